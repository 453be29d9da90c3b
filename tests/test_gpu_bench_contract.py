"""bench.py prints ONE JSON line with the agreed fields; a run on more than one GPU is refused with a message."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args, timeout=300):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=timeout, cwd=ROOT)


def test_more_than_one_gpu_is_refused():
    out = _run("--gpus", "2")
    assert out.returncode != 0 and "one GPU" in (out.stdout + out.stderr)


@pytest.mark.gpu
def test_one_json_line_with_roofline_and_cpu_baseline(device):
    # a small workload keeps this to seconds; the default run is the 200k-primitive frame
    out = _run("--workload", "cfg1_5k_160x120", "--steps", "4", "--warmup", "2", "--wake-seconds", "0.1", "--poses", "4")
    assert out.returncode == 0, out.stderr[-2000:]
    lines = [l for l in out.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    # the timed region is whole passes of --steps until --min-seconds have gone by; "steps" is what was timed
    assert d["steps_per_pass"] == 4 and d["steps"] >= 4 and d["steps"] % 4 == 0
    assert d["n_gpus"] == 1 and d["warmup"] == 2 and d["higher_is_better"] is True
    assert d["vs_baseline"] is None and d["data"] == "synthetic" and d["config"]["workload"] == "cfg1_5k_160x120"
    assert d["value"] > 0 and abs(d["ms_per_step"] * d["value"] - 1000.0) < 1.0
    roof = d["roofline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in roof, key
    assert roof["bound"] in ("hbm", "mfma") and roof["peak"] > 0 and abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-4
    exact = json.loads([l for l in _run("--workload", "cfg1_5k_160x120", "--steps", "4", "--warmup", "1", "--wake-seconds", "0.1",
                                        "--poses", "4", "--min-seconds", "0").stdout.splitlines() if l.startswith("{")][0])
    assert exact["steps"] == 4
    cpu = d["cpu_baseline"]
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in cpu, key
    assert cpu["kind"] in ("port", "reference") and cpu["cores"] >= 1 and cpu["value"] > 0
