"""The committed frame of tests/golden/ (made by tests/golden/make_frame_fixture.py): every input array of the
forward renderer for a small seeded scene and the outputs recorded for it.

On the CPU the oracle has to reproduce the recorded outputs bit for bit (it cannot drift unnoticed); on the GPU the
HIP path is held to the recorded outputs directly, through the C ABI, without the oracle at run time: integer
work and the f32 image to the bit, the matrix-core images within 5e-3 (bf16) / 5e-4 (fp16) of the recorded
emulation of their rounding points.
"""
import os

import numpy as np
import pytest
import torch

from conftest import to_dev
from helpers import bits

FIXTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "frame_160_56x40.npz")


@pytest.fixture(scope="module")
def gold():
    with np.load(FIXTURE, allow_pickle=False) as z:
        g = {k: z[k] for k in z.files}
    g["W"], g["H"], g["tile"] = (int(v) for v in g["dims"])
    g["thr"] = float(g["threshold"])
    return g


def _same_bits(got, want, what):
    got = got.detach().cpu().numpy() if torch.is_tensor(got) else got
    differing = int((bits(got) != bits(want)).sum())
    assert differing == 0, f"{what}: {differing} of {want.size} values differ"


def _scene(g):
    return [g[k] for k in ("positions", "log_scales", "quats")]


def _mlp(g):
    return [g[k] for k in ("W1", "b1", "W2", "b2", "W3", "b3")]


def test_fixture_is_a_meaningful_frame(gold):
    g = gold
    off = g["tile_offsets"]
    assert off.shape == ((g["W"] // g["tile"]) * (g["H"] // g["tile"]) + 1,) and off[0] == 0 and off[-1] == g["candidates"].size
    assert 0.5 < g["alpha"].mean() < 0.95 and g["alpha"].max() > 0.999       # open and saturated pixels both occur
    assert g["stats"][1] < g["stats"][0]                                     # early termination left pairs unprocessed
    assert not np.array_equal(g["sorted_ids_depth"], g["candidates"])
    assert 1e-5 < np.abs(g["rgb_bf16"] - g["rgb"]).max() < 5e-3


def test_oracle_reproduces_the_recorded_frame(oracle_mod, gold):
    g = gold
    dims = (g["W"], g["H"], g["tile"])
    cand, off = oracle_mod.bin_legacy(g["positions"], g["log_scales"], g["view"][None], g["proj"], *dims, g["thr"])
    np.testing.assert_array_equal(cand, g["candidates"])
    np.testing.assert_array_equal(off, g["tile_offsets"])
    for family, tag in ((1, "depth"), (2, "tstar")):
        ids, keys = oracle_mod.sort_tiles(g["rays_o"], g["rays_d"], *_scene(g), cand, off, g["W"], g["H"], g["tile"],
                                          g["tile"], family=family)
        np.testing.assert_array_equal(ids, g[f"sorted_ids_{tag}"])
        _same_bits(keys, g[f"sorted_keys_{tag}"], f"{tag} keys")
    base = (g["rays_o"], g["rays_d"], *_scene(g), cand, off, g["freq"], g["att"], *_mlp(g), g["W"], g["H"], g["tile"],
            g["tile"], g["thr"])
    img = oracle_mod.render_tilecenter(*base)
    _same_bits(img["rgb"], g["rgb"], "rgb")
    _same_bits(img["alpha"], g["alpha"], "alpha")
    np.testing.assert_array_equal(img["stats"], g["stats"])
    img = oracle_mod.render_tilecenter(*base, family=2, with_t=True)
    _same_bits(img["rgb"], g["rgb_tstar"], "rgb (t* order)")
    _same_bits(img["t"], g["t_tstar"], "expected depth")
    for precision, tag in ((1, "bf16"), (2, "fp16")):
        _same_bits(oracle_mod.render_tilecenter(*base, precision=precision)["rgb"], g[f"rgb_{tag}"], f"rgb {tag} emulation")


@pytest.mark.gpu
def test_hip_path_reproduces_the_recorded_frame(device, gold):
    from mlp_splatting_amd import ops
    g = gold
    t = lambda a: to_dev(a, device)
    W, H, tile, thr = g["W"], g["H"], g["tile"], g["thr"]
    pos, ls, qu = (t(a) for a in _scene(g))
    cand, off = ops.bin_legacy(pos, ls, torch.from_numpy(g["view"])[None], torch.from_numpy(g["proj"]), W, H, tile, thr)
    np.testing.assert_array_equal(cand.cpu().numpy(), g["candidates"])
    np.testing.assert_array_equal(off.cpu().numpy(), g["tile_offsets"])
    rec = ops.prepare_primitives(pos, ls, qu)
    ro, rd = t(g["rays_o"]), t(g["rays_d"])
    freq, att, ws = t(g["freq"]), t(g["att"]), [t(w) for w in _mlp(g)]
    orders = {}
    for family, tag in ((1, "depth"), (2, "tstar")):
        ids, keys = ops.sort_tiles(ro, rd, rec, cand, off, W, H, tile, tile, family=family, want_keys=True)
        np.testing.assert_array_equal(ids.cpu().numpy(), g[f"sorted_ids_{tag}"])
        _same_bits(keys, g[f"sorted_keys_{tag}"], f"{tag} keys")
        orders[tag] = ids
    counters = torch.zeros(4, dtype=torch.int64, device=device)
    rgb, alpha, _ = ops.render_tilecenter_f32(ro, rd, rec, orders["depth"], off, freq, att, *ws, W, H, tile, tile, thr,
                                              counters=counters)
    _same_bits(rgb, g["rgb"], "rgb")
    _same_bits(alpha, g["alpha"], "alpha")
    np.testing.assert_array_equal(counters.cpu().numpy()[1:], g["stats"][1:])
    rgb, _, depth = ops.render_tilecenter_f32(ro, rd, rec, orders["tstar"], off, freq, att, *ws, W, H, tile, tile, thr,
                                              with_t=True)
    _same_bits(rgb, g["rgb_tstar"], "rgb (t* order)")
    _same_bits(depth, g["t_tstar"], "expected depth")
    # the culled order renders the same image
    culled, _ = ops.sort_tiles(ro, rd, rec, cand, off, W, H, tile, tile, family=1, cull_threshold=thr)
    assert int((culled < 0).sum()) > 0
    rgb, alpha, _ = ops.render_tilecenter_f32(ro, rd, rec, culled, off, freq, att, *ws, W, H, tile, tile, thr)
    _same_bits(rgb, g["rgb"], "rgb from the culled order")
    for bf16, tag, tol in ((True, "bf16", 5e-3), (False, "fp16", 5e-4)):
        rgb, alpha, nonfinite = ops.render_tilecenter_mfma(ro, rd, rec, culled, off, freq, att, *ws, W, H, thr, bf16=bf16)
        assert not nonfinite
        err = float(np.abs(rgb.cpu().numpy() - g[f"rgb_{tag}"]).max())
        assert err < tol, f"{tag}: {err:.3e}"
