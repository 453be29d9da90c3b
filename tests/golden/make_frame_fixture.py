"""Writes tests/golden/frame_160_56x40.npz: one small seeded frame with every input array of the forward
renderer and what the CPU oracle returns for it (tile lists, sorted order and keys, RGB, alpha, expected depth,
the matrix-core emulations of the image).

The reference renderer exists only as CUDA and holds no output vectors of its own, so these vectors come from
this build's CPU restatement; they pin it (and the HIP path, which tests/test_golden_frame.py holds to the same
bits without the oracle at run time) against drifting, not against the reference.

    python tests/golden/make_frame_fixture.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from helpers import Frame  # noqa: E402
from mlp_splatting_amd import synthetic as syn  # noqa: E402
import oracle  # noqa: E402

NAME = "frame_160_56x40.npz"


def main():
    # 160 primitives clustered in front of the camera: the fixture stays under 3 MB (14 KB of weights each)
    fr = Frame("cfg1_5k_160x120", n=8, hidden=32, width=56, height=40, eye=(0.3, -0.2, -0.9), target=(0.0, 0.0, 0.0))
    fr.scene = sc = syn.make_scene(160, 32, 11, -2.7, cluster_frac=1.0)
    cand, off = fr.oracle_lists(oracle)
    out = {"rays_o": fr.rays_o, "rays_d": fr.rays_d, "view": fr.view, "proj": fr.proj,
           "positions": sc.positions, "log_scales": sc.log_scales, "quats": sc.quats, "freq": sc.freq, "att": sc.att,
           "dims": np.array([fr.W, fr.H, fr.tile], np.int32), "threshold": np.float32(fr.thr),
           "candidates": cand, "tile_offsets": off}
    for k, w in zip(("W1", "b1", "W2", "b2", "W3", "b3"), sc.mlp()):
        out[k] = w
    for family, tag in ((1, "depth"), (2, "tstar")):
        ids, keys = oracle.sort_tiles(fr.rays_o, fr.rays_d, sc.positions, sc.log_scales, sc.quats, cand, off, fr.W, fr.H,
                                      fr.tile, fr.tile, family=family)
        out[f"sorted_ids_{tag}"], out[f"sorted_keys_{tag}"] = ids, keys
    img = oracle.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims)
    out["rgb"], out["alpha"], out["stats"] = img["rgb"], img["alpha"], img["stats"]
    img = oracle.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims, family=2, with_t=True)
    out["rgb_tstar"], out["t_tstar"] = img["rgb"], img["t"]
    for precision, tag in ((1, "bf16"), (2, "fp16")):
        out[f"rgb_{tag}"] = oracle.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims, precision=precision)["rgb"]
    print("pairs", off[-1], "longest", int(np.diff(off).max()), "alpha", out["alpha"].mean(), "stats", out["stats"])
    np.savez_compressed(os.path.join(HERE, NAME), **out)
    print(NAME, {k: np.asarray(v).shape for k, v in out.items()})


if __name__ == "__main__":
    main()
