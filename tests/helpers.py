"""Shared builders for the parity tests: a seeded scene + camera + oracle tile lists."""
import numpy as np

from mlp_splatting_amd import synthetic as syn


class Frame:
    def __init__(self, name="cfg1_5k_160x120", n=None, eye=(0.3, -0.2, -0.5), target=(0.0, 0.0, 0.4), seed=0,
                 hidden=None, feature_dim=0, feature_slots=4, tile=8, width=None, height=None):
        cfg = dict(syn.CONFIGS[name])
        if cfg["log_scale_mean"] is None:
            cfg["log_scale_mean"] = syn.LOG_SCALE_MEAN_200K
        self.cfg = cfg
        self.W = width or cfg["width"]
        self.H = height or cfg["height"]
        self.f = cfg["focal"] * self.W / cfg["width"]
        self.thr = cfg["threshold"]
        self.tile = tile
        self.scene = syn.make_scene(n or cfg["n"], hidden or cfg["hidden"], seed, cfg["log_scale_mean"], feature_dim,
                                    feature_slots, cfg["cluster_frac"])
        self.c2w = syn.look_at(eye, target)
        ro, rd = syn.pinhole_rays(self.W, self.H, self.f, self.c2w)
        self.rays_o, self.rays_d = ro, syn.normalize_rays(rd)
        self.view = syn.view_matrix(self.c2w)
        self.proj = syn.projection_matrix(self.f, self.W, self.H)

    def oracle_lists(self, oracle):
        return oracle.bin_legacy(self.scene.positions, self.scene.log_scales, self.view[None], self.proj, self.W, self.H,
                                 self.tile, self.thr)

    def base_numpy(self, cand, offsets):
        s = self.scene
        return (self.rays_o, self.rays_d, s.positions, s.log_scales, s.quats, cand, offsets, s.freq, s.att, *s.mlp())

    def base_torch(self, cand, offsets, device):
        import torch
        out = []
        for a in self.base_numpy(cand, offsets):
            out.append(torch.from_numpy(np.ascontiguousarray(a)).to(device))
        return tuple(out)

    @property
    def dims(self):
        return (self.W, self.H, self.tile, self.tile, self.thr)


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def ulp_diff(a, b):
    """Distance in units in the last place between two float32 arrays of the same sign pattern."""
    ia = bits(a).astype(np.int64)
    ib = bits(b).astype(np.int64)
    ia = np.where(ia < 0x80000000, ia, 0x80000000 - ia)
    ib = np.where(ib < 0x80000000, ib, 0x80000000 - ib)
    return np.abs(ia - ib)
