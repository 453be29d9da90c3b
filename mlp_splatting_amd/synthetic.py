"""Seeded synthetic scenes and pinhole cameras for parity tests and the benchmark.

Scene tensors follow the parameter layout of the reference scene module
(scannet/cumodel.py:712-752): ``positions[N,3] log_scales[N,3] quats[N,4](w,x,y,z)
W1[N,H,12F] b1[N,H] W2[N,H,H] b2[N,H] W3[N,4,H] b3[N,4] feat_attr[N,S,C]``.
The "opacity logit" of a primitive is the bias of MLP output channel 3, ``b3[:,3]``
(scannet/cuda/np_tile_kernels.cu:2092-2095).

Draw order from ``numpy.random.default_rng(seed)`` (all float32 unless noted):
positions U(-2,2) -> [cluster redraw] -> log_scales N(mean,0.5) -> quats N(0,1) normalised ->
W1, b1, W2, b2, W3 N(0,0.1) -> b3[:, :3] N(0,0.1) -> b3[:,3] N(0,1) -> feat_attr N(0,0.05).
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import numpy as np

# name -> (primitives, width, height, focal, hidden, log-scale mean, threshold, feature dim, clustered fraction)
CONFIGS = {
    # 5k primitives, 160x120: the CPU-runnable regression case
    "cfg1_5k_160x120": dict(n=5000, width=160, height=120, focal=150.0, hidden=16, log_scale_mean=-3.0,
                            threshold=1e-3, feature_dim=0, cluster_frac=0.0),
    # 50k primitives, 640x480, RGB only, f32: bit-exact tile-list counts and order
    "cfg2_50k_640x480": dict(n=50000, width=640, height=480, focal=600.0, hidden=32, log_scale_mean=-3.0,
                             threshold=1e-3, feature_dim=0, cluster_frac=0.0),
    # 200k primitives, 1200x680: the headline configuration.  With log-scale mean -3.0 every tile
    # exceeds the 1,536-candidate capacity; LOG_SCALE_MEAN_200K is the shifted mean that fits.
    "cfg3_200k_1200x680": dict(n=200000, width=1200, height=680, focal=600.0, hidden=32, log_scale_mean=None,
                               threshold=5e-3, feature_dim=0, cluster_frac=0.0),
    "cfg4_200k_mosaic4": dict(n=200000, width=2400, height=1360, focal=600.0, hidden=32, log_scale_mean=None,
                              threshold=5e-3, feature_dim=0, cluster_frac=0.3),
    "cfg5_200k_feat512": dict(n=200000, width=1200, height=680, focal=600.0, hidden=32, log_scale_mean=None,
                              threshold=5e-3, feature_dim=512, cluster_frac=0.0),
}

# Mean of the natural-log scales used for the 200k-primitive scenes (sigma stays 0.5).
LOG_SCALE_MEAN_200K = -3.85
LOG_SCALE_MEAN_200K_CLUSTERED = -6.0


@dataclass
class Scene:
    positions: np.ndarray
    log_scales: np.ndarray
    quats: np.ndarray
    W1: np.ndarray
    b1: np.ndarray
    W2: np.ndarray
    b2: np.ndarray
    W3: np.ndarray
    b3: np.ndarray
    feat_attr: np.ndarray | None
    freq: np.ndarray
    att: np.ndarray

    @property
    def n(self) -> int:
        return int(self.positions.shape[0])

    @property
    def hidden(self) -> int:
        return int(self.W2.shape[1])

    def mlp(self):
        return self.W1, self.b1, self.W2, self.b2, self.W3, self.b3


def frequency_bands(num_frequencies: int = 6, sigma: float = 0.01):
    """freq_k = 2^k*pi, att_k = exp(-0.5*freq_k^2*sigma^2) (scannet/cumodel.py:138, 1078-1081)."""
    freq = (2.0 ** np.arange(num_frequencies, dtype=np.float32) * np.float32(math.pi)).astype(np.float32)
    att = np.exp(np.float32(-0.5) * (freq * freq) * np.float32(sigma * sigma)).astype(np.float32)
    return freq, att


def make_scene(n: int, hidden: int = 32, seed: int = 0, log_scale_mean: float = -3.0, feature_dim: int = 0,
               feature_slots: int = 4, cluster_frac: float = 0.0, num_frequencies: int = 6) -> Scene:
    rng = np.random.default_rng(seed)
    f32 = np.float32

    def normal(shape, std, mean=0.0):
        out = rng.standard_normal(shape, dtype=f32)
        out *= f32(std)
        if mean:
            out += f32(mean)
        return out

    positions = (rng.random((n, 3), dtype=f32) * f32(4.0) - f32(2.0)).astype(f32)
    if cluster_frac > 0.0:
        k = int(round(n * cluster_frac))
        positions[:k] = rng.random((k, 3), dtype=f32) * f32(0.5) - f32(0.25)
    log_scales = normal((n, 3), 0.5, log_scale_mean)
    q = rng.standard_normal((n, 4), dtype=f32)
    quats = (q / np.maximum(np.linalg.norm(q, axis=1, keepdims=True), f32(1e-12))).astype(f32)
    enc = 12 * num_frequencies
    W1 = normal((n, hidden, enc), 0.1)
    b1 = normal((n, hidden), 0.1)
    W2 = normal((n, hidden, hidden), 0.1)
    b2 = normal((n, hidden), 0.1)
    W3 = normal((n, 4, hidden), 0.1)
    b3 = np.empty((n, 4), f32)
    b3[:, :3] = normal((n, 3), 0.1)
    b3[:, 3] = normal((n,), 1.0)
    feat = normal((n, feature_slots, feature_dim), 0.05) if feature_dim > 0 else None
    freq, att = frequency_bands(num_frequencies)
    return Scene(positions, log_scales, quats, W1, b1, W2, b2, W3, b3, feat, freq, att)


def scene_for_config(name: str, seed: int = 0, n_override: int | None = None,
                     with_features: bool = True) -> tuple[Scene, dict]:
    cfg = dict(CONFIGS[name])
    if cfg["log_scale_mean"] is None:
        cfg["log_scale_mean"] = LOG_SCALE_MEAN_200K_CLUSTERED if cfg["cluster_frac"] > 0 else LOG_SCALE_MEAN_200K
    n = cfg["n"] if n_override is None else int(n_override)
    scene = make_scene(n, cfg["hidden"], seed, cfg["log_scale_mean"], cfg["feature_dim"] if with_features else 0, 4,
                       cfg["cluster_frac"])
    return scene, cfg


# ---------------------------------------------------------------------------------------------
# cameras
# ---------------------------------------------------------------------------------------------
def look_at(eye, target=(0.0, 0.0, 0.0), up=(0.0, 1.0, 0.0)) -> np.ndarray:
    """Camera-to-world [3,4] with columns (right, down, forward, eye): +z looks at the target."""
    eye = np.asarray(eye, np.float64)
    fwd = np.asarray(target, np.float64) - eye
    fwd /= np.linalg.norm(fwd)
    right = np.cross(fwd, np.asarray(up, np.float64))
    if np.linalg.norm(right) < 1e-6:
        right = np.cross(fwd, np.array([1.0, 0.0, 0.0]))
    right /= np.linalg.norm(right)
    down = np.cross(fwd, right)
    c2w = np.stack([right, down, fwd, eye], axis=1)
    return c2w.astype(np.float32)


def random_poses(count: int, seed: int = 0, extent: float = 1.5) -> list[np.ndarray]:
    """Camera centres U(-extent, extent)^3 looking at the cube centre, up = +y."""
    rng = np.random.default_rng(seed + 1000003)
    eyes = rng.uniform(-extent, extent, (count, 3))
    return [look_at(e) for e in eyes]


def pinhole_rays(width: int, height: int, focal: float, c2w: np.ndarray):
    """Legacy-centred rays d_cam = ((i-W/2)/f, (j-H/2)/f, 1), d = R d_cam, o = eye
    (replica/replica_loader.py:461-476).  Directions are NOT normalised here."""
    i, j = np.meshgrid(np.arange(width, dtype=np.float32), np.arange(height, dtype=np.float32), indexing="xy")
    dirs = np.stack([(i - np.float32(width * 0.5)) / np.float32(focal),
                     (j - np.float32(height * 0.5)) / np.float32(focal),
                     np.ones_like(i)], -1).astype(np.float32)
    R = c2w[:3, :3].astype(np.float32)
    rays_d = (dirs[..., None, :] * R).sum(-1).reshape(-1, 3).astype(np.float32)
    rays_o = np.broadcast_to(c2w[:3, 3].astype(np.float32), rays_d.shape).copy()
    return rays_o, rays_d


def normalize_rays(rays_d: np.ndarray) -> np.ndarray:
    n = np.maximum(np.linalg.norm(rays_d, axis=-1, keepdims=True), np.float32(1e-12))
    return (rays_d / n).astype(np.float32)


def view_matrix(c2w: np.ndarray) -> np.ndarray:
    """inverse([c2w; 0 0 0 1]) = [R^T, -R^T t] (scannet/eval_rgb_psnr.py:90-93)."""
    R = c2w[:3, :3].astype(np.float64)
    t = c2w[:3, 3].astype(np.float64)
    V = np.eye(4)
    V[:3, :3] = R.T
    V[:3, 3] = -R.T @ t
    return V.astype(np.float32)


def projection_matrix(focal: float, width: int, height: int, near: float = 1e-3, far: float = 100.0) -> np.ndarray:
    """scannet/eval_rgb_psnr.py:68-87."""
    fov_y = 2.0 * math.atan((0.5 * height) / (focal + 1e-8))
    t = math.tan(fov_y / 2.0)
    r = t * (float(width) / float(height))
    P = np.zeros((4, 4), np.float32)
    P[0, 0] = 1.0 / r
    P[1, 1] = 1.0 / t
    P[2, 2] = -(far + near) / (far - near)
    P[3, 2] = 1.0
    P[2, 3] = -(2 * far * near) / (far - near)
    return P


def mosaic_frame(width: int, height: int, focal: float, poses: list[np.ndarray], tile: int = 8):
    """Four views of width x height laid out as one 2*width x 2*height frame (quadrant q uses
    poses[q]); returns rays, per-tile view ids and the K view matrices, the form in which the
    reference expresses several views per call (scannet/cumodel.py:838-949)."""
    assert len(poses) == 4 and width % tile == 0 and height % tile == 0
    W2, H2 = 2 * width, 2 * height
    rays_o = np.empty((H2, W2, 3), np.float32)
    rays_d = np.empty((H2, W2, 3), np.float32)
    for q, c2w in enumerate(poses):
        o, d = pinhole_rays(width, height, focal, c2w)
        qy, qx = divmod(q, 2)
        rays_o[qy * height:(qy + 1) * height, qx * width:(qx + 1) * width] = o.reshape(height, width, 3)
        rays_d[qy * height:(qy + 1) * height, qx * width:(qx + 1) * width] = d.reshape(height, width, 3)
    ntx, nty = W2 // tile, H2 // tile
    ty, tx = np.meshgrid(np.arange(nty), np.arange(ntx), indexing="ij")
    tile_view_ids = ((ty >= nty // 2) * 2 + (tx >= ntx // 2)).reshape(-1).astype(np.int32)
    # The culling rule projects with ONE matrix whose principal point is the centre of the whole
    # 2W x 2H frame.  A quadrant's own principal point sits (qx-1/2)W, (qy-1/2)H pixels away; that
    # offset is a shear of view space along z and is folded into the quadrant's view matrix, which
    # leaves the view-space depth and hence the projected radius untouched.
    views = []
    for q, c2w in enumerate(poses):
        qy, qx = divmod(q, 2)
        shear = np.eye(4, dtype=np.float64)
        shear[0, 2] = (qx - 0.5) * width / focal
        shear[1, 2] = (qy - 0.5) * height / focal
        views.append((shear @ view_matrix(c2w).astype(np.float64)).astype(np.float32))
    return rays_o.reshape(-1, 3), rays_d.reshape(-1, 3), tile_view_ids, np.stack(views)
