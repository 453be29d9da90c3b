"""numpy front end of the CPU oracle (``mlpsp_oracle.cpp``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``; never by the shipped package.  The shared object is built by
``oracle/Makefile`` (``build()`` here runs it) into ``oracle/_build/``.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libmlpsp_oracle.so")
_lib = None

_f = C.POINTER(C.c_float)
_i = C.POINTER(C.c_int32)
_l = C.POINTER(C.c_int64)
_b = C.POINTER(C.c_uint8)


def build(force: bool = False) -> str:
    """Compile the oracle with g++ (idempotent unless ``force``)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
        _lib.mlpsp_oracle_key.restype = C.c_float
        _lib.mlpsp_oracle_bin_legacy.restype = C.c_int64
        _lib.mlpsp_oracle_bin_raycone.restype = C.c_int64
    return _lib


def _fa(x):
    return np.ascontiguousarray(x, dtype=np.float32)


def _ia(x):
    return np.ascontiguousarray(x, dtype=np.int32)


def _p(a, t):
    return None if a is None else a.ctypes.data_as(t)


# ---------------------------------------------------------------------------------------------
# elementary functions
# ---------------------------------------------------------------------------------------------
_MATH = {"exp": 0, "sincos": 1, "log1p": 2, "sigmoid": 3, "softplus": 4, "round_bf16": 5, "round_f16": 6}


def math(which: str, x):
    x = _fa(x).ravel()
    y = np.empty_like(x)
    y2 = np.empty_like(x)
    lib().mlpsp_oracle_math(_MATH[which], _p(x, _f), _p(y, _f), _p(y2, _f), C.c_int64(x.size))
    return (y, y2) if which == "sincos" else y


def hit(ray_o, ray_d, pos, log_s, quat, thr):
    """One ray against one primitive -> (hit, dict(t, d[3], q[3], decay))."""
    out = np.zeros(8, np.float32)
    h = lib().mlpsp_oracle_hit(_p(_fa(ray_o), _f), _p(_fa(ray_d), _f), _p(_fa(pos), _f), _p(_fa(log_s), _f),
                               _p(_fa(quat), _f), C.c_float(thr), _p(out, _f))
    return bool(h), {"t": out[0], "d": out[1:4].copy(), "q": out[4:7].copy(), "decay": out[7]}


def key(family, ray_o, ray_d, pos, log_s, quat):
    return float(lib().mlpsp_oracle_key(int(family), _p(_fa(ray_o), _f), _p(_fa(ray_d), _f), _p(_fa(pos), _f),
                                        _p(_fa(log_s), _f), _p(_fa(quat), _f)))


def gates(ql, log_s, beta, temp):
    g = np.zeros(4, np.float32)
    lib().mlpsp_oracle_gates(_p(_fa(ql), _f), _p(_fa(log_s), _f), C.c_float(beta), C.c_float(temp), _p(g, _f))
    return g


def mlp(x6, prim_ids, freq, att, W1, b1, W2, b2, W3, b3, precision=0):
    x6 = _fa(x6)
    ids = _ia(prim_ids)
    W1, b1, W2, b2, W3, b3 = map(_fa, (W1, b1, W2, b2, W3, b3))
    freq, att = _fa(freq), _fa(att)
    out = np.zeros((x6.shape[0], 4), np.float32)
    lib().mlpsp_oracle_mlp(_p(x6, _f), _p(ids, _i), C.c_int64(x6.shape[0]), _p(freq, _f), _p(att, _f),
                           int(freq.size), _p(W1, _f), _p(b1, _f), _p(W2, _f), _p(b2, _f), _p(W3, _f), _p(b3, _f),
                           int(W2.shape[1]), int(precision), _p(out, _f))
    return out


def validate(offsets, cand, num_tiles, capacity, num_prims):
    offsets, cand = _ia(offsets), _ia(cand)
    status = np.zeros(2, np.int32)
    lib().mlpsp_oracle_validate(_p(offsets, _i), _p(cand, _i), int(num_tiles), int(cand.size), int(capacity),
                                int(num_prims), _p(status, _i))
    return status


# ---------------------------------------------------------------------------------------------
# binning
# ---------------------------------------------------------------------------------------------
def bin_legacy(pos, log_s, view_mats, proj, W, H, ts, thr, tile_view_ids=None):
    pos, log_s = _fa(pos), _fa(log_s)
    V = _fa(view_mats).reshape(-1, 4, 4)
    Pm = _fa(proj).reshape(4, 4)
    tv = None if tile_view_ids is None else _ia(tile_view_ids)
    T = ((W + ts - 1) // ts) * ((H + ts - 1) // ts)
    offsets = np.zeros(T + 1, np.int32)
    args = (_p(pos, _f), _p(log_s, _f), int(pos.shape[0]), _p(V, _f), int(V.shape[0]), _p(tv, _i), _p(Pm, _f),
            int(W), int(H), int(ts), C.c_float(thr), _p(offsets, _i))
    total = lib().mlpsp_oracle_bin_legacy(*args, None)
    cand = np.zeros(max(int(total), 0), np.int32)
    if total > 0:
        lib().mlpsp_oracle_bin_legacy(*args, _p(cand, _i))
    return cand, offsets


def bin_legacy_dense(pos, log_s, view_mats, proj, W, H, ts, thr, tile_view_ids=None):
    pos, log_s = _fa(pos), _fa(log_s)
    V = _fa(view_mats).reshape(-1, 4, 4)
    Pm = _fa(proj).reshape(4, 4)
    tv = None if tile_view_ids is None else _ia(tile_view_ids)
    T = ((W + ts - 1) // ts) * ((H + ts - 1) // ts)
    mask = np.zeros((T, pos.shape[0]), np.uint8)
    lib().mlpsp_oracle_bin_legacy_dense(_p(pos, _f), _p(log_s, _f), int(pos.shape[0]), _p(V, _f), int(V.shape[0]),
                                        _p(tv, _i), _p(Pm, _f), int(W), int(H), int(ts), C.c_float(thr), _p(mask, _b))
    return mask


def bin_raycone(rays_o, rays_d, pos, log_s, W, H, ts, thr):
    rays_o, rays_d, pos, log_s = map(_fa, (rays_o, rays_d, pos, log_s))
    T = ((W + ts - 1) // ts) * ((H + ts - 1) // ts)
    offsets = np.zeros(T + 1, np.int32)
    args = (_p(rays_o, _f), _p(rays_d, _f), _p(pos, _f), _p(log_s, _f), int(pos.shape[0]), int(W), int(H), int(ts),
            C.c_float(thr), _p(offsets, _i))
    total = lib().mlpsp_oracle_bin_raycone(*args, None)
    if total == -1:
        raise ValueError("Each tile must use a single camera origin")
    if total == -2:
        raise ValueError("Tile ray cone spans >=90 degrees")
    cand = np.zeros(int(total), np.int32)
    if total > 0:
        lib().mlpsp_oracle_bin_raycone(*args, _p(cand, _i))
    return cand, offsets


# ---------------------------------------------------------------------------------------------
# sort + render
# ---------------------------------------------------------------------------------------------
def sort_tiles(rays_o, rays_d, pos, log_s, quats, cand, offsets, W, H, TW, TH, family=1, capacity=1536):
    rays_o, rays_d, pos, log_s, quats = map(_fa, (rays_o, rays_d, pos, log_s, quats))
    cand, offsets = _ia(cand), _ia(offsets)
    ids = np.zeros_like(cand)
    keys = np.zeros(cand.shape, np.float32)
    lib().mlpsp_oracle_sort_tiles(_p(rays_o, _f), _p(rays_d, _f), _p(pos, _f), _p(log_s, _f), _p(quats, _f),
                                  _p(cand, _i), _p(offsets, _i), int(W), int(H), int(TW), int(TH), int(family),
                                  int(capacity), _p(ids, _i), _p(keys, _f))
    return ids, keys


def _scene_args(rays_o, rays_d, pos, log_s, quats, cand, offsets, freq, att, W1, b1, W2, b2, W3, b3):
    arrs = list(map(_fa, (rays_o, rays_d, pos, log_s, quats)))
    cand, offsets = _ia(cand), _ia(offsets)
    freq, att = _fa(freq), _fa(att)
    Ws = list(map(_fa, (W1, b1, W2, b2, W3, b3)))
    keep = arrs + [cand, offsets, freq, att] + Ws
    args = [_p(a, _f) for a in arrs] + [_p(cand, _i), _p(offsets, _i), _p(freq, _f), _p(att, _f), int(freq.size)]
    args += [_p(a, _f) for a in Ws] + [int(arrs[2].shape[0]), int(Ws[2].shape[1])]
    return args, keep


def _feat_args(feat_attr, beta, temp):
    if feat_attr is None:
        return [None, 0, 0, C.c_float(beta), C.c_float(temp)], None
    fa = _fa(feat_attr)
    slots, ch = (1, fa.shape[1]) if fa.ndim == 2 else (fa.shape[1], fa.shape[2])
    return [_p(fa, _f), int(slots), int(ch), C.c_float(beta), C.c_float(temp)], fa


def render_tilecenter(rays_o, rays_d, pos, log_s, quats, cand, offsets, freq, att, W1, b1, W2, b2, W3, b3,
                      W, H, TW, TH, thr, *, family=1, precision=0, capacity=1536, feat_attr=None, beta=1.5,
                      temp=2.0, with_t=False, nthreads=0):
    """Returns dict(rgb[B,3], alpha[B,1], t[B,1]|None, feat[B,C]|None, stats[4])."""
    args, keep = _scene_args(rays_o, rays_d, pos, log_s, quats, cand, offsets, freq, att, W1, b1, W2, b2, W3, b3)
    fargs, fa = _feat_args(feat_attr, beta, temp)
    B = W * H
    rgb = np.zeros((B, 3), np.float32)
    alpha = np.zeros((B, 1), np.float32)
    t = np.zeros((B, 1), np.float32) if with_t else None
    feat = np.zeros((B, fargs[2]), np.float32) if fa is not None else None
    stats = np.zeros(4, np.int64)
    lib().mlpsp_oracle_render_tilecenter(*args, *fargs, int(W), int(H), int(TW), int(TH), C.c_float(thr), int(family),
                                         int(precision), int(capacity), _p(rgb, _f), _p(alpha, _f), _p(t, _f),
                                         _p(feat, _f), _p(stats, _l), int(nthreads))
    del keep
    return {"rgb": rgb, "alpha": alpha, "t": t, "feat": feat, "stats": stats}


def render_stats(rays_o, rays_d, pos, log_s, quats, cand, offsets, freq, att, W1, b1, W2, b2, W3, b3,
                 W, H, TW, TH, thr, gt_rgb, *, capacity=1536, nthreads=0):
    """Pruning-statistics forward -> dict(rgb, alpha, sum_w, max_w, hits, sum_werr, contrib), the five
    statistics as the increments one call adds to zeroed per-primitive buffers (float64 / int64)."""
    args, keep = _scene_args(rays_o, rays_d, pos, log_s, quats, cand, offsets, freq, att, W1, b1, W2, b2, W3, b3)
    gt = _fa(gt_rgb)
    B, n = W * H, int(np.asarray(pos).shape[0])
    rgb = np.zeros((B, 3), np.float32)
    alpha = np.zeros((B, 1), np.float32)
    sum_w, max_w, sum_werr = (np.zeros(n, np.float64) for _ in range(3))
    hits, contrib = np.zeros(n, np.int64), np.zeros(n, np.int64)
    _d = C.POINTER(C.c_double)
    lib().mlpsp_oracle_render_stats(*args, int(W), int(H), int(TW), int(TH), C.c_float(thr), int(capacity), _p(gt, _f),
                                    _p(rgb, _f), _p(alpha, _f), _p(sum_w, _d), _p(max_w, _d), _p(hits, _l),
                                    _p(sum_werr, _d), _p(contrib, _l), int(nthreads))
    del keep
    return {"rgb": rgb, "alpha": alpha, "sum_w": sum_w, "max_w": max_w, "hits": hits, "sum_werr": sum_werr,
            "contrib": contrib}


def records(rays_o, rays_d, pos, log_s, quats, cand, offsets, freq, att, W1, b1, W2, b2, W3, b3,
            W, H, TW, TH, thr, *, capacity=1536, max_hits=128, beta=1.5, temp=2.0, nthreads=0):
    """Training-records forward -> dict(rgb, alpha, ids[R], x6[R,6], raw[R,8], masks[R,2], gates[R,4],
    offsets[B+1] int64, overflow: bool)."""
    args, keep = _scene_args(rays_o, rays_d, pos, log_s, quats, cand, offsets, freq, att, W1, b1, W2, b2, W3, b3)
    B = W * H
    counts = np.zeros(B, np.int32)
    ovf = np.zeros(1, np.int32)
    tail = (int(W), int(H), int(TW), int(TH), C.c_float(thr), int(capacity), int(max_hits), C.c_float(beta),
            C.c_float(temp))
    lib().mlpsp_oracle_records(*args, *tail, _p(counts, _i), _p(ovf, _i), None, None, None, None, None, None, None,
                               None, int(nthreads))
    offs = np.zeros(B + 1, np.int64)
    np.cumsum(counts, out=offs[1:])
    R = int(offs[-1])
    ids = np.zeros(R, np.int32)
    x6 = np.zeros((R, 6), np.float32)
    masks = np.zeros((R, 2), np.int32)
    raw = np.zeros((R, 8), np.float32)
    gates = np.zeros((R, 4), np.float32)
    rgb = np.zeros((B, 3), np.float32)
    alpha = np.zeros((B, 1), np.float32)
    lib().mlpsp_oracle_records(*args, *tail, _p(counts, _i), _p(ovf, _i), _p(offs, _l), _p(ids, _i), _p(x6, _f),
                               _p(masks, _i), _p(raw, _f), _p(gates, _f), _p(rgb, _f), _p(alpha, _f), int(nthreads))
    del keep
    return {"rgb": rgb, "alpha": alpha, "ids": ids, "x6": x6, "raw": raw, "masks": masks, "gates": gates,
            "offsets": offs, "overflow": bool(ovf[0])}


def records_per_pixel(rays_o, rays_d, pos, log_s, quats, cand, offsets, freq, att, W1, b1, W2, b2, W3, b3,
                      W, H, TW, TH, thr, *, beta=1.5, temp=2.0, nthreads=0):
    """Training records in per-pixel order -> the dict of :func:`records` (overflow: a pixel met a 257th hit)."""
    args, keep = _scene_args(rays_o, rays_d, pos, log_s, quats, cand, offsets, freq, att, W1, b1, W2, b2, W3, b3)
    B = W * H
    counts = np.zeros(B, np.int32)
    tail = (int(W), int(H), int(TW), int(TH), C.c_float(thr), C.c_float(beta), C.c_float(temp))
    fn = lib().mlpsp_oracle_records_per_pixel
    fn.restype = C.c_int
    ovf = fn(*args, *tail, _p(counts, _i), None, None, None, None, None, None, None, None, int(nthreads))
    offs = np.zeros(B + 1, np.int64)
    np.cumsum(counts, out=offs[1:])
    R = int(offs[-1])
    ids = np.zeros(R, np.int32)
    x6 = np.zeros((R, 6), np.float32)
    masks = np.zeros((R, 2), np.int32)
    raw = np.zeros((R, 8), np.float32)
    gates = np.zeros((R, 4), np.float32)
    rgb = np.zeros((B, 3), np.float32)
    alpha = np.zeros((B, 1), np.float32)
    fn(*args, *tail, _p(counts, _i), _p(offs, _l), _p(ids, _i), _p(x6, _f), _p(masks, _i), _p(raw, _f), _p(gates, _f),
       _p(rgb, _f), _p(alpha, _f), int(nthreads))
    del keep
    return {"rgb": rgb, "alpha": alpha, "ids": ids, "x6": x6, "raw": raw, "masks": masks, "gates": gates,
            "offsets": offs, "overflow": bool(ovf)}


def render_per_pixel(rays_o, rays_d, pos, log_s, quats, cand, offsets, freq, att, W1, b1, W2, b2, W3, b3,
                     W, H, TW, TH, thr, *, feat_attr=None, beta=1.5, temp=2.0, nthreads=0):
    """Returns dict(rgb, alpha, feat|None, overflow: bool)."""
    args, keep = _scene_args(rays_o, rays_d, pos, log_s, quats, cand, offsets, freq, att, W1, b1, W2, b2, W3, b3)
    fargs, fa = _feat_args(feat_attr, beta, temp)
    B = W * H
    rgb = np.zeros((B, 3), np.float32)
    alpha = np.zeros((B, 1), np.float32)
    feat = np.zeros((B, fargs[2]), np.float32) if fa is not None else None
    ov = lib().mlpsp_oracle_render_per_pixel(*args, *fargs, int(W), int(H), int(TW), int(TH), C.c_float(thr),
                                             _p(rgb, _f), _p(alpha, _f), _p(feat, _f), int(nthreads))
    del keep
    return {"rgb": rgb, "alpha": alpha, "feat": feat, "overflow": bool(ov)}


def records_reverse(ids, offsets, x6, raw, log_s, quats, grad_rgb, grad_t):
    """Reverse compositing over saved records -> (d4[R,4], grad_positions[N,3], grad_log_scales[N,3],
    grad_quats[N,4]), f32, summed sequentially."""
    ids = np.ascontiguousarray(ids, np.int32)
    offsets = np.ascontiguousarray(offsets, np.int64)
    x6, raw = np.ascontiguousarray(x6, np.float32), np.ascontiguousarray(raw, np.float32)
    log_s, quats = np.ascontiguousarray(log_s, np.float32), np.ascontiguousarray(quats, np.float32)
    grad_rgb, grad_t = np.ascontiguousarray(grad_rgb, np.float32), np.ascontiguousarray(grad_t, np.float32)
    d4 = np.zeros((ids.size, 4), np.float32)
    gp, gs, gq = np.zeros_like(log_s), np.zeros_like(log_s), np.zeros_like(quats)
    lib().mlpsp_oracle_records_reverse(_p(ids, _i), _p(offsets, _l), _p(x6, _f), _p(raw, _f), _p(log_s, _f),
                                       _p(quats, _f), _p(grad_rgb, _f), _p(grad_t, _f), C.c_int64(grad_t.size),
                                       _p(d4, _f), _p(gp, _f), _p(gs, _f), _p(gq, _f))
    return d4, gp, gs, gq


def num_threads() -> int:
    return int(lib().mlpsp_oracle_num_threads())
