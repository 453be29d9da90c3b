"""Ray-cone tile culling for native (non-centred, possibly distorted) cameras.

Same function name, arguments, return values and exceptions as ``ray_cone_candidates`` in the
reference's ``scannet/camera.py:102-146``; the work runs in ``libmlpsp_hip.so``.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from .ops import _check, _f32c, _ptr, _stream, num_tiles


@torch.no_grad()
def ray_cone_candidates(ray_o, ray_d, positions, log_scales, width, height, tile_size, score_threshold,
                        tile_chunk=128):
    """Conservative tile lists from the actual rays -> (ids int32 [P], offsets int32 [T+1]).

    ``tile_chunk`` is accepted for signature compatibility; the kernels need no chunking.
    """
    if not 0 < score_threshold < 1:
        raise ValueError("score_threshold must be in (0,1)")
    if tuple(ray_o.shape) != (height * width, 3) or ray_d.shape != ray_o.shape:
        raise ValueError("ray shape mismatch")
    device = positions.device
    if ray_o.device != device or ray_d.device != device:
        raise ValueError("device mismatch")
    ray_o, ray_d = _f32c(ray_o, "ray_o"), _f32c(ray_d, "ray_d")
    positions, log_scales = _f32c(positions.detach(), "positions"), _f32c(log_scales.detach(), "log_scales")
    lib = _lib.load()
    n, T = positions.shape[0], num_tiles(width, height, tile_size, tile_size)
    offsets = torch.empty(T + 1, dtype=torch.int32, device=device)
    nbytes = lib.mlpsp_bin_raycone_scratch_bytes(n, width, height, tile_size)
    scratch = torch.empty(nbytes, dtype=torch.uint8, device=device)
    total = C.c_int64(0)
    with torch.cuda.device(device):
        code = lib.mlpsp_bin_raycone_count(_ptr(ray_o), _ptr(ray_d), _ptr(positions), _ptr(log_scales), n, width, height,
                                           tile_size, float(score_threshold), _ptr(scratch), nbytes, _ptr(offsets),
                                           C.byref(total), _stream(device))
        if code == _lib.E_MIXED_ORIGINS:
            raise ValueError("Each tile must use a single camera origin")
        if code == _lib.E_WIDE_CONE:
            raise ValueError("Tile ray cone spans >=90 degrees")
        _check(code, "mlpsp_bin_raycone_count")
        if total.value >= 2 ** 31:
            raise OverflowError("Tile candidate count exceeds int32 capacity")
        ids = torch.empty(int(total.value), dtype=torch.int32, device=device)
        if total.value > 0:
            code = lib.mlpsp_bin_raycone_fill(n, width, height, tile_size, _ptr(scratch), nbytes, _ptr(offsets), _ptr(ids),
                                              _stream(device))
            _check(code, "mlpsp_bin_raycone_fill")
    return ids, offsets
