"""Torch-level wrappers of the C ABI: tensors in, tensors out, kernels on the current stream.

PyTorch is used for device memory and the stream only.  Every function here ends in a call into
``libmlpsp_hip.so``; none has a PyTorch or CPU fallback.
"""
from __future__ import annotations

import ctypes as C
import math
import os

import torch

from . import _lib

TILE_CAPACITY_DEFAULT = 1536  # scannet/cumodel.py:102


def _check(code: int, what: str) -> None:
    if code != 0:
        msgs = [_lib.strerror(bit) for bit in (1, 2, 4, 8, 16, 32, 64, 128) if code & bit]
        raise RuntimeError(f"{what}: " + "; ".join(msgs))


def _ptr(t):
    """The device (or host) address of a tensor as the bound functions take it: every pointer argument is declared
    ``c_void_p`` in ``_lib.SIGNATURES``, which converts an int or None itself."""
    return None if t is None else t.data_ptr()


def _stream(device):
    """The raw handle of torch's current stream on ``device`` (the launches of a call go there)."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    return torch._C._cuda_getCurrentRawStream(index)


def _f32c(t, name):
    if not (t.is_cuda and t.dtype == torch.float32):
        raise RuntimeError(f"{name} must be a float32 tensor on the GPU")
    return t if t.is_contiguous() else t.contiguous()


def num_tiles(W: int, H: int, TW: int, TH: int) -> int:
    return ((W + TW - 1) // TW) * ((H + TH - 1) // TH)


def prepare_primitives(positions, log_scales, quats):
    """[N,3],[N,3],[N,4] -> opaque per-primitive geometry records (uint8 [N*64])."""
    positions, log_scales, quats = _f32c(positions, "positions"), _f32c(log_scales, "log_scales"), _f32c(quats, "quats")
    n = positions.shape[0]
    rec = torch.empty(max(n, 1) * _lib.PRIM_RECORD_BYTES, dtype=torch.uint8, device=positions.device)
    code = _lib.load().mlpsp_prepare_primitives(_ptr(positions), _ptr(log_scales), _ptr(quats), n, _ptr(rec),
                                                _stream(positions.device))
    _check(code, "mlpsp_prepare_primitives")
    return rec


def normalize_rays(rays_d):
    """[B,3] float32 on the device -> unit directions, the bits of ``F.normalize(rays_d, dim=-1)`` in one launch."""
    rays_d = _f32c(rays_d, "rays_d")
    if rays_d.dim() != 2 or rays_d.shape[1] != 3:
        raise ValueError("rays_d must be [B, 3]")
    out = torch.empty_like(rays_d)
    code = _lib.load().mlpsp_normalize_rays(_ptr(rays_d), rays_d.shape[0], _ptr(out), _stream(rays_d.device))
    _check(code, "mlpsp_normalize_rays")
    return out


def frame_prologue(rays_o, rays_d, W, H, TW=8, TH=8, records=None):
    """(unit directions, tile pyramids, frame records | None) of a W x H frame in one launch: what
    :func:`normalize_rays` returns; the per-tile ray pyramids :func:`sort_tiles` takes as ``tile_pyramids``; and, with
    the geometry ``records`` of the scene, the per-primitive records it takes as ``frame_records`` (written for the
    origin of ray 0)."""
    rays_d, rays_o = _f32c(rays_d, "rays_d"), _f32c(rays_o, "rays_o")
    if rays_d.dim() != 2 or rays_d.shape[1] != 3 or rays_o.shape != rays_d.shape or rays_d.shape[0] != W * H:
        raise ValueError("rays_o and rays_d must be [W * H, 3]")
    lib = _lib.load()
    dev = rays_d.device
    unit = torch.empty_like(rays_d)
    pyramids = torch.empty(_tile_pyramids_bytes(W, H, TW, TH), dtype=torch.uint8, device=dev)
    n, frame = 0, None
    if records is not None:
        n = records.numel() // _lib.PRIM_RECORD_BYTES
        frame = torch.empty(lib.mlpsp_sort_frame_records_bytes(n), dtype=torch.uint8, device=dev)
    code = lib.mlpsp_frame_prologue(_ptr(rays_d), _ptr(unit), _ptr(rays_o), W, H, TW, TH, _ptr(pyramids), _ptr(records), n,
                                    _ptr(frame), _stream(dev))
    _check(code, "mlpsp_frame_prologue")
    return unit, pyramids, frame


_pyramid_bytes = {}


def _tile_pyramids_bytes(W, H, TW, TH):
    key = (W, H, TW, TH)
    got = _pyramid_bytes.get(key)
    if got is None:
        if len(_pyramid_bytes) > 64:
            _pyramid_bytes.clear()
        got = _pyramid_bytes[key] = _lib.load().mlpsp_tile_pyramids_bytes(W, H, TW, TH)
    return got


def validate_tile_lists(candidates, tile_offsets, n_tiles: int, capacity: int, num_primitives: int, path_name: str):
    """Raise the reference's RuntimeError texts (np_tile_kernels.cu:4578-4588) for a bad tile list."""
    for t, nm in ((candidates, "culled_prim_indices"), (tile_offsets, "tile_offsets")):
        if not (t.is_cuda and t.dtype == torch.int32 and t.dim() == 1 and t.is_contiguous()):
            raise RuntimeError(f"{path_name}: {nm} must be a contiguous CUDA int32 vector")
    if tile_offsets.numel() != n_tiles + 1:
        raise RuntimeError(f"{path_name}: tile_offsets length mismatch (got {tile_offsets.numel()}, "
                           f"expected {n_tiles + 1})")
    status_dev = torch.empty(2, dtype=torch.int32, device=candidates.device)
    status = (C.c_int32 * 2)()
    code = _lib.load().mlpsp_validate_tile_lists(_ptr(tile_offsets), _ptr(candidates), n_tiles, candidates.numel(),
                                                 int(capacity), int(num_primitives), _ptr(status_dev), status,
                                                 _stream(candidates.device))
    if code & _lib.E_OFFSETS:
        raise RuntimeError(f"{path_name}: tile_offsets must start at zero, end at the candidate-list length, "
                           "and be monotonic/in bounds")
    if code & _lib.E_CAPACITY:
        raise RuntimeError(f"{path_name}: tile candidate capacity {capacity} exceeded (maximum observed tile length "
                           f"{status[1]}); refusing to truncate or use an inconsistent forward/backward order")
    if code & _lib.E_IDS:
        raise RuntimeError(f"{path_name}: candidate primitive IDs must be in [0, num_primitives)")
    _check(code, path_name)


def bin_legacy(positions, log_scales, view_matrices, proj_matrix, W: int, H: int, tile: int, threshold: float,
               tile_view_ids=None, with_longest=False):
    """Sparse form of the reference's screen-space culling (scannet/cumodel.py:994-1070, 838-949).

    view_matrices [K,4,4] / proj_matrix [4,4] may live on any device (they are read on the host).
    Returns (culled_prim_indices int32 [P], tile_offsets int32 [T+1]); ids ascend inside a tile.
    ``with_longest`` appends the length of the longest tile list (known from the same read-back).
    """
    positions, log_scales = _f32c(positions, "positions"), _f32c(log_scales, "log_scales")
    dev = positions.device
    vm = view_matrices.detach().to("cpu", torch.float32).reshape(-1, 4, 4).contiguous()
    pm = proj_matrix.detach().to("cpu", torch.float32).reshape(4, 4).contiguous()
    K, n = vm.shape[0], positions.shape[0]
    T = num_tiles(W, H, tile, tile)
    tv = None
    if tile_view_ids is not None:
        tv = tile_view_ids.to(device=dev, dtype=torch.int32).contiguous()
        if tv.numel() != T:
            raise ValueError(f"tile_view_ids length mismatch: got {tv.numel()}, expected {T}")
    lib = _lib.load()
    # ordinary (version-counted) tensors even under torch.inference_mode(): a later in-place edit of the
    # lists must be detectable by whoever skips re-validating them
    with torch.inference_mode(False):
        offsets = torch.empty(T + 1, dtype=torch.int32, device=dev)
    fp = C.POINTER(C.c_float)
    nbytes = lib.mlpsp_bin_scratch_bytes(n, K, W, H, tile)
    counts = (C.c_int64 * 2)()
    for _ in range(6):
        scratch = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        code = lib.mlpsp_bin_legacy_count(_ptr(positions), _ptr(log_scales), n, C.cast(vm.data_ptr(), fp), K, _ptr(tv),
                                          C.cast(pm.data_ptr(), fp), W, H, tile, float(threshold), _ptr(scratch),
                                          nbytes, _ptr(offsets), counts, _stream(dev))
        if code != _lib.E_SCRATCH:
            break
        nbytes *= 4
    _check(code, "mlpsp_bin_legacy_count")
    with torch.inference_mode(False):
        cand = torch.empty(int(counts[0]), dtype=torch.int32, device=dev)
    if counts[0] > 0:
        code = lib.mlpsp_bin_legacy_fill(n, K, _ptr(tv), W, H, tile, _ptr(scratch), nbytes, _ptr(offsets), _ptr(cand),
                                         _stream(dev))
        _check(code, "mlpsp_bin_legacy_fill")
    if with_longest:
        return cand, offsets, int(counts[1])
    return cand, offsets


def _host_f32(t):
    """A contiguous float32 host tensor of `t` (itself when it already is one)."""
    if t.device.type == "cpu" and t.dtype == torch.float32 and t.is_contiguous() and not t.requires_grad:
        return t
    return t.detach().to("cpu", torch.float32).contiguous()


_scratch_bytes = {}


def _bin_scratch_bytes(n, K, W, H, tile):
    key = (n, K, W, H, tile)
    got = _scratch_bytes.get(key)
    if got is None:
        if len(_scratch_bytes) > 64:
            _scratch_bytes.clear()
        got = _scratch_bytes[key] = _lib.load().mlpsp_bin_scratch_bytes(n, K, W, H, tile)
    return got


def bin_legacy_async(positions, log_scales, view_matrices, proj_matrix, W: int, H: int, tile: int, threshold: float,
                     cand_capacity: int, tile_view_ids=None, scratch_scale: int = 1, counts=None, reuse=None):
    """:func:`bin_legacy` without any host synchronisation -> (candidates [cand_capacity], tile_offsets [T+1],
    counts int64 [4] on the device = pairs, longest tile list, level-1 entries, guard).  If guard is set the
    lists are empty: read ``counts`` at the next synchronisation, enlarge ``cand_capacity`` (pairs) or
    ``scratch_scale`` (level-1 entries) and repeat.  ``counts``: an int64 [4] device tensor to write them to (e.g. a
    view of a buffer that is read back in one copy together with other results).  ``reuse``: a dict the caller keeps
    between calls whose launches follow each other on one stream; the candidate, offset and scratch buffers are
    then allocated once and handed out again while their sizes stay the same (four allocations less between the
    end of one frame and the first launch of the next)."""
    positions, log_scales = _f32c(positions, "positions"), _f32c(log_scales, "log_scales")
    dev = positions.device
    on_device = (tile_view_ids is None and all(m.is_cuda and m.dtype == torch.float32 and m.numel() == 16 and
                                               m.is_contiguous() for m in (view_matrices, proj_matrix)))
    if on_device:               # one view, both matrices already on the device: nothing is brought to the host
        vm, pm = view_matrices, proj_matrix
        K = 1
    else:
        vm, pm = _host_f32(view_matrices).reshape(-1, 4, 4), _host_f32(proj_matrix).reshape(4, 4)
        K = vm.shape[0]
    n = positions.shape[0]
    T = num_tiles(W, H, tile, tile)
    tv = None
    if tile_view_ids is not None:
        tv = tile_view_ids.to(device=dev, dtype=torch.int32).contiguous()
        if tv.numel() != T:
            raise ValueError(f"tile_view_ids length mismatch: got {tv.numel()}, expected {T}")
    lib = _lib.load()
    fp = C.POINTER(C.c_float)
    nbytes = _bin_scratch_bytes(n, K, W, H, tile) * int(scratch_scale)
    held = reuse.get("bin") if reuse is not None else None
    if held is not None and held[0] == (T, int(cand_capacity), nbytes, dev):
        offsets, cand, scratch = held[1]
    else:
        with torch.inference_mode(False):
            offsets = torch.empty(T + 1, dtype=torch.int32, device=dev)
            cand = torch.empty(int(cand_capacity), dtype=torch.int32, device=dev)
        scratch = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        if reuse is not None:
            reuse["bin"] = ((T, int(cand_capacity), nbytes, dev), (offsets, cand, scratch))
    if counts is None:
        counts = torch.empty(4, dtype=torch.int64, device=dev)
    elif not (counts.is_cuda and counts.dtype == torch.int64 and counts.numel() == 4 and counts.is_contiguous()):
        raise ValueError("counts must be a contiguous int64 [4] tensor on the device")
    if on_device:
        code = lib.mlpsp_bin_legacy_async_device_matrices(_ptr(positions), _ptr(log_scales), n, _ptr(vm), _ptr(pm), W, H,
                                                          tile, float(threshold), _ptr(scratch), nbytes, _ptr(offsets),
                                                          _ptr(cand), int(cand_capacity), _ptr(counts), _stream(dev))
    else:
        code = lib.mlpsp_bin_legacy_async(_ptr(positions), _ptr(log_scales), n, C.cast(vm.data_ptr(), fp), K, _ptr(tv),
                                          C.cast(pm.data_ptr(), fp), W, H, tile, float(threshold), _ptr(scratch), nbytes,
                                          _ptr(offsets), _ptr(cand), int(cand_capacity), _ptr(counts), _stream(dev))
    _check(code, "mlpsp_bin_legacy_async")
    return cand, offsets, counts


def bin_segments_async(positions, log_scales, view_matrix, proj_matrix, W: int, H: int, tile: int, threshold: float,
                       stride: int = TILE_CAPACITY_DEFAULT, scratch_scale: int = 1, counts=None, reuse=None):
    """The lists of :func:`bin_legacy_async` for one view (both matrices float32 device tensors of 16 elements) in
    segments of ``stride`` entries per tile, without any host synchronisation and without a count of the candidates
    before they are written -> (candidates [T * stride], tile_offsets [T + 1] = t * stride, tile_ends [T], counts
    int64 [4] on the device = 0, the longest list if one exceeds ``stride`` (else 0), level-1 entries, guard).  Tile
    t's list -- the same ids in the same order -- is ``candidates[tile_offsets[t]:tile_ends[t]]``; a list longer
    than ``stride`` keeps its first ``stride`` entries.  :func:`sort_tiles` and :func:`render_tilecenter_mfma` take
    such lists with ``tile_ends``.  ``counts``, ``reuse``: as in :func:`bin_legacy_async`."""
    positions, log_scales = _f32c(positions, "positions"), _f32c(log_scales, "log_scales")
    dev = positions.device
    for m in (view_matrix, proj_matrix):
        if not (m.is_cuda and m.dtype == torch.float32 and m.numel() == 16 and m.is_contiguous()):
            raise ValueError("view_matrix and proj_matrix must be contiguous float32 device tensors of 16 elements")
    n = positions.shape[0]
    T = num_tiles(W, H, tile, tile)
    stride = int(stride)
    if stride <= 0 or T * stride > 2**31 - 1:
        raise ValueError(f"segment stride {stride} does not fit {T} tiles")
    lib = _lib.load()
    nbytes = _bin_scratch_bytes(n, 1, W, H, tile) * int(scratch_scale)
    held = reuse.get("segments") if reuse is not None else None
    if held is not None and held[0] == (T, stride, nbytes, dev):
        offsets, ends, cand, scratch = held[1]
    else:
        with torch.inference_mode(False):
            offsets = torch.empty(T + 1, dtype=torch.int32, device=dev)
            ends = torch.empty(T, dtype=torch.int32, device=dev)
            cand = torch.empty(T * stride, dtype=torch.int32, device=dev)
        scratch = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        if reuse is not None:
            reuse["segments"] = ((T, stride, nbytes, dev), (offsets, ends, cand, scratch))
    if counts is None:
        counts = torch.empty(4, dtype=torch.int64, device=dev)
    elif not (counts.is_cuda and counts.dtype == torch.int64 and counts.numel() == 4 and counts.is_contiguous()):
        raise ValueError("counts must be a contiguous int64 [4] tensor on the device")
    code = lib.mlpsp_bin_segments_async_device_matrices(_ptr(positions), _ptr(log_scales), n, _ptr(view_matrix),
                                                        _ptr(proj_matrix), W, H, tile, float(threshold), _ptr(scratch),
                                                        nbytes, stride, _ptr(offsets), _ptr(ends), _ptr(cand),
                                                        _ptr(counts), _stream(dev))
    _check(code, "mlpsp_bin_segments_async_device_matrices")
    return cand, offsets, ends, counts


def compact_segments(order, tile_offsets, tile_ends):
    """(lists, offsets [T + 1]) of segment lists written one after the other (torch; for the rare caller that needs
    the reference's layout of lists that came in segments)."""
    starts = tile_offsets[:-1].long()
    lengths = tile_ends.long() - starts
    offsets = torch.zeros(starts.numel() + 1, dtype=torch.int64, device=order.device)
    offsets[1:] = torch.cumsum(lengths, 0)
    total = int(offsets[-1].item())
    tile_of = torch.repeat_interleave(torch.arange(starts.numel(), device=order.device), lengths, output_size=total)
    within = torch.arange(total, device=order.device) - offsets[:-1][tile_of]
    return order[starts[tile_of] + within].contiguous(), offsets.to(torch.int32)


def sort_tiles(rays_o, rays_d, records, candidates, tile_offsets, W, H, TW, TH, family=_lib.KEY_TSTAR,
               capacity=TILE_CAPACITY_DEFAULT, want_keys=False, cull_threshold=0.0, frame_records=None,
               tile_pyramids=None, tile_ends=None, ids_ascend=False):
    """Materialised per-tile depth order: (sorted_ids [P], sorted_keys [P] | None).

    With ``cull_threshold`` (the render's score threshold) candidates that provably hit no ray of their
    tile come back as ``~id``; the render kernels skip them, the image is unchanged.  ``frame_records``: the records
    :func:`frame_prologue` wrote for these rays and primitives (a fifth fewer vector instructions in the sort; keys
    and order do not depend on it), or True to let this call write them first (one more launch, which on one MI355X
    costs a frame more than the sort kernel gains), or False.  None = what ``MLPSP_SORT_FRAME_RECORDS`` says, off
    unless it is 1.  ``tile_pyramids``: what :func:`frame_prologue` returned for these rays and this tile size (the
    culling's per-tile planes, which the sort otherwise builds in every wavefront of a tile; same output).
    ``tile_ends``: the int32 [T] ends of lists that lie in segments (:func:`bin_segments_async`); the sorted lists
    come back in the same places, what lies between them is not written.  ``ids_ascend``: the caller vouches that
    the ids of every list ascend, as the binning entry points write them (same output, no gather of the ids at the
    end; lists in any other order must leave it False)."""
    dev = rays_o.device
    if tile_ends is not None and not (tile_ends.is_cuda and tile_ends.dtype == torch.int32 and tile_ends.is_contiguous()
                                      and tile_ends.numel() == tile_offsets.numel() - 1):
        raise ValueError("tile_ends must be a contiguous int32 device tensor with one entry per tile")
    sorted_ids = torch.empty_like(candidates)
    keys = torch.empty(candidates.numel(), dtype=torch.float32, device=dev) if want_keys else None
    if candidates.numel() == 0:
        return sorted_ids, keys
    num_primitives = records.numel() // _lib.PRIM_RECORD_BYTES
    lib = _lib.load()
    scratch, ready = None, 0
    if frame_records is None:
        frame_records = os.environ.get("MLPSP_SORT_FRAME_RECORDS", "0") == "1"
    if torch.is_tensor(frame_records):
        if not (frame_records.is_cuda and frame_records.dtype == torch.uint8 and frame_records.is_contiguous()
                and frame_records.numel() == lib.mlpsp_sort_frame_records_bytes(num_primitives)):
            raise ValueError("frame_records must be the uint8 buffer frame_prologue() returned for these primitives")
        scratch, ready = frame_records, 1
    elif frame_records:
        scratch = torch.empty(lib.mlpsp_sort_frame_records_bytes(num_primitives), dtype=torch.uint8, device=dev)
    if tile_pyramids is not None and not (tile_pyramids.is_cuda and tile_pyramids.dtype == torch.uint8
                                          and tile_pyramids.is_contiguous()
                                          and tile_pyramids.numel() == _tile_pyramids_bytes(W, H, TW, TH)):
        raise ValueError("tile_pyramids must be the uint8 buffer frame_prologue() returned for this frame and tile size")
    code = lib.mlpsp_sort_tiles(_ptr(rays_o), _ptr(rays_d), _ptr(records), num_primitives, _ptr(candidates),
                                _ptr(tile_offsets), W, H, TW, TH, int(family), int(capacity), float(cull_threshold),
                                _ptr(scratch), ready, _ptr(tile_pyramids), _ptr(tile_ends), int(bool(ids_ascend)),
                                _ptr(sorted_ids), _ptr(keys), _stream(dev))
    _check(code, "mlpsp_sort_tiles")
    return sorted_ids, keys


def render_tilecenter_f32(rays_o, rays_d, records, order, tile_offsets, freq, att, W1, b1, W2, b2, W3, b3, W, H, TW,
                          TH, threshold, with_t=False, counters=None):
    """Scalar-f32 tile-centre forward over materialised per-tile orders -> (rgb, alpha, t|None)."""
    dev = rays_o.device
    B = W * H
    rgb = torch.empty(B, 3, dtype=torch.float32, device=dev)
    alpha = torch.empty(B, 1, dtype=torch.float32, device=dev)
    t = torch.empty(B, 1, dtype=torch.float32, device=dev) if with_t else None
    n, hidden, F = W1.shape[0], W2.shape[1], freq.shape[0]
    code = _lib.load().mlpsp_render_tilecenter_f32(
        _ptr(rays_o), _ptr(rays_d), _ptr(records), _ptr(order), _ptr(tile_offsets), _ptr(freq), _ptr(att), F,
        _ptr(W1), _ptr(b1), _ptr(W2), _ptr(b2), _ptr(W3), _ptr(b3), n, hidden, W, H, TW, TH, float(threshold),
        _ptr(rgb), _ptr(alpha), _ptr(t), _ptr(counters), _stream(dev))
    _check(code, "mlpsp_render_tilecenter_f32")
    return rgb, alpha, t


def radius_multiplier(threshold: float) -> float:
    return math.sqrt(-2.0 * math.log(threshold))


def render_tilecenter_stats_f32(rays_o, rays_d, records, order, tile_offsets, freq, att, W1, b1, W2, b2, W3, b3, W, H,
                                TW, TH, threshold, gt_rgb, stat_sum_w, stat_max_w, stat_hits, stat_sum_werr=None,
                                stat_contrib=None):
    """Scalar-f32 tile-centre forward that also accumulates the five pruning statistics in place -> (rgb, alpha)."""
    dev = rays_o.device
    B = W * H
    rgb = torch.empty(B, 3, dtype=torch.float32, device=dev)
    alpha = torch.empty(B, 1, dtype=torch.float32, device=dev)
    n, hidden, F = W1.shape[0], W2.shape[1], freq.shape[0]
    code = _lib.load().mlpsp_render_tilecenter_stats_f32(
        _ptr(rays_o), _ptr(rays_d), _ptr(records), _ptr(order), _ptr(tile_offsets), _ptr(freq), _ptr(att), F,
        _ptr(W1), _ptr(b1), _ptr(W2), _ptr(b2), _ptr(W3), _ptr(b3), n, hidden, W, H, TW, TH, float(threshold),
        _ptr(gt_rgb), _ptr(rgb), _ptr(alpha), _ptr(stat_sum_w), _ptr(stat_max_w), _ptr(stat_hits),
        _ptr(stat_sum_werr), _ptr(stat_contrib), _stream(dev))
    _check(code, "mlpsp_render_tilecenter_stats_f32")
    return rgb, alpha


def training_records(rays_o, rays_d, records, order, tile_offsets, freq, att, W1, b1, W2, b2, W3, b3, W, H, TW, TH,
                     threshold, beta, temp, max_hits, path_name="render_tiles_training_records", render_order=False,
                     counts_only=False):
    """Training-records forward -> (rgb, alpha, ids, x6, raw, masks, gates, offsets int64 [B+1]);
    raises the reference's hit-capacity error (np_tile_kernels.cu:4601-4609).  ``render_order``: layer 2 rounded as
    the render kernels round it, which makes image and records those of the f32 render bit for bit."""
    dev = rays_o.device
    lib = _lib.load()
    B = W * H
    n, hidden, F = W1.shape[0], W2.shape[1], freq.shape[0]
    counts = torch.zeros(B, dtype=torch.int32, device=dev)
    overflow = torch.empty(1, dtype=torch.int32, device=dev)
    head = (_ptr(rays_o), _ptr(rays_d), _ptr(records), _ptr(order), _ptr(tile_offsets), _ptr(freq), _ptr(att), F,
            _ptr(W1), _ptr(b1), _ptr(W2), _ptr(b2), _ptr(W3), _ptr(b3), n, hidden, W, H, TW, TH, float(threshold),
            int(max_hits), 1 if render_order else 0)

    def refuse():
        raise RuntimeError(f"{path_name}: tile-center backward hit capacity {int(max_hits)} reached before "
                           "transmittance termination; refusing to return truncated gradients")

    _check(lib.mlpsp_records_count(*head, _ptr(counts), _ptr(overflow), _stream(dev)), "mlpsp_records_count")
    offsets = torch.zeros(B + 1, dtype=torch.int64, device=dev)
    torch.cumsum(counts, 0, out=offsets[1:])
    total, over = int(offsets[-1].item()), int(overflow.item())
    if over:
        refuse()
    if counts_only:
        return counts
    ids = torch.empty(total, dtype=torch.int32, device=dev)
    x6 = torch.empty(total, 6, dtype=torch.float32, device=dev)
    masks = torch.empty(total, 2, dtype=torch.int32, device=dev)
    raw = torch.empty(total, 8, dtype=torch.float32, device=dev)
    gates = torch.empty(total, 4, dtype=torch.float32, device=dev)
    rgb = torch.zeros(B, 3, dtype=torch.float32, device=dev)
    alpha = torch.zeros(B, 1, dtype=torch.float32, device=dev)
    if total:
        _check(lib.mlpsp_records_emit(*head, float(beta), float(temp), _ptr(offsets), _ptr(ids), _ptr(x6), _ptr(masks),
                                      _ptr(raw), _ptr(gates), _ptr(rgb), _ptr(alpha), _ptr(overflow), _stream(dev)),
               "mlpsp_records_emit")
    return rgb, alpha, ids, x6, raw, masks, gates, offsets


def all_finite_flag(tensors):
    """int32 device flag [1]: 1 if any element of the float32 tensors (at most 16, one device) is NaN or infinite.
    One fused scan; reading the flag is the caller's (single) synchronisation."""
    tensors = [t for t in tensors if t.numel()]
    dev = tensors[0].device if tensors else torch.device("cuda", torch.cuda.current_device())
    flag = torch.empty(1, dtype=torch.int32, device=dev)
    for t in tensors:
        if not (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.device == dev):
            raise RuntimeError("all_finite_flag expects contiguous float32 CUDA tensors on one device")
    pointers = (C.c_void_p * max(len(tensors), 1))(*[t.data_ptr() for t in tensors])
    lengths = (C.c_int64 * max(len(tensors), 1))(*[t.numel() for t in tensors])
    _check(_lib.load().mlpsp_all_finite(pointers, lengths, len(tensors), _ptr(flag), _stream(dev)), "mlpsp_all_finite")
    return flag


def training_records_mfma(rays_o, rays_d, records, order, tile_offsets, freq, att, packed, n, W, H, threshold, beta,
                          temp, max_hits, bf16):
    """Matrix-core training-records forward -> (status bits, (rgb, alpha, ids, x6, raw, masks, gates, offsets) or
    None).  Bits: 1 numeric, 2 hit capacity, 4 count/emit disagreement (training_wmma.cuh:21-22); the policy --
    retry in f32, raise -- is the caller's.  A non-zero status after the count step skips the emit step."""
    dev = rays_o.device
    lib = _lib.load()
    B = W * H
    counts = torch.zeros(B, dtype=torch.int32, device=dev)
    status = torch.zeros(1, dtype=torch.int32, device=dev)
    head = (_ptr(rays_o), _ptr(rays_d), _ptr(records), _ptr(order), _ptr(tile_offsets), _ptr(freq), _ptr(att),
            _ptr(packed), int(n), W, H, float(threshold), int(max_hits), 1 if bf16 else 0)
    _check(lib.mlpsp_records_mfma_count(*head, _ptr(counts), _ptr(status), _stream(dev)), "mlpsp_records_mfma_count")
    offsets = torch.zeros(B + 1, dtype=torch.int64, device=dev)
    torch.cumsum(counts, 0, out=offsets[1:])
    total, bits = torch.cat([offsets[-1:], status.to(torch.int64)]).tolist()
    if bits:
        return int(bits), None
    if not 0 <= total <= B * int(max_hits):
        raise RuntimeError("Training WMMA count total is outside the bounded allocation contract")
    ids = torch.empty(total, dtype=torch.int32, device=dev)
    x6 = torch.empty(total, 6, dtype=torch.float32, device=dev)
    masks = torch.empty(total, 2, dtype=torch.int32, device=dev)
    raw = torch.empty(total, 8, dtype=torch.float32, device=dev)
    gates = torch.empty(total, 4, dtype=torch.float32, device=dev)
    rgb = torch.zeros(B, 3, dtype=torch.float32, device=dev)
    alpha = torch.zeros(B, 1, dtype=torch.float32, device=dev)
    # launched for an empty record set too: the emit step then checks that every pixel's count is zero
    _check(lib.mlpsp_records_mfma_emit(*head, float(beta), float(temp), _ptr(offsets), int(total), _ptr(ids), _ptr(x6),
                                       _ptr(masks), _ptr(raw), _ptr(gates), _ptr(rgb), _ptr(alpha), _ptr(status),
                                       _stream(dev)), "mlpsp_records_mfma_emit")
    return int(status.item()), (rgb, alpha, ids, x6, raw, masks, gates, offsets)


def _feat_shape(feat_attr, allow_half=False):
    """(slots, channels) with the reference's checks (np_tile_kernels.cu:6158-6169).  ``allow_half``: attributes
    stored as fp16 (an inference export) are accepted by the matrix-core path, which reads them as they are."""
    dtypes = (torch.float32, torch.float16) if allow_half else (torch.float32,)
    if not (feat_attr.is_cuda and feat_attr.dtype in dtypes and feat_attr.dim() in (2, 3)):
        raise RuntimeError("feat_attr must be a float32 CUDA tensor of 2 or 3 dimensions")
    if feat_attr.dim() == 2:
        slots, ch = 1, feat_attr.shape[1]
    else:
        slots, ch = feat_attr.shape[1], feat_attr.shape[2]
        if slots not in (4, 5):
            raise RuntimeError("3D feat_attr expects slots in {4,5}")
    if ch <= 0:
        raise RuntimeError("feat_attr feature dimension must be positive")
    if ch > 512:
        raise RuntimeError("feat_attr feature dimension must be <= 512")
    return int(slots), int(ch)


def _feat_pool_sizes(pairs: int):
    """Record-pool sizes to try in turn: a quarter of the candidates (at the 200k-primitive benchmark scene
    8 % of them hit before their tile saturates), then the worst case, which cannot run out."""
    first = max(pairs // 4, 1 << 16)
    return (first, -1) if first < pairs else (-1,)


def render_tilecenter_feat_f32(rays_o, rays_d, records, order, tile_offsets, freq, att, W1, b1, W2, b2, W3, b3,
                               feat_attr, beta, temp, W, H, TW, TH, threshold):
    """Scalar-f32 tile-centre forward with the gated feature channel -> (rgb, alpha, feat [B,C])."""
    dev = rays_o.device
    slots, ch = _feat_shape(feat_attr)
    B = W * H
    lib = _lib.load()
    rgb = torch.empty(B, 3, dtype=torch.float32, device=dev)
    alpha = torch.empty(B, 1, dtype=torch.float32, device=dev)
    feat = torch.empty(B, ch, dtype=torch.float32, device=dev)
    status = torch.empty(1, dtype=torch.int32, device=dev)
    n, hidden, F = W1.shape[0], W2.shape[1], freq.shape[0]
    pairs = int(order.numel())
    for pool in _feat_pool_sizes(pairs):
        nbytes = lib.mlpsp_feat_workspace_bytes(pairs, W, H, TW, TH, slots, 0, pool)
        if nbytes == 0:
            raise RuntimeError("mlpsp_feat_workspace_bytes: bad arguments")
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        code = lib.mlpsp_render_tilecenter_feat_f32(
            _ptr(rays_o), _ptr(rays_d), _ptr(records), _ptr(order), _ptr(tile_offsets), _ptr(freq), _ptr(att), F,
            _ptr(W1), _ptr(b1), _ptr(W2), _ptr(b2), _ptr(W3), _ptr(b3), n, hidden, _ptr(feat_attr), slots, ch,
            float(beta), float(temp), W, H, TW, TH, float(threshold), pairs, _ptr(workspace), nbytes, _ptr(rgb),
            _ptr(alpha), _ptr(feat), _ptr(status), _stream(dev))
        _check(code, "mlpsp_render_tilecenter_feat_f32")
        if pool < 0 or int(status.item()) == 0:
            break
    return rgb, alpha, feat


def render_per_pixel_f32(rays_o, rays_d, records, candidates, tile_offsets, freq, att, W1, b1, W2, b2, W3, b3, W, H,
                         TW, TH, threshold, path_name, feat_attr=None, beta=1.5, temp=2.0):
    """Per-pixel-order forward -> (rgb, alpha, feat|None); raises the reference's overflow error."""
    dev = rays_o.device
    lib = _lib.load()
    B = W * H
    slots, ch = _feat_shape(feat_attr) if feat_attr is not None else (0, 0)
    rgb = torch.empty(B, 3, dtype=torch.float32, device=dev)
    alpha = torch.empty(B, 1, dtype=torch.float32, device=dev)
    feat = torch.empty(B, ch, dtype=torch.float32, device=dev) if feat_attr is not None else None
    nbytes = lib.mlpsp_per_pixel_workspace_bytes(W, H, TW, TH)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    n, hidden, F = W1.shape[0], W2.shape[1], freq.shape[0]
    code = lib.mlpsp_render_per_pixel_f32(
        _ptr(rays_o), _ptr(rays_d), _ptr(records), _ptr(candidates), _ptr(tile_offsets), _ptr(freq), _ptr(att), F,
        _ptr(W1), _ptr(b1), _ptr(W2), _ptr(b2), _ptr(W3), _ptr(b3), n, hidden, _ptr(feat_attr), slots, ch,
        float(beta), float(temp), W, H, TW, TH, float(threshold), _ptr(ws), nbytes, _ptr(rgb), _ptr(alpha),
        _ptr(feat), _stream(dev))
    if code & _lib.E_PIXEL_OVERFLOW:
        raise RuntimeError(f"{path_name}: per-pixel intersection capacity {_lib.PIXEL_HIT_CAPACITY} exceeded; "
                           "refusing to return a silently truncated result")
    _check(code, path_name)
    return rgb, alpha, feat


def records_per_pixel(rays_o, rays_d, records, candidates, tile_offsets, freq, att, W1, b1, W2, b2, W3, b3, W, H, TW,
                      TH, threshold, beta, temp, path_name, counts_only=False):
    """Training records in per-pixel order -> (rgb, alpha, ids, x6, raw, masks, gates, offsets int64 [B+1]), or the
    per-pixel counts (int32 [B]) alone; raises the reference's per-pixel overflow error."""
    dev = rays_o.device
    lib = _lib.load()
    B = W * H
    n, hidden, F = W1.shape[0], W2.shape[1], freq.shape[0]
    nbytes = lib.mlpsp_per_pixel_workspace_bytes(W, H, TW, TH)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    head = (_ptr(rays_o), _ptr(rays_d), _ptr(records), _ptr(candidates), _ptr(tile_offsets), _ptr(freq), _ptr(att), F,
            _ptr(W1), _ptr(b1), _ptr(W2), _ptr(b2), _ptr(W3), _ptr(b3), n, hidden)

    def check(code, what):
        if code & _lib.E_PIXEL_OVERFLOW:
            raise RuntimeError(f"{path_name}: per-pixel intersection capacity {_lib.PIXEL_HIT_CAPACITY} exceeded; "
                               "refusing to return a silently truncated result")
        _check(code, what)

    counts = torch.zeros(B, dtype=torch.int32, device=dev)
    check(lib.mlpsp_records_per_pixel_count(*head, W, H, TW, TH, float(threshold), _ptr(ws), nbytes, _ptr(counts),
                                            _stream(dev)), "mlpsp_records_per_pixel_count")
    if counts_only:
        return counts
    offsets = torch.zeros(B + 1, dtype=torch.int64, device=dev)
    torch.cumsum(counts, 0, out=offsets[1:])
    total = int(offsets[-1].item())
    ids = torch.empty(total, dtype=torch.int32, device=dev)
    x6 = torch.empty(total, 6, dtype=torch.float32, device=dev)
    masks = torch.empty(total, 2, dtype=torch.int32, device=dev)
    raw = torch.empty(total, 8, dtype=torch.float32, device=dev)
    gates = torch.empty(total, 4, dtype=torch.float32, device=dev)
    rgb = torch.zeros(B, 3, dtype=torch.float32, device=dev)
    alpha = torch.zeros(B, 1, dtype=torch.float32, device=dev)
    check(lib.mlpsp_records_per_pixel_emit(*head, float(beta), float(temp), W, H, TW, TH, float(threshold), _ptr(ws),
                                           nbytes, _ptr(offsets), total, _ptr(ids), _ptr(x6), _ptr(masks), _ptr(raw),
                                           _ptr(gates), _ptr(rgb), _ptr(alpha), _stream(dev)),
          "mlpsp_records_per_pixel_emit")
    return rgb, alpha, ids, x6, raw, masks, gates, offsets


def pack_mfma_weights(W1, b1, W2, b2, W3, b3, bf16=True):
    """Weights of the 72->32->32->4 MLP in matrix-core operand order (uint8 [N*7808]); once per scene."""
    n = W1.shape[0]
    if tuple(W1.shape[1:]) != (32, 72) or tuple(W2.shape[1:]) != (32, 32) or tuple(W3.shape[1:]) != (4, 32):
        raise RuntimeError("the matrix-core path supports the 72->32->32->4 MLP only")
    lib = _lib.load()
    packed = torch.empty(lib.mlpsp_mfma_pack_bytes(n), dtype=torch.uint8, device=W1.device)
    if all(w.is_cuda and w.dtype == torch.float16 for w in (W1, b1, W2, b2, W3, b3)):
        # stored as fp16 (an inference export): packed straight from that storage, no f32 copy in between
        ws = [w.contiguous() for w in (W1, b1, W2, b2, W3, b3)]
        code = lib.mlpsp_pack_mfma_weights_half(*[_ptr(w) for w in ws], n, int(bool(bf16)), _ptr(packed),
                                                _stream(W1.device))
    else:
        ws = [_f32c(w, "weights") for w in (W1, b1, W2, b2, W3, b3)]
        code = lib.mlpsp_pack_mfma_weights(*[_ptr(w) for w in ws], n, int(bool(bf16)), _ptr(packed), _stream(W1.device))
    _check(code, "mlpsp_pack_mfma_weights")
    return packed


def render_tilecenter_mfma(rays_o, rays_d, records, order, tile_offsets, freq, att, W1, b1, W2, b2, W3, b3, W, H,
                           threshold, bf16=True, counters=None, packed=None, check=True, status=None,
                           status_is_clear=False, tile_ends=None):
    """Matrix-core tile-centre forward (8x8 tiles) -> (rgb, alpha, nonfinite).

    ``nonfinite`` is a bool when ``check`` (one 4-byte readback) or the int32 device flag otherwise.  ``status``: an
    int32 [16] device tensor for the flag words (word 0 = non-finite), allocated here when omitted.
    ``status_is_clear``: the caller read all 16 words of ``status`` back as zero after the previous call that used
    it, so no clear is queued in front of the kernel.  ``tile_ends``: as in :func:`sort_tiles`.
    """
    dev = rays_o.device
    if freq.numel() != 6:
        raise RuntimeError("the matrix-core path supports 6 frequencies only")
    if packed is None:
        packed = pack_mfma_weights(W1, b1, W2, b2, W3, b3, bf16)
    B = W * H
    rgb = torch.empty(B, 3, dtype=torch.float32, device=dev)
    alpha = torch.empty(B, 1, dtype=torch.float32, device=dev)
    flag = status if status is not None else torch.empty(16, dtype=torch.int32, device=dev)
    if not (flag.is_cuda and flag.dtype == torch.int32 and flag.numel() == 16 and flag.is_contiguous()):
        raise ValueError("status must be a contiguous int32 [16] tensor on the device")
    if (status_is_clear and status is not None) or tile_ends is not None:
        # (the RGB entry point is the feature entry point without features; only that one takes the stage word and
        # the ends of lists in segments)
        stage = _lib.STAGE_STATUS_IS_CLEAR if (status_is_clear and status is not None) else 0
        code = _lib.load().mlpsp_render_tilecenter_mfma_feat(
            _ptr(rays_o), _ptr(rays_d), _ptr(records), _ptr(order), _ptr(tile_offsets), 0, _ptr(freq), _ptr(att),
            _ptr(packed), W1.shape[0], int(bool(bf16)), None, 0, 0, 0.0, 0.0, W, H, float(threshold), None, 0, _ptr(rgb),
            _ptr(alpha), None, _ptr(flag), _ptr(counters), stage, _ptr(tile_ends), _stream(dev))
    else:
        code = _lib.load().mlpsp_render_tilecenter_mfma(
            _ptr(rays_o), _ptr(rays_d), _ptr(records), _ptr(order), _ptr(tile_offsets), _ptr(freq), _ptr(att),
            _ptr(packed), W1.shape[0], int(bool(bf16)), W, H, float(threshold), _ptr(rgb), _ptr(alpha), _ptr(flag),
            _ptr(counters), _stream(dev))
    _check(code, "mlpsp_render_tilecenter_mfma")
    return rgb, alpha, (bool(flag[0].item()) if check else flag)


def pack_mfma_feat(feat_attr):
    """fp16 matrix-core operand copy of the feature attributes -> (packed uint8 tensor, nonfinite flag)."""
    dev = feat_attr.device
    slots, ch = _feat_shape(feat_attr, allow_half=True)
    lib = _lib.load()
    n = feat_attr.shape[0]
    packed = torch.empty(lib.mlpsp_mfma_feat_pack_bytes(n, slots, ch), dtype=torch.uint8, device=dev)
    flag = torch.empty(1, dtype=torch.int32, device=dev)
    entry = lib.mlpsp_pack_mfma_feat_half if feat_attr.dtype == torch.float16 else lib.mlpsp_pack_mfma_feat
    feat_attr = feat_attr.contiguous()
    _check(entry(_ptr(feat_attr), n, slots, ch, _ptr(packed), _ptr(flag), _stream(dev)), "mlpsp_pack_mfma_feat")
    return packed, bool(flag.item())


def render_tilecenter_mfma_feat(rays_o, rays_d, records, order, tile_offsets, freq, att, W1, b1, W2, b2, W3, b3,
                                feat_attr, beta, temp, W, H, threshold, bf16=True, packed=None, packed_feat=None,
                                check=True, status=None, counters=None, stages=None, status_is_clear=False,
                                tile_ends=None):
    """Matrix-core tile-centre forward with the gated feature channel -> (rgb, alpha, feat, nonfinite).
    ``packed_feat`` is the result of :func:`pack_mfma_feat` for ``feat_attr`` (built here when omitted;
    non-finite rounded attributes raise).  ``status`` (an int32 [16] device tensor): ONE attempt with the first
    record-pool size and no read-back -- word 0 = non-finite, word 1 = the pool ran out (the feature image is then
    incomplete and the caller repeats the call without ``status``); returns (rgb, alpha, feat, status).
    ``counters``: int64 [4] work counters of the render launch, accumulated.  ``stages``: a callable
    ``stages(which)`` invoked before the render launch (1), before the feature product (2) and after it (3) -- the
    two launches are then queued by separate calls, with the worst-case record pool, so that a caller can bracket
    each with events.  ``status_is_clear``: as in :func:`render_tilecenter_mfma` (with ``status`` only).
    ``tile_ends``: as in :func:`sort_tiles` (the record pool is then sized by the segments' total length)."""
    dev = rays_o.device
    if freq.numel() != 6:
        raise RuntimeError("the matrix-core path supports 6 frequencies only")
    slots, ch = _feat_shape(feat_attr, allow_half=True)
    if packed is None:
        packed = pack_mfma_weights(W1, b1, W2, b2, W3, b3, bf16)
    if packed_feat is None:
        packed_feat, bad = pack_mfma_feat(feat_attr)
        if bad:
            raise RuntimeError("feature attributes are not finite in fp16")
    lib = _lib.load()
    B = W * H
    pairs = int(order.numel())
    rgb = torch.empty(B, 3, dtype=torch.float32, device=dev)
    alpha = torch.empty(B, 1, dtype=torch.float32, device=dev)
    feat = torch.empty(B, ch, dtype=torch.float32, device=dev)
    if status is not None and not (status.is_cuda and status.dtype == torch.int32 and status.numel() == 16
                                   and status.is_contiguous()):
        raise ValueError("status must be a contiguous int32 [16] tensor on the device")
    flag = status if status is not None else torch.empty(16, dtype=torch.int32, device=dev)
    clear_bit = _lib.STAGE_STATUS_IS_CLEAR if (status_is_clear and status is not None and stages is None) else 0
    def launch(workspace, ws_bytes, stage):
        code = lib.mlpsp_render_tilecenter_mfma_feat(
            _ptr(rays_o), _ptr(rays_d), _ptr(records), _ptr(order), _ptr(tile_offsets), pairs, _ptr(freq), _ptr(att),
            _ptr(packed), W1.shape[0], int(bool(bf16)), _ptr(packed_feat), slots, ch, float(beta), float(temp), W, H,
            float(threshold), _ptr(workspace), ws_bytes, _ptr(rgb), _ptr(alpha), _ptr(feat), _ptr(flag), _ptr(counters),
            stage | clear_bit, _ptr(tile_ends), _stream(dev))
        _check(code, "mlpsp_render_tilecenter_mfma_feat")
        return code

    if stages is not None:
        ws_bytes = lib.mlpsp_feat_workspace_bytes(pairs, W, H, 8, 8, slots, 1, -1)
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        stages(1)
        launch(workspace, ws_bytes, 1)
        stages(2)
        launch(workspace, ws_bytes, 2)
        stages(3)
        return rgb, alpha, feat, (bool(flag[0].item()) if check else flag)
    for pool in _feat_pool_sizes(pairs):
        ws_bytes = lib.mlpsp_feat_workspace_bytes(pairs, W, H, 8, 8, slots, 1, pool)
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        code = launch(workspace, ws_bytes, 0)
        if status is not None:
            return rgb, alpha, feat, status
        if pool < 0:
            break
        host_flag = flag[:2].tolist()               # one read-back: [non-finite, pool ran out]
        if host_flag[1] == 0:
            return rgb, alpha, feat, (bool(host_flag[0]) if check else flag)
    _check(code, "mlpsp_render_tilecenter_mfma_feat")
    return rgb, alpha, feat, (bool(flag[0].item()) if check else flag)


def records_reverse(ids, offsets, x6, raw, log_scales, quats, grad_rgb, grad_t):
    """Reverse compositing over saved records -> (d4 [R,4], grad_positions, grad_log_scales, grad_quats)."""
    dev = ids.device
    total, pixels, n = ids.numel(), grad_rgb.shape[0], log_scales.shape[0]
    d4 = torch.empty((total, 4), dtype=torch.float32, device=dev)
    gp, gs = torch.empty_like(log_scales), torch.empty_like(log_scales)
    gq = torch.empty_like(quats)
    with torch.cuda.device(dev):
        _check(_lib.load().mlpsp_records_reverse(_ptr(ids), _ptr(offsets), _ptr(x6), _ptr(raw), _ptr(log_scales),
                                                 _ptr(quats), _ptr(grad_rgb), _ptr(grad_t), pixels, n, _ptr(d4), _ptr(gp),
                                                 _ptr(gs), _ptr(gq), _stream(dev)), "mlpsp_records_reverse")
    return d4, gp, gs, gq


def records_reverse_adjoints(ids, offsets, raw, grad_rgb, grad_t):
    """(d4 [R,4], falloff_adjoint [R]) of the reverse walk, without the atomic geometry sums."""
    dev = ids.device
    d4 = torch.empty((ids.numel(), 4), dtype=torch.float32, device=dev)
    adj = torch.empty(ids.numel(), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        _check(_lib.load().mlpsp_records_reverse_adjoints(_ptr(ids), _ptr(offsets), _ptr(raw), _ptr(grad_rgb), _ptr(grad_t),
                                                          grad_rgb.shape[0], _ptr(d4), _ptr(adj), _stream(dev)),
               "mlpsp_records_reverse_adjoints")
    return d4, adj


def geometry_gradients(csr_offsets, record_indices, x6_sorted, falloff_adjoint, log_scales, quats, groups):
    """(grad_positions, grad_log_scales, grad_quats) from records in primitive-major order; ``groups`` is the
    segment layout of primitive_gemm.prepare_groups for the same CSR."""
    dev = log_scales.device
    gp, gs, gq = torch.empty_like(log_scales), torch.empty_like(log_scales), torch.empty_like(quats)
    primitives, starts, group_offsets = groups
    num_groups = int(primitives.numel())
    partial = torch.empty((max(num_groups, 1), 16), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        _check(_lib.load().mlpsp_geometry_gradients(_ptr(csr_offsets), _ptr(record_indices), _ptr(x6_sorted),
                                                    _ptr(falloff_adjoint), _ptr(log_scales), _ptr(quats),
                                                    _ptr(primitives), _ptr(starts), _ptr(group_offsets), num_groups,
                                                    int(groups.segment_size), log_scales.shape[0], _ptr(partial),
                                                    _ptr(gp), _ptr(gs), _ptr(gq), _stream(dev)),
               "mlpsp_geometry_gradients")
    return gp, gs, gq
