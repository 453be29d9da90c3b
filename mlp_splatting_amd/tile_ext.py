"""The renderer extension object: same entry-point names, positional signatures, return values and
error texts as the reference's pybind11 module (scannet/cuda/np_tile_kernels.cu:7224-7252,
forward entry points), implemented on the C ABI of ``libmlpsp_hip.so``.

``TileExt()`` is what ``cumodel._ensure_tile_ext_static()`` returns and what a test installs with
``monkeypatch.setattr(cumodel, "_tile_ext", ...)``.  The entry points of the reference's fused backward
kernels that are not provided raise ``NotImplementedError`` naming them; the record pipeline (records forward in
f32 or on the matrix cores, reverse compositing, grouped gradients) is.
"""
from __future__ import annotations

import contextlib
import os
import struct
import sys
import threading
import warnings

import torch

from . import _lib, ops

MAX_TILE_PRIMS = 1536          # MLPSP_MAX_TILE_PRIMS as built by scannet/cumodel.py:102-118
MAX_H_TILECENTER = 32          # MLPSP_MAX_H (np_tile_kernels.cu:36-38)

_BACKWARD_ONLY = (
    "render_tiles_mlp_records",
    "render_tiles_backward_tilecenter_traversal",
    "render_tiles_backward_tilecenter_backprop_noatomic",
)


def _chk(cond, msg="Expected condition to be true"):
    if not cond:
        raise RuntimeError(msg)


def _is_f32_2d(t, cols):
    return t.is_cuda and t.dtype == torch.float32 and t.dim() == 2 and t.shape[1] == cols



_SIXTEEN_ZERO_WORDS = (0,) * 16
_TAIL_WORDS = struct.Struct("<4q16i")      # the 96 bytes a queued frame reads back


def _on_device(device):
    """``torch.cuda.device(device)``, or nothing when that device is current already (saves two device switches)."""
    if device.index is None or torch.cuda.current_device() == device.index:
        return contextlib.nullcontext()
    return torch.cuda.device(device)


class QueuedFrame:
    """A frame whose launches are queued and whose 96-byte read-back has not been looked at yet
    (``TileExt.render_frame_queued(defer=True)`` -> ``TileExt.finish_frame_queued``)."""
    __slots__ = ("name", "precision", "with_feat", "images", "tail", "held", "cap", "scale", "inputs", "lists", "host",
                 "landed", "counts")

    def __init__(self, name, precision, with_feat, images, tail, held, cap, scale, inputs, lists):
        self.name, self.precision, self.with_feat, self.images = name, precision, with_feat, images
        self.tail, self.held, self.cap, self.scale, self.inputs, self.lists = tail, held, cap, scale, inputs, lists
        self.host = self.landed = self.counts = None


class TileExt:
    """Forward entry points of the tile renderer on one MI355X."""

    def __init__(self, max_tile_prims: int = MAX_TILE_PRIMS, max_hits: int = 512):
        _lib.load()  # fail now, loudly, if the HIP library is absent
        self.max_tile_prims = int(max_tile_prims)
        self.max_hits = int(max_hits)          # MLPSP_TILECENTER_MAX_HITS (np_tile_kernels.cu:48-50, 67-69)
        self._lock = threading.Lock()
        self._mfma_calls = 0
        self._queued_buffers = {}
        self._mfma_fallbacks = 0
        self._training_mfma_stats = [0, 0, 0, 0, 0]
        self._uncached = threading.local()
        self._pack = None                 # cache slots: lists of (key, value, source tensors) -- see _derived
        self._feat_pack = None
        self._rec = None
        self._binned = None
        self._queue_capacity = 0          # candidate-buffer estimate of render_frame_queued (0: not seeded yet)
        self._queue_scratch_scale = 1

    # ------------------------------------------------------------------------------------------
    # derived-tensor caches (geometry records, matrix-core operand copies)
    # ------------------------------------------------------------------------------------------
    def invalidate_caches(self):
        """Forget every derived tensor.  The caches are keyed on the identity, shape and in-place version of
        their source tensors -- enough while a scene is only rendered, but a fused optimizer step
        (``torch.optim.Adam(..., fused=True)``) rewrites parameters WITHOUT advancing their version counter.
        Every training entry point therefore works uncached and leaves the caches empty; call this after
        changing parameters by any other means that does not advance the version."""
        with self._lock:
            self._pack = self._feat_pack = self._rec = None
        # (the note about freshly binned tile lists is keyed on the list tensors themselves, not on parameters)

    @contextlib.contextmanager
    def uncached(self):
        """Inside: derived tensors are rebuilt from their sources on every use and not kept (training steps:
        the parameters change between calls in ways a version counter does not always show)."""
        self.invalidate_caches()
        depth = getattr(self._uncached, "depth", 0)
        self._uncached.depth = depth + 1
        try:
            yield self
        finally:
            self._uncached.depth = depth
            self.invalidate_caches()

    def _caching(self):
        return getattr(self._uncached, "depth", 0) == 0

    def __getattr__(self, name):
        if name in _BACKWARD_ONLY:
            def _missing(*_a, **_k):
                raise NotImplementedError(f"{name} is one of the reference's fused backward entry points, which this build does not provide")
            return _missing
        raise AttributeError(name)

    # ------------------------------------------------------------------------------------------
    # shared argument checks (np_tile_kernels.cu:5242-5275)
    # ------------------------------------------------------------------------------------------
    # ------------------------------------------------------------------------------------------
    # tile-list validation
    # ------------------------------------------------------------------------------------------
    @staticmethod
    def _list_key(cand, offsets, n):
        try:
            versions = (cand._version, offsets._version)
        except RuntimeError:          # inference tensors carry no version counter: an edit could not be seen
            return None
        return (cand.data_ptr(), cand.numel(), offsets.data_ptr(), offsets.numel(), versions, str(cand.device), int(n))

    def note_binned_lists(self, cand, offsets, longest, num_primitives):
        """Tile lists that this library's own binning kernels have just written are well-formed by
        construction (offsets monotonic and covering the list, ids in range); ``longest`` is the length
        of their longest tile list, which the binning read back together with the pair count.  The next
        render call that receives these very tensors, unmodified, checks the capacity against
        ``longest`` on the host instead of running the device validation pass with its blocking
        read-back (np_tile_kernels.cu:4553-4588).  Anything else is validated on the device."""
        key = self._list_key(cand, offsets, num_primitives)
        with self._lock:
            # (the note keeps the two tensors: their addresses identify them only while they are allocated)
            self._binned = None if key is None else (key, int(longest), cand, offsets)

    def _validate(self, cand, offsets, n_tiles, capacity, n, name):
        with self._lock:
            binned = self._binned
        if (binned is not None and cand.is_cuda and offsets.is_cuda and cand.dtype == torch.int32
                and offsets.dtype == torch.int32 and offsets.numel() == n_tiles + 1
                and binned[0] == self._list_key(cand, offsets, n)):   # (a None key never matches)
            if capacity > 0 and binned[1] > capacity:
                raise RuntimeError(f"{name}: tile candidate capacity {capacity} exceeded (maximum observed tile length "
                                   f"{binned[1]}); refusing to truncate or use an inconsistent forward/backward order")
            return
        ops.validate_tile_lists(cand, offsets, n_tiles, capacity, n, name)

    @staticmethod
    def _check_base(rays_o, rays_d, positions, log_scales, quats, cand, offsets, freq, att):
        _chk(_is_f32_2d(rays_o, 3), "rays_o must be a CUDA float32 [B,3] tensor")
        _chk(_is_f32_2d(rays_d, 3), "rays_d must be a CUDA float32 [B,3] tensor")
        _chk(_is_f32_2d(positions, 3), "positions must be a CUDA float32 [N,3] tensor")
        _chk(_is_f32_2d(log_scales, 3), "log_scales must be a CUDA float32 [N,3] tensor")
        _chk(_is_f32_2d(quats, 4), "quats must be a CUDA float32 [N,4] tensor")
        _chk(cand.is_cuda and cand.dtype == torch.int32 and cand.dim() == 1, "culled_prim_indices must be CUDA int32 1-D")
        _chk(offsets.is_cuda and offsets.dtype == torch.int32 and offsets.dim() == 1, "tile_offsets must be CUDA int32 1-D")
        _chk(freq.is_cuda and freq.dtype == torch.float32 and freq.dim() == 1, "freq_bands must be CUDA float32 1-D")
        _chk(att.is_cuda and att.dtype == torch.float32 and att.dim() == 1, "attenuation must be CUDA float32 1-D")

    @staticmethod
    def _weights_f32(ws, allow_low_precision):
        W1 = ws[0]
        _chk(all(w.is_cuda for w in ws), "MLP tensors must be CUDA tensors")
        _chk(all(w.dtype == W1.dtype for w in ws), "W/b tensors must share the same dtype")
        ok = (torch.float32, torch.float16, torch.bfloat16) if allow_low_precision else (torch.float32,)
        _chk(W1.dtype in ok, "W/b tensors must be float32, float16, or bfloat16" if allow_low_precision
             else "W/b tensors must be float32")
        # Stored half/bfloat16 weights are widened exactly, as the reference's cast_copy does when
        # it stages them (np_tile_kernels.cu:2016-2021).
        return [w.float().contiguous() for w in ws]

    def _prepare(self, args, name, capacity, tile_limit, low_precision=False, hidden_limit=64):
        (rays_o, rays_d, positions, log_scales, quats, cand, offsets, freq, att, W1, b1, W2, b2, W3, b3,
         Wimg, Himg, TW, TH, thr) = args
        Wimg, Himg, TW, TH = int(Wimg), int(Himg), int(TW), int(TH)
        if tile_limit is not None:
            _chk(0 < TW * TH <= tile_limit[0], tile_limit[1])
        self._check_base(rays_o, rays_d, positions, log_scales, quats, cand, offsets, freq, att)
        ws = self._weights_f32([W1, b1, W2, b2, W3, b3], low_precision)
        _chk(rays_o.shape[0] == Wimg * Himg, "B must equal W*H for tile renderer")
        _chk(Wimg > 0 and Himg > 0 and TW > 0 and TH > 0, f"{name}: image and tile dimensions must be positive")
        n_tiles = ops.num_tiles(Wimg, Himg, TW, TH)
        cand = cand.contiguous()
        offsets = offsets.contiguous()
        with torch.cuda.device(rays_o.device):
            self._validate(cand, offsets, n_tiles, capacity, positions.shape[0], name)
        F = freq.shape[0]
        _chk(W1.shape[2] == 6 * F * 2, "Encoded dim must be 6*F*2")
        _chk(W2.shape[1] <= hidden_limit, f"{name} currently supports hidden_dim <= {hidden_limit}")
        geo = (rays_o.contiguous(), rays_d.contiguous(), positions.contiguous(), log_scales.contiguous(),
               quats.contiguous())
        return geo, cand, offsets, freq.contiguous(), att.contiguous(), ws, (Wimg, Himg, TW, TH, float(thr))

    # ------------------------------------------------------------------------------------------
    # tile-centre order
    # ------------------------------------------------------------------------------------------
    def _tilecenter(self, args, name, family, capacity, with_t=False, low_precision=False, hidden_limit=MAX_H_TILECENTER,
                    stats=None):
        geo, cand, offsets, freq, att, ws, (W, H, TW, TH, thr) = self._prepare(
            args, name, capacity,
            (256, "Tile-center order kernel requires 0 < TW*TH <= MLPSP_TILECENTER_BLOCK_THREADS"),
            low_precision, hidden_limit)
        rays_o, rays_d, positions, log_scales, quats = geo
        with torch.cuda.device(rays_o.device):
            rec = self._records(positions, log_scales, quats)
            if family == _lib.KEY_LIST_ORDER or cand.numel() == 0:
                order = cand
            else:
                order, _ = ops.sort_tiles(rays_o, rays_d, rec, cand, offsets, W, H, TW, TH, family, capacity,
                                          cull_threshold=thr)
            if stats is not None:
                rgb, alpha = ops.render_tilecenter_stats_f32(rays_o, rays_d, rec, order, offsets, freq, att, *ws, W, H,
                                                             TW, TH, thr, *stats)
                return rgb, alpha, None
            return ops.render_tilecenter_f32(rays_o, rays_d, rec, order, offsets, freq, att, *ws, W, H, TW, TH, thr,
                                             with_t=with_t)

    def render_tiles_forward_tilecenter(self, *args):
        """(rgb [B,3], alpha [B,1]); np_tile_kernels.cu:5225-5347."""
        rgb, alpha, _ = self._tilecenter(args, "render_tiles_forward_tilecenter", _lib.KEY_TSTAR,
                                         self.max_tile_prims, low_precision=True)
        return rgb, alpha

    def render_tiles_autograd_tilecenter(self, *args):
        """Forward-only alias (np_tile_kernels.cu:4780-4860, 5040-5061)."""
        rgb, alpha, _ = self._tilecenter(args, "render_tiles_autograd_tilecenter", _lib.KEY_TSTAR, self.max_tile_prims)
        return rgb, alpha

    def render_tiles_autograd_tilecenter_presorted(self, *args):
        """Consumes host-sorted lists of any length (np_tile_kernels.cu:4880-4948, kernel :4242-4478)."""
        rgb, alpha, _ = self._tilecenter(args, "render_tiles_autograd_tilecenter_presorted", _lib.KEY_LIST_ORDER, 0)
        return rgb, alpha

    def render_tiles_forward_tilecenter_with_t(self, *args):
        """(rgb, alpha, t [B,1]); plain centre-depth order (np_tile_kernels.cu:5432-5792)."""
        return self._tilecenter(args, "render_tiles_forward_tilecenter_with_t", _lib.KEY_DEPTH, self.max_tile_prims,
                                with_t=True, hidden_limit=64)

    def render_tiles_forward_tilecenter_with_feat(self, *args):
        """(rgb, alpha, feat [B,C]); np_tile_kernels.cu:6114-6204."""
        base, (feat_attr, beta, temp), dims = args[:15], args[15:18], args[18:]
        name = "render_tiles_forward_tilecenter_with_feat"
        _chk(feat_attr.is_cuda and feat_attr.dtype == torch.float32 and feat_attr.dim() in (2, 3),
             "feat_attr must be a CUDA float32 tensor with 2 or 3 dimensions")
        geo, cand, offsets, freq, att, ws, (W, H, TW, TH, thr) = self._prepare(
            (*base, *dims), name, self.max_tile_prims,
            (256, "Tile-center feature kernel requires 0 < TW*TH <= MLPSP_TILECENTER_BLOCK_THREADS"))
        rays_o, rays_d, positions, log_scales, quats = geo
        _chk(feat_attr.shape[0] == positions.shape[0], "feat_attr first dimension must match primitive count")
        ops._feat_shape(feat_attr)
        with torch.cuda.device(rays_o.device):
            rec = self._records(positions, log_scales, quats)
            order = cand
            if cand.numel() > 0:
                order, _ = ops.sort_tiles(rays_o, rays_d, rec, cand, offsets, W, H, TW, TH, _lib.KEY_TSTAR,
                                          self.max_tile_prims, cull_threshold=thr)
            return ops.render_tilecenter_feat_f32(rays_o, rays_d, rec, order, offsets, freq, att, *ws,
                                                  feat_attr.contiguous(), beta, temp, W, H, TW, TH, thr)

    # ------------------------------------------------------------------------------------------
    # per-pixel order
    # ------------------------------------------------------------------------------------------
    def _per_pixel(self, args, name, feat=None):
        geo, cand, offsets, freq, att, ws, (W, H, TW, TH, thr) = self._prepare(args, name, 0, None, False, MAX_H_TILECENTER)
        _chk(0 < TW * TH <= 256, "Tile size too large")
        rays_o, rays_d, positions, log_scales, quats = geo
        with torch.cuda.device(rays_o.device):
            rec = self._records(positions, log_scales, quats)
            if feat is None:
                return ops.render_per_pixel_f32(rays_o, rays_d, rec, cand, offsets, freq, att, *ws, W, H, TW, TH, thr, name)
            feat_attr, beta, temp = feat
            return ops.render_per_pixel_f32(rays_o, rays_d, rec, cand, offsets, freq, att, *ws, W, H, TW, TH, thr, name,
                                            feat_attr=feat_attr.contiguous(), beta=beta, temp=temp)

    def render_tiles_forward(self, *args):
        """(rgb, alpha), per-pixel order; np_tile_kernels.cu:5064-5132."""
        rgb, alpha, _ = self._per_pixel(args, "render_tiles_forward")
        return rgb, alpha

    def render_tiles_autograd(self, *args):
        """Forward-only alias of the per-pixel renderer (np_tile_kernels.cu:4989-5038)."""
        rgb, alpha, _ = self._per_pixel(args, "render_tiles_autograd")
        return rgb, alpha

    def render_tiles_backward_count_per_pixel(self, *args):
        """counts [B] int32: the hits every pixel blends in its own depth order before its transmittance falls below
        1e-3 -- the record count of the per-pixel backward (np_tile_kernels.cu:1424-1566, wrapper :6210-6290)."""
        return self.render_tiles_per_pixel_records(args[:15], *args[15:], 1.5, 2.0, counts_only=True,
                                                   name="render_tiles_backward_count_per_pixel")

    def render_tiles_per_pixel_records(self, base, Wimg, Himg, TW, TH, thr, beta, temp, *, counts_only=False,
                                       name="render_tiles_backward_emit_per_pixel"):
        """[rgb, alpha, ids, x6, raw, masks, gates, offsets] as :meth:`render_tiles_training_records`, every pixel's
        records in the order of its own t: what the reference's per-pixel backward kernels traverse
        (np_tile_kernels.cu:1211-1836).  Tile lists are validated without a capacity (:6238), a 257th hit of a pixel
        raises the per-pixel overflow error."""
        geo, cand, offsets, freq, att, ws, (W, H, TW, TH, thr) = self._prepare((*base, Wimg, Himg, TW, TH, thr), name, 0,
                                                                               None, False, MAX_H_TILECENTER)
        _chk(0 < TW * TH <= 256, "Tile size too large")
        rays_o, rays_d, positions, log_scales, quats = geo
        with torch.cuda.device(rays_o.device), self.uncached():
            rec = self._records(positions, log_scales, quats)
            out = ops.records_per_pixel(rays_o, rays_d, rec, cand, offsets, freq, att, *ws, W, H, TW, TH, thr, float(beta),
                                        float(temp), name, counts_only=counts_only)
        return out if counts_only else list(out)

    def render_tiles_forward_per_pixel_with_feat(self, *args):
        """(rgb, alpha, feat); np_tile_kernels.cu:5134-5222."""
        base, (feat_attr, beta, temp), dims = args[:15], args[15:18], args[18:]
        _chk(feat_attr.is_cuda and feat_attr.dtype == torch.float32 and feat_attr.dim() in (2, 3),
             "feat_attr must be a CUDA float32 tensor with 2 or 3 dimensions")
        _chk(feat_attr.shape[0] == base[2].shape[0], "feat_attr first dimension must match primitive count")
        ops._feat_shape(feat_attr)
        return self._per_pixel((*base, *dims), "render_tiles_forward_per_pixel_with_feat", (feat_attr, beta, temp))

    # ------------------------------------------------------------------------------------------
    # a whole frame queued without a host synchronisation in its middle (no counterpart in the reference)
    # ------------------------------------------------------------------------------------------
    def frame_binning_queued(self, positions, log_scales, view_matrices, proj_matrix, width, height, threshold,
                             segments=False):
        """First half of :meth:`render_frame_queued`: the frame's binning, queued.  It needs nothing but the
        primitives and the camera, so a caller queues it before it prepares anything else for the frame (ray
        directions, weights): the device works through the binning while the host does that.  Returns what
        :meth:`render_frame_queued` takes as ``binned``, or None when no candidate-buffer estimate exists yet.
        ``segments``: every tile's list in a segment of ``max_tile_prims`` entries of its own
        (:func:`ops.bin_segments_async`: one launch less, no estimate needed), when the camera's matrices are on the
        device; for frames whose render takes such lists (the matrix cores')."""
        with self._lock:
            cap, scale = self._queue_capacity, self._queue_scratch_scale
        # (not for screens whose segments would take more than 2 GiB per array: those keep the lists one after the other)
        segments = (segments and all(m.is_cuda and m.dtype == torch.float32 and m.numel() == 16 and m.is_contiguous()
                                     for m in (view_matrices, proj_matrix))
                    and ops.num_tiles(int(width), int(height), 8, 8) * self.max_tile_prims <= 1 << 29)
        if cap <= 0 and not segments:
            return None
        with _on_device(positions.device):
            # counts of the binning (4 x int64) and flag words of the render (16 x int32) share one buffer: the
            # frame's single read-back is one 96-byte copy.  The buffers a queued frame keeps to itself (this one,
            # lists, offsets, scratch) are handed out again to the next frame of the same thread on the same stream:
            # that frame starts after this one's read-back, and its first launch is four allocations nearer.
            held = self._frame_buffers(positions.device)
            if "tail" not in held:
                fresh = torch.empty(96, dtype=torch.uint8, device=positions.device)
                held["tail"] = (fresh, fresh[:32].view(torch.int64))
                held["flags_clear"] = False
            tail, counts_view = held["tail"]
            if segments:
                cand, offsets, ends, counts = ops.bin_segments_async(
                    positions, log_scales, view_matrices, proj_matrix, int(width), int(height), 8, float(threshold),
                    stride=self.max_tile_prims, scratch_scale=scale, counts=counts_view, reuse=held)
                return cand, offsets, counts, tail, cap, scale, held, ends
            cand, offsets, counts = ops.bin_legacy_async(positions, log_scales, view_matrices, proj_matrix, int(width),
                                                         int(height), 8, float(threshold), cap, scratch_scale=scale,
                                                         counts=counts_view, reuse=held)
        return cand, offsets, counts, tail, cap, scale, held, None

    def _frame_buffers(self, device):
        """The reusable buffers of queued frames, per (thread, device, stream)."""
        index = device.index if device.index is not None else torch.cuda.current_device()
        key = (threading.get_ident(), index, torch._C._cuda_getCurrentRawStream(index))
        held = self._queued_buffers.get(key)
        if held is None:
            with self._lock:
                if len(self._queued_buffers) > 16:
                    self._queued_buffers.clear()
                held = self._queued_buffers.setdefault(key, {})
        return held

    def frame_prologue(self, rays_o, rays_d, width, height, geometry=None):
        """(unit ray directions, tile pyramids of the sort, frame records of the sort | None) for a queued frame of
        8x8 tiles, in one launch (:func:`ops.frame_prologue`).  ``geometry`` = (positions, log_scales, unit_quats) asks
        for the frame records too; the geometry records they are made from are the cached ones.  ``rays_o`` and
        ``rays_d`` must be float32 [width * height, 3] device tensors."""
        with _on_device(rays_o.device):
            records = None if geometry is None else self._records(*geometry)
            return ops.frame_prologue(rays_o, rays_d, int(width), int(height), 8, 8, records)

    def render_frame_queued(self, rays_o, unit_dirs, positions, log_scales, unit_quats, freq, att, ws, view_matrices,
                            proj_matrix, width, height, threshold, precision, binned=None, feat=None,
                            frame_records=None, tile_pyramids=None, defer=False):
        """(rgb, alpha) of one 8x8-tile, tile-centre-order RGB frame: binning, sort and render are queued
        back to back and ONE read-back at the end brings the pair count, the longest tile list and the
        non-finite flag.  The candidate buffer is sized from the previous frame's count; if this frame
        needs more (or the level-1 scratch overflows) every list was left empty on the device: the
        estimate is enlarged and None is returned, and the caller renders the frame the synchronous way.
        ``binned``: the result of :meth:`frame_binning_queued` for the same primitives and camera, when the caller
        has queued the binning already.  ``feat`` = (feat_attr, beta, temp) adds the gated feature image (matrix-core
        precisions only): (rgb, alpha, feat); None is also returned when the record pool of the first size ran out
        or the attributes do not fit fp16 (the step-by-step path then decides what to do).  ``tile_pyramids``,
        ``frame_records``: what :meth:`frame_prologue` returned beside ``unit_dirs`` for these rays and primitives.
        ``defer``: queue the frame, start its read-back into pinned memory and return a :class:`QueuedFrame` instead of
        waiting; :meth:`finish_frame_queued` then waits, decides and returns what this method would have.  A caller
        that has the next camera at hand queues that frame on another stream in between, so the device never waits
        for the host (matrix-core precisions; an exact frame is finished before it is returned either way).
        Errors are those of the entry points it stands for (capacity text of np_tile_kernels.cu:4578-4588,
        fallback policy of rgb_wmma.cuh:260-272)."""
        name = "render_tiles_rgb_wmma" if precision != "f32" else "render_tiles_forward_tilecenter"
        width, height, threshold = int(width), int(height), float(threshold)
        if feat is not None and precision == "f32":
            return None                                   # (the exact feature path is not queued)
        if feat is not None:
            _chk(feat[0].is_cuda and feat[0].dtype in (torch.float32, torch.float16) and feat[0].dim() in (2, 3),
                 "feat_attr must be a CUDA float32 tensor with 2 or 3 dimensions")
            _chk(feat[0].shape[0] == positions.shape[0], "feat_attr first dimension must match primitive count")
        if binned is None:
            binned = self.frame_binning_queued(positions, log_scales, view_matrices, proj_matrix, width, height,
                                               threshold)
            if binned is None:
                return None
        cand, offsets, counts, tail, cap, scale, held, ends = binned
        if ends is not None and precision == "f32":
            raise ValueError("lists in segments are for frames on the matrix cores")
        status = tail[32:].view(torch.int32)
        # The flag words live in a buffer that this thread's frames use one after the other, and every frame ends by
        # reading them back: if the last frame read sixteen zeros they are still zero, and the render's own clear (a
        # launch between the sort and the render) is left out.  The mark is taken down while a frame is under way.
        flags_clear = held.get("flags_clear", False) and held.get("tail", (None,))[0] is tail
        held["flags_clear"] = False
        n = positions.shape[0]
        with _on_device(rays_o.device):
            rec = self._records(positions, log_scales, unit_quats)
            order, _ = ops.sort_tiles(rays_o, unit_dirs, rec, cand, offsets, width, height, 8, 8, _lib.KEY_TSTAR,
                                      self.max_tile_prims, cull_threshold=threshold, frame_records=frame_records,
                                      tile_pyramids=tile_pyramids, tile_ends=ends, ids_ascend=True)
            fmap, pool_ran_out = None, 0
            if precision != "f32":
                packed = self._packed_weights(list(ws), precision == "bf16")
                if feat is None:
                    rgb, alpha, _ = ops.render_tilecenter_mfma(rays_o, unit_dirs, rec, order, offsets, freq, att, *ws,
                                                               width, height, threshold, bf16=(precision == "bf16"),
                                                               packed=packed, check=False, status=status,
                                                               status_is_clear=flags_clear, tile_ends=ends)
                else:
                    packed_feat, bad_attr = self._packed_feat(feat[0])
                    if bad_attr:
                        return None
                    rgb, alpha, fmap, _ = ops.render_tilecenter_mfma_feat(
                        rays_o, unit_dirs, rec, order, offsets, freq, att, *ws, feat[0], feat[1], feat[2], width, height,
                        threshold, bf16=(precision == "bf16"), packed=packed, packed_feat=packed_feat, status=status,
                        status_is_clear=flags_clear, tile_ends=ends)
                frame = QueuedFrame(name, precision, feat is not None, (rgb, alpha, fmap), tail, held, cap, scale,
                                    (rays_o, unit_dirs, positions, log_scales, unit_quats, freq, att, ws),
                                    (rec, order, offsets, width, height, threshold, ends))
                if defer:
                    pinned = held.get("pinned")
                    if pinned is None:
                        pinned = held["pinned"] = torch.empty(96, dtype=torch.uint8, pin_memory=True)
                    pinned.copy_(tail, non_blocking=True)
                    frame.landed = torch.cuda.Event()
                    frame.landed.record()
                    frame.host = pinned.numpy()
                    return frame
                frame.host = tail.cpu().numpy()
                return self.finish_frame_queued(frame)
            rgb, alpha, _ = ops.render_tilecenter_f32(rays_o, unit_dirs, rec, order, offsets, freq, att, *ws, width,
                                                      height, 8, 8, threshold)
            frame = QueuedFrame(name, precision, False, (rgb, alpha, None), tail, held, cap, scale, (), ())
            frame.counts = counts.tolist()
            return self.finish_frame_queued(frame)

    def finish_frame_queued(self, frame):
        """Second half of a frame that :meth:`render_frame_queued` returned as a :class:`QueuedFrame`: waits for its
        read-back and returns (rgb, alpha[, feat]), None (the caller renders the frame the synchronous way) or raises,
        as :meth:`render_frame_queued` documents.  Call it with the frame's stream current: a fallback render is
        queued there."""
        name, precision, held, cap, scale = frame.name, frame.precision, frame.held, frame.cap, frame.scale
        rgb, alpha, fmap = frame.images
        if frame.counts is None:
            if frame.landed is not None:
                frame.landed.synchronize()
            # (four int64 counts of the binning, sixteen int32 flag words of the render: one unpacking)
            words = _TAIL_WORDS.unpack_from(frame.host)
            pairs, longest, l1_entries, guard = words[:4]
            held["flags_clear"] = words[4:] == _SIXTEEN_ZERO_WORDS
            nonfinite = words[4]
            pool_ran_out = words[5] if frame.with_feat else 0
        else:
            pairs, longest, l1_entries, guard = frame.counts
            nonfinite = pool_ran_out = 0
        with self._lock:
            if guard:
                if pairs > cap:
                    self._queue_capacity = int(pairs * 1.3) + 65536
                else:
                    self._queue_scratch_scale = scale * 4
                return None
            if pairs > 0.9 * cap:                       # stay ahead of a slowly growing scene
                self._queue_capacity = int(pairs * 1.3) + 65536
            redo = frame.with_feat and bool(nonfinite or pool_ran_out)
            if precision != "f32" and not redo:
                self._mfma_calls += 1
        if redo:
            return None                               # rare: the step-by-step path repeats the frame
        if longest > self.max_tile_prims:
            raise RuntimeError(f"{name}: tile candidate capacity {self.max_tile_prims} exceeded (maximum observed "
                               f"tile length {longest}); refusing to truncate or use an inconsistent "
                               "forward/backward order")
        if nonfinite:
            rays_o, unit_dirs, positions, log_scales, unit_quats, freq, att, ws = frame.inputs
            rec, order, offsets, width, height, threshold, ends = frame.lists
            with _on_device(rays_o.device):
                if ends is not None:      # (the f32 kernel reads lists that follow one another)
                    order, offsets = ops.compact_segments(order, offsets, ends)
                for t in (rays_o, unit_dirs, positions, log_scales, unit_quats, freq, att, *ws):
                    _chk(bool(torch.isfinite(t).all()), "WMMA input is nonfinite; refusing fallback")
                warnings.warn("WMMA operand/activation overflow: rendering this frame with scalar FP32 instead")
                with self._lock:
                    self._mfma_fallbacks += 1
                rgb, alpha, _ = ops.render_tilecenter_f32(rays_o, unit_dirs, rec, order, offsets, freq, att,
                                                          *[w.float() for w in ws], width, height, 8, 8, threshold)
                _chk(bool(torch.isfinite(rgb).all()) and bool(torch.isfinite(alpha).all()),
                     "Scalar FP32 fallback output is nonfinite")
        return (rgb, alpha) if not frame.with_feat else (rgb, alpha, fmap)

    def note_frame_pairs(self, pairs: int):
        """Seed the candidate-buffer estimate of :meth:`render_frame_queued` from a synchronous frame."""
        with self._lock:
            if pairs * 1.1 > self._queue_capacity:
                self._queue_capacity = int(pairs * 1.3) + 65536

    # ------------------------------------------------------------------------------------------
    # training-records forward (np_tile_kernels.cu:6897-6998, forward_only = true)
    # ------------------------------------------------------------------------------------------
    def render_tiles_training_records(self, x, width, height, tile, threshold, beta, temp, *, render_order=False,
                                      any_tile=False, counts_only=False, name="render_tiles_mlp_records"):
        """[rgb, alpha, ids, x6, raw, masks, gates, offsets]: one record per hit and pixel, in each
        pixel's compositing order.  ``x`` = the 15 scene tensors + two adjoint placeholders that the
        forward-only mode never reads (scannet/csr_training.py:37-39).  ``render_order`` (not in the reference):
        image and records in the rounding of ``render_tiles_forward_tilecenter`` instead of the record kernels'
        own; see :meth:`records_forward_matches_render`."""
        _chk(len(x) == 17, "Expected 15 scene inputs and RGB/T adjoints")
        width, height, tile = int(width), int(height), int(tile)
        # any_tile: the backward entry points, whose reference kernels take any square tile of up to 256 pixels
        _chk(width > 0 and height > 0 and (tile in (8, 16) or (any_tile and 0 < tile * tile <= 256)),
             "the records forward supports 8x8 and 16x16 tiles")
        for i, t in enumerate(x):
            _chk(t.is_cuda and t.is_contiguous(), "Inputs must be contiguous CUDA tensors")
            _chk(t.device == x[0].device, "Inputs must share a device")
            _chk(t.dtype == (torch.int32 if i in (5, 6) else torch.float32),
                 "Records path requires FP32 inputs and int32 tile lists")
        pixels, n = width * height, x[2].shape[0]
        _chk(tuple(x[0].shape) == (pixels, 3) and x[1].shape == x[0].shape)
        _chk(x[2].dim() == 2 and x[2].shape[1] == 3 and x[3].shape == x[2].shape and tuple(x[4].shape) == (n, 4))
        _chk(x[7].dim() == 1 and x[8].shape == x[7].shape and x[9].dim() == 3 and x[9].shape[0] == n)
        h, inp, f = x[9].shape[1], x[9].shape[2], x[7].numel()
        _chk(0 < h <= 32 and f > 0 and inp == 12 * f)
        _chk(tuple(x[10].shape) == (n, h) and tuple(x[11].shape) == (n, h, h) and x[12].shape == x[10].shape)
        _chk(tuple(x[13].shape) == (n, 4, h) and tuple(x[14].shape) == (n, 4))
        _chk(x[15].shape == x[0].shape and x[16].dim() == 1 and x[16].numel() == pixels)
        with torch.cuda.device(x[0].device), self.uncached():
            self._validate(x[5], x[6], ops.num_tiles(width, height, tile, tile), self.max_tile_prims, n, name)
            rec = self._records(x[2], x[3], x[4])
            order = x[5]
            if x[5].numel() > 0:
                order, _ = ops.sort_tiles(x[0], x[1], rec, x[5], x[6], width, height, tile, tile, _lib.KEY_TSTAR,
                                          self.max_tile_prims, cull_threshold=float(threshold))
            out = ops.training_records(x[0], x[1], rec, order, x[6], x[7], x[8], *x[9:15], width, height, tile, tile,
                                       float(threshold), float(beta), float(temp), self.max_hits, name,
                                       render_order=bool(render_order), counts_only=counts_only)
            return out if counts_only else list(out)

    @staticmethod
    def records_forward_matches_render(freq, W1, b1, W2, b2, tile):
        """True if ``render_tiles_training_records(..., render_order=True)`` is available for this frame: 8x8 tiles
        and the 72->32->32->4 MLP with six frequencies in 16-byte aligned f32 tensors.  Its rgb/alpha are then the
        bits of ``render_tiles_forward_tilecenter``, and a differentiable render can keep the records of its
        forward pass for the backward instead of traversing the frame again."""
        return (int(tile) == 8 and freq.numel() == 6 and tuple(W1.shape[1:]) == (32, 72) and tuple(W2.shape[1:]) == (32, 32)
                and all(t.dtype == torch.float32 and t.is_contiguous() and t.data_ptr() % 16 == 0 for t in (W1, b1, W2, b2)))

    def training_wmma_safety_stats(self):
        """[calls, frame_fallbacks, fp32_nonfinite_failures, count_emit_failures, capacity_failures] of
        :meth:`render_tiles_training_records_wmma` since this object was made (training_wmma.cuh:7-19: calls
        are accepted count-pass launches; rejected arguments and candidate lists are not counted)."""
        with self._lock:
            return list(self._training_mfma_stats)

    def _count_training_mfma(self, index):
        with self._lock:
            self._training_mfma_stats[index] += 1

    def render_tiles_training_records_wmma(self, x, width, height, tile, threshold, beta, temp, precision):
        """The records of :meth:`render_tiles_training_records` with the MLP on the matrix cores in ``precision``
        ("float16" or "bfloat16") and everything else in the same f32 expressions (wrapper and policy of
        training_wmma.cuh:267-357): non-finite inputs are refused, a numeric overflow of the reduced-precision
        pass discards it and repeats the whole frame with the scalar f32 record forward, hit capacity and a
        count/emit disagreement raise."""
        import math
        _chk(len(x) == 17, "Training WMMA requires 15 scene inputs and two RGB/T adjoint placeholders")
        _chk(int(tile) == 8, "Training WMMA requires tile8")
        _chk(precision in ("float16", "bfloat16"), "Training WMMA precision must be float16 or bfloat16")
        width, height = int(width), int(height)
        _chk(0 < width <= 2147483647 and 0 < height <= 2147483647 and width <= 2147483647 // height,
             "Training WMMA image dimensions exceed int32 pixel indexing")
        thr32 = torch.tensor(float(threshold), dtype=torch.float32).item()
        _chk(math.isfinite(threshold) and 0.0 < thr32 < 1.0,
             "Training WMMA threshold must remain in (0,1) after FP32 conversion")
        for v in (beta, temp):
            _chk(math.isfinite(v) and math.isfinite(torch.tensor(float(v), dtype=torch.float32).item()),
                 "Training WMMA gating parameters must be finite FP32 values")
        for i, t in enumerate(x):
            _chk(t.is_cuda and t.is_contiguous() and t.device == x[0].device,
                 "Training WMMA inputs must be contiguous CUDA tensors on one device")
            _chk(t.dtype == (torch.int32 if i in (5, 6) else torch.float32),
                 "Training WMMA requires FP32 inputs and int32 tile lists")
        pixels, n = width * height, x[2].shape[0] if x[2].dim() == 2 else -1
        _chk(tuple(x[0].shape) == (pixels, 3) and x[1].shape == x[0].shape)
        _chk(x[2].dim() == 2 and x[2].shape[1] == 3 and x[3].shape == x[2].shape and tuple(x[4].shape) == (n, 4))
        _chk(x[7].dim() == 1 and x[7].numel() == 6 and x[8].shape == x[7].shape)
        _chk(tuple(x[9].shape) == (n, 32, 72) and tuple(x[10].shape) == (n, 32) and tuple(x[11].shape) == (n, 32, 32))
        _chk(x[12].shape == x[10].shape and tuple(x[13].shape) == (n, 4, 32) and tuple(x[14].shape) == (n, 4))
        _chk(x[15].shape == x[0].shape and x[16].dim() == 1 and x[16].numel() == pixels)
        name = "render_tiles_training_records_wmma"
        with torch.cuda.device(x[0].device), self.uncached():
            self._validate(x[5], x[6], ops.num_tiles(width, height, 8, 8), self.max_tile_prims, n, name)
            nonfinite = ops.all_finite_flag([t for i, t in enumerate(x) if i not in (5, 6)])
            _chk(int(nonfinite.item()) == 0, "Training WMMA input is nonfinite; refusing unsafe forward/fallback")
            self._count_training_mfma(0)
            bf16 = precision == "bfloat16"
            rec = self._records(x[2], x[3], x[4])
            order = x[5]
            if x[5].numel() > 0:
                order, _ = ops.sort_tiles(x[0], x[1], rec, x[5], x[6], width, height, 8, 8, _lib.KEY_TSTAR,
                                          self.max_tile_prims, cull_threshold=float(threshold))
            packed = self._packed_weights(list(x[9:15]), bf16)
            bits, records = ops.training_records_mfma(x[0], x[1], rec, order, x[6], x[7], x[8], packed, n, width, height,
                                                      float(threshold), float(beta), float(temp), self.max_hits, bf16)
            if bits & 2:
                self._count_training_mfma(4)
                raise RuntimeError(f"Training WMMA hit capacity {self.max_hits} exceeded; refusing truncated records")
            if bits & 4:
                self._count_training_mfma(3)
                raise RuntimeError("Training WMMA count/emit mismatch; bounded partial records were discarded")
            if bits & 1:
                self._count_training_mfma(1)
                warnings.warn("Training WMMA numeric overflow: discarding both mixed passes and rerunning the whole "
                              "FP32 record forward")
                del records
                records = self.render_tiles_training_records(x, width, height, 8, threshold, beta, temp)
                if int(ops.all_finite_flag([t for t in records if t.is_floating_point()]).item()):
                    self._count_training_mfma(2)
                    raise RuntimeError("Training WMMA scalar FP32 fallback records are nonfinite")
            return list(records)

    def primitive_records_reverse(self, ids, offsets, x6, raw, logs, quats, grgb, gt):
        """[d4, grad_positions, grad_log_scales, grad_quats] from saved forward records
        (scannet/cuda/primitive_records.cuh:48-74: same argument checks, then one reverse walk per pixel)."""
        tensors = (ids, offsets, x6, raw, logs, quats, grgb, gt)
        for t in tensors:
            _chk(t.is_cuda and t.is_contiguous() and t.device == ids.device)
        _chk(ids.dtype == torch.int32 and offsets.dtype == torch.int64)
        for t in (x6, raw, logs, quats, grgb, gt):
            _chk(t.dtype == torch.float32)
        total, pixels, n = ids.numel(), grgb.shape[0], logs.shape[0]
        _chk(ids.dim() == 1 and offsets.dim() == 1 and offsets.numel() == pixels + 1)
        _chk(x6.dim() == 2 and tuple(x6.shape) == (total, 6))
        _chk(raw.dim() == 2 and tuple(raw.shape) == (total, 8))
        _chk(logs.dim() == 2 and logs.shape[1] == 3)
        _chk(quats.dim() == 2 and tuple(quats.shape) == (n, 4))
        _chk(grgb.dim() == 2 and grgb.shape[1] == 3 and gt.dim() == 1 and gt.numel() == pixels)
        _chk(int(offsets[0]) == 0 and int(offsets[-1]) == total)
        _chk(bool((offsets[1:] >= offsets[:-1]).all()))
        if total:
            lo, hi = torch.aminmax(ids)
            _chk(int(lo) >= 0 and int(hi) < n)
        return list(ops.records_reverse(ids, offsets, x6, raw, logs, quats, grgb, gt))

    def primitive_records_reverse_adjoints(self, ids, offsets, raw, grgb, gt):
        """(d4 [R,4], falloff adjoint [R]): the reverse walk of ``primitive_records_reverse`` without its atomic
        geometry sums (no counterpart in the reference; ``primitive_geometry_gradients`` completes it)."""
        for t in (ids, offsets, raw, grgb, gt):
            _chk(t.is_cuda and t.is_contiguous() and t.device == ids.device)
        _chk(ids.dtype == torch.int32 and offsets.dtype == torch.int64 and raw.dtype == torch.float32)
        _chk(raw.dim() == 2 and tuple(raw.shape) == (ids.numel(), 8) and offsets.numel() == grgb.shape[0] + 1)
        _chk(grgb.dim() == 2 and grgb.shape[1] == 3 and gt.numel() == grgb.shape[0])
        with torch.cuda.device(ids.device):
            return ops.records_reverse_adjoints(ids, offsets, raw, grgb, gt)

    def primitive_geometry_gradients(self, csr, falloff_adjoint, log_scales, quats, groups):
        """(grad_positions, grad_log_scales, grad_quats) from a primitive-major CSR of the records and the
        per-record falloff adjoints, one wavefront per segment of ``groups`` (no atomics)."""
        with torch.cuda.device(log_scales.device):
            return ops.geometry_gradients(csr.offsets, csr.record_indices, csr.x6, falloff_adjoint, log_scales, quats,
                                          groups)

    def render_tiles_backward_tilecenter_full(self, rays_o, rays_d, positions, log_scales, quats, cand, offsets,
                                              freq, att, W1, b1, W2, b2, W3, b3, grad_rgb, grad_t, Wimg, Himg, TW, TH,
                                              thr):
        """[gW1, gb1, gW2, gb2, gW3, gb3, grad_positions, grad_log_scales, grad_quats] of the tile-centre-order
        render for the image adjoint ``grad_rgb`` [B,3] and the adjoint ``grad_t`` [B] of the final transmittance
        (np_tile_kernels.cu:2928-3530, wrapper :6765-6895).  The reference fuses everything into one kernel;
        here the same quantities come from the record pipeline it is tested against (tests/test_primitive_csr.py:
        44-50: equal within 5e-4): records forward -> reverse compositing -> grouped weight gradients in IEEE f32."""
        from .primitive_csr import group_records, reference_weight_gradients
        from . import primitive_gemm
        _chk(int(TW) == int(TH), "square tiles only")
        x = [rays_o, rays_d, positions, log_scales, quats, cand, offsets, freq, att, W1, b1, W2, b2, W3, b3,
             grad_rgb.contiguous(), grad_t.contiguous()]
        records = self.render_tiles_training_records(x, Wimg, Himg, TW, thr, 1.5, 2.0, any_tile=True,
                                                     name="render_tiles_backward_tilecenter_full")
        return self.backward_from_records(records, positions, log_scales, quats, freq, att, W1, b1, W2, b2, W3, b3,
                                          x[15], x[16])

    def render_tiles_backward_tilecenter_full_with_feat(self, rays_o, rays_d, positions, log_scales, quats, cand, offsets,
                                                        freq, att, W1, b1, W2, b2, W3, b3, feat_attr, grad_rgb, grad_t,
                                                        grad_feat, beta, temp, Wimg, Himg, TW, TH, thr):
        """The nine gradients of :meth:`render_tiles_backward_tilecenter_full` and grad_feat_attr of
        :meth:`render_tiles_backward_featattr_tilecenter` from one traversal (np_tile_kernels.cu:7005-7114): here one
        records forward and one grouping of its records."""
        _chk(int(TW) == int(TH), "square tiles only")
        self._check_feature_adjoint(feat_attr, grad_feat, positions, int(Wimg) * int(Himg))
        x = [rays_o, rays_d, positions, log_scales, quats, cand, offsets, freq, att, W1, b1, W2, b2, W3, b3,
             grad_rgb.contiguous(), grad_t.contiguous()]
        records = self.render_tiles_training_records(x, Wimg, Himg, TW, thr, float(beta), float(temp), any_tile=True,
                                                     name="render_tiles_backward_tilecenter_full_with_feat")
        return self.backward_from_records(records, positions, log_scales, quats, freq, att, W1, b1, W2, b2, W3, b3,
                                          x[15], x[16], feat_attr=feat_attr, grad_feat=grad_feat.contiguous())

    @staticmethod
    def _check_feature_adjoint(feat_attr, grad_out_feat, positions, pixels):
        _chk(feat_attr.is_cuda and feat_attr.dtype == torch.float32 and feat_attr.is_contiguous())
        _chk(feat_attr.dim() in (2, 3) and feat_attr.shape[0] == positions.shape[0],
             "feat_attr first dimension must match primitive count")
        _chk(feat_attr.dim() == 2 or feat_attr.shape[1] in (4, 5), "3D feat_attr expects slots in {4,5}")
        _chk(grad_out_feat.is_cuda and grad_out_feat.dtype == torch.float32
             and tuple(grad_out_feat.shape) == (pixels, feat_attr.shape[-1]), "grad_out_feat must be [B, C]")

    def render_tiles_backward_count_tilecenter(self, rays_o, rays_d, positions, log_scales, quats, cand, offsets, freq,
                                               att, W1, b1, W2, b2, W3, b3, Wimg, Himg, TW, TH, thr):
        """counts [B] int32 of the tile-centre-order backward: the hits every pixel blends before its transmittance
        falls below 1e-3 (np_tile_kernels.cu:6275-6340)."""
        _chk(int(TW) == int(TH), "square tiles only")
        pixels = int(Wimg) * int(Himg)
        x = [rays_o, rays_d, positions, log_scales, quats, cand, offsets, freq, att, W1, b1, W2, b2, W3, b3,
             torch.zeros_like(rays_o), torch.zeros(pixels, device=rays_o.device)]
        return self.render_tiles_training_records(x, Wimg, Himg, TW, thr, 1.5, 2.0, any_tile=True, counts_only=True,
                                                  name="render_tiles_backward_count_tilecenter")

    def _emit(self, records, log_scales, quats, grad_rgb, grad_t, counts, offsets, total):
        """The emit entry points' outputs from records: (prim_id, x6, grad_rgb, grad_sigma_raw, grad_positions,
        grad_log_scales, grad_quats) with record k of pixel p at offsets[p] + k for k < counts[p]
        (np_tile_kernels.cu:1568-1836: out_grad_rgb = T alpha grad_out_rgb[p], out_grad_sigma_raw = the adjoint of
        softplus(o3))."""
        _, _, ids, x6, raw, _, _, rec_off = records
        pixels = rec_off.numel() - 1
        _chk(counts.dtype == torch.int32 and counts.numel() == pixels, "counts must have size B")
        _chk(offsets.dtype == torch.int32 and offsets.numel() == pixels, "offsets must have size B")
        dev = ids.device
        total = int(total)
        with torch.cuda.device(dev):
            d4, gp, gs, gq = ops.records_reverse(ids, rec_off, x6, raw, log_scales, quats, grad_rgb.contiguous(),
                                                 grad_t.contiguous())
            pix = torch.repeat_interleave(torch.arange(pixels, device=dev), rec_off.diff(), output_size=ids.numel())
            k = torch.arange(ids.numel(), device=dev) - rec_off[pix]
            dest = offsets.long()[pix] + k
            keep = (k < counts.long()[pix]) & (dest < total)
            dest = dest[keep]
            weight = (raw[:, 4] * raw[:, 5])[:, None]
            sigma_adjoint = d4[:, 3:4] / torch.sigmoid(raw[:, 7:8]).clamp_min(1e-38)
            out_ids = torch.zeros(total, dtype=torch.int32, device=dev)
            out_x6 = torch.zeros(total, 6, device=dev)
            out_rgb = torch.zeros(total, 3, device=dev)
            out_sigma = torch.zeros(total, 1, device=dev)
            out_ids[dest] = ids[keep]
            out_x6[dest] = x6[keep]
            out_rgb[dest] = (weight * grad_rgb[pix])[keep]
            out_sigma[dest] = sigma_adjoint[keep]
        return [out_ids, out_x6, out_rgb, out_sigma, gp, gs, gq]

    def render_tiles_backward_emit_tilecenter(self, rays_o, rays_d, positions, log_scales, quats, cand, offsets, freq,
                                              att, W1, b1, W2, b2, W3, b3, grad_rgb, grad_t, counts, record_offsets,
                                              total_records, Wimg, Himg, TW, TH, thr):
        """(prim_id, x6, grad_rgb, grad_sigma_raw, grad_positions, grad_log_scales) of the tile-centre order
        (np_tile_kernels.cu:6443-6535)."""
        _chk(int(TW) == int(TH), "square tiles only")
        x = [rays_o, rays_d, positions, log_scales, quats, cand, offsets, freq, att, W1, b1, W2, b2, W3, b3,
             grad_rgb.contiguous(), grad_t.contiguous()]
        records = self.render_tiles_training_records(x, Wimg, Himg, TW, thr, 1.5, 2.0, any_tile=True,
                                                     name="render_tiles_backward_emit_tilecenter")
        return self._emit(records, log_scales, quats, x[15], x[16], counts, record_offsets, total_records)[:6]

    def render_tiles_backward_emit_per_pixel(self, rays_o, rays_d, positions, log_scales, quats, cand, offsets, freq, att,
                                             W1, b1, W2, b2, W3, b3, grad_rgb, grad_t, counts, record_offsets,
                                             total_records, Wimg, Himg, TW, TH, thr):
        """(prim_id, x6, grad_rgb, grad_sigma_raw, grad_positions, grad_log_scales, grad_quats) of the per-pixel order
        (np_tile_kernels.cu:6344-6400)."""
        base = (rays_o, rays_d, positions, log_scales, quats, cand, offsets, freq, att, W1, b1, W2, b2, W3, b3)
        _chk(grad_rgb.is_cuda and grad_rgb.dtype == torch.float32 and tuple(grad_rgb.shape) == (int(Wimg) * int(Himg), 3))
        _chk(grad_t.is_cuda and grad_t.dtype == torch.float32 and grad_t.numel() == int(Wimg) * int(Himg),
             "grad_T_end must have size B")
        records = self.render_tiles_per_pixel_records(base, Wimg, Himg, TW, TH, thr, 1.5, 2.0)
        return self._emit(records, log_scales, quats, grad_rgb, grad_t, counts, record_offsets, total_records)

    def render_tiles_backward_featattr_tilecenter(self, rays_o, rays_d, positions, log_scales, quats, cand, offsets,
                                                  freq, att, W1, b1, W2, b2, W3, b3, feat_attr, grad_out_feat, beta,
                                                  temp, Wimg, Himg, TW, TH, thr):
        """grad_feat_attr (shaped like ``feat_attr``) of the tile-centre-order feature image for its adjoint
        ``grad_out_feat`` [B,C] (np_tile_kernels.cu:3531-3760, wrapper :6537-6620): every hit adds
        T * alpha * gate_slot * grad_out_feat[pixel] to its primitive's slot rows; geometry, MLP and gates get no
        gradient from the feature image.  The reference traverses the frame with atomics; here the hits come from
        the records forward and are summed per primitive in a fixed order."""
        _chk(int(TW) == int(TH), "square tiles only")
        _chk(feat_attr.is_cuda and feat_attr.dtype == torch.float32 and feat_attr.is_contiguous())
        _chk(feat_attr.dim() in (2, 3) and feat_attr.shape[0] == positions.shape[0])
        _chk(feat_attr.dim() == 2 or feat_attr.shape[1] in (4, 5), "3D feat_attr expects slots in {4,5}")
        pixels = int(Wimg) * int(Himg)
        _chk(grad_out_feat.is_cuda and grad_out_feat.dtype == torch.float32
             and tuple(grad_out_feat.shape) == (pixels, feat_attr.shape[-1]), "grad_out_feat must be [B, C]")
        placeholders = [torch.zeros_like(rays_o), torch.zeros(pixels, device=rays_o.device)]
        x = [rays_o, rays_d, positions, log_scales, quats, cand, offsets, freq, att, W1, b1, W2, b2, W3, b3, *placeholders]
        records = self.render_tiles_training_records(x, Wimg, Himg, TW, thr, float(beta), float(temp), any_tile=True,
                                                     name="render_tiles_backward_featattr_tilecenter")
        return self.feature_gradients_from_records(records, feat_attr, grad_out_feat.contiguous())

    def render_tiles_backward_featattr_per_pixel(self, rays_o, rays_d, positions, log_scales, quats, cand, offsets,
                                                 freq, att, W1, b1, W2, b2, W3, b3, feat_attr, grad_out_feat, beta, temp,
                                                 Wimg, Himg, TW, TH, thr):
        """:meth:`render_tiles_backward_featattr_tilecenter` for the per-pixel order (np_tile_kernels.cu:1211-1422,
        wrapper :6629-6720): the same sums over every pixel's hits in its own depth order."""
        _chk(feat_attr.is_cuda and feat_attr.dtype == torch.float32 and feat_attr.is_contiguous())
        _chk(feat_attr.dim() in (2, 3) and feat_attr.shape[0] == positions.shape[0])
        _chk(feat_attr.dim() == 2 or feat_attr.shape[1] in (4, 5), "3D feat_attr expects slots in {4,5}")
        _chk(grad_out_feat.is_cuda and grad_out_feat.dtype == torch.float32
             and tuple(grad_out_feat.shape) == (int(Wimg) * int(Himg), feat_attr.shape[-1]), "grad_out_feat must be [B, C]")
        base = (rays_o, rays_d, positions, log_scales, quats, cand, offsets, freq, att, W1, b1, W2, b2, W3, b3)
        records = self.render_tiles_per_pixel_records(base, Wimg, Himg, TW, TH, thr, float(beta), float(temp),
                                                      name="render_tiles_backward_featattr_per_pixel")
        return self.feature_gradients_from_records(records, feat_attr, grad_out_feat.contiguous())

    @staticmethod
    def feature_gradients_from_records(records, feat_attr, grad_out_feat, csr=None, groups=None):
        """:meth:`render_tiles_backward_featattr_tilecenter` from records that the caller already holds; ``csr`` and
        ``groups`` when it has grouped them by primitive as well."""
        from .primitive_csr import group_records
        from . import primitive_gemm
        from .record_feature_loss import dense_feature_attribute_gradients
        ids, x6 = records[2], records[3]
        with torch.cuda.device(ids.device):
            if csr is None:
                csr = group_records(ids, x6, torch.empty((ids.numel(), 0), device=ids.device), feat_attr.shape[0])
                groups = None
            if groups is None:
                groups = primitive_gemm.prepare_groups(csr)
            return dense_feature_attribute_gradients(records, csr, grad_out_feat, feat_attr, groups=groups)

    def backward_from_records(self, records, positions, log_scales, quats, freq, att, W1, b1, W2, b2, W3, b3,
                              grad_rgb, grad_t, feat_attr=None, grad_feat=None):
        """The nine gradients of :meth:`render_tiles_backward_tilecenter_full` from records that a forward pass
        already holds (no counterpart in the reference, whose fused backward traverses the frame again).  With
        ``feat_attr`` and ``grad_feat`` the gradient of :meth:`render_tiles_backward_featattr_tilecenter` is appended,
        from the same grouping of the records."""
        from .primitive_csr import group_records, reference_weight_gradients
        from . import primitive_gemm
        rgb, alpha, ids, x6, raw, masks, gates, pixel_offsets = records
        x = {15: grad_rgb.contiguous(), 16: grad_t.contiguous()}
        # reverse walk without atomics; the geometry sums are formed from the primitive-major order that the
        # weight gradients need anyway
        with torch.cuda.device(ids.device):
            d4, falloff_adjoint = ops.records_reverse_adjoints(ids, pixel_offsets, raw, x[15], x[16])
            weights = [W1, b1, W2, b2, W3, b3]
            csr = group_records(ids, x6, d4, positions.shape[0], masks)
            groups = primitive_gemm.prepare_groups(csr)
            gp, gs, gq = ops.geometry_gradients(csr.offsets, csr.record_indices, csr.x6, falloff_adjoint, log_scales,
                                                quats, groups)
        if tuple(W1.shape[1:]) == (32, 72) and freq.numel() == 6:
            grads = primitive_gemm.grouped_weight_gradients(csr, freq, att, weights, dtype=torch.float32, groups=groups)
        else:   # other MLP shapes: the dense chain per primitive (small scenes and tests only)
            grads = reference_weight_gradients(csr, freq, att, weights)
        if feat_attr is not None and grad_feat is not None:
            return [*grads, gp, gs, gq, self.feature_gradients_from_records(records, feat_attr, grad_feat, csr, groups)]
        return [*grads, gp, gs, gq]

    # ------------------------------------------------------------------------------------------
    # statistics forward (pruning statistics are not rebuilt; the render itself is)
    # ------------------------------------------------------------------------------------------
    def render_tiles_forward_tilecenter_stats(self, rays_o, rays_d, positions, log_scales, quats, cand, offsets,
                                              freq, att, F, W1, b1, W2, b2, W3, b3, N, H, IN, Wimg, Himg, TW, TH, thr,
                                              gt_rgb, stat_sum_w, stat_max_w, stat_hits, stat_sum_werr,
                                              stat_contrib_count):
        """(rgb, alpha) in centre-depth order; the five per-primitive statistic buffers are updated in
        place (np_tile_kernels.cu:2139-2519, wrapper :5349-5428)."""
        _chk(0 < int(TW) * int(TH) <= 256, "Tile-center order kernel currently supports 0 < TW*TH <= 256")
        for t in (stat_sum_w, stat_max_w, stat_sum_werr):
            _chk(t.is_cuda and t.dtype == torch.float32 and t.numel() == N and t.is_contiguous())
        for t in (stat_hits, stat_contrib_count):
            _chk(t.is_cuda and t.dtype == torch.int32 and t.numel() == N and t.is_contiguous())
        _chk(int(N) == positions.shape[0], "N must be the primitive count")
        _chk(gt_rgb.is_cuda and gt_rgb.dtype == torch.float32 and tuple(gt_rgb.shape) == (int(Himg) * int(Wimg), 3))
        args = (rays_o, rays_d, positions, log_scales, quats, cand, offsets, freq, att, W1, b1, W2, b2, W3, b3,
                Wimg, Himg, TW, TH, thr)
        rgb, alpha, _ = self._tilecenter(args, "render_tiles_forward_tilecenter_stats", _lib.KEY_DEPTH,
                                         self.max_tile_prims, hidden_limit=64,
                                         stats=(gt_rgb.contiguous(), stat_sum_w, stat_max_w, stat_hits, stat_sum_werr,
                                                stat_contrib_count))
        return rgb, alpha

    # ------------------------------------------------------------------------------------------
    # reduced-precision matrix-core path (rgb_wmma.cuh:225-274)
    # ------------------------------------------------------------------------------------------
    def rgb_wmma_safety_stats(self):
        return [self._mfma_calls, self._mfma_fallbacks]

    @staticmethod
    def _source_key(tensors, extra=()):
        """Cache key of a derived tensor: address, in-place version, shape and device of every source.  None for
        inference tensors, which carry no version counter (an edit could not be seen: no caching)."""
        try:
            return tuple(extra) + tuple((t.data_ptr(), t._version, tuple(t.shape), str(t.device)) for t in tensors)
        except RuntimeError:
            return None

    @staticmethod
    def _held_only_here(sources):
        """True when the cache entry's own references are all that keeps the sources' memory allocated (their
        owner -- a scene module -- is gone): nobody else holds these tensor objects, and nobody holds another tensor
        on their storages (a tensor handed in is usually a fresh ``detach()`` of a parameter: then the tensor object
        is the entry's alone and the parameter shows in the storage's holder count)."""
        count = getattr(torch._C, "_storage_Use_Count", None)
        if count is None:
            return False
        try:
            mine = {}
            for t in sources:
                # the entry's tuple (once per occurrence), this loop variable and getrefcount's own argument
                if sys.getrefcount(t) > sum(1 for u in sources if u is t) + 2:
                    return False
                mine.setdefault(t.untyped_storage()._cdata, set()).add(id(t))
            # (+1: the wrapper untyped_storage() makes for the question itself)
            return all(count(c) <= len(tensors) + 1 for c, tensors in mine.items())
        except Exception:
            return False

    def _derived(self, slot, sources, extra, build):
        """``build()`` once per state of ``sources``; a slot keeps the derived tensors of the last
        ``MLPSP_CACHE_SCENES`` (default 2) source states, most recent first, so that two scenes rendered in turn
        do not rebuild each other's copies.  An entry keeps the source tensors themselves: while it lives their
        memory cannot be freed and handed to another scene's tensors of the same shape, whose key would then match
        (the address is only an identity for memory that is still allocated).  Entries whose sources nothing else
        holds any more are dropped on the next call; :meth:`invalidate_caches` drops everything."""
        if not self._caching():
            return build()
        key = self._source_key(sources, extra)
        if key is None:
            return build()
        with self._lock:
            entries = getattr(self, slot) or []
            for i, entry in enumerate(entries):
                if entry[0] == key:
                    if i:
                        entries.insert(0, entries.pop(i))
                    return entry[1]
            depth = max(1, int(os.environ.get("MLPSP_CACHE_SCENES", "2")))
            entries = [e for e in entries if not self._held_only_here(e[2])][:depth - 1]
            entry = (key, build(), tuple(sources))
            setattr(self, slot, [entry] + entries)
            return entry[1]

    def _records(self, positions, log_scales, quats):
        """Per-primitive geometry records, rebuilt only when one of the three tensors changed."""
        return self._derived("_rec", (positions, log_scales, quats), (),
                             lambda: ops.prepare_primitives(positions, log_scales, quats))

    def _packed_weights(self, ws, bf16):
        """Matrix-core operand copy of the six weight tensors, rebuilt only when one of them changed
        (identity, shape or in-place version) -- the scene's weights are constant during inference."""
        return self._derived("_pack", tuple(ws), (bool(bf16),), lambda: ops.pack_mfma_weights(*ws, bf16=bf16))

    def _packed_feat(self, feat_attr):
        """fp16 operand copy of the feature attributes, cached like the weights -> (packed, nonfinite)."""
        return self._derived("_feat_pack", (feat_attr,), (), lambda: ops.pack_mfma_feat(feat_attr))

    def render_tiles_rgb_wmma(self, x, width, height, threshold, bf16):
        """[rgb, alpha] with the 72->32->32->4 MLP on the matrix cores, f32 everywhere else."""
        return self._rgb_wmma(x, None, width, height, threshold, bf16, "render_tiles_rgb_wmma")

    def render_tiles_rgb_wmma_with_feat(self, x, feat_attr, beta, temp, width, height, threshold, bf16):
        """[rgb, alpha, feat]: the matrix-core render with the gated feature channel composited by the
        same weights (feature semantics of np_tile_kernels.cu:6036-6075; the reference's tensor-core
        kernel itself is RGB only)."""
        _chk(feat_attr.is_cuda and feat_attr.dtype in (torch.float32, torch.float16) and feat_attr.dim() in (2, 3),
             "feat_attr must be a CUDA float32 tensor with 2 or 3 dimensions")
        _chk(feat_attr.shape[0] == x[2].shape[0], "feat_attr first dimension must match primitive count")
        ops._feat_shape(feat_attr, allow_half=True)
        return self._rgb_wmma(x, (feat_attr.contiguous(), float(beta), float(temp)), width, height, threshold, bf16,
                              "render_tiles_rgb_wmma_with_feat")

    def _rgb_wmma(self, x, feat, width, height, threshold, bf16, name):
        _chk(len(x) == 15, "WMMA requires the 15 scene tensors")
        width, height, threshold = int(width), int(height), float(threshold)
        _chk(width > 0 and height > 0 and 0.0 < threshold < 1.0)
        _chk(width <= 2147483647 and height <= 2147483647 and width <= 2147483647 // height,
             "WMMA image dimensions exceed int32 pixel indexing")
        # The six MLP tensors may all be stored as fp16 (an inference export kept as it is on disk: the operand blocks
        # are then packed straight from that storage); everything else is f32 as in the reference's entry point.
        half_weights = all(t.dtype == torch.float16 for t in x[9:15])
        for i, t in enumerate(x):
            _chk(t.is_cuda and t.is_contiguous() and t.device == x[0].device)
            _chk(t.dtype == (torch.int32 if i in (5, 6) else torch.float16 if (half_weights and i >= 9) else torch.float32))
        pixels, n = width * height, x[2].shape[0]
        _chk(tuple(x[0].shape) == (pixels, 3) and x[1].shape == x[0].shape)
        _chk(x[2].dim() == 2 and x[2].shape[1] == 3 and x[3].shape == x[2].shape)
        _chk(tuple(x[4].shape) == (n, 4))
        _chk(x[7].dim() == 1 and x[7].numel() == 6 and x[8].shape == x[7].shape)
        _chk(tuple(x[9].shape) == (n, 32, 72) and tuple(x[10].shape) == (n, 32))
        _chk(tuple(x[11].shape) == (n, 32, 32) and x[12].shape == x[10].shape)
        _chk(tuple(x[13].shape) == (n, 4, 32) and tuple(x[14].shape) == (n, 4))
        with torch.cuda.device(x[0].device):
            self._validate(x[5], x[6], ops.num_tiles(width, height, 8, 8), self.max_tile_prims, n, name)
            with self._lock:
                self._mfma_calls += 1
            rec = self._records(x[2], x[3], x[4])
            order = x[5]
            if x[5].numel() > 0:
                order, _ = ops.sort_tiles(x[0], x[1], rec, x[5], x[6], width, height, 8, 8, _lib.KEY_TSTAR,
                                          self.max_tile_prims, cull_threshold=threshold)
            packed = self._packed_weights(list(x[9:15]), bool(bf16))
            packed_feat = None
            if feat is not None:
                packed_feat, bad_attr = self._packed_feat(feat[0])
                if bad_attr:                      # e.g. |attr| beyond the fp16 range: exact path instead
                    warnings.warn("feature attributes overflow fp16: "
                                  "rendering this frame with scalar FP32 instead")
                    with self._lock:
                        self._mfma_fallbacks += 1
                    return list(ops.render_tilecenter_feat_f32(x[0], x[1], rec, order, x[6], x[7], x[8],
                                                               *[w.float() for w in x[9:15]], feat[0].float(), feat[1],
                                                               feat[2], width, height, 8, 8, threshold))
            if feat is None:
                rgb, alpha, nonfinite = ops.render_tilecenter_mfma(x[0], x[1], rec, order, x[6], x[7], x[8], *x[9:15],
                                                                   width, height, threshold, bf16=bool(bf16),
                                                                   packed=packed)
                out = [rgb, alpha]
            else:
                rgb, alpha, fmap, nonfinite = ops.render_tilecenter_mfma_feat(
                    x[0], x[1], rec, order, x[6], x[7], x[8], *x[9:15], feat[0], feat[1], feat[2], width, height,
                    threshold, bf16=bool(bf16), packed=packed, packed_feat=packed_feat)
                out = [rgb, alpha, fmap]
            if nonfinite:
                for i, t in enumerate(x):
                    if i not in (5, 6):
                        _chk(bool(torch.isfinite(t).all()), "WMMA input is nonfinite; refusing fallback")
                warnings.warn("WMMA operand/activation overflow: rendering this frame with scalar FP32 instead")
                with self._lock:
                    self._mfma_fallbacks += 1
                wide = [w.float() for w in x[9:15]]
                if feat is None:
                    out = list(ops.render_tilecenter_f32(x[0], x[1], rec, order, x[6], x[7], x[8], *wide, width,
                                                         height, 8, 8, threshold))[:2]
                else:
                    out = list(ops.render_tilecenter_feat_f32(x[0], x[1], rec, order, x[6], x[7], x[8], *wide,
                                                              feat[0].float(), feat[1], feat[2], width, height, 8, 8,
                                                              threshold))
                _chk(all(bool(torch.isfinite(t).all()) for t in out), "Scalar FP32 fallback output is nonfinite")
        return out
