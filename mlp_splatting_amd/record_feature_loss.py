"""Streamed feature L1 loss from saved splat records, with the API of the reference's
``scannet/record_feature_loss.py`` (``streaming_feature_l1``, ``feature_weight_gradients``).

The exact high-resolution feature blend is sampled with the bilinear down-sampling operator
(``F.interpolate(..., mode="bilinear", align_corners=False)``) without ever materialising the 512-D image; only
int8 signs of the residual and scalar loss partials are kept.  Geometry, alpha and the MLP are constants of this
loss (scannet/record_feature_loss.py:1-6).  The kernels are libmlpsp_hip's ``mlpsp_stream_feature_l1`` and
``mlpsp_feature_attribute_gradients``.
"""
from __future__ import annotations

import os

import torch

from . import _lib


def _ptr(t):
    return None if t is None else t.data_ptr()


def _launch_order(pixels, csr, starts):
    """Segments sorted by their first pixels (int64 permutation, or None): workgroups that run together then read
    neighbouring rows of the adjoint (or sign) image and find them in L2.  MLPSP_FEATURE_VJP_ORDER=primitive keeps
    the primitive-major launch order; the sums do not depend on it."""
    if len(starts) < 2 or os.environ.get("MLPSP_FEATURE_VJP_ORDER", "pixel") == "primitive":
        return None
    return torch.argsort(pixels[csr.record_indices[starts]].to(torch.int64))


def _loss_geometry(attributes, target, record_tensors, width, height):
    """(target height, target width, channels, slots) after the argument checks of the streamed loss
    (the conditions and texts of scannet/record_feature_loss.py:66-82, which callers and tests match)."""
    on_one_gpu = all(t.is_cuda and t.device == attributes.device for t in (*record_tensors, attributes, target))
    slots = attributes.shape[1] if attributes.ndim == 3 else 1
    shape_ok = target.ndim == 3 and min(target.shape) > 0
    for ok, text in (
            (shape_ok, "feature target must have nonempty HWC dimensions"),
            (attributes.dtype == torch.float32 and attributes.is_contiguous(),
             "feature master attributes must be contiguous FP32"),
            (target.dtype in (torch.float16, torch.float32), "feature target must be FP16 or FP32"),
            (on_one_gpu, "feature tensors and records must share a CUDA device"),
            (slots in (1, 4, 5) and shape_ok and attributes.shape[-1] == target.shape[-1],
             "feature shape does not match the 1/4/5-slot renderer"),
            (shape_ok and target.shape[0] <= height and target.shape[1] <= width,
             "streamed feature loss supports downsampling only")):
        if not ok:
            raise ValueError(text)
    return target.shape[0], target.shape[1], target.shape[2], slots


def streaming_feature_l1(records, attributes, target, width, height, *, debug=False):
    """(loss, signs int8 [hf, wf, C], prediction or None) -- scannet/record_feature_loss.py:66-89."""
    ids, raw, gates, offsets = records[2], records[4], records[6], records[7]
    hf, wf, channels, slots = _loss_geometry(attributes, target, (ids, offsets, raw, gates), width, height)
    target = target.contiguous()
    device = target.device
    signs = torch.empty(target.shape, device=device, dtype=torch.int8)
    partial = torch.empty((hf * wf, (channels + 127) // 128), device=device, dtype=torch.float32)
    pred = torch.empty(target.shape, device=device, dtype=torch.float32) if debug else None
    with torch.cuda.device(device):
        rc = _lib.load().mlpsp_stream_feature_l1(
            _ptr(ids), _ptr(offsets), _ptr(raw), _ptr(gates), _ptr(attributes), _ptr(target),
            int(target.dtype == torch.float16), int(width), int(height), int(wf), int(hf), int(channels), int(slots),
            _ptr(signs), _ptr(partial), _ptr(pred), torch.cuda.current_stream(device).cuda_stream)
    if rc != 0:
        raise RuntimeError(f"mlpsp_stream_feature_l1: {_lib.strerror(rc)}")
    return partial.sum(), signs, pred


class _SegmentPlan:
    """What both attribute-gradient kernels need beside their adjoint: the segments of the primitive-major record
    grouping, the pixel of every record, the buffer of per-segment sums and the launch order."""

    def __init__(self, records, csr, num_pixels, attributes, segment_size, groups):
        from .primitive_gemm import resolve_groups
        ids, pixel_offsets = records[2], records[7]
        dev = ids.device
        self.primitives, self.starts, self.group_offsets = resolve_groups(csr, segment_size, groups)
        # record -> pixel: pixel p owns records [pixel_offsets[p], pixel_offsets[p + 1])
        self.pixels = torch.repeat_interleave(torch.arange(num_pixels, device=dev, dtype=torch.int32),
                                              pixel_offsets.diff(), output_size=len(ids))
        self.slots = attributes.shape[1] if attributes.ndim == 3 else 1
        self.channels = attributes.shape[-1]
        # per-segment sums followed by the chunk sums of the reduction over a primitive's segments
        rows = int(_lib.load().mlpsp_segment_reduce_rows(len(self.primitives)))
        self.partial = torch.empty((max(rows, 1), self.slots, self.channels), device=dev, dtype=torch.float32)
        self.order = _launch_order(self.pixels, csr, self.starts)
        self.device = dev


def feature_weight_gradients(records, csr, signs, attributes, width, height, *, mixed=True, segment_size=512,
                             groups=None):
    """d loss / d attributes, shaped like ``attributes``, from the residual signs the streamed loss kept
    (API, checks and error texts of scannet/record_feature_loss.py:164-185)."""
    if signs.dtype != torch.int8 or not signs.is_contiguous():
        raise ValueError("feature loss signs must be contiguous int8")
    low_h, low_w, channels = signs.shape
    if low_h > height or low_w > width:
        raise ValueError("streamed feature loss supports downsampling only")
    plan = _SegmentPlan(records, csr, width * height, attributes, segment_size, groups)
    raw, gates = records[4], records[6]
    result = torch.empty_like(attributes)
    with torch.cuda.device(plan.device):
        rc = _lib.load().mlpsp_feature_attribute_gradients(
            _ptr(signs), _ptr(csr.record_indices), _ptr(plan.pixels), _ptr(raw), _ptr(gates), _ptr(csr.offsets),
            _ptr(plan.primitives), _ptr(plan.starts), _ptr(plan.group_offsets), _ptr(plan.order),
            int(len(plan.primitives)), int(len(attributes)), int(width), int(height), int(low_w), int(low_h),
            int(channels), int(plan.slots), int(segment_size), int(bool(mixed)), _ptr(plan.partial), _ptr(result),
            torch.cuda.current_stream(plan.device).cuda_stream)
    if rc != 0:
        raise RuntimeError(f"mlpsp_feature_attribute_gradients: {_lib.strerror(rc)}")
    return result


@torch.no_grad()
def dense_feature_attribute_gradients(records, csr, grad_feature, attributes, *, segment_size=512, groups=None):
    """Adjoint of the dense feature image with respect to ``attributes`` (shaped like them), from saved records:
    what ``render_tiles_backward_featattr_tilecenter`` returns to ``_TileRenderWithFeatAutogradFn.backward``
    (scannet/cumodel.py:466-477; kernel scannet/cuda/np_tile_kernels.cu:3531-3760).  ``grad_feature`` [pixels, C]
    f32; geometry, alpha and the gates are constants of the feature image, as in the reference."""
    num_pixels = records[7].numel() - 1
    slots = 1 if attributes.ndim == 2 else attributes.shape[1]
    if slots not in (1, 4, 5):
        raise RuntimeError("feat_attr must be [N,C] or [N,S,C] with slots in {4,5}")
    if (grad_feature.dtype != torch.float32 or not grad_feature.is_contiguous()
            or tuple(grad_feature.shape) != (num_pixels, attributes.shape[-1])):
        raise ValueError("the feature adjoint must be contiguous float32 [pixels, channels]")
    if attributes.dtype != torch.float32:
        raise ValueError("feature attributes must be float32")
    plan = _SegmentPlan(records, csr, num_pixels, attributes, segment_size, groups)
    raw, gates = records[4], records[6]
    result = torch.empty(attributes.shape, device=plan.device, dtype=torch.float32)
    with torch.cuda.device(plan.device):
        rc = _lib.load().mlpsp_feature_dense_attribute_gradients(
            _ptr(grad_feature), _ptr(csr.record_indices), _ptr(plan.pixels), _ptr(raw), _ptr(gates), _ptr(csr.offsets),
            _ptr(plan.primitives), _ptr(plan.starts), _ptr(plan.group_offsets), _ptr(plan.order),
            int(len(plan.primitives)), int(len(attributes)), int(plan.channels), int(slots), int(segment_size),
            _ptr(plan.partial), _ptr(result), torch.cuda.current_stream(plan.device).cuda_stream)
    if rc != 0:
        raise RuntimeError(f"mlpsp_feature_dense_attribute_gradients: {_lib.strerror(rc)}")
    return result
