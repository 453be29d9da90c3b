"""Host-side policy of the grouped MLP weight-gradient path, with the API of the reference's
``scannet/primitive_gemm.py``: segment layout of a primitive-major CSR, its identity/version guards, the
non-finite retry policy and its counters, and argument validation of ``grouped_weight_gradients``.

The device kernels behind ``_launch_grouped_vjp`` (Triton in the reference, scannet/primitive_gemm.py:101-183)
are the HIP kernels ``mlpsp_grouped_vjp`` / ``mlpsp_reduce_partials`` of libmlpsp_hip: one wavefront per segment,
32x32 MFMA tiles, f32 accumulation over the segment.
"""
from __future__ import annotations

import math
import warnings
from dataclasses import dataclass

import torch

PACKED_GRADIENT_SIZES = (2304, 32, 1024, 32, 128, 4)   # W1 | b1 | W2 | b2 | W3 | b3 = 3524 (scannet/primitive_gemm.py:160-166)
_EXPECTED_SHAPES = [(32, 72), (32,), (32, 32), (32,), (4, 32), (4,)]


def _require_segment_size(segment_size) -> None:
    if isinstance(segment_size, bool) or not isinstance(segment_size, int) or segment_size <= 0:
        raise ValueError("segment_size must be a positive integer")


@dataclass(frozen=True)
class GroupLayout:
    """Segments of at most ``segment_size`` records, each owned by one primitive, tied to the CSR they
    were cut from (scannet/primitive_gemm.py:21-52)."""
    primitives: torch.Tensor
    starts: torch.Tensor
    offsets: torch.Tensor
    segment_size: int
    source_offsets: torch.Tensor
    num_records: int
    tensor_versions: tuple

    def __iter__(self):
        yield self.primitives
        yield self.starts
        yield self.offsets

    def _guarded(self):
        return (self.source_offsets, self.primitives, self.starts, self.offsets)

    def validate(self, csr, segment_size):
        if segment_size != self.segment_size:
            raise ValueError(f"Prepared groups use segment_size={self.segment_size}, "
                             f"but the consumer requested {segment_size}")
        if csr.offsets is not self.source_offsets or len(csr.x6) != self.num_records:
            raise ValueError("Prepared groups belong to a different CSR layout")
        if tuple(t._version for t in self._guarded()) != tuple(self.tensor_versions):
            raise ValueError("Prepared groups or their CSR offsets were modified in place")
        return self


_SAFETY_STATS = {"calls": 0, "mixed_calls": 0, "fp32_fallbacks": 0, "fp32_nonfinite_failures": 0}


def get_grouped_vjp_safety_stats(*, reset=False):
    """Copy of the process-local counters; ``reset=True`` zeroes them afterwards."""
    stats = dict(_SAFETY_STATS)
    if reset:
        for name in list(_SAFETY_STATS):
            _SAFETY_STATS[name] = 0
    return stats


def _checked_grouped_vjp(launch, dtype, loss_scale):
    """Run ``launch(dtype, loss_scale) -> (result, nonfinite_flag)``; a non-finite reduced-precision result is
    retried once in unscaled f32, a non-finite f32 result raises (scannet/primitive_gemm.py:67-98).
    A finite result is returned untouched."""
    reduced = dtype != torch.float32
    _SAFETY_STATS["calls"] += 1
    if reduced:
        _SAFETY_STATS["mixed_calls"] += 1
    result, flag = launch(dtype, loss_scale)
    if not bool(flag.item()):
        return result
    if reduced:
        _SAFETY_STATS["fp32_fallbacks"] += 1
        warnings.warn(f"[CSR safety] Nonfinite {dtype} MLP VJP; retrying with IEEE FP32 before Adam "
                      f"(FP32 fallbacks={_SAFETY_STATS['fp32_fallbacks']}).", RuntimeWarning, stacklevel=2)
        result, flag = launch(torch.float32, 1.0)
        if not bool(flag.item()):
            return result
    _SAFETY_STATS["fp32_nonfinite_failures"] += 1
    raise FloatingPointError("[CSR safety] IEEE FP32 MLP VJP is nonfinite; no gradients were returned and Adam must "
                             "not step. Inspect the saved model, records and loss. "
                             f"Safety counters: {get_grouped_vjp_safety_stats()}")


def prepare_groups(csr, segment_size=512):
    """Cut every primitive's record range into ceil(count / segment_size) segments (scannet/primitive_gemm.py:186-201)."""
    _require_segment_size(segment_size)
    off = csr.offsets
    if off.ndim != 1 or off.dtype != torch.int64 or not off.is_contiguous():
        raise ValueError("CSR offsets must be contiguous int64")
    if off.numel() < 1:
        raise ValueError("CSR offsets must include the initial zero")
    per_primitive = (off.diff() + (segment_size - 1)) // segment_size
    group_offsets = torch.zeros(per_primitive.numel() + 1, dtype=per_primitive.dtype, device=per_primitive.device)
    group_offsets[1:] = per_primitive.cumsum(0)
    total = int(group_offsets[-1])
    owner = torch.repeat_interleave(torch.arange(per_primitive.numel(), device=off.device), per_primitive,
                                    output_size=total)
    within = torch.arange(total, device=off.device) - group_offsets[owner]
    starts = off[owner] + within * segment_size
    versions = tuple(t._version for t in (off, owner, starts, group_offsets))
    return GroupLayout(owner, starts, group_offsets, segment_size, off, len(csr.x6), versions)


def resolve_groups(csr, segment_size=512, groups=None):
    """``groups`` if it is a layout of this CSR and segment size, else a fresh one (scannet/primitive_gemm.py:204-212)."""
    _require_segment_size(segment_size)
    if groups is None:
        return prepare_groups(csr, segment_size)
    if not isinstance(groups, GroupLayout):
        raise TypeError("groups must be a GroupLayout returned by prepare_groups")
    return groups.validate(csr, segment_size)


_PRECISION_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def _launch_grouped_vjp(csr, freq, attenuation, weights, groups, dtype, block_size, scale, split=False):
    """(result [n,3524] f32, nonfinite flag [1] int32): per-segment partial gradients, then their sum per
    primitive (scannet/primitive_gemm.py:214-230).  ``block_size`` only chose the Triton tile height; the
    HIP kernel always walks a segment in blocks of 32 records.  ``split``: the result is the list of the six
    gradient tensors, written in place by the summing kernel instead of being cut out of packed rows."""
    from . import _lib
    lib = _lib.load()
    group_primitives, group_starts, group_offsets = groups
    device = weights[0].device
    n = len(weights[0])
    num_groups = int(group_primitives.numel())
    partial = torch.empty((max(int(lib.mlpsp_segment_reduce_rows(num_groups)), 1), sum(PACKED_GRADIENT_SIZES)),
                          dtype=torch.float32, device=device)       # per-segment sums + the reduction's chunk sums
    if split:
        result = [torch.empty_like(w) for w in weights]
    else:
        result = torch.empty((n, sum(PACKED_GRADIENT_SIZES)), dtype=torch.float32, device=device)
    flag = torch.zeros(1, dtype=torch.int32, device=device)
    stream = torch.cuda.current_stream(device).cuda_stream
    masks = csr.relu_masks
    with torch.cuda.device(device):
        rc = lib.mlpsp_grouped_vjp(csr.x6.data_ptr(), csr.grad4.data_ptr(), masks.data_ptr() if masks is not None else None,
                                   csr.offsets.data_ptr(), group_primitives.data_ptr(), group_starts.data_ptr(),
                                   num_groups, freq.data_ptr(), attenuation.data_ptr(), *[w.data_ptr() for w in weights[:5]],
                                   _PRECISION_CODE[dtype], float(scale), int(groups.segment_size), partial.data_ptr(),
                                   stream)
        if rc != 0:
            raise RuntimeError(f"mlpsp_grouped_vjp: {_lib.strerror(rc)}")
        if split:
            rc = lib.mlpsp_reduce_partials_split(partial.data_ptr(), group_primitives.data_ptr(), group_offsets.data_ptr(),
                                                 num_groups, n, *[r.data_ptr() for r in result], flag.data_ptr(), stream)
        else:
            rc = lib.mlpsp_reduce_partials(partial.data_ptr(), group_primitives.data_ptr(), group_offsets.data_ptr(),
                                           num_groups, n, result.data_ptr(), flag.data_ptr(), stream)
        if rc != 0:
            raise RuntimeError(f"mlpsp_reduce_partials: {_lib.strerror(rc)}")
    return result, flag


@torch.no_grad()
def grouped_weight_gradients(csr, freq, attenuation, weights, *, dtype=torch.float16, segment_size=512, block_size=32,
                             loss_scale=None, groups=None):
    """Argument contract of scannet/primitive_gemm.py:233-279 for the 72->32->32->4 MLP, then the guarded launch."""
    n = len(weights[0])
    if [tuple(w.shape[1:]) for w in weights] != _EXPECTED_SHAPES:
        raise ValueError("grouped backward requires the 72→32→32→4 architecture")
    if any(len(w) != n for w in weights) or csr.offsets.numel() != n + 1:
        raise ValueError("CSR offsets and all master tensors must have the same primitive count")
    if csr.x6.ndim != 2 or csr.x6.shape[1] != 6 or tuple(csr.grad4.shape) != (len(csr.x6), 4):
        raise ValueError("CSR inputs/adjoints must have shapes (records,6) and (records,4)")
    if freq.numel() != 6 or attenuation.numel() != 6:
        raise ValueError("grouped backward requires six positional frequencies")
    if dtype not in (torch.float32, torch.float16, torch.bfloat16):
        raise ValueError("unsupported GEMM operand dtype")
    if block_size not in (32, 64) or segment_size <= 0 or segment_size % block_size:
        raise ValueError("segment size must be a positive multiple of the 32/64-row block")
    device = weights[0].device
    for t in (csr.offsets, csr.x6, csr.grad4, freq, attenuation, *weights):
        if not t.is_cuda or not t.is_contiguous() or t.device != device:
            raise ValueError("all inputs must be contiguous tensors on one CUDA device")
    if any(t.dtype != torch.float32 for t in (csr.x6, csr.grad4, freq, attenuation, *weights)):
        raise ValueError("master weights, records and encoding parameters must be FP32")
    masks = csr.relu_masks
    if masks is not None and (masks.dtype != torch.int32 or not masks.is_contiguous() or masks.device != device
                              or tuple(masks.shape) != (len(csr.x6), 2)):
        raise ValueError("saved ReLU masks must be contiguous CUDA int32 with shape (records,2)")
    groups = resolve_groups(csr, segment_size, groups)
    if loss_scale is None:
        scale = 4096.0 if dtype == torch.float16 else 1.0
    else:
        scale = float(loss_scale)
    if not math.isfinite(scale) or scale <= 0:
        raise ValueError("loss_scale must be finite and strictly positive")

    def launch(operand_dtype, operand_scale):
        return _launch_grouped_vjp(csr, freq, attenuation, weights, groups, operand_dtype, block_size, operand_scale,
                                   split=True)

    return _checked_grouped_vjp(launch, dtype, scale)
