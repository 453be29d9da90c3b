"""Primitive-major grouping of per-hit records, with the API of the reference's
``scannet/primitive_csr.py`` (``PrimitiveCSR``, ``group_records``, ``reference_weight_gradients``).

These are host/torch-level helpers of the training side; they are kept so that code importing them keeps
working.  The forward renderer itself does not use them.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from .cumodel import _encode_x6


@dataclass
class PrimitiveCSR:
    """Records sorted by primitive: primitive p owns rows offsets[p]:offsets[p+1] (scannet/primitive_csr.py:14-20)."""
    offsets: torch.Tensor
    record_indices: torch.Tensor
    x6: torch.Tensor
    grad4: torch.Tensor
    relu_masks: Optional[torch.Tensor] = None


def _gather_rows(t, perm):
    """t[perm] for a 2-D tensor.  Rows of four float32 are gathered as one 16-byte element each: torch's row
    gather takes 8 ms for 39 M such rows on an MI355X, the same bytes as single elements 0.9 ms."""
    if t.dim() == 2 and t.shape[1] == 4 and t.dtype == torch.float32 and t.is_contiguous() and t.is_cuda and t.shape[0] > 0:
        as_elements = torch.view_as_complex(t.view(torch.float64).view(t.shape[0], 1, 2)).reshape(t.shape[0])
        return torch.view_as_real(as_elements[perm]).view(torch.float32).view(t.shape[0], 4)
    return t[perm]


def group_records(primitive_ids, x6, grad4, num_primitives: int, relu_masks=None) -> PrimitiveCSR:
    """Stable grouping by primitive id: inside a group the records keep their original (pixel) order
    (scannet/primitive_csr.py:23-29)."""
    # stable sort once; the per-primitive offsets are then 200k binary searches in the sorted ids (a histogram
    # of 39 M ids takes 10 ms on an MI355X, the sort 1.7 ms)
    sorted_ids, perm = torch.sort(primitive_ids, stable=True)
    bounds = torch.arange(num_primitives + 1, device=primitive_ids.device, dtype=primitive_ids.dtype)
    offsets = torch.searchsorted(sorted_ids, bounds, right=False).to(torch.int64)
    masks = relu_masks[perm] if relu_masks is not None else None
    return PrimitiveCSR(offsets=offsets, record_indices=perm, x6=x6[perm], grad4=_gather_rows(grad4, perm),
                        relu_masks=masks)


@torch.no_grad()
def reference_weight_gradients(csr: PrimitiveCSR, freq, attenuation, weights):
    """[dW1, db1, dW2, db2, dW3, db3] by one dense matmul chain per primitive (scannet/primitive_csr.py:32-58).

    ``grad4`` is the adjoint of the four pre-activation outputs; sigmoid/softplus are already accounted for.
    """
    W1, b1, W2, b2, W3, b3 = weights
    out = [torch.zeros_like(t) for t in weights]
    bounds = csr.offsets.cpu().tolist()
    for p in range(len(bounds) - 1):
        lo, hi = bounds[p], bounds[p + 1]
        if hi == lo:
            continue
        enc = _encode_x6(csr.x6[lo:hi], freq, attenuation)
        a1 = torch.relu(enc @ W1[p].T + b1[p])
        a2 = torch.relu(a1 @ W2[p].T + b2[p])
        g3 = csr.grad4[lo:hi]
        g2 = (g3 @ W3[p]) * (a2 > 0)
        g1 = (g2 @ W2[p]) * (a1 > 0)
        out[0][p], out[1][p] = g1.T @ enc, g1.sum(0)
        out[2][p], out[3][p] = g2.T @ a1, g2.sum(0)
        out[4][p], out[5][p] = g3.T @ a2, g3.sum(0)
    return out
