"""One training step on saved splat records: image + streamed feature L1 loss from a single records forward.

What the reference's ``scannet/csr_training.py`` provides to ``scannet/cumodel.py:1098-1108``: a differentiable
``(rgb, feature_loss)`` whose backward never traverses the frame again.  The adjoints come from the records the
forward kept -- reverse compositing, one primitive-major grouping, grouped MLP weight gradients, geometry sums
and the attribute gradient of the streamed loss -- all libmlpsp_hip kernels.

Environment (names shared with the reference so that its launch scripts keep working):
  MLPSP_CSR_FORWARD_BACKEND  scalar | wmma_fp16 | wmma_bf16   which records forward runs
  MLPSP_CSR_MLP_PRECISION    float32 | float16 | bfloat16     operand precision of the grouped weight gradients
"""
from __future__ import annotations

import os
from dataclasses import dataclass

import torch

from . import primitive_csr, primitive_gemm, record_feature_loss

_FORWARD_BACKENDS = {"scalar": None, "wmma_fp16": "float16", "wmma_bf16": "bfloat16"}
_GRADIENT_PRECISIONS = ("float32", "float16", "bfloat16")
_NUM_SCENE_TENSORS = 15      # rays_o .. b3, the extension's positional order


@dataclass(frozen=True)
class Frame:
    width: int
    height: int
    threshold: float
    gating_beta: float
    gating_temp: float


def records_forward(ext, scene_tensors, frame: Frame):
    """[rgb, alpha, ids, x6, raw, masks, gates, offsets] from the records forward that
    MLPSP_CSR_FORWARD_BACKEND names.  ``scene_tensors``: the 15 scene tensors; the two adjoint placeholders the
    extension's signature carries are appended here."""
    name = os.environ.get("MLPSP_CSR_FORWARD_BACKEND", "scalar").strip().lower()
    if name not in _FORWARD_BACKENDS:
        raise ValueError("MLPSP_CSR_FORWARD_BACKEND must be scalar, wmma_fp16 or wmma_bf16")
    rays = scene_tensors[0]
    x = [*scene_tensors[:_NUM_SCENE_TENSORS], torch.zeros_like(rays), rays.new_zeros(rays.shape[0])]
    geometry = (frame.width, frame.height, 8, frame.threshold, frame.gating_beta, frame.gating_temp)
    operand = _FORWARD_BACKENDS[name]
    if operand is None:
        return ext.render_tiles_training_records(x, *geometry)
    return ext.render_tiles_training_records_wmma(x, *geometry, operand)


def _gradient_precision():
    name = os.environ.get("MLPSP_CSR_MLP_PRECISION", "float16")
    if name not in _GRADIENT_PRECISIONS:
        raise ValueError("MLPSP_CSR_MLP_PRECISION must be float32, float16 or bfloat16")
    return name


class _RecordStep(torch.autograd.Function):
    """inputs: frame, background (tensor or None), attributes, target, then the 15 scene tensors."""

    @staticmethod
    def forward(ctx, frame, background, attributes, target, *scene_tensors):
        from .cumodel import NeuralPrimitiveSceneTileCUDA
        if scene_tensors[7].numel() != 6 or tuple(scene_tensors[9].shape[1:]) != (32, 72):
            raise ValueError("CSR training currently supports only the released 72→32→32→4 MLP")
        ctx.gradient_precision = _gradient_precision()
        ext = NeuralPrimitiveSceneTileCUDA._ensure_tile_ext_static(8)
        records = records_forward(ext, list(scene_tensors), frame)
        loss, signs, _ = record_feature_loss.streaming_feature_l1(records, attributes, target, frame.width, frame.height)
        image, alpha = records[0], records[1]
        if background is not None:
            image = image + (1 - alpha).clamp(0, 1) * background.reshape(1, -1)
        ctx.frame, ctx.background, ctx.ext = frame, background, ext
        ctx.save_for_backward(attributes, signs, *records, *scene_tensors)
        ctx.set_materialize_grads(False)
        return image, loss

    @staticmethod
    def backward(ctx, image_adjoint, loss_adjoint):
        attributes, signs, *rest = ctx.saved_tensors
        records, scene = rest[:8], rest[8:]
        _, _, ids, x6, raw, masks, _, pixel_offsets = records
        log_scales, quats, freq, att = scene[3], scene[4], scene[7], scene[8]
        ext, frame = ctx.ext, ctx.frame
        num_primitives = attributes.shape[0]

        geometry = [None, None, None]
        weights = [None] * 6
        if image_adjoint is None:
            d4, falloff = x6.new_zeros((ids.numel(), 4)), None
        else:
            image_adjoint = image_adjoint.contiguous()
            # the background term makes the final transmittance an output: dL/dT_end = <adjoint, background>
            end_adjoint = (image_adjoint.new_zeros(image_adjoint.shape[0]) if ctx.background is None
                           else (image_adjoint * ctx.background.reshape(1, -1)).sum(-1))
            d4, falloff = ext.primitive_records_reverse_adjoints(ids, pixel_offsets, raw, image_adjoint, end_adjoint)
        by_primitive = primitive_csr.group_records(ids, x6, d4, num_primitives, masks)
        segments = primitive_gemm.prepare_groups(by_primitive)
        if falloff is not None:
            geometry = list(ext.primitive_geometry_gradients(by_primitive, falloff, log_scales, quats, segments))
            weights = list(primitive_gemm.grouped_weight_gradients(
                by_primitive, freq, att, scene[9:15], dtype=getattr(torch, ctx.gradient_precision), groups=segments))
        attribute_gradient = None
        if loss_adjoint is not None:
            attribute_gradient = record_feature_loss.feature_weight_gradients(
                records, by_primitive, signs, attributes, frame.width, frame.height, groups=segments,
                mixed=ctx.gradient_precision != "float32") * loss_adjoint
        #        frame bg    attributes          target  rays_o rays_d  positions..quats  lists+tables (4)
        return (None, None, attribute_gradient, None, None, None, *geometry, None, None, None, None, *weights)


def feature_training_step(scene_tensors, attributes, target, frame: Frame, background=None):
    """(rgb [B,3], streamed feature L1 loss) with gradients for positions, log-scales, quaternions, the six MLP
    tensors and the attributes."""
    if len(scene_tensors) != _NUM_SCENE_TENSORS:
        raise ValueError("expected the 15 scene tensors")
    return _RecordStep.apply(frame, background, attributes, target, *scene_tensors)


def render_training_csr(base, attr, target, width, height, threshold, beta, temp, bg):
    """The reference's call signature (scannet/cumodel.py:1103-1108) on :func:`feature_training_step`."""
    return feature_training_step(list(base), attr, target,
                                 Frame(int(width), int(height), float(threshold), float(beta), float(temp)), bg)
