"""Scene module with the Python-facing API of the reference's ``scannet/cumodel.py``.

Same module-level names (``_tile_ext``, ``_tile_ext_key``, ``_tile_ext_build_config``, the two
encodings, ``_encode_x6``, ``_mlp_forward_indexed``) and the same class
``NeuralPrimitiveSceneTileCUDA`` (constructor arguments, parameter names and shapes, methods,
error behaviour), so that code written against the reference module -- an evaluator, a benchmark
harness, a test that monkeypatches ``_tile_ext`` -- runs against this one.  What differs is below
the API: culling is the sparse HIP binning instead of a dense [tiles x primitives] tensor
expression, and the extension object is ``tile_ext.TileExt`` on ``libmlpsp_hip.so``.

``forward`` renders without a graph under ``torch.no_grad()``; in grad mode with parameters that require
grad it goes through ``_TileRenderAutogradFn`` (RGB) or, with a feature target, through the record-based
training step of ``record_training``.  The dense feature-image backward of the reference is not provided.
"""
from __future__ import annotations

import os
import weakref

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops
from .camera import ray_cone_candidates

# Extension object, created on first use; tests may install their own (scannet/cumodel.py:78-80).
_tile_ext = None
_tile_error = None
_tile_ext_key = None


# The environment is read on every call, as the reference does (a test or a caller may change it between two frames);
# these reads sit between the end of one frame and the first launch of the next, where the device waits for the
# host.  CPython keeps the encoded environment in a plain dict behind os.environ: reading that dict costs a tenth of
# os.environ.get (no key encoding, no default handling in Python code).
_ENV_DATA = getattr(os.environ, "_data", None)
_ENV_KEYS = {}


def _env(name: str, default: str) -> str:
    data = _ENV_DATA
    if type(data) is dict and os.name == "posix":
        key = _ENV_KEYS.get(name)
        if key is None:
            key = _ENV_KEYS[name] = os.fsencode(name)
        value = data.get(key)
        return default if value is None else os.fsdecode(value)
    return os.environ.get(name, default)


_BUILD_CONFIGS = {}


def _tile_ext_build_config(tile_size=None):
    """(key, name, flags) naming the extension build selected by the environment
    (scannet/cumodel.py:96-130).  The capacities the reference bakes in at compile time are run-time
    arguments of this library, but names, accepted values and errors are kept."""
    raw = (_env("MLPSP_NVCC_MAXRREGCOUNT", ""), _env("MLPSP_TILE_CANDIDATE_CAPACITY", "1536"),
           _env("MLPSP_TRAINING_BACKEND", "legacy"), _env("MLPSP_CSR_MAX_HITS", "128"))
    known = _BUILD_CONFIGS.get(raw)
    if known is not None:
        return known[0], known[1], list(known[2])
    config = _tile_ext_build_config_of(*raw)
    if len(_BUILD_CONFIGS) < 64:
        _BUILD_CONFIGS[raw] = (config[0], config[1], tuple(config[2]))
    return config


def _tile_ext_build_config_of(rreg, capacity, backend, csr_hits):
    rreg = rreg.strip()
    flags = []
    suffix = "default"
    capacity = int(capacity)
    if capacity not in {768, 1536}:
        raise ValueError("MLPSP_TILE_CANDIDATE_CAPACITY must be 768 or 1536")
    if backend == "csr":
        hits = int(csr_hits)
        if hits not in {128, 256, 512}:
            raise ValueError("MLPSP_CSR_MAX_HITS must be 128, 256 or 512; overflow is an error")
        flags += ["-DMLPSP_TILECENTER_BLOCK_THREADS=64", "-DMLPSP_BACKWARD_RECOMPUTE_GEOMETRY=1",
                  f"-DMLPSP_TILECENTER_MAX_HITS={hits}", "-DMLPSP_BACKWARD_MIN_BLOCKS_PER_SM=8"]
        suffix = f"csr_h{hits}"
    if capacity != 768:
        flags.append(f"-DMLPSP_MAX_TILE_PRIMS={capacity}")
        suffix += f"_c{capacity}"
    if rreg:
        try:
            value = int(rreg)
        except ValueError:
            value = 0
        if value > 0:
            flags.append(f"-maxrregcount={value}")
            suffix += f"_rreg{value}"
    name = f"np_tile_kernels_{suffix}"
    return (name, tuple(flags)), name, flags


_host_copies = {}


def _unit_directions(ray_d):
    """``F.normalize(ray_d, dim=-1)`` (scannet/cumodel.py:1088); for float32 rays on the device one libmlpsp_hip
    launch that returns the same bits."""
    if ray_d.is_cuda and ray_d.dtype == torch.float32 and ray_d.dim() == 2 and ray_d.shape[1] == 3 \
            and not ray_d.requires_grad:
        from . import ops
        return ops.normalize_rays(ray_d)
    return F.normalize(ray_d, dim=-1).contiguous()


def _frame_matrix(t):
    """The matrix as the queued frame takes it: a float32 device tensor stays where it is (the binning reads it
    there; no copy to the host, no synchronisation), anything else becomes a host copy."""
    if torch.is_tensor(t) and t.is_cuda and t.dtype == torch.float32 and t.numel() == 16:
        return t.detach().contiguous()
    return _host_matrix(t)


def _host_matrix(t):
    """A float32 host copy of a small device tensor (view / projection matrices), remembered for as long
    as that very tensor object is alive and unmodified: the binning reads its matrices on the host, and a
    device-to-host copy per frame is a synchronisation per frame.  The entry is keyed by the object and
    checked through a weak reference and the in-place version, so a new tensor at a recycled address
    never hits."""
    if not torch.is_tensor(t) or not t.is_cuda:
        return t
    try:
        version = t._version
    except RuntimeError:                              # inference tensors carry no version counter
        return t.detach().to("cpu", torch.float32)
    hit = _host_copies.get(id(t))
    if hit is not None and hit[0]() is t and hit[1] == version:
        return hit[2]
    if len(_host_copies) > 512:
        _host_copies.clear()
    host = t.detach().to("cpu", torch.float32)
    try:
        _host_copies[id(t)] = (weakref.ref(t), version, host)
    except TypeError:
        pass
    return host


def _tile_capacity_from_env() -> int:
    return int(os.environ.get("MLPSP_TILE_CANDIDATE_CAPACITY", "1536"))


def _max_hits_from_env() -> int:
    """MLPSP_TILECENTER_MAX_HITS of the selected build: MLPSP_CSR_MAX_HITS in the csr backend
    (scannet/cumodel.py:106-113), else the kernel's default 512 (np_tile_kernels.cu:48-50)."""
    if os.environ.get("MLPSP_TRAINING_BACKEND", "legacy") == "csr":
        return int(os.environ.get("MLPSP_CSR_MAX_HITS", "128"))
    return 512


class IntegratedPositionalEncoding(nn.Module):
    """freq_k = 2^k pi; the attenuation exp(-freq^2 sigma^2 / 2) scales the phase
    (scannet/cumodel.py:132-155)."""

    def __init__(self, in_dim=6, num_frequencies=10, sigma=0.01):
        super().__init__()
        self.in_dim = in_dim
        self.num_frequencies = num_frequencies
        self.sigma2 = sigma ** 2
        self.register_buffer("freq_bands", 2.0 ** torch.linspace(0.0, num_frequencies - 1, num_frequencies) * torch.pi)
        self.register_buffer("runtime_frequency_weights", torch.ones(num_frequencies), persistent=False)

    def set_runtime_frequency_weights(self, weights: torch.Tensor):
        with torch.no_grad():
            self.runtime_frequency_weights.copy_(
                weights.to(device=self.runtime_frequency_weights.device, dtype=self.runtime_frequency_weights.dtype))

    def forward(self, x):
        att = torch.exp(-0.5 * (self.freq_bands ** 2) * self.sigma2) * self.runtime_frequency_weights
        phase = (x[..., None] * self.freq_bands * att).view(*x.shape[:-1], -1)
        return torch.cat([torch.sin(phase), torch.cos(phase)], dim=-1)

    @property
    def out_dim(self):
        return self.in_dim * self.num_frequencies * 2


class FourierFeatureEncoding(nn.Module):
    """freq_k = 2^k, amplitude weights (scannet/cumodel.py:158-180)."""

    def __init__(self, in_dim=6, num_frequencies=10):
        super().__init__()
        self.in_dim = in_dim
        self.num_frequencies = num_frequencies
        self.register_buffer("freq_bands", 2.0 ** torch.linspace(0.0, num_frequencies - 1, num_frequencies))
        self.register_buffer("runtime_frequency_weights", torch.ones(num_frequencies), persistent=False)

    def set_runtime_frequency_weights(self, weights: torch.Tensor):
        with torch.no_grad():
            self.runtime_frequency_weights.copy_(
                weights.to(device=self.runtime_frequency_weights.device, dtype=self.runtime_frequency_weights.dtype))

    def forward(self, x):
        phase = x[..., None] * self.freq_bands
        w = self.runtime_frequency_weights.view(*([1] * (phase.ndim - 1)), self.num_frequencies)
        s = (torch.sin(phase) * w).view(*x.shape[:-1], -1)
        c = (torch.cos(phase) * w).view(*x.shape[:-1], -1)
        return torch.cat([s, c], dim=-1)

    @property
    def out_dim(self):
        return self.in_dim * self.num_frequencies * 2


def _encode_x6(x6: torch.Tensor, freq: torch.Tensor, att: torch.Tensor) -> torch.Tensor:
    """[M,6] -> [M,12F]: all sines (index c*F+f) then all cosines (scannet/cumodel.py:183-190)."""
    phase = x6[:, :, None] * freq[None, None, :] * att[None, None, :]
    m = x6.shape[0]
    return torch.cat([torch.sin(phase).reshape(m, -1), torch.cos(phase).reshape(m, -1)], dim=-1)


def _mlp_forward_indexed(x_enc, prim_ids, W1, b1, W2, b2, W3, b3):
    """Per-record MLP with gathered weights -> (rgb [M,3], sigma_raw [M,1]) (scannet/cumodel.py:193-216)."""
    hcap = min(int(W1.shape[1]), 64)
    w1 = W1.index_select(0, prim_ids)[:, :hcap, :]
    c1 = b1.index_select(0, prim_ids)[:, :hcap]
    w2 = W2.index_select(0, prim_ids)[:, :hcap, :hcap]
    c2 = b2.index_select(0, prim_ids)[:, :hcap]
    w3 = W3.index_select(0, prim_ids)[:, :, :hcap]
    c3 = b3.index_select(0, prim_ids)
    h = F.relu(torch.einsum("mhi,mi->mh", w1, x_enc) + c1)
    h = F.relu(torch.einsum("moh,mh->mo", w2, h) + c2)
    o = torch.einsum("moh,mh->mo", w3, h) + c3
    return torch.sigmoid(o[:, :3]), F.softplus(o[:, 3:4])


_LANES: dict = {}


def _render_lanes(device, count):
    """The streams (default priority) on which ``render_frames`` keeps ``count`` frames in flight on ``device``."""
    key = (device.index if device.index is not None else torch.cuda.current_device(), count)
    lanes = _LANES.get(key)
    if lanes is None:
        lanes = _LANES[key] = [torch.cuda.Stream(device) for _ in range(count)]
    return lanes


def _add_background(rgb, alpha, bg):
    """rgb + clamp(1 - alpha, 0, 1) * bg (scannet/cumodel.py:252-256)."""
    if bg is None:
        return rgb
    if bg.numel() == 1:
        bg = bg.repeat(3)
    return rgb + (1.0 - alpha).clamp(0.0, 1.0) * bg.view(1, 3)


def _uncached(ext):
    """``ext.uncached()`` where the extension object has derived-tensor caches (``tile_ext.TileExt``), else nothing."""
    import contextlib
    manager = getattr(ext, "uncached", None)
    return manager() if callable(manager) else contextlib.nullcontext()


class _TileRenderAutogradFn(torch.autograd.Function):
    """RGB render with gradients for geometry and MLP weights (scannet/cumodel.py:219-378).  The forward is the
    ordinary f32 render; the backward re-traverses the frame (``render_tiles_backward_tilecenter_full``)."""

    @staticmethod
    def forward(ctx, rays_o, rays_d, positions, log_scales, quats, culled_prim_indices, tile_offsets, freq, att,
                W1, b1, W2, b2, W3, b3, Wimg, Himg, TW, TH, threshold, mode, bg_color):
        ext = NeuralPrimitiveSceneTileCUDA._ensure_tile_ext_static()
        args = (rays_o, rays_d, positions, log_scales, quats, culled_prim_indices, tile_offsets, freq, att,
                W1, b1, W2, b2, W3, b3)
        dims = (int(Wimg), int(Himg), int(TW), int(TH), float(threshold))
        # a training step: nothing derived from the parameters may be reused from, or kept for, another call
        records = None
        with _uncached(ext):
            if mode == 0:
                rgb, alpha = ext.render_tiles_forward(*args, *dims)
            elif mode == 1:
                matches = getattr(ext, "records_forward_matches_render", None)
                if (dims[2] == dims[3] and callable(matches) and matches(freq, W1, b1, W2, b2, dims[2])
                        and os.environ.get("MLPSP_AUTOGRAD_KEEP_RECORDS", "1") != "0"):
                    # the records forward in the render kernels' rounding IS this forward (same bits), and its
                    # records serve the backward: one traversal of the frame less per step
                    placeholders = [torch.zeros_like(rays_o), torch.zeros(rays_o.shape[0], device=rays_o.device)]
                    records = ext.render_tiles_training_records(list(args) + placeholders, dims[0], dims[1], dims[2],
                                                                dims[4], 1.5, 2.0, render_order=True)
                    rgb, alpha = records[0], records[1]
                else:
                    rgb, alpha = ext.render_tiles_forward_tilecenter(*args, *dims)
            else:
                raise ValueError("Unsupported tile mode for backward")
        rgb = _add_background(rgb, alpha, bg_color)
        ctx.save_for_backward(*args, *(records[2:] if records is not None else ()))
        ctx.has_records = records is not None
        ctx.dims, ctx.mode, ctx.bg_color = dims, int(mode), bg_color
        return rgb

    @staticmethod
    def backward(ctx, grad_out_rgb):
        args, kept = ctx.saved_tensors[:15], ctx.saved_tensors[15:]
        grad_out_rgb = grad_out_rgb.contiguous()
        if ctx.bg_color is None:
            grad_t_end = torch.zeros(args[0].shape[0], device=grad_out_rgb.device, dtype=grad_out_rgb.dtype)
        else:
            bg = ctx.bg_color.to(device=grad_out_rgb.device, dtype=grad_out_rgb.dtype)
            if bg.numel() == 1:
                bg = bg.repeat(3)
            grad_t_end = (grad_out_rgb * bg.view(1, 3)).sum(dim=-1)
        ext = NeuralPrimitiveSceneTileCUDA._ensure_tile_ext_static()
        if ctx.mode == 0:
            # per-pixel order (scannet/cumodel.py:297-364): the records of every pixel in its own depth order, then
            # the same reverse walk and grouped weight gradients as the tile-centre order
            with _uncached(ext):
                records = ext.render_tiles_per_pixel_records(args, *ctx.dims, 1.5, 2.0)
                gW1, gb1, gW2, gb2, gW3, gb3, gp, gs, gq = ext.backward_from_records(
                    records, args[2], args[3], args[4], args[7], args[8], *args[9:15], grad_out_rgb, grad_t_end)
        elif ctx.has_records:
            gW1, gb1, gW2, gb2, gW3, gb3, gp, gs, gq = ext.backward_from_records(
                [None, None, *kept], args[2], args[3], args[4], args[7], args[8], *args[9:15], grad_out_rgb, grad_t_end)
        else:
            gW1, gb1, gW2, gb2, gW3, gb3, gp, gs, gq = ext.render_tiles_backward_tilecenter_full(
                *args, grad_out_rgb, grad_t_end, *ctx.dims)
        return (None, None, gp, gs, gq, None, None, None, None, gW1, gb1, gW2, gb2, gW3, gb3,
                None, None, None, None, None, None, None)


class _TileRenderWithFeatAutogradFn(torch.autograd.Function):
    """(rgb, feature image) in tile-centre order with gradients (scannet/cumodel.py:381-489): the RGB adjoint reaches
    geometry and MLP weights as in :class:`_TileRenderAutogradFn`, the feature adjoint reaches ``feat_attr`` only.
    An output without an adjoint contributes nothing (``set_materialize_grads(False)``), so its parameters get
    ``None`` and an optimizer leaves them and their moments alone.  The backward runs the records forward once and
    serves both adjoints from it."""

    @staticmethod
    def forward(ctx, rays_o, rays_d, positions, log_scales, quats, culled_prim_indices, tile_offsets, freq, att,
                W1, b1, W2, b2, W3, b3, feat_attr, gating_beta, gating_temp, Wimg, Himg, TW, TH, threshold, bg_color):
        ext = NeuralPrimitiveSceneTileCUDA._ensure_tile_ext_static()
        args = (rays_o, rays_d, positions, log_scales, quats, culled_prim_indices, tile_offsets, freq, att,
                W1, b1, W2, b2, W3, b3)
        dims = (int(Wimg), int(Himg), int(TW), int(TH), float(threshold))
        with _uncached(ext):
            rgb, alpha, feat = ext.render_tiles_forward_tilecenter_with_feat(*args, feat_attr, float(gating_beta),
                                                                             float(gating_temp), *dims)
        rgb = _add_background(rgb, alpha, bg_color)
        ctx.save_for_backward(*args, feat_attr)
        ctx.dims, ctx.bg_color, ctx.gating = dims, bg_color, (float(gating_beta), float(gating_temp))
        ctx.set_materialize_grads(False)
        return rgb, feat

    @staticmethod
    def backward(ctx, grad_out_rgb, grad_out_feat):
        args, feat_attr = ctx.saved_tensors[:15], ctx.saved_tensors[15]
        ext = NeuralPrimitiveSceneTileCUDA._ensure_tile_ext_static()
        W, H, TW, TH, thr = ctx.dims
        grads = [None] * 9
        grad_attr = None
        if grad_out_rgb is None and grad_out_feat is None:
            return (None,) * 24
        if grad_out_feat is not None:
            grad_out_feat = grad_out_feat.contiguous()
        if grad_out_rgb is None:
            with _uncached(ext):
                grad_attr = ext.render_tiles_backward_featattr_tilecenter(*args, feat_attr, grad_out_feat, *ctx.gating,
                                                                          W, H, TW, TH, thr)
        else:
            grad_out_rgb = grad_out_rgb.contiguous()
            if ctx.bg_color is None:
                grad_t_end = torch.zeros(args[0].shape[0], device=grad_out_rgb.device, dtype=grad_out_rgb.dtype)
            else:
                bg = ctx.bg_color.to(device=grad_out_rgb.device, dtype=grad_out_rgb.dtype)
                if bg.numel() == 1:
                    bg = bg.repeat(3)
                grad_t_end = (grad_out_rgb * bg.view(1, 3)).sum(dim=-1)
            with _uncached(ext):
                if grad_out_feat is None:
                    grads = ext.render_tiles_backward_tilecenter_full(*args, grad_out_rgb, grad_t_end, W, H, TW, TH, thr)
                else:
                    x = [*args, grad_out_rgb, grad_t_end]
                    records = ext.render_tiles_training_records(x, W, H, TW, thr, *ctx.gating)
                    *grads, grad_attr = ext.backward_from_records(
                        records, args[2], args[3], args[4], args[7], args[8], *args[9:15], grad_out_rgb, grad_t_end,
                        feat_attr=feat_attr, grad_feat=grad_out_feat)
        gW1, gb1, gW2, gb2, gW3, gb3, gp, gs, gq = grads
        return (None, None, gp, gs, gq, None, None, None, None, gW1, gb1, gW2, gb2, gW3, gb3, grad_attr,
                None, None, None, None, None, None, None, None)


class _TileRenderWithFeatPerPixelAutogradFn(torch.autograd.Function):
    """(rgb, feature image) in per-pixel order under autograd (scannet/cumodel.py:492-600).  The forward is the
    per-pixel render; the backward takes the records of every pixel in its own depth order and serves both adjoints
    from them, as :class:`_TileRenderWithFeatAutogradFn` does in tile-centre order."""

    @staticmethod
    def forward(ctx, rays_o, rays_d, positions, log_scales, quats, culled_prim_indices, tile_offsets, freq, att,
                W1, b1, W2, b2, W3, b3, feat_attr, gating_beta, gating_temp, Wimg, Himg, TW, TH, threshold, bg_color):
        ext = NeuralPrimitiveSceneTileCUDA._ensure_tile_ext_static()
        with _uncached(ext):
            rgb, alpha, feat = ext.render_tiles_forward_per_pixel_with_feat(
                rays_o, rays_d, positions, log_scales, quats, culled_prim_indices, tile_offsets, freq, att,
                W1, b1, W2, b2, W3, b3, feat_attr, float(gating_beta), float(gating_temp), int(Wimg), int(Himg), int(TW),
                int(TH), float(threshold))
        ctx.save_for_backward(rays_o, rays_d, positions, log_scales, quats, culled_prim_indices, tile_offsets, freq, att,
                              W1, b1, W2, b2, W3, b3, feat_attr)
        ctx.dims = (int(Wimg), int(Himg), int(TW), int(TH), float(threshold))
        ctx.bg_color, ctx.gating = bg_color, (float(gating_beta), float(gating_temp))
        ctx.set_materialize_grads(False)
        return _add_background(rgb, alpha, bg_color), feat

    @staticmethod
    def backward(ctx, grad_out_rgb, grad_out_feat):
        args, feat_attr = ctx.saved_tensors[:15], ctx.saved_tensors[15]
        if grad_out_rgb is None and grad_out_feat is None:
            return (None,) * 24
        ext = NeuralPrimitiveSceneTileCUDA._ensure_tile_ext_static()
        grads, grad_attr = [None] * 9, None
        with _uncached(ext):
            records = ext.render_tiles_per_pixel_records(args, *ctx.dims, *ctx.gating)
            if grad_out_rgb is None:
                grad_attr = ext.feature_gradients_from_records(records, feat_attr, grad_out_feat.contiguous())
            else:
                grad_out_rgb = grad_out_rgb.contiguous()
                if ctx.bg_color is None:
                    grad_t_end = torch.zeros(args[0].shape[0], device=grad_out_rgb.device, dtype=grad_out_rgb.dtype)
                else:
                    bg = ctx.bg_color.to(device=grad_out_rgb.device, dtype=grad_out_rgb.dtype)
                    if bg.numel() == 1:
                        bg = bg.repeat(3)
                    grad_t_end = (grad_out_rgb * bg.view(1, 3)).sum(dim=-1)
                out = ext.backward_from_records(
                    records, args[2], args[3], args[4], args[7], args[8], *args[9:15], grad_out_rgb, grad_t_end,
                    feat_attr=feat_attr if grad_out_feat is not None else None,
                    grad_feat=grad_out_feat.contiguous() if grad_out_feat is not None else None)
                grads = out[:9]
                grad_attr = out[9] if len(out) > 9 else None
        gW1, gb1, gW2, gb2, gW3, gb3, gp, gs, gq = grads
        return (None, None, gp, gs, gq, None, None, None, None, gW1, gb1, gW2, gb2, gW3, gb3, grad_attr,
                None, None, None, None, None, None, None, None)


class NeuralPrimitiveSceneTileCUDA(nn.Module):
    """Tile-based single-pass MLP-splatting renderer: full-frame rays in, image out.

    Call ``set_image_size`` first; ``forward`` needs ``B == W*H`` rays.
    """

    requires_full_image = True

    def __init__(self, num_primitives=1024, hidden_dim=32, pe_frequencies=6, initial_positions=None,
                 use_integrated_pe=True, pe_sigma: float = 0.01, min_points: int = 10, tile_size: int = 8,
                 feature_dim_low: int = 0, feature_slots: int = 4, feature_gating_beta: float = 1.5,
                 feature_gating_temp: float = 2.0):
        super().__init__()
        if int(hidden_dim) > 32:
            raise ValueError("NeuralPrimitiveSceneTileCUDA currently supports hidden_dim <= 32 "
                             "(kernel scratch-cap tuning in backward/full path).")
        self.num_primitives = num_primitives
        self.hidden_dim = hidden_dim
        self.pe_frequencies = pe_frequencies
        self.use_integrated_pe = bool(use_integrated_pe)
        self.pe_sigma = float(pe_sigma)
        if self.pe_sigma <= 0.0:
            raise ValueError("pe_sigma must be > 0.")
        self.image_size = None
        self.tile_size = int(tile_size)
        if self.tile_size <= 0:
            raise ValueError("tile_size must be a positive integer.")
        if self.tile_size not in (8, 16):
            raise ValueError("NeuralPrimitiveSceneTileCUDA supports tile_size in {8, 16}.")
        self.tile_order_mode_override = None
        # MLP arithmetic of the RGB tile-centre render: "f32" (scalar, the reference's default kernel) or
        # "bf16"/"fp16" (matrix cores; needs the 72->32->32->4 MLP and 8x8 tiles, else f32 is used).
        self.render_precision = os.environ.get("MLPSP_RENDER_PRECISION", "f32")
        self.feature_dim_low = int(max(0, feature_dim_low))
        self.feature_slots = int(max(1, feature_slots))
        self.feature_gating_beta = float(feature_gating_beta)
        self.feature_gating_temp = float(feature_gating_temp)
        if self.feature_dim_low > 0 and self.feature_slots not in (4, 5):
            raise ValueError("feature_slots must be 4 (canonical) or 5 (legacy) when features are enabled.")
        if self.feature_gating_beta <= 0.0:
            raise ValueError("feature_gating_beta must be > 0.")
        if self.feature_gating_temp <= 0.0:
            raise ValueError("feature_gating_temp must be > 0.")

        if initial_positions is not None:
            raise NotImplementedError("octree initialisation from a point cloud belongs to the training side; "
                                      "construct with num_primitives and load a state dict instead")
        n = int(num_primitives)
        self.positions = nn.Parameter(torch.rand(n, 3) * 2.0 - 1.0)
        self.log_scales = nn.Parameter(torch.log(torch.ones(n) * 0.1).unsqueeze(-1).repeat(1, 3))
        self.quats = nn.Parameter(torch.tensor([1.0, 0.0, 0.0, 0.0]).view(1, 4).repeat(n, 1))
        if self.use_integrated_pe:
            self.encoder = IntegratedPositionalEncoding(in_dim=6, num_frequencies=pe_frequencies, sigma=self.pe_sigma)
        else:
            self.encoder = FourierFeatureEncoding(in_dim=6, num_frequencies=pe_frequencies)
        enc, h = self.encoder.out_dim, hidden_dim
        self.W1 = nn.Parameter(torch.randn(n, h, enc) * 0.01)
        self.b1 = nn.Parameter(torch.zeros(n, h))
        self.W2 = nn.Parameter(torch.randn(n, h, h) * 0.01)
        self.b2 = nn.Parameter(torch.zeros(n, h))
        self.W3 = nn.Parameter(torch.randn(n, 4, h) * 0.01)
        self.b3 = nn.Parameter(torch.zeros(n, 4))
        if self.feature_dim_low > 0:
            if self.feature_slots == 5:
                feat = torch.zeros(n, 5, self.feature_dim_low)
                feat[:, 0, :].normal_(mean=0.0, std=0.01)
            else:
                feat = torch.randn(n, self.feature_slots, self.feature_dim_low) * 0.01
            self.feat_attr = nn.Parameter(feat)
        else:
            self.feat_attr = None
        self.register_buffer("stat_sum_w", torch.zeros(n, dtype=torch.float32))
        self.register_buffer("stat_max_w", torch.zeros(n, dtype=torch.float32))
        self.register_buffer("stat_hits", torch.zeros(n, dtype=torch.int32))
        self.register_buffer("stat_contrib_count", torch.zeros(n, dtype=torch.int32))
        self.register_buffer("stat_sum_werr", torch.zeros(n, dtype=torch.float32))
        self.register_buffer("alpha_accum", torch.zeros(n, dtype=torch.float32))

    # ------------------------------------------------------------------------------------------
    @torch.no_grad()
    def reset_w_stats(self):
        n, dev = self.positions.shape[0], self.positions.device
        self.stat_sum_w = torch.zeros(n, device=dev, dtype=torch.float32)
        self.stat_hits = torch.zeros(n, device=dev, dtype=torch.int32)
        self.stat_max_w = torch.zeros(n, device=dev, dtype=torch.float32)
        self.stat_sum_werr = torch.zeros(n, device=dev, dtype=torch.float32)
        self.stat_contrib_count = torch.zeros(n, device=dev, dtype=torch.int32)

    def set_image_size(self, W: int, H: int):
        self.image_size = (int(W), int(H))

    def _activate_cuda_device(self) -> torch.device:
        positions = self._parameters.get("positions")
        device = (positions if positions is not None else self.positions).device
        if device.type != "cuda":
            raise RuntimeError("NeuralPrimitiveSceneTileCUDA must be moved to a CUDA device before rendering.")
        if device.index is None:
            device = torch.device("cuda", torch.cuda.current_device())
        elif torch.cuda.current_device() != device.index:
            torch.cuda.set_device(device.index)
        return device

    def _resolve_tile_order_mode(self) -> str:
        mode = self.tile_order_mode_override
        if mode is None or str(mode).strip() == "":
            mode = _env("MLPSP_TILE_ORDER", "tilecenter")
        if mode == "tilecenter":
            return mode
        mode = str(mode).strip().lower()
        mode = {"tile_center": "tilecenter", "tile-center": "tilecenter"}.get(mode, mode)
        if mode not in {"tilecenter", "per_pixel"}:
            raise ValueError(f"Unsupported tile order {mode!r}; use 'tilecenter' or 'per_pixel'.")
        return mode

    def _ensure_tile_ext(self):
        return self._ensure_tile_ext_static()

    @staticmethod
    def _ensure_tile_ext_static(tile_size=None):
        """The extension object for the build the environment selects; cached in the module globals
        ``_tile_ext`` / ``_tile_ext_key`` exactly where the reference caches its JIT module."""
        global _tile_ext, _tile_ext_key
        key, _name, _flags = _tile_ext_build_config()
        if _tile_ext is None or _tile_ext_key != key:
            from .tile_ext import TileExt
            _tile_ext = TileExt(max_tile_prims=_tile_capacity_from_env(), max_hits=_max_hits_from_env())
            _tile_ext_key = key
        return _tile_ext

    # ------------------------------------------------------------------------------------------
    def _cached(self, name, sources, extra, build):
        """``build()`` once per state of the ``sources`` tensors (identity, shape, in-place version): the
        scene is constant while rendering, and every small torch op skipped is a kernel launch less per
        frame.  The value is built outside inference mode so that it carries a version counter itself."""
        try:
            key = tuple((t.data_ptr(), t._version, t.shape, t.device) for t in sources) + tuple(extra)
        except RuntimeError:                      # inference tensors have no version counter: do not cache
            return build()
        cache = self.__dict__.setdefault("_mlpsp_cache", {})
        hit = cache.get(name)
        if hit is None or hit[0] != key:
            with torch.inference_mode(False), torch.no_grad():
                hit = (key, build())
            cache[name] = hit
        return hit[1]

    def _frequency_tables(self, device):
        """freq and att as the kernels take them (scannet/cumodel.py:1078-1086)."""
        # (once per frame, while the device may be waiting for the host: the encoder and its buffers are taken from
        # the modules' own tables, which a plain attribute read reaches only after a failed instance look-up)
        encoder = self._modules.get("encoder")
        if encoder is None:
            encoder = self.encoder
        buffers = encoder._buffers
        bands = buffers.get("freq_bands")
        sources = [bands if bands is not None else encoder.freq_bands]
        weights = buffers.get("runtime_frequency_weights")
        if weights is None and hasattr(encoder, "runtime_frequency_weights"):
            weights = encoder.runtime_frequency_weights
        if weights is not None:
            sources.append(weights)
        sigma2 = encoder.__dict__.get("sigma2")
        if sigma2 is None:
            sigma2 = getattr(encoder, "sigma2", 0.0) if hasattr(type(encoder), "sigma2") else 0.0
        extra = (device, float(sigma2))
        return self._cached("frequency_tables", sources, extra, lambda: self._build_frequency_tables(device))

    def _build_frequency_tables(self, device):
        freq = self.encoder.freq_bands.to(device=device, dtype=torch.float32)
        if isinstance(self.encoder, IntegratedPositionalEncoding):
            att = torch.exp(-0.5 * (freq * freq) * float(self.encoder.sigma2))
        else:
            att = torch.ones_like(freq)
        if hasattr(self.encoder, "runtime_frequency_weights"):
            att = att * self.encoder.runtime_frequency_weights.to(device=device, dtype=torch.float32)
        return freq.contiguous(), att.contiguous()

    def _legacy_culling(self, view_matrices, proj_matrix, score_threshold, tile_size, tile_view_ids=None):
        """Screen-space tile lists: same rule as scannet/cumodel.py:994-1070, evaluated sparsely on the GPU."""
        W, H = self.image_size
        cand, offsets, longest = ops.bin_legacy(self.positions.detach(), self.log_scales.detach(),
                                                _host_matrix(view_matrices), _host_matrix(proj_matrix), W, H,
                                                int(tile_size), float(score_threshold),
                                                tile_view_ids, with_longest=True)
        # lists fresh from the binning kernels need no second validation pass on the device
        note = getattr(self._ensure_tile_ext(), "note_binned_lists", None)
        if note is not None:
            note(cand, offsets, longest, self.positions.shape[0])
        return cand, offsets

    @torch.no_grad()
    def build_tilecenter_culling_from_tile_views(self, tile_view_ids, view_matrices, proj_matrix,
                                                 score_threshold: float = 1e-3, tile_size: int | None = None):
        """Tile lists when every tile takes its rays from one of K views (scannet/cumodel.py:838-949)."""
        if getattr(self, "camera_mode", "legacy-centered") == "colmap-native":
            return None, None
        if self.image_size is None:
            raise ValueError("image_size must be set before building tile culling.")
        W, H = self.image_size
        device = self._activate_cuda_device()
        tile_size = int(self.tile_size if tile_size is None else tile_size)
        if tile_size <= 0:
            raise ValueError("tile_size must be a positive integer.")
        num_tiles = ops.num_tiles(W, H, tile_size, tile_size)
        given = tile_view_ids
        tile_view_ids = tile_view_ids.to(device=device, dtype=torch.long).reshape(-1)
        if tile_view_ids.numel() != num_tiles:
            raise ValueError(f"tile_view_ids length mismatch: got {tile_view_ids.numel()}, expected {num_tiles}")
        if view_matrices.ndim != 3 or view_matrices.shape[1:] != (4, 4):
            raise ValueError("view_matrices must have shape (K,4,4)")
        if int(view_matrices.shape[0]) <= 0:
            raise ValueError("view_matrices must contain at least one view")
        # one read-back for both bounds, and -- with the int32 copy the binning takes -- only once per state of the
        # caller's tensor (a mosaic's layout is the same frame after frame; the check is a reduction and a
        # synchronisation)
        lo, hi, ids32 = self._tile_view_check(given, tile_view_ids)
        if lo < 0 or hi >= int(view_matrices.shape[0]):
            raise ValueError("tile_view_ids contains out-of-range view indices")
        return self._legacy_culling(view_matrices, proj_matrix, score_threshold, tile_size, ids32)

    def _tile_view_check(self, given, ids):
        """(smallest id, largest id, int32 copy) of a caller's tile_view_ids, remembered for the last few tensors seen
        (a renderer cycles through a handful of mosaic layouts).  An entry keeps the caller's tensor itself: while it
        lives its memory cannot be handed to another tensor, whose address, shape and version would match."""
        try:
            key = (given.data_ptr(), given._version, tuple(given.shape), given.dtype, str(given.device))
        except RuntimeError:                      # inference tensors have no version counter: do not remember
            key = None
        memo = self.__dict__.setdefault("_mlpsp_tile_views", {})
        hit = memo.get(key) if key is not None else None
        if hit is None:
            with torch.inference_mode(False), torch.no_grad():
                lo, hi = torch.stack(torch.aminmax(ids)).tolist()
                hit = (lo, hi, ids.to(torch.int32).contiguous(), given)
            if key is not None:
                if len(memo) >= 16:
                    memo.pop(next(iter(memo)))
                memo[key] = hit
        return hit[:3]

    def _tile_lists(self, ray_o, ray_d, score_threshold, view_matrix, proj_matrix, culled_prim_indices, tile_offsets,
                    device, allow_native=True):
        W, H = self.image_size
        tile_size = int(self.tile_size)
        num_tiles = ops.num_tiles(W, H, tile_size, tile_size)
        external = (culled_prim_indices is not None) or (tile_offsets is not None)
        if allow_native and getattr(self, "camera_mode", "legacy-centered") == "colmap-native":
            if external:
                raise ValueError("Native camera culling must be derived from the actual rays")
            culled_prim_indices, tile_offsets = ray_cone_candidates(
                ray_o, ray_d, self.positions, self.log_scales, W, H, tile_size, score_threshold)
            external = True
        if external:
            if culled_prim_indices is None or tile_offsets is None:
                raise ValueError("Both culled_prim_indices and tile_offsets must be provided together.")
            culled_prim_indices = culled_prim_indices.to(device=device, dtype=torch.int32)
            tile_offsets = tile_offsets.to(device=device, dtype=torch.int32)
            if tile_offsets.numel() != num_tiles + 1:
                raise ValueError(f"tile_offsets length mismatch: got {tile_offsets.numel()}, expected {num_tiles + 1}")
            return culled_prim_indices, tile_offsets
        if view_matrix is None or proj_matrix is None:
            raise ValueError("Tile renderer requires view_matrix/proj_matrix unless external culling is provided.")
        return self._legacy_culling(_host_matrix(view_matrix).reshape(1, 4, 4), _host_matrix(proj_matrix),
                                    score_threshold, tile_size)

    def _unit_quats(self):
        quats = self._parameters.get("quats")
        if quats is None:
            quats = self.quats
        return self._cached("unit_quats", [quats], (), lambda: F.normalize(quats.detach(), dim=-1).contiguous())

    def _base_args(self, ray_o, ray_d, culled_prim_indices, tile_offsets, device, unit_dirs=None):
        freq, att = self._frequency_tables(device)
        if unit_dirs is None:
            unit_dirs = _unit_directions(ray_d)
        return (ray_o.contiguous(), unit_dirs, self.positions.detach().contiguous(),
                self.log_scales.detach().contiguous(), self._unit_quats(),
                culled_prim_indices, tile_offsets.to(torch.int32), freq, att,
                self.W1.detach().contiguous(), self.b1.detach().contiguous(), self.W2.detach().contiguous(),
                self.b2.detach().contiguous(), self.W3.detach().contiguous(), self.b3.detach().contiguous())

    @staticmethod
    def _background(bg_color, ray_o):
        if bg_color is None:
            return None
        if not torch.is_tensor(bg_color):
            return torch.tensor(bg_color, dtype=ray_o.dtype, device=ray_o.device)
        return bg_color.to(ray_o.device, dtype=ray_o.dtype)

    # ------------------------------------------------------------------------------------------
    def forward(self, ray_o, ray_d, score_threshold=1e-3, bg_color=None, view_matrix=None, proj_matrix=None,
                culled_prim_indices=None, tile_offsets=None, return_feature: bool = False, feature_target=None):
        """rgb [B,3], or (rgb, feat [B,C]) with ``return_feature`` (scannet/cumodel.py:951-1160)."""
        if self.image_size is None:
            raise ValueError("image_size must be set on NeuralPrimitiveSceneTileCUDA before calling forward.")
        W, H = self.image_size
        assert ray_o.shape[0] == W * H, "Tile renderer requires full-frame rays (B == W*H)"
        device = self._activate_cuda_device()
        ts = int(self.tile_size)
        if feature_target is not None:
            return self._forward_csr_training(ray_o, ray_d, score_threshold, bg_color, view_matrix, proj_matrix,
                                              culled_prim_indices, tile_offsets, return_feature, feature_target, device)
        if torch.is_grad_enabled():
            trainable = (self.positions, self.log_scales, self.quats, self.W1, self.b1, self.W2, self.b2, self.W3,
                         self.b3)
            if return_feature and self.feat_attr is not None:
                if any(t.requires_grad for t in (*trainable, self.feat_attr)):
                    return self._forward_differentiable_with_feat(ray_o, ray_d, score_threshold, bg_color, view_matrix,
                                                                  proj_matrix, culled_prim_indices, tile_offsets, device)
            elif any(t.requires_grad for t in trainable):
                return self._forward_differentiable(ray_o, ray_d, score_threshold, bg_color, view_matrix, proj_matrix,
                                                    culled_prim_indices, tile_offsets, return_feature, device)
        with torch.no_grad():
            use_tilecenter = self._resolve_tile_order_mode() == "tilecenter"
            ext = self._ensure_tile_ext()
            # (plain attributes live in the module's __dict__; getattr with a default on a module that lacks the name
            # walks parameters, buffers and submodules first)
            plain = self.__dict__
            own_lists = (culled_prim_indices is None and tile_offsets is None and view_matrix is not None
                         and proj_matrix is not None
                         and plain.get("camera_mode", "legacy-centered") != "colmap-native")
            with_feat = return_feature and self.feat_attr is not None
            if (own_lists and use_tilecenter and ts == 8 and (with_feat or not return_feature)
                    and feature_target is None and plain.get("queued_frames", True)
                    and hasattr(ext, "render_frame_queued")):
                done = self._forward_queued(ext, ray_o, ray_d, score_threshold, view_matrix, proj_matrix, bg_color,
                                            device, with_feat)
                if done is not None:
                    return done
            # queued before the binning, whose pair count is a blocking read-back: the device then has
            # this work to do while the host waits, instead of idling while the host issues it afterwards
            unit_dirs = _unit_directions(ray_d)
            culled_prim_indices, tile_offsets = self._tile_lists(
                ray_o, ray_d, score_threshold, view_matrix, proj_matrix, culled_prim_indices, tile_offsets, device)
            if own_lists and hasattr(ext, "note_frame_pairs"):
                ext.note_frame_pairs(int(culled_prim_indices.numel()))
            base = self._base_args(ray_o, ray_d, culled_prim_indices, tile_offsets, device, unit_dirs)
            bg = self._background(bg_color, ray_o)
            dims = (int(W), int(H), ts, ts, float(score_threshold))
            precision = str(getattr(self, "render_precision", "f32")).lower()
            if precision not in {"f32", "bf16", "fp16"}:
                raise ValueError(f"Unsupported render_precision {precision!r}; use 'f32', 'bf16' or 'fp16'.")
            matrix_cores = (use_tilecenter and precision != "f32" and ts == 8 and int(self.hidden_dim) == 32
                            and int(self.pe_frequencies) == 6)
            if (not return_feature) or (self.feat_attr is None):
                if matrix_cores:
                    rgb, alpha = ext.render_tiles_rgb_wmma(list(base), int(W), int(H), float(score_threshold),
                                                           precision == "bf16")
                elif use_tilecenter:
                    rgb, alpha = ext.render_tiles_forward_tilecenter(*base, *dims)
                else:
                    rgb, alpha = ext.render_tiles_forward(*base, *dims)
                rgb = _add_background(rgb, alpha, bg)
                if return_feature and self.feat_attr is None:
                    raise RuntimeError("return_feature=True requested but feat_attr is not initialized.")
                return rgb
            feat_attr = self.feat_attr.detach()
            if not matrix_cores and feat_attr.dtype != torch.float32:
                feat_attr = feat_attr.float()          # fp16-stored attributes: only the matrix-core path reads them as they are
            feat_args = (feat_attr.contiguous(), float(self.feature_gating_beta), float(self.feature_gating_temp))
            if matrix_cores:
                rgb, alpha, feat = ext.render_tiles_rgb_wmma_with_feat(list(base), *feat_args, int(W), int(H),
                                                                       float(score_threshold), precision == "bf16")
            elif use_tilecenter:
                rgb, alpha, feat = ext.render_tiles_forward_tilecenter_with_feat(*base, *feat_args, *dims)
            else:
                rgb, alpha, feat = ext.render_tiles_forward_per_pixel_with_feat(*base, *feat_args, *dims)
            return _add_background(rgb, alpha, bg), feat

    def invalidate_render_caches(self):
        """Drop everything derived from the parameters (unit quaternions, geometry records, matrix-core operand
        copies).  Called by every grad-mode forward: the caches are keyed on the parameters' identity and in-place
        version, which a fused optimizer step (``Adam(fused=True)``) does not advance.  Call it yourself after
        changing parameters in any other way that leaves ``tensor._version`` unchanged."""
        self.__dict__.pop("_mlpsp_cache", None)
        self.__dict__.pop("_mlpsp_tile_views", None)
        ext = _tile_ext
        if ext is not None and callable(getattr(ext, "invalidate_caches", None)):
            ext.invalidate_caches()

    def _forward_csr_training(self, ray_o, ray_d, score_threshold, bg_color, view_matrix, proj_matrix,
                              culled_prim_indices, tile_offsets, return_feature, feature_target, device):
        """(rgb, streamed feature L1 loss) through the record-based training function
        (scannet/cumodel.py:1098-1108)."""
        self.invalidate_render_caches()
        W, H = self.image_size
        ts = int(self.tile_size)
        use_tilecenter = self._resolve_tile_order_mode() == "tilecenter"
        if not return_feature or self.feat_attr is None or not use_tilecenter or ts != 8:
            raise ValueError("CSR feature training requires tilecenter8 and direct feature attributes")
        from .record_training import Frame, feature_training_step
        with torch.no_grad():
            unit_dirs = _unit_directions(ray_d)
            culled_prim_indices, tile_offsets = self._tile_lists(
                ray_o, ray_d, score_threshold, view_matrix, proj_matrix, culled_prim_indices, tile_offsets, device)
            freq, att = self._frequency_tables(device)
        base = [ray_o.contiguous(), unit_dirs, self.positions.contiguous(), self.log_scales.contiguous(),
                F.normalize(self.quats, dim=-1).contiguous(), culled_prim_indices, tile_offsets.to(torch.int32), freq, att,
                self.W1.contiguous(), self.b1.contiguous(), self.W2.contiguous(), self.b2.contiguous(),
                self.W3.contiguous(), self.b3.contiguous()]
        frame = Frame(int(W), int(H), float(score_threshold), float(self.feature_gating_beta),
                      float(self.feature_gating_temp))
        return feature_training_step(base, self.feat_attr.contiguous(), feature_target, frame,
                                     self._background(bg_color, ray_o))

    def _forward_differentiable(self, ray_o, ray_d, score_threshold, bg_color, view_matrix, proj_matrix,
                                culled_prim_indices, tile_offsets, return_feature, device):
        """RGB with autograd (scannet/cumodel.py:1110-1131): tile lists and encodings are constants, positions,
        log-scales, normalised quaternions and MLP weights carry gradients."""
        self.invalidate_render_caches()
        W, H = self.image_size
        ts = int(self.tile_size)
        with torch.no_grad():
            unit_dirs = _unit_directions(ray_d)
            culled_prim_indices, tile_offsets = self._tile_lists(
                ray_o, ray_d, score_threshold, view_matrix, proj_matrix, culled_prim_indices, tile_offsets, device)
            freq, att = self._frequency_tables(device)
        mode = 1 if self._resolve_tile_order_mode() == "tilecenter" else 0
        rgb = _TileRenderAutogradFn.apply(
            ray_o.contiguous(), unit_dirs, self.positions.contiguous(), self.log_scales.contiguous(),
            F.normalize(self.quats, dim=-1).contiguous(), culled_prim_indices, tile_offsets.to(torch.int32), freq, att,
            self.W1.contiguous(), self.b1.contiguous(), self.W2.contiguous(), self.b2.contiguous(),
            self.W3.contiguous(), self.b3.contiguous(), int(W), int(H), ts, ts, float(score_threshold), mode,
            self._background(bg_color, ray_o))
        if return_feature and self.feat_attr is None:
            raise RuntimeError("return_feature=True requested but feat_attr is not initialized.")
        return rgb

    def _forward_differentiable_with_feat(self, ray_o, ray_d, score_threshold, bg_color, view_matrix, proj_matrix,
                                          culled_prim_indices, tile_offsets, device):
        """(rgb, feature image) with autograd (scannet/cumodel.py:1128-1160), in either order."""
        fn = (_TileRenderWithFeatAutogradFn if self._resolve_tile_order_mode() == "tilecenter"
              else _TileRenderWithFeatPerPixelAutogradFn)
        self.invalidate_render_caches()
        W, H = self.image_size
        ts = int(self.tile_size)
        with torch.no_grad():
            unit_dirs = _unit_directions(ray_d)
            culled_prim_indices, tile_offsets = self._tile_lists(
                ray_o, ray_d, score_threshold, view_matrix, proj_matrix, culled_prim_indices, tile_offsets, device)
            freq, att = self._frequency_tables(device)
        return fn.apply(
            ray_o.contiguous(), unit_dirs, self.positions.contiguous(), self.log_scales.contiguous(),
            F.normalize(self.quats, dim=-1).contiguous(), culled_prim_indices, tile_offsets.to(torch.int32), freq, att,
            self.W1.contiguous(), self.b1.contiguous(), self.W2.contiguous(), self.b2.contiguous(),
            self.W3.contiguous(), self.b3.contiguous(), self.feat_attr.contiguous(), float(self.feature_gating_beta),
            float(self.feature_gating_temp), int(W), int(H), ts, ts, float(score_threshold),
            self._background(bg_color, ray_o))

    def _forward_queued(self, ext, ray_o, ray_d, score_threshold, view_matrix, proj_matrix, bg_color, device,
                        with_feat=False, defer=False):
        """The RGB frame with binning, sort and render queued back to back and one read-back at the end
        (``TileExt.render_frame_queued``); None when that path does not apply or has to be repeated the
        synchronous way.  Same images and errors as the step-by-step path.  The binning goes first: it needs only
        the primitives and the camera, and the device is busy with it while the host prepares the rest of the
        frame (unit ray directions, tables, weights).  ``defer``: return a callable that finishes the frame (waits for
        its read-back, returns the images or None) instead of finishing it here."""
        precision = str(getattr(self, "render_precision", "f32")).lower()
        if precision not in {"f32", "bf16", "fp16"}:
            raise ValueError(f"Unsupported render_precision {precision!r}; use 'f32', 'bf16' or 'fp16'.")
        if precision != "f32" and not (int(self.hidden_dim) == 32 and int(self.pe_frequencies) == 6):
            precision = "f32"
        if with_feat and precision == "f32":
            return None                       # the exact feature frame goes step by step
        # (up to the binning call below the device waits for the host: parameters are taken from the module's own
        # table, which a plain attribute read reaches only after a failed instance look-up)
        registered = self._parameters
        try:
            params = (registered["W1"], registered["b1"], registered["W2"], registered["b2"], registered["W3"],
                      registered["b3"])
            positions, log_scales = registered["positions"], registered["log_scales"]
        except KeyError:
            params = (self.W1, self.b1, self.W2, self.b2, self.W3, self.b3)
            positions, log_scales = self.positions, self.log_scales
        f32 = torch.float32
        if params[0].dtype != f32 and not (precision != "f32" and params[0].dtype == torch.float16):
            return None                       # stored half-precision weights: only the matrix-core frame reads them as they are
        W, H = self.image_size
        # (the kernels take addresses: no detached aliases are made on the way to the first launch)
        if not positions.is_contiguous():
            positions = positions.contiguous()
        if not log_scales.is_contiguous():
            log_scales = log_scales.contiguous()
        views, proj = _frame_matrix(view_matrix).reshape(1, 4, 4), _frame_matrix(proj_matrix)
        binned = None
        if hasattr(ext, "frame_binning_queued"):
            # (a frame on the matrix cores takes its lists in per-tile segments: one binning launch less)
            segments = precision != "f32" and _env("MLPSP_FRAME_SEGMENTS", "1") != "0"
            binned = ext.frame_binning_queued(positions, log_scales, views, proj, int(W), int(H), float(score_threshold),
                                              **({"segments": True} if segments else {}))
            if binned is None:
                return None
        # (the other weight tensors are looked at now that the device has the binning to work on; a mixed set goes the
        # step-by-step way, whose own binning then repeats what was queued here)
        if not (params[1].dtype == f32 and params[2].dtype == f32 and params[3].dtype == f32 and params[4].dtype == f32
                and params[5].dtype == f32 and params[0].dtype == f32):
            half = all(w.dtype == torch.float16 for w in params)
            if not (half and precision != "f32"):
                return None
        ws = [p.detach().contiguous() for p in params]
        more = {"binned": binned} if binned is not None else {}
        ray_o = ray_o.contiguous()
        if (hasattr(ext, "frame_prologue") and ray_d.is_cuda and ray_d.dtype == torch.float32 and ray_d.dim() == 2
                and ray_d.shape[1] == 3 and not ray_d.requires_grad and ray_o.dtype == torch.float32
                and ray_o.shape == ray_d.shape and ray_o.is_cuda):
            # unit directions and the tiles' ray pyramids for the sort's culling in one launch; with
            # MLPSP_SORT_FRAME_RECORDS=1 also the sort's per-frame records (opt-in: measured 6 us per frame slower than
            # the full key evaluation on one MI355X)
            geometry = None
            if _env("MLPSP_SORT_FRAME_RECORDS", "0") == "1":
                geometry = (positions, log_scales, self._unit_quats())
            unit_dirs, more["tile_pyramids"], records = ext.frame_prologue(ray_o, ray_d, int(W), int(H), geometry)
            if records is not None:
                more["frame_records"] = records
        else:
            unit_dirs = _unit_directions(ray_d)
        freq, att = self._frequency_tables(device)
        if with_feat:
            more["feat"] = (self.feat_attr.detach().contiguous(), float(self.feature_gating_beta),
                            float(self.feature_gating_temp))
        if defer:
            more["defer"] = True
        out = ext.render_frame_queued(ray_o, unit_dirs, positions, log_scales, self._unit_quats(), freq, att,
                                      ws, views, proj, int(W), int(H), float(score_threshold), precision, **more)

        def finish(out=out):
            if out is not None and not isinstance(out, tuple):
                out = ext.finish_frame_queued(out)
            if out is None:
                return None
            rgb = _add_background(out[0], out[1], self._background(bg_color, ray_o))
            return (rgb, out[2]) if with_feat else rgb
        return finish if defer else finish()

    def render_frames(self, frames, score_threshold=1e-3, bg_color=None, return_feature: bool = False,
                      frames_in_flight: int = 2):
        """``[self(ray_o, ray_d, score_threshold, bg_color, view_matrix, proj_matrix, return_feature=...) for (ray_o,
        ray_d, view_matrix, proj_matrix) in frames]`` without gradients, with up to ``frames_in_flight`` frames queued
        on the device at once (no counterpart in the reference, whose callers render camera after camera,
        tools/benchmark_inference.py:264-313).  One frame alone leaves the device idle twice: at its end, where the
        last tiles of the render run on a chip that has nothing else to do, and between frames, while the host reads
        the frame's 96 status bytes and issues the next launches.  Here frame k+1 is queued on a second stream before
        the host waits for frame k, so its binning and sort run beside the end of frame k's render.  Same images as
        ``forward`` (each frame runs the same launches in the same order on its stream); the inputs must be ready
        on the current stream when the call is made, and the results are ready on it when the call returns."""
        frames = list(frames)
        W, H = self.image_size if self.image_size is not None else (0, 0)
        plain = self.__dict__
        with_feat = return_feature and self.feat_attr is not None

        def one(f):
            with torch.no_grad():
                return self.forward(f[0], f[1], score_threshold, bg_color, f[2], f[3], return_feature=return_feature)
        eligible = (frames_in_flight > 1 and len(frames) > 1 and self.image_size is not None
                    and self._resolve_tile_order_mode() == "tilecenter" and int(self.tile_size) == 8
                    and (with_feat or not return_feature) and plain.get("queued_frames", True)
                    and plain.get("camera_mode", "legacy-centered") != "colmap-native"
                    and str(getattr(self, "render_precision", "f32")).lower() in {"bf16", "fp16"}
                    and all(f[2] is not None and f[3] is not None and f[0].shape[0] == W * H for f in frames))
        if not eligible:
            return [one(f) for f in frames]
        device = self._activate_cuda_device()
        ext = self._ensure_tile_ext()
        if not (hasattr(ext, "render_frame_queued") and hasattr(ext, "finish_frame_queued")):
            return [one(f) for f in frames]
        main = torch.cuda.current_stream(device)
        lanes = _render_lanes(device, min(int(frames_in_flight), 4))
        ready = torch.cuda.Event()
        ready.record(main)
        for lane in lanes:
            lane.wait_event(ready)
        results, waiting = [], []          # waiting: (lane, frame, finish) in queue order

        def finish_oldest():
            lane, f, finish = waiting.pop(0)
            with torch.cuda.stream(lane):
                out = finish() if finish is not None else None
                if out is None:
                    out = one(f)           # rare: the synchronous way, on the frame's own stream
            results.append(out)
        try:
            with torch.no_grad():
                for i, f in enumerate(frames):
                    lane = lanes[i % len(lanes)]
                    with torch.cuda.stream(lane):
                        finish = self._forward_queued(ext, f[0], f[1], score_threshold, f[2], f[3], bg_color, device,
                                                      with_feat, defer=True)
                    waiting.append((lane, f, finish))
                    if i == 0:
                        # Whatever is derived from the parameters (geometry records, operand copies of the weights,
                        # tables) is built by the first frame, on its lane: the other lanes start after it.
                        if finish is None:
                            finish_oldest()
                        built = torch.cuda.Event()
                        built.record(lane)
                        for other in lanes[1:]:
                            other.wait_event(built)
                    if len(waiting) >= len(lanes):
                        finish_oldest()
                while waiting:
                    finish_oldest()
        finally:
            for lane in lanes:
                main.wait_stream(lane)
        for out in results:
            for t in (out if isinstance(out, tuple) else (out,)):
                t.record_stream(main)
        return results

    def render_feature_map(self, ray_o, ray_d, score_threshold: float = 1e-3, view_matrix=None, proj_matrix=None,
                           culled_prim_indices=None, tile_offsets=None):
        """The feature image alone, through ``forward`` (scannet/cumodel.py:1162-1193)."""
        if self.feat_attr is None:
            raise RuntimeError("Feature rendering requested but feature_dim_low == 0.")
        if self.image_size is None:
            raise ValueError("image_size must be set before calling render_feature_map.")
        W, H = self.image_size
        if ray_o.shape[0] != W * H:
            raise ValueError("render_feature_map requires full-frame rays (B == W*H).")
        _rgb, feat = self.forward(ray_o=ray_o, ray_d=ray_d, score_threshold=score_threshold, bg_color=None,
                                  view_matrix=view_matrix, proj_matrix=proj_matrix,
                                  culled_prim_indices=culled_prim_indices, tile_offsets=tile_offsets,
                                  return_feature=True)
        return feat

    @torch.no_grad()
    def render_rgb_alpha_no_grad(self, ray_o, ray_d, score_threshold: float = 1e-3, bg_color=None, view_matrix=None,
                                 proj_matrix=None, collect_w_stats: bool = False, gt_rgb=None):
        """(rgb, alpha) under the tile-centre pipeline (scannet/cumodel.py:1196-1383)."""
        if getattr(self, "camera_mode", "legacy-centered") == "colmap-native":
            raise NotImplementedError("Native camera statistics rendering is not implemented; use forward for RGB/features")
        if self.image_size is None:
            raise ValueError("image_size must be set on NeuralPrimitiveSceneTileCUDA before calling render_rgb_alpha_no_grad.")
        if view_matrix is None or proj_matrix is None:
            raise ValueError("Tile renderer requires view_matrix and proj_matrix for culling.")
        W, H = self.image_size
        B = ray_o.shape[0]
        assert B == W * H, "Tile renderer requires full-frame rays (B == W*H)"
        device = self._activate_cuda_device()
        ts = int(self.tile_size)
        cand, offsets = self._legacy_culling(_host_matrix(view_matrix).reshape(1, 4, 4), _host_matrix(proj_matrix),
                                             score_threshold, ts)
        ext = self._ensure_tile_ext()
        base = self._base_args(ray_o, ray_d, cand, offsets, device)
        dims = (int(W), int(H), ts, ts, float(score_threshold))
        if collect_w_stats:
            if gt_rgb is None:
                raise ValueError("collect_w_stats=True requires gt_rgb (shape=(B,3), B=W*H) to compute pixel_error "
                                 "inside the CUDA kernel.")
            if gt_rgb.dim() != 2 or gt_rgb.shape[0] != B or gt_rgb.shape[1] != 3:
                raise ValueError(f"gt_rgb must have shape (B,3) with B=W*H={B}, got {tuple(gt_rgb.shape)}")
            gt_rgb = gt_rgb.to(device=device, dtype=torch.float32).contiguous()
            rgb, alpha = ext.render_tiles_forward_tilecenter_stats(
                *base[:9], int(base[7].numel()), *base[9:], int(self.W1.shape[0]), int(self.W1.shape[1]),
                int(self.W1.shape[2]), *dims, gt_rgb, self.stat_sum_w.contiguous(), self.stat_max_w.contiguous(),
                self.stat_hits.contiguous(), self.stat_sum_werr.contiguous(), self.stat_contrib_count.contiguous())
        else:
            rgb, alpha = ext.render_tiles_forward_tilecenter(*base, *dims)
        return _add_background(rgb, alpha, self._background(bg_color, ray_o)), alpha

    @torch.no_grad()
    def render_rgb_t_no_grad(self, ray_o, ray_d, score_threshold: float = 1e-3, bg_color=None, view_matrix=None,
                             proj_matrix=None):
        """(rgb, t, alpha) with t the expected depth (scannet/cumodel.py:1385-1525)."""
        if getattr(self, "camera_mode", "legacy-centered") == "colmap-native":
            raise NotImplementedError("Native camera depth rendering is not implemented; use forward for RGB/features")
        if self.image_size is None:
            raise ValueError("image_size must be set on NeuralPrimitiveSceneTileCUDA before calling render_rgb_t_no_grad.")
        if view_matrix is None or proj_matrix is None:
            raise ValueError("Tile renderer requires view_matrix and proj_matrix for culling.")
        W, H = self.image_size
        assert ray_o.shape[0] == W * H, "Tile renderer requires full-frame rays (B == W*H)"
        device = self._activate_cuda_device()
        ts = int(self.tile_size)
        cand, offsets = self._legacy_culling(_host_matrix(view_matrix).reshape(1, 4, 4), _host_matrix(proj_matrix),
                                             score_threshold, ts)
        ext = self._ensure_tile_ext()
        base = self._base_args(ray_o, ray_d, cand, offsets, device)
        rgb, alpha, t = ext.render_tiles_forward_tilecenter_with_t(*base, int(W), int(H), ts, ts, float(score_threshold))
        return _add_background(rgb, alpha, self._background(bg_color, ray_o)), t, alpha
