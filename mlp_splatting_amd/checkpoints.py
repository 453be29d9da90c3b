"""Scene checkpoints -> a ready ``NeuralPrimitiveSceneTileCUDA`` (the loading half of scannet/checkpoints.py and
of ``_load_scene_tile_cuda``, scannet/eval_rgb_psnr.py:156-235).  No renderer dependency except in
:func:`scene_from_checkpoint`.

Accepted on disk: a bare scene ``state_dict`` or a training wrapper holding it under ``scene_state_dict`` /
``state_dict``; ``module.`` / ``_orig_mod.`` key prefixes; the old ``mlps.lin{1,2,3}.{weight,bias}`` names;
MLP weights and feature attributes stored as float16 (the inference export, scannet/checkpoints.py:317-381),
geometry always float32.  Files are read with ``torch.load(weights_only=True)`` only.
"""
from __future__ import annotations

from collections.abc import Mapping
from dataclasses import dataclass
from typing import Any

import torch

WRAPPER_KEYS = ("scene_state_dict", "state_dict")
KEY_PREFIXES = ("module.", "_orig_mod.")
LEGACY_NAMES = {"mlps.lin1.weight": "W1", "mlps.lin1.bias": "b1", "mlps.lin2.weight": "W2", "mlps.lin2.bias": "b2",
                "mlps.lin3.weight": "W3", "mlps.lin3.bias": "b3"}
HALF_STORAGE_OK = frozenset(("W1", "b1", "W2", "b2", "W3", "b3", "feat_attr"))
# buffers a checkpoint may lack without harm (scannet/eval_rgb_psnr.py:215-224)
BENIGN_MISSING = frozenset(("encoder.freq_bands", "stat_sum_w", "stat_max_w", "stat_hits", "stat_contrib_count",
                            "stat_sum_werr", "alpha_accum"))


@dataclass(frozen=True)
class SceneSpec:
    """What the tensor shapes alone say about a scene (scannet/checkpoints.py:42-52)."""
    num_primitives: int
    hidden_dim: int
    encoded_dim: int
    pe_frequencies: int
    feature_dim: int
    feature_slots: int


def _looks_like_scene_state(value) -> bool:
    return (isinstance(value, Mapping) and len(value) > 0 and
            any(isinstance(k, str) and k.endswith(("positions", "W1", "mlps.lin1.weight")) for k in value))


def split_checkpoint(checkpoint) -> tuple[dict, str | None]:
    """(scene state dict, wrapper key or None) of a bare or wrapped checkpoint (scannet/checkpoints.py:71-96)."""
    if not isinstance(checkpoint, Mapping):
        raise TypeError(f"checkpoint must be a mapping, got {type(checkpoint).__name__}")
    for key in WRAPPER_KEYS:
        if _looks_like_scene_state(checkpoint.get(key)):
            return dict(checkpoint[key]), key
    if _looks_like_scene_state(checkpoint):
        return dict(checkpoint), None
    raise ValueError("could not find a scene state_dict; expected a bare scene state_dict or a "
                     "'scene_state_dict'/'state_dict' wrapper")


def normalize_scene_state_dict(state_dict, *, remap_legacy_mlp: bool = True) -> dict:
    """Drop DDP / torch.compile key prefixes and rename the old MLP parameters; everything else is kept.
    Two keys that collapse onto one name must be the same object (scannet/checkpoints.py:110-149)."""
    if not isinstance(state_dict, Mapping):
        raise TypeError("state_dict must be a mapping")
    out: dict[str, Any] = {}
    for key, value in state_dict.items():
        if not isinstance(key, str):
            raise TypeError(f"state_dict key must be str, got {type(key).__name__}")
        name = key
        stripped = True
        while stripped:
            stripped = False
            for prefix in KEY_PREFIXES:
                if name.startswith(prefix):
                    name, stripped = name[len(prefix):], True
        if name in out and out[name] is not value:
            raise ValueError(f"key collision after prefix removal: {key!r} -> {name!r}")
        out[name] = value
    if not remap_legacy_mlp:
        return out
    old_present = [k for k in LEGACY_NAMES if k in out]
    if old_present and len(old_present) != len(LEGACY_NAMES):
        raise KeyError(f"incomplete legacy MLP state; missing {sorted(set(LEGACY_NAMES) - set(old_present))}")
    for old, new in LEGACY_NAMES.items():
        if old not in out:
            continue
        value = out.pop(old)
        if new in out and out[new] is not value:
            same = (torch.is_tensor(out[new]) and torch.is_tensor(value) and out[new].shape == value.shape
                    and torch.equal(out[new], value))
            if not same:
                raise ValueError(f"both legacy key {old!r} and canonical key {new!r} differ")
        else:
            out[new] = value
    return out


def _need(state, key) -> torch.Tensor:
    value = state.get(key)
    if not torch.is_tensor(value):
        raise KeyError(f"required tensor {key!r} is missing")
    return value


def infer_scene_spec(state_dict) -> SceneSpec:
    """N, hidden width, encoding width and feature layout from the tensor shapes, with every other tensor
    checked against them (scannet/checkpoints.py:165-216)."""
    state = normalize_scene_state_dict(state_dict)
    w1 = _need(state, "W1")
    if w1.ndim != 3:
        raise ValueError(f"W1 must have shape [N,H,encoded_dim], got {tuple(w1.shape)}")
    n, hidden, enc = (int(v) for v in w1.shape)
    if min(n, hidden, enc) <= 0:
        raise ValueError("scene dimensions must be positive")
    if enc % 12:
        raise ValueError(f"encoded_dim={enc} is not divisible by 12 (6D input x sin/cos positional encoding)")
    expected = {"b1": (n, hidden), "W2": (n, hidden, hidden), "b2": (n, hidden), "W3": (n, 4, hidden), "b3": (n, 4),
                "positions": (n, 3), "log_scales": (n, 3), "quats": (n, 4)}
    for name, shape in expected.items():
        got = tuple(_need(state, name).shape)
        if got != shape:
            raise ValueError(f"{name} has shape {got}, expected {shape}")
    feature_dim = feature_slots = 0
    feat = state.get("feat_attr")
    if feat is not None:
        if not torch.is_tensor(feat):
            raise TypeError("feat_attr must be a tensor")
        if feat.ndim == 2 and int(feat.shape[0]) == n:
            feature_dim, feature_slots = int(feat.shape[1]), 1
        elif feat.ndim == 3:
            if int(feat.shape[0]) != n:
                raise ValueError(f"feat_attr has N={feat.shape[0]}, expected {n}")
            feature_slots, feature_dim = int(feat.shape[1]), int(feat.shape[2])
        else:
            raise ValueError(f"feat_attr must have shape [N,D] or [N,S,D], got {tuple(feat.shape)}")
        if feature_dim <= 0 or feature_slots <= 0:
            raise ValueError("feature dimensions must be positive")
    return SceneSpec(n, hidden, enc, enc // 12, feature_dim, feature_slots)


def convert_feature_slots(feature: torch.Tensor, target_slots: int) -> torch.Tensor:
    """4 <-> 5 directional feature slots without changing the rendered feature: the five-slot layout is a
    base plus four deltas, and the four gates sum to one, so ``slot_k = base + delta_k`` is the same image;
    the way back takes a zero base, which makes 4 -> 5 -> 4 exact (scannet/checkpoints.py:219-241)."""
    if not torch.is_tensor(feature) or feature.ndim != 3:
        raise ValueError("feature must be a tensor with shape [N,S,D]")
    if target_slots not in (4, 5):
        raise ValueError("target_slots must be 4 or 5")
    have = int(feature.shape[1])
    if have == target_slots:
        return feature.clone()
    if have == 5:
        return feature[:, :1, :] + feature[:, 1:, :]
    if have == 4:
        return torch.cat((torch.zeros_like(feature[:, :1, :]), feature), dim=1)
    raise ValueError(f"cannot convert {have}-slot features to {target_slots} slots")


def restore_scene_state_dict(state_dict) -> dict:
    """float32 copies of every floating tensor; float16 is storage for MLP weights and features only, never
    for geometry (scannet/checkpoints.py:299-314).  The input is not modified."""
    state = normalize_scene_state_dict(state_dict)
    for name, value in state.items():
        if not torch.is_tensor(value) or not value.is_floating_point():
            continue
        if value.dtype == torch.float16 and name not in HALF_STORAGE_OK:
            raise TypeError(f"{name}: FP16 storage is only supported for MLP weights and features")
        if value.dtype not in (torch.float16, torch.float32, torch.float64):
            raise TypeError(f"{name}: unsupported scene storage dtype {value.dtype}")
        state[name] = value.float()
    return state


def checkpoint_camera_mode(checkpoint) -> str:
    """``legacy-centered`` or ``colmap-native`` from the wrapper metadata, with the native mode's
    consistency requirements (scannet/camera.py:11-23)."""
    metadata = checkpoint.get("metadata", {})
    if not isinstance(metadata, Mapping):
        raise ValueError("Checkpoint metadata must be a dictionary")
    mode = metadata.get("camera_mode", "legacy-centered")
    if mode not in {"legacy-centered", "colmap-native"}:
        raise ValueError(f"Unsupported checkpoint camera_mode={mode!r}")
    if mode == "colmap-native":
        if metadata.get("camera_pixel_center") != 0.5 or metadata.get("camera_culling") != "raycone-v1":
            raise ValueError("Native camera checkpoint has incompatible pixel-center/culling metadata")
        if not isinstance(metadata.get("camera_intrinsics"), Mapping):
            raise ValueError("Native camera checkpoint must record its COLMAP calibration")
    return mode


def load_checkpoint(path):
    """The checkpoint mapping of a file, read without executing anything it contains."""
    return torch.load(path, map_location="cpu", weights_only=True)


def half_stored_tensors(state_dict) -> dict:
    """The tensors of a checkpoint that an inference export stores as float16 (MLP weights, biases, feature
    attributes; scannet/checkpoints.py:317-381), under their canonical names and exactly as stored."""
    state = normalize_scene_state_dict(state_dict)
    return {name: value for name, value in state.items()
            if name in HALF_STORAGE_OK and torch.is_tensor(value) and value.dtype == torch.float16}


def scene_from_checkpoint(checkpoint, device, *, min_points: int = 10, tile_size: int = 8, feature_gating_beta=None,
                          feature_gating_temp=None, feature_slots: int | None = None, render_precision: str | None = None,
                          keep_half_storage: bool = False):
    """Build the renderer module for a checkpoint (mapping or path), the way the reference's evaluators do
    (scannet/eval_rgb_psnr.py:156-235): dimensions from the tensors, encoding and gating constants from the
    wrapper's ``metadata``, float16-stored tensors widened, ``load_state_dict(strict=False)`` with the benign
    missing buffers, ``camera_mode`` from the metadata, ``eval()``.  ``feature_slots`` re-expresses 4/5-slot
    features in the other layout first.

    ``keep_half_storage``: the tensors an inference export stores as float16 stay float16 on the device (half the
    memory of the scene), and the matrix-core render (``render_precision`` "bf16" / "fp16") packs its operand blocks
    and its fp16 attribute layout straight from them -- the checkpoint's values reach the kernels without an f32
    copy in between.  All six MLP tensors must be stored that way; the f32 render paths widen per call."""
    from .cumodel import NeuralPrimitiveSceneTileCUDA
    if not isinstance(checkpoint, Mapping):
        checkpoint = load_checkpoint(checkpoint)
    if not isinstance(checkpoint, Mapping):
        raise TypeError("Unsupported checkpoint format")
    state, _wrapper = split_checkpoint(checkpoint)
    metadata = checkpoint.get("metadata", {})
    if not isinstance(metadata, Mapping):
        metadata = {}
    kind = str(metadata.get("encoding_kind", "attenuated_phase_v1"))
    if kind not in {"attenuated_phase_v1", "fourier_features_v1"}:
        raise ValueError(f"Unsupported checkpoint encoding_kind={kind!r}")
    stored_half = half_stored_tensors(state) if keep_half_storage else {}
    state = restore_scene_state_dict(state)
    spec = infer_scene_spec(state)
    if feature_slots is not None and spec.feature_slots in (4, 5) and feature_slots != spec.feature_slots:
        state["feat_attr"] = convert_feature_slots(state["feat_attr"], int(feature_slots))
        stored_half.pop("feat_attr", None)          # re-expressed in f32: no longer the stored tensor
        spec = infer_scene_spec(state)
    mlp_names = ("W1", "b1", "W2", "b2", "W3", "b3")
    if stored_half and not all(k in stored_half for k in mlp_names):
        for k in mlp_names:                         # a mixture of storage types is widened as a whole
            stored_half.pop(k, None)
    beta = float(metadata.get("feature_gating_beta", 1.5) if feature_gating_beta is None else feature_gating_beta)
    temp = float(metadata.get("feature_gating_temperature", 2.0) if feature_gating_temp is None else feature_gating_temp)
    scene = NeuralPrimitiveSceneTileCUDA(
        num_primitives=spec.num_primitives, hidden_dim=spec.hidden_dim, pe_frequencies=spec.pe_frequencies,
        use_integrated_pe=(kind == "attenuated_phase_v1"), pe_sigma=float(metadata.get("encoding_sigma", 0.01)),
        initial_positions=None, min_points=int(min_points), tile_size=int(tile_size),
        feature_dim_low=spec.feature_dim, feature_slots=spec.feature_slots if spec.feature_slots in (4, 5) else 4,
        feature_gating_beta=beta, feature_gating_temp=temp).to(device)
    missing, unexpected = scene.load_state_dict(state, strict=False)
    missing = [k for k in missing if k not in BENIGN_MISSING]
    if missing:
        raise RuntimeError(f"Checkpoint is missing required scene tensors: {missing[:10]} (total={len(missing)})")
    if unexpected:
        print(f"[Warn] Unexpected keys while loading scene: {unexpected[:10]} (total={len(unexpected)})")
    for name, value in stored_half.items():
        setattr(scene, name, torch.nn.Parameter(value.to(device).contiguous(), requires_grad=False))
    scene.camera_mode = checkpoint_camera_mode(checkpoint)
    scene.checkpoint_metadata = dict(metadata)
    if render_precision is not None:
        scene.render_precision = render_precision
    scene.eval()
    return scene
