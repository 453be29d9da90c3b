"""Checkpoint loading (host logic, CPU): the cases of the reference's tests/test_checkpoints.py:43-139,
202-213, 287-300 that concern reading a scene, restated on this package's loader."""
import numpy as np
import pytest
import torch

from mlp_splatting_amd import checkpoints as ck


def _state(n=5, hidden=4, freqs=2, feature=None, dtype=torch.float32):
    g = torch.Generator().manual_seed(0)
    r = lambda *shape: torch.randn(*shape, generator=g)
    s = {"positions": r(n, 3), "log_scales": r(n, 3), "quats": r(n, 4), "W1": r(n, hidden, 12 * freqs).to(dtype),
         "b1": r(n, hidden).to(dtype), "W2": r(n, hidden, hidden).to(dtype), "b2": r(n, hidden).to(dtype),
         "W3": r(n, 4, hidden).to(dtype), "b3": r(n, 4).to(dtype)}
    if feature is not None:
        s["feat_attr"] = r(n, *feature).to(dtype)
    return s


def test_infer_dimensions_and_validate_shapes():
    spec = ck.infer_scene_spec(_state(7, 8, 3, feature=(5, 16)))
    assert spec == ck.SceneSpec(7, 8, 36, 3, 16, 5)
    assert ck.infer_scene_spec(_state(feature=(9,))).feature_slots == 1
    assert ck.infer_scene_spec(_state()).feature_dim == 0
    bad = _state()
    bad["b2"] = torch.zeros(5, 3)
    with pytest.raises(ValueError, match="b2 has shape"):
        ck.infer_scene_spec(bad)
    bad = _state()
    bad["W1"] = torch.zeros(5, 4, 25)
    with pytest.raises(ValueError, match="not divisible by 12"):
        ck.infer_scene_spec(bad)
    bad = _state()
    del bad["quats"]
    with pytest.raises(KeyError, match="quats"):
        ck.infer_scene_spec(bad)


def test_prefixes_and_legacy_mlp_names():
    s = _state()
    renamed = {"module._orig_mod." + k: v for k, v in s.items() if not k.startswith(("W", "b"))}
    for old, new in ck.LEGACY_NAMES.items():
        renamed["module." + old] = s[new]
    out = ck.normalize_scene_state_dict(renamed)
    assert set(out) == set(s) and all(out[k] is s[k] for k in s)
    del renamed["module.mlps.lin2.bias"]
    with pytest.raises(KeyError, match="incomplete legacy MLP state"):
        ck.normalize_scene_state_dict(renamed)
    with pytest.raises(ValueError, match="key collision"):
        ck.normalize_scene_state_dict({"module.positions": s["positions"], "positions": s["positions"].clone()})


def test_five_to_four_is_the_same_feature_and_four_to_five_round_trips():
    f5 = _state(feature=(5, 6))["feat_attr"]
    f4 = ck.convert_feature_slots(f5, 4)
    gates = torch.softmax(torch.randn(5, 4), dim=1)                       # any gates that sum to one
    five = f5[:, 0] + (gates[:, :, None] * f5[:, 1:]).sum(1)
    four = (gates[:, :, None] * f4).sum(1)
    torch.testing.assert_close(five, four, rtol=1e-6, atol=1e-6)
    back = ck.convert_feature_slots(ck.convert_feature_slots(f4, 5), 4)
    assert torch.equal(back, f4) and ck.convert_feature_slots(f4, 4) is not f4
    with pytest.raises(ValueError, match="target_slots"):
        ck.convert_feature_slots(f4, 8)
    with pytest.raises(ValueError, match="cannot convert"):
        ck.convert_feature_slots(torch.zeros(2, 3, 4), 4)


def test_wrappers_and_bare_states():
    s = _state()
    assert ck.split_checkpoint(s) == (s, None)
    assert ck.split_checkpoint({"scene_state_dict": s, "epoch": 3})[1] == "scene_state_dict"
    assert ck.split_checkpoint({"state_dict": s})[1] == "state_dict"
    with pytest.raises(ValueError, match="could not find a scene state_dict"):
        ck.split_checkpoint({"epoch": 1})
    with pytest.raises(TypeError):
        ck.split_checkpoint([1, 2])


def test_restore_widens_half_storage_and_rejects_half_geometry():
    s = _state(dtype=torch.float16, feature=(4, 8))
    out = ck.restore_scene_state_dict(s)
    assert all(v.dtype == torch.float32 for v in out.values()) and s["W1"].dtype == torch.float16
    assert torch.equal(out["W1"], s["W1"].float())
    s["positions"] = s["positions"].half()
    with pytest.raises(TypeError, match="positions: FP16 storage is only supported"):
        ck.restore_scene_state_dict(s)
    s = _state()
    s["b3"] = s["b3"].to(torch.bfloat16)
    with pytest.raises(TypeError, match="unsupported scene storage dtype"):
        ck.restore_scene_state_dict(s)


def test_camera_mode_metadata():
    assert ck.checkpoint_camera_mode({}) == "legacy-centered"
    native = {"metadata": {"camera_mode": "colmap-native", "camera_pixel_center": 0.5, "camera_culling": "raycone-v1",
                           "camera_intrinsics": {"fx": 1.0}}}
    assert ck.checkpoint_camera_mode(native) == "colmap-native"
    native["metadata"]["camera_culling"] = "other"
    with pytest.raises(ValueError, match="incompatible pixel-center/culling"):
        ck.checkpoint_camera_mode(native)
    with pytest.raises(ValueError, match="Unsupported checkpoint camera_mode"):
        ck.checkpoint_camera_mode({"metadata": {"camera_mode": "fisheye"}})


@pytest.mark.parametrize("wrapped", [False, True])
def test_scene_from_a_saved_checkpoint_is_float32_and_complete(tmp_path, wrapped):
    s = _state(6, 32, 6, feature=(5, 12), dtype=torch.float16)
    meta = {"feature_gating_beta": 1.25, "feature_gating_temperature": 3.0, "encoding_sigma": 0.02,
            "encoding_kind": "attenuated_phase_v1"}
    path = tmp_path / "scene_epoch_1.pt"
    torch.save({"scene_state_dict": {"module." + k: v for k, v in s.items()}, "metadata": meta, "epoch": 1}
               if wrapped else s, path)
    scene = ck.scene_from_checkpoint(str(path), "cpu", feature_slots=4, render_precision="bf16")
    assert not scene.training and scene.camera_mode == "legacy-centered" and scene.render_precision == "bf16"
    assert scene.num_primitives == 6 and scene.hidden_dim == 32 and scene.pe_frequencies == 6
    assert all(p.dtype == torch.float32 for p in scene.parameters())
    assert torch.equal(scene.W2.detach(), s["W2"].float())
    assert tuple(scene.feat_attr.shape) == (6, 4, 12)                    # 5 slots folded into 4
    torch.testing.assert_close(scene.feat_attr.detach(), (s["feat_attr"].float()[:, :1] + s["feat_attr"].float()[:, 1:]))
    if wrapped:
        assert scene.feature_gating_beta == 1.25 and scene.feature_gating_temp == 3.0
        assert abs(float(scene.encoder.sigma2) - 0.02 ** 2) < 1e-12
    missing = dict(s)
    del missing["b3"]
    with pytest.raises((RuntimeError, KeyError), match="b3"):
        ck.scene_from_checkpoint(missing, "cpu")
    with pytest.raises(ValueError, match="encoding_kind"):
        ck.scene_from_checkpoint({"scene_state_dict": s, "metadata": {"encoding_kind": "hash"}}, "cpu")
