"""A saved fp16 inference export rendered on the matrix cores without an f32 copy of its weights in between.

The reference's export keeps MLP weights, biases and feature attributes as float16 and everything else as float32
(scannet/checkpoints.py:317-381), and its loader widens them again (:299-314).  ``scene_from_checkpoint(...,
keep_half_storage=True)`` keeps them as stored; the matrix-core render packs its operand blocks and its fp16
attribute layout straight from that storage.  Checked here on a seeded scene saved that way:
  * the packed blocks equal, bit for bit, those packed from the widened (f32-loaded) tensors;
  * the image and the feature image equal, bit for bit, those of the f32-loaded scene in the same precision;
  * the image agrees with the oracle's emulation of the operand rounding, evaluated on the widened weights, to the
    tolerance of the path (5e-3 bf16, 5e-4 fp16).
"""
import numpy as np
import pytest
import torch

from conftest import to_dev
from helpers import Frame

pytestmark = pytest.mark.gpu

MLP = ("W1", "b1", "W2", "b2", "W3", "b3")


def _inference_export(fr, path):
    """The file an inference export of this scene is: wrapper with metadata, geometry f32, MLP + attributes fp16."""
    sc = fr.scene
    state = {"positions": sc.positions, "log_scales": sc.log_scales, "quats": sc.quats}
    state.update({k: getattr(sc, k) for k in MLP})
    state["feat_attr"] = sc.feat_attr
    tensors = {k: torch.from_numpy(np.ascontiguousarray(v)) for k, v in state.items()}
    for k in (*MLP, "feat_attr"):
        tensors[k] = tensors[k].half()
    torch.save({"scene_state_dict": tensors,
                "metadata": {"inference_only": True, "feature_slots": 4, "feature_dim": int(sc.feat_attr.shape[2]),
                             "storage_precision": "float16_mlp_and_features_float32_geometry",
                             "encoding_kind": "attenuated_phase_v1", "encoding_sigma": 0.01}}, path)
    return tensors


def _render(scene, fr, device, **kw):
    with torch.inference_mode():
        return scene(to_dev(fr.rays_o, device), to_dev(fr.rays_d, device), score_threshold=fr.thr,
                     view_matrix=to_dev(fr.view, device), proj_matrix=to_dev(fr.proj, device), **kw)


@pytest.mark.parametrize("precision", ["bf16", "fp16"])
def test_fp16_export_renders_from_its_own_storage(device, oracle_mod, tmp_path, precision):
    from mlp_splatting_amd import ops
    from mlp_splatting_amd.checkpoints import scene_from_checkpoint
    fr = Frame("cfg1_5k_160x120", n=1500, hidden=32, width=64, height=48, feature_dim=24)
    path = tmp_path / "scene_inference.pt"
    stored = _inference_export(fr, path)

    kept = scene_from_checkpoint(str(path), device, render_precision=precision, keep_half_storage=True)
    wide = scene_from_checkpoint(str(path), device, render_precision=precision)
    for scene in (kept, wide):
        scene.set_image_size(fr.W, fr.H)
    for k in (*MLP, "feat_attr"):
        assert getattr(kept, k).dtype == torch.float16 and getattr(wide, k).dtype == torch.float32
        assert torch.equal(getattr(kept, k).cpu(), stored[k])                      # the stored bits, untouched
        assert torch.equal(getattr(wide, k).cpu(), stored[k].float())
    assert kept.positions.dtype == torch.float32

    # operand blocks: straight from fp16 storage == from the widened tensors
    bf16 = precision == "bf16"
    from_half = ops.pack_mfma_weights(*[getattr(kept, k).detach() for k in MLP], bf16=bf16)
    from_wide = ops.pack_mfma_weights(*[getattr(wide, k).detach() for k in MLP], bf16=bf16)
    assert from_half.numel() == 1500 * 7808 and torch.equal(from_half, from_wide)
    attr_half, bad_half = ops.pack_mfma_feat(kept.feat_attr.detach())
    attr_wide, bad_wide = ops.pack_mfma_feat(wide.feat_attr.detach())
    assert not bad_half and not bad_wide and torch.equal(attr_half, attr_wide)

    # images: the queued RGB frame and the RGB + feature frame
    rgb_kept, rgb_wide = _render(kept, fr, device), _render(wide, fr, device)
    assert torch.equal(rgb_kept, rgb_wide)
    both_kept, both_wide = _render(kept, fr, device, return_feature=True), _render(wide, fr, device, return_feature=True)
    assert torch.equal(both_kept[0], both_wide[0]) and torch.equal(both_kept[1], both_wide[1])
    assert float(both_kept[1].abs().max()) > 0

    # against the oracle on the widened weights
    sc = fr.scene
    cand, off = fr.oracle_lists(oracle_mod)
    q = torch.nn.functional.normalize(to_dev(sc.quats, device), dim=-1).cpu().numpy()
    rd = torch.nn.functional.normalize(to_dev(fr.rays_d, device), dim=-1).cpu().numpy()
    freq, att = (t.cpu().numpy() for t in kept._frequency_tables(device))
    widened = [stored[k].float().numpy() for k in MLP]
    want = oracle_mod.render_tilecenter(fr.rays_o, rd, sc.positions, sc.log_scales, q, cand, off, freq, att, *widened,
                                        *fr.dims, precision=1 if bf16 else 2)
    tol = 5e-3 if bf16 else 5e-4
    err = float(np.abs(rgb_kept.cpu().numpy() - want["rgb"]).max())
    print(f"{precision}: max |image - oracle on widened weights| = {err:.2e}")
    assert err <= tol and want["alpha"].mean() > 0.3


def test_mixed_storage_is_widened_and_f32_render_of_half_storage_matches(device, tmp_path):
    """Half storage of only some MLP tensors is widened as a whole; and the f32 render of a half-stored scene (which
    widens per call) equals the f32 render of the f32-loaded scene."""
    from mlp_splatting_amd.checkpoints import scene_from_checkpoint
    fr = Frame("cfg1_5k_160x120", n=600, hidden=32, width=32, height=24, feature_dim=8)
    path = tmp_path / "scene_inference.pt"
    stored = _inference_export(fr, path)
    kept = scene_from_checkpoint(str(path), device, keep_half_storage=True)
    wide = scene_from_checkpoint(str(path), device)
    for scene in (kept, wide):
        scene.set_image_size(fr.W, fr.H)
    assert torch.equal(_render(kept, fr, device), _render(wide, fr, device))
    mixed = {"scene_state_dict": {**stored, "W2": stored["W2"].float()}}
    scene = scene_from_checkpoint(mixed, device, keep_half_storage=True)
    assert all(getattr(scene, k).dtype == torch.float32 for k in MLP) and scene.feat_attr.dtype == torch.float16
