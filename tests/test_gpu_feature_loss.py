"""Streamed feature L1 loss and its attribute gradients (HIP) against the dense definition: the feature image of
the exact render kernel (bit-identical to the oracle, tests/test_gpu_parity.py), torch's bilinear
``F.interpolate(align_corners=False)``, ``F.l1_loss`` and autograd through a float64 framebuffer built from the
records.  Cases and tolerances follow the reference's tests (tests/test_record_feature_loss.py:8-51,
tests/test_record_feature_512.py:130-200): prediction 3e-6, loss 2e-7 / 2e-6, signs exact, f32 gradients
2e-6 / 2e-5, mixed gradients relative L2 < 0.003."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from conftest import to_dev
from helpers import Frame

pytestmark = pytest.mark.gpu


def _frame_records(device, oracle_mod, width, height, n=500, seed_eye=(0.3, 0.2, -2.0)):
    from mlp_splatting_amd.tile_ext import TileExt
    fr = Frame("cfg1_5k_160x120", n=n, hidden=32, width=width, height=height, eye=seed_eye, target=(0.0, 0.0, 0.0))
    cand, off = fr.oracle_lists(oracle_mod)
    base = [to_dev(a, device) for a in fr.base_numpy(cand, off)]
    ext = TileExt()
    x = base + [torch.zeros_like(base[0]), torch.zeros(width * height, device=device)]
    records = ext.render_tiles_training_records(x, width, height, 8, fr.thr, 1.5, 2.0)
    return fr, ext, base, records


def _framebuffer64(records, attributes, width, height):
    """Dense feature image from records, float64, differentiable in ``attributes`` only."""
    _, _, ids, x6, raw, masks, gates, offsets = [t.cpu() if torch.is_tensor(t) else t for t in records]
    ids = ids.long()
    w = (raw[:, 4] * raw[:, 5]).double()
    g = gates.double()
    a = attributes
    if a.dim() == 2:
        mix = a[ids]
    elif a.shape[1] == 4:
        mix = (g[:, :, None] * a[ids]).sum(1)
    else:
        mix = a[ids, 0] + (g[:, :, None] * a[ids, 1:]).sum(1)
    pix = torch.repeat_interleave(torch.arange(width * height), offsets.diff())
    out = torch.zeros(width * height, a.shape[-1], dtype=torch.float64)
    return out.index_add(0, pix, w[:, None] * mix)


def _resize(dense, width, height, wf, hf):
    image = dense.view(height, width, -1).permute(2, 0, 1).unsqueeze(0)
    return F.interpolate(image, size=(hf, wf), mode="bilinear", align_corners=False).squeeze(0).permute(1, 2, 0)


_SIZES = [(9, 7, 7, 5), (8, 8, 8, 8), (33, 19, 23, 11), (9, 7, 1, 1), (15, 1, 8, 1), (1, 13, 1, 7)]
# f32 targets for every slot count and size; fp16 targets with four slots on the sizes whose width is 9 or 33
_CASES = ([(slots, size, False) for slots in (1, 4, 5) for size in _SIZES]
          + [(4, size, True) for size in _SIZES if size[0] in (9, 33)])


@pytest.mark.parametrize("slots,size,half_target", _CASES)
def test_streamed_l1_and_attribute_gradients_match_the_dense_definition(device, oracle_mod, slots, size, half_target):
    from mlp_splatting_amd import primitive_gemm as gemm
    from mlp_splatting_amd.primitive_csr import group_records
    from mlp_splatting_amd.record_feature_loss import feature_weight_gradients, streaming_feature_l1
    width, height, wf, hf = size
    fr, ext, base, records = _frame_records(device, oracle_mod, width, height)
    n, channels = fr.scene.n, 150
    torch.manual_seed(482 + slots)
    attr = torch.randn((n, channels) if slots == 1 else (n, slots, channels), device=device) * 0.2
    target = torch.randn(hf, wf, channels, device=device) * 0.2
    if half_target:
        target = target.half()
    assert records[2].numel() > 0
    # the dense image of the exact render kernel and torch's resampling
    _, _, dense = ext.render_tiles_forward_tilecenter_with_feat(*base, attr, 1.5, 2.0, width, height, 8, 8, fr.thr)
    expected_prediction = _resize(dense, width, height, wf, hf)
    expected_loss = F.l1_loss(expected_prediction, target.float())
    loss, signs, prediction = streaming_feature_l1(records, attr, target, width, height, debug=True)
    torch.testing.assert_close(prediction, expected_prediction, atol=3e-6, rtol=3e-6)
    torch.testing.assert_close(loss, expected_loss, atol=2e-7, rtol=2e-6)
    expected_signs = (expected_prediction - target.float()).sign().to(torch.int8)
    settled = (expected_prediction - target.float()).abs() > 1e-5     # a residual within rounding of zero may flip
    assert torch.equal(signs[settled], expected_signs[settled]) and float(settled.float().mean()) > 0.999
    loss2, signs2, none = streaming_feature_l1(records, attr, target, width, height)
    assert none is None and torch.equal(signs2, signs) and torch.equal(loss2, loss)
    # gradient: autograd through the float64 framebuffer, with the kernel's own signs as the L1 subgradient
    leaf = attr.detach().cpu().double().requires_grad_(True)
    pred64 = _resize(_framebuffer64(records, leaf, width, height), width, height, wf, hf)
    torch.testing.assert_close(pred64.float(), prediction.cpu(), atol=3e-6, rtol=3e-6)
    (pred64 * signs.cpu().double()).sum().div(hf * wf * channels).backward()
    ids, x6 = records[2:4]
    csr = group_records(ids, x6, torch.zeros((len(ids), 4), device=device), n, records[5])
    for segment in (32, 512):
        for mixed in (False, True):
            actual = feature_weight_gradients(records, csr, signs, attr, width, height, mixed=mixed,
                                              segment_size=segment).cpu().double()
            assert actual.shape == leaf.grad.shape
            if not mixed:
                torch.testing.assert_close(actual, leaf.grad, atol=2e-6, rtol=2e-5)
            else:
                assert float((actual - leaf.grad).norm() / leaf.grad.norm().clamp_min(1e-30)) < 0.003
            untouched = torch.bincount(ids.long().cpu(), minlength=n) == 0
            assert untouched.any() and not actual[untouched].any()


def test_feature_loss_argument_checks(device, oracle_mod):
    from mlp_splatting_amd.record_feature_loss import feature_weight_gradients, streaming_feature_l1
    fr, ext, base, records = _frame_records(device, oracle_mod, 16, 8, n=100)
    attr = torch.zeros(fr.scene.n, 4, 6, device=device)
    with pytest.raises(ValueError, match="nonempty HWC"):
        streaming_feature_l1(records, attr, torch.zeros(4, 6, device=device), 16, 8)
    with pytest.raises(ValueError, match="contiguous FP32"):
        streaming_feature_l1(records, attr.half(), torch.zeros(4, 8, 6, device=device), 16, 8)
    with pytest.raises(ValueError, match="FP16 or FP32"):
        streaming_feature_l1(records, attr, torch.zeros(4, 8, 6, device=device, dtype=torch.float64), 16, 8)
    with pytest.raises(ValueError, match="1/4/5-slot"):
        streaming_feature_l1(records, torch.zeros(fr.scene.n, 3, 6, device=device), torch.zeros(4, 8, 6, device=device), 16, 8)
    with pytest.raises(ValueError, match="downsampling only"):
        streaming_feature_l1(records, attr, torch.zeros(9, 8, 6, device=device), 16, 8)
    with pytest.raises(ValueError, match="contiguous int8"):
        feature_weight_gradients(records, None, torch.zeros(4, 8, 6, device=device), attr, 16, 8)


@pytest.mark.parametrize("precision", ["float32", "float16"])
@pytest.mark.parametrize("feature_only", [False, True])
def test_scene_csr_training_contract(device, oracle_mod, monkeypatch, precision, feature_only):
    """scene(..., feature_target=...) returns (rgb, streamed loss); its gradients equal those of the dense
    definition (feature image -> bilinear resize -> L1) for the attributes and those of the RGB autograd path
    for everything else (tests/test_record_feature_loss.py:54-101)."""
    from test_gpu_scene import _scene_from
    monkeypatch.setenv("MLPSP_CSR_MLP_PRECISION", precision)
    fr = Frame("cfg1_5k_160x120", n=300, hidden=32, width=24, height=16)
    fr.scene.feat_attr = (np.random.default_rng(3).standard_normal((fr.scene.n, 4, 17)) * 0.1).astype(np.float32)
    scene = _scene_from(fr, device, feature=True).train()
    assert scene.feat_attr is not None and scene.feat_attr.shape[1] == 4
    args = (to_dev(fr.rays_o, device), to_dev(fr.rays_d, device))
    kw = dict(score_threshold=fr.thr, view_matrix=to_dev(fr.view, device), proj_matrix=to_dev(fr.proj, device),
              bg_color=0.3)
    torch.manual_seed(165)
    target = torch.randn(11, 17, 17, device=device) * 0.1
    rgb_target = torch.randn(fr.W * fr.H, 3, device=device) * 0.1
    scene.zero_grad(set_to_none=True)
    rgb, feature_loss = scene(*args, return_feature=True, feature_target=target, **kw)
    assert rgb.shape == (fr.W * fr.H, 3) and feature_loss.dim() == 0
    loss = 0.7 * feature_loss
    if not feature_only:
        loss = loss + F.l1_loss(rgb, rgb_target)
    loss.backward()
    got = {k: (None if p.grad is None else p.grad.clone()) for k, p in scene.named_parameters()}
    # dense definition of the feature part
    with torch.no_grad():
        _, dense = scene(*args, return_feature=True, **kw)
    dense = dense.detach().requires_grad_()
    small = _resize(dense, fr.W, fr.H, 17, 11)
    dense_loss = F.l1_loss(small, target)
    torch.testing.assert_close(feature_loss.detach(), dense_loss.detach(), atol=2e-6, rtol=2e-6)
    # attribute gradient by autograd through the float64 framebuffer of the records
    ext = scene._ensure_tile_ext()
    with torch.no_grad():
        rd = F.normalize(args[1], dim=-1).contiguous()
        cand, off = scene._tile_lists(args[0], rd, fr.thr, kw["view_matrix"], kw["proj_matrix"], None, None, device)
        freq, att = scene._frequency_tables(device)
        x = [args[0], rd, scene.positions.detach(), scene.log_scales.detach(), F.normalize(scene.quats.detach(), dim=-1),
             cand, off.to(torch.int32), freq, att, *[getattr(scene, k).detach() for k in ("W1", "b1", "W2", "b2", "W3", "b3")]]
        x = [t.contiguous() for t in x] + [torch.zeros_like(args[0]), torch.zeros(fr.W * fr.H, device=device)]
        records = ext.render_tiles_training_records(x, fr.W, fr.H, 8, fr.thr, float(scene.feature_gating_beta),
                                                    float(scene.feature_gating_temp))
    leaf = scene.feat_attr.detach().cpu().double().requires_grad_(True)
    pred64 = _resize(_framebuffer64(records, leaf, fr.W, fr.H), fr.W, fr.H, 17, 11)
    (0.7 * F.l1_loss(pred64, target.cpu().double())).backward()
    a, b = got["feat_attr"].cpu().double(), leaf.grad
    if precision == "float32":
        torch.testing.assert_close(a, b, atol=5e-6, rtol=5e-5)
    else:
        assert float((a - b).norm() / b.norm().clamp_min(1e-30)) < 0.003
    # everything else: the RGB autograd path
    geometry_and_mlp = ("positions", "log_scales", "quats", "W1", "b1", "W2", "b2", "W3", "b3")
    if feature_only:
        assert all(got[k] is None for k in geometry_and_mlp)
        return
    scene.zero_grad(set_to_none=True)
    F.l1_loss(scene(*args, **kw), rgb_target).backward()
    for k in geometry_and_mlp:
        want = getattr(scene, k).grad
        if precision == "float32" or k in ("positions", "log_scales", "quats"):
            torch.testing.assert_close(got[k], want, atol=5e-6, rtol=5e-4)
        else:
            assert float((got[k] - want).norm() / want.norm().clamp_min(1e-30)) < 0.003, k
