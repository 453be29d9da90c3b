"""The differentiable RGB render: scene(...) under autograd, backward through the record pipeline (records
forward -> reverse compositing -> grouped weight gradients).

What pins it: the record structure (which primitive hits which pixel, in which order, and the hit offsets) is
taken from the forward records, everything else -- MLP from the weights, falloff from positions, log-scales and
normalised quaternions, compositing, background -- is recomputed in float64 with torch autograd.  The
gradients the reference defines flow through the MLP outputs and through the Gaussian falloff at a fixed hit
offset (scannet/cuda/primitive_records.cuh:3-46); the restatement detaches exactly those inputs."""
import numpy as np
import pytest
import torch

from conftest import to_dev
from helpers import Frame
from test_gpu_scene import _scene_from

pytestmark = pytest.mark.gpu

PARAMS = ("positions", "log_scales", "quats", "W1", "b1", "W2", "b2", "W3", "b3")


def _float64_gradients(scene, fr, device, weight_img, bg, per_pixel=False):
    """d/dparams of  sum(weight_img * rgb)  with rgb recomposed from the frame's records in float64."""
    ext = scene._ensure_tile_ext()
    with torch.no_grad():
        rd = torch.nn.functional.normalize(to_dev(fr.rays_d, device), dim=-1).contiguous()
        cand, off = scene._tile_lists(to_dev(fr.rays_o, device), rd, fr.thr, to_dev(fr.view, device),
                                      to_dev(fr.proj, device), None, None, device)
        freq, att = scene._frequency_tables(device)
        x = [to_dev(fr.rays_o, device), rd, scene.positions.detach().contiguous(), scene.log_scales.detach().contiguous(),
             torch.nn.functional.normalize(scene.quats.detach(), dim=-1).contiguous(), cand, off.to(torch.int32), freq, att,
             *[getattr(scene, k).detach().contiguous() for k in PARAMS[3:]]]
        x += [torch.zeros_like(x[0]), torch.zeros(fr.W * fr.H, device=device)]
        if per_pixel:
            rgb, alpha, ids, x6, raw, masks, gates, offsets = ext.render_tiles_per_pixel_records(x[:15], fr.W, fr.H, 8, 8,
                                                                                                 fr.thr, 1.5, 2.0)
        else:
            rgb, alpha, ids, x6, raw, masks, gates, offsets = ext.render_tiles_training_records(x, fr.W, fr.H, 8, fr.thr,
                                                                                                1.5, 2.0)
    ids, x6, offsets = ids.cpu().long(), x6.cpu().double(), offsets.cpu()
    leaves = {k: getattr(scene, k).detach().cpu().double().requires_grad_(True) for k in PARAMS}
    freq, att = freq.cpu().double(), att.cpu().double()
    phase = (x6[:, :, None] * freq * att).reshape(len(ids), 36)
    enc = torch.cat([torch.sin(phase), torch.cos(phase)], 1)
    h1 = torch.relu(torch.einsum("rhk,rk->rh", leaves["W1"][ids], enc) + leaves["b1"][ids])
    h2 = torch.relu(torch.einsum("roh,rh->ro", leaves["W2"][ids], h1) + leaves["b2"][ids])
    out = torch.einsum("roh,rh->ro", leaves["W3"][ids], h2) + leaves["b3"][ids]
    colour, sigma_raw = torch.sigmoid(out[:, :3]), torch.nn.functional.softplus(out[:, 3])
    q = torch.nn.functional.normalize(leaves["quats"], dim=-1)[ids]
    w, qx, qy, qz = q.unbind(1)
    rot = torch.stack([torch.stack([1 - 2 * (qy * qy + qz * qz), 2 * (qx * qy - w * qz), 2 * (qx * qz + w * qy)], 1),
                       torch.stack([2 * (qx * qy + w * qz), 1 - 2 * (qx * qx + qz * qz), 2 * (qy * qz - w * qx)], 1),
                       torch.stack([2 * (qx * qz - w * qy), 2 * (qy * qz + w * qx), 1 - 2 * (qx * qx + qy * qy)], 1)], 1)
    pos = leaves["positions"][ids]
    local = torch.einsum("rji,rj->ri", rot, x6[:, 3:6] + (pos - pos.detach()))
    decay = torch.exp(-0.5 * (torch.exp(-2 * leaves["log_scales"][ids]) * local * local).sum(1))
    a = 1 - torch.exp(-sigma_raw * decay)
    wimg = weight_img.cpu().double()
    loss = torch.zeros((), dtype=torch.float64)
    for pix in range(fr.W * fr.H):
        t = torch.ones((), dtype=torch.float64)
        for r in range(int(offsets[pix]), int(offsets[pix + 1])):
            loss = loss + (wimg[pix] * colour[r]).sum() * t * a[r]
            t = t * (1 - a[r])
        if bg is not None:
            loss = loss + (wimg[pix] * bg.cpu().double()).sum() * t
    loss.backward()
    return {k: v.grad for k, v in leaves.items()}, int(len(ids)), rgb


@pytest.mark.parametrize("with_bg", [False, True])
def test_scene_gradients_match_float64_autograd_over_the_same_records(device, oracle_mod, with_bg):
    fr = Frame("cfg1_5k_160x120", n=600, hidden=32, width=32, height=24)
    scene = _scene_from(fr, device).train()
    torch.manual_seed(0)
    weight_img = torch.randn(fr.W * fr.H, 3, device=device)
    bg = torch.tensor([0.2, 0.5, 0.9], device=device) if with_bg else None
    rgb = scene(to_dev(fr.rays_o, device), to_dev(fr.rays_d, device), score_threshold=fr.thr, bg_color=bg,
                view_matrix=to_dev(fr.view, device), proj_matrix=to_dev(fr.proj, device))
    assert rgb.requires_grad
    (rgb * weight_img).sum().backward()
    want, num_records, rgb_records = _float64_gradients(scene, fr, device, weight_img, bg)
    assert num_records > 1500
    for k in PARAMS:
        got = getattr(scene, k).grad
        assert got is not None and got.shape == getattr(scene, k).shape, k
        g, w = got.cpu().double(), want[k]
        scale = float(w.abs().max())
        assert scale > 1e-4, k
        assert float((g - w).abs().max()) <= 2e-3 * scale, (k, float((g - w).abs().max()), scale)
        assert float((g - w).norm() / w.norm()) < 1e-3, k


def test_per_pixel_order_gradients_match_float64_autograd_over_its_records(device, oracle_mod, monkeypatch):
    """MLPSP_TILE_ORDER=per_pixel: the backward of the per-pixel order (scannet/cumodel.py:297-364) through the
    per-pixel records, against the same float64 restatement over those records; the forward is the per-pixel
    render."""
    monkeypatch.setenv("MLPSP_TILE_ORDER", "per_pixel")
    fr = Frame("cfg1_5k_160x120", n=600, hidden=32, width=32, height=24)
    scene = _scene_from(fr, device).train()
    torch.manual_seed(1)
    weight_img = torch.randn(fr.W * fr.H, 3, device=device)
    bg = torch.tensor([0.3, 0.1, 0.7], device=device)
    args = dict(score_threshold=fr.thr, bg_color=bg, view_matrix=to_dev(fr.view, device),
                proj_matrix=to_dev(fr.proj, device))
    rgb = scene(to_dev(fr.rays_o, device), to_dev(fr.rays_d, device), **args)
    with torch.no_grad():
        plain = scene(to_dev(fr.rays_o, device), to_dev(fr.rays_d, device), **args)
    assert rgb.requires_grad and torch.equal(rgb, plain)
    (rgb * weight_img).sum().backward()
    want, num_records, _ = _float64_gradients(scene, fr, device, weight_img, bg, per_pixel=True)
    assert num_records > 1500
    for k in PARAMS:
        got = getattr(scene, k).grad
        assert got is not None and got.shape == getattr(scene, k).shape, k
        g, w = got.cpu().double(), want[k]
        scale = float(w.abs().max())
        assert scale > 1e-4, k
        assert float((g - w).abs().max()) <= 2e-3 * scale, (k, float((g - w).abs().max()), scale)
        assert float((g - w).norm() / w.norm()) < 1e-3, k
    monkeypatch.setenv("MLPSP_TILE_ORDER", "tilecenter")
    scene.zero_grad(set_to_none=True)
    other = scene(to_dev(fr.rays_o, device), to_dev(fr.rays_d, device), **args)
    assert float((other.detach() - rgb.detach()).abs().max()) > 1e-5            # the two orders are different images here


def test_reference_style_per_pixel_backward_through_count_and_emit(device, oracle_mod, monkeypatch):
    """The reference's own mode-0 backward (scannet/cumodel.py:297-364), spelled out against this build's entry
    points: count -> exclusive scan -> emit -> torch autograd through the MLP of the emitted (prim_id, x6) with the
    emitted adjoints of (rgb, sigma_raw).  It must give the gradients of the scene module's per-pixel backward."""
    from mlp_splatting_amd.cumodel import _encode_x6, _mlp_forward_indexed
    monkeypatch.setenv("MLPSP_TILE_ORDER", "per_pixel")
    fr = Frame("cfg1_5k_160x120", n=500, hidden=32, width=24, height=16)
    scene = _scene_from(fr, device).train()
    ro, rd = to_dev(fr.rays_o, device), to_dev(fr.rays_d, device)
    view, proj = to_dev(fr.view, device), to_dev(fr.proj, device)
    torch.manual_seed(5)
    weight_img = torch.randn(fr.W * fr.H, 3, device=device)
    rgb = scene(ro, rd, score_threshold=fr.thr, view_matrix=view, proj_matrix=proj)
    (rgb * weight_img).sum().backward()
    mine = {k: getattr(scene, k).grad.clone() for k in PARAMS}
    ext = scene._ensure_tile_ext()
    with torch.no_grad():
        unit = torch.nn.functional.normalize(rd, dim=-1).contiguous()
        cand, off = scene._tile_lists(ro, unit, fr.thr, view, proj, None, None, device)
        base = scene._base_args(ro, rd, cand, off, device)
        dims = (fr.W, fr.H, 8, 8, fr.thr)
        counts = ext.render_tiles_backward_count_per_pixel(*base, *dims)
        offsets = torch.zeros_like(counts)
        offsets[1:] = torch.cumsum(counts[:-1], 0)
        total = int(offsets[-1] + counts[-1])
        prim_id, x6, g_rgb, g_sigma, gp, gs, gq = ext.render_tiles_backward_emit_per_pixel(
            *base, weight_img, torch.zeros(fr.W * fr.H, device=device), counts, offsets, total, *dims)
    assert total > 1000 and prim_id.numel() == total
    weights = [getattr(scene, k).detach().clone().requires_grad_(True) for k in PARAMS[3:]]
    colour, sigma_raw = _mlp_forward_indexed(_encode_x6(x6, base[7], base[8]), prim_id.long(), *weights)
    grads = torch.autograd.grad([colour, sigma_raw], weights, [g_rgb, g_sigma])
    for k, g in zip(PARAMS[3:], grads):
        scale = float(mine[k].abs().max())
        assert scale > 1e-5, k
        assert float((g - mine[k]).abs().max()) <= 2e-3 * scale, (k, float((g - mine[k]).abs().max()), scale)
    # geometry: positions and log-scales directly; the module differentiates through the quaternion normalisation
    torch.testing.assert_close(gp, mine["positions"], atol=1e-6, rtol=1e-4)
    torch.testing.assert_close(gs, mine["log_scales"], atol=1e-6, rtol=1e-4)


def test_inference_calls_are_untouched_by_the_training_path(device, oracle_mod):
    fr = Frame("cfg1_5k_160x120", n=300, hidden=32, width=32, height=24)
    scene = _scene_from(fr, device)
    args = (to_dev(fr.rays_o, device), to_dev(fr.rays_d, device))
    kw = dict(score_threshold=fr.thr, view_matrix=to_dev(fr.view, device), proj_matrix=to_dev(fr.proj, device))
    with torch.no_grad():
        a = scene(*args, **kw)
    b = scene(*args, **kw)                       # grad mode, parameters require grad: autograd path
    assert not a.requires_grad and b.requires_grad and torch.equal(a, b.detach())
    for p in scene.parameters():
        p.requires_grad_(False)
    c = scene(*args, **kw)
    assert not c.requires_grad and torch.equal(a, c)


def test_a_few_optimiser_steps_reduce_an_image_loss(device, oracle_mod):
    fr = Frame("cfg1_5k_160x120", n=400, hidden=32, width=48, height=32)
    scene = _scene_from(fr, device).train()
    args = (to_dev(fr.rays_o, device), to_dev(fr.rays_d, device))
    kw = dict(score_threshold=fr.thr, view_matrix=to_dev(fr.view, device), proj_matrix=to_dev(fr.proj, device))
    with torch.no_grad():
        target = (scene(*args, **kw) * 0.5 + 0.2).clamp(0, 1)
    opt = torch.optim.Adam([{"params": [scene.W1, scene.b1, scene.W2, scene.b2, scene.W3, scene.b3], "lr": 5e-3},
                            {"params": [scene.positions, scene.log_scales, scene.quats], "lr": 1e-3}])
    losses = []
    for _ in range(12):
        opt.zero_grad(set_to_none=True)
        loss = (scene(*args, **kw) - target).abs().mean()
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    assert all(np.isfinite(losses)) and losses[-1] < 0.7 * losses[0], losses


@pytest.mark.parametrize("precision", ["f32", "bf16"])
def test_fused_optimiser_steps_are_seen_by_the_next_render(device, oracle_mod, precision):
    """Adam(fused=True) rewrites parameters without advancing ``tensor._version``, the key of the derived-tensor
    caches (geometry records, unit quaternions, matrix-core operand copies): the grad-mode forward must leave no
    cache behind, so that the render after the step uses the new parameters, as a scene built from them does."""
    fr = Frame("cfg1_5k_160x120", n=400, hidden=32, width=48, height=32)
    scene = _scene_from(fr, device).train()
    scene.render_precision = precision
    args = (to_dev(fr.rays_o, device), to_dev(fr.rays_d, device))
    kw = dict(score_threshold=fr.thr, view_matrix=to_dev(fr.view, device), proj_matrix=to_dev(fr.proj, device))
    with torch.no_grad():
        before = scene(*args, **kw)              # fills the caches
    target = (before * 0.5 + 0.2).clamp(0, 1)
    opt = torch.optim.Adam([{"params": [scene.W1, scene.b1, scene.W2, scene.b2, scene.W3, scene.b3], "lr": 2e-2},
                            {"params": [scene.positions, scene.log_scales, scene.quats], "lr": 5e-3}], fused=True)
    versions = [p._version for p in scene.parameters()]
    for _ in range(2):
        opt.zero_grad(set_to_none=True)
        (scene(*args, **kw) - target).abs().mean().backward()
        opt.step()
    with torch.no_grad():
        after = scene(*args, **kw)
        fresh = _scene_from(fr, device)
        fresh.render_precision = precision
        fresh.load_state_dict(scene.state_dict())
        from mlp_splatting_amd.tile_ext import TileExt
        fresh_ext = TileExt()
        rd = torch.nn.functional.normalize(args[1], dim=-1).contiguous()
        cand, off = fresh._tile_lists(args[0], rd, fr.thr, kw["view_matrix"], kw["proj_matrix"], None, None, device)
        base = fresh._base_args(args[0], args[1], cand, off, device)
        if precision == "f32":
            expected = fresh_ext.render_tiles_forward_tilecenter(*base, fr.W, fr.H, 8, 8, fr.thr)[0]
        else:
            expected = fresh_ext.render_tiles_rgb_wmma(list(base), fr.W, fr.H, fr.thr, True)[0]
    assert float((after - before).abs().max()) > 1e-3             # the steps did change the image
    assert torch.equal(after, expected)
    if [p._version for p in scene.parameters()] != versions:
        pytest.skip("this torch build advances the version in fused steps; the caches would have seen them anyway")


def test_records_forward_in_render_order_is_the_render(device, oracle_mod):
    """render_tiles_training_records(render_order=True): image and alpha are the bits of the f32 tile-centre render
    (itself bit-exact against the oracle), the record topology is that of the ordinary records forward."""
    from mlp_splatting_amd.tile_ext import TileExt
    fr = Frame("cfg1_5k_160x120", n=1500, hidden=32, width=80, height=48)
    cand, off = fr.oracle_lists(oracle_mod)
    base = [to_dev(a, device) for a in fr.base_numpy(cand, off)]
    x = base + [torch.zeros_like(base[0]), torch.zeros(fr.W * fr.H, device=device)]
    ext = TileExt()
    assert ext.records_forward_matches_render(base[7], base[9], base[10], base[11], base[12], 8)
    rgb, alpha = ext.render_tiles_forward_tilecenter(*base, fr.W, fr.H, 8, 8, fr.thr)
    kept = ext.render_tiles_training_records(x, fr.W, fr.H, 8, fr.thr, 1.5, 2.0, render_order=True)
    plain = ext.render_tiles_training_records(x, fr.W, fr.H, 8, fr.thr, 1.5, 2.0)
    assert kept[2].numel() > 5000
    assert torch.equal(kept[0], rgb) and torch.equal(kept[1], alpha)
    same_lists = torch.equal(kept[7], plain[7])
    assert float((kept[7].diff() == plain[7].diff()).float().mean()) > 0.999
    if same_lists:
        for index in (2, 3, 6):
            assert torch.equal(kept[index], plain[index])
        torch.testing.assert_close(kept[4], plain[4], atol=2e-6, rtol=2e-6)
    # other shapes are refused rather than silently rendered in the other rounding
    fr16 = Frame("cfg1_5k_160x120", n=200, hidden=16, width=32, height=24)
    cand16, off16 = fr16.oracle_lists(oracle_mod)
    base16 = [to_dev(a, device) for a in fr16.base_numpy(cand16, off16)]
    assert not ext.records_forward_matches_render(base16[7], base16[9], base16[10], base16[11], base16[12], 8)
    x16 = base16 + [torch.zeros_like(base16[0]), torch.zeros(fr16.W * fr16.H, device=device)]
    with pytest.raises(RuntimeError):
        ext.render_tiles_training_records(x16, fr16.W, fr16.H, 8, fr16.thr, 1.5, 2.0, render_order=True)


def test_gradients_with_and_without_kept_records_agree(device, oracle_mod, monkeypatch):
    """The autograd forward that keeps its records against the one that renders first and re-traverses the frame
    in the backward: same image bits, gradients equal to the rounding of the two record forwards."""
    fr = Frame("cfg1_5k_160x120", n=600, hidden=32, width=32, height=24)
    args = (to_dev(fr.rays_o, device), to_dev(fr.rays_d, device))
    kw = dict(score_threshold=fr.thr, view_matrix=to_dev(fr.view, device), proj_matrix=to_dev(fr.proj, device))
    torch.manual_seed(4)
    weight = torch.randn(fr.W * fr.H, 3, device=device)
    results = {}
    for keep in ("1", "0"):
        monkeypatch.setenv("MLPSP_AUTOGRAD_KEEP_RECORDS", keep)
        scene = _scene_from(fr, device).train()
        rgb = scene(*args, **kw)
        (rgb * weight).sum().backward()
        results[keep] = (rgb.detach(), {k: getattr(scene, k).grad.clone() for k in PARAMS})
    assert torch.equal(results["1"][0], results["0"][0])
    for k in PARAMS:
        a, b = results["1"][1][k], results["0"][1][k]
        assert float(b.abs().max()) > 0
        assert float((a - b).abs().max()) <= 1e-4 * float(b.abs().max()), k
