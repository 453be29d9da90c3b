"""The scene module on the GPU: the call an evaluator makes (scannet/eval_rgb_psnr.py:443-493,
tools/benchmark_inference.py:121-149) against the oracle, plus the no-grad helpers."""
import numpy as np
import pytest
import torch

from conftest import to_dev
from helpers import Frame, bits

pytestmark = pytest.mark.gpu


def _scene_from(fr, device, feature=False, tile=8):
    from mlp_splatting_amd.cumodel import NeuralPrimitiveSceneTileCUDA
    sc = fr.scene
    C = sc.feat_attr.shape[2] if (feature and sc.feat_attr is not None) else 0
    scene = NeuralPrimitiveSceneTileCUDA(num_primitives=sc.n, hidden_dim=sc.hidden, tile_size=tile, feature_dim_low=C)
    state = {"positions": sc.positions, "log_scales": sc.log_scales, "quats": sc.quats, "W1": sc.W1, "b1": sc.b1,
             "W2": sc.W2, "b2": sc.b2, "W3": sc.W3, "b3": sc.b3}
    if C:
        state["feat_attr"] = sc.feat_attr
    missing, unexpected = scene.load_state_dict({k: torch.from_numpy(v) for k, v in state.items()}, strict=False)
    assert not unexpected and set(missing) <= {"stat_sum_w", "stat_max_w", "stat_hits", "stat_contrib_count",
                                               "stat_sum_werr", "alpha_accum", "encoder.freq_bands"}
    scene = scene.to(device).eval()
    scene.set_image_size(fr.W, fr.H)
    return scene


def _call(scene, fr, device, **kw):
    with torch.inference_mode():
        return scene(to_dev(fr.rays_o, device), to_dev(fr.rays_d, device), score_threshold=fr.thr,
                     view_matrix=to_dev(fr.view, device), proj_matrix=to_dev(fr.proj, device), **kw)


def test_forward_matches_oracle_end_to_end(device, oracle_mod):
    fr = Frame("cfg1_5k_160x120")
    scene = _scene_from(fr, device)
    rgb = _call(scene, fr, device)
    cand, off = fr.oracle_lists(oracle_mod)
    sc = fr.scene
    # The module normalises quaternions and ray directions itself, with torch on the device
    # (scannet/cumodel.py:1088, 1114); the oracle is fed the very same normalised values.
    q = torch.nn.functional.normalize(to_dev(sc.quats, device), dim=-1).cpu().numpy()
    rd = torch.nn.functional.normalize(to_dev(fr.rays_d, device), dim=-1).cpu().numpy()
    # ... and the module's own frequency tables (torch's exp on the device, scannet/cumodel.py:1078-1086)
    freq, att = (t.cpu().numpy() for t in scene._frequency_tables(device))
    np.testing.assert_allclose(freq, sc.freq, rtol=1e-6)
    np.testing.assert_allclose(att, sc.att, rtol=1e-6)
    want = oracle_mod.render_tilecenter(fr.rays_o, rd, sc.positions, sc.log_scales, q, cand, off, freq, att,
                                        *sc.mlp(), *fr.dims)
    assert rgb.shape == (fr.W * fr.H, 3) and not rgb.requires_grad
    assert np.array_equal(bits(rgb.cpu().numpy()), bits(want["rgb"]))
    img = rgb.view(fr.H, fr.W, 3).clamp(0.0, 1.0)
    assert float(img.mean()) > 0.1


def test_background_and_external_lists(device, oracle_mod):
    fr = Frame("cfg1_5k_160x120", n=800, width=40, height=24)
    scene = _scene_from(fr, device)
    cand, off = fr.oracle_lists(oracle_mod)
    plain = _call(scene, fr, device)
    ext_lists = _call(scene, fr, device, culled_prim_indices=to_dev(cand, device).long(), tile_offsets=to_dev(off, device).long())
    assert torch.equal(plain, ext_lists)       # int64 lists are accepted and cast (scannet/cumodel.py:986-987)
    rgb_a = scene.render_rgb_alpha_no_grad(to_dev(fr.rays_o, device), to_dev(fr.rays_d, device), fr.thr,
                                           view_matrix=to_dev(fr.view, device), proj_matrix=to_dev(fr.proj, device))
    bg = _call(scene, fr, device, bg_color=[0.2, 0.4, 0.6])
    want = rgb_a[0] + (1 - rgb_a[1]).clamp(0, 1) * torch.tensor([0.2, 0.4, 0.6], device=device)
    torch.testing.assert_close(bg, want, rtol=0, atol=1e-7)
    with pytest.raises(ValueError, match="provided together"):
        _call(scene, fr, device, culled_prim_indices=to_dev(cand, device))
    with pytest.raises(ValueError, match="tile_offsets length mismatch"):
        _call(scene, fr, device, culled_prim_indices=to_dev(cand, device), tile_offsets=to_dev(off[:-1], device))
    with pytest.raises(RuntimeError, match="feat_attr is not initialized"):
        _call(scene, fr, device, return_feature=True)


def test_feature_path_returns_the_same_rgb_as_the_rgb_only_path(device, oracle_mod):
    # the benchmark's parity block (tools/benchmark_inference.py:287-311)
    fr = Frame("cfg1_5k_160x120", n=800, width=40, height=24, feature_dim=64)
    scene = _scene_from(fr, device, feature=True)
    rgb = _call(scene, fr, device)
    rgb_f, feat = _call(scene, fr, device, return_feature=True)
    assert torch.equal(rgb, rgb_f) and feat.shape == (fr.W * fr.H, 64)
    cand, off = fr.oracle_lists(oracle_mod)
    sc = fr.scene
    want = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims, feat_attr=sc.feat_attr)
    np.testing.assert_allclose(feat.cpu().numpy(), want["feat"], atol=1e-6)
    torch.testing.assert_close(scene.render_feature_map(to_dev(fr.rays_o, device), to_dev(fr.rays_d, device), fr.thr,
                                                        view_matrix=to_dev(fr.view, device),
                                                        proj_matrix=to_dev(fr.proj, device)), feat, rtol=0, atol=0)


def test_per_pixel_mode_and_tile16(device, oracle_mod):
    fr = Frame("cfg1_5k_160x120", n=800, width=48, height=32)
    scene = _scene_from(fr, device)
    scene.tile_order_mode_override = "per_pixel"
    rgb_pp = _call(scene, fr, device)
    cand, off = fr.oracle_lists(oracle_mod)
    want = oracle_mod.render_per_pixel(*fr.base_numpy(cand, off), *fr.dims)
    np.testing.assert_allclose(rgb_pp.cpu().numpy(), want["rgb"], atol=1e-6)
    fr16 = Frame("cfg1_5k_160x120", n=800, width=48, height=32, tile=16)
    scene16 = _scene_from(fr16, device, tile=16)
    rgb16 = _call(scene16, fr16, device)
    c16, o16 = fr16.oracle_lists(oracle_mod)
    want16 = oracle_mod.render_tilecenter(*fr16.base_numpy(c16, o16), *fr16.dims)
    np.testing.assert_allclose(rgb16.cpu().numpy(), want16["rgb"], atol=1e-6)


def test_public_no_grad_helpers_return_finite_detached_outputs(device):
    # tests/test_cuda_renderer.py:48-89
    from mlp_splatting_amd.cumodel import NeuralPrimitiveSceneTileCUDA
    scene = NeuralPrimitiveSceneTileCUDA(num_primitives=1).to(device)
    scene.set_image_size(1, 1)
    scene.tile_order_mode_override = "tilecenter"
    with torch.no_grad():
        scene.positions.zero_()
        scene.positions[:, 2] = 1.0
        scene.log_scales.fill_(-2.0)
    rays_o = torch.zeros((1, 3), device=device)
    rays_d = torch.tensor([[0.0, 0.0, 1.0]], device=device)
    view, projection = torch.eye(4, device=device), torch.eye(4, device=device)
    rgb, alpha = scene.render_rgb_alpha_no_grad(rays_o, rays_d, view_matrix=view, proj_matrix=projection)
    rgb_d, depth, alpha_d = scene.render_rgb_t_no_grad(rays_o, rays_d, view_matrix=view, proj_matrix=projection)
    for out in (rgb, alpha, rgb_d, depth, alpha_d):
        assert out.device == device and torch.isfinite(out).all() and not out.requires_grad
    assert abs(float(depth) - 1.0) < 1e-6 and float(alpha) > 0
    out = scene(rays_o, rays_d, view_matrix=view, proj_matrix=projection)
    assert out.shape == (1, 3)


def test_native_camera_mode_uses_ray_cone_lists(device, oracle_mod):
    # tests/test_camera_cuda.py:34-41: conservative culling leaves the image unchanged
    fr = Frame("cfg1_5k_160x120", n=600, width=40, height=24)
    scene = _scene_from(fr, device)
    scene.camera_mode = "colmap-native"
    rgb_native = _call(scene, fr, device)
    T = (fr.W // 8) * (fr.H // 8)
    every = torch.arange(600, dtype=torch.int32, device=device).repeat(T)
    offs = torch.arange(T + 1, dtype=torch.int32, device=device) * 600
    scene.camera_mode = "legacy-centered"
    rgb_all = _call(scene, fr, device, culled_prim_indices=every, tile_offsets=offs)
    torch.testing.assert_close(rgb_native, rgb_all, rtol=0, atol=1e-6)
    scene.camera_mode = "colmap-native"
    with pytest.raises(ValueError, match="derived from the actual rays"):
        _call(scene, fr, device, culled_prim_indices=every, tile_offsets=offs)


def test_lists_from_the_own_binning_skip_device_validation_but_keep_the_capacity_check(device, oracle_mod, monkeypatch):
    from mlp_splatting_amd import cumodel, ops
    from mlp_splatting_amd.tile_ext import TileExt
    fr = Frame("cfg1_5k_160x120", n=1500, hidden=32, width=64, height=48)
    scene = _scene_from(fr, device)
    ref = _call(scene, fr, device)
    calls = []
    real = ops.validate_tile_lists
    monkeypatch.setattr(ops, "validate_tile_lists", lambda *a, **k: (calls.append(a[-1]), real(*a, **k))[1])
    for precision in ("f32", "bf16"):
        scene.render_precision = precision
        out = _call(scene, fr, device)
        assert precision == "bf16" or torch.equal(out, ref)
    assert calls == []                                   # no device pass for lists the binning just wrote
    scene.render_precision = "f32"
    # the same lists handed in by the caller are validated on the device, as the reference does
    cand, off = fr.oracle_lists(oracle_mod)
    ext_lists = dict(culled_prim_indices=to_dev(cand, device), tile_offsets=to_dev(off, device))
    assert torch.equal(_call(scene, fr, device, **ext_lists), ref) and len(calls) == 1
    # ... and a list edited after the binning noted it is validated again (and rejected)
    ext = cumodel.NeuralPrimitiveSceneTileCUDA._ensure_tile_ext_static()
    c, o, longest = ops.bin_legacy(to_dev(fr.scene.positions, device), to_dev(fr.scene.log_scales, device),
                                   torch.from_numpy(fr.view[None]), torch.from_numpy(fr.proj), fr.W, fr.H, 8, fr.thr,
                                   with_longest=True)
    assert longest == int(np.diff(off).max())
    ext.note_binned_lists(c, o, longest, fr.scene.n)
    c[0] = fr.scene.n + 5
    with pytest.raises(RuntimeError, match="candidate primitive IDs must be in"):
        _call(scene, fr, device, culled_prim_indices=c, tile_offsets=o)
    # the capacity check needs no device pass: it uses the longest list the binning reported
    monkeypatch.setattr(cumodel, "_tile_ext", TileExt(max_tile_prims=longest - 1))
    with pytest.raises(RuntimeError, match=f"capacity {longest - 1} exceeded \\(maximum observed tile length {longest}\\)"):
        _call(scene, fr, device)
    monkeypatch.setattr(cumodel, "_tile_ext", TileExt(max_tile_prims=longest))
    assert torch.equal(_call(scene, fr, device), ref)


def test_cached_scene_derivatives_follow_in_place_parameter_updates(device, oracle_mod):
    # unit quaternions, frequency tables, geometry records and packed weights are cached per tensor
    # version: an optimiser-style in-place update must show in the very next frame
    fr = Frame("cfg1_5k_160x120", n=1200, hidden=32, width=48, height=32)
    for precision in ("f32", "bf16"):
        scene = _scene_from(fr, device)
        scene.render_precision = precision
        a = _call(scene, fr, device)
        assert torch.equal(_call(scene, fr, device), a)
        with torch.no_grad():
            scene.log_scales.add_(0.2)
            scene.quats.mul_(torch.tensor([1.0, -1.0, 1.0, 1.0], device=device))
            scene.b3.add_(0.3)
        b = _call(scene, fr, device)
        fresh = _scene_from(fr, device)
        fresh.render_precision = precision
        fresh.load_state_dict(scene.state_dict())
        assert not torch.equal(a, b) and torch.equal(_call(fresh, fr, device), b)
        scene.encoder.set_runtime_frequency_weights(torch.tensor([1.0, 0.9, 0.8, 0.7, 0.6, 0.5]))
        c = _call(scene, fr, device)
        assert not torch.equal(c, b)


def test_statistics_collection_through_the_scene_module(device, oracle_mod):
    # scannet/cumodel.py:1196-1383: render_rgb_alpha_no_grad(collect_w_stats=True, gt_rgb=...) accumulates
    # into the module's five statistic buffers; reset_w_stats() clears them
    fr = Frame("cfg1_5k_160x120", n=1500, hidden=32, width=64, height=48)
    scene = _scene_from(fr, device)
    gt = np.random.default_rng(9).random((fr.W * fr.H, 3), dtype=np.float32)
    kw = dict(view_matrix=to_dev(fr.view, device), proj_matrix=to_dev(fr.proj, device))
    ro, rd = to_dev(fr.rays_o, device), to_dev(fr.rays_d, device)
    rgb0, alpha0 = scene.render_rgb_alpha_no_grad(ro, rd, fr.thr, **kw)
    assert float(scene.stat_sum_w.sum()) == 0.0
    with pytest.raises(ValueError, match="requires gt_rgb"):
        scene.render_rgb_alpha_no_grad(ro, rd, fr.thr, collect_w_stats=True, **kw)
    rgb, alpha = scene.render_rgb_alpha_no_grad(ro, rd, fr.thr, collect_w_stats=True, gt_rgb=to_dev(gt, device), **kw)
    cand, off = fr.oracle_lists(oracle_mod)
    q = torch.nn.functional.normalize(to_dev(fr.scene.quats, device), dim=-1).cpu().numpy()
    rdn = torch.nn.functional.normalize(rd, dim=-1).cpu().numpy()
    freq, att = (t.cpu().numpy() for t in scene._frequency_tables(device))
    sc = fr.scene
    want = oracle_mod.render_stats(fr.rays_o, rdn, sc.positions, sc.log_scales, q, cand, off, freq, att, *sc.mlp(),
                                   *fr.dims, gt)
    assert np.array_equal(bits(rgb.cpu().numpy()), bits(want["rgb"]))
    assert np.array_equal(scene.stat_hits.cpu().numpy(), want["hits"])
    assert np.array_equal(scene.stat_contrib_count.cpu().numpy(), want["contrib"])
    np.testing.assert_allclose(scene.stat_sum_w.cpu().numpy(), want["sum_w"], rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(scene.stat_sum_werr.cpu().numpy(), want["sum_werr"], rtol=1e-5, atol=1e-7)
    assert np.array_equal(scene.stat_max_w.cpu().numpy(), want["max_w"].astype(np.float32))
    # the depth-ordered image differs from the t*-ordered one only where the two orders differ
    assert float((rgb - rgb0).abs().max()) < 0.5
    scene.reset_w_stats()
    assert int(scene.stat_hits.sum()) == 0 and float(scene.stat_sum_werr.sum()) == 0.0


def test_queued_feature_frames_equal_step_by_step_frames(device, oracle_mod, monkeypatch):
    # the matrix-core frame with its feature image, queued without a mid-frame read-back, is the same frame
    from mlp_splatting_amd import cumodel
    from mlp_splatting_amd.tile_ext import TileExt
    fr = Frame("cfg1_5k_160x120", n=1500, hidden=32, width=64, height=48, feature_dim=48)
    monkeypatch.setattr(cumodel, "_tile_ext", TileExt())
    scene = _scene_from(fr, device, feature=True)
    scene.render_precision = "bf16"
    scene.queued_frames = False
    ref_rgb, ref_feat = _call(scene, fr, device, return_feature=True)
    scene.queued_frames = True
    ext = cumodel._tile_ext
    assert ext._queue_capacity > 0                       # seeded by the step-by-step frame
    calls = []
    real = ext.render_frame_queued
    monkeypatch.setattr(ext, "render_frame_queued", lambda *a, **k: (calls.append(k.get("feat") is not None), real(*a, **k))[1])
    rgb, feat = _call(scene, fr, device, return_feature=True)
    assert calls == [True] and torch.equal(rgb, ref_rgb) and torch.equal(feat, ref_feat)
    assert float(feat.abs().max()) > 1e-2
    # a candidate-buffer estimate that is too small: repeated step by step, same images (lists one after the other:
    # lists in segments, the default, need no estimate)
    monkeypatch.setenv("MLPSP_FRAME_SEGMENTS", "0")
    ext._queue_capacity = 16
    rgb, feat = _call(scene, fr, device, return_feature=True)
    assert torch.equal(rgb, ref_rgb) and torch.equal(feat, ref_feat) and ext._queue_capacity > 1000
    # the exact path is not queued
    scene.render_precision = "f32"
    calls.clear()
    exact = _call(scene, fr, device, return_feature=True)
    assert calls == [] and float((exact[1] - ref_feat).abs().max()) < 5e-2


def test_queued_frames_equal_step_by_step_frames(device, oracle_mod, monkeypatch):
    # the frame queued without a mid-frame read-back (TileExt.render_frame_queued) is the same frame
    from mlp_splatting_amd import cumodel
    from mlp_splatting_amd.tile_ext import TileExt
    fr = Frame("cfg1_5k_160x120", n=1500, hidden=32, width=64, height=48)
    monkeypatch.setenv("MLPSP_FRAME_SEGMENTS", "0")
    for precision in ("f32", "bf16"):
        monkeypatch.setattr(cumodel, "_tile_ext", TileExt())
        scene = _scene_from(fr, device)
        scene.render_precision = precision
        scene.queued_frames = False
        ref = _call(scene, fr, device)
        scene.queued_frames = True
        ext = cumodel._tile_ext
        ext._queue_capacity = 0
        first = _call(scene, fr, device)                 # seeds the candidate-buffer estimate, step by step
        assert ext._queue_capacity > 0 and torch.equal(first, ref)
        calls = []
        real = ext.render_frame_queued
        monkeypatch.setattr(ext, "render_frame_queued", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
        assert torch.equal(_call(scene, fr, device), ref) and calls == [1]
        # an estimate that is too small: the lists were left empty on the device, the frame is repeated
        # step by step and the estimate grows (lists in segments, which RGB frames on the matrix cores take, need
        # no estimate: switched off for this test)
        ext._queue_capacity = 16
        assert torch.equal(_call(scene, fr, device), ref) and ext._queue_capacity > 1000
        assert torch.equal(_call(scene, fr, device), ref)
        # a view matrix edited in place is a new view (the host copy is keyed by the tensor's version)
        view = to_dev(fr.view, device)
        kw = dict(score_threshold=fr.thr, proj_matrix=to_dev(fr.proj, device))
        ro, rd = to_dev(fr.rays_o, device), to_dev(fr.rays_d, device)
        with torch.no_grad():      # (in grad mode a scene whose parameters require grad renders differentiably, in f32)
            a = scene(ro, rd, view_matrix=view, **kw)
            view[0, 3] += 0.5
            b = scene(ro, rd, view_matrix=view, **kw)
            scene.queued_frames = False
            assert torch.equal(a, ref) and torch.equal(scene(ro, rd, view_matrix=view, **kw), b) and not torch.equal(a, b)
    # the capacity error comes out of the queued path too
    monkeypatch.setattr(cumodel, "_tile_ext", TileExt())
    scene = _scene_from(fr, device)
    _call(scene, fr, device)
    cand, off = fr.oracle_lists(oracle_mod)
    longest = int(np.diff(off).max())
    cumodel._tile_ext.max_tile_prims = longest - 1
    with pytest.raises(RuntimeError, match=f"capacity {longest - 1} exceeded \\(maximum observed tile length {longest}\\)"):
        _call(scene, fr, device)


def test_queued_rgb_frames_take_their_lists_in_segments(device, oracle_mod, monkeypatch):
    # An RGB frame on the matrix cores is queued with every tile's list in a segment of its own: no candidate-buffer
    # estimate, so the very first frame is queued too; the same image as the step-by-step frame; a tile beyond the
    # capacity raises the reference's error with the length observed; MLPSP_FRAME_SEGMENTS=0 takes the other lists.
    from mlp_splatting_amd import cumodel, ops
    from mlp_splatting_amd.tile_ext import TileExt
    fr = Frame("cfg1_5k_160x120", n=1500, hidden=32, width=64, height=48)
    monkeypatch.setattr(cumodel, "_tile_ext", TileExt())
    scene = _scene_from(fr, device)
    scene.render_precision = "bf16"
    scene.queued_frames = False
    ref = _call(scene, fr, device)
    scene.queued_frames = True
    ext = cumodel._tile_ext
    ext._queue_capacity = 0
    used = []
    real = ops.bin_segments_async
    monkeypatch.setattr(ops, "bin_segments_async", lambda *a, **k: (used.append(k.get("stride")), real(*a, **k))[1])
    assert torch.equal(_call(scene, fr, device), ref) and used == [ext.max_tile_prims] and ext._queue_capacity == 0
    assert torch.equal(_call(scene, fr, device), ref) and len(used) == 2
    monkeypatch.setenv("MLPSP_FRAME_SEGMENTS", "0")
    assert torch.equal(_call(scene, fr, device), ref) and len(used) == 2
    monkeypatch.delenv("MLPSP_FRAME_SEGMENTS")
    cand, off = fr.oracle_lists(oracle_mod)
    longest = int(np.diff(off).max())
    ext.max_tile_prims = longest - 1
    with pytest.raises(RuntimeError, match=f"capacity {longest - 1} exceeded \\(maximum observed tile length {longest}\\)"):
        _call(scene, fr, device)
    assert used[-1] == longest - 1
    ext.max_tile_prims = longest
    assert torch.equal(_call(scene, fr, device), ref)


def test_a_flag_raised_by_one_queued_frame_does_not_reach_the_next(device, oracle_mod, monkeypatch):
    # Queued frames of a thread share their flag words and skip the clear while the last read-back showed zeros.
    # A frame that raises the non-finite flag (fp16 cannot hold 1e5) is rendered by the f32 kernel; the frame after
    # it, with the weight back in range, must come from the matrix cores again, unflagged.
    import warnings
    from mlp_splatting_amd import cumodel
    from mlp_splatting_amd.tile_ext import TileExt
    fr = Frame("cfg1_5k_160x120", n=1500, hidden=32, width=64, height=48)
    monkeypatch.setattr(cumodel, "_tile_ext", TileExt())
    scene = _scene_from(fr, device)
    scene.render_precision = "fp16"
    ext = cumodel._tile_ext
    _call(scene, fr, device)                             # seeds the candidate-buffer estimate
    clean = _call(scene, fr, device)
    again = _call(scene, fr, device)                     # (this one ran without the clear)
    held = ext._frame_buffers(device)
    assert torch.equal(again, clean) and held["flags_clear"] is True
    cand, _ = fr.oracle_lists(oracle_mod)
    with torch.no_grad():
        kept = scene.W2[int(cand[0]), 3, 5].item()
        scene.W2[int(cand[0]), 3, 5] = 1.0e5
    calls0, fb0 = ext.rgb_wmma_safety_stats()
    with pytest.warns(UserWarning, match="scalar FP32 instead"):
        flagged = _call(scene, fr, device)
    assert held["flags_clear"] is False and ext.rgb_wmma_safety_stats() == [calls0 + 1, fb0 + 1]
    with torch.no_grad():
        scene.W2[int(cand[0]), 3, 5] = kept
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        after = _call(scene, fr, device)
    assert torch.equal(after, clean) and not torch.equal(flagged, clean)
    assert ext.rgb_wmma_safety_stats() == [calls0 + 2, fb0 + 1] and held["flags_clear"] is True


def _camera_frames(fr, device, count):
    """`count` pinhole cameras around the frame's scene: (rays_o, rays_d, view matrix, projection) on the device."""
    from mlp_splatting_amd import synthetic as syn
    frames = []
    for k in range(count):
        a = 0.35 * k
        c2w = syn.look_at((0.3 + 0.4 * np.sin(a), -0.2 + 0.1 * k, -0.5 - 0.3 * np.cos(a)), (0.0, 0.0, 0.4))
        ro, rd = syn.pinhole_rays(fr.W, fr.H, fr.f, c2w)
        frames.append((to_dev(ro, device), to_dev(rd, device), to_dev(syn.view_matrix(c2w), device),
                       to_dev(fr.proj, device)))
    return frames


def _same_images(got, want):
    assert len(got) == len(want)
    for g, w in zip(got, want):
        g, w = (g if isinstance(g, tuple) else (g,)), (w if isinstance(w, tuple) else (w,))
        assert len(g) == len(w) and all(torch.equal(a, b) for a, b in zip(g, w))


@pytest.mark.parametrize("precision,feature_dim", [("bf16", 0), ("fp16", 0), ("bf16", 48)])
def test_frames_in_flight_equal_frames_rendered_one_by_one(device, oracle_mod, monkeypatch, precision, feature_dim):
    # render_frames keeps two (or three) frames queued on streams of its own; every frame is the frame forward() renders
    from mlp_splatting_amd import cumodel
    from mlp_splatting_amd.tile_ext import TileExt
    fr = Frame("cfg1_5k_160x120", n=1500, hidden=32, width=64, height=48, feature_dim=feature_dim)
    monkeypatch.setattr(cumodel, "_tile_ext", TileExt())
    scene = _scene_from(fr, device, feature=bool(feature_dim))
    scene.render_precision = precision
    frames = _camera_frames(fr, device, 7)
    kw = dict(score_threshold=fr.thr, return_feature=bool(feature_dim))
    with torch.inference_mode():
        want = [scene(f[0], f[1], view_matrix=f[2], proj_matrix=f[3], **kw) for f in frames]
    assert not torch.equal(want[0][0] if feature_dim else want[0], want[3][0] if feature_dim else want[3])
    ext = cumodel._tile_ext
    deferred = []
    real = ext.render_frame_queued
    monkeypatch.setattr(ext, "render_frame_queued", lambda *a, **k: (deferred.append(k.get("defer", False)), real(*a, **k))[1])
    for in_flight in (2, 3):
        deferred.clear()
        _same_images(scene.render_frames(frames, fr.thr, return_feature=bool(feature_dim),
                                         frames_in_flight=in_flight), want)
        assert deferred == [True] * 7
    # one frame at a time, or a single frame: plain calls
    deferred.clear()
    _same_images(scene.render_frames(frames[:4], fr.thr, return_feature=bool(feature_dim), frames_in_flight=1), want[:4])
    _same_images(scene.render_frames(frames[:1], fr.thr, return_feature=bool(feature_dim)), want[:1])
    _same_images(scene.render_frames(frames[:2], fr.thr, return_feature=bool(feature_dim)), want[:2])
    assert deferred == [False] * 5 + [True] * 2
    # a frame in flight whose candidate buffer turns out too small is repeated the synchronous way on its stream
    # (with lists in segments, which RGB frames take, there is no such buffer: switched off from here on)
    monkeypatch.setenv("MLPSP_FRAME_SEGMENTS", "0")
    _same_images(scene.render_frames(frames[:3], fr.thr, return_feature=bool(feature_dim)), want[:3])
    calls = []
    real_bin = ext.frame_binning_queued

    def small_third(*a, **k):
        calls.append(1)
        if len(calls) == 3:
            ext._queue_capacity = 16
        return real_bin(*a, **k)
    monkeypatch.setattr(ext, "frame_binning_queued", small_third)
    _same_images(scene.render_frames(frames, fr.thr, return_feature=bool(feature_dim)), want)
    assert ext._queue_capacity > 1000
    monkeypatch.setattr(ext, "frame_binning_queued", real_bin)
    # forward() afterwards, on the caller's stream, is undisturbed
    with torch.inference_mode():
        _same_images([scene(frames[5][0], frames[5][1], view_matrix=frames[5][2], proj_matrix=frames[5][3], **kw)], want[5:6])


def test_frames_in_flight_take_the_f32_fallback_on_their_own_stream(device, oracle_mod, monkeypatch):
    # fp16 cannot hold 1e5: every frame raises the non-finite flag and is rendered again by the f32 kernel, in flight
    # as in forward(); with the weight back in range the frames come from the matrix cores again
    import warnings
    from mlp_splatting_amd import cumodel
    from mlp_splatting_amd.tile_ext import TileExt
    fr = Frame("cfg1_5k_160x120", n=1500, hidden=32, width=64, height=48)
    monkeypatch.setattr(cumodel, "_tile_ext", TileExt())
    scene = _scene_from(fr, device)
    scene.render_precision = "fp16"
    frames = _camera_frames(fr, device, 5)
    clean = scene.render_frames(frames, fr.thr)
    with torch.no_grad():
        kept = scene.W2[:, 3, 5].clone()
        scene.W2[:, 3, 5] = 1.0e5
    ext = cumodel._tile_ext
    calls0, fb0 = ext.rgb_wmma_safety_stats()
    with pytest.warns(UserWarning, match="scalar FP32 instead"):
        with torch.inference_mode():
            want = [scene(f[0], f[1], score_threshold=fr.thr, view_matrix=f[2], proj_matrix=f[3]) for f in frames]
        flagged = scene.render_frames(frames, fr.thr)
    _same_images(flagged, want)
    assert ext.rgb_wmma_safety_stats() == [calls0 + 10, fb0 + 10]
    with torch.no_grad():
        scene.W2[:, 3, 5] = kept
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        _same_images(scene.render_frames(frames, fr.thr), clean)
    assert not torch.equal(flagged[1], clean[1])


def test_harness_renders_times_and_scores_a_view(device, oracle_mod):
    """mlp_splatting_amd.harness: the timed view of tools/benchmark_inference.py:121-149, its statistics, PSNR and
    the RGB parity of the feature render, on a frame whose image the oracle pins."""
    from mlp_splatting_amd import harness
    fr = Frame("cfg1_5k_160x120", n=800, width=40, height=24, feature_dim=64)
    scene = _scene_from(fr, device, feature=True).eval()
    frame = (to_dev(fr.rays_o, device), to_dev(fr.rays_d, device), to_dev(fr.view, device), to_dev(fr.proj, device),
             fr.W, fr.H, fr.thr)
    rgb, wall_ms, device_ms, shape = harness.render_view(scene, *frame)
    assert tuple(rgb.shape) == (fr.H, fr.W, 3) and shape is None and wall_ms > 0 and 0 < device_ms <= wall_ms * 1.5
    cand, off = fr.oracle_lists(oracle_mod)
    sc = fr.scene
    # the oracle is fed the module's own normalised directions, quaternions and frequency tables, as above
    q = torch.nn.functional.normalize(to_dev(sc.quats, device), dim=-1).cpu().numpy()
    rd = torch.nn.functional.normalize(to_dev(fr.rays_d, device), dim=-1).cpu().numpy()
    freq, att = (t.cpu().numpy() for t in scene._frequency_tables(device))
    want = oracle_mod.render_tilecenter(fr.rays_o, rd, sc.positions, sc.log_scales, q, cand, off, freq, att, *sc.mlp(),
                                        *fr.dims)["rgb"].reshape(fr.H, fr.W, 3).clip(0.0, 1.0)
    assert np.array_equal(rgb.cpu().numpy(), want)
    _, _, _, shape = harness.render_view(scene, *frame, return_feature=True)
    assert shape == [fr.W * fr.H, 64]
    assert harness.rgb_parity_with_features(scene, *frame) == 0.0
    q = harness.quality([rgb, rgb], [torch.from_numpy(want).to(device), (rgb + 0.1)])
    assert q["per_view_psnr_db"][0] == float("inf") and abs(q["per_view_psnr_db"][1] - 20.0) < 1e-4
    st = harness.timing_stats([harness.render_view(scene, *frame)[1] for _ in range(5)])
    assert st["samples"] == 5 and st["mean_ms"] > 0 and st["std_ms"] >= 0
