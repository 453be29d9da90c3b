"""Host-side behaviour of the scene module that needs no GPU (mirrors the reference's CPU tests:
tests/test_config.py:97-105, tests/test_cuda_renderer.py:38-45, tests/test_camera.py:104-110)."""
import math

import numpy as np
import pytest
import torch

from mlp_splatting_amd import cumodel, synthetic as syn
from mlp_splatting_amd.cumodel import NeuralPrimitiveSceneTileCUDA


def test_public_scene_defaults_match_release_architecture():
    scene = NeuralPrimitiveSceneTileCUDA(num_primitives=2)
    assert scene.hidden_dim == 32 and scene.pe_frequencies == 6
    assert scene.encoder.out_dim == 72
    assert scene.W1.shape == (2, 32, 72) and scene.W2.shape == (2, 32, 32) and scene.W3.shape == (2, 4, 32)
    assert scene.quats.tolist() == [[1, 0, 0, 0]] * 2
    assert torch.allclose(scene.log_scales, torch.full((2, 3), math.log(0.1)))
    assert scene.feat_attr is None and scene.requires_full_image
    assert set(dict(scene.named_buffers())) >= {"stat_sum_w", "stat_max_w", "stat_hits", "stat_contrib_count",
                                                "stat_sum_werr", "alpha_accum", "encoder.freq_bands"}


def test_constructor_constraints():
    with pytest.raises(ValueError, match="hidden_dim <= 32"):
        NeuralPrimitiveSceneTileCUDA(num_primitives=1, hidden_dim=33)
    with pytest.raises(ValueError, match="tile_size in"):
        NeuralPrimitiveSceneTileCUDA(num_primitives=1, tile_size=4)
    with pytest.raises(ValueError, match="feature_slots"):
        NeuralPrimitiveSceneTileCUDA(num_primitives=1, feature_dim_low=8, feature_slots=8)
    with pytest.raises(ValueError, match="pe_sigma"):
        NeuralPrimitiveSceneTileCUDA(num_primitives=1, pe_sigma=0.0)
    s5 = NeuralPrimitiveSceneTileCUDA(num_primitives=3, feature_dim_low=8, feature_slots=5)
    assert s5.feat_attr.shape == (3, 5, 8) and not s5.feat_attr[:, 1:].any()


def test_build_config_names(monkeypatch):
    for var in ("MLPSP_NVCC_MAXRREGCOUNT", "MLPSP_TILE_CANDIDATE_CAPACITY", "MLPSP_TRAINING_BACKEND", "MLPSP_CSR_MAX_HITS"):
        monkeypatch.delenv(var, raising=False)
    key, name, flags = cumodel._tile_ext_build_config()
    assert name == "np_tile_kernels_default_c1536" and "-DMLPSP_MAX_TILE_PRIMS=1536" in flags and key == (name, tuple(flags))
    monkeypatch.setenv("MLPSP_TRAINING_BACKEND", "csr")
    monkeypatch.setenv("MLPSP_CSR_MAX_HITS", "512")
    assert cumodel._tile_ext_build_config()[1] == "np_tile_kernels_csr_h512_c1536"
    monkeypatch.setenv("MLPSP_TILE_CANDIDATE_CAPACITY", "768")
    assert cumodel._tile_ext_build_config()[1] == "np_tile_kernels_csr_h512"
    monkeypatch.setenv("MLPSP_NVCC_MAXRREGCOUNT", "96")
    assert cumodel._tile_ext_build_config()[1] == "np_tile_kernels_csr_h512_rreg96"
    monkeypatch.setenv("MLPSP_TILE_CANDIDATE_CAPACITY", "1000")
    with pytest.raises(ValueError, match="768 or 1536"):
        cumodel._tile_ext_build_config()
    monkeypatch.setenv("MLPSP_TILE_CANDIDATE_CAPACITY", "1536")
    monkeypatch.setenv("MLPSP_CSR_MAX_HITS", "100")
    with pytest.raises(ValueError, match="128, 256 or 512"):
        cumodel._tile_ext_build_config()


def test_tile_order_resolution(monkeypatch):
    scene = NeuralPrimitiveSceneTileCUDA(num_primitives=1)
    monkeypatch.delenv("MLPSP_TILE_ORDER", raising=False)
    assert scene._resolve_tile_order_mode() == "tilecenter"
    monkeypatch.setenv("MLPSP_TILE_ORDER", "per_pixel")
    assert scene._resolve_tile_order_mode() == "per_pixel"
    scene.tile_order_mode_override = "Tile-Center"
    assert scene._resolve_tile_order_mode() == "tilecenter"
    scene.tile_order_mode_override = "globaldepth"
    with pytest.raises(ValueError, match="Unsupported tile order"):
        scene._resolve_tile_order_mode()


def test_forward_preconditions_on_the_host():
    scene = NeuralPrimitiveSceneTileCUDA(num_primitives=1)
    with pytest.raises(ValueError, match="image_size must be set"):
        scene(torch.zeros(1, 3), torch.ones(1, 3))
    scene.set_image_size(2, 2)
    with pytest.raises(AssertionError, match="full-frame rays"):
        scene(torch.zeros(1, 3), torch.ones(1, 3))
    scene.set_image_size(1, 1)
    with pytest.raises(RuntimeError, match="must be moved to a CUDA device"):
        scene(torch.zeros(1, 3), torch.ones(1, 3), view_matrix=torch.eye(4), proj_matrix=torch.eye(4))
    with pytest.raises(RuntimeError, match="feature_dim_low == 0"):
        scene.render_feature_map(torch.zeros(1, 3), torch.ones(1, 3))


@pytest.mark.parametrize("method", ["render_rgb_alpha_no_grad", "render_rgb_t_no_grad"])
def test_unsupported_native_analysis_helpers_fail_closed(method):
    scene = NeuralPrimitiveSceneTileCUDA(num_primitives=1)
    scene.camera_mode = "colmap-native"
    with pytest.raises(NotImplementedError, match="Native camera"):
        getattr(scene, method)(torch.zeros(1, 3), torch.ones(1, 3))


def test_encoding_layout_and_indexed_mlp_agree_with_the_module_encoder():
    enc = cumodel.IntegratedPositionalEncoding(in_dim=6, num_frequencies=6, sigma=0.01)
    x = torch.randn(5, 6)
    att = torch.exp(-0.5 * enc.freq_bands ** 2 * enc.sigma2)
    torch.testing.assert_close(cumodel._encode_x6(x, enc.freq_bands, att), enc(x))
    assert enc.out_dim == 72
    fe = cumodel.FourierFeatureEncoding(in_dim=6, num_frequencies=4)
    assert fe(x).shape == (5, 48) and torch.equal(fe.freq_bands, torch.tensor([1.0, 2.0, 4.0, 8.0]))
    scene = NeuralPrimitiveSceneTileCUDA(num_primitives=3)
    ids = torch.tensor([2, 0, 1, 2, 2])
    rgb, sigma = cumodel._mlp_forward_indexed(enc(x), ids, scene.W1, scene.b1, scene.W2, scene.b2, scene.W3, scene.b3)
    assert rgb.shape == (5, 3) and sigma.shape == (5, 1) and (sigma > 0).all() and ((rgb > 0) & (rgb < 1)).all()


def test_indexed_mlp_matches_the_oracle(oracle_mod):
    sc = syn.make_scene(4, 32, seed=9)
    x6 = np.random.default_rng(2).standard_normal((16, 6)).astype(np.float32) * 0.3
    ids = np.arange(16) % 4
    enc = cumodel._encode_x6(torch.from_numpy(x6), torch.from_numpy(sc.freq), torch.from_numpy(sc.att))
    rgb, sigma = cumodel._mlp_forward_indexed(enc, torch.from_numpy(ids), *map(torch.from_numpy, sc.mlp()))
    o = oracle_mod.mlp(x6, ids, sc.freq, sc.att, *sc.mlp())
    np.testing.assert_allclose(rgb.numpy(), 1 / (1 + np.exp(-o[:, :3])), atol=1e-5)
    np.testing.assert_allclose(sigma.numpy()[:, 0], np.log1p(np.exp(o[:, 3])), atol=1e-5)


def test_extension_can_be_injected_like_the_reference_tests_do(monkeypatch):
    sentinel = object()
    monkeypatch.setattr(cumodel, "_tile_ext", sentinel)
    monkeypatch.setattr(cumodel, "_tile_ext_key", cumodel._tile_ext_build_config()[0])
    assert NeuralPrimitiveSceneTileCUDA._ensure_tile_ext_static() is sentinel


def test_synthetic_scene_is_seeded_and_geometry_does_not_depend_on_the_mlp_width():
    a = syn.make_scene(100, 8, seed=0)
    b = syn.make_scene(100, 32, seed=0)
    c = syn.make_scene(100, 8, seed=1)
    np.testing.assert_array_equal(a.positions, b.positions)
    np.testing.assert_array_equal(a.quats, b.quats)
    assert not np.array_equal(a.positions, c.positions)
    np.testing.assert_allclose(np.linalg.norm(a.quats, axis=1), 1, atol=1e-6)
    assert abs(a.b3[:, 3].std() - 1) < 0.2 and abs(a.W1.std() - 0.1) < 0.01
    np.testing.assert_allclose(a.freq, [math.pi * 2 ** k for k in range(6)], rtol=1e-6)
    np.testing.assert_allclose(a.att, np.exp(-0.5 * a.freq.astype(np.float64) ** 2 * 1e-4), rtol=1e-6)


def test_camera_helpers_closed_forms():
    c2w = syn.look_at((1.0, -0.5, 2.0), (0.0, 0.2, 0.0))
    R = c2w[:, :3].astype(np.float64)
    np.testing.assert_allclose(R.T @ R, np.eye(3), atol=1e-6)
    assert abs(np.linalg.det(R) - 1) < 1e-6
    V = syn.view_matrix(c2w)
    full = np.eye(4); full[:3] = c2w
    np.testing.assert_allclose(V.astype(np.float64) @ full, np.eye(4), atol=1e-6)   # inverse of a rigid transform
    P = syn.projection_matrix(600.0, 1200, 680)
    # P00*W/2 = P11*H/2 = focal, so the culling's focal equals the camera's (scannet/eval_rgb_psnr.py:68-87)
    assert abs(P[0, 0] * 600 - 600) < 1e-3 and abs(P[1, 1] * 340 - 600) < 1e-3 and P[3, 2] == 1
    ro, rd = syn.pinhole_rays(8, 6, 10.0, c2w)
    centre = rd[3 * 8 + 4]      # pixel (4, 3) = (W/2, H/2): straight ahead
    np.testing.assert_allclose(centre, c2w[:, 2], atol=1e-6)
    np.testing.assert_allclose(ro[0], c2w[:, 3])
    # a point on a pixel's ray projects back onto that pixel
    pix = 5 * 8 + 2
    pt = ro[pix] + 3.0 * rd[pix]
    pv = V @ np.append(pt, 1.0)
    P8 = syn.projection_matrix(10.0, 8, 6)
    clip = P8 @ pv
    assert abs((clip[0] / clip[3] + 1) * 0.5 * 8 - 2) < 1e-4 and abs((clip[1] / clip[3] + 1) * 0.5 * 6 - 5) < 1e-4


def test_mosaic_frame_quadrants_project_into_their_own_quadrant():
    poses = syn.random_poses(4, seed=3)
    W, H, f = 64, 48, 40.0
    ro, rd, tv, views = syn.mosaic_frame(W, H, f, poses)
    assert ro.shape == (4 * W * H, 3) and tv.shape == ((2 * W // 8) * (2 * H // 8),) and set(tv.tolist()) == {0, 1, 2, 3}
    P = syn.projection_matrix(f, 2 * W, 2 * H)
    for q, (px, py) in enumerate([(10, 7), (W + 20, 30), (5, H + 11), (W + 40, H + 40)]):
        pix = py * 2 * W + px
        pt = ro[pix] + 2.5 * rd[pix]
        clip = P @ (views[q] @ np.append(pt, 1.0))
        assert abs((clip[0] / clip[3] + 1) * W - px) < 1e-3 and abs((clip[1] / clip[3] + 1) * H - py) < 1e-3
        assert tv[(py // 8) * (2 * W // 8) + px // 8] == q


def test_training_paths_leave_no_derived_tensor_behind():
    """TileExt.uncached(): caches are emptied on entry and exit, nothing is kept inside, and nesting holds."""
    from mlp_splatting_amd.tile_ext import TileExt
    ext = TileExt()

    def fill():
        ext._pack = ext._rec = ext._feat_pack = (("k",), object(), ())

    def empty():
        return all(v is None for v in (ext._pack, ext._rec, ext._feat_pack))

    fill()
    assert ext._caching() and not empty()
    with ext.uncached():
        assert empty() and not ext._caching()
        fill()                                   # whatever a call inside might have stored ...
        with ext.uncached():
            assert empty() and not ext._caching()
        assert not ext._caching()
        fill()
    assert empty() and ext._caching()            # ... is gone afterwards
    fill()
    with pytest.raises(ValueError):
        with ext.uncached():
            raise ValueError("a failing training call")
    assert empty() and ext._caching()
    ext._binned = ("lists", 7, None, None)
    ext.invalidate_caches()
    assert ext._binned == ("lists", 7, None, None)     # keyed on the list tensors, not on parameters


def test_scene_invalidation_reaches_the_extension(monkeypatch):
    from mlp_splatting_amd.tile_ext import TileExt
    ext = TileExt()
    monkeypatch.setattr(cumodel, "_tile_ext", ext)
    scene = NeuralPrimitiveSceneTileCUDA(num_primitives=4, hidden_dim=32)
    scene.__dict__["_mlpsp_cache"] = {"unit_quats": (("key",), object())}
    ext._rec = [(("k",), object(), ())]
    scene.invalidate_render_caches()
    assert "_mlpsp_cache" not in scene.__dict__ and ext._rec is None


def test_derived_tensor_cache_cannot_be_served_to_recycled_memory():
    """A cache entry is keyed on the sources' addresses and versions -- an identity only while that memory stays
    allocated -- so the entry keeps the source tensors: with the first scene's tensor dropped by its owner, a second
    tensor of the same shape cannot land on its address, and a faked collision of the key alone never happens.
    Inference tensors (no version counter) are never cached."""
    from mlp_splatting_amd.tile_ext import TileExt
    ext = TileExt()
    built = []

    def build(tag):
        built.append(tag)
        return tag

    first = torch.zeros(8)
    address = first.data_ptr()
    assert ext._derived("_rec", (first,), (), lambda: build("first")) == "first"
    assert ext._derived("_rec", (first,), (), lambda: build("again")) == "first"        # served from the cache
    del first                                               # the owner lets go; the entry still holds the memory
    assert ext._rec[0][2][0].data_ptr() == address
    second = torch.zeros(8)
    assert second.data_ptr() != address                      # so an equal-shaped newcomer lives elsewhere
    assert ext._derived("_rec", (second,), (), lambda: build("second")) == "second"
    second.add_(1)                                           # an in-place edit is seen through the version counter
    assert ext._derived("_rec", (second,), (), lambda: build("edited")) == "edited"
    with torch.inference_mode():
        frozen = torch.zeros(8)
    assert ext._source_key((frozen,)) is None
    assert ext._derived("_pack", (frozen,), (True,), lambda: build("a")) == "a"
    assert ext._derived("_pack", (frozen,), (True,), lambda: build("b")) == "b" and ext._pack is None
    assert built == ["first", "second", "edited", "a", "b"]
    # the entry of the tensor nobody else holds any more went when the next one was built
    assert all(e[1] != "first" for e in ext._rec)
    # the note about freshly binned lists holds its two tensors for the same reason
    cand, offsets = torch.zeros(4, dtype=torch.int32), torch.zeros(3, dtype=torch.int32)
    ext.note_binned_lists(cand, offsets, 2, 10)
    assert ext._binned[2] is cand and ext._binned[3] is offsets


def test_derived_tensor_cache_keeps_two_scenes_and_drops_the_least_recent(monkeypatch):
    from mlp_splatting_amd.tile_ext import TileExt
    ext = TileExt()
    built = []

    def derived(t, tag):
        return ext._derived("_pack", (t,), (True,), lambda: built.append(tag) or tag)

    a, b, c = torch.zeros(8), torch.zeros(8), torch.zeros(8)
    assert [derived(a, "a"), derived(b, "b"), derived(a, "a2"), derived(b, "b2")] == ["a", "b", "a", "b"]
    assert built == ["a", "b"]                               # two scenes rendered in turn rebuild nothing
    assert derived(c, "c") == "c" and [e[1] for e in ext._pack] == ["c", "b"]      # the least recent one goes
    assert derived(a, "a3") == "a3" and [e[1] for e in ext._pack] == ["a3", "c"]
    monkeypatch.setenv("MLPSP_CACHE_SCENES", "1")
    assert derived(b, "b3") == "b3" and [e[1] for e in ext._pack] == ["b3"]
    ext.invalidate_caches()
    assert ext._pack is None


def test_harness_statistics_closed_forms():
    from mlp_splatting_amd.harness import quality, timing_stats
    st = timing_stats([1.0, 2.0, 3.0, 4.0, 10.0])
    assert st["samples"] == 5 and st["mean_ms"] == 4.0 and st["median_ms"] == 3.0
    assert math.isclose(st["std_ms"], math.sqrt(50.0 / 4.0)) and math.isclose(st["coefficient_of_variation"], st["std_ms"] / 4.0)
    assert math.isclose(st["p95_ms"], 8.8) and st["fps_from_mean"] == 250.0 and math.isclose(st["fps_from_median"], 1000.0 / 3.0)
    assert timing_stats([2.5])["std_ms"] == 0.0
    with pytest.raises(ValueError):
        timing_stats([])
    # a uniform error of 0.1 is 20 dB, of 0.01 is 40 dB; pooled: mse = (0.01 + 0.0001) / 2
    a, b = torch.zeros(4, 5, 3), torch.zeros(2, 2, 3)
    q = quality([a + 0.1, b + 0.01, b], [a, b, b])
    assert math.isclose(q["per_view_psnr_db"][0], 20.0, abs_tol=1e-5) and math.isclose(q["per_view_psnr_db"][1], 40.0, abs_tol=1e-4)
    assert q["per_view_psnr_db"][2] == float("inf") and q["median_psnr_db"] == q["per_view_psnr_db"][1]
    pooled = (60 * 0.01 + 12 * 0.0001) / (60 + 12 + 12)
    assert math.isclose(q["global_psnr_db"], -10.0 * math.log10(pooled), abs_tol=1e-5)
    with pytest.raises(ValueError):
        quality([a], [])


def test_compact_segments_writes_segment_lists_one_after_the_other():
    """ops.compact_segments (plain torch): lists that lie in per-tile segments, with gaps and an empty tile, come out
    as the reference's layout -- ids in tile order and T + 1 offsets."""
    import torch
    from mlp_splatting_amd import ops
    stride = 5
    lists = [[7, 9], [], [1, 2, 3, 4, 5], [11]]
    order = torch.full((len(lists) * stride,), -99, dtype=torch.int32)
    ends = torch.empty(len(lists), dtype=torch.int32)
    for t, ids in enumerate(lists):
        order[t * stride:t * stride + len(ids)] = torch.tensor(ids, dtype=torch.int32)
        ends[t] = t * stride + len(ids)
    offsets = torch.arange(len(lists) + 1, dtype=torch.int32) * stride
    flat, off = ops.compact_segments(order, offsets, ends)
    assert flat.tolist() == [7, 9, 1, 2, 3, 4, 5, 11] and off.tolist() == [0, 2, 2, 7, 8]
    assert flat.dtype == torch.int32 and off.dtype == torch.int32
    none, off0 = ops.compact_segments(order, offsets, offsets[:-1].clone())
    assert none.numel() == 0 and off0.tolist() == [0, 0, 0, 0, 0]
