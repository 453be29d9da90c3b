"""The matrix-core render path (bf16 / fp16 MFMA, f32 accumulate) against the oracle.

Tolerances, on the final image (absolute): 5e-3 with bf16 operands, 5e-4 with fp16 operands, against
BOTH the oracle's emulation of the reference's rounding points (rgb_wmma.cuh:144-213) and the plain f32
oracle.  The hit geometry is the f32 path's, so the work counters must agree exactly with the f32 oracle
except where a pixel's transmittance lands on the 1e-3 floor.
"""
import numpy as np
import pytest
import torch

from conftest import to_dev
from helpers import Frame

pytestmark = pytest.mark.gpu

TOL = {True: 5e-3, False: 5e-4}


def _mfma(fr, device, cand, off, bf16, counters=None):
    from mlp_splatting_amd import ops
    sc = fr.scene
    t = lambda a: to_dev(a, device)
    rec = ops.prepare_primitives(t(sc.positions), t(sc.log_scales), t(sc.quats))
    ro, rd, c, o = t(fr.rays_o), t(fr.rays_d), t(cand), t(off)
    order, _ = ops.sort_tiles(ro, rd, rec, c, o, fr.W, fr.H, 8, 8)
    return ops.render_tilecenter_mfma(ro, rd, rec, order, o, t(sc.freq), t(sc.att), *[t(w) for w in sc.mlp()], fr.W,
                                      fr.H, fr.thr, bf16=bf16, counters=counters)


@pytest.mark.parametrize("bf16", [True, False])
@pytest.mark.parametrize("width,height", [(160, 120), (52, 44)])
def test_matrix_core_render_against_oracle(device, oracle_mod, bf16, width, height):
    fr = Frame("cfg1_5k_160x120", hidden=32, width=width, height=height)
    cand, off = fr.oracle_lists(oracle_mod)
    emu = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims, precision=1 if bf16 else 2)
    f32 = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims)
    counters = torch.zeros(4, dtype=torch.int64, device=device)
    rgb, alpha, nonfinite = _mfma(fr, device, cand, off, bf16, counters)
    assert not nonfinite and f32["alpha"].mean() > 0.5
    got, got_a = rgb.cpu().numpy(), alpha.cpu().numpy()
    tol = TOL[bf16]
    print(f"bf16={bf16}: max|gpu-emu|={np.abs(got - emu['rgb']).max():.2e} max|gpu-f32|={np.abs(got - f32['rgb']).max():.2e}")
    assert np.abs(got - emu["rgb"]).max() <= tol and np.abs(got_a - emu["alpha"]).max() <= tol
    assert np.abs(got - f32["rgb"]).max() <= tol and np.abs(got_a - f32["alpha"]).max() <= tol
    assert np.abs(got - f32["rgb"]).max() > 0            # it is not the f32 kernel in disguise
    c = counters.cpu().numpy()
    assert abs(int(c[3]) - int(emu["stats"][3])) <= 0.002 * emu["stats"][3]
    assert c[1] >= c[2] > 0


@pytest.mark.parametrize("bf16", [True, False])
def test_rays_from_separate_origins_take_the_per_pixel_form_with_the_same_bits(device, oracle_mod, bf16):
    # A tile whose rays share an origin reads centre - origin and its rotated image per list entry; any other tile
    # computes them per pixel.  One pixel per tile moved to another origin sends every tile down the per-pixel form:
    # all the other pixels must come out bit-identical, and the moved ones must still match the oracle.
    fr = Frame("cfg1_5k_160x120", hidden=32, width=88, height=60)          # ragged on both edges
    cand, off = fr.oracle_lists(oracle_mod)
    shared = _mfma(fr, device, cand, off, bf16)
    ys, xs = np.meshgrid(np.arange(fr.H), np.arange(fr.W), indexing="ij")
    moved = ((ys % 8 == 4) & (xs % 8 == 5)).ravel()
    pinhole_o = fr.rays_o.copy()
    fr.rays_o = pinhole_o.copy()
    fr.rays_o[moved] += np.float32([0.02, -0.015, 0.01])
    counters = torch.zeros(4, dtype=torch.int64, device=device)
    mixed = _mfma(fr, device, cand, off, bf16, counters)
    assert not shared[2] and not mixed[2]
    keep = torch.from_numpy(~moved).to(device)
    assert torch.equal(mixed[0][keep], shared[0][keep]) and torch.equal(mixed[1][keep], shared[1][keep])
    assert not torch.equal(mixed[0][~keep], shared[0][~keep])
    emu = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims, precision=1 if bf16 else 2)
    assert np.abs(mixed[0].cpu().numpy() - emu["rgb"]).max() <= TOL[bf16]
    assert np.abs(mixed[1].cpu().numpy() - emu["alpha"]).max() <= TOL[bf16]
    c = counters.cpu().numpy()
    assert abs(int(c[3]) - int(emu["stats"][3])) <= 0.002 * emu["stats"][3]
    # every origin different: no pixel shares anything with its neighbours
    rng = np.random.default_rng(3)
    fr.rays_o = pinhole_o + rng.uniform(-0.01, 0.01, pinhole_o.shape).astype(np.float32)
    loose = _mfma(fr, device, cand, off, bf16)
    emu = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims, precision=1 if bf16 else 2)
    assert not loose[2] and np.abs(loose[0].cpu().numpy() - emu["rgb"]).max() <= TOL[bf16]


@pytest.mark.parametrize("threshold,log_scale,depth,zoom", [(5e-3, -3.0, 1.0, 0.9), (5e-3, -5.5, 20.0, 40.0),
                                                            (0.2, -4.5, 6.0, 10.0), (1e-4, -4.0, 2.0, 2.0)])
def test_hit_sets_equal_the_exact_path_for_near_and_far_primitives(device, oracle_mod, threshold, log_scale, depth,
                                                                   zoom):
    # The reduced path decides hits with fast arithmetic and re-tests, exactly, only what lies within a band around
    # the threshold whose width follows the distance to the primitive (in units of its scales).  With zero weights
    # and a faint density no pixel ever saturates, so the hit counters depend on the hit decisions alone and must
    # equal the exact kernel's to the last hit -- for primitives a few dozen scales away (the first case) and ten
    # thousand (the second: a long lens on small far primitives) alike.
    from mlp_splatting_amd import ops, synthetic as syn
    W, H, n = 320, 240, 6000
    sc = syn.make_scene(n, 32, seed=11, log_scale_mean=log_scale)
    rng = np.random.default_rng(12)
    f = zoom * W
    z = rng.random(n, dtype=np.float32) * np.float32(3.0 * depth) + np.float32(depth)
    sc.positions[:, 2] = z
    sc.positions[:, 0] = (rng.random(n, dtype=np.float32) - np.float32(0.5)) * z * np.float32(W / f)
    sc.positions[:, 1] = (rng.random(n, dtype=np.float32) - np.float32(0.5)) * z * np.float32(H / f)
    for w in (sc.W1, sc.b1, sc.W2, sc.b2, sc.W3):
        w[...] = 0
    sc.b3[:, :3] = 0.3
    sc.b3[:, 3] = -12.0                                                   # softplus ~ 6e-6: transmittance stays ~1
    c2w = syn.look_at((0.0, 0.0, 0.0), (0.0, 0.0, 1.0))
    ro, rd = syn.pinhole_rays(W, H, f, c2w)
    rd = syn.normalize_rays(rd)
    view, proj = syn.view_matrix(c2w), syn.projection_matrix(f, W, H)
    cand, off = oracle_mod.bin_legacy(sc.positions, sc.log_scales, view[None], proj, W, H, 8, threshold)
    assert len(cand) > 20000
    t = lambda a: to_dev(a, device)
    rec = ops.prepare_primitives(t(sc.positions), t(sc.log_scales), t(sc.quats))
    ro_t, rd_t, c, o = t(ro), t(rd), t(cand), t(off)
    order, _ = ops.sort_tiles(ro_t, rd_t, rec, c, o, W, H, 8, 8, cull_threshold=threshold)
    ws = [t(w) for w in sc.mlp()]
    exact_counters = torch.zeros(4, dtype=torch.int64, device=device)
    ops.render_tilecenter_f32(ro_t, rd_t, rec, order, o, t(sc.freq), t(sc.att), *ws, W, H, 8, 8, threshold,
                              counters=exact_counters)
    for bf16 in (True, False):
        counters = torch.zeros(4, dtype=torch.int64, device=device)
        _, alpha, bad = ops.render_tilecenter_mfma(ro_t, rd_t, rec, order, o, t(sc.freq), t(sc.att), *ws, W, H, threshold,
                                                   bf16=bf16, counters=counters)
        assert not bad and float(alpha.max()) < 0.05
        assert int(counters[3]) == int(exact_counters[3]) > 10000


def test_matrix_core_matches_rounded_closed_form(device):
    # zero weights: colour = sigmoid(b3), independent of the operand rounding -> must equal the f32 kernel
    from mlp_splatting_amd.tile_ext import TileExt
    ext = TileExt()
    n = 6
    pos = torch.zeros(n, 3, device=device); pos[:, 2] = torch.arange(1, n + 1, device=device)
    quats = torch.zeros(n, 4, device=device); quats[:, 0] = 1
    b3 = torch.tensor([[0.3, -0.4, 1.1, 0.2]], device=device).repeat(n, 1)
    W, H = 8, 8
    ro = torch.zeros(W * H, 3, device=device)
    rd = torch.nn.functional.normalize(torch.tensor([[0.0, 0.0, 1.0]], device=device).repeat(W * H, 1) +
                                       0.01 * torch.randn(W * H, 3, device=device), dim=-1).contiguous()
    x = [ro, rd, pos, torch.full((n, 3), -1.0, device=device), quats, torch.arange(n, dtype=torch.int32, device=device),
         torch.tensor([0, n], dtype=torch.int32, device=device), torch.ones(6, device=device), torch.ones(6, device=device),
         torch.zeros(n, 32, 72, device=device), torch.zeros(n, 32, device=device), torch.zeros(n, 32, 32, device=device),
         torch.zeros(n, 32, device=device), torch.zeros(n, 4, 32, device=device), b3]
    rgb, alpha = ext.render_tiles_rgb_wmma(x, W, H, 1e-3, True)
    want = ext.render_tiles_forward_tilecenter(*x, W, H, 8, 8, 1e-3)
    torch.testing.assert_close(rgb, want[0], rtol=0, atol=1e-6)
    torch.testing.assert_close(alpha, want[1], rtol=0, atol=1e-6)
    assert float(alpha.mean()) > 0.5


def test_overflow_falls_back_to_f32_for_the_whole_frame(device, oracle_mod):
    # rgb_wmma.cuh:260-272 / tests/test_training_wmma.py:308-339: a weight beyond the fp16 range makes
    # the rounded operand infinite -> flag -> the frame is rendered by the scalar f32 kernel instead
    from mlp_splatting_amd.tile_ext import TileExt
    fr = Frame("cfg1_5k_160x120", n=400, hidden=32, width=32, height=24)
    cand, off = fr.oracle_lists(oracle_mod)
    sc = fr.scene
    sc.W2[cand[0], 3, 5] = 1.0e5           # finite in f32 and bf16, infinite in fp16
    ext = TileExt()
    x = [to_dev(a, device) for a in fr.base_numpy(cand, off)]
    calls0, fb0 = ext.rgb_wmma_safety_stats()
    with pytest.warns(UserWarning, match="scalar FP32 instead"):
        rgb, alpha = ext.render_tiles_rgb_wmma(x, fr.W, fr.H, fr.thr, False)
    want = ext.render_tiles_forward_tilecenter(*x, fr.W, fr.H, 8, 8, fr.thr)
    assert torch.equal(rgb, want[0]) and torch.equal(alpha, want[1])
    assert ext.rgb_wmma_safety_stats() == [calls0 + 1, fb0 + 1]
    rgb_b, _ = ext.render_tiles_rgb_wmma(x, fr.W, fr.H, fr.thr, True)       # bf16 holds 1e5: no fallback
    assert ext.rgb_wmma_safety_stats() == [calls0 + 2, fb0 + 1]
    # non-finite INPUT is an error, not a fallback
    x[9] = x[9].clone()
    x[9][int(cand[0]), 0, 0] = float("nan")
    with pytest.raises(RuntimeError, match="input is nonfinite"):
        ext.render_tiles_rgb_wmma(x, fr.W, fr.H, fr.thr, True)


def test_hit_offsets_beyond_the_sincos_table_range_fall_back_to_f32(device, oracle_mod):
    # the bf16 path takes the position half of the encoding from a table that is exact for up to 500 periods of the
    # highest frequency (2^5 pi: 31 scene units of |dx| + |dy| + |dz|); a primitive 60 units across that the rays
    # pass 40 units off its centre is beyond it -> flag -> the frame comes from the f32 kernel, bit for bit.
    # fp16 operands use the sin/cos instructions and render the same frame themselves.
    from mlp_splatting_amd.tile_ext import TileExt
    fr = Frame("cfg1_5k_160x120", n=64, hidden=32, width=32, height=24)
    sc = fr.scene
    ahead = fr.rays_d[(fr.H // 2) * fr.W + fr.W // 2]
    side = np.cross(ahead, [0.0, 1.0, 0.0])
    sc.positions[0] = fr.rays_o[0] + 10.0 * ahead + 40.0 * side / np.linalg.norm(side)
    sc.log_scales[0] = np.log(60.0)
    cand, off = fr.oracle_lists(oracle_mod)
    assert (cand == 0).sum() == (fr.W // 8) * (fr.H // 8)          # the large primitive is on every tile's list
    ext = TileExt()
    x = [to_dev(a, device) for a in fr.base_numpy(cand, off)]
    calls0, fb0 = ext.rgb_wmma_safety_stats()
    with pytest.warns(UserWarning, match="scalar FP32 instead"):
        rgb, alpha = ext.render_tiles_rgb_wmma(x, fr.W, fr.H, fr.thr, True)
    want = ext.render_tiles_forward_tilecenter(*x, fr.W, fr.H, 8, 8, fr.thr)
    assert torch.equal(rgb, want[0]) and torch.equal(alpha, want[1])
    assert float(alpha.max()) > 0.0
    assert ext.rgb_wmma_safety_stats() == [calls0 + 1, fb0 + 1]
    rgb_h, alpha_h = ext.render_tiles_rgb_wmma(x, fr.W, fr.H, fr.thr, False)
    assert ext.rgb_wmma_safety_stats() == [calls0 + 2, fb0 + 1]
    assert float((rgb_h - want[0]).abs().max()) <= TOL[False]


def test_packed_weights_are_cached_until_a_tensor_changes(device, oracle_mod):
    from mlp_splatting_amd.tile_ext import TileExt
    fr = Frame("cfg1_5k_160x120", n=300, hidden=32, width=24, height=16)
    cand, off = fr.oracle_lists(oracle_mod)
    ext = TileExt()
    x = [to_dev(a, device) for a in fr.base_numpy(cand, off)]
    a, _ = ext.render_tiles_rgb_wmma(x, fr.W, fr.H, fr.thr, True)
    pack1 = ext._pack
    b, _ = ext.render_tiles_rgb_wmma(x, fr.W, fr.H, fr.thr, True)
    assert ext._pack is pack1 and torch.equal(a, b)
    x[14].add_(0.5)                                          # in-place edit bumps the tensor version
    c, _ = ext.render_tiles_rgb_wmma(x, fr.W, fr.H, fr.thr, True)
    assert ext._pack is not pack1 and not torch.equal(a, c)


def test_scene_module_precision_switch(device, oracle_mod):
    from test_gpu_scene import _call, _scene_from
    fr = Frame("cfg1_5k_160x120", n=1500, hidden=32, width=64, height=48)
    scene = _scene_from(fr, device)
    ref = _call(scene, fr, device)
    scene.render_precision = "bf16"
    fast = _call(scene, fr, device)
    assert 0 < float((fast - ref).abs().max()) <= 5e-3
    scene.render_precision = "int8"
    with pytest.raises(ValueError, match="render_precision"):
        _call(scene, fr, device)


@pytest.mark.parametrize("slots,channels", [(4, 200), (5, 512), (1, 36), (4, 37), (4, 509), (5, 3)])
@pytest.mark.parametrize("bf16", [True, False])
def test_matrix_core_feature_render_against_oracle(device, oracle_mod, bf16, slots, channels):
    # the feature image shares the weights w of the RGB image, so it inherits the same tolerance scaled
    # by the attribute magnitude (|feat_attr| <= ~4 in this scene -> measured against max|feat|)
    from mlp_splatting_amd import ops
    fr = Frame("cfg1_5k_160x120", n=1200, hidden=32, width=56, height=40, feature_dim=channels,
               feature_slots=slots if slots > 1 else 4)
    sc = fr.scene
    fa = sc.feat_attr if slots > 1 else np.ascontiguousarray(sc.feat_attr[:, 0])
    cand, off = fr.oracle_lists(oracle_mod)
    want = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims, feat_attr=fa, beta=1.3, temp=2.2)
    t = lambda a: to_dev(a, device)
    rec = ops.prepare_primitives(t(sc.positions), t(sc.log_scales), t(sc.quats))
    ro, rd, c, o = t(fr.rays_o), t(fr.rays_d), t(cand), t(off)
    order, _ = ops.sort_tiles(ro, rd, rec, c, o, fr.W, fr.H, 8, 8, cull_threshold=fr.thr)
    ws = [t(w) for w in sc.mlp()]
    rgb, alpha, feat, nonfinite = ops.render_tilecenter_mfma_feat(ro, rd, rec, order, o, t(sc.freq), t(sc.att), *ws,
                                                                  t(fa), 1.3, 2.2, fr.W, fr.H, fr.thr, bf16=bf16)
    rgb0, alpha0, _ = ops.render_tilecenter_mfma(ro, rd, rec, order, o, t(sc.freq), t(sc.att), *ws, fr.W, fr.H, fr.thr,
                                                 bf16=bf16)
    assert not nonfinite
    assert torch.equal(rgb, rgb0) and torch.equal(alpha, alpha0)         # every channel chunk walks the same hits
    scale = float(np.abs(want["feat"]).max())
    err = float(np.abs(feat.cpu().numpy() - want["feat"]).max())
    print(f"bf16={bf16} slots={slots} C={channels}: max|feat err|={err:.2e} of max|feat|={scale:.2e}")
    assert scale > 1e-2 and 0 < err <= TOL[bf16] * max(1.0, scale)
    assert np.abs(rgb.cpu().numpy() - want["rgb"]).max() <= TOL[bf16]


@pytest.mark.parametrize("channels", [260, 37])
def test_matrix_core_feature_image_on_a_ragged_frame(device, oracle_mod, channels):
    # image sides that are no multiples of the tile side; 260 channels: the second slice of 256 holds a single
    # 16-byte piece per pixel; 37: a pixel's channels do not start on a 16-byte boundary.  The product writes the image
    # 16 bytes per lane and has to leave out the pixels beyond the image and the channels beyond the last.
    from mlp_splatting_amd import ops
    fr = Frame("cfg1_5k_160x120", n=1200, hidden=32, width=52, height=44, feature_dim=channels, feature_slots=4)
    sc = fr.scene
    cand, off = fr.oracle_lists(oracle_mod)
    want = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims, feat_attr=sc.feat_attr, beta=1.3, temp=2.2)
    t = lambda a: to_dev(a, device)
    rec = ops.prepare_primitives(t(sc.positions), t(sc.log_scales), t(sc.quats))
    ro, rd, c, o = t(fr.rays_o), t(fr.rays_d), t(cand), t(off)
    order, _ = ops.sort_tiles(ro, rd, rec, c, o, fr.W, fr.H, 8, 8, cull_threshold=fr.thr)
    ws = [t(w) for w in sc.mlp()]
    rgb, alpha, feat, nonfinite = ops.render_tilecenter_mfma_feat(ro, rd, rec, order, o, t(sc.freq), t(sc.att), *ws,
                                                                  t(sc.feat_attr), 1.3, 2.2, fr.W, fr.H, fr.thr, bf16=True)
    assert not nonfinite and feat.shape == (fr.W * fr.H, channels)
    scale = float(np.abs(want["feat"]).max())
    err = float(np.abs(feat.cpu().numpy() - want["feat"]).max())
    assert scale > 1e-2 and 0 < err <= TOL[True] * max(1.0, scale)


def test_matrix_core_feature_render_with_separate_origins(device, oracle_mod):
    from mlp_splatting_amd import ops
    fr = Frame("cfg1_5k_160x120", n=1200, hidden=32, width=56, height=40, feature_dim=72, feature_slots=4)
    rng = np.random.default_rng(5)
    fr.rays_o = fr.rays_o + rng.uniform(-0.01, 0.01, fr.rays_o.shape).astype(np.float32)
    sc = fr.scene
    cand, off = fr.oracle_lists(oracle_mod)
    want = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims, feat_attr=sc.feat_attr, beta=1.3, temp=2.2)
    t = lambda a: to_dev(a, device)
    rec = ops.prepare_primitives(t(sc.positions), t(sc.log_scales), t(sc.quats))
    ro, rd, c, o = t(fr.rays_o), t(fr.rays_d), t(cand), t(off)
    order, _ = ops.sort_tiles(ro, rd, rec, c, o, fr.W, fr.H, 8, 8, cull_threshold=fr.thr)
    rgb, alpha, feat, nonfinite = ops.render_tilecenter_mfma_feat(ro, rd, rec, order, o, t(sc.freq), t(sc.att),
                                                                  *[t(w) for w in sc.mlp()], t(sc.feat_attr), 1.3, 2.2,
                                                                  fr.W, fr.H, fr.thr, bf16=True)
    assert not nonfinite
    scale = float(np.abs(want["feat"]).max())
    assert scale > 1e-2 and np.abs(feat.cpu().numpy() - want["feat"]).max() <= TOL[True] * max(1.0, scale)
    assert np.abs(rgb.cpu().numpy() - want["rgb"]).max() <= TOL[True]


@pytest.mark.parametrize("bf16", [True, False])
@pytest.mark.parametrize("slots", [0, 4, 5])
def test_repeated_launches_give_the_same_bits(device, oracle_mod, bf16, slots):
    # Every value the kernel reads is either loaded and waited for or computed: nothing depends on timing.  (The walk
    # keeps a scalar load in flight across a whole step; a register of it read too early shows as run-to-run noise.)
    from mlp_splatting_amd import ops
    fr = Frame("cfg2_50k_640x480", n=20000, hidden=32, width=320, height=240, feature_dim=40 if slots else 0,
               feature_slots=max(slots, 4))
    sc = fr.scene
    cand, off = fr.oracle_lists(oracle_mod)
    t = lambda a: to_dev(a, device)
    rec = ops.prepare_primitives(t(sc.positions), t(sc.log_scales), t(sc.quats))
    ro, rd, c, o = t(fr.rays_o), t(fr.rays_d), t(cand), t(off)
    order, _ = ops.sort_tiles(ro, rd, rec, c, o, fr.W, fr.H, 8, 8, cull_threshold=fr.thr)
    ws = [t(w) for w in sc.mlp()]
    fa = t(sc.feat_attr) if slots else None

    def once():
        if not slots:
            return ops.render_tilecenter_mfma(ro, rd, rec, order, o, t(sc.freq), t(sc.att), *ws, fr.W, fr.H, fr.thr,
                                              bf16=bf16)[:2]
        return ops.render_tilecenter_mfma_feat(ro, rd, rec, order, o, t(sc.freq), t(sc.att), *ws, fa, 1.3, 2.2, fr.W,
                                               fr.H, fr.thr, bf16=bf16)[:3]
    first = once()
    assert float(first[1].mean()) > 0.2
    for _ in range(4):
        again = once()
        assert all(torch.equal(a, b) for a, b in zip(first, again))


def test_scene_module_feature_precision_switch(device, oracle_mod):
    from test_gpu_scene import _call, _scene_from
    fr = Frame("cfg1_5k_160x120", n=800, width=40, height=24, hidden=32, feature_dim=64)
    scene = _scene_from(fr, device, feature=True)
    rgb, feat = _call(scene, fr, device, return_feature=True)
    scene.render_precision = "bf16"
    rgb_b, feat_b = _call(scene, fr, device, return_feature=True)
    assert torch.equal(rgb_b, _call(scene, fr, device))
    assert 0 < float((rgb_b - rgb).abs().max()) <= 5e-3
    assert 0 < float((feat_b - feat).abs().max()) <= 5e-3 * max(1.0, float(feat.abs().max()))


def test_feature_attributes_beyond_fp16_fall_back_to_the_exact_kernel(device, oracle_mod):
    from mlp_splatting_amd.tile_ext import TileExt
    fr = Frame("cfg1_5k_160x120", n=400, hidden=32, width=32, height=24, feature_dim=40)
    cand, off = fr.oracle_lists(oracle_mod)
    x = [to_dev(a, device) for a in fr.base_numpy(cand, off)]
    fa = to_dev(fr.scene.feat_attr, device).clone()
    ext = TileExt()
    rgb, alpha, feat = ext.render_tiles_rgb_wmma_with_feat(x, fa, 1.0, 4.0, fr.W, fr.H, fr.thr, True)
    exact = ext.render_tiles_forward_tilecenter_with_feat(*x, fa, 1.0, 4.0, fr.W, fr.H, 8, 8, fr.thr)
    assert 0 < float((feat - exact[2]).abs().max()) <= 5e-3 * max(1.0, float(exact[2].abs().max()))
    fa[int(cand[0]), 2, 7] = 1.0e5                      # finite in f32, infinite in fp16
    calls0, fb0 = ext.rgb_wmma_safety_stats()
    with pytest.warns(UserWarning, match="overflow fp16"):
        out = ext.render_tiles_rgb_wmma_with_feat(x, fa, 1.0, 4.0, fr.W, fr.H, fr.thr, True)
    exact = ext.render_tiles_forward_tilecenter_with_feat(*x, fa, 1.0, 4.0, fr.W, fr.H, 8, 8, fr.thr)
    assert all(torch.equal(a, b) for a, b in zip(out, exact))
    assert ext.rgb_wmma_safety_stats() == [calls0 + 1, fb0 + 1]
