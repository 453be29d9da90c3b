"""Pins the oracle's MLP, compositing, ordering, capacity and feature arithmetic.

References: numpy float64 restatements of the MLP (einsum form, scannet/cumodel.py:193-216) and the
closed forms and cases held by the reference's own tests (tests/test_cuda_renderer.py,
tests/test_candidate_capacity.py, tests/test_training_wmma.py, tests/test_record_feature_512.py).
"""
import math

import numpy as np
import pytest
import torch

from mlp_splatting_amd import synthetic as syn


# ---------------------------------------------------------------------------------------------
# scenes in the style of the reference's _renderer_inputs (tests/test_cuda_renderer.py:111-141):
# n primitives at (0,0,1), unit scale, one pixel, ray along +z, H = F = 1, zero weights
# ---------------------------------------------------------------------------------------------
def stack_scene(n, hidden=1, freqs=1, b3=None, feat=None):
    enc = 12 * freqs
    s = dict(
        rays_o=np.zeros((1, 3), np.float32), rays_d=np.array([[0, 0, 1]], np.float32),
        positions=np.tile(np.array([[0, 0, 1]], np.float32), (n, 1)), log_scales=np.zeros((n, 3), np.float32),
        quats=np.tile(np.array([[1, 0, 0, 0]], np.float32), (n, 1)),
        cand=np.arange(n, dtype=np.int32), offsets=np.array([0, n], np.int32),
        freq=np.ones(freqs, np.float32), att=np.ones(freqs, np.float32),
        W1=np.zeros((n, hidden, enc), np.float32), b1=np.zeros((n, hidden), np.float32),
        W2=np.zeros((n, hidden, hidden), np.float32), b2=np.zeros((n, hidden), np.float32),
        W3=np.zeros((n, 4, hidden), np.float32), b3=np.zeros((n, 4), np.float32))
    if b3 is not None:
        s["b3"][:] = np.asarray(b3, np.float32)
    return s


def base(s):
    return (s["rays_o"], s["rays_d"], s["positions"], s["log_scales"], s["quats"], s["cand"], s["offsets"], s["freq"],
            s["att"], s["W1"], s["b1"], s["W2"], s["b2"], s["W3"], s["b3"])


DIMS1 = (1, 1, 1, 1, 1e-3)


# ---------------------------------------------------------------------------------------------
# MLP
# ---------------------------------------------------------------------------------------------
def _mlp_f64(x6, ids, freq, att, W1, b1, W2, b2, W3, b3):
    phase = x6[:, :, None].astype(np.float64) * freq[None, None, :] * att[None, None, :]
    enc = np.concatenate([np.sin(phase).reshape(len(x6), -1), np.cos(phase).reshape(len(x6), -1)], -1)
    h = np.maximum(np.einsum("mhi,mi->mh", W1[ids].astype(np.float64), enc) + b1[ids], 0)
    h = np.maximum(np.einsum("moh,mh->mo", W2[ids].astype(np.float64), h) + b2[ids], 0)
    return np.einsum("moh,mh->mo", W3[ids].astype(np.float64), h) + b3[ids]


@pytest.mark.parametrize("hidden,freqs", [(32, 6), (16, 6), (5, 3), (1, 1)])
def test_mlp_matches_einsum_restatement(oracle_mod, hidden, freqs):
    sc = syn.make_scene(7, hidden, seed=3, num_frequencies=freqs)
    rng = np.random.default_rng(0)
    x6 = np.concatenate([syn.normalize_rays(rng.standard_normal((64, 3)).astype(np.float32)),
                         (rng.standard_normal((64, 3)) * 0.2).astype(np.float32)], 1)
    ids = rng.integers(0, 7, 64).astype(np.int32)
    got = oracle_mod.mlp(x6, ids, sc.freq, sc.att, *sc.mlp())
    ref = _mlp_f64(x6, ids, sc.freq.astype(np.float64), sc.att.astype(np.float64), *sc.mlp())
    np.testing.assert_allclose(got, ref, atol=3e-5, rtol=0)


def test_mlp_encoding_layout_is_sines_then_cosines(oracle_mod):
    # one-hot W1 rows expose which input feeds which slot: slot c*F+f is sin, slot 6F+c*F+f is cos
    F, H = 6, 32
    freq, att = syn.frequency_bands(F)
    x6 = np.array([[0.3, -0.2, 0.9, 0.05, -0.07, 0.02]], np.float32)
    for c, f in [(0, 0), (2, 5), (4, 3)]:
        for cos_part in (0, 1):
            W1 = np.zeros((1, H, 12 * F), np.float32)
            W1[0, 0, cos_part * 6 * F + c * F + f] = 1.0
            W2 = np.zeros((1, H, H), np.float32); W2[0, 0, 0] = 1.0
            W3 = np.zeros((1, 4, H), np.float32); W3[0, 1, 0] = 1.0
            zb = np.zeros((1, H), np.float32)
            out = oracle_mod.mlp(x6, [0], freq, att, W1, zb, W2, zb, W3, np.zeros((1, 4), np.float32))
            phase = float(x6[0, c]) * float(freq[f]) * float(att[f])
            want = max(math.cos(phase) if cos_part else math.sin(phase), 0.0)
            assert abs(out[0, 1] - want) < 1e-6 and out[0, 0] == 0 and out[0, 2] == 0


@pytest.mark.parametrize("precision,dtype", [(1, torch.bfloat16), (2, torch.float16)])
def test_mixed_precision_mlp_rounding_points(oracle_mod, precision, dtype):
    # rgb_wmma.cuh:144-213: operands rounded, f32 accumulate, bias in f32, hidden re-rounded
    sc = syn.make_scene(5, 32, seed=4)
    rng = np.random.default_rng(1)
    x6 = np.concatenate([syn.normalize_rays(rng.standard_normal((48, 3)).astype(np.float32)),
                         (rng.standard_normal((48, 3)) * 0.1).astype(np.float32)], 1)
    ids = rng.integers(0, 5, 48).astype(np.int32)
    got = oracle_mod.mlp(x6, ids, sc.freq, sc.att, *sc.mlp(), precision=precision)

    def q(a):
        return torch.from_numpy(np.asarray(a, np.float32)).to(dtype).float().numpy().astype(np.float64)

    phase = x6[:, :, None].astype(np.float64) * sc.freq[None, None, :] * sc.att[None, None, :]
    enc = q(np.concatenate([np.sin(phase).reshape(48, -1), np.cos(phase).reshape(48, -1)], -1))
    W1, b1, W2, b2, W3, b3 = sc.mlp()
    h = q(np.maximum(np.einsum("mhi,mi->mh", q(W1)[ids], enc) + b1[ids], 0))
    h = q(np.maximum(np.einsum("moh,mh->mo", q(W2)[ids], h) + b2[ids], 0))
    ref = np.einsum("moh,mh->mo", q(W3)[ids], h) + b3[ids]
    # a hidden value sitting on a rounding boundary may round the other way in f32 vs f64 accumulation
    tol = 2e-3 if precision == 1 else 3e-4
    np.testing.assert_allclose(got, ref, atol=tol, rtol=0)
    full = oracle_mod.mlp(x6, ids, sc.freq, sc.att, *sc.mlp(), precision=0)
    assert np.abs(got - full).max() < (3e-2 if precision == 1 else 4e-3)
    assert np.abs(got - full).max() > 0  # the rounding is really applied


# ---------------------------------------------------------------------------------------------
# compositing and termination
# ---------------------------------------------------------------------------------------------
def test_zero_weight_stack_is_a_geometric_series(oracle_mod):
    # colour = sigmoid(b3[:3]); alpha = 1 - exp(-softplus(b3[3])) (decay = 1 through the centre)
    b3 = [0.3, -0.4, 1.1, 0.2]
    s = stack_scene(40, b3=b3)
    out = oracle_mod.render_tilecenter(*base(s), *DIMS1)
    a = 1 - math.exp(-math.log1p(math.exp(b3[3])))
    k = next(i for i in range(1, 100) if (1 - a) ** i < 1e-3)  # first step that drops below the floor
    assert k < 40
    colour = 1 / (1 + np.exp(-np.array(b3[:3])))
    np.testing.assert_allclose(out["rgb"][0], colour * (1 - (1 - a) ** k), atol=2e-6)
    np.testing.assert_allclose(out["alpha"][0, 0], 1 - (1 - a) ** k, atol=2e-6)
    assert out["stats"][1] == k and out["stats"][3] == k  # the tile stops processing once its pixel is done


def test_opaque_stops_after_first_and_transparent_never_stops(oracle_mod):
    # tests/test_training_wmma.py:194, 283
    out = oracle_mod.render_tilecenter(*base(stack_scene(10, b3=[0, 0, 0, 8.0])), *DIMS1)
    assert out["stats"][3] == 1
    out = oracle_mod.render_tilecenter(*base(stack_scene(10, b3=[0, 0, 0, -20.0])), *DIMS1)
    assert out["stats"][3] == 10


def test_transmittance_boundary_at_exactly_the_floor(oracle_mod):
    # tests/test_training_wmma.py:234-252: alpha = 0.999 gives T ~ 1e-3 after one blend; the pixel
    # stays active iff the f32 value of T is >= 1e-3f.  sigma = -ln(T1) makes exp(-sigma) = T1.
    for target, expect_second in [(np.float32(1e-3), None), (np.float32(1.2e-3), True), (np.float32(0.8e-3), False)]:
        sigma = -math.log(float(target))
        logit = math.log(math.expm1(sigma))  # softplus^-1
        out = oracle_mod.render_tilecenter(*base(stack_scene(2, b3=[0, 0, 0, logit])), *DIMS1)
        hits = int(out["stats"][3])
        t1 = np.float32(1.0) - np.float32(out["alpha"][0, 0]) if hits == 1 else None
        if expect_second is None:
            # on the boundary the decision must agree with the f32 transmittance the oracle itself produced
            if hits == 1:
                assert t1 < np.float32(1e-3)
            else:
                assert hits == 2
        else:
            assert hits == (2 if expect_second else 1)


def test_empty_tile_and_empty_scene(oracle_mod):
    s = stack_scene(0)
    out = oracle_mod.render_tilecenter(*base(s), *DIMS1)
    assert not out["rgb"].any() and not out["alpha"].any()


def test_expected_depth(oracle_mod):
    # identical primitives at depth 1 -> t = 1 wherever something was hit; family 2 key
    s = stack_scene(5, b3=[0, 0, 0, 0.5])
    out = oracle_mod.render_tilecenter(*base(s), *DIMS1, family=2, with_t=True)
    assert abs(out["t"][0, 0] - 1.0) < 1e-6
    s["positions"][:, 2] = [1, 2, 3, 4, 5]
    out = oracle_mod.render_tilecenter(*base(s), *DIMS1, family=2, with_t=True)
    a = 1 - math.exp(-math.log1p(math.exp(0.5)))
    w = np.array([a * (1 - a) ** i for i in range(5)])
    live = np.cumprod(np.concatenate([[1.0], np.full(4, 1 - a)])) >= 1e-3
    w = w * live
    assert abs(out["t"][0, 0] - (w * np.arange(1, 6)).sum() / w.sum()) < 1e-5


# ---------------------------------------------------------------------------------------------
# ordering
# ---------------------------------------------------------------------------------------------
def test_sort_is_ascending_and_stable_with_list_order_ties(oracle_mod):
    # tests/test_training_wmma.py:179-201: coincident primitives, list reversed -> first processed is id 11
    n = 12
    s = stack_scene(n, b3=[0, 0, 0, 8.0])
    s["b3"][:, 0] = np.linspace(-3, 3, n)          # a different red per primitive
    s["cand"] = np.arange(n - 1, -1, -1, dtype=np.int32)
    ids, keys = oracle_mod.sort_tiles(s["rays_o"], s["rays_d"], s["positions"], s["log_scales"], s["quats"], s["cand"],
                                      s["offsets"], 1, 1, 1, 1)
    np.testing.assert_array_equal(ids, s["cand"])   # all keys equal: list order kept
    assert np.all(keys == keys[0])
    out = oracle_mod.render_tilecenter(*base(s), *DIMS1)
    assert abs(out["rgb"][0, 0] / out["alpha"][0, 0] - 1 / (1 + math.exp(-s["b3"][11, 0]))) < 1e-5
    # distinct depths: nearest first whatever the list order; primitives behind the ray go last in list order
    s["positions"][:, 2] = np.array([5, 3, -1, 9, 1, 7, -2, 2, 8, 4, 6, 10], np.float32)
    ids, keys = oracle_mod.sort_tiles(s["rays_o"], s["rays_d"], s["positions"], s["log_scales"], s["quats"], s["cand"],
                                      s["offsets"], 1, 1, 1, 1)
    z = s["positions"][ids, 2]
    front = z > 0
    assert np.all(np.diff(z[front]) > 0) and np.all(front[:10]) and not front[10:].any()
    np.testing.assert_array_equal(ids[10:], [6, 2])  # reversed list visits 6 before 2
    np.testing.assert_array_equal(keys[10:], np.float32(1e30))
    both = np.lexsort((np.arange(n), np.where(s["positions"][s["cand"], 2] > 0, s["positions"][s["cand"], 2], 1e30)))
    np.testing.assert_array_equal(ids, s["cand"][both])


@pytest.mark.parametrize("n", [768, 769, 1024, 1536])
def test_only_the_last_candidate_hits_is_not_truncated(oracle_mod, n):
    # tests/test_candidate_capacity.py:7-19
    s = stack_scene(n, b3=[0.5, 0.5, 0.5, 2.0])
    s["positions"][:-1, 0] = 100.0
    out = oracle_mod.render_tilecenter(*base(s), *DIMS1)
    one = oracle_mod.render_tilecenter(*base(stack_scene(1, b3=[0.5, 0.5, 0.5, 2.0])), *DIMS1)
    assert one["alpha"][0, 0] > 0
    np.testing.assert_array_equal(out["rgb"], one["rgb"])
    np.testing.assert_array_equal(out["alpha"], one["alpha"])


def test_presorted_streams_past_capacity(oracle_mod):
    # tests/test_cuda_renderer.py:374-388: list order, no cap, the only hit is entry 1537
    s = stack_scene(1537, b3=[0.5, 0.5, 0.5, 2.0])
    s["positions"][:-1, 0] = 100.0
    out = oracle_mod.render_tilecenter(*base(s), *DIMS1, family=0, capacity=0)
    one = oracle_mod.render_tilecenter(*base(stack_scene(1, b3=[0.5, 0.5, 0.5, 2.0])), *DIMS1, family=0, capacity=0)
    np.testing.assert_array_equal(out["rgb"], one["rgb"])


# ---------------------------------------------------------------------------------------------
# validation
# ---------------------------------------------------------------------------------------------
def test_validation_status_bits(oracle_mod):
    ok = oracle_mod.validate([0, 1536], np.zeros(1536), 1, 1536, 1)
    assert ok[0] == 0
    over = oracle_mod.validate([0, 1537], np.zeros(1537), 1, 1536, 1)
    assert over[0] == 2 and over[1] == 1537
    assert oracle_mod.validate([0, 1537], np.zeros(1537), 1, 0, 1)[0] == 0          # capacity 0 = no cap
    assert oracle_mod.validate([1, 2], [0, 0], 1, 1536, 2)[0] & 1                     # must start at zero
    assert oracle_mod.validate([0, 1], [0, 0], 1, 1536, 2)[0] & 1                     # must end at the list length
    assert oracle_mod.validate([0, 2, 1, 2], [0, 0], 3, 1536, 2)[0] & 1               # monotone
    assert oracle_mod.validate([0, 2], [-1, 0], 1, 1536, 2)[0] == 4
    assert oracle_mod.validate([0, 2], [0, 2], 1, 1536, 2)[0] == 4
    assert oracle_mod.validate([0, 2], [0, 1], 1, 1536, 2)[0] == 0
    assert oracle_mod.validate([0, 0], [], 1, 1536, 0)[0] == 0                        # N = 0 accepted


# ---------------------------------------------------------------------------------------------
# per-pixel order
# ---------------------------------------------------------------------------------------------
def test_per_pixel_capacity(oracle_mod):
    # tests/test_cuda_renderer.py:250-305: 257 real hits overflow, 256 fit, 386 candidates with 256 hits fit
    assert oracle_mod.render_per_pixel(*base(stack_scene(257)), *DIMS1)["overflow"]
    assert not oracle_mod.render_per_pixel(*base(stack_scene(256)), *DIMS1)["overflow"]
    s = stack_scene(386)
    s["positions"][256:, 0] = 100.0
    assert not oracle_mod.render_per_pixel(*base(s), *DIMS1)["overflow"]


def test_per_pixel_orders_by_each_pixels_own_t(oracle_mod):
    # two opaque primitives, the farther one first in the list: per-pixel order still shows the near one
    s = stack_scene(2, b3=[0, 0, 0, 8.0])
    s["positions"][:, 2] = [3.0, 1.0]
    s["b3"][:, 0] = [-4.0, 4.0]
    out = oracle_mod.render_per_pixel(*base(s), *DIMS1)
    assert abs(out["rgb"][0, 0] / out["alpha"][0, 0] - 1 / (1 + math.exp(-4.0))) < 1e-5
    # the single-pixel tile-centre render agrees (its centre ray IS the pixel ray)
    tc = oracle_mod.render_tilecenter(*base(s), *DIMS1)
    np.testing.assert_array_equal(out["rgb"], tc["rgb"])


def test_per_pixel_equals_tile_centre_on_one_pixel_tiles(oracle_mod):
    # with 1x1 tiles the tile-centre ray is the pixel's own ray, so both orders coincide exactly
    from helpers import Frame
    fr = Frame("cfg1_5k_160x120", n=600, width=16, height=12, tile=1)
    cand, off = fr.oracle_lists(oracle_mod)
    a = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims)
    b = oracle_mod.render_per_pixel(*fr.base_numpy(cand, off), *fr.dims)
    assert a["alpha"].max() > 0.5
    np.testing.assert_array_equal(a["rgb"], b["rgb"])
    np.testing.assert_array_equal(a["alpha"], b["alpha"])


def test_per_pixel_records_are_each_pixels_hits_in_its_own_depth_order(oracle_mod):
    """Pins records_per_pixel by properties that do not restate it: on 1x1 tiles it IS the tile-centre records
    forward; on 8x8 tiles every pixel's ids are a prefix of ALL its hits (brute force through the scalar hit
    function) in ascending own-t order with list-order ties, cut where the transmittance falls below 1e-3; the
    image recomposes from the raw fields and agrees with the per-pixel render (another MLP rounding: 2e-6)."""
    from helpers import Frame
    one = Frame("cfg1_5k_160x120", n=600, hidden=16, width=16, height=12, tile=1)
    cand, off = one.oracle_lists(oracle_mod)
    a = oracle_mod.records(*one.base_numpy(cand, off), *one.dims, max_hits=512, beta=1.3, temp=2.2)
    b = oracle_mod.records_per_pixel(*one.base_numpy(cand, off), *one.dims, beta=1.3, temp=2.2)
    assert a["offsets"][-1] > 300 and not b["overflow"]
    for k in ("rgb", "alpha", "ids", "x6", "raw", "masks", "gates", "offsets"):
        np.testing.assert_array_equal(a[k], b[k], err_msg=k)

    from mlp_splatting_amd import synthetic as syn
    fr = Frame("cfg1_5k_160x120", n=8, hidden=16, width=24, height=16, eye=(0.3, -0.2, -0.9), target=(0.0, 0.0, 0.0))
    fr.scene = sc = syn.make_scene(160, 16, 11, -2.4, cluster_frac=1.0)      # dense cluster: some pixels saturate
    cand, off = fr.oracle_lists(oracle_mod)
    out = oracle_mod.records_per_pixel(*fr.base_numpy(cand, off), *fr.dims)
    ren = oracle_mod.render_per_pixel(*fr.base_numpy(cand, off), *fr.dims)
    np.testing.assert_allclose(out["rgb"], ren["rgb"], atol=2e-6)
    np.testing.assert_allclose(out["alpha"], ren["alpha"], atol=2e-6)
    offs, raw, ids = out["offsets"], out["raw"].astype(np.float64), out["ids"]
    assert offs[-1] > 2000
    ntx = (fr.W + 7) // 8
    cut_short = 0
    for pix in range(fr.W * fr.H):
        tile = (pix // fr.W // 8) * ntx + (pix % fr.W) // 8
        lst = cand[off[tile]:off[tile + 1]]
        hit, t = [], []
        for p in lst:
            is_hit, h = oracle_mod.hit(fr.rays_o[pix], fr.rays_d[pix], sc.positions[p], sc.log_scales[p], sc.quats[p], fr.thr)
            if is_hit:
                hit.append(int(p))
                t.append(np.float32(h["t"]))
        order = np.argsort(np.asarray(t, np.float32), kind="stable")
        want = np.asarray(hit, np.int64)[order]
        got = ids[offs[pix]:offs[pix + 1]]
        assert len(got) <= len(want) and np.array_equal(got, want[:len(got)]), pix
        if len(got) < len(want):                       # stopped early: only because the pixel is saturated
            last = raw[offs[pix + 1] - 1]
            assert last[4] * (1 - last[5]) < 1e-3 and last[4] >= 1e-3
            cut_short += 1
    assert cut_short > 0
    pix_of = np.repeat(np.arange(fr.W * fr.H), np.diff(offs))
    rgb = np.zeros((fr.W * fr.H, 3))
    np.add.at(rgb, pix_of, (raw[:, 4] * raw[:, 5])[:, None] * raw[:, :3])
    np.testing.assert_allclose(rgb, out["rgb"], atol=2e-6)
    assert np.array_equal(out["x6"][:, :3], fr.rays_d[pix_of])


# ---------------------------------------------------------------------------------------------
# feature channel
# ---------------------------------------------------------------------------------------------
def test_feature_is_the_weighted_sum_of_gated_mixes(oracle_mod):
    # independent framebuffer restatement in float64 (tests/test_record_feature_512.py:80-98): replay the
    # blend from the oracle's per-hit quantities obtained one primitive at a time
    from helpers import Frame
    fr = Frame("cfg1_5k_160x120", n=300, width=24, height=16, feature_dim=20)
    cand, off = fr.oracle_lists(oracle_mod)
    sc = fr.scene
    out = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims, feat_attr=sc.feat_attr)
    rgb_only = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims)
    np.testing.assert_array_equal(out["rgb"], rgb_only["rgb"])     # same w as RGB
    ids, _ = oracle_mod.sort_tiles(fr.rays_o, fr.rays_d, sc.positions, sc.log_scales, sc.quats, cand, off, fr.W, fr.H, 8, 8)
    feat = np.zeros((fr.W * fr.H, 20))
    ntx = (fr.W + 7) // 8
    for pix in range(0, fr.W * fr.H, 7):
        x, y = pix % fr.W, pix // fr.W
        tile = (y // 8) * ntx + x // 8
        T = 1.0
        for p in ids[off[tile]:off[tile + 1]]:
            if T < 1e-3:
                break
            hit, h = oracle_mod.hit(fr.rays_o[pix], fr.rays_d[pix], sc.positions[p], sc.log_scales[p], sc.quats[p], fr.thr)
            if not hit:
                continue
            x6 = np.concatenate([fr.rays_d[pix], h["d"]])[None]
            o = oracle_mod.mlp(x6, [p], sc.freq, sc.att, *sc.mlp())[0].astype(np.float64)
            sigma = (o[3] if o[3] > 20 else math.log1p(math.exp(o[3]))) * float(h["decay"])
            alpha = 1 - math.exp(-sigma)
            g = oracle_mod.gates(h["q"], sc.log_scales[p], 1.5, 2.0).astype(np.float64)
            feat[pix] += T * alpha * (g[:, None] * sc.feat_attr[p].astype(np.float64)).sum(0)
            T *= 1 - alpha
        np.testing.assert_allclose(out["feat"][pix], feat[pix], atol=2e-6)
    assert np.abs(out["feat"]).max() > 1e-3


def test_five_slot_equals_four_slot_after_folding(oracle_mod):
    # scannet/checkpoints.py:234-235: slot_k(4) = base + delta_k  <=>  5-slot (base, deltas), since gates sum to 1
    from helpers import Frame
    fr = Frame("cfg1_5k_160x120", n=200, width=16, height=16, feature_dim=8, feature_slots=5)
    cand, off = fr.oracle_lists(oracle_mod)
    f5 = fr.scene.feat_attr
    f4 = f5[:, :1] + f5[:, 1:]
    a = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims, feat_attr=f5)
    b = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims, feat_attr=f4)
    np.testing.assert_allclose(a["feat"], b["feat"], atol=2e-6)
    assert np.abs(a["feat"]).max() > 1e-3


def test_two_dimensional_feature_attribute_is_ungated(oracle_mod):
    s = stack_scene(3, b3=[0, 0, 0, 0.0])
    fa = np.array([[1.0, 2.0], [3.0, 4.0], [5.0, 6.0]], np.float32)
    out = oracle_mod.render_tilecenter(*base(s), *DIMS1, feat_attr=fa)
    a = 1 - math.exp(-math.log(2.0))
    w = np.array([a * (1 - a) ** i for i in range(3)])
    np.testing.assert_allclose(out["feat"][0], (w[:, None] * fa).sum(0), atol=1e-6)


# ---------------------------------------------------------------------------------------------
# pruning statistics (np_tile_kernels.cu:2139-2519)
# ---------------------------------------------------------------------------------------------
def test_statistics_of_a_zero_weight_stack_follow_the_geometric_series(oracle_mod):
    # n identical primitives on one pixel: w_i = a (1-a)^i, colour after step i = c (1 - (1-a)^(i+1))
    n = 12
    b3 = [0.4, -0.3, 0.9, 0.5]
    s = stack_scene(n, b3=b3)
    gt = np.array([[0.2, 0.6, 0.1]], np.float32)
    out = oracle_mod.render_stats(*base(s), *DIMS1, gt)
    plain = oracle_mod.render_tilecenter(*base(s), *DIMS1, family=2)
    assert np.array_equal(out["rgb"], plain["rgb"]) and np.array_equal(out["alpha"], plain["alpha"])
    a = 1.0 - np.exp(-np.log1p(np.exp(b3[3])))             # decay = 1 on the centre ray
    c = 1.0 / (1.0 + np.exp(-np.array(b3[:3])))
    w = a * (1.0 - a) ** np.arange(n)
    live = np.concatenate([[True], (1.0 - a) ** np.arange(1, n) >= 1e-3])   # transmittance before step i
    w = np.where(live, w, 0.0)
    np.testing.assert_allclose(out["sum_w"], w, rtol=2e-6, atol=1e-9)
    np.testing.assert_allclose(out["max_w"], w, rtol=2e-6, atol=1e-9)          # one pixel: max = sum
    assert np.array_equal(out["hits"], (w > 1e-8).astype(np.int64))
    assert np.array_equal(out["contrib"], (w > 0.1).astype(np.int64)) and 0 < out["contrib"].sum() < live.sum()
    colour = c[None, :] * (1.0 - (1.0 - a) ** (np.arange(n) + 1))[:, None]
    err = np.abs(colour - gt.astype(np.float64)).sum(axis=1)
    np.testing.assert_allclose(out["sum_werr"], np.where(w > 0.1, w * err, 0.0), rtol=5e-6, atol=1e-9)


def test_statistics_sum_to_the_image_alpha_and_order_by_plain_depth(oracle_mod):
    from helpers import Frame
    fr = Frame("cfg1_5k_160x120", n=600, width=40, height=24)
    cand, off = fr.oracle_lists(oracle_mod)
    gt = np.random.default_rng(3).random((fr.W * fr.H, 3), dtype=np.float32)
    out = oracle_mod.render_stats(*fr.base_numpy(cand, off), *fr.dims, gt)
    plain = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims, family=2)
    assert np.array_equal(out["rgb"], plain["rgb"]) and np.array_equal(out["alpha"], plain["alpha"])
    # every pixel's weights sum to its alpha = 1 - T
    np.testing.assert_allclose(out["sum_w"].sum(), plain["alpha"].astype(np.float64).sum(), rtol=1e-5)
    assert 0 < out["hits"].sum() <= plain["stats"][3]      # hits with w > 1e-8 among all evaluated hits
    assert (out["max_w"] <= out["sum_w"] + 1e-12).all() and (out["contrib"] <= out["hits"]).all()
    assert (out["sum_werr"] <= 3.0 * out["sum_w"] + 1e-9).all() and out["contrib"].sum() > 0


# ---------------------------------------------------------------------------------------------
# training records (np_tile_kernels.cu:2925-3206 modes 1/3, wrapper :6897-6998)
# ---------------------------------------------------------------------------------------------
def test_records_of_a_zero_weight_stack(oracle_mod):
    # tests/test_training_wmma.py:103-139 style: n coincident primitives on one pixel
    n, b3 = 9, [0.4, -0.3, 0.9, 0.5]
    s = stack_scene(n, b3=b3)
    out = oracle_mod.records(*base(s), *DIMS1)
    a = 1.0 - np.exp(-np.log1p(np.exp(b3[3])))
    k = next(i for i in range(1, 100) if (1 - a) ** i < 1e-3)
    m = min(n, k)
    assert not out["overflow"] and out["offsets"].tolist() == [0, m] and out["ids"].tolist() == list(range(m))
    raw = out["raw"]
    np.testing.assert_allclose(raw[:, :3], np.tile(1 / (1 + np.exp(-np.array(b3[:3]))), (m, 1)), rtol=2e-6)
    np.testing.assert_allclose(raw[:, 3], np.log1p(np.exp(b3[3])), rtol=2e-6)       # softplus
    np.testing.assert_allclose(raw[:, 4], (1 - a) ** np.arange(m), rtol=1e-5)        # T before each hit
    np.testing.assert_allclose(raw[:, 5], a, rtol=2e-6)
    assert np.all(raw[:, 6] == 1.0) and np.all(raw[:, 7] == np.float32(b3[3]))       # decay on the centre ray, logit
    assert np.array_equal(out["x6"], np.tile(np.array([[0, 0, 1, 0, 0, 0]], np.float32), (m, 1)))
    assert np.all(out["masks"] == 0)                                                  # zero weights, zero biases
    np.testing.assert_allclose(out["gates"], 0.25)                                    # q = 0: uniform gates
    # hit capacity (np_tile_kernels.cu:3166-3168): a pixel that is still live with max_hits records overflows,
    # even at the end of its list; one that saturated in time does not
    assert oracle_mod.records(*base(s), *DIMS1, max_hits=3)["overflow"]
    assert oracle_mod.records(*base(stack_scene(3, b3=b3)), *DIMS1, max_hits=3)["overflow"]
    opaque = oracle_mod.records(*base(stack_scene(5, b3=[0, 0, 0, 20.0])), *DIMS1, max_hits=1)
    assert not opaque["overflow"] and opaque["offsets"].tolist() == [0, 1]


def test_records_recompose_the_image_and_match_the_forward_render(oracle_mod):
    from helpers import Frame
    fr = Frame("cfg1_5k_160x120", n=700, hidden=16, width=40, height=24)
    sc = fr.scene
    cand, off = fr.oracle_lists(oracle_mod)
    out = oracle_mod.records(*fr.base_numpy(cand, off), *fr.dims, max_hits=512, beta=1.3, temp=2.2)
    fwd = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims)
    assert not out["overflow"] and out["offsets"][-1] == fwd["stats"][3] > 5000      # one record per evaluated hit
    # tests/test_primitive_csr.py:49-53: records-forward image == tile-centre forward within 2e-6
    np.testing.assert_allclose(out["rgb"], fwd["rgb"], atol=2e-6)
    np.testing.assert_allclose(out["alpha"], fwd["alpha"], atol=2e-6)
    offs, raw, ids = out["offsets"], out["raw"].astype(np.float64), out["ids"]
    pix_of = np.repeat(np.arange(fr.W * fr.H), np.diff(offs))
    first = np.zeros(len(ids), bool)
    first[offs[:-1][np.diff(offs) > 0]] = True
    assert np.all(raw[first, 4] == 1.0)                                               # T starts at one
    nxt = ~first[1:]                                                                  # record i+1 continues pixel of i
    np.testing.assert_allclose(raw[1:, 4][nxt], (raw[:-1, 4] * (1 - raw[:-1, 5]))[nxt], rtol=3e-7)
    np.testing.assert_allclose(raw[:, 5], 1 - np.exp(-raw[:, 3] * raw[:, 6]), atol=2e-7)
    np.testing.assert_allclose(raw[:, 3], np.log1p(np.exp(raw[:, 7])), rtol=3e-6)
    rgb = np.zeros((fr.W * fr.H, 3))
    np.add.at(rgb, pix_of, (raw[:, 4] * raw[:, 5])[:, None] * raw[:, :3])
    np.testing.assert_allclose(rgb, out["rgb"], atol=2e-6)
    assert np.array_equal(out["x6"][:, :3], fr.rays_d[pix_of])                        # tests/test_training_wmma.py:123-125
    np.testing.assert_allclose(out["gates"].sum(1), 1.0, atol=1e-6)
    assert (raw[:, 6] > fr.thr).all() and (raw[:, 4] >= 1e-3).all()
    # ReLU masks against an independent float64 evaluation (units whose pre-activation is not near zero)
    enc = np.concatenate([np.sin(out["x6"][:, :, None] * (sc.freq * sc.att)[None, None, :]).reshape(len(ids), -1),
                          np.cos(out["x6"][:, :, None] * (sc.freq * sc.att)[None, None, :]).reshape(len(ids), -1)], 1)
    pre1 = np.einsum("rhi,ri->rh", sc.W1[ids].astype(np.float64), enc.astype(np.float64)) + sc.b1[ids]
    pre2 = np.einsum("roh,rh->ro", sc.W2[ids].astype(np.float64), np.maximum(pre1, 0)) + sc.b2[ids]
    for layer, pre in enumerate((pre1, pre2)):
        bitsm = (out["masks"][:, layer].astype(np.int64)[:, None] >> np.arange(sc.hidden)[None, :]) & 1
        sure = np.abs(pre) > 1e-5
        assert np.array_equal(bitsm[sure], (pre > 0)[sure].astype(np.int64)) and sure.mean() > 0.99
    o3 = np.einsum("rh,rh->r", sc.W3[ids, 3].astype(np.float64), np.maximum(pre2, 0)) + sc.b3[ids, 3]
    np.testing.assert_allclose(raw[:, 7], o3, atol=2e-5)


def _synthetic_records(seed, pixels=40, n=12, max_per_pixel=9):
    """Random per-pixel record lists with every raw field computed in float64 from leaves, plus the float64
    autograd gradients of  sum_pix (grad_rgb . rgb + grad_t * T_final)."""
    g = torch.Generator().manual_seed(seed)
    counts = torch.randint(0, max_per_pixel + 1, (pixels,), generator=g)
    counts[0], counts[1] = 0, max_per_pixel
    offsets = torch.zeros(pixels + 1, dtype=torch.int64)
    offsets[1:] = counts.cumsum(0)
    R = int(offsets[-1])
    ids = torch.randint(0, n, (R,), generator=g)
    d = (torch.randn(R, 3, generator=g) * 0.08).double()
    o = torch.randn(R, 4, generator=g).double().requires_grad_(True)
    dpos = torch.zeros(n, 3, dtype=torch.float64, requires_grad=True)
    log_s = (torch.randn(n, 3, generator=g) * 0.3 - 2.3).double().requires_grad_(True)
    q0 = torch.randn(n, 4, generator=g).double()
    quats = (q0 / q0.norm(dim=1, keepdim=True)).requires_grad_(True)
    grad_rgb = torch.randn(pixels, 3, generator=g).double()
    grad_t = torch.randn(pixels, generator=g).double()

    w, x, y, z = quats[ids].unbind(1)
    rot = torch.stack([torch.stack([1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y)], 1),
                       torch.stack([2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x)], 1),
                       torch.stack([2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)], 1)], 1)
    local = torch.einsum("rji,rj->ri", rot, d + dpos[ids])                 # R(q)^T (offset)
    decay = torch.exp(-0.5 * (torch.exp(-2 * log_s[ids]) * local * local).sum(1))
    colour = torch.sigmoid(o[:, :3])
    sigma_raw = torch.nn.functional.softplus(o[:, 3])
    alpha = 1 - torch.exp(-sigma_raw * decay)
    trans = torch.ones(R, dtype=torch.float64)
    loss = torch.zeros((), dtype=torch.float64)
    trans_rows = []
    for pix in range(pixels):
        t = torch.ones((), dtype=torch.float64)
        for r in range(int(offsets[pix]), int(offsets[pix + 1])):
            trans_rows.append(t)
            loss = loss + (grad_rgb[pix] * colour[r]).sum() * t * alpha[r]
            t = t * (1 - alpha[r])
        loss = loss + grad_t[pix] * t
    loss.backward()
    trans = torch.stack(trans_rows) if trans_rows else trans
    raw = torch.cat([colour, sigma_raw[:, None], trans[:, None], alpha[:, None], decay[:, None], o[:, 3:4]], 1).detach()
    x6 = torch.cat([torch.zeros(R, 3, dtype=torch.float64), d], 1)
    want = (o.grad, dpos.grad, log_s.grad, quats.grad)
    inputs = (ids.int().numpy(), offsets.numpy(), x6.float().numpy(), raw.float().numpy(), log_s.detach().float().numpy(),
              quats.detach().float().numpy(), grad_rgb.float().numpy(), grad_t.float().numpy())
    return inputs, [w.numpy() for w in want]


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_reverse_compositing_matches_float64_autograd(oracle_mod, seed):
    # primitive_records.cuh:3-46: d4 = dL/d(pre-activation outputs); geometry gradients through the falloff
    # only (the hit offset is an input), which is exactly what differentiating the restatement above gives
    inputs, want = _synthetic_records(seed)
    got = oracle_mod.records_reverse(*inputs)
    for name, a, b in zip(("d4", "grad_positions", "grad_log_scales", "grad_quats"), got, want):
        scale = max(1.0, float(np.abs(b).max()))
        assert np.abs(a - b).max() <= 2e-5 * scale, (name, float(np.abs(a - b).max()), scale)
        assert np.abs(b).max() > 1e-3, name      # a gradient that is identically zero would pin nothing


def test_reverse_compositing_of_empty_pixels_is_zero(oracle_mod):
    z = np.zeros
    d4, gp, gs, gq = oracle_mod.records_reverse(z(0, np.int32), z(5, np.int64), z((0, 6), np.float32), z((0, 8), np.float32),
                                                z((3, 3), np.float32), np.tile(np.float32([1, 0, 0, 0]), (3, 1)),
                                                np.ones((4, 3), np.float32), np.ones(4, np.float32))
    assert d4.shape == (0, 4) and not gp.any() and not gs.any() and not gq.any()
