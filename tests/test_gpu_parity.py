"""Parity of the HIP path against the CPU oracle on the same seeded inputs, through the C ABI.

f32 paths are held to bit equality (tolerance 0): the kernels perform the oracle's operations in the
oracle's order, with no native transcendental instruction and no contraction.
"""
import numpy as np
import pytest
import torch

from conftest import to_dev
from helpers import Frame, bits

pytestmark = pytest.mark.gpu


def _t(a, device):
    return to_dev(a, device)


def _assert_bits(got, want, what):
    got = got.detach().cpu().numpy() if torch.is_tensor(got) else got
    same = np.array_equal(bits(got), bits(want))
    if not same:
        d = np.abs(got.astype(np.float64) - want.astype(np.float64))
        raise AssertionError(f"{what}: {int((bits(got) != bits(want)).sum())} of {got.size} values differ, max abs {d.max():.3e}")


@pytest.fixture(scope="module")
def frame1(oracle_mod):
    fr = Frame("cfg1_5k_160x120")
    fr.lists = fr.oracle_lists(oracle_mod)
    return fr


def test_binning_matches_oracle_bit_exactly(device, oracle_mod, frame1):
    from mlp_splatting_amd import ops
    fr = frame1
    sc = fr.scene
    cand, off = ops.bin_legacy(_t(sc.positions, device), _t(sc.log_scales, device), torch.from_numpy(fr.view)[None],
                               torch.from_numpy(fr.proj), fr.W, fr.H, 8, fr.thr)
    np.testing.assert_array_equal(off.cpu().numpy(), fr.lists[1])
    np.testing.assert_array_equal(cand.cpu().numpy(), fr.lists[0])
    assert cand.dtype == torch.int32 and off.dtype == torch.int32


# (the last two frames have 504 and 510 super-tiles: more than one LDS bitmap of the by-primitive counting pass of
# level 1 holds, so it runs in two bands of super-tile rows)
@pytest.mark.parametrize("width,height,tile", [(100, 76, 8), (100, 76, 16), (33, 17, 8), (3000, 2600, 16),
                                               (1920, 1080, 8)])
def test_binning_ragged_frames_and_tile_sizes(device, oracle_mod, width, height, tile):
    from mlp_splatting_amd import ops
    fr = Frame("cfg1_5k_160x120", n=3000, width=width, height=height, tile=tile, eye=(1.0, 0.8, -1.2), target=(0, 0, 0))
    sc = fr.scene
    want = fr.oracle_lists(oracle_mod)
    cand, off = ops.bin_legacy(_t(sc.positions, device), _t(sc.log_scales, device), torch.from_numpy(fr.view)[None],
                               torch.from_numpy(fr.proj), fr.W, fr.H, tile, fr.thr)
    np.testing.assert_array_equal(off.cpu().numpy(), want[1])
    np.testing.assert_array_equal(cand.cpu().numpy(), want[0])


@pytest.mark.parametrize("n,grow", [(4500, 2.5), (2049, 4.0), (1, 3.0), (63, 0.0)])
def test_binning_with_primitives_that_span_many_super_tiles(device, oracle_mod, n, grow):
    """Level 1 by primitive hands every primitive that overlaps more than four super-tiles to a whole wavefront: here
    (log-scales raised by `grow`) most or all primitives of a 2048-chunk are such, on a 20-super-tile screen, and the
    chunk boundaries fall at 2048 + 1 and inside a single wavefront."""
    from mlp_splatting_amd import ops
    fr = Frame("cfg1_5k_160x120", n=n, width=320, height=200, eye=(0.2, 0.1, -1.0), target=(0, 0, 0.2))
    sc = fr.scene
    logs = (sc.log_scales + np.float32(grow)).astype(np.float32)
    want = oracle_mod.bin_legacy(sc.positions, logs, fr.view[None], fr.proj, fr.W, fr.H, 8, fr.thr)
    cand, off = ops.bin_legacy(_t(sc.positions, device), _t(logs, device), torch.from_numpy(fr.view)[None],
                               torch.from_numpy(fr.proj), fr.W, fr.H, 8, fr.thr)
    if grow >= 2.5 and n > 1000:
        assert want[0].size > 100 * n          # (a primitive lands in hundreds of tiles: the case is what it says)
    np.testing.assert_array_equal(off.cpu().numpy(), want[1])
    np.testing.assert_array_equal(cand.cpu().numpy(), want[0])


@pytest.mark.parametrize("n", [300000, 2200000])
def test_binning_with_more_chunks_than_a_workgroup_takes_at_once(device, oracle_mod, n):
    """The level-1 fill places a super-tile's list itself: a workgroup adds up the counts before it and scans its row
    of (chunk, super-tile) counts, 1,024 chunks per pass, the ballots of each wavefront's first eight chunks requested
    ahead.  147 chunks (300 k primitives) go beyond those eight, 1,075 chunks (2.2 M) into a second pass; both entry
    points, the two-call one and the asynchronous one with its guard, against the oracle."""
    from mlp_splatting_amd import ops, synthetic as syn
    rng = np.random.default_rng(3)
    pos = (rng.random((n, 3), dtype=np.float32) * 4 - 2).astype(np.float32)
    logs = (rng.standard_normal((n, 3)).astype(np.float32) * np.float32(0.3) - np.float32(5.5)).astype(np.float32)
    W, H, f, thr = 96, 64, 60.0, 5e-3
    view = syn.view_matrix(syn.look_at((0.3, -0.2, -2.5), (0.0, 0.0, 0.4)))
    proj = syn.projection_matrix(f, W, H)
    want_cand, want_off = oracle_mod.bin_legacy(pos, logs, view[None], proj, W, H, 8, thr)
    assert want_cand.size > n // 2
    p, l = _t(pos, device), _t(logs, device)
    cand, off = ops.bin_legacy(p, l, torch.from_numpy(view)[None], torch.from_numpy(proj), W, H, 8, thr)
    np.testing.assert_array_equal(off.cpu().numpy(), want_off)
    np.testing.assert_array_equal(cand.cpu().numpy(), want_cand)
    cand2, off2, counts = ops.bin_legacy_async(p, l, _t(view, device), _t(proj, device), W, H, 8, thr, want_cand.size + 7)
    pairs, longest, _, guard = counts.tolist()
    assert (pairs, longest, guard) == (want_cand.size, int(np.diff(want_off).max()), 0)
    np.testing.assert_array_equal(off2.cpu().numpy(), want_off)
    np.testing.assert_array_equal(cand2.cpu().numpy()[:pairs], want_cand)


@pytest.mark.parametrize("n,width,height", [(5000, 160, 120), (300000, 96, 64), (1500, 21, 13)])
def test_lists_in_segments_are_the_oracles_lists(device, oracle_mod, n, width, height):
    """mlpsp_bin_segments_async_device_matrices: every tile's list in a segment of its own, written by a level 2 that
    tests and writes in one launch.  The same ids in the same order as the oracle's lists; a stride below the longest
    list keeps the first `stride` entries and reports the full length; the sort and the matrix-core render read such
    lists through their ends and give what they give for the lists written one after the other."""
    from mlp_splatting_amd import ops, synthetic as syn
    if n == 300000:
        rng = np.random.default_rng(3)
        pos = (rng.random((n, 3), dtype=np.float32) * 4 - 2).astype(np.float32)
        logs = (rng.standard_normal((n, 3)).astype(np.float32) * np.float32(0.3) - np.float32(5.5)).astype(np.float32)
        view = syn.view_matrix(syn.look_at((0.3, -0.2, -2.5), (0.0, 0.0, 0.4)))
        proj, thr = syn.projection_matrix(60.0, width, height), 5e-3
        fr = None
    else:
        fr = Frame("cfg1_5k_160x120", n=n, hidden=32, width=width, height=height)
        pos, logs, view, proj, thr = fr.scene.positions, fr.scene.log_scales, fr.view, fr.proj, fr.thr
    want_cand, want_off = oracle_mod.bin_legacy(pos, logs, view[None], proj, width, height, 8, thr)
    lengths = np.diff(want_off)
    T, longest = lengths.size, int(lengths.max())
    p, l, v, pr = _t(pos, device), _t(logs, device), _t(view, device), _t(proj, device)
    for stride in (longest, longest + 37, max(longest // 2, 1)):
        cand, off, ends, counts = ops.bin_segments_async(p, l, v, pr, width, height, 8, thr, stride=stride)
        off_h, ends_h, cand_h = off.cpu().numpy(), ends.cpu().numpy(), cand.cpu().numpy()
        np.testing.assert_array_equal(off_h, np.arange(T + 1) * stride)
        np.testing.assert_array_equal(ends_h - off_h[:-1], np.minimum(lengths, stride))
        for t in range(T):
            np.testing.assert_array_equal(cand_h[off_h[t]:ends_h[t]], want_cand[want_off[t]:want_off[t] + min(lengths[t], stride)])
        pairs, over, l1_entries, guard = counts.tolist()
        assert (pairs, over, guard) == (0, longest if longest > stride else 0, 0) and l1_entries > 0
    if fr is None:
        return
    # sort and render through the ends
    sc = fr.scene
    stride = longest + 5
    cand, off, ends, _ = ops.bin_segments_async(p, l, v, pr, width, height, 8, thr, stride=stride)
    rec = ops.prepare_primitives(p, l, _t(sc.quats, device))
    ro, rd = _t(fr.rays_o, device), _t(fr.rays_d, device)
    c, o = _t(want_cand, device), _t(want_off, device)
    plain, plain_keys = ops.sort_tiles(ro, rd, rec, c, o, width, height, 8, 8, cull_threshold=thr, want_keys=True)
    seg, seg_keys = ops.sort_tiles(ro, rd, rec, cand, off, width, height, 8, 8, cull_threshold=thr, want_keys=True, tile_ends=ends)
    # lists whose ids ascend (these do) may be sorted as (key, id) words, with the tiles' pyramids from the prologue:
    # the same order, and the same lists with or without the vouching
    _, pyramids, _ = ops.frame_prologue(ro, rd, width, height, 8, 8)
    for c_, o_, e_ in ((c, o, None), (cand, off, ends)):
        a = ops.sort_tiles(ro, rd, rec, c_, o_, width, height, 8, 8, cull_threshold=thr, want_keys=True, tile_pyramids=pyramids,
                           tile_ends=e_)
        b = ops.sort_tiles(ro, rd, rec, c_, o_, width, height, 8, 8, cull_threshold=thr, want_keys=True, tile_pyramids=pyramids,
                           tile_ends=e_, ids_ascend=True)
        ends_h = (o_[1:] if e_ is None else e_).cpu().numpy()
        for t in range(T):
            lo, hi = int(o_[t]), int(ends_h[t])
            assert torch.equal(a[0][lo:hi], b[0][lo:hi]) and torch.equal(a[1][lo:hi], b[1][lo:hi])
    plain, seg, plain_keys, seg_keys = plain.cpu().numpy(), seg.cpu().numpy(), plain_keys.cpu().numpy(), seg_keys.cpu().numpy()
    for t in range(T):
        np.testing.assert_array_equal(seg[t * stride:t * stride + lengths[t]], plain[want_off[t]:want_off[t + 1]])
        assert np.array_equal(bits(seg_keys[t * stride:t * stride + lengths[t]]), bits(plain_keys[want_off[t]:want_off[t + 1]]))
    args = (_t(sc.freq, device), _t(sc.att, device), *[_t(w, device) for w in sc.mlp()], width, height, thr)
    for bf16 in (True, False):
        a = ops.render_tilecenter_mfma(ro, rd, rec, _t(plain, device), o, *args, bf16=bf16)
        b = ops.render_tilecenter_mfma(ro, rd, rec, _t(seg, device), off, *args, bf16=bf16, tile_ends=ends)
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1]) and a[2] == b[2]
        assert float(a[1].mean()) > 0.2
    comp, comp_off = ops.compact_segments(_t(seg, device), off, ends)
    np.testing.assert_array_equal(comp.cpu().numpy(), plain)
    np.testing.assert_array_equal(comp_off.cpu().numpy(), want_off)


def test_level1_overflow_empties_the_lists_in_segments_too(device):
    """Primitives so large that each overlaps every super-tile overflow the level-1 lists of a scratch of the ordinary
    size (room for eight super-tiles per primitive): guard = 1, the number of level-1 entries is reported, every list
    is empty -- from the segment entry as from the asynchronous entry with a candidate buffer --, and four times the
    scratch holds them."""
    from mlp_splatting_amd import ops, synthetic as syn
    n, width, height, thr = 12000, 640, 480, 1e-3
    rng = np.random.default_rng(5)
    pos = (rng.random((n, 3), dtype=np.float32) - 0.5).astype(np.float32)
    logs = np.full((n, 3), -0.5, np.float32)
    view = syn.view_matrix(syn.look_at((0.0, 0.0, -3.0), (0.0, 0.0, 0.0)))
    proj = syn.projection_matrix(500.0, width, height)
    p, l, v, pr = _t(pos, device), _t(logs, device), _t(view, device), _t(proj, device)
    cand, off, ends, counts = ops.bin_segments_async(p, l, v, pr, width, height, 8, thr, stride=64)
    pairs, over, l1_entries, guard = counts.tolist()
    assert guard == 1 and l1_entries > 8 * n + 65536 and torch.equal(ends, off[:-1])
    _, off2, counts2 = ops.bin_legacy_async(p, l, v, pr, width, height, 8, thr, 1 << 20)
    assert counts2.tolist()[2:] == [l1_entries, 1] and not off2.any()
    _, off4, ends4, counts4 = ops.bin_segments_async(p, l, v, pr, width, height, 8, thr, stride=64, scratch_scale=16)
    pairs, over, l1_entries4, guard = counts4.tolist()
    assert guard == 0 and l1_entries4 == l1_entries and over > 64 and bool((ends4 - off4[:-1] == 64).all())


def test_lists_in_segments_without_primitives(device):
    from mlp_splatting_amd import ops
    none = torch.empty(0, 3, dtype=torch.float32, device=device)
    eye = torch.eye(4, dtype=torch.float32, device=device)
    cand, off, ends, counts = ops.bin_segments_async(none, none, eye, eye.clone(), 40, 24, 8, 1e-3, stride=16)
    assert cand.numel() == 15 * 16 and counts.tolist() == [0, 0, 0, 0]
    assert not off.any() and not ends.any()


def test_binning_with_several_views_and_no_view_per_tile(device, oracle_mod):
    """Several view matrices without tile_view_ids: every tile is binned against view 0 (level 1 then runs the walk
    over (chunk, super-tile) pairs with all the views, a superset that level 2 cuts down)."""
    from mlp_splatting_amd import ops, synthetic as syn
    fr = Frame("cfg1_5k_160x120", n=5000, width=200, height=136)
    sc = fr.scene
    views = np.stack([fr.view, syn.view_matrix(syn.look_at((1.0, 0.3, -0.8), (0, 0, 0)))]).astype(np.float32)
    want = oracle_mod.bin_legacy(sc.positions, sc.log_scales, views, fr.proj, fr.W, fr.H, 8, fr.thr)
    cand, off = ops.bin_legacy(_t(sc.positions, device), _t(sc.log_scales, device), torch.from_numpy(views),
                               torch.from_numpy(fr.proj), fr.W, fr.H, 8, fr.thr)
    assert want[0].size > 1000
    np.testing.assert_array_equal(off.cpu().numpy(), want[1])
    np.testing.assert_array_equal(cand.cpu().numpy(), want[0])
    one = oracle_mod.bin_legacy(sc.positions, sc.log_scales, views[:1], fr.proj, fr.W, fr.H, 8, fr.thr)
    np.testing.assert_array_equal(one[0], want[0])


def test_tile_view_binning_matches_oracle(device, oracle_mod):
    from mlp_splatting_amd import ops, synthetic as syn
    fr = Frame("cfg1_5k_160x120", n=4000, width=96, height=64)
    sc = fr.scene
    ro, rd, tv, views = syn.mosaic_frame(48, 32, fr.f, syn.random_poses(4, seed=2))
    proj = syn.projection_matrix(fr.f, 96, 64)
    want = oracle_mod.bin_legacy(sc.positions, sc.log_scales, views, proj, 96, 64, 8, fr.thr, tile_view_ids=tv)
    cand, off = ops.bin_legacy(_t(sc.positions, device), _t(sc.log_scales, device), torch.from_numpy(views),
                               torch.from_numpy(proj), 96, 64, 8, fr.thr, tile_view_ids=_t(tv, device))
    assert want[0].size > 500
    np.testing.assert_array_equal(off.cpu().numpy(), want[1])
    np.testing.assert_array_equal(cand.cpu().numpy(), want[0])


def test_binning_empty_cases(device):
    from mlp_splatting_amd import ops
    pos = torch.zeros(0, 3, device=device)
    cand, off = ops.bin_legacy(pos, pos.clone(), torch.eye(4)[None], torch.eye(4), 16, 16, 8, 1e-3)
    assert cand.numel() == 0 and off.tolist() == [0] * 5
    # everything behind the camera
    pos = torch.tensor([[0.0, 0.0, -3.0]], device=device)
    cand, off = ops.bin_legacy(pos, torch.zeros(1, 3, device=device), torch.eye(4)[None], torch.eye(4), 16, 16, 8, 1e-3)
    assert cand.numel() == 0 and off.tolist() == [0] * 5


def test_raycone_binning_matches_oracle(device, oracle_mod):
    from mlp_splatting_amd.camera import ray_cone_candidates
    fr = Frame("cfg1_5k_160x120", n=2500, width=80, height=56)
    sc = fr.scene
    want = oracle_mod.bin_raycone(fr.rays_o, fr.rays_d, sc.positions, sc.log_scales, fr.W, fr.H, 8, 0.005)
    ids, off = ray_cone_candidates(_t(fr.rays_o, device), _t(fr.rays_d, device), _t(sc.positions, device),
                                   _t(sc.log_scales, device), fr.W, fr.H, 8, 0.005)
    assert 0 < want[0].size < 2500 * 70
    np.testing.assert_array_equal(off.cpu().numpy(), want[1])
    np.testing.assert_array_equal(ids.cpu().numpy(), want[0])
    ro = torch.zeros(64, 3, device=device)
    ro[1, 0] = 1
    with pytest.raises(ValueError, match="single camera"):
        ray_cone_candidates(ro, torch.ones_like(ro), torch.ones(1, 3, device=device), torch.zeros(1, 3, device=device), 8, 8, 8, 0.005)


@pytest.mark.parametrize("rays,scale", [(1200 * 680, 1.0), (160 * 120, 1e-4), (999_983, 250.0), (5, 1.0)])
def test_unit_directions_are_the_bits_of_torch_normalize(device, rays, scale):
    """The render's ray directions are F.normalize(ray_d, dim=-1) (scannet/cumodel.py:1088); the one-launch kernel
    must return exactly those bits (its order of summing the squares is the library's), zero and tiny rays included."""
    from mlp_splatting_amd import ops
    g = torch.Generator(device="cpu").manual_seed(rays)
    d = (torch.randn(rays, 3, generator=g) * scale).to(device)
    d[0] = 0.0                                             # |d| below eps: divided by eps, stays zero
    if rays > 4:
        d[1] = torch.tensor([3e-13, -4e-13, 0.0])
        d[2] = torch.tensor([1e19, 1e19, -1e19])           # squares overflow: inf norm, zero direction
        d[3] = torch.tensor([1e-23, 2e-23, 2e-23])         # squares underflow
    want = torch.nn.functional.normalize(d, dim=-1)
    got = ops.normalize_rays(d)
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    sliced = torch.randn(64, 6, generator=g).to(device)[:, :3]           # not contiguous: copied first
    assert torch.equal(ops.normalize_rays(sliced), torch.nn.functional.normalize(sliced, dim=-1))


@pytest.mark.parametrize("frame_records", [True, False, "prologue"], ids=["frame_records", "full_key", "prologue"])
@pytest.mark.parametrize("family", [1, 2])
def test_sorted_tile_lists_match_oracle_keys_and_order(device, oracle_mod, frame1, family, frame_records):
    # frame_records: the rotated offset centre - origin of the key comes from per-frame records (one per primitive,
    # written for the common ray origin) instead of being evaluated per candidate; the key bits must not depend on it
    from mlp_splatting_amd import ops
    fr = frame1
    sc = fr.scene
    cand, off = fr.lists
    rec = ops.prepare_primitives(_t(sc.positions, device), _t(sc.log_scales, device), _t(sc.quats, device))
    pyramids = None
    if frame_records == "prologue":
        # the records written beside the unit directions, in one launch; the directions are normalize_rays' bits
        unit, pyramids, frame_records = ops.frame_prologue(_t(fr.rays_o, device), _t(fr.rays_d, device), fr.W, fr.H, 8, 8,
                                                           rec)
        assert torch.equal(unit.view(torch.int32), ops.normalize_rays(_t(fr.rays_d, device)).view(torch.int32))
    ids, keys = ops.sort_tiles(_t(fr.rays_o, device), _t(fr.rays_d, device), rec, _t(cand, device), _t(off, device),
                               fr.W, fr.H, 8, 8, family=family, want_keys=True, frame_records=frame_records,
                               tile_pyramids=pyramids)
    want_ids, want_keys = oracle_mod.sort_tiles(fr.rays_o, fr.rays_d, sc.positions, sc.log_scales, sc.quats, cand, off,
                                                fr.W, fr.H, 8, 8, family=family)
    np.testing.assert_array_equal(ids.cpu().numpy(), want_ids)
    _assert_bits(keys, want_keys, "sort keys")


@pytest.mark.parametrize("case", ["spread", "ties", "behind", "clusters", "beyond_invalid", "two", "capacity",
                                  "ties:64", "behind:64", "beyond_invalid:63", "spread:65", "clusters:1",
                                  "spread:2000", "clusters:1800", "behind:2048"])
@pytest.mark.parametrize("frame_records", [True, False], ids=["frame_records", "full_key"])
@pytest.mark.parametrize("family", [1, 2])
def test_sort_is_the_stable_key_order_for_every_key_distribution(device, oracle_mod, case, family, frame_records):
    """One 8x8 tile with a hand-made list.  The kernel ranks survivors inside 256 key buckets and falls back to a
    sorting network when keys pile up in few buckets or a key exceeds the invalid key; each case below steers it
    down one of those routes, and the result must be the oracle's stable sort by key every time.  A list of at most
    64 entries is sorted by one wavefront in registers: the cases with a length after the colon go that way (65:
    the first length that does not).  Lists longer than the default capacity of 1536 are sorted with the capacity
    of the interface, 2048: a workgroup's memory is laid out for the one or the other."""
    from mlp_splatting_amd import ops
    rng = np.random.default_rng(11)
    fr = Frame("cfg1_5k_160x120", n=8, width=8, height=8, eye=(0, 0, -2.0), target=(0, 0, 0))
    case, _, short = case.partition(":")
    n = {"spread": 1500, "ties": 700, "behind": 900, "clusters": 1200, "beyond_invalid": 300, "two": 2, "capacity": 1536}[case]
    n = int(short) if short else n
    pos = np.zeros((n, 3), np.float32)
    pos[:, :2] = rng.uniform(-0.05, 0.05, (n, 2))
    if case in ("spread", "capacity"):
        pos[:, 2] = rng.uniform(-1.5, 6.0, n)
    elif case == "ties":
        pos[:] = (0.01, -0.02, 0.75)                       # every key equal: list order decides
        pos[n // 2:] = (0.0, 0.0, 1.25)
    elif case == "behind":
        pos[:, 2] = np.where(rng.random(n) < 0.5, rng.uniform(-6.0, -2.5, n), rng.uniform(-1.0, 3.0, n))
    elif case == "clusters":
        pos[:, 2] = rng.choice([-0.5, 0.8, 0.8000001, 3.0], n) + rng.normal(0, 1e-6, n)
    elif case == "beyond_invalid":
        pos[:, 2] = rng.uniform(-1.0, 3.0, n)
        pos[::5, 2] = rng.uniform(2e30, 9e31, pos[::5].shape[0])     # in front, but farther than the invalid key
        pos[1::7, 2] = -5.0                                          # behind: the invalid key itself
    else:
        pos[:, 2] = (1.0, 0.5)
    pos = pos.astype(np.float32)
    log_s = rng.uniform(-3.0, -2.0, (n, 3)).astype(np.float32)
    quat = rng.normal(size=(n, 4)).astype(np.float32)
    quat /= np.linalg.norm(quat, axis=1, keepdims=True)
    cand = rng.permutation(n).astype(np.int32) if case != "capacity" else np.arange(n, dtype=np.int32)
    cand = np.sort(cand)
    off = np.array([0, n], np.int32)
    rec = ops.prepare_primitives(_t(pos, device), _t(log_s, device), _t(quat, device))
    more = {"capacity": 2048} if n > 1536 else {}
    ids, keys = ops.sort_tiles(_t(fr.rays_o, device), _t(fr.rays_d, device), rec, _t(cand, device), _t(off, device),
                               8, 8, 8, 8, family=family, want_keys=True, frame_records=frame_records, **more)
    want_ids, want_keys = oracle_mod.sort_tiles(fr.rays_o, fr.rays_d, pos, log_s, quat, cand, off, 8, 8, 8, 8, family=family,
                                                **more)
    if case == "beyond_invalid":
        assert (want_keys > 1e30).any() and (want_keys == np.float32(1e30)).any()
    if case == "behind":
        assert 0.2 < (want_keys == np.float32(1e30)).mean() < 0.8
    np.testing.assert_array_equal(ids.cpu().numpy(), want_ids)
    _assert_bits(keys, want_keys, "sort keys")


@pytest.mark.parametrize("name,n,width,height,tile,eye", [
    ("cfg1_5k_160x120", None, 160, 120, 8, (0.3, -0.2, -0.5)), ("cfg1_5k_160x120", 4000, 100, 76, 16, (1.0, 0.8, -1.2)),
    ("cfg2_50k_640x480", 20000, 200, 136, 8, (-0.7, 0.4, 0.9)), ("cfg1_5k_160x120", 1500, 21, 13, 8, (0.1, 0.1, -0.2))])
@pytest.mark.parametrize("frame_records", [True, False, "pyramids"], ids=["frame_records", "full_key", "pyramids"])
def test_conservative_tile_culling_never_drops_a_hit(device, oracle_mod, name, n, width, height, tile, eye, frame_records):
    # per tile: the survivors, in front, are the plain sorted list with the culled ids struck out; the
    # culled ones follow as ~id in reverse list (descending id) order; (2) it is a real saving, and (3) no bit
    # of the image changes: the oracle, which tests every candidate, is the witness
    from mlp_splatting_amd import ops
    fr = Frame(name, n=n, width=width, height=height, tile=tile, eye=eye, target=(0, 0, 0.1))
    sc = fr.scene
    cand, off = fr.oracle_lists(oracle_mod)
    rec = ops.prepare_primitives(_t(sc.positions, device), _t(sc.log_scales, device), _t(sc.quats, device))
    ro, rd, c, o = _t(fr.rays_o, device), _t(fr.rays_d, device), _t(cand, device), _t(off, device)
    # (with frame records the ellipsoid's support along a face normal comes from a stored covariance, rounded up;
    # without, from the face normal rotated into the primitive's axes: two forms of the same conservative test)
    pyramids = None
    if frame_records == "pyramids":
        # the tiles' ray pyramids built once per tile by the frame prologue (from the same directions, normalised
        # again on the way with a reciprocal square root: the planes agree with the sort's own to a few ulps)
        frame_records = False
        _, pyramids, none = ops.frame_prologue(ro, rd, fr.W, fr.H, tile, tile)
        assert none is None and pyramids.numel() == (off.size - 1) * 160
    plain, _ = ops.sort_tiles(ro, rd, rec, c, o, fr.W, fr.H, tile, tile, frame_records=frame_records, tile_pyramids=pyramids)
    culled, _ = ops.sort_tiles(ro, rd, rec, c, o, fr.W, fr.H, tile, tile, cull_threshold=fr.thr, frame_records=frame_records,
                               tile_pyramids=pyramids)
    plain, culled = plain.cpu().numpy(), culled.cpu().numpy()
    for t in range(off.size - 1):
        a, b = plain[off[t]:off[t + 1]], culled[off[t]:off[t + 1]]
        gone = ~b[b < 0]
        k = b.size - gone.size
        assert (b[:k] >= 0).all() and np.array_equal(gone, np.sort(gone)[::-1])
        assert np.array_equal(b[:k], a[~np.isin(a, gone)])
    frac = (culled < 0).mean()
    assert frac > 0.15, frac
    if frame_records or pyramids is not None:      # the stored covariance, or planes that differ in their last bits,
        # cost next to nothing in culled candidates
        other, _ = ops.sort_tiles(ro, rd, rec, c, o, fr.W, fr.H, tile, tile, cull_threshold=fr.thr, frame_records=False)
        assert frac > 0.97 * float((other < 0).float().mean()), (frac, float((other < 0).float().mean()))
    want = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims)
    rgb, alpha, _ = ops.render_tilecenter_f32(ro, rd, rec, _t(culled, device), o, _t(sc.freq, device), _t(sc.att, device),
                                              *[_t(w, device) for w in sc.mlp()], fr.W, fr.H, tile, tile, fr.thr)
    _assert_bits(rgb, want["rgb"], "rgb with culled lists")
    _assert_bits(alpha, want["alpha"], "alpha with culled lists")
    # the witness again, entry by entry: no culled (tile, primitive) has a hitting pixel
    ntx = (fr.W + tile - 1) // tile
    bad = 0
    rng = np.random.default_rng(0)
    for t in rng.choice(off.size - 1, size=min(40, off.size - 1), replace=False):
        tx, ty = t % ntx, t // ntx
        pix = [y * fr.W + x for y in range(ty * tile, min((ty + 1) * tile, fr.H)) for x in range(tx * tile, min((tx + 1) * tile, fr.W))]
        for p in ~culled[off[t]:off[t + 1]][culled[off[t]:off[t + 1]] < 0][:25]:
            for q in pix:
                hit, _ = oracle_mod.hit(fr.rays_o[q], fr.rays_d[q], sc.positions[p], sc.log_scales[p], sc.quats[p], fr.thr)
                bad += int(hit)
    assert bad == 0


def test_culling_is_off_for_tiles_with_mixed_origins_or_degenerate_pyramids(device, oracle_mod):
    from mlp_splatting_amd import ops
    fr = Frame("cfg1_5k_160x120", n=1500, width=32, height=24)
    sc = fr.scene
    cand, off = fr.oracle_lists(oracle_mod)
    rec = ops.prepare_primitives(_t(sc.positions, device), _t(sc.log_scales, device), _t(sc.quats, device))
    ro = fr.rays_o.copy()
    ro[::7, 0] += 1e-3                                    # per-pixel origins: no common apex
    c, o = _t(cand, device), _t(off, device)
    ids, _ = ops.sort_tiles(_t(ro, device), _t(fr.rays_d, device), rec, c, o, fr.W, fr.H, 8, 8, cull_threshold=fr.thr)
    assert int((ids < 0).sum()) == 0
    # ... and so it is when the pyramids come from the frame prologue: those of such tiles are marked unusable
    _, pyramids, _ = ops.frame_prologue(_t(ro, device), _t(fr.rays_d, device), fr.W, fr.H)
    faces = pyramids.view(torch.int32).view(-1, 40)[:, 15]
    assert int(faces.abs().sum()) == 0
    with_records, _ = ops.sort_tiles(_t(ro, device), _t(fr.rays_d, device), rec, c, o, fr.W, fr.H, 8, 8, cull_threshold=fr.thr,
                                     tile_pyramids=pyramids)
    assert torch.equal(with_records, ids)
    _, usable, _ = ops.frame_prologue(_t(fr.rays_o, device), _t(fr.rays_d, device), fr.W, fr.H)
    assert int((usable.view(torch.int32).view(-1, 40)[:, 15] == 15).sum()) == (fr.W // 8) * (fr.H // 8)
    fr1 = Frame("cfg1_5k_160x120", n=300, width=12, height=6, tile=1)           # 1x1 tiles: no pyramid
    c1, o1 = fr1.oracle_lists(oracle_mod)
    rec1 = ops.prepare_primitives(_t(fr1.scene.positions, device), _t(fr1.scene.log_scales, device), _t(fr1.scene.quats, device))
    ids1, _ = ops.sort_tiles(_t(fr1.rays_o, device), _t(fr1.rays_d, device), rec1, _t(c1, device), _t(o1, device), 12, 6, 1, 1,
                             cull_threshold=fr1.thr)
    assert int((ids1 < 0).sum()) == 0


@pytest.mark.parametrize("family", [1, 2])
def test_frame_records_serve_only_tiles_that_share_their_origin(device, oracle_mod, family):
    """The per-frame records are written for the origin of ray 0.  A tile whose centre ray starts elsewhere must
    evaluate its keys in full: with every seventh pixel's origin moved, both kinds of tile occur, and all keys are
    still the oracle's bits.  Flat and needle-shaped primitives, far from and near the origin, stay sorted and are
    culled conservatively with the stored covariance."""
    from mlp_splatting_amd import ops
    fr = Frame("cfg1_5k_160x120", n=1500, width=48, height=32)
    sc = fr.scene
    cand, off = fr.oracle_lists(oracle_mod)
    rec = ops.prepare_primitives(_t(sc.positions, device), _t(sc.log_scales, device), _t(sc.quats, device))
    ro = fr.rays_o.copy()
    ro[3::7, 1] -= 2e-3
    ids, keys = ops.sort_tiles(_t(ro, device), _t(fr.rays_d, device), rec, _t(cand, device), _t(off, device), fr.W, fr.H,
                               8, 8, family=family, want_keys=True, cull_threshold=fr.thr)
    want_ids, want_keys = oracle_mod.sort_tiles(ro, fr.rays_d, sc.positions, sc.log_scales, sc.quats, cand, off, fr.W,
                                                fr.H, 8, 8, family=family)
    centre_moved = [(min(ty * 8 + 4, fr.H - 1) * fr.W + min(tx * 8 + 4, fr.W - 1)) % 7 == 3
                    for ty in range(fr.H // 8) for tx in range(fr.W // 8)]
    assert any(centre_moved) and not all(centre_moved)
    assert int((ids < 0).sum()) == 0                      # mixed origins inside every tile: no pyramid, nothing culled
    np.testing.assert_array_equal(ids.cpu().numpy(), want_ids)
    _assert_bits(keys, want_keys, "sort keys with mixed origins")

    # extreme shapes: axis ratios up to e^8, with and without the records
    rng = np.random.default_rng(5)
    log_s = sc.log_scales.copy()
    log_s[::3, 0] -= 6.0
    log_s[1::3, 1:] -= 5.0
    log_s[2::9] += 2.0
    log_s = log_s.astype(np.float32)
    rec2 = ops.prepare_primitives(_t(sc.positions, device), _t(log_s, device), _t(sc.quats, device))
    cand2, off2 = oracle_mod.bin_legacy(sc.positions, log_s, fr.view[None], fr.proj, fr.W, fr.H, 8, fr.thr)
    c2, o2 = _t(cand2, device), _t(off2, device)
    plain_ids, plain_keys = oracle_mod.sort_tiles(fr.rays_o, fr.rays_d, sc.positions, log_s, sc.quats, cand2, off2, fr.W,
                                                  fr.H, 8, 8, family=family)
    want = oracle_mod.render_tilecenter(fr.rays_o, fr.rays_d, sc.positions, log_s, sc.quats, cand2, off2, sc.freq, sc.att,
                                        *sc.mlp(), *fr.dims)
    for with_records in (True, False):
        got, _ = ops.sort_tiles(_t(fr.rays_o, device), _t(fr.rays_d, device), rec2, c2, o2, fr.W, fr.H, 8, 8, family=family,
                                cull_threshold=fr.thr, frame_records=with_records)
        got_np = got.cpu().numpy()
        for t in range(off2.size - 1):
            b = got_np[off2[t]:off2[t + 1]]
            gone = ~b[b < 0]
            a = plain_ids[off2[t]:off2[t + 1]]
            assert np.array_equal(b[:b.size - gone.size], a[~np.isin(a, gone)])
        if family == 1:
            rgb, alpha, _ = ops.render_tilecenter_f32(_t(fr.rays_o, device), _t(fr.rays_d, device), rec2, got, o2,
                                                      _t(sc.freq, device), _t(sc.att, device),
                                                      *[_t(w, device) for w in sc.mlp()], fr.W, fr.H, 8, 8, fr.thr)
            _assert_bits(rgb, want["rgb"], "rgb, extreme shapes, culled")
            _assert_bits(alpha, want["alpha"], "alpha, extreme shapes, culled")


def _render_gpu(fr, device, cand, off, family=1, with_t=False):
    from mlp_splatting_amd import ops
    sc = fr.scene
    rec = ops.prepare_primitives(_t(sc.positions, device), _t(sc.log_scales, device), _t(sc.quats, device))
    ro, rd, c, o = _t(fr.rays_o, device), _t(fr.rays_d, device), _t(cand, device), _t(off, device)
    order = c
    if family:
        order, _ = ops.sort_tiles(ro, rd, rec, c, o, fr.W, fr.H, fr.tile, fr.tile, family=family)
    counters = torch.zeros(4, dtype=torch.int64, device=device)
    rgb, alpha, t = ops.render_tilecenter_f32(ro, rd, rec, order, o, _t(sc.freq, device), _t(sc.att, device),
                                              *[_t(w, device) for w in sc.mlp()], fr.W, fr.H, fr.tile, fr.tile, fr.thr,
                                              with_t=with_t, counters=counters)
    return rgb, alpha, t, counters.cpu().numpy()


def test_tilecentre_render_is_bit_exact_config1(device, oracle_mod, frame1):
    fr = frame1
    cand, off = fr.lists
    want = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims)
    rgb, alpha, _, counters = _render_gpu(fr, device, cand, off)
    assert want["alpha"].mean() > 0.5
    _assert_bits(rgb, want["rgb"], "rgb")
    _assert_bits(alpha, want["alpha"], "alpha")
    np.testing.assert_array_equal(counters[1:], want["stats"][1:])   # processed, with-hit, hits


def test_scalar_and_matrix_core_f32_evaluations_agree_bit_for_bit(device, oracle_mod, frame1, monkeypatch):
    """The 72-32-32-4 and 72-16-16-4 shapes (this frame: 16 hidden units, half-filled tiles) run on the matrix
    cores; MLPSP_F32_SCALAR=1 and weight arrays that are not 16-byte aligned select the scalar kernel.  All three
    must produce the oracle's bits."""
    from mlp_splatting_amd import ops
    fr = frame1
    cand, off = fr.lists
    want = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims)
    monkeypatch.setenv("MLPSP_F32_SCALAR", "1")
    rgb, alpha, _, _ = _render_gpu(fr, device, cand, off)
    monkeypatch.delenv("MLPSP_F32_SCALAR")
    _assert_bits(rgb, want["rgb"], "rgb (scalar kernel)")
    _assert_bits(alpha, want["alpha"], "alpha (scalar kernel)")
    sc = fr.scene
    rec = ops.prepare_primitives(_t(sc.positions, device), _t(sc.log_scales, device), _t(sc.quats, device))
    ro, rd, c, o = _t(fr.rays_o, device), _t(fr.rays_d, device), _t(cand, device), _t(off, device)
    order, _ = ops.sort_tiles(ro, rd, rec, c, o, fr.W, fr.H, fr.tile, fr.tile)
    weights = []
    for w in sc.mlp():                      # every array starts 4 bytes past a 16-byte boundary
        flat = torch.empty(w.size + 1, dtype=torch.float32, device=device)
        flat[1:] = _t(w, device).reshape(-1)
        weights.append(flat[1:].view(*w.shape))
        assert weights[-1].data_ptr() % 16 == 4 and weights[-1].is_contiguous()
    rgb2, alpha2, _ = ops.render_tilecenter_f32(ro, rd, rec, order, o, _t(sc.freq, device), _t(sc.att, device),
                                                *weights, fr.W, fr.H, fr.tile, fr.tile, fr.thr)
    _assert_bits(rgb2, want["rgb"], "rgb (unaligned weights)")
    _assert_bits(alpha2, want["alpha"], "alpha (unaligned weights)")


@pytest.mark.parametrize("hidden,tile,width,height", [(16, 8, 160, 120), (32, 8, 90, 70), (32, 16, 100, 76)])
def test_small_launches_take_kernels_that_look_ahead_with_the_same_bits(device, oracle_mod, monkeypatch, hidden, tile,
                                                                       width, height):
    """A launch of at most 512 items runs two wavefronts per item, each on 32 of its pixels; up to 1,024 items one
    wavefront per item with the next entry requested ahead; with work counters never the split form.
    MLPSP_F32_AHEAD=0/1/2 picks one by hand: the oracle's bits from all three, on lists that carry culled (negative)
    ids behind the survivors, with edge tiles that are cut by the image border, and the oracle's work counters from
    the two forms that keep them."""
    from mlp_splatting_amd import ops
    fr = Frame("cfg1_5k_160x120", n=3000, hidden=hidden, width=width, height=height, tile=tile, eye=(0.5, -0.3, -0.9))
    sc = fr.scene
    cand, off = fr.oracle_lists(oracle_mod)
    want = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims)
    rec = ops.prepare_primitives(_t(sc.positions, device), _t(sc.log_scales, device), _t(sc.quats, device))
    ro, rd, c, o = _t(fr.rays_o, device), _t(fr.rays_d, device), _t(cand, device), _t(off, device)
    order, _ = ops.sort_tiles(ro, rd, rec, c, o, fr.W, fr.H, tile, tile, cull_threshold=fr.thr)
    assert 0.1 < float((order < 0).float().mean()) < 0.9
    args = (ro, rd, rec, order, o, _t(sc.freq, device), _t(sc.att, device), *[_t(w, device) for w in sc.mlp()], fr.W, fr.H,
            tile, tile, fr.thr)
    for mode in ("0", "1", "2", None):
        if mode is None:
            monkeypatch.delenv("MLPSP_F32_AHEAD")
        else:
            monkeypatch.setenv("MLPSP_F32_AHEAD", mode)
        rgb, alpha, _ = ops.render_tilecenter_f32(*args)
        _assert_bits(rgb, want["rgb"], f"rgb (MLPSP_F32_AHEAD={mode})")
        _assert_bits(alpha, want["alpha"], f"alpha (MLPSP_F32_AHEAD={mode})")
        counters = torch.zeros(4, dtype=torch.int64, device=device)
        rgb, alpha, _ = ops.render_tilecenter_f32(*args, counters=counters)
        _assert_bits(rgb, want["rgb"], f"rgb with counters (MLPSP_F32_AHEAD={mode})")
        if tile == 8:      # steps with a hit and hits (the culled entries the oracle also walks through never hit)
            np.testing.assert_array_equal(counters.cpu().numpy()[2:], want["stats"][2:])
    assert want["alpha"].mean() > 0.3


def test_non_finite_activations_take_the_same_path_in_both_f32_evaluations(device, oracle_mod, monkeypatch):
    """Huge and non-finite weights of a few primitives (inf - inf, NaN through a ReLU, overflow to inf) must
    give the oracle's image -- NaN positions included -- from the matrix-core and the scalar kernel."""
    fr = Frame("cfg1_5k_160x120", n=1200, width=64, height=48)
    sc = fr.scene
    cand, off = fr.oracle_lists(oracle_mod)
    t = int(np.argmax(np.diff(off)))
    ids = [int(v) for v in dict.fromkeys(cand[off[t]:off[t + 1]].tolist())][:6]     # primitives of the fullest tile
    W1, b1, W2, b2, W3, b3 = [w.copy() for w in sc.mlp()]
    W1[ids[0], 5, :] = 3e38
    W1[ids[0], 6, :] = -3e38
    b1[ids[1], 0] = np.nan
    W2[ids[2], 2, 3] = np.inf
    W2[ids[3], :, :] = 1e30
    W3[ids[4], 3, :] = -np.inf
    W3[ids[5], 0, 7] = np.nan
    sc.W1, sc.b1, sc.W2, sc.b2, sc.W3, sc.b3 = W1, b1, W2, b2, W3, b3
    weights = sc.mlp()
    want = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims)
    from mlp_splatting_amd import ops
    rec = ops.prepare_primitives(_t(sc.positions, device), _t(sc.log_scales, device), _t(sc.quats, device))
    ro, rd, c, o = _t(fr.rays_o, device), _t(fr.rays_d, device), _t(cand, device), _t(off, device)
    order, _ = ops.sort_tiles(ro, rd, rec, c, o, fr.W, fr.H, fr.tile, fr.tile)
    outs = []
    for scalar in (False, True):
        if scalar:
            monkeypatch.setenv("MLPSP_F32_SCALAR", "1")
        rgb, alpha, _ = ops.render_tilecenter_f32(ro, rd, rec, order, o, _t(sc.freq, device), _t(sc.att, device),
                                                  *[_t(w, device) for w in weights], fr.W, fr.H, fr.tile, fr.tile, fr.thr)
        outs.append((rgb.cpu().numpy(), alpha.cpu().numpy()))
    monkeypatch.delenv("MLPSP_F32_SCALAR")
    nan_a, nan_b = np.isnan(outs[0][0]), np.isnan(outs[1][0])
    np.testing.assert_array_equal(nan_a, nan_b)
    assert np.array_equal(bits(outs[0][0])[~nan_a], bits(outs[1][0])[~nan_b])
    assert np.array_equal(bits(outs[0][1])[~np.isnan(outs[0][1])], bits(outs[1][1])[~np.isnan(outs[1][1])])
    assert (~nan_a).mean() > 0.5 and nan_a.any()
    np.testing.assert_array_equal(np.isnan(want["rgb"]), nan_a)
    assert np.array_equal(bits(want["rgb"])[~nan_a], bits(outs[0][0])[~nan_a])


def test_expected_depth_render_is_bit_exact(device, oracle_mod, frame1):
    fr = frame1
    cand, off = fr.lists
    want = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims, family=2, with_t=True)
    rgb, alpha, t, _ = _render_gpu(fr, device, cand, off, family=2, with_t=True)
    _assert_bits(rgb, want["rgb"], "rgb")
    _assert_bits(t, want["t"], "t")
    assert float(t.max()) > 0.5


@pytest.mark.parametrize("hidden,freqs,tile,width,height", [(32, 6, 8, 72, 40), (32, 6, 16, 72, 40), (16, 6, 8, 50, 30),
                                                            (7, 3, 8, 40, 24), (1, 1, 4, 20, 12), (32, 6, 1, 12, 6)])
def test_render_shapes_tiles_and_ragged_edges(device, oracle_mod, hidden, freqs, tile, width, height):
    from mlp_splatting_amd import synthetic as syn
    fr = Frame("cfg1_5k_160x120", n=1500, width=width, height=height, tile=tile, hidden=hidden)
    if freqs != 6:
        fr.scene = syn.make_scene(1500, hidden, 0, -3.0, num_frequencies=freqs)
    cand, off = fr.oracle_lists(oracle_mod)
    want = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims)
    rgb, alpha, _, _ = _render_gpu(fr, device, cand, off)
    assert want["alpha"].max() > 0.3
    _assert_bits(rgb, want["rgb"], "rgb")
    _assert_bits(alpha, want["alpha"], "alpha")


def test_tilecentre_render_is_bit_exact_config2(device, oracle_mod):
    # 50k primitives, 640x480: tile-list counts, order and the image, all bit-exact
    from mlp_splatting_amd import ops
    fr = Frame("cfg2_50k_640x480")
    sc = fr.scene
    want_lists = fr.oracle_lists(oracle_mod)
    cand, off = ops.bin_legacy(_t(sc.positions, device), _t(sc.log_scales, device), torch.from_numpy(fr.view)[None],
                               torch.from_numpy(fr.proj), fr.W, fr.H, 8, fr.thr)
    np.testing.assert_array_equal(off.cpu().numpy(), want_lists[1])
    np.testing.assert_array_equal(cand.cpu().numpy(), want_lists[0])
    assert 1000 < np.diff(want_lists[1]).max() <= 1536
    rec = ops.prepare_primitives(_t(sc.positions, device), _t(sc.log_scales, device), _t(sc.quats, device))
    ids, keys = ops.sort_tiles(_t(fr.rays_o, device), _t(fr.rays_d, device), rec, cand, off, fr.W, fr.H, 8, 8, want_keys=True)
    want_ids, want_keys = oracle_mod.sort_tiles(fr.rays_o, fr.rays_d, sc.positions, sc.log_scales, sc.quats, *want_lists,
                                                fr.W, fr.H, 8, 8)
    np.testing.assert_array_equal(ids.cpu().numpy(), want_ids)
    _assert_bits(keys, want_keys, "keys")
    want = oracle_mod.render_tilecenter(*fr.base_numpy(*want_lists), *fr.dims)
    rgb, alpha, _, counters = _render_gpu(fr, device, *want_lists)
    _assert_bits(rgb, want["rgb"], "rgb")
    _assert_bits(alpha, want["alpha"], "alpha")
    np.testing.assert_array_equal(counters[1:], want["stats"][1:])


@pytest.mark.parametrize("slots,channels", [(4, 20), (5, 8), (1, 12), (4, 512), (4, 130)])
def test_feature_render_is_bit_exact(device, oracle_mod, slots, channels):
    from mlp_splatting_amd import ops
    fr = Frame("cfg1_5k_160x120", n=900, width=48, height=32, feature_dim=channels, feature_slots=slots if slots > 1 else 4)
    sc = fr.scene
    fa = sc.feat_attr if slots > 1 else np.ascontiguousarray(sc.feat_attr[:, 0])
    cand, off = fr.oracle_lists(oracle_mod)
    want = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims, feat_attr=fa, beta=1.3, temp=2.2)
    rec = ops.prepare_primitives(_t(sc.positions, device), _t(sc.log_scales, device), _t(sc.quats, device))
    ro, rd, c, o = _t(fr.rays_o, device), _t(fr.rays_d, device), _t(cand, device), _t(off, device)
    order, _ = ops.sort_tiles(ro, rd, rec, c, o, fr.W, fr.H, 8, 8)
    rgb, alpha, feat = ops.render_tilecenter_feat_f32(ro, rd, rec, order, o, _t(sc.freq, device), _t(sc.att, device),
                                                      *[_t(w, device) for w in sc.mlp()], _t(fa, device), 1.3, 2.2,
                                                      fr.W, fr.H, 8, 8, fr.thr)
    assert np.abs(want["feat"]).max() > 1e-3
    _assert_bits(rgb, want["rgb"], "rgb")
    _assert_bits(alpha, want["alpha"], "alpha")
    _assert_bits(feat, want["feat"], "feat")


@pytest.mark.parametrize("with_feat", [False, True])
def test_per_pixel_render_is_bit_exact(device, oracle_mod, with_feat):
    from mlp_splatting_amd import ops
    fr = Frame("cfg1_5k_160x120", n=1200, width=56, height=40, feature_dim=24 if with_feat else 0)
    sc = fr.scene
    cand, off = fr.oracle_lists(oracle_mod)
    want = oracle_mod.render_per_pixel(*fr.base_numpy(cand, off), *fr.dims, feat_attr=sc.feat_attr)
    assert not want["overflow"] and want["alpha"].max() > 0.3
    rec = ops.prepare_primitives(_t(sc.positions, device), _t(sc.log_scales, device), _t(sc.quats, device))
    rgb, alpha, feat = ops.render_per_pixel_f32(
        _t(fr.rays_o, device), _t(fr.rays_d, device), rec, _t(cand, device), _t(off, device), _t(sc.freq, device),
        _t(sc.att, device), *[_t(w, device) for w in sc.mlp()], fr.W, fr.H, 8, 8, fr.thr, "test",
        feat_attr=_t(sc.feat_attr, device) if with_feat else None)
    _assert_bits(rgb, want["rgb"], "rgb")
    _assert_bits(alpha, want["alpha"], "alpha")
    if with_feat:
        _assert_bits(feat, want["feat"], "feat")
    # per-pixel and tile-centre orders differ on real scenes: the two oracles must not coincide here
    tc = oracle_mod.render_tilecenter(*fr.base_numpy(cand, off), *fr.dims)
    assert np.abs(tc["rgb"] - want["rgb"]).max() > 1e-4


@pytest.mark.parametrize("tile,hidden,n,size,seed,eye", [
    (8, 32, 1200, (56, 40), 0, (0.3, -0.2, -0.5)), (16, 16, 900, (50, 30), 0, (0.3, -0.2, -0.5)),
    (8, 7, 700, (33, 17), 0, (0.3, -0.2, -0.5)), (4, 32, 500, (21, 13), 0, (0.3, -0.2, -0.5)),
    (8, 32, 2500, (64, 48), 3, (1.0, 0.8, -1.2)), (8, 16, 1800, (40, 56), 7, (-0.7, 0.4, 0.9)),
    (16, 32, 1500, (47, 33), 11, (0.1, 0.1, -0.2))])
def test_per_pixel_records_are_bit_exact(device, oracle_mod, tile, hidden, n, size, seed, eye):
    """mlpsp_records_per_pixel_count / _emit against the oracle's records_per_pixel: counts, offsets, every record
    field and the image, to the bit."""
    from mlp_splatting_amd.tile_ext import TileExt
    fr = Frame("cfg1_5k_160x120", n=n, hidden=hidden, width=size[0], height=size[1], tile=tile, seed=seed, eye=eye,
               target=(0.0, 0.0, 0.4) if seed == 0 else (0.0, 0.0, 0.0))
    cand, off = fr.oracle_lists(oracle_mod)
    want = oracle_mod.records_per_pixel(*fr.base_numpy(cand, off), *fr.dims, beta=1.3, temp=2.2)
    assert not want["overflow"] and want["offsets"][-1] > 300
    ext = TileExt()
    base = fr.base_torch(cand, off, device)
    counts = ext.render_tiles_backward_count_per_pixel(*base, fr.W, fr.H, tile, tile, fr.thr)
    assert counts.dtype == torch.int32
    np.testing.assert_array_equal(counts.cpu().numpy(), np.diff(want["offsets"]))
    rgb, alpha, ids, x6, raw, masks, gates, offsets = ext.render_tiles_per_pixel_records(base, fr.W, fr.H, tile, tile,
                                                                                         fr.thr, 1.3, 2.2)
    np.testing.assert_array_equal(offsets.cpu().numpy(), want["offsets"])
    np.testing.assert_array_equal(ids.cpu().numpy(), want["ids"])
    np.testing.assert_array_equal(masks.cpu().numpy(), want["masks"])
    for got, key in ((x6, "x6"), (raw, "raw"), (gates, "gates"), (rgb, "rgb"), (alpha, "alpha")):
        _assert_bits(got, want[key], key)
    # the order differs from the tile-centre records on a real frame
    tc = oracle_mod.records(*fr.base_numpy(cand, off), *fr.dims, max_hits=512)
    assert tile == 4 or not (len(tc["ids"]) == len(want["ids"]) and np.array_equal(tc["ids"], want["ids"]))


def test_per_pixel_records_refuse_a_257th_hit(device):
    from mlp_splatting_amd.tile_ext import TileExt
    from test_gpu_contract import _renderer_inputs, _base
    ext = TileExt()
    d = _renderer_inputs(257, device)
    with pytest.raises(RuntimeError, match="per-pixel intersection capacity 256 exceeded"):
        ext.render_tiles_backward_count_per_pixel(*_base(d), 1, 1, 1, 1, 0.005)
    ok = ext.render_tiles_backward_count_per_pixel(*_base(_renderer_inputs(256, device)), 1, 1, 1, 1, 0.005)
    assert 0 < int(ok[0]) <= 256


@pytest.mark.parametrize("tile,hidden", [(8, 32), (16, 16), (8, 8)])
def test_statistics_forward_against_oracle(device, oracle_mod, tile, hidden):
    # np_tile_kernels.cu:2139-2519.  Image bit-exact; integer statistics and the maximum exact; the two
    # float sums are reductions in an unspecified order (wavefront shuffles + atomics here, block
    # reduce + atomics in the reference): relative 1e-5 against the oracle's double-precision sums.
    from mlp_splatting_amd import ops
    fr = Frame("cfg1_5k_160x120", n=2500, hidden=hidden, width=72, height=48, tile=tile)
    sc = fr.scene
    cand, off = fr.oracle_lists(oracle_mod)
    gt = np.random.default_rng(5).random((fr.W * fr.H, 3), dtype=np.float32)
    want = oracle_mod.render_stats(*fr.base_numpy(cand, off), *fr.dims, gt)
    rec = ops.prepare_primitives(_t(sc.positions, device), _t(sc.log_scales, device), _t(sc.quats, device))
    ro, rd, c, o = _t(fr.rays_o, device), _t(fr.rays_d, device), _t(cand, device), _t(off, device)
    order, _ = ops.sort_tiles(ro, rd, rec, c, o, fr.W, fr.H, tile, tile, family=2, cull_threshold=fr.thr)
    n = sc.n
    st = [torch.zeros(n, device=device, dtype=dt) for dt in (torch.float32, torch.float32, torch.int32, torch.float32, torch.int32)]
    args = (ro, rd, rec, order, o, _t(sc.freq, device), _t(sc.att, device), *[_t(w, device) for w in sc.mlp()],
            fr.W, fr.H, tile, tile, fr.thr, _t(gt, device))
    rgb, alpha = ops.render_tilecenter_stats_f32(*args, *st)
    _assert_bits(rgb, want["rgb"], "rgb")
    _assert_bits(alpha, want["alpha"], "alpha")
    sum_w, max_w, hits, sum_werr, contrib = (t.cpu().numpy() for t in st)
    assert np.array_equal(hits, want["hits"]) and np.array_equal(contrib, want["contrib"])
    assert np.array_equal(max_w, want["max_w"].astype(np.float32)) and want["contrib"].sum() > 50
    np.testing.assert_allclose(sum_w, want["sum_w"], rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(sum_werr, want["sum_werr"], rtol=1e-5, atol=1e-7)
    # a second frame accumulates: sums and counts double, the maximum stays
    ops.render_tilecenter_stats_f32(*args, *st)
    assert np.array_equal(st[2].cpu().numpy(), 2 * want["hits"]) and np.array_equal(st[1].cpu().numpy(), max_w)
    np.testing.assert_allclose(st[0].cpu().numpy(), 2 * want["sum_w"], rtol=1e-5, atol=1e-7)
    # the two optional buffers may be absent
    st2 = [torch.zeros(n, device=device, dtype=dt) for dt in (torch.float32, torch.float32, torch.int32)]
    ops.render_tilecenter_stats_f32(*args, *st2)
    assert np.array_equal(st2[2].cpu().numpy(), want["hits"])


@pytest.mark.parametrize("tile,hidden,n,size", [(8, 32, 1500, (72, 48)), (16, 16, 2500, (72, 48)), (8, 8, 900, (72, 48)),
                                                (16, 32, 2000, (72, 48)), (8, 32, 1500, (69, 43)), (16, 32, 1200, (37, 50))])
def test_training_records_are_bit_exact(device, oracle_mod, tile, hidden, n, size):
    # np_tile_kernels.cu:2925-3206 (record modes 1/3): counts, order, every record field, rgb, alpha; 8x8 and 16x16
    # tiles, scalar and matrix-core MLP (the latter stages its records in LDS before writing them), image sizes that
    # are and are not multiples of the tile
    from mlp_splatting_amd.tile_ext import TileExt
    fr = Frame("cfg1_5k_160x120", n=n, hidden=hidden, width=size[0], height=size[1], tile=tile)
    cand, off = fr.oracle_lists(oracle_mod)
    want = oracle_mod.records(*fr.base_numpy(cand, off), *fr.dims, max_hits=512, beta=1.3, temp=2.2)
    x = [_t(a, device) for a in fr.base_numpy(cand, off)]
    x += [torch.zeros_like(x[0]), torch.zeros(fr.W * fr.H, device=device)]
    ext = TileExt()
    rgb, alpha, ids, x6, raw, masks, gates, offsets = ext.render_tiles_training_records(x, fr.W, fr.H, tile, fr.thr, 1.3, 2.2)
    assert offsets.dtype == torch.int64 and np.array_equal(offsets.cpu().numpy(), want["offsets"])
    assert want["offsets"][-1] > 3000 and np.array_equal(ids.cpu().numpy(), want["ids"])
    assert np.array_equal(masks.cpu().numpy(), want["masks"])
    for got, key in ((rgb, "rgb"), (alpha, "alpha"), (x6, "x6"), (raw, "raw"), (gates, "gates")):
        _assert_bits(got, want[key], key)
    # primitive-major grouping of those records (scannet/primitive_csr.py:14-29)
    from mlp_splatting_amd.primitive_csr import group_records
    csr = group_records(ids, x6, raw[:, :4].contiguous(), fr.scene.n, masks)
    counts = np.bincount(want["ids"], minlength=fr.scene.n)
    assert np.array_equal(np.diff(csr.offsets.cpu().numpy()), counts)
    order = csr.record_indices.cpu().numpy()
    assert np.array_equal(want["ids"][order], np.sort(want["ids"], kind="stable"))
    assert np.array_equal(order, np.argsort(want["ids"], kind="stable"))


def test_training_records_hit_capacity_is_an_error(device, oracle_mod):
    from mlp_splatting_amd.tile_ext import TileExt
    fr = Frame("cfg1_5k_160x120", n=1500, hidden=32, width=32, height=24)
    cand, off = fr.oracle_lists(oracle_mod)
    want = oracle_mod.records(*fr.base_numpy(cand, off), *fr.dims, max_hits=512)
    deepest = int(np.diff(want["offsets"]).max())
    assert deepest > 8
    x = [_t(a, device) for a in fr.base_numpy(cand, off)]
    x += [torch.zeros_like(x[0]), torch.zeros(fr.W * fr.H, device=device)]
    assert oracle_mod.records(*fr.base_numpy(cand, off), *fr.dims, max_hits=deepest - 1)["overflow"]
    with pytest.raises(RuntimeError, match=f"hit capacity {deepest - 1} reached before transmittance termination"):
        TileExt(max_hits=deepest - 1).render_tiles_training_records(x, fr.W, fr.H, 8, fr.thr, 1.5, 2.0)
    # empty lists: empty records, zero image
    x[5], x[6] = torch.zeros(0, dtype=torch.int32, device=device), torch.zeros_like(x[6])
    out = TileExt().render_tiles_training_records(x, fr.W, fr.H, 8, fr.thr, 1.5, 2.0)
    assert out[2].numel() == 0 and int(out[7][-1]) == 0 and float(out[0].abs().max()) == 0.0


def test_async_binning_with_device_matrices_equals_host_matrices(device, oracle_mod):
    """The asynchronous binning takes one view's matrices from the host or straight from device tensors (what the
    reference's evaluators hold); lists and counts are the same bits, and equal the oracle's."""
    from mlp_splatting_amd import ops
    fr = Frame("cfg1_5k_160x120", n=3000, width=104, height=72, eye=(0.4, 0.1, -0.7))
    sc = fr.scene
    pos, logs = _t(sc.positions, device), _t(sc.log_scales, device)
    view_host, proj_host = torch.from_numpy(fr.view), torch.from_numpy(fr.proj)
    want_cand, want_off = fr.oracle_lists(oracle_mod)
    results = []
    for view, proj in ((view_host[None], proj_host), (view_host.to(device), proj_host.to(device))):
        cand, off, counts = ops.bin_legacy_async(pos, logs, view, proj, fr.W, fr.H, 8, fr.thr, want_cand.size + 100)
        pairs, longest, _, guard = counts.tolist()
        assert guard == 0 and pairs == want_cand.size
        results.append((cand[:pairs].cpu().numpy(), off.cpu().numpy(), longest))
    for cand, off, longest in results:
        np.testing.assert_array_equal(off, want_off)
        np.testing.assert_array_equal(cand, want_cand)
        assert longest == int(np.diff(want_off).max())
