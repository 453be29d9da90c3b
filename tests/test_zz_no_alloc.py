"""mlpsp_bin_legacy_async_noalloc -- the binning whose scratch is a device array inside the library -- against
mlpsp_bin_legacy_async with a caller-provided scratch buffer, through the C ABI: tile offsets, candidate lists and
the counts word must be bit-identical, on two calls in a row of which the second is the smaller one (the array keeps
the first call's contents), for one view and for a four-view mosaic, for an empty scene, and beyond the fixed
maximum the call must refuse."""
import ctypes as C

import numpy as np
import pytest
import torch

from mlp_splatting_amd import _lib, synthetic as syn

pytestmark = pytest.mark.gpu


def _frame(n, width, height, focal, views, seed):
    poses = syn.random_poses(max(views, 1), seed)
    vm = np.stack([syn.view_matrix(p) for p in poses[:views]]).astype(np.float32)
    proj = np.asarray(syn.projection_matrix(focal, width, height), dtype=np.float32)
    if n == 0:
        empty = np.zeros((0, 3), np.float32)
        return empty, empty.copy(), np.ascontiguousarray(vm), np.ascontiguousarray(proj)
    sc = syn.make_scene(n, 16, seed=seed, log_scale_mean=-3.0)
    return sc.positions, sc.log_scales, np.ascontiguousarray(vm), np.ascontiguousarray(proj)


def _tile_views(width, height, device):
    ntx, nty = (width + 7) // 8, (height + 7) // 8
    tx, ty = np.meshgrid(np.arange(ntx), np.arange(nty))
    quadrant = (tx >= ntx // 2).astype(np.int32) + 2 * (ty >= nty // 2).astype(np.int32)
    return torch.from_numpy(np.ascontiguousarray(quadrant.reshape(-1))).to(device)


def _run(entry, device, positions, log_scales, vm, proj, width, height, thr, capacity, tile_views=None, scratch=True):
    lib = _lib.load()
    fp = C.POINTER(C.c_float)
    pos, logs = torch.from_numpy(positions).to(device), torch.from_numpy(log_scales).to(device)
    n, views = positions.shape[0], vm.shape[0]
    tiles = ((width + 7) // 8) * ((height + 7) // 8)
    offsets = torch.full((tiles + 1,), -7, dtype=torch.int32, device=device)
    cand = torch.full((capacity,), -7, dtype=torch.int32, device=device)
    counts = torch.full((4,), -7, dtype=torch.int64, device=device)
    stream = C.c_void_p(torch.cuda.current_stream(device).cuda_stream)
    ptr = lambda t: None if t is None else C.c_void_p(t.data_ptr())
    head = (ptr(pos), ptr(logs), n, C.cast(vm.ctypes.data, fp), views, ptr(tile_views), C.cast(proj.ctypes.data, fp), width,
            height, 8, float(thr))
    tail = (ptr(offsets), ptr(cand), capacity, ptr(counts), stream)
    if scratch:
        nbytes = lib.mlpsp_bin_scratch_bytes(n, views, width, height, 8)
        buf = torch.empty(nbytes, dtype=torch.uint8, device=device)
        rc = getattr(lib, entry)(*head, ptr(buf), nbytes, *tail)
    else:
        rc = getattr(lib, entry)(*head, *tail)
    torch.cuda.synchronize(device)
    return rc, offsets.cpu().numpy(), cand.cpu().numpy(), counts.cpu().numpy()


def _assert_same(device, case, capacity):
    width, height, thr, tile_views = case["width"], case["height"], case["thr"], case.get("tile_views")
    frame = _frame(case["n"], width, height, case["focal"], case["views"], case["seed"])
    want = _run("mlpsp_bin_legacy_async", device, *frame, width, height, thr, capacity, tile_views, scratch=True)
    got = _run("mlpsp_bin_legacy_async_noalloc", device, *frame, width, height, thr, capacity, tile_views, scratch=False)
    assert want[0] == 0 and got[0] == 0
    assert np.array_equal(got[3], want[3]), (got[3], want[3])                      # pairs, longest, level-1 entries, guard
    assert want[3][3] == 0 and want[3][0] > 0
    assert np.array_equal(got[1], want[1])                                         # tile offsets
    pairs = int(want[3][0])
    assert np.array_equal(got[2][:pairs], want[2][:pairs])                         # candidate lists
    assert (got[2][pairs:] == -7).all()                                            # nothing written past them
    return pairs


def test_two_calls_in_a_row_the_second_smaller(device):
    big = dict(n=50000, width=640, height=480, focal=600.0, views=1, seed=0, thr=1e-3)
    small = dict(n=3000, width=160, height=120, focal=150.0, views=1, seed=1, thr=5e-3)
    first = _assert_same(device, big, 6_000_000)
    second = _assert_same(device, small, 400_000)
    assert second < first
    third = _assert_same(device, big, 6_000_000)                                   # and back up again
    assert third == first


def test_the_call_allocates_nothing_on_the_device(device):
    """After one warm-up call (the library takes the array's address once per device), a call changes neither the
    allocator's books nor the free memory the driver reports."""
    lib = _lib.load()
    fp = C.POINTER(C.c_float)
    for views in (1, 4):
        n, width, height = 20000, 320, 240
        positions, log_scales, vm, proj = _frame(n, width, height, 300.0, views, 4)
        pos, logs = torch.from_numpy(positions).to(device), torch.from_numpy(log_scales).to(device)
        tiles = ((width + 7) // 8) * ((height + 7) // 8)
        offsets = torch.empty(tiles + 1, dtype=torch.int32, device=device)
        cand = torch.empty(4_000_000, dtype=torch.int32, device=device)
        counts = torch.empty(4, dtype=torch.int64, device=device)
        tv = _tile_views(width, height, device) if views > 1 else None
        stream = C.c_void_p(torch.cuda.current_stream(device).cuda_stream)
        ptr = lambda t: None if t is None else C.c_void_p(t.data_ptr())
        args = (ptr(pos), ptr(logs), n, C.cast(vm.ctypes.data, fp), views, ptr(tv), C.cast(proj.ctypes.data, fp), width,
                height, 8, 5e-3, ptr(offsets), ptr(cand), cand.numel(), ptr(counts), stream)
        assert lib.mlpsp_bin_legacy_async_noalloc(*args) == 0            # warm-up
        torch.cuda.synchronize(device)
        before = (torch.cuda.memory_allocated(device), torch.cuda.memory_reserved(device), torch.cuda.mem_get_info(device)[0])
        for _ in range(3):
            assert lib.mlpsp_bin_legacy_async_noalloc(*args) == 0
        torch.cuda.synchronize(device)
        after = (torch.cuda.memory_allocated(device), torch.cuda.memory_reserved(device), torch.cuda.mem_get_info(device)[0])
        assert after == before, (before, after)
        assert int(counts[3]) == 0 and int(counts[0]) > 0


def test_four_views_travel_as_kernel_arguments(device):
    case = dict(n=20000, width=320, height=240, focal=300.0, views=4, seed=2, thr=5e-3)
    case["tile_views"] = _tile_views(case["width"], case["height"], device)
    _assert_same(device, case, 4_000_000)


def test_guard_empties_the_lists_like_the_ordinary_entry_point(device):
    case = dict(n=20000, width=320, height=240, focal=300.0, views=1, seed=3, thr=1e-3)
    frame = _frame(case["n"], 320, 240, 300.0, 1, 3)
    want = _run("mlpsp_bin_legacy_async", device, *frame, 320, 240, 1e-3, 1000, None, scratch=True)
    got = _run("mlpsp_bin_legacy_async_noalloc", device, *frame, 320, 240, 1e-3, 1000, None, scratch=False)
    assert want[0] == 0 and got[0] == 0 and want[3][3] == 1
    assert np.array_equal(got[3], want[3]) and np.array_equal(got[1], want[1]) and not got[1].any()
    assert (got[2] == -7).all()


def test_empty_scene_and_refusals(device):
    lib = _lib.load()
    frame = _frame(0, 160, 120, 150.0, 1, 0)
    rc, offsets, _, counts = _run("mlpsp_bin_legacy_async_noalloc", device, *frame, 160, 120, 1e-3, 16, None, scratch=False)
    assert rc == 0 and not offsets.any() and not counts.any()
    # beyond the fixed maximum: refused before anything is launched
    assert lib.mlpsp_bin_scratch_bytes(400000, 1, 1200, 680, 8) > lib.mlpsp_bin_static_scratch_bytes()
    huge = _frame(16, 1200, 680, 600.0, 1, 0)
    pos = np.zeros((400000, 3), np.float32)
    rc, *_ = _run("mlpsp_bin_legacy_async_noalloc", device, pos, pos.copy(), huge[2], huge[3], 1200, 680, 5e-3, 16, None,
                  scratch=False)
    assert rc == _lib.E_SCRATCH
    nine = np.ascontiguousarray(np.repeat(huge[2], 9, axis=0))
    small = _frame(100, 160, 120, 150.0, 1, 0)
    rc, *_ = _run("mlpsp_bin_legacy_async_noalloc", device, small[0], small[1], nine, small[3], 160, 120, 5e-3, 16,
                  _tile_views(160, 120, device), scratch=False)
    assert rc == _lib.E_ARGUMENT
