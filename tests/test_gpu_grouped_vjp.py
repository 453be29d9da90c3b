"""Grouped MLP weight gradients (HIP kernels behind primitive_gemm.grouped_weight_gradients) against the
per-primitive dense chain in float64, which tests/test_record_grouping.py pins to autograd.  Cases, sizes and
tolerances are those of the reference's own tests (tests/test_primitive_csr.py:98-133: f32 atol 1e-4*scale,
rtol 3e-4; relative L2 error below 0.01 for fp16 and 0.04 for bf16; tests/test_csr_safety.py:153-209)."""
import pytest
import torch

from mlp_splatting_amd import primitive_gemm as gemm
from mlp_splatting_amd.cumodel import _encode_x6
from mlp_splatting_amd.primitive_csr import group_records, reference_weight_gradients

pytestmark = pytest.mark.gpu

SHAPES = [(32, 72), (32,), (32, 32), (32,), (4, 32), (4,)]


@pytest.fixture(autouse=True)
def isolated_counters(monkeypatch):
    monkeypatch.setattr(gemm, "_SAFETY_STATS", {k: 0 for k in gemm._SAFETY_STATS})


def _float64_expected(csr, freq, att, weights):
    from types import SimpleNamespace
    c = SimpleNamespace(offsets=csr.offsets.cpu(), x6=csr.x6.double().cpu(), grad4=csr.grad4.double().cpu())
    return reference_weight_gradients(c, freq.double().cpu(), att.double().cpu(), [w.double().cpu() for w in weights])


def _saved_masks(csr, freq, att, weights):
    """The exact f32 activation masks a record emitter would have saved."""
    masks = torch.zeros((len(csr.x6), 2), device=csr.x6.device, dtype=torch.int32)
    bit = 1 << torch.arange(32, device=csr.x6.device, dtype=torch.int64)
    for p in range(len(weights[0])):
        lo, hi = map(int, csr.offsets[p:p + 2])
        if lo == hi:
            continue
        enc = _encode_x6(csr.x6[lo:hi], freq, att)
        h1 = torch.relu(enc @ weights[0][p].T + weights[1][p])
        h2 = torch.relu(h1 @ weights[2][p].T + weights[3][p])
        masks[lo:hi, 0] = ((h1 > 0) * bit).sum(1).to(torch.int32)
        masks[lo:hi, 1] = ((h2 > 0) * bit).sum(1).to(torch.int32)
    return masks


def _case(device, scale, seed=92):
    torch.manual_seed(seed)
    counts = torch.tensor([0, 1, 31, 32, 33, 511, 512, 513, 1700, 0], device=device)
    ids = torch.repeat_interleave(torch.arange(10, device=device, dtype=torch.int32), counts)
    ids = ids[torch.randperm(ids.numel(), device=device)]
    x6 = torch.randn((len(ids), 6), device=device) * 0.2
    d3 = torch.randn((len(ids), 4), device=device) * scale
    csr = group_records(ids, x6, d3, 10)
    freq = 2.0 ** torch.arange(6, device=device, dtype=torch.float32)
    att = torch.exp(-0.5 * freq.square() * 1e-4)
    weights = [torch.randn((10, *shape), device=device) * 0.1 for shape in SHAPES]
    return csr, freq, att, weights


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("scale", [1.0, 1e-6])
@pytest.mark.parametrize("saved_masks", [True, False])
def test_grouped_vjp_matches_the_dense_chain(device, dtype, scale, saved_masks):
    csr, freq, att, weights = _case(device, scale)
    if saved_masks:
        csr.relu_masks = _saved_masks(csr, freq, att, weights)
    expected = _float64_expected(csr, freq, att, weights)
    actual = gemm.grouped_weight_gradients(csr, freq, att, weights, dtype=dtype)
    for a, b, w in zip(actual, expected, weights):
        assert a.shape == w.shape and a.dtype == torch.float32 and bool(torch.isfinite(a).all())
        a = a.double().cpu()
        if dtype == torch.float32:
            torch.testing.assert_close(a, b, atol=1e-4 * scale, rtol=3e-4)
        else:
            # without saved masks the 16-bit forward pass decides which units are active, and units whose
            # pre-activation is within rounding of zero flip against the exact chain: the reference states no
            # tolerance for that mode, five times the saved-mask one is what is asserted here
            rel = (a - b).norm() / b.norm().clamp_min(1e-30)
            limit = (0.01 if dtype == torch.float16 else 0.04) * (1.0 if saved_masks else 5.0)
            assert float(rel) < limit, float(rel)
    for empty in (0, 9):
        assert all(bool((g[empty] == 0).all()) for g in actual)
    assert gemm.get_grouped_vjp_safety_stats()["fp32_fallbacks"] == 0


@pytest.mark.parametrize("segment_size,block_size", [(32, 32), (64, 64), (512, 32), (2048, 64)])
def test_segment_size_only_changes_the_summation_order(device, segment_size, block_size):
    csr, freq, att, weights = _case(device, 1.0, seed=5)
    expected = _float64_expected(csr, freq, att, weights)
    actual = gemm.grouped_weight_gradients(csr, freq, att, weights, dtype=torch.float32, segment_size=segment_size,
                                           block_size=block_size)
    for a, b in zip(actual, expected):
        torch.testing.assert_close(a.double().cpu(), b, atol=1e-4, rtol=3e-4)


def test_gradients_of_real_training_records(device, oracle_mod):
    """Records emitted by the training-records forward (ids, x6, ReLU masks), grouped and differentiated."""
    from helpers import Frame
    from mlp_splatting_amd.tile_ext import TileExt
    from conftest import to_dev
    fr = Frame("cfg1_5k_160x120", n=400, width=64, height=48, hidden=32)
    sc = fr.scene
    cand, off = fr.oracle_lists(oracle_mod)
    t = lambda a: to_dev(a, device)
    ext = TileExt()
    args = [t(a) for a in fr.base_numpy(cand, off)]
    args += [torch.zeros_like(args[0]), torch.zeros(fr.W * fr.H, device=device)]
    out = ext.render_tiles_training_records(args, fr.W, fr.H, fr.tile, fr.thr, 1.5, 2.0)
    rgb, alpha, ids, x6, raw, masks, gates, pixel_offsets = out
    assert ids.numel() > 1000
    torch.manual_seed(3)
    grad4 = torch.randn((ids.numel(), 4), device=device)
    csr = group_records(ids, x6, grad4, sc.n, masks)
    weights = [t(w) for w in sc.mlp()]
    expected = _float64_expected(csr, t(sc.freq), t(sc.att), weights)
    for dtype in (torch.float32, torch.float16):
        actual = gemm.grouped_weight_gradients(csr, t(sc.freq), t(sc.att), weights, dtype=dtype)
        for a, b in zip(actual, expected):
            a = a.double().cpu()
            if dtype == torch.float32:
                torch.testing.assert_close(a, b, atol=5e-4, rtol=5e-4)
            else:
                assert float((a - b).norm() / b.norm().clamp_min(1e-30)) < 0.003


# ---- the safety policy on real kernels (tests/test_csr_safety.py:153-209)

@pytest.fixture
def vjp_inputs(device):
    counts = torch.tensor([33, 0, 513], dtype=torch.int64, device=device)
    from types import SimpleNamespace
    offsets = torch.cat((counts.new_zeros(1), counts.cumsum(0)))
    n = int(offsets[-1])
    csr = SimpleNamespace(offsets=offsets, x6=torch.zeros(n, 6, device=device), grad4=torch.ones(n, 4, device=device),
                          relu_masks=torch.full((n, 2), -1, device=device, dtype=torch.int32))
    freq = 2.0 ** torch.arange(6, device=device, dtype=torch.float32)
    weights = [torch.full((3, *shape), 0.01, device=device) for shape in SHAPES]
    return csr, freq, torch.ones_like(freq), weights


def test_finite_flag_does_not_change_a_finite_result(vjp_inputs):
    csr, freq, att, weights = vjp_inputs
    groups = gemm.prepare_groups(csr)
    raw, flag = gemm._launch_grouped_vjp(csr, freq, att, weights, groups, torch.float16, 32, 4096.0)
    actual = gemm.grouped_weight_gradients(csr, freq, att, weights, groups=groups)
    assert int(flag) == 0
    expected = [v.reshape(w.shape).contiguous() for v, w in zip(raw.split([2304, 32, 1024, 32, 128, 4], dim=1), weights)]
    assert all(torch.equal(a, b) for a, b in zip(actual, expected))
    assert gemm.get_grouped_vjp_safety_stats()["fp32_fallbacks"] == 0


def test_fp16_overflow_falls_back_to_exact_fp32(vjp_inputs):
    csr, freq, att, weights = vjp_inputs
    csr.grad4.fill_(20.0)       # finite in f32, overflows only after the default fp16 scaling by 4096
    before = [w.clone() for w in weights]
    expected = gemm.grouped_weight_gradients(csr, freq, att, weights, dtype=torch.float32)
    with pytest.warns(RuntimeWarning, match="retrying with IEEE FP32 before Adam"):
        actual = gemm.grouped_weight_gradients(csr, freq, att, weights, dtype=torch.float16)
    assert all(torch.equal(a, b) for a, b in zip(actual, expected))
    assert all(torch.equal(a, b) for a, b in zip(weights, before))
    assert all(bool(torch.isfinite(g).all()) for g in actual)
    assert gemm.get_grouped_vjp_safety_stats()["fp32_fallbacks"] == 1


def test_non_finite_fp32_gradients_fail_closed(vjp_inputs):
    csr, freq, att, weights = vjp_inputs
    csr.grad4[0, 0] = float("nan")
    with pytest.raises(FloatingPointError, match="Adam must not step"):
        gemm.grouped_weight_gradients(csr, freq, att, weights, dtype=torch.float32)


@pytest.mark.parametrize("invalid_scale", [0, -1, float("inf"), float("nan")])
def test_invalid_loss_scale_is_rejected(vjp_inputs, invalid_scale):
    csr, freq, att, weights = vjp_inputs
    with pytest.raises(ValueError, match="finite and strictly positive"):
        gemm.grouped_weight_gradients(csr, freq, att, weights, loss_scale=invalid_scale)


def test_c_abi_rejects_bad_arguments(device):
    from mlp_splatting_amd import _lib
    lib = _lib.load()
    buf = torch.zeros(8192, device=device)
    i64 = torch.zeros(8, dtype=torch.int64, device=device)
    p, q = buf.data_ptr(), i64.data_ptr()
    ok = lambda **kw: lib.mlpsp_grouped_vjp(p, p, None, q, q, q, kw.get("groups", 1), p, p, p, p, p, p, p,
                                            kw.get("precision", 0), kw.get("scale", 1.0), kw.get("segment", 512), p, None)
    assert ok(segment=500) != 0 and ok(segment=0) != 0 and ok(precision=3) != 0 and ok(scale=0.0) != 0
    assert ok(groups=-1) != 0
    assert ok(groups=0) == 0
    torch.cuda.synchronize()


@pytest.mark.parametrize("counts", [
    [0, 1, 31, 32, 33, 0, 64, 100, 1, 0],          # runs that start/end on, before and after chunk boundaries
    [32, 32, 32],                                  # every primitive is exactly one chunk
    [5] * 40,                                      # several whole primitives per chunk, some straddling
    [0, 0, 700, 0, 3],                             # one primitive over 22 chunks
    [0, 0, 0],                                     # no segment at all
    [1],
])
def test_segment_sums_per_primitive(device, counts):
    """mlpsp_reduce_partials / _split: chunked two-pass sums against a float64 index_add, and the non-finite flag."""
    from mlp_splatting_amd import _lib
    lib = _lib.load()
    n, total = len(counts), sum(counts)
    counts_t = torch.tensor(counts, dtype=torch.int64, device=device)
    owners = torch.repeat_interleave(torch.arange(n, device=device), counts_t)
    offsets = torch.cat((counts_t.new_zeros(1), counts_t.cumsum(0)))
    rows = int(lib.mlpsp_segment_reduce_rows(total))
    assert rows == total + 2 * ((total + 31) // 32)
    torch.manual_seed(len(counts) + total)
    partial = torch.full((max(rows, 1), 3524), float("nan"), device=device)       # the scratch rows start as garbage
    partial[:total] = torch.randn(total, 3524, device=device)
    expected = torch.zeros(n, 3524, dtype=torch.float64, device=device).index_add_(0, owners, partial[:total].double())
    stream = torch.cuda.current_stream(device).cuda_stream
    packed = torch.full((n, 3524), float("nan"), device=device)
    flag = torch.ones(1, dtype=torch.int32, device=device)
    assert lib.mlpsp_reduce_partials(partial.data_ptr(), owners.data_ptr(), offsets.data_ptr(), total, n, packed.data_ptr(),
                                     flag.data_ptr(), stream) == 0
    assert int(flag) == 0
    torch.testing.assert_close(packed.double(), expected, atol=2e-5, rtol=1e-5)
    parts = [torch.full((n, *shape), float("nan"), device=device) for shape in SHAPES]
    assert lib.mlpsp_reduce_partials_split(partial.data_ptr(), owners.data_ptr(), offsets.data_ptr(), total, n,
                                           *[t.data_ptr() for t in parts], flag.data_ptr(), stream) == 0
    assert int(flag) == 0
    assert torch.equal(torch.cat([t.reshape(n, -1) for t in parts], dim=1), packed)
    if total:
        partial[total // 2, 1234] = float("inf")
        assert lib.mlpsp_reduce_partials(partial.data_ptr(), owners.data_ptr(), offsets.data_ptr(), total, n,
                                         packed.data_ptr(), flag.data_ptr(), stream) == 0
        assert int(flag) == 1
