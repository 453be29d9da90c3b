"""Host logic kept from the reference's record/gradient helpers (scannet/primitive_csr.py,
scannet/primitive_gemm.py): grouping, segment layout guards and the non-finite retry policy, as its CPU
tests state them (tests/test_csr_safety.py:24-151)."""
from types import SimpleNamespace

import pytest
import torch

from mlp_splatting_amd import primitive_gemm as gemm
from mlp_splatting_amd.primitive_csr import group_records, reference_weight_gradients


@pytest.fixture(autouse=True)
def isolated_counters(monkeypatch):
    monkeypatch.setattr(gemm, "_SAFETY_STATS", {k: 0 for k in gemm._SAFETY_STATS})


def _csr(counts):
    counts = torch.tensor(counts, dtype=torch.int64)
    offsets = torch.cat((counts.new_zeros(1), counts.cumsum(0)))
    n = int(offsets[-1])
    return SimpleNamespace(offsets=offsets, x6=torch.zeros(n, 6), grad4=torch.ones(n, 4), relu_masks=None)


def test_group_records_is_stable_and_offsets_are_exclusive_sums():
    ids = torch.tensor([2, 0, 2, 1, 0, 2], dtype=torch.int32)
    x6 = torch.arange(36, dtype=torch.float32).view(6, 6)
    g4 = torch.arange(24, dtype=torch.float32).view(6, 4)
    csr = group_records(ids, x6, g4, 4)
    assert csr.offsets.tolist() == [0, 2, 3, 6, 6]
    assert csr.record_indices.tolist() == [1, 4, 3, 0, 2, 5]      # original order kept inside each primitive
    assert torch.equal(csr.x6, x6[csr.record_indices]) and torch.equal(csr.grad4, g4[csr.record_indices])
    assert csr.relu_masks is None


def test_reference_weight_gradients_match_autograd():
    torch.manual_seed(0)
    n, m = 3, 20
    ws = [torch.randn(n, 32, 72) * 0.1, torch.randn(n, 32) * 0.1, torch.randn(n, 32, 32) * 0.1, torch.randn(n, 32) * 0.1,
          torch.randn(n, 4, 32) * 0.1, torch.randn(n, 4) * 0.1]
    ids = torch.randint(0, n, (m,), dtype=torch.int32)
    x6, g4 = torch.randn(m, 6) * 0.3, torch.randn(m, 4)
    freq, att = 2.0 ** torch.arange(6) * torch.pi, torch.ones(6)
    csr = group_records(ids, x6, g4, n)
    got = reference_weight_gradients(csr, freq, att, ws)
    from mlp_splatting_amd.cumodel import _encode_x6
    leaves = [w.clone().requires_grad_(True) for w in ws]
    enc = _encode_x6(x6, freq, att)
    idx = ids.long()
    h1 = torch.relu(torch.einsum("mhi,mi->mh", leaves[0][idx], enc) + leaves[1][idx])
    h2 = torch.relu(torch.einsum("moh,mh->mo", leaves[2][idx], h1) + leaves[3][idx])
    out = torch.einsum("moh,mh->mo", leaves[4][idx], h2) + leaves[5][idx]
    (out * g4).sum().backward()
    for a, b in zip(got, leaves):
        torch.testing.assert_close(a, b.grad, rtol=1e-4, atol=1e-5)


def test_group_layout_carries_exact_segment_boundaries():
    counts = [0, 1, 511, 512, 513, 1024]
    csr = _csr(counts)
    groups = gemm.prepare_groups(csr, 512)
    prims, starts, base = [], [], 0
    for p, c in enumerate(counts):
        for local in range(0, c, 512):
            prims.append(p)
            starts.append(base + local)
        base += c
    assert groups.segment_size == 512 and groups.primitives.tolist() == prims and groups.starts.tolist() == starts
    assert groups.offsets.tolist() == [0, 0, 1, 2, 3, 5, 7]
    assert gemm.resolve_groups(csr, 512, groups) is groups
    assert [t is u for t, u in zip(tuple(groups), (groups.primitives, groups.starts, groups.offsets))] == [True] * 3


def test_group_layout_guards():
    csr = _csr([513])
    groups = gemm.prepare_groups(csr, 512)
    for other in (256, 1024):
        with pytest.raises(ValueError, match="Prepared groups use segment_size=512"):
            gemm.resolve_groups(csr, other, groups)
    with pytest.raises(TypeError, match="GroupLayout"):
        gemm.resolve_groups(csr, 512, tuple(groups))
    with pytest.raises(ValueError, match="different CSR"):
        gemm.resolve_groups(_csr([513]), 512, groups)
    for bad in (0, -1, 1.5, True):
        with pytest.raises(ValueError, match="positive integer"):
            gemm.prepare_groups(_csr([1]), bad)
    with pytest.raises(ValueError, match="positive integer"):
        gemm.resolve_groups(csr, 512.0, groups)


@pytest.mark.parametrize("tensor", ["source_offsets", "primitives", "starts", "offsets"])
def test_group_layout_rejects_inplace_mutation(tensor):
    csr = _csr([1, 2])
    groups = gemm.prepare_groups(csr)
    getattr(groups, tensor)[0] += 1
    with pytest.raises(ValueError, match="modified in place"):
        gemm.resolve_groups(csr, 512, groups)


def test_retry_policy():
    good = torch.tensor([1.25, -2.0])
    calls = []

    def finite(dt, s):
        calls.append((dt, s))
        return good, torch.tensor(0, dtype=torch.int32)

    assert gemm._checked_grouped_vjp(finite, torch.bfloat16, 4096.0) is good and calls == [(torch.bfloat16, 4096.0)]
    assert gemm.get_grouped_vjp_safety_stats() == {"calls": 1, "mixed_calls": 1, "fp32_fallbacks": 0,
                                                   "fp32_nonfinite_failures": 0}
    calls.clear()

    def overflow_then_ok(dt, s):
        calls.append((dt, s))
        bad = dt != torch.float32
        return (torch.tensor([float("inf")]) if bad else good), torch.tensor(int(bad), dtype=torch.int32)

    with pytest.warns(RuntimeWarning, match="retrying with IEEE FP32 before Adam"):
        assert gemm._checked_grouped_vjp(overflow_then_ok, torch.float16, 4096.0) is good
    assert calls == [(torch.float16, 4096.0), (torch.float32, 1.0)]

    def always_bad(dt, s):
        return torch.tensor([float("nan")]), torch.tensor(1, dtype=torch.int32)

    with pytest.raises(FloatingPointError, match="Adam must not step"):
        gemm._checked_grouped_vjp(always_bad, torch.float32, 1.0)
    stats = gemm.get_grouped_vjp_safety_stats(reset=True)
    assert stats["fp32_fallbacks"] == 1 and stats["fp32_nonfinite_failures"] == 1
    assert all(v == 0 for v in gemm.get_grouped_vjp_safety_stats().values())


def test_grouped_weight_gradients_validates_before_any_launch():
    ws = [torch.zeros(2, 32, 72), torch.zeros(2, 32), torch.zeros(2, 32, 32), torch.zeros(2, 32), torch.zeros(2, 4, 32),
          torch.zeros(2, 4)]
    csr = _csr([1, 2])
    f = torch.ones(6)
    with pytest.raises(ValueError, match="72→32→32→4"):
        gemm.grouped_weight_gradients(csr, f, f, [torch.zeros(2, 16, 72)] + ws[1:])
    with pytest.raises(ValueError, match="same primitive count"):
        gemm.grouped_weight_gradients(_csr([1]), f, f, ws)
    with pytest.raises(ValueError, match="six positional frequencies"):
        gemm.grouped_weight_gradients(csr, torch.ones(4), f, ws)
    with pytest.raises(ValueError, match="multiple of the 32/64-row block"):
        gemm.grouped_weight_gradients(csr, f, f, ws, segment_size=500)
    with pytest.raises(ValueError, match="one CUDA device"):
        gemm.grouped_weight_gradients(csr, f, f, ws)
    assert sum(gemm.PACKED_GRADIENT_SIZES) == 3524
