"""Reverse compositing over saved records (HIP) against the CPU oracle, which tests/test_oracle_render.py pins
to float64 autograd.  Tolerance: the per-primitive sums are f32 atomics in no fixed order; the reference's own
cross-check of this kernel uses atol = rtol = 5e-5 (tests/test_primitive_csr.py:60-63)."""
import numpy as np
import pytest
import torch

from conftest import to_dev
from helpers import Frame
from test_oracle_render import _synthetic_records

pytestmark = pytest.mark.gpu


def _close(got, want, what, tol=5e-5):
    got = got.cpu().numpy()
    scale = max(1.0, float(np.abs(want).max()))
    assert got.shape == want.shape and np.abs(got - want).max() <= tol * scale, (what, float(np.abs(got - want).max()), scale)


@pytest.mark.parametrize("seed", [0, 3])
def test_reverse_matches_oracle_on_synthetic_records(device, oracle_mod, seed):
    from mlp_splatting_amd.tile_ext import TileExt
    inputs, autograd = _synthetic_records(seed, pixels=300, n=20, max_per_pixel=12)
    want = oracle_mod.records_reverse(*inputs)
    got = TileExt().primitive_records_reverse(*[to_dev(a, device) for a in inputs])
    for name, a, b, c in zip(("d4", "grad_positions", "grad_log_scales", "grad_quats"), got, want, autograd):
        _close(a, b, name)
        _close(a, c.astype(np.float32), name + " vs autograd", tol=1e-4)


def test_reverse_on_records_of_a_rendered_frame(device, oracle_mod):
    from mlp_splatting_amd.tile_ext import TileExt
    fr = Frame("cfg1_5k_160x120", n=1500, hidden=32, width=72, height=48)
    cand, off = fr.oracle_lists(oracle_mod)
    x = [to_dev(a, device) for a in fr.base_numpy(cand, off)]
    x += [torch.zeros_like(x[0]), torch.zeros(fr.W * fr.H, device=device)]
    ext = TileExt()
    rgb, alpha, ids, x6, raw, masks, gates, offsets = ext.render_tiles_training_records(x, fr.W, fr.H, 8, fr.thr, 1.5, 2.0)
    assert ids.numel() > 5000
    torch.manual_seed(1)
    grgb = torch.randn(fr.W * fr.H, 3, device=device)
    gt = torch.randn(fr.W * fr.H, device=device)
    got = ext.primitive_records_reverse(ids, offsets, x6, raw, x[3], x[4], grgb, gt)
    want = oracle_mod.records_reverse(ids.cpu().numpy(), offsets.cpu().numpy(), x6.cpu().numpy(), raw.cpu().numpy(),
                                      fr.scene.log_scales, fr.scene.quats, grgb.cpu().numpy(), gt.cpu().numpy())
    for name, a, b in zip(("d4", "grad_positions", "grad_log_scales", "grad_quats"), got, want):
        assert float(np.abs(b).max()) > 1e-3
        _close(a, b, name)
    # d4 is written record by record, without atomics: same bits
    assert np.array_equal(got[0].cpu().numpy().view(np.uint32), want[0].view(np.uint32))
    # the atomic-free split (adjoints per record, then one wavefront per primitive) gives the same gradients
    from mlp_splatting_amd import ops
    from mlp_splatting_amd.primitive_csr import group_records as _group
    d4b, adjoint = ops.records_reverse_adjoints(ids, offsets, raw, grgb, gt)
    assert torch.equal(d4b, got[0])
    csr_b = _group(ids, x6, d4b, fr.scene.n, masks)
    from mlp_splatting_amd import primitive_gemm
    for segment in (32, 512):
        split = ops.geometry_gradients(csr_b.offsets, csr_b.record_indices, csr_b.x6, adjoint, x[3], x[4],
                                       primitive_gemm.prepare_groups(csr_b, segment))
        for name, a, b in zip(("grad_positions", "grad_log_scales", "grad_quats"), split, want[1:]):
            _close(a, b, name + f" (split, segment {segment})")
    for name, a, b in zip(("grad_positions", "grad_log_scales", "grad_quats"), split, want[1:]):
        _close(a, b, name + " (split)")
    # and it feeds the grouped weight gradients
    from mlp_splatting_amd import primitive_gemm as gemm
    from mlp_splatting_amd.primitive_csr import group_records
    csr = group_records(ids, x6, got[0], fr.scene.n, masks)
    grads = gemm.grouped_weight_gradients(csr, x[7], x[8], x[9:15], dtype=torch.float32)
    assert all(bool(torch.isfinite(g).all()) for g in grads) and float(grads[0].abs().max()) > 0


def test_reverse_argument_checks_and_empty_inputs(device):
    from mlp_splatting_amd.tile_ext import TileExt
    ext = TileExt()
    z = lambda *shape, dtype=torch.float32: torch.zeros(*shape, dtype=dtype, device=device)
    quats = z(3, 4)
    quats[:, 0] = 1
    empty = (z(0, dtype=torch.int32), z(5, dtype=torch.int64), z(0, 6), z(0, 8), z(3, 3), quats, z(4, 3) + 1, z(4) + 1)
    d4, gp, gs, gq = ext.primitive_records_reverse(*empty)
    assert tuple(d4.shape) == (0, 4) and not gp.any() and not gs.any() and not gq.any()
    ids = torch.tensor([0, 5], dtype=torch.int32, device=device)
    off = torch.tensor([0, 1, 2, 2, 2], dtype=torch.int64, device=device)
    with pytest.raises(RuntimeError):            # id 5 of 3 primitives
        ext.primitive_records_reverse(ids, off, z(2, 6), z(2, 8), z(3, 3), quats, z(4, 3), z(4))
    ids[1] = 2
    with pytest.raises(RuntimeError):            # offsets must end at the record count
        ext.primitive_records_reverse(ids, off + 1, z(2, 6), z(2, 8), z(3, 3), quats, z(4, 3), z(4))
    with pytest.raises(RuntimeError):            # offsets must be int64
        ext.primitive_records_reverse(ids, off.int(), z(2, 6), z(2, 8), z(3, 3), quats, z(4, 3), z(4))
    out = ext.primitive_records_reverse(ids, off, z(2, 6), z(2, 8), z(3, 3), quats, z(4, 3), z(4))
    assert float(out[0].abs().max()) == 0.0
