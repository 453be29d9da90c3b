"""Matrix-core training-records forward (TileExt.render_tiles_training_records_wmma) against the scalar f32 record
forward, which tests/test_gpu_parity.py holds bit-exact to the CPU oracle.  The contracts are those of the
reference's tests/test_training_wmma.py: record topology (ids, offsets), x6, decay and gates are exact; R, G, B,
sigma, alpha and the image follow the reduced-precision MLP within atol = rtol = 5e-4 (fp16) / 3e-3 (bf16)
(:133-135); a constant MLP (zero weights, output biases only) is exact in every field; the saved masks are those
of the reduced-precision forward actually run; count and emit agree; capacities raise; numeric overflow repeats
the whole frame in f32; invalid arguments are rejected before anything is counted."""
import math

import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu

PRECISIONS = ("float16", "bfloat16")
WEIGHTS = ("W1", "b1", "W2", "b2", "W3", "b3")
SHAPES = ((32, 72), (32,), (32, 32), (32,), (4, 32), (4,))
STATS = ("calls", "frame_fallbacks", "fp32_nonfinite_failures", "count_emit_failures", "capacity_failures")


@pytest.fixture(scope="module")
def ext(device):
    from mlp_splatting_amd.tile_ext import TileExt
    return TileExt()


def _stats(ext):
    values = ext.training_wmma_safety_stats()
    assert len(values) == len(STATS)
    return dict(zip(STATS, map(int, values)))


def _delta(ext, before):
    after = _stats(ext)
    return {k: after[k] - before[k] for k in STATS}


def _case(device, n=13, width=9, height=7, *, constant=False, mosaic=False):
    """A slab of n primitives in front of a near-orthographic camera; every tile lists every primitive."""
    g = torch.Generator(device="cpu").manual_seed(42157 + n + width + height)
    rnd = lambda *shape: torch.randn(*shape, generator=g).to(device)
    uni = lambda lo, hi, *shape: (torch.rand(*shape, generator=g) * (hi - lo) + lo).to(device)
    d = {}
    yy, xx = torch.meshgrid(torch.linspace(-.45, .45, height, device=device),
                            torch.linspace(-.55, .55, width, device=device), indexing="ij")
    d["rays_o"] = torch.stack((xx.flatten(), yy.flatten(), torch.zeros(width * height, device=device)), -1).contiguous()
    d["rays_d"] = torch.tensor([.025, -.015, 1.], device=device).repeat(width * height, 1)
    if mosaic:
        # origins AND directions differ inside a tile, with a view boundary that is not a tile edge
        ix = torch.arange(width * height, device=device)
        quadrant = (ix % width >= width // 2).long() + 2 * (ix // width >= height // 2).long()
        cameras = torch.tensor([[0., 0., 0.], [.19, 0., -.12], [0., -.17, .09], [-.14, .13, -.08]], device=device)
        directions = torch.tensor([[0., 0., 1.], [-.09, .04, 1.], [.07, .08, 1.], [.12, -.05, 1.]], device=device)
        d["rays_o"] = (d["rays_o"] + cameras[quadrant]).contiguous()
        d["rays_d"] = directions[quadrant]
    d["rays_d"] = F.normalize(d["rays_d"], dim=-1).contiguous()
    d["positions"] = torch.cat((uni(-.2, .2, n, 2), torch.linspace(.75, 1.75, n, device=device)[:, None]), 1).contiguous()
    d["log_scales"] = uni(-.45, .15, n, 3)
    d["quats"] = F.normalize(rnd(n, 4), dim=-1).contiguous() if n else torch.zeros(0, 4, device=device)
    d["freq"] = 2. ** torch.arange(6, device=device, dtype=torch.float32)
    d["attenuation"] = torch.exp(-.5 * d["freq"].square() * .0001)
    for name, shape in zip(WEIGHTS, SHAPES):
        d[name] = rnd(n, *shape) * .035
    d["b3"][:, 3] = -2.          # far from termination: the record topology must match the f32 path
    if constant:
        for name in WEIGHTS:
            d[name].zero_()
        d["b3"][:, 0] = torch.linspace(-1., 1., n, device=device)
        d["b3"][:, 1] = -.25
        d["b3"][:, 2] = .5
        d["b3"][:, 3] = -2.
    tiles = ((width + 7) // 8) * ((height + 7) // 8)
    d["candidates"] = torch.arange(n, device=device, dtype=torch.int32).repeat(tiles)
    d["offsets"] = torch.arange(tiles + 1, device=device, dtype=torch.int32) * n
    d["grad_rgb"] = rnd(width * height, 3) * .1
    d["grad_t"] = rnd(width * height) * .1
    return d


def _args(d):
    return [d["rays_o"], d["rays_d"], d["positions"], d["log_scales"], d["quats"], d["candidates"], d["offsets"],
            d["freq"], d["attenuation"]] + [d[k] for k in WEIGHTS] + [d["grad_rgb"], d["grad_t"]]


def _render(ext, d, width, height, precision, threshold=.001):
    return ext.render_tiles_training_records_wmma(_args(d), width, height, 8, threshold, 1.5, 2., precision)


def _scalar(ext, d, width, height, threshold=.001):
    return ext.render_tiles_training_records(_args(d), width, height, 8, threshold, 1.5, 2.)


def _schema(records, d, width, height):
    assert len(records) == 8
    rgb, alpha, ids, x6, raw, masks, gates, offsets = records
    count = len(ids)
    shapes = ((width * height, 3), (width * height, 1), (count,), (count, 6), (count, 8), (count, 2), (count, 4),
              (width * height + 1,))
    dtypes = (torch.float32, torch.float32, torch.int32, torch.float32, torch.float32, torch.int32, torch.float32,
              torch.int64)
    for value, shape, dtype in zip(records, shapes, dtypes):
        assert tuple(value.shape) == shape and value.dtype == dtype and value.device == d["positions"].device
        assert value.is_contiguous() and bool(torch.isfinite(value).all())
    assert int(offsets[0]) == 0 and int(offsets[-1]) == count and bool((offsets.diff() >= 0).all())
    assert bool(((ids >= 0) & (ids < len(d["positions"]))).all())
    if count:
        assert bool(((raw[:, 4:6] >= 0) & (raw[:, 4:6] <= 1)).all())
        torch.testing.assert_close(gates.sum(-1), torch.ones(count, device=ids.device), atol=2e-6, rtol=2e-6)
        pixels = torch.repeat_interleave(torch.arange(width * height, device=ids.device), offsets.diff(), output_size=count)
        assert torch.equal(x6[:, :3], d["rays_d"][pixels])


def _parity(actual, expected, precision, exact=False):
    for index in (2, 3, 6, 7):                        # ids, x6, gates, offsets: the f32 expression path
        assert torch.equal(actual[index], expected[index]), index
    assert torch.equal(actual[4][:, 6], expected[4][:, 6])        # decay
    if exact:
        for index, (a, b) in enumerate(zip(actual, expected)):
            assert torch.equal(a, b), index
    else:
        tol = .003 if precision == "bfloat16" else .0005
        for index in (0, 1, 4):
            torch.testing.assert_close(actual[index], expected[index], atol=tol, rtol=tol)


@pytest.mark.parametrize("precision", PRECISIONS)
@pytest.mark.parametrize("width,height,mosaic", [(1, 1, False), (8, 8, False), (13, 11, False), (17, 9, True)])
@pytest.mark.parametrize("constant", [False, True])
def test_schema_geometry_and_full_records(ext, device, precision, width, height, mosaic, constant):
    d = _case(device, width=width, height=height, constant=constant, mosaic=mosaic)
    originals = [(t.clone(), t._version) for t in _args(d)]
    expected = _scalar(ext, d, width, height)
    before = _stats(ext)
    actual = _render(ext, d, width, height, precision)
    _schema(actual, d, width, height)
    assert len(actual[2]) > 0
    _parity(actual, expected, precision, exact=constant)
    if not constant:
        assert not torch.equal(actual[4][:, :3], expected[4][:, :3])     # it really is the reduced-precision MLP
    assert _delta(ext, before) == dict(zip(STATS, (1, 0, 0, 0, 0)))
    for t, (saved, version) in zip(_args(d), originals):
        assert torch.equal(t, saved) and t._version == version


@pytest.mark.parametrize("precision", PRECISIONS)
def test_a_rendered_frame_matches_the_scalar_records(ext, device, oracle_mod, precision):
    """A perspective frame of the 5k-primitive scene with binned lists: 10^5 records over 60 tiles."""
    from conftest import to_dev
    from helpers import Frame
    fr = Frame("cfg1_5k_160x120", n=1500, hidden=32, width=80, height=48)
    cand, off = fr.oracle_lists(oracle_mod)
    x = [to_dev(a, device) for a in fr.base_numpy(cand, off)]
    x += [torch.zeros_like(x[0]), torch.zeros(fr.W * fr.H, device=device)]
    expected = ext.render_tiles_training_records(x, fr.W, fr.H, 8, fr.thr, 1.5, 2.0)
    actual = ext.render_tiles_training_records_wmma(x, fr.W, fr.H, 8, fr.thr, 1.5, 2.0, precision)
    assert actual[2].numel() > 5000
    tol = .003 if precision == "bfloat16" else .0005
    # pixels whose early termination falls on the other side of T = 1e-3 may differ by their last records;
    # everything up to the shorter of the two lists is the same record
    same = actual[7].diff() == expected[7].diff()
    assert float(same.float().mean()) > 0.995
    torch.testing.assert_close(actual[0], expected[0], atol=tol, rtol=tol)
    torch.testing.assert_close(actual[1], expected[1], atol=tol, rtol=tol)
    if bool(same.all()):
        _parity(actual, expected, precision)
    # masks: the reduced-precision forward may flip units whose pre-activation is within rounding of zero
    if bool(same.all()):
        flipped = (actual[5] ^ expected[5]).to(torch.int64) & 0xFFFFFFFF
        bits = sum(int(((flipped >> b) & 1).sum()) for b in range(32))
        assert bits < 0.01 * 64 * actual[5].shape[0], bits


@pytest.mark.parametrize("precision", PRECISIONS)
@pytest.mark.parametrize("kind", ["empty_scene", "empty_lists", "no_hits"])
def test_empty_outputs_are_initialised(ext, device, precision, kind):
    width, height = 13, 11
    d = _case(device, 0 if kind == "empty_scene" else 5, width, height)
    if kind == "empty_lists":
        d["candidates"] = d["candidates"].new_empty(0)
        d["offsets"].zero_()
    elif kind == "no_hits":
        d["rays_o"][:, 0] = 100.
    actual = _render(ext, d, width, height, precision)
    _schema(actual, d, width, height)
    assert len(actual[2]) == 0
    for index in (0, 1, 7):
        assert bool((actual[index] == 0).all())
    _parity(actual, _scalar(ext, d, width, height), precision, exact=True)


def _stack_at_origin(d):
    d["positions"].zero_()
    d["positions"][:, 2] = 1.
    d["log_scales"].zero_()
    d["quats"].zero_()
    d["quats"][:, 0] = 1.
    d["rays_o"].zero_()
    d["rays_d"].zero_()
    d["rays_d"][:, 2] = 1.


@pytest.mark.parametrize("precision", PRECISIONS)
def test_stable_depth_ties_and_divergent_early_stop(ext, device, precision):
    d = _case(device, 12, 8, 8, constant=True)
    _stack_at_origin(d)
    d["rays_o"][:, 0] = 100.
    selected = [0, 15, 16, 31, 32, 47, 48, 63]
    d["rays_o"][selected] = 0.
    d["candidates"] = d["candidates"].flip(0).contiguous()
    d["b3"][:, 3] = 8.           # every active pixel stops after the first of the tied primitives
    actual = _render(ext, d, 8, 8, precision)
    _schema(actual, d, 8, 8)
    _parity(actual, _scalar(ext, d, 8, 8), precision, exact=True)
    counts = torch.zeros(64, device=device, dtype=torch.int64)
    counts[selected] = 1
    assert torch.equal(actual[7].diff(), counts)
    assert actual[2].tolist() == [11] * len(selected)


@pytest.mark.parametrize("precision", PRECISIONS)
def test_masks_follow_the_reduced_precision_forward(ext, device, precision):
    from mlp_splatting_amd.primitive_csr import group_records
    from mlp_splatting_amd.primitive_gemm import grouped_weight_gradients
    d = _case(device, 1, 1, 1, constant=True)
    epsilon = 2. ** (-12 if precision == "float16" else -9)
    d["b1"][0, 1] = 1. + epsilon
    d["W2"][0] = torch.eye(32, device=device)
    d["b2"][0, 1] = -(1. + epsilon / 2.)
    d["W3"][0, :, 1] = .125
    # h1 rounds to 1 in the operand type, so the h2 really computed is negative although the f32 one is positive
    actual = _render(ext, d, 1, 1, precision)
    scalar = _scalar(ext, d, 1, 1)
    assert len(actual[2]) == 1
    assert actual[5].tolist() == [[2, 0]]
    assert scalar[5].tolist() == [[2, 2]]
    torch.testing.assert_close(actual[0], scalar[0], atol=.0001, rtol=.0001)
    csr = group_records(actual[2], actual[3], torch.ones(1, 4, device=device), 1, actual[5])
    gradients = grouped_weight_gradients(csr, d["freq"], d["attenuation"], [d[k] for k in WEIGHTS], dtype=torch.float32)
    for gradient in gradients[:4]:          # only the saved mask keeps the adjoint away from W1, b1, W2, b2
        assert bool((gradient == 0).all())


@pytest.mark.parametrize("precision", PRECISIONS)
def test_every_mask_bit_maps_to_its_unit(ext, device, precision):
    """One active unit at a time in each hidden layer: bit u of the saved mask is hidden unit u."""
    d = _case(device, 32, 1, 1, constant=True)
    _stack_at_origin(d)
    d["b3"][:, 3] = -6.
    for u in range(32):
        d["b1"][u].fill_(-1.)
        d["b1"][u, u] = 1.
        d["b2"][u].fill_(-1.)
        d["b2"][u, 31 - u] = 1.
    actual = _render(ext, d, 1, 1, precision)
    assert len(actual[2]) == 32
    masks = actual[5].to(torch.int64) & 0xFFFFFFFF
    ids = actual[2].tolist()
    for row, u in enumerate(ids):
        assert masks[row].tolist() == [1 << u, 1 << (31 - u)], (u, masks[row].tolist())
    assert torch.equal(actual[5], _scalar(ext, d, 1, 1)[5])


@pytest.mark.parametrize("precision", PRECISIONS)
@pytest.mark.parametrize("bias_offset", [-.001, 0., .001])
def test_count_and_emit_agree_at_the_transmittance_boundary(ext, device, precision, bias_offset):
    d = _case(device, 2, 1, 1, constant=True)
    _stack_at_origin(d)
    d["positions"][:, 2] = torch.tensor([1., 2.], device=device)
    d["b3"][0, 3] = math.log(999.) + bias_offset
    before = _stats(ext)
    actual = _render(ext, d, 1, 1, precision)
    _schema(actual, d, 1, 1)
    _parity(actual, _scalar(ext, d, 1, 1), precision, exact=True)
    still_active = bool((1. - actual[4][0, 5]) >= .001)       # the f32 update itself, not a float64 estimate
    assert actual[7].tolist() == [0, 2 if still_active else 1]
    assert _delta(ext, before) == dict(zip(STATS, (1, 0, 0, 0, 0)))


@pytest.mark.parametrize("precision", PRECISIONS)
@pytest.mark.parametrize("kind", ["candidate", "hit"])
def test_capacity_raises_instead_of_truncating(ext, device, precision, kind):
    capacity = ext.max_tile_prims if kind == "candidate" else ext.max_hits
    d = _case(device, capacity + 1, 1, 1, constant=True)
    _stack_at_origin(d)
    d["b3"][:, 3] = -20. if kind == "hit" else 8.
    before = _stats(ext)
    with pytest.raises(RuntimeError, match="capacity"):
        _render(ext, d, 1, 1, precision)
    expected = (0, 0, 0, 0, 0) if kind == "candidate" else (1, 0, 0, 0, 1)
    assert _delta(ext, before) == dict(zip(STATS, expected))


@pytest.mark.parametrize("precision", PRECISIONS)
def test_just_below_hit_capacity_keeps_every_record(ext, device, precision):
    count = ext.max_hits - 1
    d = _case(device, count, 1, 1, constant=True)
    _stack_at_origin(d)
    d["b3"][:, 3] = -20.
    actual = _render(ext, d, 1, 1, precision)
    assert actual[7].tolist() == [0, count]
    _parity(actual, _scalar(ext, d, 1, 1), precision, exact=True)


@pytest.mark.parametrize("precision", PRECISIONS)
@pytest.mark.parametrize("kind", ["weight", "hidden"])
def test_numeric_failure_repeats_the_whole_frame_in_f32(ext, device, precision, kind):
    d = _case(device, 3, 9, 7, constant=True, mosaic=True)
    large = 70000. if precision == "float16" else 3.4e38
    if kind == "weight":
        # zero x phase: the f32 product large * sin(0) is finite, the rounded weight is not
        d["rays_d"][:, 0] = 0.
        d["W1"][0, 0, 0] = large
    else:
        d["b1"][0, 0] = large
    expected = _scalar(ext, d, 9, 7)
    before = _stats(ext)
    with pytest.warns(UserWarning, match="rerunning the whole FP32 record forward"):
        actual = _render(ext, d, 9, 7, precision)
    _schema(actual, d, 9, 7)
    _parity(actual, expected, precision, exact=True)
    assert _delta(ext, before) == dict(zip(STATS, (1, 1, 0, 0, 0)))


@pytest.mark.parametrize("precision", PRECISIONS)
def test_non_finite_f32_retry_raises_without_records(ext, device, precision):
    d = _case(device, 1, 1, 1, constant=True)
    d["b1"][0, 0] = 3.e38
    d["W2"][0, 0, 0] = 3.e38
    before = _stats(ext)
    with pytest.warns(UserWarning), pytest.raises(RuntimeError, match="[Nn]onfinite|finite"):
        _render(ext, d, 1, 1, precision)
    delta = _delta(ext, before)
    assert delta["frame_fallbacks"] == 1 and delta["fp32_nonfinite_failures"] == 1
    assert delta["count_emit_failures"] == delta["capacity_failures"] == 0


@pytest.mark.parametrize("kind", ["half_master", "half_geometry", "invalid_id", "invalid_offset", "tile16", "precision",
                                  "shape", "nonfinite_unused_geometry", "threshold"])
def test_invalid_contract_is_rejected(ext, device, kind):
    d = _case(device, 3, 9, 7)
    tile, precision, threshold = 8, "float16", .001
    if kind == "half_master":
        d["W1"] = d["W1"].half()
    elif kind == "half_geometry":
        d["log_scales"] = d["log_scales"].half()
    elif kind == "invalid_id":
        d["candidates"][-1] = 3
    elif kind == "invalid_offset":
        d["offsets"][0] = 1
    elif kind == "tile16":
        tile = 16
    elif kind == "precision":
        precision = "float32"
    elif kind == "shape":
        d["W1"] = d["W1"][:, :, :71].contiguous()
    elif kind == "threshold":
        threshold = 1.0
    else:
        d["positions"][-1, 0] = 100.
        d["log_scales"][-1, 1] = float("nan")
    before = _stats(ext)
    with pytest.raises(RuntimeError):
        ext.render_tiles_training_records_wmma(_args(d), 9, 7, tile, threshold, 1.5, 2., precision)
    assert _delta(ext, before) == dict(zip(STATS, (0, 0, 0, 0, 0)))


def test_per_call_stream_and_record_lifetime(ext, device):
    d = _case(device, 4, 9, 7)
    original = _render(ext, d, 9, 7, "float16")
    saved = [v.clone() for v in original]
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        # in-place edits of the master tensors, geometry included, must reach this call
        d["b3"][:, 0].add_(.7)
        d["log_scales"].add_(.15)
        changed = _render(ext, d, 9, 7, "float16")
        expected = _scalar(ext, d, 9, 7)
    torch.cuda.current_stream().wait_stream(stream)
    _parity(changed, expected, "float16")
    assert not torch.equal(changed[0], original[0])
    for value, snapshot in zip(original, saved):
        assert torch.equal(value, snapshot)


def _f32_vjp_with_saved_masks(csr, d):
    """Dense per-primitive chain in torch that takes the ReLU decisions from the saved masks."""
    from mlp_splatting_amd.cumodel import _encode_x6
    weights = [d[k] for k in WEIGHTS]
    result = [torch.zeros_like(w) for w in weights]
    bits = torch.arange(32, device=csr.x6.device, dtype=torch.int64)
    for p in range(len(weights[0])):
        lo, hi = map(int, csr.offsets[p:p + 2])
        if lo == hi:
            continue
        x = _encode_x6(csr.x6[lo:hi], d["freq"], d["attenuation"])
        w1, b1, w2, b2, w3, _ = [w[p] for w in weights]
        h1 = torch.relu(x @ w1.T + b1)
        h2 = torch.relu(h1 @ w2.T + b2)
        masks = csr.relu_masks[lo:hi].long()
        m1 = ((masks[:, :1] >> bits) & 1).bool()
        m2 = ((masks[:, 1:] >> bits) & 1).bool()
        d3 = csr.grad4[lo:hi]
        d2 = (d3 @ w3) * m2
        d1 = (d2 @ w2) * m1
        for out, grad in zip(result, (d1.T @ x, d1.sum(0), d2.T @ h1, d2.sum(0), d3.T @ h2, d3.sum(0))):
            out[p] = grad
    return result


@pytest.mark.parametrize("precision", PRECISIONS)
@pytest.mark.parametrize("constant", [False, True])
def test_saved_records_feed_reverse_and_grouped_vjp(ext, device, precision, constant):
    from mlp_splatting_amd.primitive_csr import group_records
    from mlp_splatting_amd.primitive_gemm import grouped_weight_gradients
    d = _case(device, 9, 9, 7, constant=constant, mosaic=True)
    d["b1"].fill_(.125)
    d["b2"].fill_(.25)
    if not constant:
        for name in ("W1", "W2", "W3"):      # strictly positive hidden activations: no mask flips to confuse the VJP check
            d[name].mul_(.1)
    records = _render(ext, d, 9, 7, precision)
    expected = ext.render_tiles_backward_tilecenter_full(*_args(d), 9, 7, 8, 8, .001)
    d4, gp, gs, gq = ext.primitive_records_reverse(records[2], records[7], records[3], records[4], d["log_scales"],
                                                   d["quats"], d["grad_rgb"], d["grad_t"])
    forward_tol = 5e-5 if constant else (.003 if precision == "bfloat16" else .0005)
    for actual, reference in zip((gp, gs, gq), expected[6:]):
        torch.testing.assert_close(actual, reference, atol=3e-5, rtol=forward_tol)
    csr = group_records(records[2], records[3], d4, len(d["positions"]), records[5])
    gradients = grouped_weight_gradients(csr, d["freq"], d["attenuation"], [d[k] for k in WEIGHTS], dtype=torch.float32)
    dense = _f32_vjp_with_saved_masks(csr, d)
    for actual, reference, scalar in zip(gradients, dense, expected[:6]):
        torch.testing.assert_close(actual, reference, atol=2e-5, rtol=5e-5)
        torch.testing.assert_close(actual, scalar, atol=3e-5, rtol=forward_tol)
    if not constant:
        assert all(bool((g != 0).any()) for g in gradients)


@pytest.mark.parametrize("backend,precision", [("wmma_fp16", "float16"), ("wmma_bf16", "bfloat16")])
def test_environment_selects_the_record_forward(ext, device, monkeypatch, backend, precision):
    from mlp_splatting_amd import csr_training
    d = _case(device, 7, 9, 7, mosaic=True)
    monkeypatch.setenv("MLPSP_CSR_FORWARD_BACKEND", backend)
    before = _stats(ext)
    chosen = csr_training._record_forward(ext, _args(d), 9, 7, .001, 1.5, 2.)
    assert _delta(ext, before)["calls"] == 1
    direct = _render(ext, d, 9, 7, precision)
    for a, b in zip(chosen, direct):
        assert torch.equal(a, b)
    monkeypatch.setenv("MLPSP_CSR_FORWARD_BACKEND", "tensor_cores")
    with pytest.raises(ValueError, match="MLPSP_CSR_FORWARD_BACKEND"):
        csr_training._record_forward(ext, _args(d), 9, 7, .001, 1.5, 2.)


@pytest.mark.parametrize("precision", PRECISIONS)
def test_training_step_on_matrix_core_records(ext, device, monkeypatch, precision):
    """CSRTrainingFunction on the reduced-precision records: the 512-channel attribute gradient equals autograd
    through a dense framebuffer of those very records, and no MLP-input adjoint exists."""
    from mlp_splatting_amd import cumodel
    from mlp_splatting_amd.csr_training import CSRTrainingFunction
    from test_gpu_feature_loss import _framebuffer64, _resize
    monkeypatch.setattr(cumodel, "_tile_ext", ext, raising=False)
    monkeypatch.setattr(cumodel, "_tile_ext_key", cumodel._tile_ext_build_config(8)[0])
    monkeypatch.setenv("MLPSP_CSR_MLP_PRECISION", "float32")
    monkeypatch.setenv("MLPSP_CSR_FORWARD_BACKEND", "wmma_fp16" if precision == "float16" else "wmma_bf16")
    d = _case(device, 7, 9, 7, mosaic=True)
    base = _args(d)[:15]
    for t in base:
        if t.dtype == torch.float32:
            t.requires_grad_()
    g = torch.Generator().manual_seed(5)
    attributes = (torch.randn(7, 5, 512, generator=g) * .2).to(device).requires_grad_()
    with torch.no_grad():
        records = _render(ext, d, 9, 7, precision)
        prediction = _resize(_framebuffer64(records, attributes.detach().cpu().double(), 9, 7), 9, 7, 5, 3)
        # every residual at least 0.01 away from zero: the L1 subgradient is the same in both evaluations
        noise = (torch.rand(prediction.shape, generator=g) * .05 + .01) * (torch.rand(prediction.shape, generator=g) < .5).double().mul(2).sub(1)
        target = (prediction + noise).float().to(device).contiguous()
    before = _stats(ext)
    rgb, feature_loss = CSRTrainingFunction.apply(*base, attributes, target, (9, 7, .001, 1.5, 2.), None)
    assert _delta(ext, before)["calls"] == 1
    (rgb.square().mean() + feature_loss).backward()
    for index in (0, 1, 7, 8):
        assert base[index].grad is None
    for index in (2, 3, 4, 9, 10, 11, 12, 13, 14):
        assert base[index].grad is not None and bool(torch.isfinite(base[index].grad).all())
    leaf = attributes.detach().cpu().double().requires_grad_()
    dense = _resize(_framebuffer64(records, leaf, 9, 7), 9, 7, 5, 3)
    torch.testing.assert_close(feature_loss.detach().cpu().double(), F.l1_loss(dense, target.cpu().double()).detach(),
                               atol=2e-7, rtol=2e-6)
    F.l1_loss(dense, target.cpu().double()).backward()
    torch.testing.assert_close(attributes.grad.cpu().double(), leaf.grad, atol=2e-8, rtol=8e-5)


def test_fused_finite_scan(device):
    """mlpsp_all_finite over several arrays of ragged length and alignment: every position of a bad value is seen."""
    from mlp_splatting_amd import ops
    base = torch.zeros(4099, device=device)
    views = [base[1:], base[2:11], base[3:3], torch.ones(70001, device=device), torch.ones(5, 3, device=device)]
    assert int(ops.all_finite_flag(views).item()) == 0
    assert int(ops.all_finite_flag([]).item()) == 0
    for tensor, index, value in [(base, 1, float("nan")), (base, 4098, float("inf")), (base, 2049, -float("inf")),
                                 (views[3], 70000, float("nan")), (views[3], 0, float("inf")), (views[4], (4, 2), float("nan"))]:
        saved = tensor[index].clone()
        tensor[index] = value
        assert int(ops.all_finite_flag(views).item()) == 1, (index, value)
        tensor[index] = saved
        assert int(ops.all_finite_flag(views).item()) == 0
    with pytest.raises(RuntimeError):
        ops.all_finite_flag([torch.zeros(4, device=device, dtype=torch.float16)])
