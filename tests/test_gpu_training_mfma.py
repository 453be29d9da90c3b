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


# Mosaic variant: four cameras, one per image quadrant (the quadrant boundary is NOT a tile edge, so origins and
# directions both change inside a tile).
_QUADRANT_ORIGIN_SHIFT = ((0., 0., 0.), (.19, 0., -.12), (0., -.17, .09), (-.14, .13, -.08))
_QUADRANT_DIRECTION = ((0., 0., 1.), (-.09, .04, 1.), (.07, .08, 1.), (.12, -.05, 1.))


def _slab_rays(device, width, height, mosaic):
    """Near-orthographic rays: origins on a width x height grid in the z = 0 plane, one shared direction (or one
    direction and origin shift per quadrant)."""
    xs = torch.linspace(-.55, .55, width, device=device)
    ys = torch.linspace(-.45, .45, height, device=device)
    origins = torch.zeros(height, width, 3, device=device)
    origins[..., 0] = xs[None, :]
    origins[..., 1] = ys[:, None]
    origins = origins.reshape(-1, 3)
    directions = torch.tensor([.025, -.015, 1.], device=device).expand(width * height, 3)
    if mosaic:
        col = torch.arange(width, device=device)[None, :].expand(height, width)
        row = torch.arange(height, device=device)[:, None].expand(height, width)
        quadrant = ((col >= width // 2).long() + 2 * (row >= height // 2).long()).reshape(-1)
        origins = origins + torch.tensor(_QUADRANT_ORIGIN_SHIFT, device=device)[quadrant]
        directions = torch.tensor(_QUADRANT_DIRECTION, device=device)[quadrant]
    return origins.contiguous(), F.normalize(directions, dim=-1).contiguous()


def _case(device, n=13, width=9, height=7, *, constant=False, mosaic=False):
    """n primitives stacked in depth (z from 0.75 to 1.75) in front of the rays of _slab_rays; every tile lists every
    primitive in id order.  Small random MLPs with the density logit pinned at -2, far from early termination, so
    that the reduced-precision forward must reproduce the f32 record topology; ``constant``: zero weights and only
    output biases, for which every record field is exact in any operand precision."""
    rng = torch.Generator(device="cpu").manual_seed(42157 + n + width + height)

    def normal(*shape, scale=1.):
        return (torch.randn(*shape, generator=rng) * scale).to(device)

    def uniform(lo, hi, *shape):
        return (lo + (hi - lo) * torch.rand(*shape, generator=rng)).to(device)

    pixels = width * height
    tiles = ((width + 7) // 8) * ((height + 7) // 8)
    d = dict(zip(("rays_o", "rays_d"), _slab_rays(device, width, height, mosaic)))
    depth = torch.linspace(.75, 1.75, n, device=device)
    d["positions"] = torch.cat((uniform(-.2, .2, n, 2), depth[:, None]), dim=1).contiguous()
    d["log_scales"] = uniform(-.45, .15, n, 3)
    d["quats"] = F.normalize(normal(n, 4), dim=-1).contiguous() if n else torch.zeros(0, 4, device=device)
    d["freq"] = torch.tensor([1., 2., 4., 8., 16., 32.], device=device)
    d["attenuation"] = torch.exp(-.5e-4 * d["freq"] ** 2)
    for name, shape in zip(WEIGHTS, SHAPES):
        d[name] = torch.zeros(n, *shape, device=device) if constant else normal(n, *shape, scale=.035)
    if constant:
        d["b3"][:, 0] = torch.linspace(-1., 1., n, device=device)
        d["b3"][:, 1] = -.25
        d["b3"][:, 2] = .5
    d["b3"][:, 3] = -2.
    d["candidates"] = torch.arange(n, device=device, dtype=torch.int32).repeat(tiles)
    d["offsets"] = (n * torch.arange(tiles + 1, device=device)).to(torch.int32)
    d["grad_rgb"] = normal(pixels, 3, scale=.1)
    d["grad_t"] = normal(pixels, scale=.1)
    return d


def _args(d):
    return [d["rays_o"], d["rays_d"], d["positions"], d["log_scales"], d["quats"], d["candidates"], d["offsets"],
            d["freq"], d["attenuation"]] + [d[k] for k in WEIGHTS] + [d["grad_rgb"], d["grad_t"]]


def _render(ext, d, width, height, precision, threshold=.001):
    return ext.render_tiles_training_records_wmma(_args(d), width, height, 8, threshold, 1.5, 2., precision)


def _scalar(ext, d, width, height, threshold=.001):
    return ext.render_tiles_training_records(_args(d), width, height, 8, threshold, 1.5, 2.)


RECORD_FIELDS = (       # name, trailing shape, dtype, leading dimension ("B" pixels, "R" records, "B+1")
    ("rgb", (3,), torch.float32, "B"), ("alpha", (1,), torch.float32, "B"), ("ids", (), torch.int32, "R"),
    ("x6", (6,), torch.float32, "R"), ("raw", (8,), torch.float32, "R"), ("masks", (2,), torch.int32, "R"),
    ("gates", (4,), torch.float32, "R"), ("offsets", (), torch.int64, "B+1"))


def _schema(records, d, width, height):
    """Layout and internal consistency of a record list: field shapes and types, a monotone offsets vector that
    covers the records, valid ids, T and alpha inside [0, 1], gates that sum to one, and x6[:, :3] equal to the
    ray direction of the record's pixel."""
    assert len(records) == len(RECORD_FIELDS)
    pixels = width * height
    fields = {name: value for (name, *_), value in zip(RECORD_FIELDS, records)}
    total = fields["ids"].numel()
    leading = {"B": pixels, "R": total, "B+1": pixels + 1}
    for (name, trailing, dtype, lead), value in zip(RECORD_FIELDS, records):
        assert value.dtype == dtype and tuple(value.shape) == (leading[lead], *trailing), name
        assert value.device == d["positions"].device and value.is_contiguous(), name
        assert bool(torch.isfinite(value).all()), name
    per_pixel = fields["offsets"].diff()
    assert int(fields["offsets"][0]) == 0 and int(fields["offsets"][-1]) == total and int(per_pixel.min()) >= 0
    if total == 0:
        return
    ids, raw = fields["ids"], fields["raw"]
    assert int(ids.min()) >= 0 and int(ids.max()) < d["positions"].shape[0]
    transmittance_and_alpha = raw[:, 4:6]
    assert float(transmittance_and_alpha.min()) >= 0. and float(transmittance_and_alpha.max()) <= 1.
    torch.testing.assert_close(fields["gates"].sum(-1), torch.ones_like(raw[:, 0]), atol=2e-6, rtol=2e-6)
    pixel_of_record = torch.repeat_interleave(torch.arange(pixels, device=ids.device), per_pixel, output_size=total)
    assert torch.equal(fields["x6"][:, :3], d["rays_d"][pixel_of_record])


def _parity(actual, expected, precision, exact=False):
    """Reduced-precision records against the f32 records: topology (ids, offsets) and everything computed by the
    f32 geometry expressions (x6, gates, decay) bit for bit; image, alpha and the raw MLP outputs within the operand
    precision's tolerance -- or every field bit for bit when the MLP is constant."""
    names = [name for name, *_ in RECORD_FIELDS]
    got, want = dict(zip(names, actual)), dict(zip(names, expected))
    for name in ("ids", "offsets", "x6", "gates"):
        assert torch.equal(got[name], want[name]), name
    assert torch.equal(got["raw"][:, 6], want["raw"][:, 6]), "decay"
    if exact:
        for name in names:
            assert torch.equal(got[name], want[name]), name
        return
    tol = {"bfloat16": 3e-3, "float16": 5e-4}[precision]
    for name in ("rgb", "alpha", "raw"):
        torch.testing.assert_close(got[name], want[name], atol=tol, rtol=tol)


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
    from mlp_splatting_amd import record_training
    frame = record_training.Frame(9, 7, .001, 1.5, 2.)
    d = _case(device, 7, 9, 7, mosaic=True)
    monkeypatch.setenv("MLPSP_CSR_FORWARD_BACKEND", backend)
    before = _stats(ext)
    chosen = record_training.records_forward(ext, _args(d)[:15], frame)
    assert _delta(ext, before)["calls"] == 1
    direct = _render(ext, d, 9, 7, precision)
    for a, b in zip(chosen, direct):
        assert torch.equal(a, b)
    monkeypatch.setenv("MLPSP_CSR_FORWARD_BACKEND", "tensor_cores")
    with pytest.raises(ValueError, match="MLPSP_CSR_FORWARD_BACKEND"):
        record_training.records_forward(ext, _args(d)[:15], frame)


@pytest.mark.parametrize("precision", PRECISIONS)
def test_training_step_on_matrix_core_records(ext, device, monkeypatch, precision):
    """The record-based training step on the reduced-precision records: the 512-channel attribute gradient equals autograd
    through a dense framebuffer of those very records, and no MLP-input adjoint exists."""
    from mlp_splatting_amd import cumodel
    from mlp_splatting_amd.record_training import Frame, feature_training_step
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
    rgb, feature_loss = feature_training_step(base, attributes, target, Frame(9, 7, .001, 1.5, 2.), None)
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
