"""The extension object's contract, case for case as the reference's renderer tests state it
(tests/test_cuda_renderer.py:250-388, tests/test_candidate_capacity.py, tests/test_training_wmma.py:370-386):
capacity and id errors are raised before any render kernel runs, with the reference's wording, and
the device stays usable afterwards."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tile_ext(device):
    from mlp_splatting_amd.tile_ext import TileExt
    return TileExt()


def _renderer_inputs(n, device):
    hidden, frequencies = 1, 1
    encoded = 12 * frequencies
    positions = torch.zeros((n, 3), device=device)
    positions[:, 2] = 1.0
    quats = torch.zeros((n, 4), device=device)
    quats[:, 0] = 1.0
    return {
        "rays_o": torch.zeros((1, 3), device=device), "rays_d": torch.tensor([[0.0, 0.0, 1.0]], device=device),
        "positions": positions, "log_scales": torch.zeros((n, 3), device=device), "quats": quats,
        "candidates": torch.arange(n, device=device, dtype=torch.int32),
        "offsets": torch.tensor([0, n], device=device, dtype=torch.int32),
        "freq": torch.ones(frequencies, device=device), "attenuation": torch.ones(frequencies, device=device),
        "W1": torch.zeros((n, hidden, encoded), device=device), "b1": torch.zeros((n, hidden), device=device),
        "W2": torch.zeros((n, hidden, hidden), device=device), "b2": torch.zeros((n, hidden), device=device),
        "W3": torch.zeros((n, 4, hidden), device=device), "b3": torch.zeros((n, 4), device=device),
        "feat_attr": torch.zeros((n, 4, 2), device=device),
        "grad_rgb": torch.ones((1, 3), device=device), "grad_t": torch.zeros(1, device=device),
        "grad_feat": torch.ones((1, 2), device=device),
    }


def _base(d):
    return tuple(d[k] for k in ("rays_o", "rays_d", "positions", "log_scales", "quats", "candidates", "offsets", "freq",
                                "attenuation", "W1", "b1", "W2", "b2", "W3", "b3"))


DIMS = (1, 1, 1, 1, 1.0e-3)
PLAIN = {"render_tiles_forward", "render_tiles_autograd", "render_tiles_autograd_tilecenter",
         "render_tiles_autograd_tilecenter_presorted", "render_tiles_forward_tilecenter",
         "render_tiles_forward_tilecenter_with_t"}
BACKWARD_COUNT = {"render_tiles_backward_count_per_pixel", "render_tiles_backward_count_tilecenter"}
PER_PIXEL_BACKWARD = ["render_tiles_backward_count_per_pixel", "render_tiles_backward_emit_per_pixel",
                      "render_tiles_backward_featattr_per_pixel"]
TILECENTER_BACKWARD = ["render_tiles_backward_count_tilecenter", "render_tiles_backward_emit_tilecenter",
                       "render_tiles_backward_featattr_tilecenter", "render_tiles_backward_tilecenter_full",
                       "render_tiles_backward_tilecenter_full_with_feat"]
ALL_FORWARD = sorted(PLAIN | {"render_tiles_forward_per_pixel_with_feat", "render_tiles_forward_tilecenter_with_feat",
                              "render_tiles_forward_tilecenter_stats"})


def _invoke(ext, name, d):
    base = _base(d)
    if name in PLAIN:
        return getattr(ext, name)(*base, *DIMS)
    if name in ("render_tiles_forward_per_pixel_with_feat", "render_tiles_forward_tilecenter_with_feat"):
        return getattr(ext, name)(*base, d["feat_attr"], 1.0, 1.0, *DIMS)
    if name in BACKWARD_COUNT:
        return (getattr(ext, name)(*base, *DIMS),)
    if name in ("render_tiles_backward_featattr_per_pixel", "render_tiles_backward_featattr_tilecenter"):
        return (getattr(ext, name)(*base, d["feat_attr"], d["grad_feat"], 1.0, 1.0, *DIMS),)
    if name in ("render_tiles_backward_emit_per_pixel", "render_tiles_backward_emit_tilecenter"):
        n = d["positions"].shape[0]
        counts = torch.full((1,), n, device=d["positions"].device, dtype=torch.int32)
        record_offsets = torch.zeros(1, device=d["positions"].device, dtype=torch.int32)
        return getattr(ext, name)(*base, d["grad_rgb"], d["grad_t"], counts, record_offsets, n, *DIMS)
    if name == "render_tiles_backward_tilecenter_full":
        return ext.render_tiles_backward_tilecenter_full(*base, d["grad_rgb"], d["grad_t"], *DIMS)
    if name == "render_tiles_backward_tilecenter_full_with_feat":
        return ext.render_tiles_backward_tilecenter_full_with_feat(*base, d["feat_attr"], d["grad_rgb"], d["grad_t"],
                                                                   d["grad_feat"], 1.0, 1.0, *DIMS)
    if name == "render_tiles_forward_tilecenter_stats":
        n = d["positions"].shape[0]
        dev = d["positions"].device
        stats = [torch.zeros(n, device=dev, dtype=dt) for dt in (torch.float32, torch.float32, torch.int32, torch.float32, torch.int32)]
        return ext.render_tiles_forward_tilecenter_stats(*base[:9], d["freq"].numel(), *base[9:], n, d["W2"].shape[1],
                                                         d["W1"].shape[2], *DIMS, torch.ones((1, 3), device=dev), *stats)
    raise AssertionError(name)


@pytest.mark.parametrize("name,capacity,error", [
    ("render_tiles_autograd", 256, "per-pixel intersection capacity 256 exceeded"),
    ("render_tiles_forward", 256, "per-pixel intersection capacity 256 exceeded"),
    ("render_tiles_forward_per_pixel_with_feat", 256, "per-pixel intersection capacity 256 exceeded"),
    ("render_tiles_forward_tilecenter", 1536, "tile candidate capacity 1536 exceeded"),
    ("render_tiles_forward_tilecenter_with_feat", 1536, "tile candidate capacity 1536 exceeded"),
    ("render_tiles_forward_tilecenter_with_t", 1536, "tile candidate capacity 1536 exceeded"),
    ("render_tiles_autograd_tilecenter", 1536, "tile candidate capacity 1536 exceeded"),
])
def test_entry_points_fail_explicitly_on_capacity_overflow(tile_ext, device, name, capacity, error):
    with pytest.raises(RuntimeError, match=error):
        _invoke(tile_ext, name, _renderer_inputs(capacity + 1, device))
    torch.cuda.synchronize()


def test_capacity_error_reports_the_observed_length(tile_ext, device):
    with pytest.raises(RuntimeError, match=r"maximum observed tile length 1600\); refusing to truncate"):
        _invoke(tile_ext, "render_tiles_forward_tilecenter", _renderer_inputs(1600, device))


@pytest.mark.parametrize("name,capacity", [("render_tiles_forward", 256), ("render_tiles_forward_tilecenter", 512),
                                           ("render_tiles_forward_tilecenter", 1536)])
def test_capacity_boundary_is_accepted(tile_ext, device, name, capacity):
    outputs = _invoke(tile_ext, name, _renderer_inputs(capacity, device))
    assert all(torch.isfinite(o).all() for o in outputs)


@pytest.mark.parametrize("name", ["render_tiles_autograd", "render_tiles_forward", "render_tiles_forward_per_pixel_with_feat"])
def test_per_pixel_allows_large_tile_candidate_lists_when_hits_fit(tile_ext, device, name):
    d = _renderer_inputs(386, device)
    d["positions"][256:, 0] = 100.0
    outputs = _invoke(tile_ext, name, d)
    assert all(torch.isfinite(o).all() for o in outputs)


@pytest.mark.parametrize("name", ["render_tiles_forward_per_pixel_with_feat", "render_tiles_forward_tilecenter_with_feat"])
def test_removed_eight_slot_cube_gating_is_rejected(tile_ext, device, name):
    d = _renderer_inputs(1, device)
    d["feat_attr"] = torch.zeros((1, 8, 2), device=device)
    with pytest.raises(RuntimeError, match=r"slots in \{4,5\}"):
        _invoke(tile_ext, name, d)


def test_feature_dimension_limit(tile_ext, device):
    d = _renderer_inputs(1, device)
    d["feat_attr"] = torch.zeros((1, 4, 513), device=device)
    with pytest.raises(RuntimeError, match="must be <= 512"):
        _invoke(tile_ext, "render_tiles_forward_tilecenter_with_feat", d)


def test_tile_offsets_must_cover_the_candidate_list(tile_ext, device):
    d = _renderer_inputs(2, device)
    d["offsets"] = torch.tensor([1, 2], device=device, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="tile_offsets must start at zero"):
        _invoke(tile_ext, "render_tiles_forward", d)
    d["offsets"] = torch.tensor([0, 1, 2], device=device, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="tile_offsets length mismatch"):
        _invoke(tile_ext, "render_tiles_forward_tilecenter", d)


@pytest.mark.parametrize("name", ALL_FORWARD)
@pytest.mark.parametrize("invalid_id", [-1, 2])
def test_entry_points_reject_invalid_primitive_ids_before_rendering(tile_ext, device, name, invalid_id):
    d = _renderer_inputs(2, device)
    d["candidates"][0] = invalid_id
    with pytest.raises(RuntimeError, match="candidate primitive IDs must be in"):
        _invoke(tile_ext, name, d)
    torch.cuda.synchronize()   # an illegal access would surface here


@pytest.mark.parametrize("name", ["render_tiles_forward", "render_tiles_forward_tilecenter"])
@pytest.mark.parametrize("n", [0, 2])
def test_primitive_id_boundaries_and_empty_scene_are_accepted(tile_ext, device, name, n):
    outputs = _invoke(tile_ext, name, _renderer_inputs(n, device))
    assert all(torch.isfinite(o).all() for o in outputs)
    if n == 0:
        assert all(not o.any() for o in outputs)


def test_presorted_streams_and_validates_candidates_beyond_shared_capacity(tile_ext, device):
    d = _renderer_inputs(1537, device)
    d["positions"][:-1, 0] = 100.0
    d["b3"][:, 3] = 1.0
    one = _renderer_inputs(1, device)
    one["b3"][:, 3] = 1.0
    name = "render_tiles_autograd_tilecenter_presorted"
    expected = _invoke(tile_ext, name, one)
    actual = _invoke(tile_ext, name, d)
    assert expected[1].item() > 0
    for value, reference in zip(actual, expected):
        torch.testing.assert_close(value, reference, rtol=0, atol=0)
    for invalid_id in (-1, 1537):
        d["candidates"][-1] = invalid_id
        with pytest.raises(RuntimeError, match="candidate primitive IDs must be in"):
            _invoke(tile_ext, name, d)
        torch.cuda.synchronize()


@pytest.mark.parametrize("n", [768, 769, 1024, 1536])
def test_only_the_last_candidate_hits_is_not_truncated(tile_ext, device, n):
    d = _renderer_inputs(n, device)
    d["positions"][:-1, 0] = 100.0
    d["b3"][:] = torch.tensor([0.5, 0.5, 0.5, 2.0], device=device)
    one = _renderer_inputs(1, device)
    one["b3"][:] = torch.tensor([0.5, 0.5, 0.5, 2.0], device=device)
    got = _invoke(tile_ext, "render_tiles_forward_tilecenter", d)
    want = _invoke(tile_ext, "render_tiles_forward_tilecenter", one)
    assert want[1].item() > 0
    for a, b in zip(got, want):
        torch.testing.assert_close(a, b, rtol=0, atol=0)


def test_stable_depth_ties_follow_list_order(tile_ext, device):
    n = 12
    d = _renderer_inputs(n, device)
    d["b3"][:, 3] = 8.0
    d["b3"][:, 0] = torch.linspace(-3, 3, n, device=device)
    d["candidates"] = torch.arange(n - 1, -1, -1, device=device, dtype=torch.int32)
    rgb, alpha = _invoke(tile_ext, "render_tiles_forward_tilecenter", d)
    assert abs(float(rgb[0, 0] / alpha[0, 0]) - float(torch.sigmoid(d["b3"][11, 0]))) < 1e-5


def test_closed_form_geometric_series(tile_ext, device):
    import math
    d = _renderer_inputs(40, device)
    b3 = [0.3, -0.4, 1.1, 0.2]
    d["b3"][:] = torch.tensor(b3, device=device)
    rgb, alpha = _invoke(tile_ext, "render_tiles_forward_tilecenter", d)
    a = 1 - math.exp(-math.log1p(math.exp(b3[3])))
    k = next(i for i in range(1, 100) if (1 - a) ** i < 1e-3)
    colour = 1 / (1 + np.exp(-np.array(b3[:3])))
    np.testing.assert_allclose(rgb.cpu().numpy()[0], colour * (1 - (1 - a) ** k), atol=2e-6)
    assert abs(alpha.item() - (1 - (1 - a) ** k)) < 2e-6


def test_stored_half_precision_weights_are_widened_exactly(tile_ext, device):
    d = _renderer_inputs(3, device)
    d["b3"][:] = torch.tensor([0.25, -0.5, 1.0, 0.75], device=device)      # exactly representable in bf16 and fp16
    want = _invoke(tile_ext, "render_tiles_forward_tilecenter", d)
    for dt in (torch.float16, torch.bfloat16):
        dd = dict(d)
        for k in ("W1", "b1", "W2", "b2", "W3", "b3"):
            dd[k] = d[k].to(dt)
        got = _invoke(tile_ext, "render_tiles_forward_tilecenter", dd)
        for a, b in zip(got, want):
            torch.testing.assert_close(a, b, rtol=0, atol=0)
    dd = dict(d)
    dd["W1"] = d["W1"].half()
    with pytest.raises(RuntimeError, match="share the same dtype"):
        _invoke(tile_ext, "render_tiles_forward_tilecenter", dd)


def test_kernels_run_on_the_current_stream(tile_ext, device):
    # tests/test_training_wmma.py:370-386: work is enqueued on the caller's current stream
    d = _renderer_inputs(4, device)
    d["b3"][:, 3] = 0.5
    want = _invoke(tile_ext, "render_tiles_forward_tilecenter", d)
    side = torch.cuda.Stream(device=device)
    side.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(side):
        got = _invoke(tile_ext, "render_tiles_forward_tilecenter", d)
    side.synchronize()
    for a, b in zip(got, want):
        torch.testing.assert_close(a, b, rtol=0, atol=0)


def test_inputs_are_not_mutated(tile_ext, device):
    d = _renderer_inputs(5, device)
    before = {k: v.clone() for k, v in d.items()}
    _invoke(tile_ext, "render_tiles_forward_tilecenter_with_feat", d)
    _invoke(tile_ext, "render_tiles_forward", d)
    for k, v in d.items():
        assert torch.equal(v, before[k]), k


@pytest.mark.parametrize("name", PER_PIXEL_BACKWARD + TILECENTER_BACKWARD)
def test_backward_entry_points_follow_the_forward_contracts(tile_ext, device, name):
    """tests/test_cuda_renderer.py:250-371 for the backward entry points: capacity refusals (256 hits per pixel /
    1,536 candidates per tile), 386 candidates with 256 hits accepted in per-pixel order, invalid ids rejected
    before anything runs, finite outputs on a valid stack."""
    per_pixel = name in PER_PIXEL_BACKWARD
    error = "per-pixel intersection capacity 256 exceeded" if per_pixel else "tile candidate capacity 1536 exceeded"
    with pytest.raises(RuntimeError, match=error):
        _invoke(tile_ext, name, _renderer_inputs((256 if per_pixel else 1536) + 1, device))
    for invalid in (-1, 2):
        d = _renderer_inputs(2, device)
        d["candidates"][0] = invalid
        with pytest.raises(RuntimeError, match="candidate primitive IDs must be in"):
            _invoke(tile_ext, name, d)
    torch.cuda.synchronize()
    d = _renderer_inputs(386 if per_pixel else 300, device)
    if per_pixel:
        d["positions"][256:, 0] = 100.0
    outputs = _invoke(tile_ext, name, d)
    assert all(torch.isfinite(o).all() for o in outputs)
    if "featattr" in name:
        d = _renderer_inputs(1, device)
        d["feat_attr"] = torch.zeros((1, 8, 2), device=device)
        with pytest.raises(RuntimeError, match=r"slots in \{4,5\}"):
            _invoke(tile_ext, name, d)


def test_emit_entry_points_return_the_adjoints_of_the_activated_outputs(tile_ext, device):
    """np_tile_kernels.cu:1568-1836: out_grad_rgb = T alpha grad_out_rgb[pixel]; out_grad_sigma_raw = the adjoint of
    softplus(o3).  On a stack of identical zero-weight primitives along one ray (R = G = B = 1/2, sigma_raw = ln 2)
    both have closed forms: alpha = 1 - 2^-decay with decay = 1, T_k = 2^-k, and with grad_out_rgb = 1, grad_t = 0
    the colour adjoint of record k is T_k alpha and d loss / d sigma_raw_k = -(1 - alpha) * sum_{j>k} T_j alpha 3/2
    + T_k (1 - alpha) 3/2."""
    n = 6
    d = _renderer_inputs(n, device)
    for name in ("render_tiles_backward_emit_per_pixel", "render_tiles_backward_emit_tilecenter"):
        out = _invoke(tile_ext, name, d)
        ids, x6, g_rgb, g_sigma = out[:4]
        assert len(out) == (7 if "per_pixel" in name else 6)
        assert ids.cpu().tolist() == list(range(n)) and tuple(x6.shape) == (n, 6)
        alpha = 0.5
        trans = torch.tensor([0.5 ** k for k in range(n)], dtype=torch.float64)
        torch.testing.assert_close(g_rgb.cpu().double(), (trans * alpha)[:, None].expand(n, 3), atol=1e-6, rtol=1e-5)
        colour = 1.5                                        # sum over channels of grad_out_rgb * (R, G, B)
        later = torch.stack([(trans[k + 1:] * alpha * colour).sum() for k in range(n)])
        # d/d sigma_k: alpha_k' = (1 - alpha) decay; the hit's own term T_k colour alpha_k', and every later term
        # scaled by (1 - alpha_k) loses (1 - alpha) decay / (1 - alpha_k) of itself
        want = (1 - alpha) * trans * colour - later
        torch.testing.assert_close(g_sigma.cpu().double().flatten(), want, atol=1e-6, rtol=1e-5)


def test_backward_entry_points_that_are_not_built_say_so(tile_ext):
    with pytest.raises(NotImplementedError, match="fused backward entry points"):
        tile_ext.render_tiles_backward_tilecenter_traversal()
    assert callable(tile_ext.render_tiles_backward_tilecenter_full) and callable(tile_ext.primitive_records_reverse)
    with pytest.raises(AttributeError):
        tile_ext.no_such_entry_point
