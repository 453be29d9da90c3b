"""The C-ABI library loads on a machine without a GPU and exports exactly what include/mlpsp.h declares."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "mlpsp.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mlpsp_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = _declared_functions()
    for required in ("mlpsp_validate_tile_lists", "mlpsp_bin_legacy_count", "mlpsp_bin_legacy_fill", "mlpsp_sort_tiles",
                     "mlpsp_render_tilecenter_f32", "mlpsp_render_tilecenter_feat_f32", "mlpsp_render_per_pixel_f32",
                     "mlpsp_bin_raycone_count", "mlpsp_prepare_primitives", "mlpsp_strerror"):
        assert required in names


def test_library_exports_every_declared_symbol():
    from mlp_splatting_amd import _lib
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared_functions():
        assert hasattr(lib, name), f"{name} is declared in include/mlpsp.h but not exported"


def test_python_binding_covers_the_header_and_nothing_else():
    from mlp_splatting_amd import _lib
    assert sorted(_lib.SIGNATURES) == _declared_functions()
    _lib.load()


def test_status_constants_agree_with_the_header():
    from mlp_splatting_amd import _lib
    text = open(os.path.join(ROOT, "include", "mlpsp.h")).read()
    consts = dict(re.findall(r"#define\s+MLPSP_(\w+)\s+(\d+)", text))
    assert int(consts["E_OFFSETS"]) == _lib.E_OFFSETS == 1
    assert int(consts["E_CAPACITY"]) == _lib.E_CAPACITY == 2
    assert int(consts["E_IDS"]) == _lib.E_IDS == 4
    assert int(consts["E_PIXEL_OVERFLOW"]) == _lib.E_PIXEL_OVERFLOW
    assert int(consts["E_NONFINITE"]) == _lib.E_NONFINITE
    assert int(consts["E_SCRATCH"]) == _lib.E_SCRATCH
    assert int(consts["E_MIXED_ORIGINS"]) == _lib.E_MIXED_ORIGINS
    assert int(consts["E_WIDE_CONE"]) == _lib.E_WIDE_CONE
    assert int(consts["TILE_CAPACITY_MAX"]) == _lib.TILE_CAPACITY_MAX
    assert int(consts["PIXEL_HIT_CAPACITY"]) == _lib.PIXEL_HIT_CAPACITY == 256
    assert int(consts["PRIM_RECORD_BYTES"]) == _lib.PRIM_RECORD_BYTES
    assert int(consts["VERSION"]) == _lib.VERSION == _lib.load().mlpsp_version()


def test_error_messages_carry_the_reference_wording():
    from mlp_splatting_amd import _lib
    assert "tile_offsets must start at zero" in _lib.strerror(_lib.E_OFFSETS)
    assert "candidate primitive IDs must be in" in _lib.strerror(_lib.E_IDS)
    assert "per-pixel intersection capacity 256 exceeded" in _lib.strerror(_lib.E_PIXEL_OVERFLOW)
    assert "capacity" in _lib.strerror(_lib.E_CAPACITY)


def test_size_queries_need_no_gpu():
    from mlp_splatting_amd import _lib
    lib = _lib.load()
    assert lib.mlpsp_version() == _lib.VERSION
    assert lib.mlpsp_per_pixel_workspace_bytes(160, 120, 8, 8) == 300 * 64 * 256 * 8 + 256
    assert lib.mlpsp_per_pixel_workspace_bytes(0, 120, 8, 8) == 0
    assert lib.mlpsp_bin_scratch_bytes(5000, 1, 160, 120, 8) > 5000 * 16
    assert lib.mlpsp_bin_raycone_scratch_bytes(5000, 160, 120, 8) > 5000 * 16


def test_product_sources_never_reach_into_the_oracle():
    # the shipped package and the library sources must not import, include or open anything under oracle/
    pkg = os.path.join(ROOT, "mlp_splatting_amd")
    for dirpath, _dirs, files in os.walk(pkg):
        if os.path.basename(dirpath) == "build":
            continue
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h", "Makefile")):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(import|from)\s+oracle\b", text, flags=re.M), f
                assert "oracle/" not in text and "mlpsp_oracle" not in text, f
