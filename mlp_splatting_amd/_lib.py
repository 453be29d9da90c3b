"""ctypes binding of ``libmlpsp_hip.so`` (the C ABI declared in ``include/mlpsp.h``).

The library is built in-tree by ``mlp_splatting_amd/csrc/Makefile``.  There is no fallback: if the
shared object is missing or does not export a declared symbol, loading raises.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmlpsp_hip.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

E_OFFSETS, E_CAPACITY, E_IDS, E_PIXEL_OVERFLOW, E_NONFINITE, E_ARGUMENT, E_RUNTIME, E_SCRATCH = 1, 2, 4, 8, 16, 32, 64, 128
E_MIXED_ORIGINS, E_WIDE_CONE = 256, 512
KEY_LIST_ORDER, KEY_TSTAR, KEY_DEPTH = 0, 1, 2
TILE_CAPACITY_MAX = 2048
PIXEL_HIT_CAPACITY = 256
PRIM_RECORD_BYTES = 128
MFMA_PACK_BYTES = 7808
VERSION = 303      # MLPSP_VERSION of include/mlpsp.h: the interface this binding was written against
STAGE_STATUS_IS_CLEAR = 4

_vp, _i, _f, _i64, _sz = C.c_void_p, C.c_int, C.c_float, C.c_int64, C.c_size_t

# name -> (restype, argtypes); one entry per function declared in include/mlpsp.h
SIGNATURES = {
    "mlpsp_version": (_i, []),
    "mlpsp_strerror": (C.c_char_p, [_i]),
    "mlpsp_prepare_primitives": (_i, [_vp, _vp, _vp, _i, _vp, _vp]),
    "mlpsp_normalize_rays": (_i, [_vp, _i64, _vp, _vp]),
    "mlpsp_validate_tile_lists": (_i, [_vp, _vp, _i, _i, _i, _i, _vp, C.POINTER(C.c_int32), _vp]),
    "mlpsp_bin_scratch_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "mlpsp_bin_legacy_count": (_i, [_vp, _vp, _i, C.POINTER(_f), _i, _vp, C.POINTER(_f), _i, _i, _i, _f, _vp, _sz, _vp,
                                    C.POINTER(_i64), _vp]),
    "mlpsp_bin_legacy_async_device_matrices": (_i, [_vp, _vp, _i, _vp, _vp, _i, _i, _i, _f, _vp, _sz, _vp, _vp, _i64, _vp,
                                                     _vp]),
    "mlpsp_bin_segments_async_device_matrices": (_i, [_vp, _vp, _i, _vp, _vp, _i, _i, _i, _f, _vp, _sz, _i, _vp, _vp, _vp,
                                                       _vp, _vp]),
    "mlpsp_bin_legacy_async": (_i, [_vp, _vp, _i, C.POINTER(_f), _i, _vp, C.POINTER(_f), _i, _i, _i, _f, _vp, _sz, _vp, _vp,
                                    _i64, _vp, _vp]),
    "mlpsp_bin_legacy_fill": (_i, [_i, _i, _vp, _i, _i, _i, _vp, _sz, _vp, _vp, _vp]),
    "mlpsp_bin_static_scratch_bytes": (_sz, []),
    "mlpsp_bin_legacy_async_noalloc": (_i, [_vp, _vp, _i, C.POINTER(_f), _i, _vp, C.POINTER(_f), _i, _i, _i, _f, _vp, _vp,
                                            _i64, _vp, _vp]),
    "mlpsp_bin_raycone_scratch_bytes": (_sz, [_i, _i, _i, _i]),
    "mlpsp_bin_raycone_count": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _f, _vp, _sz, _vp, C.POINTER(_i64), _vp]),
    "mlpsp_bin_raycone_fill": (_i, [_i, _i, _i, _i, _vp, _sz, _vp, _vp, _vp]),
    "mlpsp_sort_frame_records_bytes": (_sz, [_i]),
    "mlpsp_tile_pyramids_bytes": (_sz, [_i, _i, _i, _i]),
    "mlpsp_frame_prologue": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _i, _vp, _vp]),
    "mlpsp_sort_tiles": (_i, [_vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _vp, _i, _vp, _vp, _i, _vp, _vp,
                              _vp]),
    "mlpsp_render_tilecenter_f32": (_i, [_vp] * 7 + [_i] + [_vp] * 6 + [_i, _i, _i, _i, _i, _i, _f, _vp, _vp, _vp,
                                                                       _vp, _vp]),
    "mlpsp_render_tilecenter_feat_f32": (_i, [_vp] * 7 + [_i] + [_vp] * 6 + [_i, _i, _vp, _i, _i, _f, _f, _i, _i, _i, _i,
                                                                            _f, _i64, _vp, _sz, _vp, _vp, _vp, _vp, _vp]),
    "mlpsp_per_pixel_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "mlpsp_render_per_pixel_f32": (_i, [_vp] * 7 + [_i] + [_vp] * 6 + [_i, _i, _vp, _i, _i, _f, _f, _i, _i, _i, _i, _f,
                                                                      _vp, _sz, _vp, _vp, _vp, _vp]),
    "mlpsp_records_per_pixel_count": (_i, [_vp] * 7 + [_i] + [_vp] * 6 + [_i, _i, _i, _i, _i, _i, _f, _vp, _sz, _vp, _vp]),
    "mlpsp_records_per_pixel_emit": (_i, [_vp] * 7 + [_i] + [_vp] * 6 + [_i, _i, _f, _f, _i, _i, _i, _i, _f, _vp, _sz, _vp,
                                                                        _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "mlpsp_mfma_pack_bytes": (_sz, [_i]),
    "mlpsp_pack_mfma_weights": (_i, [_vp] * 6 + [_i, _i, _vp, _vp]),
    "mlpsp_pack_mfma_weights_half": (_i, [_vp] * 6 + [_i, _i, _vp, _vp]),
    "mlpsp_pack_mfma_feat_half": (_i, [_vp, _i, _i, _i, _vp, _vp, _vp]),
    "mlpsp_render_tilecenter_mfma": (_i, [_vp] * 8 + [_i, _i, _i, _i, _f, _vp, _vp, _vp, _vp, _vp]),
    "mlpsp_mfma_feat_pack_bytes": (_sz, [_i, _i, _i]),
    "mlpsp_pack_mfma_feat": (_i, [_vp, _i, _i, _i, _vp, _vp, _vp]),
    "mlpsp_render_tilecenter_stats_f32": (_i, [_vp] * 7 + [_i] + [_vp] * 6 + [_i, _i, _i, _i, _i, _i, _f] + [_vp] * 9),
    "mlpsp_records_count": (_i, [_vp] * 7 + [_i] + [_vp] * 6 + [_i, _i, _i, _i, _i, _i, _f, _i, _i, _vp, _vp, _vp]),
    "mlpsp_records_emit": (_i, [_vp] * 7 + [_i] + [_vp] * 6 + [_i, _i, _i, _i, _i, _i, _f, _i, _i, _f, _f] + [_vp] * 10),
    "mlpsp_records_mfma_count": (_i, [_vp] * 8 + [_i, _i, _i, _f, _i, _i, _vp, _vp, _vp]),
    "mlpsp_records_mfma_emit": (_i, [_vp] * 8 + [_i, _i, _i, _f, _i, _i, _f, _f, _vp, _i64] + [_vp] * 9),
    "mlpsp_all_finite": (_i, [_vp, _vp, _i, _vp, _vp]),
    "mlpsp_feat_workspace_bytes": (_sz, [_i64, _i, _i, _i, _i, _i, _i, _i64]),
    "mlpsp_render_tilecenter_mfma_feat": (_i, [_vp] * 5 + [_i64, _vp, _vp, _vp, _i, _i, _vp, _i, _i, _f, _f, _i, _i, _f,
                                               _vp, _sz, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp]),
    "mlpsp_probe_mfma_bf16": (_i64, [_i, _vp, _vp]),
    "mlpsp_probe_issue": (_i, [C.POINTER(C.c_int32), _i, _vp, _vp, _vp]),
    "mlpsp_grouped_vjp": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _f, _i, _vp,
                               _vp]),
    "mlpsp_segment_reduce_rows": (_i64, [_i64]),
    "mlpsp_reduce_partials": (_i, [_vp, _vp, _vp, _i64, _i, _vp, _vp, _vp]),
    "mlpsp_reduce_partials_split": (_i, [_vp, _vp, _vp, _i64, _i] + [_vp] * 8),
    "mlpsp_stream_feature_l1": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "mlpsp_feature_attribute_gradients": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i, _i, _i, _i, _i,
                                               _i, _i, _i, _i, _vp, _vp, _vp]),
    "mlpsp_feature_dense_attribute_gradients": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i, _i, _i,
                                                     _i, _vp, _vp, _vp]),
    "mlpsp_records_reverse_adjoints": (_i, [_vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp]),
    "mlpsp_geometry_gradients": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i, _i, _vp, _vp, _vp, _vp,
                                      _vp]),
    "mlpsp_records_reverse": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i, _vp, _vp, _vp, _vp, _vp]),
}

_lib = None


def build(verbose: bool = False) -> str:
    """Compile every HIP source for gfx950 into ``libmlpsp_hip.so`` (hipcc cross-compiles; no GPU needed)."""
    out = None if verbose else subprocess.DEVNULL
    subprocess.check_call(["make", "-C", CSRC_DIR, "-j8"], stdout=out, stderr=out)
    return LIB_PATH


def load():
    """Return the loaded library with argument types set; raise if it is absent or incomplete."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"libmlpsp_hip.so not found at {LIB_PATH}; build it with `make -C {CSRC_DIR}` "
            "(there is no CPU or PyTorch fallback for the renderer)")
    lib = C.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as exc:
            raise RuntimeError(f"libmlpsp_hip.so does not export {name}; rebuild the library") from exc
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.mlpsp_version() != VERSION:
        raise RuntimeError(f"libmlpsp_hip.so is version {lib.mlpsp_version()}, this binding expects {VERSION}: "
                           f"rebuild the library (`make -C {CSRC_DIR}`)")
    _lib = lib
    return lib


def strerror(code: int) -> str:
    return load().mlpsp_strerror(int(code)).decode()
