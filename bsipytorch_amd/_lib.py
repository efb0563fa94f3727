"""ctypes binding of ``libbsi_hip.so`` (the C ABI declared in ``include/bsi_hip.h``).

The library is the only compute path: if it is missing or fails to load, importing this module
raises -- there is no CPU or PyTorch fallback.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# BSI_HIP_LIBRARY names another build of the same library (the timeline build, say); it must exist like the default.
LIB_PATH = os.environ.get("BSI_HIP_LIBRARY") or os.path.join(_HERE, "libbsi_hip.so")

BSI_OK = 0
DTYPE_F32, DTYPE_F16, DTYPE_BF16 = 0, 1, 2
CORE_AUTO, CORE_VALU, CORE_MFMA = 0, 1, 2
LAYOUT_CANONICAL, LAYOUT_TILED16, LAYOUT_INT8, LAYOUT_INT8_TILED = 0, 1, 2, 3
OPT_I8_TILE = 1
OPT_DIGITS_ROUTE = 2
OPT_BUILD_ITEMS = 3
OPT_OUTPUT_STORES = 4
OPT_I8_SPLIT = 5

_vp = ctypes.c_void_p
_i = ctypes.c_int
_i64 = ctypes.c_int64
_f = ctypes.c_float
_d = ctypes.c_double
_sz = ctypes.c_size_t

# name -> argument types, in header order (all return int unless listed in _RESTYPES)
PROTOTYPES = {
    "bsi_hip_device_info": [ctypes.c_char_p, _i, ctypes.POINTER(_i), ctypes.POINTER(_i)],
    "bsi_hip_quantize_round_to_int64": [_vp, _i, _i64, _d, _vp, _vp],
    "bsi_hip_compute_row_shift_scale": [_vp, _i64, _i64, _i, _f, _vp, _vp, _vp],
    "bsi_hip_compute_chunk_shift_scale": [_vp, _i64, _i64, _i, _i, _f, _vp, _vp, _vp],
    "bsi_hip_apply_row_shift_clamp": [_vp, _i64, _i64, _vp, _i, _vp],
    "bsi_hip_apply_chunk_shift_clamp": [_vp, _i64, _i64, _i, _vp, _i, _vp],
    "bsi_hip_compute_row_shift_scale_from_input": [_vp, _i, _i64, _i64, _d, _i, _f, _vp, _vp, _vp],
    "bsi_hip_compute_chunk_shift_scale_from_input": [_vp, _i, _i64, _i64, _i, _d, _i, _f, _vp, _vp, _vp],
    "bsi_hip_quantize_shift_pack_row_batch": [_vp, _i, _i64, _i64, _i, _i, _d, _i, _vp, _vp, _vp],
    "bsi_hip_quantize_shift_pack_chunk_batch": [_vp, _i, _i64, _i64, _i, _i, _i, _d, _i, _vp, _vp, _vp],
    "bsi_hip_pack_bits_batch": [_vp, _i64, _i64, _i, _i, _vp, _vp],
    "bsi_hip_decimal_stats": [_vp, _i64, _i64, _vp, _vp, _vp],
    "bsi_hip_build_fixed": [_vp, _i, _i64, _i64, _i, _i, _i, _f, _vp, _vp, _vp, _vp, _vp],
    "bsi_hip_slice_popcount_sum": [_vp, _i, _i, _vp, _vp],
    "bsi_hip_compress_flags_from_density": [_vp, _i, _i, _d, _vp, _vp],
    "bsi_hip_ewah_size": [_vp, _i, _i, _vp, _vp, _vp],
    "bsi_hip_ewah_emit": [_vp, _i, _i, _vp, _vp, _vp, _vp, _vp],
    "bsi_hip_ewah_decompress": [_vp, _i, _i, _vp, _vp],
    "bsi_hip_ewah_decompress_batch": [_vp, _vp, _vp, _i, _i, _vp, _vp],
    "bsi_hip_tile_key_planes": [_vp, _i64, _i, _i, _vp, _vp],
    "bsi_hip_planes_to_int8": [_vp, _i64, _i, _i, _vp, _vp],
    "bsi_hip_set_option": [_i, _i],
    "bsi_hip_stream_capture_id": [_vp, ctypes.POINTER(ctypes.c_ulonglong)],
    "bsi_hip_dot_workspace_bytes": [_i64, _i, _i],
    "bsi_hip_dot_split_scratch_bytes": [],
    "bsi_hip_dot_attach_split_scratch": [_vp, _sz],
    "bsi_hip_dot_split_plan": [_i64, _i64, _i, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)],
    "bsi_hip_dot": [_vp, _vp, _vp, _i, _i, _i, _vp, _i, _vp, _i, _i64, _i64, _f, _i64, _vp, _vp, _i, _vp, _sz, _vp],
    "bsi_hip_dot_static_scratch": [_vp, _vp, _i, _i, _i, _vp, _i, _vp, _i, _i64, _i64, _f, _i64, _vp, _vp, _vp],
    "bsi_hip_add_bias": [_vp, _vp, _i64, _i64, _i64, _vp],
    "bsi_hip_dot_bias": [_vp, _vp, _vp, _i, _i, _i, _vp, _i, _vp, _i, _i64, _i64, _f, _i64, _vp, _vp, _i, _vp, _sz, _vp],
    "bsi_hip_dot_bias_warm": [_vp, _vp, _vp, _i, _i, _i, _vp, _i, _vp, _i, _i64, _i64, _f, _i64, _vp, _vp, _i, _vp, _sz, _vp, _sz, _vp],
    "bsi_hip_linear_few_rows": [_vp, _i, _i64, _i64, _i, _i, _vp, _vp, _i, _i64, _f, _i64, _vp, _vp, _vp],
    "bsi_hip_linear_few_rows_upfront": [_i64, _i64, _i64],
    "bsi_hip_linear_workspace_bytes": [_i64, _i64, _i],
    "bsi_hip_linear": [_vp, _i, _i64, _i64, _i, _i, _i, _vp, _sz, _vp, _i, _vp, _i, _i64, _f, _i64, _vp, _vp, _i, _vp,
                       _sz, _vp],
    "bsi_hip_dot_ewah_query": [_vp, _vp, _vp, _i, _i, _vp, _i, _vp, _vp, _i, _i64, _f, _vp, _vp, _vp],
    "bsi_hip_dot_ewah_batch_workspace_bytes": [_i64, _i],
    "bsi_hip_dot_ewah_batch": [_vp, _vp, _vp, _i, _i, _vp, _i, _vp, _i, _vp, _i, _i64, _i64, _f, _i64, _vp, _vp, _vp, _vp,
                               _sz, _vp],
    "bsi_hip_planes_to_int8_digits": [_vp, _i64, _i, _i, _vp, _vp],
    "bsi_hip_dot_digits_workspace_bytes": [_i64, _i, _i64, _i],
    "bsi_hip_dot_digits": [_vp, _i, _vp, _i, _vp, _i, _i, _vp, _i, _i, _i64, _i64, _vp, _f, _i64, _vp, _vp, _vp,
                           _sz, _i, _vp],
    "bsi_hip_int8_tiled_bytes": [_i64, _i],
    "bsi_hip_planes_to_int8_tiled": [_vp, _i64, _i, _i, _vp, _vp],
    "bsi_hip_dot_weighted": [_vp, _vp, _i, _i, _vp, _i, _vp, _i, _i64, _i64, _vp, _f, _i64, _vp, _vp],
    "bsi_hip_dot_weighted_f64": [_vp, _vp, _i, _i, _vp, _i, _vp, _i, _i64, _i64, _vp, _i64, _vp, _vp],
    "bsi_hip_quantize_trunc_to_int64": [_vp, _i, _i64, _f, _vp, _vp],
    "bsi_hip_dot_timed": [_vp, _vp, _vp, _i, _i, _i, _vp, _i, _vp, _i, _i64, _i64, _f, _i64, _vp, _i, _vp, _sz, _i,
                          ctypes.POINTER(_f), _vp],
    "bsi_hip_probe_valu_popcount": [ctypes.POINTER(_d), _vp],
    "bsi_hip_probe_mfma_i8": [ctypes.POINTER(_d), _vp],
    "bsi_hip_probe_mfma_i8_operands": [_i, ctypes.POINTER(_d), _vp],
    "bsi_hip_probe_stream_read": [_vp, _sz, ctypes.POINTER(_d), _vp],
    "bsi_hip_probe_l2_to_lds": [_vp, _sz, _i, ctypes.POINTER(_d), _vp],
    "bsi_hip_timeline_read": [ctypes.POINTER(ctypes.c_ulonglong), _i],
    "bsi_hip_timeline_read_cycles": [ctypes.POINTER(ctypes.c_ulonglong), _i],
    "bsi_hip_version": [],
    "bsi_hip_last_error": [],
}
_RESTYPES = {
    "bsi_hip_version": ctypes.c_char_p,
    "bsi_hip_last_error": ctypes.c_char_p,
    "bsi_hip_dot_workspace_bytes": _sz,
    "bsi_hip_dot_split_scratch_bytes": _sz,
    "bsi_hip_dot_ewah_batch_workspace_bytes": _sz,
    "bsi_hip_linear_workspace_bytes": _sz,
    "bsi_hip_dot_digits_workspace_bytes": _sz,
    "bsi_hip_int8_tiled_bytes": _sz,
}


class BsiHipError(RuntimeError):
    """An entry point of libbsi_hip.so returned a non-zero code."""


def _load() -> ctypes.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C bsipytorch_amd/csrc`. There is no fallback path.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in PROTOTYPES.items():
        fn = getattr(lib, name)  # AttributeError here = the library does not export a declared symbol
        fn.argtypes = argtypes
        fn.restype = _RESTYPES.get(name, ctypes.c_int)
    return lib


lib = _load()


def check(rc: int, what: str) -> None:
    if rc != BSI_OK:
        msg = lib.bsi_hip_last_error()
        raise BsiHipError(f"{what}: {msg.decode() if msg else 'error'} (code {rc})")


def version() -> str:
    return lib.bsi_hip_version().decode()
