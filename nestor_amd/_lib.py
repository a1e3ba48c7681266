"""ctypes binding of ``libnestor_hip.so`` (the C ABI in ``include/nestor_hip.h``).

The library is loaded lazily on first use and a missing or stale build is a hard
error: there is no CPU or PyTorch fallback behind these entry points.
"""

from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_int32, c_int64, c_size_t, c_void_p
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libnestor_hip.so"
ABI_VERSION = 16

F32 = 0
BF16 = 1
ROW_ALIGN = 16
TILE_M = 128

_P = c_void_p
_I32 = c_int32
_I64 = c_int64

# name -> argument types (every function returns int unless listed in _RESTYPES)
_SIGNATURES: dict[str, list] = {
    "nestor_hip_abi_version": [],
    "nestor_hip_strerror": [_I32],
    "nestor_hip_index_build_workspace_bytes": [_I64, _I32],
    "nestor_hip_max_tiles": [_I64, _I32],
    "nestor_hip_index_build": [
        _P, _I64, _I32, _I32, _I64, _I64, _I32,  # ids rows banks slots rows_pad capacity valid_dtype
        _P, _P, _P, _P, _P,                      # order counts raw_starts padded_starts offs
        _P, _P, _P, _P, _P, _P,                  # row_dest pad_token pad_src_row eid_pad pad_valid row_kept
        _P, _I64, _P, c_size_t, _P,              # tile_table max_tiles workspace bytes stream
    ],
    "nestor_hip_index_build_static_capacity_bytes": [],
    "nestor_hip_index_build_static": [
        _P, _I64, _I32, _I32, _I64, _I64, _I32,
        _P, _P, _P, _P, _P,
        _P, _P, _P, _P, _P, _P,
        _P, _I64, _P,                            # tile_table max_tiles stream
    ],
    "nestor_hip_build_dispatch_maps": [
        _P, _P, _P, _P, _I64, _I32, _I32, _I64, _I32, _P, _P, _P, _P, _P, _P,
    ],
    "nestor_hip_tile_table_ints": [_I64, _I32],
    "nestor_hip_tile_schedule": [_P, _I32, _I64, _P, _I64, _P],
    "nestor_hip_dispatch_rows_fwd": [_P, _I32, _P, _P, _I32, _P, _I64, _I64, _P, _I64, _I32, _P],
    "nestor_hip_dispatch_rows_bwd": [_P, _P, _P, _I32, _I64, _I32, _I64, _P],
    "nestor_hip_swiglu_fwd": [_P, _P, _P, _I64, _I64, _I64, _I64, _P],
    "nestor_hip_swiglu_bwd": [_P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _P],
    "nestor_hip_cat_cast_fwd": [_P, _P, _P, _I64, _I64, _P],
    "nestor_hip_cat_cast_bwd": [_P, _P, _P, _I64, _I64, _P],
    "nestor_hip_combine_rows_fwd": [_P, _P, _P, _I32, _P, _I32, _I64, _I32, _I64, _I32, _P],
    "nestor_hip_combine_rows_bwd": [
        _P, _I32, _P, _P, _P, _I32, _P, _I32, _P, _P, _I64, _I32, _I64, _P, _I64, _P,
    ],
    "nestor_hip_grouped_gemm_nn": [_P, _P, _P, _I64, _I64, _I64, _I32, _P, _I64, _P],
    "nestor_hip_grouped_gemm_upgate_swiglu": [
        _P, _P, _P, _P, _P, _I64, _I64, _I64, _I32, _P, _I64, _P,
    ],
    "nestor_hip_grouped_gemm_nt": [_P, _P, _P, _I64, _I64, _I64, _I32, _P, _I64, _P],
    "nestor_hip_grouped_gemm_nt_upgate": [
        _P, _P, _P, _P, _I64, _I64, _I64, _I32, _P, _I64, _P,
    ],
    "nestor_hip_grouped_gemm_tn": [
        _P, _I64, _P, _I64, _P, _I64, _I64, _I64, _I64, _I64, _I32, _P, _P, _P, _I32, _P,
    ],
    "nestor_hip_grouped_gemm_tn_pair": [
        _P, _I64, _P, _I64, _P, _P, _I64, _I64, _I64, _I64, _I64, _I32, _P, _P, _P, _I32, _P,
    ],
    "nestor_hip_grouped_gemm_fp8w_nn": [_P, _P, _P, _P, _I64, _I64, _I64, _I32, _P, _I64, _I32, _P],
    "nestor_hip_grouped_gemm_fp8w_upgate_swiglu": [
        _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I32, _P, _I64, _I32, _P,
    ],
    "nestor_hip_router_topk": [
        _P, _I32, _P, _I32, _P, _P, _P, _P, _I64, _I32, _I32, _I32, _P,
    ],
    "nestor_hip_router_gates_bwd": [_P, _I32, _P, _P, _P, _P, _P, _I64, _I32, _I32, _I32, _P],
    "nestor_hip_router_choice_counts": [_P, _P, _P, _I64, _I32, _I32, _P],
    "nestor_hip_private_slots_fwd": [
        _P, _P, _I32, _P, _P, _P, _P, _P, _I64, _I32, _I32, _I32, _I32, _P,
    ],
    "nestor_hip_private_slots_bwd": [
        _P, _P, _P, _I32, _P, _P, _P, _P, _I64, _I32, _I32, _I32, _I32, _P,
    ],
    "nestor_hip_path_mix_fwd": [_P, _P, _P, _P, _I32, _I64, _I64, _P],
    "nestor_hip_path_mix_bwd": [_P, _P, _P, _P, _P, _P, _P, _I32, _I64, _I64, _P],
    "nestor_hip_bias_rows_fwd": [_P, _P, _P, _P, _I32, _P, _I64, _I64, _P],
    "nestor_hip_segment_colsum": [_P, _P, _P, _P, _P, _I32, _P, _I32, _I64, _P],
    "nestor_hip_gate_slots_fwd": [_P, _P, _P, _P, _P, _P, _I32, _I64, _I64, _P],
    "nestor_hip_gate_slots_bwd": [_P, _I32, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, _P],
    "nestor_hip_path_scale_fwd": [_P, _P, _I32, _P, _P, _I32, _I64, _I32, _I32, _I64, _P],
    "nestor_hip_path_scale_bwd": [
        _P, _P, _P, _I32, _P, _P, _P, _I32, _I64, _I32, _I32, _I64, _P,
    ],
}
_RESTYPES = {
    "nestor_hip_strerror": c_char_p,
    "nestor_hip_index_build_workspace_bytes": c_size_t,
    "nestor_hip_index_build_static_capacity_bytes": c_size_t,
    "nestor_hip_max_tiles": _I64,
    "nestor_hip_tile_table_ints": _I64,
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib: ctypes.CDLL | None = None


class NestorHipError(RuntimeError):
    """A ``nestor_hip_*`` entry point returned a negative status."""


def library_available() -> bool:
    return LIB_PATH.exists()


def load() -> ctypes.CDLL:
    """The loaded library; raises if it has not been built."""

    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise NestorHipError(
            f"{LIB_PATH} is missing: build it with `python -m nestor_amd.build` "
            "(there is no fallback path)"
        )
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, argtypes in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = _RESTYPES.get(name, c_int32)
    version = lib.nestor_hip_abi_version()
    if version != ABI_VERSION:
        raise NestorHipError(f"libnestor_hip.so ABI {version} != expected {ABI_VERSION}; rebuild")
    _lib = lib
    return lib


def call(name: str, *args) -> None:
    """Call an int-status entry point and raise on failure."""

    lib = load()
    status = getattr(lib, name)(*args)
    if status != 0:
        msg = lib.nestor_hip_strerror(status).decode()
        raise NestorHipError(f"{name} failed: {msg} ({status})")
