"""ctypes binding of ``libnestor_hip_probes.so`` (``include/nestor_hip_probes.h``): the
measurement library.  Nothing in the package imports this module; ``bench.py`` and the
tests of the probes do.

Besides the probes, the library holds an instrumented build of the bf16 grouped GEMMs
under the product's entry-point names.  ``instrumented(sink)`` routes the package's GEMM
calls there for the duration of a ``with`` block and switches the kernels' clock hook on,
so the same ops, on the same tensors, report the shader clock they ran at.
"""

from __future__ import annotations

import contextlib
import ctypes
from ctypes import c_int32, c_int64, c_void_p
from pathlib import Path

from . import _lib

LIB_PATH = Path(__file__).resolve().parent / "libnestor_hip_probes.so"

_P, _I32, _I64 = c_void_p, c_int32, c_int64
GEMM_ENTRY_POINTS = (
    "nestor_hip_grouped_gemm_nn", "nestor_hip_grouped_gemm_upgate_swiglu",
    "nestor_hip_grouped_gemm_nt", "nestor_hip_grouped_gemm_nt_upgate",
    "nestor_hip_grouped_gemm_tn", "nestor_hip_grouped_gemm_tn_pair",
)
_SIGNATURES: dict[str, list] = {
    "nestor_hip_dma_stream_probe": [_P, _I64, _I64, _I64, _I32, _I32, _P],
    "nestor_hip_mfma_clock_probe": [_I32, _I32, _P, _P],
    "nestor_hip_mfma_mix_probe": [_I32, _I32, _I32, _P, _I64, _I64, _P, _P],
    "nestor_hip_wall_clock_khz": [],
    "nestor_hip_gemm_clock_sink": [_P],
    **{name: _lib._SIGNATURES[name] for name in GEMM_ENTRY_POINTS},
}

_cdll: ctypes.CDLL | None = None


def load() -> ctypes.CDLL:
    global _cdll
    if _cdll is None:
        if not LIB_PATH.exists():
            raise _lib.NestorHipError(f"{LIB_PATH} is missing: build it with `python -m nestor_amd.build`")
        lib = ctypes.CDLL(str(LIB_PATH))
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = c_int32
        _cdll = lib
    return _cdll


def call(name: str, *args) -> None:
    status = getattr(load(), name)(*args)
    if status != 0:
        raise _lib.NestorHipError(f"{name} (measurement library) failed with status {status}")


def wall_clock_khz() -> int:
    return int(load().nestor_hip_wall_clock_khz())


@contextlib.contextmanager
def instrumented(sink_ptr: int):
    """Inside the block the package's bf16 grouped-GEMM calls run the measurement
    library's instrumented build, which adds each workgroup's {shader cycles, wall ticks,
    1, K steps} to the 64 x 4 uint64 device array at ``sink_ptr`` (zeroed by the caller).
    Synchronise the device before entering and before leaving."""

    load()
    original = _lib.call

    def routed(name, *args):
        if name in GEMM_ENTRY_POINTS:
            return call(name, *args)
        return original(name, *args)

    call("nestor_hip_gemm_clock_sink", c_void_p(sink_ptr))
    _lib.call = routed
    try:
        yield
    finally:
        _lib.call = original
        call("nestor_hip_gemm_clock_sink", c_void_p(0))
