"""Compile ``libnestor_hip.so`` (gfx950) from ``nestor_amd/csrc`` with hipcc.

The library has no Python or torch dependency: it is a plain C-ABI shared object
(``include/nestor_hip.h``) built in-tree next to this file, so it travels with
the source tree to any machine that runs the tests or the benchmark.

A second, separate library is built beside it: ``libnestor_hip_probes.so``
(``include/nestor_hip_probes.h``), the measurement aids that only ``bench.py`` loads --
the counter yardsticks, the matrix-core clock probes and an instrumented build of the
bf16 GEMM translation unit (``-DNESTOR_GEMM_CLOCK_HOOK=1``).  None of it is in the
product library.

Run ``python -m nestor_amd.build`` to (re)build both.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
REPO_ROOT = PKG_DIR.parent
CSRC = PKG_DIR / "csrc"
INCLUDE = REPO_ROOT / "include"
LIB_PATH = PKG_DIR / "libnestor_hip.so"
PROBES_LIB_PATH = PKG_DIR / "libnestor_hip_probes.so"

SOURCES = ["index_build.hip", "rows.hip", "grouped_gemm.hip", "fp8_stream.hip", "router.hip"]
# (source, object stem, extra flags) of the measurement library
PROBE_SOURCES = [
    ("probes.hip", "probes", []),
    ("grouped_gemm.hip", "grouped_gemm_hooked", ["-DNESTOR_GEMM_CLOCK_HOOK=1"]),
]

# -packed-fp32-ops off: the compiler must not form packed fp32 VALU ops.
HIP_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # The LDS-DMA statements clobber m0 on purpose; tests/test_library_abi.py checks on the
    # generated assembly that nothing else in these kernels touches it.
    "-Wno-inline-asm",
]


def _hipcc() -> str:
    found = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(found):
        raise RuntimeError("hipcc not found; cannot build libnestor_hip.so")
    return found


def _compile(src: str, obj_dir: Path, stem: str | None = None, extra: list[str] | None = None) -> Path:
    obj = obj_dir / ((stem or Path(src).stem) + ".o")
    cmd = [_hipcc(), *HIP_FLAGS, *(extra or []), f"-I{INCLUDE}", f"-I{CSRC}", "-c", str(CSRC / src),
           "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(line for line in proc.stderr.splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def _link(objs: list[Path], lib: Path) -> None:
    tmp = lib.with_suffix(".so.tmp")
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    os.replace(tmp, lib)


def build_library(verbose: bool = True) -> Path:
    """Compile every HIP source and link ``libnestor_hip.so`` and the measurement
    library ``libnestor_hip_probes.so``; returns the path of the former."""

    obj_dir = PKG_DIR / "build"
    obj_dir.mkdir(exist_ok=True)
    jobs = [(s, None, None) for s in SOURCES] + list(PROBE_SOURCES)
    with ThreadPoolExecutor(max_workers=min(7, len(jobs))) as pool:
        objs = list(pool.map(lambda j: _compile(j[0], obj_dir, j[1], j[2]), jobs))
    _link(objs[:len(SOURCES)], LIB_PATH)
    _link(objs[len(SOURCES):], PROBES_LIB_PATH)
    if verbose:
        for lib in (LIB_PATH, PROBES_LIB_PATH):
            print(f"built {lib} ({lib.stat().st_size} bytes)")
    return LIB_PATH


if __name__ == "__main__":
    build_library()
