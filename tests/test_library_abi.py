"""The C-ABI library loads and exports every entry point the header declares
(no compute: runs without a GPU)."""

import ctypes
import os
import re

from nestor_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header: str = "nestor_hip.h") -> list[str]:
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nestor_hip_\w+)\s*\(", text)))


def test_header_symbols_exported_and_bound():
    names = _declared()
    assert len(names) >= 35
    assert _lib.LIB_PATH.exists(), "build the library first: python -m nestor_amd.build"
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in names:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert sorted(_lib.EXPORTED_SYMBOLS) == names, "ctypes table and header disagree"


def test_measurement_aids_live_in_their_own_library():
    """The probes and the instrumented GEMM build are a separate library with its own
    header; the product library exports none of them."""

    from nestor_amd import build

    probes = _declared("nestor_hip_probes.h")
    assert "nestor_hip_gemm_clock_sink" in probes and "nestor_hip_mfma_clock_probe" in probes
    assert build.PROBES_LIB_PATH.exists(), "build the libraries first: python -m nestor_amd.build"
    plib = ctypes.CDLL(str(build.PROBES_LIB_PATH))
    for name in probes:
        assert hasattr(plib, name), f"{name} declared in nestor_hip_probes.h but not exported"
    # the instrumented GEMM entry points carry the product's names and signatures
    for name in ("nestor_hip_grouped_gemm_nn", "nestor_hip_grouped_gemm_upgate_swiglu",
                 "nestor_hip_grouped_gemm_nt", "nestor_hip_grouped_gemm_nt_upgate",
                 "nestor_hip_grouped_gemm_tn", "nestor_hip_grouped_gemm_tn_pair"):
        assert hasattr(plib, name)
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in probes:
        assert not hasattr(lib, name), f"{name} leaked into the product library"
    assert not set(probes) & set(_declared())
    # the probes that walk a caller's buffer take its size and refuse to leave it
    null, one = ctypes.c_void_p(0), ctypes.c_void_p(1)
    i64, i32 = ctypes.c_int64, ctypes.c_int32
    plib.nestor_hip_dma_stream_probe.argtypes = [ctypes.c_void_p, i64, i64, i64, i32, i32, ctypes.c_void_p]
    assert plib.nestor_hip_dma_stream_probe(one, 1 << 20, 1024, 8192, 512, 1, null) == -22
    plib.nestor_hip_mfma_mix_probe.argtypes = [i32, i32, i32, ctypes.c_void_p, i64, i64,
                                               ctypes.c_void_p, ctypes.c_void_p]
    assert plib.nestor_hip_mfma_mix_probe(16, 8, 10, one, (8 << 20) - 1, 1 << 20, one, null) == -22


def test_version_and_error_strings():
    lib = _lib.load()
    assert lib.nestor_hip_abi_version() == _lib.ABI_VERSION
    assert lib.nestor_hip_strerror(0) == b"ok"
    assert b"invalid" in lib.nestor_hip_strerror(-22)
    assert lib.nestor_hip_max_tiles(67584, 128) == 67584 // 128 + 128 + 2
    from nestor_amd import ops

    assert lib.nestor_hip_tile_table_ints(67584, 128) == ops.tile_table_ints(67584, 128)
    assert lib.nestor_hip_tile_table_ints(16, 1) == ops.tile_table_ints(16, 1)
    assert lib.nestor_hip_index_build_workspace_bytes(65536, 128) == 128 * 128 * 4


def test_argument_checks_fail_before_any_launch():
    """Bad sizes are rejected with EINVAL on the host (null pointers, no GPU needed)."""

    lib = _lib.load()
    null = ctypes.c_void_p(0)
    assert lib.nestor_hip_dispatch_rows_fwd(null, 1, null, null, 1, null, 16, 12, null, 0, 0, null) == -22  # dim % 8
    assert lib.nestor_hip_swiglu_fwd(null, null, null, 4, 20, 20, 20, null) == -22
    assert lib.nestor_hip_grouped_gemm_nn(null, null, null, 16, 12, 8, 1, null, 4, null) == -22
    assert lib.nestor_hip_router_topk(null, 1, null, 1, null, null, null, null, 4, 65, 1, 0, null) == -22
    assert lib.nestor_hip_index_build(null, 10, 5000, 1, 0, 0, 1, null, null, null, null, null, null,
                                      null, null, null, null, null, null, 0, null, 0, null) == -34
    assert lib.nestor_hip_router_gates_bwd(null, 1, null, null, null, null, null, 4, 8, 9, 0, null) == -22  # k > C
    assert lib.nestor_hip_private_slots_fwd(null, null, 1, null, null, null, null, null, 4, 65, 4, 2, 1, null) == -22  # G > 64
    assert lib.nestor_hip_private_slots_bwd(null, null, null, 1, null, null, null, null, 4, 8, 4, 9, 1, null) == -22  # k_a > G
    assert lib.nestor_hip_router_choice_counts(null, null, null, 4, 2, 65, null) == -22
    # pool epilogues and biased banks
    assert lib.nestor_hip_path_mix_fwd(null, null, null, null, 1, 4, 12, null) == -22  # dim % 8
    assert lib.nestor_hip_path_mix_bwd(null, null, null, null, null, null, null, 7, 4, 16, null) == -22  # dtype
    assert lib.nestor_hip_path_scale_fwd(null, null, 2, null, null, 1, 4, 2, 2, 16, null) == -22  # which
    assert lib.nestor_hip_path_scale_fwd(null, null, 1, null, null, 1, 4, 2, 8, 16, null) == -22  # null operands
    assert lib.nestor_hip_path_scale_bwd(null, null, null, 1, null, null, null, 1, 4, 65, 65, 16, null) == -22  # slots > 64
    assert lib.nestor_hip_bias_rows_fwd(null, null, null, null, 0, null, 4, 12, null) == -22
    assert lib.nestor_hip_segment_colsum(null, null, null, null, null, 0, null, 4, 16, null) == -22  # splits
    assert lib.nestor_hip_path_mix_fwd(null, null, null, null, 1, 0, 16, null) == 0  # nothing to do


def test_m0_is_only_touched_by_the_dma_statements(tmp_path):
    """The LDS-DMA transfers are inline assembly that writes ``m0`` (the destination
    register of ``global_load_lds``) and lists it as clobbered.  ``m0`` is a register the
    compiler reserves for its own use (LDS-DMA builtins, register-indexed moves, message
    sends), which is why it warns about the clobber; the statements are safe as long as
    the compiler holds no value of its own in ``m0`` across them.  In these kernels it
    never uses ``m0`` at all: every reference in the generated gfx950 assembly sits inside
    one of the asm statements.  A compiler that starts using it shows up here."""

    import re
    import shutil
    import subprocess

    from nestor_amd import build

    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    total = 0
    for src in ("grouped_gemm.hip", "fp8_stream.hip", "probes.hip"):
        out = tmp_path / (src + ".s")
        cmd = [hipcc, *[f for f in build.HIP_FLAGS if f != "-fPIC"], "--cuda-device-only", "-S",
               f"-I{build.INCLUDE}", f"-I{build.CSRC}", str(build.CSRC / src), "-o", str(out)]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        assert proc.returncode == 0, proc.stderr[-2000:]
        inside, stray = False, []
        for number, line in enumerate(out.read_text().splitlines(), 1):
            text = line.strip()
            if text.startswith(";;#ASMSTART"):
                inside = True
            elif text.startswith(";;#ASMEND"):
                inside = False
            elif re.search(r"\bm0\b", text.split(";")[0]):
                total += inside
                if not inside:
                    stray.append((src, number, text))
        assert not stray, stray[:5]
    assert total > 100  # the statements are there (and were recognised)
