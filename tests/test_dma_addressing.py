"""Host-side range check of the direct-to-LDS transfers' address arithmetic (no GPU).

``tests/dma_addressing_check.cpp`` includes the header the kernels take their per-lane
offsets and buffer-descriptor sizes from (``nestor_amd/csrc/dma_addressing.hpp``) and walks
every wavefront, lane, transfer and K step of ragged shapes: tiles of 1..320 rows, widths
that are not a multiple of the tile, segments shorter than a K step, operands that end
with a segment.  An address out of range on the GPU is a memory fault, so this has to
pass before a change to that arithmetic is run there.
"""

import os
import shutil
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_every_transfer_stays_inside_its_operand(tmp_path):
    gxx = shutil.which("g++")
    assert gxx, "g++ is part of the toolchain this library is built with"
    exe = tmp_path / "dma_addressing_check"
    build = subprocess.run(
        [gxx, "-O1", "-std=c++17", f"-I{os.path.join(ROOT, 'nestor_amd', 'csrc')}",
         os.path.join(ROOT, "tests", "dma_addressing_check.cpp"), "-o", str(exe)],
        capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-2000:]
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stdout[-2000:]
    assert run.stdout.strip().startswith("ok:")
