"""The index build that allocates nothing (``nestor_hip_index_build_static``: chunk
histograms in a fixed device array inside the library) against the entry point that
takes a caller workspace, through the C ABI: all twelve outputs bit-identical, on two
calls in a row (the second with a smaller input, so the array still holds the first
call's histograms), on a capacity-limited plan, and the size limit is refused."""

import ctypes

import pytest
import torch

from nestor_amd import _lib, ops

pytestmark = pytest.mark.gpu

_NAMES = ("order", "counts", "raw_starts", "padded_starts", "offs", "row_dest", "pad_token",
          "pad_src_row", "eid_pad", "pad_valid", "row_kept", "tile_table")


def _outputs(rows, num_banks, dev):
    rows_pad = ops.rows_pad_for(rows, num_banks)
    max_tiles = ops.max_tiles_for(rows_pad, num_banks)
    i64 = dict(dtype=torch.long, device=dev)
    # poisoned, so an entry a call fails to write shows up in the comparison
    outs = [
        torch.full((rows,), -7, **i64), torch.full((num_banks,), -7, **i64),
        torch.full((num_banks,), -7, **i64), torch.full((num_banks,), -7, **i64),
        torch.full((num_banks,), -7, dtype=torch.int32, device=dev),
        torch.full((rows,), -7, **i64), torch.full((rows_pad,), -7, **i64),
        torch.full((rows_pad,), -7, **i64), torch.full((rows_pad,), -7, **i64),
        torch.full((rows_pad,), -7.0, dtype=torch.bfloat16, device=dev),
        torch.full((rows,), 9, dtype=torch.uint8, device=dev),
        torch.full((ops.tile_table_ints(rows_pad, num_banks),), -7, dtype=torch.int32, device=dev),
    ]
    return outs, rows_pad, max_tiles


def _run(entry, ids, num_banks, slots, capacity):
    dev = ids.device
    rows = ids.numel()
    outs, rows_pad, max_tiles = _outputs(rows, num_banks, dev)
    ptr = [ctypes.c_void_p(t.data_ptr()) for t in outs]
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    head = (ctypes.c_void_p(ids.data_ptr()), rows, num_banks, slots, rows_pad, capacity, _lib.BF16,
            *ptr, max_tiles)
    if entry == "nestor_hip_index_build":
        nbytes = _lib.load().nestor_hip_index_build_workspace_bytes(rows, num_banks)
        work = torch.empty(max(nbytes, 4), dtype=torch.uint8, device=dev)
        _lib.call(entry, *head, ctypes.c_void_p(work.data_ptr()), work.numel(), stream)
    else:
        _lib.call(entry, *head, stream)
    torch.cuda.synchronize()
    # entries of the tile tables beyond each table's count are unspecified in both entry
    # points: compare what the contract defines
    from tests.helpers import tile_tables

    outs[11] = tile_tables(outs[11], rows_pad, num_banks)[1]
    return outs


@pytest.mark.parametrize("capacity_factor", [0.0, 1.25])
def test_static_scratch_index_build_matches_workspace_entry(cuda, capacity_factor):
    g = torch.Generator().manual_seed(5)
    # 65536 routed rows over 128 banks (the private call of the 1b-like shape), then a
    # smaller and differently shaped call that reuses the array
    cases = [(32768, 2, 128), (3001, 3, 20), (65, 1, 1), (0, 2, 4)]
    for tokens, slots, num_banks in cases:
        ids = torch.randint(0, num_banks, (tokens * slots,), generator=g).to(cuda)
        capacity = 0
        if capacity_factor > 0 and tokens > 0:
            capacity = int(-(-capacity_factor * tokens * slots // num_banks))
        want = _run("nestor_hip_index_build", ids, num_banks, slots, capacity)
        got = _run("nestor_hip_index_build_static", ids, num_banks, slots, capacity)
        for name, a, b in zip(_NAMES, got, want):
            assert torch.equal(a, b), (name, tokens, slots, num_banks, capacity)


def test_static_scratch_limit_is_refused(cuda):
    lib = _lib.load()
    cap = lib.nestor_hip_index_build_static_capacity_bytes()
    assert cap == 128 * 2048 * 4
    rows, num_banks = 1 << 16, 2049   # 128 chunks x 2049 banks x 4 B > the array
    assert lib.nestor_hip_index_build_workspace_bytes(rows, num_banks) > cap
    ids = torch.zeros(rows, dtype=torch.long, device=cuda)
    outs, rows_pad, max_tiles = _outputs(rows, num_banks, cuda)
    ptr = [ctypes.c_void_p(t.data_ptr()) for t in outs]
    status = lib.nestor_hip_index_build_static(
        ctypes.c_void_p(ids.data_ptr()), rows, num_banks, 1, rows_pad, 0, _lib.BF16, *ptr,
        max_tiles, ctypes.c_void_p(torch.cuda.current_stream(cuda).cuda_stream))
    assert status == -34


def test_static_entry_allocates_nothing(cuda):
    """The entry point is for callers that cannot allocate.  Two observations: the device's
    free memory is the same before and after a call (``hipMemGetInfo``), and the call can be
    recorded into a HIP graph -- capture refuses allocations -- whose replays (with eager
    work and synchronisations in between) give the workspace entry point's results."""

    g = torch.Generator().manual_seed(9)
    tokens, slots, num_banks = 4096, 2, 32
    ids = torch.randint(0, num_banks, (tokens * slots,), generator=g).to(cuda)
    want = _run("nestor_hip_index_build", ids, num_banks, slots, 0)
    _run("nestor_hip_index_build_static", ids, num_banks, slots, 0)   # set-up happens here, once
    outs, rows_pad, max_tiles = _outputs(tokens * slots, num_banks, cuda)
    ptr = [ctypes.c_void_p(t.data_ptr()) for t in outs]
    lib = _lib.load()

    def call(stream):
        status = lib.nestor_hip_index_build_static(
            ctypes.c_void_p(ids.data_ptr()), tokens * slots, num_banks, slots, rows_pad, 0, _lib.BF16,
            *ptr, max_tiles, ctypes.c_void_p(stream.cuda_stream))
        assert status == 0

    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info(cuda)
    call(torch.cuda.current_stream(cuda))
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(cuda)
    assert free_after == free_before

    from tests.helpers import tile_tables

    def check():
        torch.cuda.synchronize()
        got = list(outs)
        got[11] = tile_tables(got[11], rows_pad, num_banks)[1]
        for name, a, b in zip(_NAMES, got, want):
            assert torch.equal(a, b), name

    check()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(torch.cuda.current_stream(cuda))
    for _ in range(3):
        for t in outs:
            t.fill_(-3)                       # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        check()
