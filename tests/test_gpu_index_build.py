"""HIP index build vs the oracle plan: every output must match bit for bit
(the bar of the reference's own map tests, tests/test_triton_index_build.py:114-115)."""

import pytest
import torch

from oracle import plan as oplan
from tests.helpers import gen, zipf_ids

pytestmark = pytest.mark.gpu

FIELDS = ["order", "counts", "raw_starts", "padded_starts", "offs", "row_dest", "pad_token",
          "pad_src_row", "eid_pad", "pad_valid", "row_kept"]


def _check(ids2d, num_banks, cuda, capacity=0, dtype=torch.bfloat16):
    from nestor_amd.dispatch import build_dispatch_maps, dispatch_plan

    slots = ids2d.shape[1]
    flat = ids2d.reshape(-1)
    want = oplan.dispatch_plan(flat, num_banks, slots, dtype, capacity)
    got = dispatch_plan(flat.to(cuda), num_banks, slots, dtype, capacity)
    assert got.rows_pad == want.rows_pad
    for name in FIELDS:
        g = getattr(got, name).cpu()
        w = getattr(want, name)
        assert g.dtype == w.dtype, name
        assert torch.equal(g, w), f"{name} differs (rows={flat.numel()}, E={num_banks}, cap={capacity})"
    # Tile tables: each of the three covers every padded row exactly once, no tile crosses
    # a segment end, and the balanced tables cut a segment of b 32-row blocks into
    # ceil(b / cap) tiles whose block counts differ by at most one.
    from tests.helpers import tile_tables

    tables, _ = tile_tables(got.tile_table, want.rows_pad, num_banks)
    kept = want.counts.clamp(max=capacity) if capacity > 0 else want.counts
    padded = (kept + 15) // 16 * 16
    seg_end_all = int((want.padded_starts + padded)[-1])
    for (bank, row0, nrows), cap_blocks in zip(tables, (4, 5, 10)):
        covered = torch.zeros(want.rows_pad, dtype=torch.int32)
        per_bank: dict[int, list[tuple[int, int]]] = {}
        for b, r0, nr in zip(bank.tolist(), row0.tolist(), nrows.tolist()):
            assert 0 < nr <= 32 * cap_blocks
            covered[r0:r0 + nr] += 1
            if b >= 0:
                assert want.padded_starts[b] <= r0 and r0 + nr <= want.padded_starts[b] + padded[b]
                per_bank.setdefault(b, []).append((r0, nr))
            else:
                assert r0 >= seg_end_all
        assert torch.equal(covered, torch.ones_like(covered))
        for b in range(num_banks):
            tiles = sorted(per_bank.get(b, []))
            blocks = (int(padded[b]) + 31) // 32
            if cap_blocks == 4:
                assert len(tiles) == (int(padded[b]) + 127) // 128
                continue
            assert len(tiles) == (blocks + cap_blocks - 1) // cap_blocks
            sizes = [(nr + 31) // 32 for _, nr in tiles]
            assert sum(sizes) == blocks
            if sizes:
                assert max(sizes) - min(sizes) <= 1
                # every tile but a segment's last is made of whole blocks
                assert all(nr % 32 == 0 for _, nr in tiles[:-1])
    if capacity == 0:
        # The reference kernel's own boundary: maps from a caller-held sort.
        maps = build_dispatch_maps(
            flat.to(cuda), want.order.to(cuda), want.padded_starts.to(cuda),
            want.raw_starts.to(cuda), slots, want.rows_pad, dtype,
        )
        for name, g in zip(["row_dest", "pad_token", "pad_src_row", "eid_pad", "pad_valid"], maps):
            assert torch.equal(g.cpu(), getattr(want, name)), f"build_dispatch_maps {name}"


def test_reference_map_cases(cuda):
    """The four input cases of the reference's map tests
    (tests/test_triton_index_build.py:117-137), drawn with its seeds."""

    torch.manual_seed(0)
    _check(torch.randint(0, 8, (300, 3)), 8, cuda)
    torch.manual_seed(1)
    ids = torch.randint(1, 5, (200, 2))
    ids[ids == 4] = 2
    _check(ids, 6, cuda)
    _check(torch.zeros(65, 1, dtype=torch.long), 1, cuda)
    torch.manual_seed(2)
    _check(torch.randint(0, 4, (341, 3)), 4, cuda)
    _check(torch.randint(0, 4, (342, 3)), 4, cuda)


@pytest.mark.parametrize("tokens,slots,banks", [
    (1, 1, 1), (7, 2, 3), (64, 1, 5), (1000, 6, 120), (4096, 1, 4), (4096, 2, 16),
    (16384, 2, 64), (32768, 1, 16), (32768, 2, 128), (5000, 16, 256), (3000, 3, 300),
    (2000, 2, 3000), (500, 1, 4096),   # more LDS than a launch gets by default in the plan scan
])
def test_uniform_routing_sizes(cuda, tokens, slots, banks):
    ids = torch.randint(0, banks, (tokens, slots), generator=gen(tokens + slots + banks))
    _check(ids, banks, cuda)
    _check(ids, banks, cuda, dtype=torch.float32)


@pytest.mark.parametrize("tokens,slots,banks", [
    (4096, 1, 512), (4097, 1, 512), (4096, 1, 513), (2048, 2, 128), (4095, 1, 7), (1, 3, 512),
    (255, 1, 2), (257, 1, 2), (3841, 1, 64),
])
def test_one_launch_build_and_its_limits(cuda, tokens, slots, banks):
    """A batch of up to 4096 rows over up to 512 banks is built by one workgroup in one
    launch, larger ones by the three launches: both sides of each limit, chunk ends
    inside and at wavefront boundaries, skew with empty banks, and a binding capacity."""

    ids = torch.randint(0, banks, (tokens, slots), generator=gen(7 * tokens + slots + banks))
    _check(ids, banks, cuda)
    skew = zipf_ids(1, tokens, slots, banks)
    _check(skew, banks, cuda, dtype=torch.float32)
    cap = oplan.capacity_for(tokens * slots, banks, 1.25)
    _check(skew, banks, cuda, capacity=cap)


def test_skewed_routing_with_empty_banks_and_capacity(cuda):
    """The skew-stress config: Zipf-ranked bank popularity (several banks get no
    rows) on the 200m shape, dropless and with capacity factor 1.25."""

    for tokens, slots, banks in [(16384, 1, 8), (16384, 2, 64)]:
        ids = zipf_ids(0, tokens, slots, banks)
        counts = torch.bincount(ids.reshape(-1), minlength=banks)
        assert (counts == 0).sum() >= 1 or banks == 8
        _check(ids, banks, cuda)
        cap = oplan.capacity_for(tokens * slots, banks, 1.25)
        assert (counts > cap).any()
        _check(ids, banks, cuda, capacity=cap)


def test_capacity_never_binding_equals_dropless(cuda):
    ids = torch.randint(0, 8, (512, 2), generator=gen(3))
    from nestor_amd.dispatch import dispatch_plan

    a = dispatch_plan(ids.reshape(-1).to(cuda), 8, 2, torch.bfloat16, 0)
    b = dispatch_plan(ids.reshape(-1).to(cuda), 8, 2, torch.bfloat16, 100000)
    for name in FIELDS:
        assert torch.equal(getattr(a, name), getattr(b, name)), name
