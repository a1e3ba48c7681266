"""Dispatch plan oracle (nestor/backbones/grouped_mm.py:222-321)."""

from __future__ import annotations

from typing import NamedTuple

import torch
from torch import Tensor

ALIGN = 16  # GROUPED_MM_ALIGN, nestor/backbones/grouped_mm.py:61


class Plan(NamedTuple):
    rows: int
    rows_pad: int
    order: Tensor
    counts: Tensor
    raw_starts: Tensor
    padded_starts: Tensor
    offs: Tensor
    row_dest: Tensor
    pad_token: Tensor
    pad_src_row: Tensor
    eid_pad: Tensor
    pad_valid: Tensor
    row_kept: Tensor


def rows_pad_for(rows: int, num_banks: int) -> int:
    """Static padded length (nestor/backbones/grouped_mm.py:270)."""

    return ((rows + ALIGN - 1) // ALIGN) * ALIGN + ALIGN * num_banks


def capacity_for(rows: int, num_banks: int, capacity_factor: float) -> int:
    """Per-bank row capacity ``ceil(cf * rows / E)`` of the skew-stress config."""

    import math

    return int(math.ceil(capacity_factor * rows / num_banks))


def dispatch_plan(
    expert_ids: Tensor, num_banks: int, slots: int, dtype: torch.dtype, capacity: int = 0
) -> Plan:
    """Stable sort by bank, aligned segment starts, and the five maps.

    ``capacity <= 0`` is the reference cascade (grouped_mm.py:253-318) op for
    op.  ``capacity > 0`` keeps, per bank, the first ``capacity`` rows in stable
    (token-major) order -- the rule of the reference's attention dispatch,
    "stable members-first argsort, keep the first cap"
    (nestor/backbones/nestor.py:3599-3607) -- and sends every other row to the
    last padded row, which is always slack.
    """

    rows = expert_ids.shape[0]
    device = expert_ids.device
    order = torch.argsort(expert_ids, stable=True)
    counts = torch.zeros(num_banks, dtype=torch.long, device=device).scatter_add_(
        0, expert_ids, torch.ones_like(expert_ids)
    )
    kept_counts = counts.clamp(max=capacity) if capacity > 0 else counts
    padded_counts = torch.div(kept_counts + ALIGN - 1, ALIGN, rounding_mode="floor") * ALIGN
    padded_starts = padded_counts.cumsum(0) - padded_counts
    raw_starts = counts.cumsum(0) - counts
    rows_pad = rows_pad_for(rows, num_banks)
    padded_ends = padded_counts.cumsum(0)
    offs = torch.cat(
        [padded_ends[:-1], torch.full((1,), rows_pad, dtype=torch.long, device=device)]
    ).to(torch.int32)

    sorted_eids = expert_ids.index_select(0, order)
    sorted_tokens = torch.div(order, slots, rounding_mode="floor")
    position = torch.arange(rows, device=device)
    rank = position - raw_starts.index_select(0, sorted_eids)
    dest = padded_starts.index_select(0, sorted_eids) + rank
    keep = rank < capacity if capacity > 0 else torch.ones_like(rank, dtype=torch.bool)

    row_dest = torch.full((rows,), rows_pad - 1, dtype=torch.long, device=device)
    row_dest[order[keep]] = dest[keep]
    pad_token = torch.zeros(rows_pad, dtype=torch.long, device=device)
    pad_token[dest[keep]] = sorted_tokens[keep]
    pad_src_row = torch.zeros(rows_pad, dtype=torch.long, device=device)
    pad_src_row[dest[keep]] = order[keep]
    eid_pad = torch.zeros(rows_pad, dtype=torch.long, device=device)
    eid_pad[dest[keep]] = sorted_eids[keep]
    pad_valid = torch.zeros(rows_pad, dtype=dtype, device=device)
    pad_valid[dest[keep]] = 1
    row_kept = torch.zeros(rows, dtype=torch.uint8, device=device)
    row_kept[order[keep]] = 1
    return Plan(
        rows, rows_pad, order, counts, raw_starts, padded_starts, offs, row_dest,
        pad_token, pad_src_row, eid_pad, pad_valid, row_kept,
    )
