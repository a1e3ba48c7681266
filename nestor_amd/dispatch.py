"""The dispatch plan of one bank call and the map build behind it.

Host-side mirror of ``_dispatch_plan`` / ``_DispatchPlan``
(nestor/backbones/grouped_mm.py:197-321) and ``build_dispatch_maps``
(nestor/backbones/triton_dispatch.py:109-160).  The whole plan -- stable sort,
counts, offsets, maps, GEMM tile table -- is one custom-op call; shapes depend
only on ``rows`` and the bank count, never on the routing.
"""

from __future__ import annotations

from typing import NamedTuple

import torch
from torch import Tensor

from nestor_amd import ops

GROUPED_MM_ALIGN = 16


class DispatchPlan(NamedTuple):
    """Reference fields first (same names, same order), then what the HIP
    kernels add: the sort itself, segment bookkeeping and the tile table."""

    rows: int
    rows_pad: int
    offs: Tensor
    row_dest: Tensor
    pad_token: Tensor
    pad_src_row: Tensor
    eid_pad: Tensor
    pad_valid: Tensor
    order: Tensor
    counts: Tensor
    raw_starts: Tensor
    padded_starts: Tensor
    row_kept: Tensor
    tile_table: Tensor
    capacity: int
    kept_counts: Tensor  # rows of each bank that own a padded slot (== counts when dropless)


def dispatch_plan(
    expert_ids: Tensor, num_banks: int, slots: int, dtype: torch.dtype, capacity: int = 0
) -> DispatchPlan:
    """Sort the routed rows by bank and build every per-row map on the GPU.

    Args:
        expert_ids: flat token-major bank index per ``(token, slot)`` row, int64.
        num_banks: bank size ``E``.
        slots: slots per token.
        dtype: dtype of ``pad_valid`` (the GEMM dtype).
        capacity: ``<= 0`` dispatches every row (the reference's behaviour);
            ``> 0`` keeps the first ``capacity`` rows of each bank in stable
            order and gives the rest no padded slot (``row_kept == 0``,
            ``row_dest == rows_pad - 1``).
    """

    rows = expert_ids.shape[0]
    (order, counts, raw_starts, padded_starts, offs, row_dest, pad_token, pad_src_row,
     eid_pad, pad_valid, row_kept, tile_table) = ops.index_build(
        expert_ids, num_banks, slots, capacity, dtype
    )
    return DispatchPlan(
        rows, ops.rows_pad_for(rows, num_banks), offs, row_dest, pad_token, pad_src_row,
        eid_pad, pad_valid, order, counts, raw_starts, padded_starts, row_kept, tile_table,
        capacity, counts.clamp(max=capacity) if capacity > 0 else counts,
    )


def build_dispatch_maps(
    expert_ids: Tensor, order: Tensor, padded_starts: Tensor, raw_starts: Tensor,
    slots: int, rows_pad: int, valid_dtype: torch.dtype,
) -> tuple[Tensor, Tensor, Tensor, Tensor, Tensor]:
    """``(row_dest, pad_token, pad_src_row, eid_pad, pad_valid)`` from a sort the
    caller already holds -- the reference kernel's exact boundary."""

    out = ops.build_dispatch_maps_op(
        expert_ids, order, padded_starts, raw_starts, slots, rows_pad, valid_dtype
    )
    return out[0], out[1], out[2], out[3], out[4]
