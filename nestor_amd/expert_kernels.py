"""Entry points of the fused row kernels, under the reference's names and
signatures (nestor/backbones/triton_expert.py:509-625).  Each is differentiable
and backed by a HIP kernel pair; there is no eager fallback."""

from __future__ import annotations

import torch
from torch import Tensor

from nestor_amd import ops


def _need_bf16(dtype: torch.dtype, what: str) -> None:
    if dtype != torch.bfloat16:
        raise NotImplementedError(
            f"{what}: the HIP expert path computes in bfloat16 (run under bf16 autocast "
            f"or pass bf16 tensors); got {dtype}"
        )


def dispatch_rows(
    x: Tensor, pad_token: Tensor, pad_valid: Tensor, row_dest: Tensor, slots: int,
    compute_dtype: torch.dtype,
) -> Tensor:
    """``x.to(compute_dtype).index_select(0, pad_token) * pad_valid`` in one kernel;
    backward is the ``slots``-way gather-sum through ``row_dest``."""

    _need_bf16(compute_dtype, "dispatch_rows")
    return ops.dispatch_rows_op(x, pad_token, pad_valid, row_dest, slots)


def cat_cast(a: Tensor, b: Tensor, dtype: torch.dtype) -> Tensor:
    """``torch.cat([a, b], -1).to(dtype)`` bit for bit; the backward writes each
    bank's fp32 gradient contiguously."""

    assert a.shape == b.shape and a.dtype == b.dtype, "cat_cast needs twin banks"
    _need_bf16(dtype, "cat_cast")
    if a.dtype != torch.float32:
        return torch.cat([a, b], dim=-1).to(dtype)
    return ops.cat_cast_op(a, b)


def swiglu(up: Tensor, gate: Tensor) -> Tensor:
    """``F.silu(gate) * up`` over two ``[rows, hidden]`` tensors."""

    _need_bf16(up.dtype, "swiglu")
    return ops.swiglu_op(up, gate)


def swiglu_fused(up_gate: Tensor, hidden: int) -> Tensor:
    """``F.silu(up_gate[:, hidden:]) * up_gate[:, :hidden]`` read in place."""

    assert up_gate.shape[1] == 2 * hidden, "up_gate must be [rows, 2*hidden]"
    _need_bf16(up_gate.dtype, "swiglu_fused")
    return ops.swiglu_fused_op(up_gate, hidden)


def combine_rows(
    y_pad: Tensor, row_dest: Tensor, pad_src_row: Tensor, pad_valid: Tensor,
    weights: Tensor, group: int, out_dtype: torch.dtype,
) -> Tensor:
    """``(y_pad[row_dest] * weights[:, None]).to(out_dtype).view(-1, group, dim).sum(1)``
    as one deterministic gather-reduce; backward yields the padded-row gradient
    and the per-row weight gradient in one pass."""

    assert row_dest.shape[0] % group == 0, "rows must be a multiple of group"
    _need_bf16(y_pad.dtype, "combine_rows")
    return ops.combine_rows_op(y_pad, row_dest, pad_src_row, pad_valid, weights, group, out_dtype)


def bank_is_fusable(experts: list, fused_gate: bool) -> bool:
    """Bias-free SwiGLU banks take the fused path
    (nestor/backbones/triton_expert.py:122-140)."""

    first = experts[0]
    return (
        bool(getattr(first, "gated", False))
        and getattr(first, "activation", None) == "silu"
        and first.layers[0].bias is None
        and first.layers[1].bias is None
    )
