"""Expert-bank oracles: the grouped path with the reference's rounding points,
an unrounded fp32/fp64 "gold" form, and the sparse per-expert loop (the
reference's CPU eager path)."""

from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import Tensor

from oracle import plan as oplan
from oracle import rows as orows


def segment_mm(a: Tensor, b: Tensor, offs: Tensor) -> Tensor:
    """Rows ``[offs[i-1], offs[i])`` of ``a`` through ``b[i]``: the host-side
    segment loop of nestor/backbones/grouped_mm.py:97-104, with the GPU
    kernel's numerics (operands as given, fp32 accumulate, result in a's dtype)."""

    bounds = [0] + offs.tolist()
    outs = [
        (a[bounds[i] : bounds[i + 1]].float() @ b[i].float()).to(a.dtype)
        for i in range(b.shape[0])
    ]
    return torch.cat(outs, dim=0)


def expert_rows_padded(
    x: Tensor, w_up: Tensor, w_gate: Tensor, w_down: Tensor, plan: oplan.Plan, dtype: torch.dtype
) -> dict[str, Tensor]:
    """Dispatch -> up|gate GEMM -> SwiGLU -> down GEMM on the padded layout
    (nestor/backbones/grouped_mm.py:398-421), every intermediate returned."""

    x_pad = orows.dispatch_rows(x, plan.pad_token, plan.pad_valid, dtype)
    w_up_gate = orows.cat_cast(w_up, w_gate, dtype)
    up_gate = segment_mm(x_pad, w_up_gate, plan.offs)
    h = w_up.shape[-1]
    hidden = orows.swiglu(up_gate[:, :h], up_gate[:, h:])
    y_pad = segment_mm(hidden, w_down.to(dtype), plan.offs)
    return {"x_pad": x_pad, "up_gate": up_gate, "hidden": hidden, "y_pad": y_pad}


def grouped_expert_combine(
    x: Tensor, w_up: Tensor, w_gate: Tensor, w_down: Tensor, expert_ids: Tensor,
    weights: Tensor, group: int, dtype: torch.dtype, capacity: int = 0,
) -> Tensor:
    """The fused call-site form (nestor/backbones/grouped_mm.py:619-637):
    ``[T, slots // group, d_out]`` in x's dtype."""

    num_tokens, slots = expert_ids.shape
    plan = oplan.dispatch_plan(expert_ids.reshape(-1), w_up.shape[0], slots, dtype, capacity)
    y_pad = expert_rows_padded(x, w_up, w_gate, w_down, plan, dtype)["y_pad"]
    w = weights.reshape(-1)
    if capacity > 0:
        w = w * plan.row_kept.to(w.dtype)
    out = orows.combine_rows(y_pad, plan.row_dest, w, group, x.dtype)
    return out.view(num_tokens, slots // group, -1)


def swiglu_expert(x: Tensor, w_up: Tensor, w_gate: Tensor, w_down: Tensor) -> Tensor:
    """One expert, ``down(silu(gate(x)) * up(x))`` with ``[d_in, h]`` / ``[h, d_out]``
    stacked-layout weights (nestor/scaling/blocks.py:306-312,
    nestor/backbones/expert_bank_stack.py:72-77)."""

    return (F.silu(x @ w_gate) * (x @ w_up)) @ w_down


_ACTIVATIONS = {"silu": F.silu, "gelu": F.gelu, "relu": F.relu}


def biased_expert(
    x: Tensor, w_up: Tensor, w_gate: Tensor | None, w_down: Tensor, b_up: Tensor | None,
    b_down: Tensor | None, activation: str = "silu",
) -> Tensor:
    """One expert of the native MoE banks: gated ``down(act(gate(x)) * up(x))`` with
    biases on up and down only (nestor/scaling/blocks.py:251-312), or the pointwise
    ``down(act(up(x)))`` when ``w_gate`` is None; stacked-layout weights."""

    up = x @ w_up if b_up is None else x @ w_up + b_up
    act = _ACTIVATIONS[activation]
    hidden = act(x @ w_gate) * up if w_gate is not None else act(up)
    out = hidden @ w_down
    return out if b_down is None else out + b_down


def gold_combine(
    x: Tensor, w_up: Tensor, w_gate: Tensor | None, w_down: Tensor, expert_ids: Tensor,
    weights: Tensor, group: int, row_kept: Tensor | None = None, *,
    b_up: Tensor | None = None, b_down: Tensor | None = None, activation: str = "silu",
) -> Tensor:
    """Unrounded reference in the dtype of its inputs (use fp32 or fp64): every
    (token, slot) row through its expert, weighted, summed over each group of
    consecutive slots.  Differentiable; built from a per-expert loop so it
    shares no indexing with the padded layout."""

    num_tokens, slots = expert_ids.shape
    flat_ids = expert_ids.reshape(-1)
    tokens = torch.arange(num_tokens, device=x.device).repeat_interleave(slots)
    rows = torch.zeros(num_tokens * slots, w_down.shape[-1], dtype=x.dtype, device=x.device)
    for e in range(w_up.shape[0]):
        sel = torch.nonzero(flat_ids == e).squeeze(-1)
        if sel.numel() == 0:
            continue
        y = biased_expert(
            x.index_select(0, tokens[sel]), w_up[e], None if w_gate is None else w_gate[e],
            w_down[e], None if b_up is None else b_up[e], None if b_down is None else b_down[e],
            activation,
        )
        rows = rows.index_add(0, sel, y)
    w = weights.reshape(-1, 1).to(x.dtype)
    if row_kept is not None:
        w = w * row_kept.reshape(-1, 1).to(x.dtype)
    return (rows * w).view(num_tokens, slots // group, group, -1).sum(2)


def accumulate_sparse_expert_bank(
    residual: Tensor, x: Tensor, w_up: Tensor, w_gate: Tensor, w_down: Tensor,
    expert_weights: Tensor,
) -> None:
    """The per-expert sparse loop, the reference's CPU eager path
    (nestor/backbones/expert_pool_dispatch.py:194-215): nonzero -> index_select
    -> expert -> weight -> index_add_ into ``residual``.  Run it under
    ``torch.autocast("cpu", torch.bfloat16)`` to match the reference tests
    (tests/test_expert_pools.py:417-422); F.linear is what autocast narrows."""

    for e in range(w_up.shape[0]):
        token_indices = torch.nonzero(expert_weights[:, e], as_tuple=False).squeeze(-1)
        if token_indices.numel() == 0:
            continue
        xe = x.index_select(0, token_indices)
        hidden = F.silu(F.linear(xe, w_gate[e].t())) * F.linear(xe, w_up[e].t())
        out = F.linear(hidden, w_down[e].t())
        weighted = out * expert_weights.index_select(0, token_indices)[:, e].unsqueeze(-1)
        residual.index_add_(0, token_indices, weighted.to(residual.dtype))


def dense_weights(expert_ids: Tensor, weights: Tensor, num_banks: int) -> Tensor:
    """``[T, E]`` gate matrix equivalent to per-slot (ids, weights); duplicate
    ids of one token add up."""

    out = torch.zeros(expert_ids.shape[0], num_banks, dtype=weights.dtype, device=weights.device)
    return out.scatter_add(1, expert_ids, weights)
