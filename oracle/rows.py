"""Row-kernel oracles: dispatch gather, SwiGLU, cat+cast, weighted combine, path mix.

Each forward is the eager chain the reference's fused kernels are held to; each
backward states the reference's backward formula with its rounding points.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import Tensor


def dispatch_rows(x: Tensor, pad_token: Tensor, pad_valid: Tensor, compute_dtype: torch.dtype) -> Tensor:
    """``x.to(dtype).index_select(0, pad_token) * pad_valid``
    (nestor/backbones/grouped_mm.py:120-124, triton_expert.py:517)."""

    return x.to(compute_dtype).index_select(0, pad_token) * pad_valid.to(compute_dtype).unsqueeze(1)


def dispatch_rows_bwd(grad_pad: Tensor, row_dest: Tensor, num_tokens: int, slots: int, x_dtype: torch.dtype) -> Tensor:
    """Slots-way gather-sum in fp32, written in x's dtype
    (nestor/backbones/triton_packed.py:160-169)."""

    g = grad_pad.index_select(0, row_dest).float()
    return g.view(num_tokens, slots, -1).sum(1).to(x_dtype)


def swiglu(up: Tensor, gate: Tensor) -> Tensor:
    """``F.silu(gate) * up`` on bf16 tensors: silu in fp32 rounded to bf16, then
    the product rounded to bf16 (nestor/backbones/triton_expert.py:172-175)."""

    return F.silu(gate) * up


def swiglu_bwd(grad_out: Tensor, up: Tensor, gate: Tensor) -> tuple[Tensor, Tensor]:
    """(grad_up, grad_gate) with the reference's three roundings
    (nestor/backbones/triton_expert.py:206-214)."""

    dt = up.dtype
    g = gate.float()
    s = torch.sigmoid(g)
    act = (g * s).to(dt)
    go = grad_out.float()
    grad_up = (go * act.float()).to(dt)
    grad_act = (go * up.float()).to(dt)
    grad_gate = (grad_act.float() * s * (1.0 + g * (1.0 - s))).to(dt)
    return grad_up, grad_gate


def cat_cast(a: Tensor, b: Tensor, dtype: torch.dtype) -> Tensor:
    """``torch.cat([a, b], -1).to(dtype)`` (nestor/backbones/triton_expert.py:547)."""

    return torch.cat([a, b], dim=-1).to(dtype)


def combine_rows(
    y_pad: Tensor, row_dest: Tensor, weights: Tensor, group: int, out_dtype: torch.dtype
) -> Tensor:
    """Gather + weight + per-term rounding + group sum, as the fused reference
    kernel does it (nestor/backbones/triton_expert.py:292-302,466-472): fp32
    product, rounded to ``out_dtype`` when the rounding flag is on (a no-op for
    an fp32 output), fp32 accumulation, final cast."""

    term = y_pad.index_select(0, row_dest).float() * weights.float().unsqueeze(1)
    promoted = torch.promote_types(y_pad.dtype, weights.dtype)
    if promoted != torch.float32 or out_dtype != torch.float32:
        term = term.to(out_dtype).float()
    n_out = row_dest.shape[0] // group
    return term.view(n_out, group, -1).sum(1).to(out_dtype)


def combine_rows_eager(
    y_pad: Tensor, row_dest: Tensor, weights: Tensor, group: int, out_dtype: torch.dtype
) -> Tensor:
    """The eager chain of grouped_expert_combine (nestor/backbones/grouped_mm.py:616-617)."""

    rows = y_pad.index_select(0, row_dest)
    weighted = (rows * weights.reshape(-1, 1)).to(out_dtype)
    return weighted.view(row_dest.shape[0] // group, group, -1).sum(1)


def combine_rows_bwd(
    grad_out: Tensor, y_pad: Tensor, pad_src_row: Tensor, pad_valid: Tensor,
    weights: Tensor, group: int, row_kept: Tensor | None = None,
) -> tuple[Tensor, Tensor]:
    """(grad_y, grad_w): ``gy[p] = bf16(go[src//group] * w[src]) * valid[p]``,
    ``gw[src] = sum_d go * y`` in fp32 (nestor/backbones/triton_expert.py:324-344)."""

    src = pad_src_row
    go = grad_out.float().index_select(0, torch.div(src, group, rounding_mode="floor"))
    w = weights.float().index_select(0, src)
    valid = pad_valid.float() != 0
    gy = (go * w.unsqueeze(1)).to(y_pad.dtype) * valid.to(y_pad.dtype).unsqueeze(1)
    dots = (go * y_pad.float()).sum(1)
    gw = torch.zeros(weights.shape[0], dtype=torch.float32, device=y_pad.device)
    gw[src[valid]] = dots[valid]
    return gy, gw


def path_mix(public_update: Tensor, private_update: Tensor, alpha: Tensor) -> Tensor:
    """``alpha[..., 0:1] * public + alpha[..., 1:2] * private`` in the operands' dtype:
    every product and the sum are rounded to it
    (nestor/backbones/expert_pools.py:1110-1113)."""

    return alpha[..., 0:1] * public_update + alpha[..., 1:2] * private_update


def path_mix_bwd(grad_out: Tensor, public_update: Tensor, private_update: Tensor,
                 alpha: Tensor) -> tuple[Tensor, Tensor, Tensor]:
    """What autograd derives from :func:`path_mix`: ``(g_public, g_private, g_alpha)``."""

    leaves = [t.detach().clone().requires_grad_(True) for t in (public_update, private_update, alpha)]
    path_mix(*leaves).backward(grad_out)
    return leaves[0].grad, leaves[1].grad, leaves[2].grad


def path_scale(inp: Tensor, alpha: Tensor, which: int, dest: Tensor | None = None,
               num_out: int = 0) -> Tensor:
    """Split layouts of the pool: ``alpha[..., which] * X`` with ``X = inp [..., slots, d]``
    (per slot, nestor/backbones/expert_pools.py:943-953) or ``inp`` scattered onto
    ``num_out`` column streams by ``dest [..., slots]``
    (``zeros.scatter_add``, expert_pools.py:758-761, scaled at :1031-1041)."""

    x = inp
    if dest is not None:
        index = dest.unsqueeze(-1).expand_as(inp)
        x = inp.new_zeros(*inp.shape[:-2], num_out, inp.shape[-1]).scatter_add(-2, index, inp)
    return alpha[..., which:which + 1].unsqueeze(-1) * x


def path_scale_bwd(grad_out: Tensor, inp: Tensor, alpha: Tensor, which: int,
                   dest: Tensor | None = None, num_out: int = 0) -> tuple[Tensor, Tensor]:
    """What autograd derives from :func:`path_scale`: ``(g_inp, g_alpha [..., 2])``."""

    leaves = [t.detach().clone().requires_grad_(True) for t in (inp, alpha)]
    path_scale(leaves[0], leaves[1], which, dest, num_out).backward(grad_out)
    return leaves[0].grad, leaves[1].grad


def gate_combine_slots(out_c: Tensor, bo: Tensor | None, gid: Tensor | None, gates: Tensor,
                       slot_rows: Tensor, out_dtype: torch.dtype) -> Tensor:
    """Packed column attention epilogue, the eager chain its fused kernel is held to
    (nestor/backbones/triton_packed.py:385-395): bias added in the GEMM dtype, the row
    upcast to the stream dtype, multiplied by the row's gate in that dtype, gathered
    into slot order."""

    val = out_c if bo is None else out_c + bo.to(out_c.dtype).index_select(0, gid)
    rows = val.to(out_dtype) * gates.to(out_dtype).unsqueeze(1)
    return rows.index_select(0, slot_rows)
