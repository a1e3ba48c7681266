"""Router and slot-construction oracles (single-linear score heads; the training-mode
exploration noise as a function of a given standard-normal draw)."""

from __future__ import annotations

from typing import NamedTuple

import torch
import torch.nn.functional as F
from torch import Tensor


class RouterOut(NamedTuple):
    scores: Tensor
    softmax_probs: Tensor
    gates: Tensor
    topk_indices: Tensor
    active_mask: Tensor
    valid_token_mask: Tensor


def stable_topk(values: Tensor, k: int) -> Tensor:
    """Indices of the k largest entries along the last dim in descending order,
    equal values lowest index first -- the one tightening of ``torch.topk``
    (whose tie order is unspecified) that both sides of every parity test share."""

    return torch.sort(values, dim=-1, descending=True, stable=True).indices[..., :k]


def explore(scores: Tensor, eps: Tensor, noise_head: Tensor, steps_done: float = 0.0,
            anneal_steps: int = 0) -> Tensor:
    """Training-mode scores of a router with a noise head
    (nestor/backbones/nestor.py:540-556; batched: batched_router.py:188-208):
    ``scores + eps * softplus(noise_head) * (1 - min(steps_done / anneal_steps, 1))``,
    with ``eps`` the standard-normal draw, ``noise_head = noise_mlp(x)`` and the anneal
    factor 1 when ``anneal_steps`` is 0.  Written with log1p/exp, not ``F.softplus``."""

    spread = torch.where(noise_head > 20, noise_head, torch.log1p(torch.exp(noise_head.clamp(max=20))))
    keep = 1.0 if anneal_steps <= 0 else 1.0 - min(steps_done / anneal_steps, 1.0)
    return scores + eps * spread * keep


def route(
    scores: Tensor, choice_bias: Tensor, k: int, gate_mode: str, valid: Tensor,
    softmax_dtype: torch.dtype | None = None,
) -> RouterOut:
    """Everything after the score head in ``Router.forward``
    (nestor/backbones/nestor.py:558-593).  ``valid`` broadcasts against
    ``scores[..., 0]``; ``choice_bias`` against ``scores``.  ``softmax_dtype``
    is the dtype ``F.softmax(scores)`` returns (fp32 under autocast, else the
    score dtype)."""

    probs32 = F.softmax(scores.float(), dim=-1)
    softmax_probs = probs32.to(softmax_dtype or scores.dtype)
    biased = scores + choice_bias
    topk = stable_topk(biased, k)
    if gate_mode == "switch":
        topk_gates = probs32.gather(-1, topk).to(scores.dtype)
    else:
        topk_gates = F.softmax(scores.gather(-1, topk).float(), dim=-1).to(scores.dtype)
    gates = torch.zeros_like(scores).scatter_add_(-1, topk, topk_gates)
    gates = gates * valid.unsqueeze(-1).to(gates.dtype)
    return RouterOut(scores, softmax_probs, gates, topk, gates > 0, valid)


def route_private_batched(
    scores: Tensor, choice_bias: Tensor, k: int, gate_mode: str, valid: Tensor,
    group_active: Tensor, softmax_dtype: torch.dtype | None = None,
) -> RouterOut:
    """The batched form on ``[B, S, G, Q]`` scores with ``[G, Q]`` biases and the
    ``valid & member`` mask (nestor/backbones/batched_router.py:210-227)."""

    member = valid.unsqueeze(-1) & group_active
    return route(scores, choice_bias, k, gate_mode, member, softmax_dtype)


def public_slots(gates: Tensor, topk: Tensor) -> tuple[Tensor, Tensor]:
    """(expert_ids, weights) ``[T, k_p]`` (nestor/backbones/expert_pools.py:416-420)."""

    return topk, gates.gather(1, topk)


def private_slots(
    gates: Tensor, choices: Tensor, group_gates: Tensor, k_a: int, selected: Tensor | None = None
) -> tuple[Tensor, Tensor, Tensor]:
    """token -> column -> expert ids ``g * Q + e`` and weights
    ``private_gate * column_gate`` (nestor/backbones/expert_pools.py:496-521).
    gates ``[T, G, Q]``, choices ``[T, G, k_q]``, group_gates ``[T, G]``."""

    num_tokens, _, num_private = gates.shape
    k_q = choices.shape[-1]
    if selected is None:
        selected = stable_topk(group_gates, k_a)
    group_gate = group_gates.gather(1, selected)
    expand = selected.unsqueeze(-1)
    chosen = choices.gather(1, expand.expand(-1, -1, k_q))
    chosen_gates = gates.gather(1, expand.expand(-1, -1, num_private)).gather(2, chosen)
    expert_ids = expand * num_private + chosen
    weights = chosen_gates * group_gate.unsqueeze(-1)
    return (
        expert_ids.reshape(num_tokens, k_a * k_q),
        weights.reshape(num_tokens, k_a * k_q),
        selected,
    )


def balancing_update(choice_bias: Tensor, topk: Tensor, valid: Tensor, rate: float) -> Tensor:
    """Loss-free balancing step (nestor/backbones/nestor.py:613-634, single rank):
    one-hot the selections, count valid tokens per choice, move every bias by
    ``rate`` towards the mean load.  Returns the new bias."""

    num_choices = choice_bias.shape[0]
    one_hot = F.one_hot(topk, num_classes=num_choices).float()
    assigned = one_hot.sum(dim=-2) * valid.unsqueeze(-1).float()
    counts = assigned.reshape(-1, num_choices).sum(0)
    return choice_bias + rate * torch.sign(counts.mean() - counts)
