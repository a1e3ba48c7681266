"""The hybrid public / column-private expert-pool MLP on the HIP path.

Mirrors ``ExpertPoolMLP`` (nestor/backbones/expert_pools.py:110-1114): for each
token

    MLP(h) = a_pub  * sum_e public_gate_e * PublicExpert_e(h)
           + a_priv * sum_g column_gate_g * sum_e private_gate_(g,e) * PrivateExpert_(g,e)(h)

with ``(a_pub, a_priv) = softmax(path_gate(h))``.  The public pool is one bank
call (``slots = k_p``), the ``G x Q`` private experts one flattened bank indexed
``g * Q + e`` (``slots = k_a * k_q``).  Three output layouts: summed
(``forward``), per column (``forward_per_group``) and per attention slot
(``forward_per_slot``).
"""

from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from nestor_amd import flags, ops
from nestor_amd.bank import Linear2, StackedBanksMixin, SwigluExpert
from nestor_amd.grouped import grouped_expert_combine
from nestor_amd.router import (
    Router, RouterOutput, check_batchable, route_private_batched, score_linear,
)


def round_to_multiple_of_8(value: float) -> int:
    """``max(8, round(value / 8) * 8)`` (nestor/backbones/expert_pool_dispatch.py:25-35)."""

    return max(8, int(round(value / 8.0)) * 8)


def public_expert_hidden_dim(dim: int, public_top_k: int, *, active_budget: float | None = None) -> int:
    """``round8(budget * d / k_p)``, budget 2 by default (expert_pool_dispatch.py:38-62)."""

    budget = 2.0 if active_budget is None else float(active_budget)
    return round_to_multiple_of_8(budget * dim / public_top_k)


def private_expert_hidden_dim(dim: int, num_groups_per_token: int, private_top_k: int, *,
                              with_public_pool: bool = True,
                              active_budget: float | None = None) -> int:
    """``round8(budget * d / (k_a * k_q))``; budget 2 beside a public pool, 4 alone
    (expert_pool_dispatch.py:65-105)."""

    if active_budget is not None:
        budget = float(active_budget)
    else:
        budget = 2.0 if with_public_pool else 4.0
    return round_to_multiple_of_8(budget * dim / (num_groups_per_token * private_top_k))


_KERNEL_STREAM_DTYPES = (torch.bfloat16, torch.float32)


class ExpertPoolMLP(StackedBanksMixin, nn.Module):
    """Public + column-private SwiGLU expert pools behind layer-local routers."""

    def __init__(self, dim: int, num_groups: int, num_groups_per_token: int,
                 num_public_experts: int, public_top_k: int, num_private_experts: int,
                 private_top_k: int, router_score_mlp_hidden_dims: list[int],
                 router_score_mlp_activation: str = "gelu",
                 router_noise_mlp_hidden_dims: list[int] | None = None,
                 router_noise_mlp_activation: str = "gelu", *,
                 loss_free_balancing: bool = False, bias_update_rate: float = 0.0,
                 active_budget: float | None = None, public_budget: float | None = None,
                 private_gate_mode: str = "renorm") -> None:
        super().__init__()
        if num_private_experts < 1:
            raise ValueError("ExpertPoolMLP requires a private pool: num_private_experts must be > 0.")
        if not 1 <= num_groups_per_token <= num_groups:
            raise ValueError("num_groups_per_token must be in [1, num_groups].")
        self.dim = dim
        self.num_groups = num_groups
        self.num_groups_per_token = num_groups_per_token
        self.num_public_experts = num_public_experts
        self.public_top_k = public_top_k
        self.num_private_experts = num_private_experts
        self.private_top_k = private_top_k
        self.private_gate_mode = private_gate_mode
        self.has_public_pool = num_public_experts > 0
        self.public_hidden_dim = (
            public_expert_hidden_dim(dim, public_top_k, active_budget=public_budget)
            if self.has_public_pool else 0
        )
        self.private_hidden_dim = private_expert_hidden_dim(
            dim, num_groups_per_token, private_top_k,
            with_public_pool=self.has_public_pool, active_budget=active_budget,
        )

        def make_router(choices: int, top_k: int, gate_mode: str = "renorm") -> Router:
            return Router(dim, choices, top_k, router_score_mlp_hidden_dims,
                          router_score_mlp_activation, router_noise_mlp_hidden_dims,
                          router_noise_mlp_activation, loss_free_balancing=loss_free_balancing,
                          bias_update_rate=bias_update_rate, gate_mode=gate_mode)

        self.public_router = make_router(num_public_experts, public_top_k) if self.has_public_pool else None
        self.private_routers = nn.ModuleList(
            [make_router(num_private_experts, private_top_k, private_gate_mode) for _ in range(num_groups)]
        )
        self.public_experts = (
            nn.ModuleList([SwigluExpert(dim, self.public_hidden_dim, dim) for _ in range(num_public_experts)])
            if self.has_public_pool else None
        )
        self.private_experts = nn.ModuleList(
            [nn.ModuleList([SwigluExpert(dim, self.private_hidden_dim, dim)
                            for _ in range(num_private_experts)]) for _ in range(num_groups)]
        )
        if self.has_public_pool:
            self.path_gate = Linear2(dim, 2, bias=False)
            with torch.no_grad():
                self.path_gate.weight.zero_()  # alpha = (0.5, 0.5) at step 0
        else:
            self.path_gate = None
        self.grouped_dispatch = False if flags.pool_grouped_mm_disabled() else None
        self.fused_gate = flags.fused_gate_requested()
        self.triton_index = flags.triton_index_requested() and flags.triton_index_available()
        self.triton_fused = flags.triton_expert_requested() and flags.triton_expert_available()
        self.triton_cat_cast = flags.triton_cat_cast_requested()
        self.batched_routers = flags.batched_routers_enabled() and num_groups > 1
        if self.batched_routers:
            check_batchable(list(self.private_routers))
        self._declare_expert_banks(
            [("stacked_public", self.public_experts), ("stacked_private", self._private_bank())]
        )

    @classmethod
    def from_stacked(cls, dim: int, num_groups: int, num_groups_per_token: int,
                     stacked_public, stacked_private, public_top_k: int, private_top_k: int,
                     *, private_gate_mode: str = "switch",
                     router_score_mlp_hidden_dims: list[int] | None = None) -> "ExpertPoolMLP":
        """A pool around banks that already exist in the stacked layout
        (``StackedExpertBank``; private bank index ``column * Q + expert``).  No
        per-expert modules are built: the banks are the only owners of the expert
        weights, which is how a stacked-layout checkpoint or a large synthetic
        bank enters without materialising ``P + G*Q`` separate modules first."""

        self = cls.__new__(cls)
        nn.Module.__init__(self)
        p = stacked_public.num_experts if stacked_public is not None else 0
        q = stacked_private.num_experts // num_groups
        self.dim, self.num_groups, self.num_groups_per_token = dim, num_groups, num_groups_per_token
        self.num_public_experts, self.public_top_k = p, public_top_k
        self.num_private_experts, self.private_top_k = q, private_top_k
        self.private_gate_mode = private_gate_mode
        self.has_public_pool = p > 0
        self.public_hidden_dim = stacked_public.w_up.shape[-1] if p > 0 else 0
        self.private_hidden_dim = stacked_private.w_up.shape[-1]
        hidden = router_score_mlp_hidden_dims or []
        self.public_router = Router(dim, p, public_top_k, hidden) if p > 0 else None
        self.private_routers = nn.ModuleList(
            [Router(dim, q, private_top_k, hidden, gate_mode=private_gate_mode)
             for _ in range(num_groups)]
        )
        self.public_experts = None
        self.private_experts = None
        if p > 0:
            self.path_gate = Linear2(dim, 2, bias=False)
            with torch.no_grad():
                self.path_gate.weight.zero_()
        else:
            self.path_gate = None
        self.grouped_dispatch = None
        self.fused_gate = True
        self.triton_index = self.triton_fused = True
        self.triton_cat_cast = True
        self.batched_routers = num_groups > 1
        self._stacked_bank_specs, self._stacked_view_sources = [], []
        self.stacked_public = stacked_public
        self.stacked_private = stacked_private
        return self

    def enable_bf16_shadow(self, enabled: bool = True) -> "ExpertPoolMLP":
        """Persistent bf16 copies of both stacked banks' fp32 owners (see
        ``StackedExpertBank.enable_bf16_shadow``); a no-op for banks that are not stacked."""

        for bank in (self.stacked_public, self.stacked_private):
            if bank is not None:
                bank.enable_bf16_shadow(enabled)
        return self

    def refresh_shadow(self, in_place: bool = False) -> None:
        """``StackedExpertBank.refresh_shadow`` on both stacked banks (after an optimizer step
        when the step is replayed as a captured graph: ``in_place=True``)."""

        for bank in (self.stacked_public, self.stacked_private):
            if bank is not None and bank.__dict__.get("_shadow_enabled", False):
                bank.refresh_shadow(in_place)

    # -- slots ---------------------------------------------------------------
    def _private_bank(self) -> list[nn.Module]:
        if self.private_experts is None:
            return self.stacked_private.expert_views()
        return [expert for column in self.private_experts for expert in column]

    def _public_bank(self) -> list[nn.Module]:
        if self.public_experts is None:
            return self.stacked_public.expert_views()
        return list(self.public_experts)

    def _public_slots(self, public_output: RouterOutput, num_tokens: int) -> tuple[Tensor, Tensor]:
        ids = public_output.topk_indices.reshape(num_tokens, self.public_top_k)
        gates = public_output.gates.reshape(num_tokens, self.num_public_experts)
        return ids, gates.gather(1, ids)

    def _private_slots(self, private_outputs: list[RouterOutput], flat_group_gates: Tensor,
                       num_tokens: int, selected: Tensor | None = None,
                       stacked: tuple[Tensor, Tensor] | None = None) -> tuple[Tensor, Tensor, Tensor]:
        """ids ``column * Q + expert`` and weights ``private_gate * column_gate`` for
        the ``k_a * k_q`` private rows of every token, slot-major."""

        k_a, k_q, q = self.num_groups_per_token, self.private_top_k, self.num_private_experts
        if stacked is None:
            gates = torch.stack([o.gates for o in private_outputs], dim=-2)
            choices = torch.stack([o.topk_indices for o in private_outputs], dim=-2)
        else:
            gates, choices = stacked
        gates = gates.reshape(num_tokens, self.num_groups, q)
        choices = choices.reshape(num_tokens, self.num_groups, k_q)
        if (flat_group_gates.is_cuda and self.num_groups <= 64
                and gates.dtype == flat_group_gates.dtype
                and gates.dtype in (torch.bfloat16, torch.float32)):
            # one launch (and one for both gate gradients) instead of top-k + gathers
            picked = None if selected is None else selected.reshape(num_tokens, k_a)
            selected, ids, weights = ops.private_slots_op(flat_group_gates, gates, choices, picked, k_a)
            return ids, weights, selected
        if selected is None:
            selected = torch.topk(flat_group_gates, k_a, dim=-1).indices
        else:
            selected = selected.reshape(num_tokens, k_a)
        column_gate = flat_group_gates.gather(1, selected)
        col = selected.unsqueeze(-1)
        chosen = choices.gather(1, col.expand(-1, -1, k_q))
        chosen_gates = gates.gather(1, col.expand(-1, -1, q)).gather(2, chosen)
        ids = col * q + chosen
        weights = chosen_gates * column_gate.unsqueeze(-1)
        return ids.reshape(num_tokens, k_a * k_q), weights.reshape(num_tokens, k_a * k_q), selected

    # -- routing -------------------------------------------------------------
    def _fused_head_scores(self, x: Tensor):
        """Scores of the public router, the ``G`` private routers and the path gate
        from ONE GEMM over ``x`` when all of them are single linear maps: they read
        the same rows, and at production widths each separate skinny GEMM costs a
        full pass over the activations (forward) and one more for its input
        gradient (backward).  ``None`` when the heads cannot be fused."""

        if not (self.batched_routers and self.public_router is not None):
            return None
        heads = [self.public_router.score_mlp, *[r.score_mlp for r in self.private_routers]]
        if any(len(h.layers) != 1 for h in heads):
            return None
        layers = [h.layers[0] for h in heads] + [self.path_gate]
        weight = torch.cat([l.weight for l in layers])
        bias = None
        if any(l.bias is not None for l in layers):
            bias = torch.cat([
                l.bias if l.bias is not None else l.weight.new_zeros(l.weight.shape[0])
                for l in layers
            ])
        out = score_linear(x.reshape(-1, self.dim), weight, bias)
        n_pub = layers[0].weight.shape[0]
        n_priv = sum(l.weight.shape[0] for l in layers[1:-1])
        return (out[:, :n_pub].reshape(*x.shape[:-1], n_pub), out[:, n_pub:n_pub + n_priv],
                out[:, n_pub + n_priv:].reshape(*x.shape[:-1], -1))

    def _route(self, x: Tensor, valid: Tensor, group_active: Tensor, router_noise=None):
        """``(public_output, private_outputs, stacked, path_logits)``: ``stacked`` holds the
        batched routers' ``[B, S, G, Q]`` gates and ``[B, S, G, k]`` choices (``None`` for
        per-column routers), ``path_logits`` the path gate's scores when the fused score
        GEMM produced them (``None``: the caller evaluates the path gate itself).

        The public router runs first, then the ``G`` private ones: routers with a noise
        head draw from the RNG in training mode, so the order is part of the contract
        (nestor/backbones/expert_pools.py:533-586).  ``router_noise``: the pre-drawn
        factors of ``draw_router_noise`` (``"public"`` ``[B, S, P]``, ``"private"``
        ``[B, S, G, Q]``); ``None`` lets each router draw its own."""

        public_noise = None if router_noise is None else router_noise.get("public")
        private_noise = None if router_noise is None else router_noise.get("private")
        fused = self._fused_head_scores(x)
        if fused is not None:
            pub_scores, priv_scores, path_logits = fused
            public_output = self.public_router(x, valid, noise=public_noise, scores=pub_scores)
            outs, gates, choices = route_private_batched(
                list(self.private_routers), x, valid, group_active, training=self.training,
                noise=private_noise, scores=priv_scores,
            )
            return public_output, outs, (gates, choices), path_logits
        public_output = (
            self.public_router(x, valid, noise=public_noise) if self.public_router is not None else None
        )
        if self.batched_routers:
            outs, gates, choices = route_private_batched(
                list(self.private_routers), x, valid, group_active, training=self.training,
                noise=private_noise,
            )
            return public_output, outs, (gates, choices), None
        outs = [
            self.private_routers[g](
                x, valid & group_active[:, :, g],
                noise=None if private_noise is None else private_noise[:, :, g],
            )
            for g in range(self.num_groups)
        ]
        return public_output, outs, None, None

    def draw_router_noise(self, batch_size: int, seq_len: int, device, dtype: torch.dtype) -> dict:
        """Every pool router's standard-normal noise factor, drawn in one place (outside an
        activation checkpoint) and handed back through ``router_noise`` so that a recompute
        routes as the forward did (nestor/backbones/expert_pools.py:588-623): ``"private"``
        ``[B, S, G, Q]`` and, with a public pool, ``"public"`` ``[B, S, P]``."""

        noise = {
            "private": torch.randn(batch_size, seq_len, self.num_groups, self.num_private_experts,
                                   device=device, dtype=dtype)
        }
        if self.public_router is not None:
            noise["public"] = self.public_router.draw_noise(batch_size, seq_len, device, dtype)
        return noise

    # -- banks ---------------------------------------------------------------
    def _bank(self, flat_x: Tensor, experts, stacked, ids: Tensor, weights: Tensor, group: int) -> Tensor:
        return grouped_expert_combine(
            flat_x, experts, ids, weights, group, fused_gate=self.fused_gate, stacked=stacked,
            triton_index=self.triton_index, triton_fused=self.triton_fused,
            triton_cat_cast=self.triton_cat_cast,
        )

    def _public_update(self, flat_x: Tensor, public_output: RouterOutput, num_tokens: int) -> Tensor:
        ids, weights = self._public_slots(public_output, num_tokens)
        return self._bank(flat_x, self._public_bank(), self.stacked_public, ids, weights,
                          self.public_top_k).reshape(num_tokens, self.dim)

    def _private_per_slot(self, flat_x: Tensor, ids: Tensor, weights: Tensor) -> Tensor:
        return self._bank(flat_x, self._private_bank(), self.stacked_private, ids, weights,
                          self.private_top_k)

    def _path_weights(self, x: Tensor, logits: Tensor | None) -> Tensor:
        if logits is None:
            logits = self.path_gate(x)
        return F.softmax(logits.float(), dim=-1).to(x.dtype)

    def _prologue(self, x: Tensor, valid: Tensor, group_gates: Tensor, group_active: Tensor,
                  router_noise=None):
        flat_x = x.reshape(-1, self.dim)
        num_tokens = flat_x.shape[0]
        flat_gates = group_gates.reshape(num_tokens, self.num_groups)
        public_output, private_outputs, stacked, path_logits = self._route(
            x, valid, group_active, router_noise)
        public_update = (
            self._public_update(flat_x, public_output, num_tokens).reshape_as(x)
            if public_output is not None else None
        )
        return (flat_x, num_tokens, flat_gates, public_output, private_outputs, stacked,
                public_update, path_logits)

    # -- forwards ------------------------------------------------------------
    def forward(self, x: Tensor, valid_token_mask: Tensor, group_gates: Tensor,
                group_active_mask: Tensor, router_noise=None):
        """Summed layout: ``(update [B,S,d], public_output, private_outputs)``."""

        flat_x, n, flat_gates, pub_out, priv_outs, stacked, public_update, path_logits = self._prologue(
            x, valid_token_mask, group_gates, group_active_mask, router_noise
        )
        ids, weights, _ = self._private_slots(priv_outs, flat_gates, n, stacked=stacked)
        private_update = self._bank(
            flat_x, self._private_bank(), self.stacked_private, ids, weights, ids.shape[1]
        ).reshape_as(x)
        if public_update is None:
            return private_update.to(x.dtype), pub_out, priv_outs
        alpha = self._path_weights(x, path_logits)
        if x.dtype in _KERNEL_STREAM_DTYPES:
            update = ops.path_mix_op(public_update, private_update, alpha)
        else:  # other stream dtypes: the reference's eager expression
            update = (alpha[..., 0:1] * public_update + alpha[..., 1:2] * private_update).to(x.dtype)
        return update, pub_out, priv_outs

    def forward_per_slot(self, x: Tensor, valid_token_mask: Tensor, group_gates: Tensor,
                         group_active_mask: Tensor, slot_groups: Tensor, router_noise=None):
        """Slot layout: ``(public [B,S,d] | None, private [B,S,k_a,d], ...)``."""

        flat_x, n, flat_gates, pub_out, priv_outs, stacked, public_update, path_logits = self._prologue(
            x, valid_token_mask, group_gates, group_active_mask, router_noise
        )
        ids, weights, _ = self._private_slots(
            priv_outs, flat_gates, n, selected=slot_groups.reshape(n, self.num_groups_per_token), stacked=stacked
        )
        per_slot = self._private_per_slot(flat_x, ids, weights).view(
            x.shape[0], x.shape[1], self.num_groups_per_token, self.dim
        )
        return self._gate_split(x, public_update, per_slot, pub_out, priv_outs, path_logits)

    def forward_per_group(self, x: Tensor, valid_token_mask: Tensor, group_gates: Tensor,
                          group_active_mask: Tensor, router_noise=None):
        """Column layout: ``(public [B,S,d] | None, private [B,S,G,d], ...)``."""

        flat_x, n, flat_gates, pub_out, priv_outs, stacked, public_update, path_logits = self._prologue(
            x, valid_token_mask, group_gates, group_active_mask, router_noise
        )
        ids, weights, selected = self._private_slots(priv_outs, flat_gates, n, stacked=stacked)
        per_slot = self._private_per_slot(flat_x, ids, weights)
        return self._gate_split(x, public_update, per_slot, pub_out, priv_outs, path_logits, columns=selected)

    def _gate_split_eager(self, x, public_update, per_slot, pub_out, priv_outs, path_logits, columns):
        """The reference's op chain (expert_pools.py:758-761,943-953), for stream dtypes
        the kernels do not take."""

        split = per_slot
        if columns is not None:
            index = columns.reshape(*x.shape[:-1], -1, 1).expand_as(per_slot)
            split = per_slot.new_zeros(*x.shape[:-1], self.num_groups, self.dim).scatter_add(
                -2, index, per_slot)
        if public_update is None:
            return None, split.to(x.dtype), pub_out, priv_outs
        alpha = self._path_weights(x, path_logits)
        return ((alpha[..., 0:1] * public_update).to(x.dtype),
                (alpha[..., 1:2].unsqueeze(-1) * split).to(x.dtype), pub_out, priv_outs)

    def _gate_split(self, x, public_update, per_slot, pub_out, priv_outs, path_logits, columns=None):
        """Outputs of the split layouts from the per-slot rows ``[n or B,S, k_a, d]``.
        ``columns [n, k_a]`` scatters the slots onto the ``G`` column streams
        (``zeros.scatter_add`` in the reference, expert_pools.py:758-761); the path
        weights scale both parts.  One launch per part."""

        lead = x.shape[:-1]
        per_slot = per_slot.reshape(*lead, self.num_groups_per_token, self.dim)
        if x.dtype not in _KERNEL_STREAM_DTYPES:
            return self._gate_split_eager(x, public_update, per_slot, pub_out, priv_outs, path_logits, columns)
        width = per_slot.shape[-2] if columns is None else self.num_groups
        dest = None if columns is None else columns.reshape(*lead, self.num_groups_per_token)
        if public_update is None:
            if dest is None:
                return None, per_slot.to(x.dtype), pub_out, priv_outs
            ones = per_slot.new_ones(*lead, 2)  # a private-only pool has the constant weight 1
            return None, ops.path_scale_op(per_slot, ones, 1, dest, width), pub_out, priv_outs
        alpha = self._path_weights(x, path_logits)
        return (
            ops.path_scale_op(public_update.reshape(*lead, 1, self.dim), alpha, 0, None, 1)
            .reshape_as(x),
            ops.path_scale_op(per_slot, alpha, 1, dest, width),
            pub_out,
            priv_outs,
        )
