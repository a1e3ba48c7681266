"""Token-choice top-k routers of the expert pools.

Mirrors ``RouterOutput`` / ``Router`` (nestor/backbones/nestor.py:320-593: score
head, training-mode exploration noise, softmax, detached choice bias, top-k,
``renorm`` / ``switch`` gate, scatter, validity mask) and the batched evaluation
of a layer's ``G`` private routers (nestor/backbones/batched_router.py:97-240).
Everything after the score GEMM -- softmax, biased top-k, gates -- is one HIP
launch for the whole ``[tokens, (G,) choices]`` block, and the gradient of the
scores is one more.  The loss-free balancing update of ``choice_bias``
(nestor/backbones/nestor.py:596-634) takes its counts from a histogram launch.
A router built with a noise head perturbs its scores in training mode
(``scores + eps * softplus(noise_mlp(x))``, nestor/backbones/nestor.py:540-556), with
``eps`` drawn there or handed in pre-drawn so that a checkpoint's recompute routes
as the forward did; a router built without one is deterministic in both modes.

``torch.topk`` leaves the order of equal scores open; this implementation (and
its oracle) take equal biased scores lowest index first.
"""

from __future__ import annotations

from typing import NamedTuple

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from nestor_amd import ops

_ACTIVATIONS = {"gelu": F.gelu, "silu": F.silu, "relu": F.relu}


class RouterOutput(NamedTuple):
    scores: Tensor
    softmax_probs: Tensor
    gates: Tensor
    topk_indices: Tensor
    active_mask: Tensor
    valid_token_mask: Tensor


def score_linear(x: Tensor, weight: Tensor, bias: Tensor | None) -> Tensor:
    """``F.linear`` for a skinny score head over rows ``x [T, d]``.  When the GEMM runs
    in bf16 on the GPU and ``x`` needs a gradient, the input gradient goes through the
    grouped GEMM kernel (``ops.score_heads_op``); the head count is padded with zero
    rows to a multiple of 32 for it.  Values are those of ``F.linear``."""

    bf16 = torch.bfloat16
    if x.is_cuda and torch.is_autocast_enabled("cuda"):
        on_bf16 = torch.get_autocast_dtype("cuda") == bf16
    else:
        on_bf16 = x.dtype == bf16 and weight.dtype == bf16
    if not (x.is_cuda and on_bf16 and x.dim() == 2 and torch.is_grad_enabled() and x.requires_grad):
        return F.linear(x, weight, bias)
    heads = weight.shape[0]
    pad = -heads % 32
    w = weight.to(bf16)
    b = None if bias is None else bias.to(bf16)
    if pad:
        w = torch.cat([w, w.new_zeros(pad, w.shape[1])])
        b = None if b is None else torch.cat([b, b.new_zeros(pad)])
    with torch.autocast("cuda", enabled=False):
        out = ops.score_heads_op(x.to(bf16), w, b)
    return out[:, :heads] if pad else out


class ScoreMLP(nn.Module):
    """Score head: ``Linear`` layers with an activation between them (none after
    the last); ``hidden_dims=[]`` is the single linear map every registered arm uses."""

    def __init__(self, input_dim: int, hidden_dims: list[int], output_dim: int,
                 activation: str = "gelu", bias: bool = True) -> None:
        super().__init__()
        dims = [input_dim, *hidden_dims, output_dim]
        self.layers = nn.ModuleList(
            [nn.Linear(dims[i], dims[i + 1], bias=bias) for i in range(len(dims) - 1)]
        )
        self.activation = activation
        self._activation_fn = _ACTIVATIONS[activation]
        with torch.no_grad():
            for layer in self.layers:
                layer.weight.normal_(0.0, 1.0 / layer.in_features)
                if layer.bias is not None:
                    layer.bias.zero_()

    def forward(self, x: Tensor) -> Tensor:
        for layer in self.layers[:-1]:
            x = self._activation_fn(layer(x))
        last = self.layers[-1]
        if x.dim() >= 2 and len(self.layers) == 1:
            flat = score_linear(x.reshape(-1, x.shape[-1]), last.weight, last.bias)
            return flat.reshape(*x.shape[:-1], flat.shape[-1])
        return last(x)


def _softmax_dtype(scores: Tensor) -> torch.dtype:
    # F.softmax is on autocast's fp32 list; outside autocast it keeps the input dtype.
    return torch.float32 if torch.is_autocast_enabled(scores.device.type) else scores.dtype


def route_scores(
    scores: Tensor, choice_bias: Tensor, top_k: int, gate_mode: str, mask: Tensor
) -> tuple[Tensor, Tensor, Tensor]:
    """``(softmax_probs, topk_indices, gates)`` for ``scores [..., C]``.

    ``choice_bias`` is ``[C]`` or, for batched routers, ``[G, C]`` matching the
    second-to-last axis of ``scores``; ``mask`` has the shape of ``scores[..., 0]``.
    One HIP launch; the op carries the gradient of the scores through the gates
    and the softmax probabilities (one more launch), which is what autograd derives
    from the reference's softmax / gather / scatter chain.
    """

    shape = scores.shape
    c = shape[-1]
    mode = 1 if gate_mode == "switch" else 0
    probs, topk, gates = ops.router_topk(
        scores.reshape(-1, c), choice_bias.detach().float().reshape(-1, c), mask.reshape(-1),
        top_k, mode,
    )
    return (probs.view(shape).to(_softmax_dtype(scores)), topk.view(*shape[:-1], top_k),
            gates.view(shape))


def _is_recomputing() -> bool:
    """True inside a backward pass, i.e. when an activation checkpoint re-runs a forward
    (nestor/backbones/nestor.py:1077-1089): per-step counters must not advance then."""

    return torch._C._current_autograd_node() is not None


def _anneal_steps_from_env() -> int:
    import os

    return int(os.environ.get("NESTOR_ROUTER_NOISE_ANNEAL_STEPS", "0"))


class Router(nn.Module):
    """Top-k router over ``num_choices`` with a detached ``choice_bias`` buffer."""

    def __init__(self, feature_dim: int, num_choices: int, num_choices_per_token: int,
                 score_mlp_hidden_dims: list[int], score_mlp_activation: str = "gelu",
                 noise_mlp_hidden_dims: list[int] | None = None,
                 noise_mlp_activation: str = "gelu", *, loss_free_balancing: bool = False,
                 bias_update_rate: float = 0.0, gate_mode: str = "renorm") -> None:
        super().__init__()
        if num_choices < 1:
            raise ValueError("num_choices must be positive.")
        if not 1 <= num_choices_per_token <= num_choices:
            raise ValueError("num_choices_per_token must be in [1, num_choices].")
        if gate_mode not in ("renorm", "switch"):
            raise ValueError(f"gate_mode must be 'renorm' or 'switch', got {gate_mode!r}.")
        self.feature_dim = feature_dim
        self.num_choices = num_choices
        self.num_choices_per_token = num_choices_per_token
        self.loss_free_balancing = loss_free_balancing
        self.bias_update_rate = bias_update_rate
        self.gate_mode = gate_mode
        self.score_mlp = ScoreMLP(feature_dim, score_mlp_hidden_dims, num_choices,
                                  score_mlp_activation)
        # ``None`` (this build's default) leaves the router without a noise head:
        # deterministic in training mode too.  The reference always builds one.
        self.noise_mlp = (
            ScoreMLP(feature_dim, noise_mlp_hidden_dims, num_choices, noise_mlp_activation)
            if noise_mlp_hidden_dims is not None else None
        )
        self.register_buffer("choice_bias", torch.zeros(num_choices))
        # NESTOR_ROUTER_NOISE_ANNEAL_STEPS=N: the noise decays linearly to zero over the
        # first N training forwards (nestor/backbones/nestor.py:469-484); the counter is
        # a persistent buffer so that it survives a resume.
        self._noise_anneal_steps = _anneal_steps_from_env()
        if self._noise_anneal_steps > 0:
            self.register_buffer("_noise_steps", torch.zeros((), dtype=torch.long))

    def draw_noise(self, batch_size: int, seq_len: int, device, dtype: torch.dtype) -> Tensor:
        """The standard-normal factor of the exploration noise, ``[B, S, C]``: drawn
        outside an activation checkpoint and passed to ``forward(noise=...)`` it makes
        the recompute route exactly as the forward did
        (nestor/backbones/nestor.py:486-518)."""

        return torch.randn(batch_size, seq_len, self.num_choices, device=device, dtype=dtype)

    def _explore(self, x: Tensor, scores: Tensor, noise: Tensor | None) -> Tensor:
        if not (self.training and self.noise_mlp is not None):
            return scores
        eps = torch.randn_like(scores) if noise is None else noise.to(scores.dtype)
        perturbation = eps * F.softplus(self.noise_mlp(x))
        if self._noise_anneal_steps > 0:
            done = (self._noise_steps.float() / self._noise_anneal_steps).clamp(max=1.0)
            perturbation = perturbation * (1.0 - done)
            if not _is_recomputing():
                self._noise_steps += 1
        return scores + perturbation

    def forward(self, x: Tensor, valid_token_mask: Tensor, noise: Tensor | None = None,
                scores: Tensor | None = None) -> RouterOutput:
        """``noise``: pre-drawn ``N(0, 1)`` factor of the training noise (``None``: drawn
        here); ignored outside training mode or without a noise head.  ``scores``: the
        score head's output when the caller already computed it (one GEMM for several
        heads that read the same rows)."""

        if scores is None:
            scores = self.score_mlp(x)
        scores = self._explore(x, scores, noise)
        probs, topk, gates = route_scores(
            scores, self.choice_bias, self.num_choices_per_token, self.gate_mode, valid_token_mask
        )
        return RouterOutput(scores, probs, gates, topk, gates > 0, valid_token_mask)

    @torch.no_grad()
    def update_detached_parameters(self, topk_indices: Tensor, valid_token_mask: Tensor) -> None:
        """Loss-free balancing (nestor/backbones/nestor.py:596-634): nudge the detached
        ``choice_bias`` by ``bias_update_rate`` towards the mean load.  The per-choice
        counts come from one histogram launch; the sum over data-parallel ranks the
        reference offers under ``NESTOR_LOSSFREE_GLOBAL_COUNTS`` belongs to a
        multi-GPU run and is not part of this build."""

        if not self.loss_free_balancing:
            return
        counts = ops.router_choice_counts(
            topk_indices.reshape(-1, topk_indices.shape[-1]), valid_token_mask.reshape(-1),
            self.num_choices,
        ).float()
        error = counts.mean() - counts
        self.choice_bias += self.bias_update_rate * torch.sign(error)


def check_batchable(routers: list[Router]) -> None:
    """Raise unless the routers can run as one batched router."""

    if not routers:
        raise ValueError("Need at least one router to batch.")

    def mlp_signature(mlp) -> tuple:
        if mlp is None:
            return ()
        return (tuple((l.in_features, l.out_features, l.bias is not None) for l in mlp.layers),
                mlp.activation)

    def signature(r: Router) -> tuple:
        return (r.num_choices, r.num_choices_per_token, r.gate_mode, mlp_signature(r.score_mlp),
                mlp_signature(r.noise_mlp))

    if any(signature(r) != signature(routers[0]) for r in routers[1:]):
        raise ValueError("Private routers differ in shape/gate mode; cannot batch them.")


def batched_mlp(x: Tensor, mlps: list[ScoreMLP]) -> Tensor:
    """``[N, G, d_out]``: ``G`` same-shaped heads on shared rows -- one GEMM for the
    first layers (weights concatenated along the output axis), one ``[G]``-batched
    matmul per later layer."""

    heads = len(mlps)
    w0 = torch.stack([m.layers[0].weight for m in mlps])
    b0 = (
        torch.stack([m.layers[0].bias for m in mlps]).reshape(-1)
        if mlps[0].layers[0].bias is not None else None
    )
    hidden = score_linear(x, w0.reshape(heads * w0.shape[1], w0.shape[2]), b0)
    hidden = hidden.view(x.shape[0], heads, w0.shape[1])
    for index in range(1, len(mlps[0].layers)):
        hidden = mlps[0]._activation_fn(hidden)
        w = torch.stack([m.layers[index].weight for m in mlps])
        hidden = torch.einsum("ngi,goi->ngo", hidden, w)
        if mlps[0].layers[index].bias is not None:
            hidden = hidden + torch.stack([m.layers[index].bias for m in mlps])
    return hidden


def route_private_batched(
    routers: list[Router], x: Tensor, valid_token_mask: Tensor, group_active_mask: Tensor,
    training: bool, noise: Tensor | None = None, scores: Tensor | None = None,
) -> tuple[list[RouterOutput], Tensor, Tensor]:
    """All ``G`` private routers of a layer in one pass: per-group outputs (views
    of the stacked tensors, masked to ``valid & member``), stacked gates
    ``[B, S, G, Q]`` and stacked choices ``[B, S, G, k]``.  ``scores``
    (``[B*S, G*Q]``, head-major) skips the score GEMM when the caller has it.
    ``training`` with noise heads: every router's scores are perturbed as in
    ``Router.forward``, from ONE draw ``[B, S, G, Q]`` (or the pre-drawn ``noise``) and
    one batched noise-head GEMM; each router's anneal counter advances as it would
    alone (nestor/backbones/batched_router.py:188-208)."""

    first = routers[0]
    groups = len(routers)
    batch, seq, dim = x.shape
    flat_x = x.reshape(batch * seq, dim)
    if scores is None:
        scores = batched_mlp(flat_x, [r.score_mlp for r in routers])
    scores = scores.reshape(batch, seq, groups, first.num_choices)
    if training and first.noise_mlp is not None:
        spread = F.softplus(batched_mlp(flat_x, [r.noise_mlp for r in routers]).view_as(scores))
        eps = torch.randn_like(scores) if noise is None else noise.to(scores.dtype)
        perturbation = eps * spread
        if any(r._noise_anneal_steps > 0 for r in routers):
            done = torch.stack([
                (r._noise_steps.float() / r._noise_anneal_steps).clamp(max=1.0)
                if r._noise_anneal_steps > 0 else torch.zeros((), device=x.device)
                for r in routers
            ])
            perturbation = perturbation * (1.0 - done).to(perturbation.dtype)[None, None, :, None]
            if not _is_recomputing():
                for r in routers:
                    if r._noise_anneal_steps > 0:
                        r._noise_steps += 1
        scores = scores + perturbation
    bias = torch.stack([r.choice_bias for r in routers])
    member = valid_token_mask.unsqueeze(-1) & group_active_mask
    probs, topk, gates = route_scores(
        scores, bias, first.num_choices_per_token, first.gate_mode, member
    )
    active = gates > 0
    outputs = [
        RouterOutput(scores[:, :, g], probs[:, :, g], gates[:, :, g], topk[:, :, g],
                     active[:, :, g], member[:, :, g])
        for g in range(groups)
    ]
    return outputs, gates, topk
