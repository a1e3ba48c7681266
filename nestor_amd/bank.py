"""Expert modules and their stacked parameter ownership.

``StackedExpertBank`` keeps the layout contract of
nestor/backbones/expert_bank_stack.py:58-213 -- ``w_up`` / ``w_gate``
``[E, d_in, hidden]`` (each expert's ``weight.t()``), ``w_down``
``[E, hidden, d_out]``, optional bias banks -- so a state dict written by one
side loads into the other.  ``SwigluExpert`` / ``Linear2`` are the minimal
modules with the attribute surface the grouped path reads
(``layers[0]``, ``layers[1]``, ``gate``, ``gated``, ``activation``;
nestor/scaling/blocks.py:251-312).
"""

from __future__ import annotations

import math
from collections.abc import Sequence

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from nestor_amd.flags import stacked_banks_requested

_ACTIVATIONS = {"silu": F.silu, "gelu": F.gelu, "relu": F.relu}


class Linear2(nn.Module):
    """A linear map with ``weight [out, in]`` and optional ``bias`` whose
    parameters can later be re-pointed at views of a stacked owner."""

    def __init__(self, in_features: int, out_features: int, bias: bool = False) -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.weight = nn.Parameter(torch.empty(out_features, in_features))
        self.bias = nn.Parameter(torch.zeros(out_features)) if bias else None
        with torch.no_grad():
            self.weight.normal_(0.0, 1.0 / math.sqrt(in_features))

    def forward(self, x: Tensor) -> Tensor:
        return F.linear(x, self.weight, self.bias)


class SwigluExpert(nn.Module):
    """``down(act(gate(x)) * up(x))``; up/down are ``layers[0]`` / ``layers[1]``."""

    gated = True

    def __init__(self, input_dim: int, hidden_dim: int, output_dim: int,
                 activation: str = "silu", bias: bool = False) -> None:
        super().__init__()
        self.input_dim, self.output_dim = input_dim, output_dim
        self.hidden_dims = [hidden_dim]
        self.activation = activation
        self.layers = nn.ModuleList(
            [Linear2(input_dim, hidden_dim, bias), Linear2(hidden_dim, output_dim, bias)]
        )
        self.gate = Linear2(input_dim, hidden_dim, False)
        self._activation_fn = _ACTIVATIONS[activation]

    def forward(self, x: Tensor) -> Tensor:
        return self.layers[1](self._activation_fn(self.gate(x)) * self.layers[0](x))


class StackedExpertBank(nn.Module):
    """One bank of shape-identical experts owned as stacked parameters."""

    def __init__(self, experts: Sequence[nn.Module]) -> None:
        super().__init__()
        first = experts[0]
        if len(first.layers) != 2:
            raise ValueError("StackedExpertBank expects 2-layer (single-hidden) experts.")
        gated = bool(getattr(first, "gated", False))
        biased = first.layers[0].bias is not None
        for e in experts:
            if bool(getattr(e, "gated", False)) != gated or len(e.layers) != 2:
                raise ValueError("StackedExpertBank expects a structurally uniform bank.")
            if any((lin.bias is not None) != biased for lin in e.layers):
                raise ValueError("StackedExpertBank expects uniform bias presence.")
            if gated and e.gate.bias is not None:
                raise ValueError("StackedExpertBank expects bias-free gates (standard SwiGLU).")
        self.num_experts = len(experts)
        self.gated = gated

        def owner(tensors: list[Tensor]) -> nn.Parameter:
            with torch.no_grad():
                return nn.Parameter(torch.stack(tensors).contiguous())

        self.w_up = owner([e.layers[0].weight.t() for e in experts])
        self.w_gate = owner([e.gate.weight.t() for e in experts]) if gated else None
        self.w_down = owner([e.layers[1].weight.t() for e in experts])
        self.b_up = owner([e.layers[0].bias for e in experts]) if biased else None
        self.b_down = owner([e.layers[1].bias for e in experts]) if biased else None
        self.install_views(experts)

    @classmethod
    def from_tensors(cls, w_up: Tensor, w_gate: Tensor | None, w_down: Tensor) -> "StackedExpertBank":
        """A bias-free bank that adopts already-stacked tensors (``[E, d_in, h]``,
        ``[E, d_in, h]`` or None, ``[E, h, d_out]``) as its owners without going
        through per-expert modules -- how a checkpoint in the stacked layout or a
        synthetic benchmark bank enters."""

        bank = cls.__new__(cls)
        nn.Module.__init__(bank)
        bank.num_experts = w_up.shape[0]
        bank.gated = w_gate is not None
        bank.w_up = nn.Parameter(w_up)
        bank.w_gate = nn.Parameter(w_gate) if w_gate is not None else None
        bank.w_down = nn.Parameter(w_down)
        bank.b_up = None
        bank.b_down = None
        return bank

    def expert_views(self, activation: str = "silu") -> list["ExpertView"]:
        """Per-expert read-only handles with the attribute surface the grouped
        path inspects (``gated``, ``activation``, ``layers[i].weight/.bias``,
        ``gate.weight``), as views of the owners."""

        cached = self.__dict__.get("_views")
        if cached is None or cached[0] != activation:
            views = [ExpertView(self, i, activation) for i in range(self.num_experts)]
            self.__dict__["_views"] = cached = (activation, views)
        return cached[1]

    def install_views(self, experts: Sequence[nn.Module]) -> None:
        """Re-point every expert's ``weight`` / ``bias`` at a view of the owners;
        the per-expert entries leave ``_parameters`` so the model exposes each
        bank once.  Re-run after any ``_apply`` (``.to()`` / ``.cuda()``)."""

        for i, e in enumerate(experts):
            pairs = [(e.layers[0], self.w_up), (e.layers[1], self.w_down)]
            if self.gated:
                pairs.append((e.gate, self.w_gate))
            for linear, bank in pairs:
                linear._parameters.pop("weight", None)
                linear.weight = bank[i].t()
            if self.b_up is not None:
                for linear, bank in ((e.layers[0], self.b_up), (e.layers[1], self.b_down)):
                    linear._parameters.pop("bias", None)
                    linear.bias = bank[i]

    def cast(self, dtype: torch.dtype) -> tuple[Tensor, Tensor | None, Tensor]:
        """``(w_up, w_gate, w_down)`` in the GEMM dtype, one cast each (none when
        the owners already are that dtype)."""

        return (
            self.w_up.to(dtype),
            self.w_gate.to(dtype) if self.w_gate is not None else None,
            self.w_down.to(dtype),
        )

    # -- bf16 shadow of fp32 owners --------------------------------------------
    def enable_bf16_shadow(self, enabled: bool = True) -> "StackedExpertBank":
        """Keep a persistent bf16 copy of fp32 owners for the GEMMs.

        Without it a bank with fp32 owners narrows all three tensors on every bank
        call and widens all three gradients again (at the 1b-like shape 22 GB of
        pure traffic per direction and micro-step).  With it the GEMMs read the
        copy, the weight-gradient GEMM writes fp32 straight into the owners'
        gradient, and the copy is rebuilt only when an owner has changed (an
        optimizer step bumps the tensor's version counter; ``refresh_shadow()``
        forces it) -- the arrangement of nestor/scaling/bf16_master.py:1-40 seen
        from the other side: fp32 masters stay the parameters, bf16 is the cache.

        What the version counter does not see is a write through ``.data``
        (``p.data.copy_(...)`` leaves ``p._version`` alone), and the reference writes
        owners exactly that way: the EMA swap around evaluation
        (nestor/train/trainer.py:974-999) and the master restore of a resumed Muon
        state (nestor/scaling/muon.py:582).  Therefore: in evaluation mode the copy is
        rebuilt on EVERY call (evaluation is where the EMA weights are swapped in and
        out with no mode change in between, trainer.py:557-563; one cast per bank call
        is what the path without a shadow pays anyway); every ``train()`` / ``eval()``
        transition and every ``load_state_dict`` drops the copy; and code that writes
        an owner through ``.data`` while the module stays in training mode (the Muon
        resume, when a forward has already run) must call ``refresh_shadow()``."""

        self.__dict__["_shadow_enabled"] = bool(enabled)
        if not enabled:
            self.__dict__.pop("_shadow", None)
        return self

    def invalidate_shadow(self) -> None:
        """Forget the bf16 copies; the next bank call rebuilds them from the owners."""

        self.__dict__.pop("_shadow", None)

    def refresh_shadow(self, in_place: bool = False) -> None:
        """Rebuild the bf16 copies from the owners now.

        ``in_place``: rewrite the existing copies instead of making new tensors, so that
        their addresses stay what a captured HIP graph of the step reads (the replays do
        not re-run this host-side check: call this after every optimizer step, outside the
        graph).  Only between steps: an autograd graph that saved the copies and has not
        run its backward yet would see them change under it."""

        owners = (self.w_up, self.w_gate, self.w_down)
        cached = self.__dict__.get("_shadow")
        with torch.no_grad():
            if in_place and cached is not None and all(
                (c is None) == (o is None) and (c is None or (c.shape == o.shape and c.device == o.device))
                for c, o in zip(cached[1], owners)
            ):
                copies = cached[1]
                for c, o in zip(copies, owners):
                    if c is not None:
                        c.copy_(o.detach())
            else:
                copies = tuple(None if o is None else o.detach().to(torch.bfloat16) for o in owners)
        key = tuple(None if o is None else (o.data_ptr(), o._version) for o in owners)
        self.__dict__["_shadow"] = (key, copies)

    def train(self, mode: bool = True):
        if bool(mode) != self.training:
            self.invalidate_shadow()
        return super().train(mode)

    def _load_from_state_dict(self, *args, **kwargs):
        self.invalidate_shadow()
        return super()._load_from_state_dict(*args, **kwargs)

    def shadowed(self, dtype: torch.dtype):
        """``((w_up, w_gate, w_down) bf16 copies, (owner_up, owner_gate, owner_down))`` when
        the shadow is on and applies (fp32 owners, bf16 GEMMs, no bias banks -- the fused
        path), else ``None``.  The copies carry no gradient: the owners receive it."""

        if not self.__dict__.get("_shadow_enabled", False):
            return None
        if dtype != torch.bfloat16 or self.w_up.dtype != torch.float32 or self.b_up is not None:
            return None
        owners = (self.w_up, self.w_gate, self.w_down)
        key = tuple(None if o is None else (o.data_ptr(), o._version) for o in owners)
        cached = self.__dict__.get("_shadow")
        if cached is None or cached[0] != key or not self.training:
            self.refresh_shadow()
            cached = self.__dict__["_shadow"]
        return cached[1], owners


class _LinearView:
    def __init__(self, weight: Tensor, bias: Tensor | None) -> None:
        self.weight = weight
        self.bias = bias


class ExpertView:
    """Expert ``index`` of a stacked bank, duck-typed like ``SwigluExpert``.  The
    weight views are formed on access, so they always reflect the bank's current
    tensors (after ``.to()`` / ``.cuda()`` too) and a list of views costs nothing
    until one is read."""

    def __init__(self, bank: StackedExpertBank, index: int, activation: str) -> None:
        self._bank = bank
        self._index = index
        self.gated = bank.gated
        self.activation = activation
        self._activation_fn = _ACTIVATIONS[activation]

    @property
    def layers(self) -> list[_LinearView]:
        b, i = self._bank, self._index
        return [
            _LinearView(b.w_up[i].t(), b.b_up[i] if b.b_up is not None else None),
            _LinearView(b.w_down[i].t(), b.b_down[i] if b.b_down is not None else None),
        ]

    @property
    def gate(self) -> _LinearView | None:
        b = self._bank
        return _LinearView(b.w_gate[self._index].t(), None) if b.gated else None


class StackedBanksMixin:
    """Declares banks at construction, stacks them on request, and re-installs
    the expert views after device / dtype moves
    (nestor/backbones/expert_bank_stack.py:216-282)."""

    def _declare_expert_banks(self, banks) -> None:
        self._stacked_bank_specs = []
        self._stacked_view_sources = []
        for name, experts in banks:
            setattr(self, name, None)
            if experts:
                self._stacked_bank_specs.append((name, list(experts)))

    def _consolidate_expert_banks(self) -> int:
        done = 0
        for name, experts in getattr(self, "_stacked_bank_specs", []):
            if getattr(self, name, None) is None:
                bank = StackedExpertBank(experts)
                setattr(self, name, bank)
                self._stacked_view_sources.append((bank, experts))
                done += 1
        return done

    def _apply(self, fn, recurse=True):
        module = super()._apply(fn, recurse)
        for bank, experts in getattr(self, "_stacked_view_sources", []):
            bank.install_views(experts)
        return module


def consolidate_stacked_expert_banks(model: nn.Module, *, force: bool = False) -> int:
    """Stack the declared banks of every module in ``model``; returns how many.
    A no-op unless ``NESTOR_STACKED_EXPERT_BANKS=1`` or ``force``."""

    if not (force or stacked_banks_requested()):
        return 0
    return sum(
        m._consolidate_expert_banks() for m in model.modules() if isinstance(m, StackedBanksMixin)
    )
