"""Synthetic workloads of the expert-MLP measurement configs.

Every config routes each token to its top-2 of ``G`` columns, to the top-1 of
``Q`` private experts inside each chosen column, and to the top-1 of ``P`` public
experts: three weighted assignments per token, issued as one public bank call
(``slots = 1``) and one private bank call (``slots = 2``).  Activations are
``N(0, 1)`` rounded to bf16, router heads ``N(0, 0.02)``, expert banks
``N(0, std)`` in the stacked layout ``w_up / w_gate [E, d, h]``,
``w_down [E, h, d]`` with the private bank indexed ``column * Q + expert``.
Draws use a seeded generator on the device the tensors live on; copy them to the
other side to compare implementations on identical bits.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch
from torch import Tensor


@dataclass(frozen=True)
class Workload:
    name: str
    tokens: int
    d_model: int
    hidden: int
    public: int      # P
    columns: int     # G
    private: int     # Q per column
    weight_std: float
    router_std: float = 0.02
    k_columns: int = 2
    k_private: int = 1
    k_public: int = 1
    backward: bool = True
    hidden_public: int = 0   # 0: the public experts are as wide as the private ones

    @property
    def h_public(self) -> int:
        return self.hidden_public or self.hidden

    @property
    def experts(self) -> int:
        return self.public + self.columns * self.private

    @property
    def assignments(self) -> int:
        return self.k_public + self.k_columns * self.k_private

    def gemm_flops(self, backward: bool | None = None) -> float:
        """``2 * rows * K * N`` per GEMM over real rows: forward ``18 T d h`` at three
        assignments per token, backward twice that."""

        per_token = (self.k_public * self.h_public + self.k_columns * self.k_private * self.hidden)
        fwd = 6.0 * self.tokens * self.d_model * per_token
        bwd = self.backward if backward is None else backward
        return fwd * (3.0 if bwd else 1.0)


WORKLOADS = {
    "tiny_100m": Workload("tiny_100m", 4096, 512, 1024, 4, 8, 2, 0.02, backward=False),
    "mlp_200m": Workload("mlp_200m", 16384, 1024, 2048, 8, 16, 4, 0.02),
    "mlp_1b": Workload("mlp_1b", 32768, 2048, 4096, 16, 32, 4, 0.014),
    # The reference's registered arms at their real widths (experiments/pretrain.py:145-150,
    # 174-193; width contract expert_pool_dispatch.py:38-105): 8 columns, top-k columns and
    # private top-k per block, 8 public experts top-2 of width d, 4 x 4096 tokens per
    # micro-batch.  One entry per block shape that differs in kind: the widest private
    # experts with the fewest slots per token, and the narrowest with the most.
    "nestor_1b_block0": Workload("nestor_1b_block0", 16384, 1280, 424, 8, 8, 15, 0.02,
                                 k_columns=3, k_private=2, k_public=2, hidden_public=1280),
    "nestor_1b_block6": Workload("nestor_1b_block6", 16384, 1280, 160, 8, 8, 15, 0.02,
                                 k_columns=8, k_private=2, k_public=2, hidden_public=1280),
    "nestor_200m_block0": Workload("nestor_200m_block0", 16384, 640, 216, 8, 8, 8, 0.02,
                                   k_columns=3, k_private=2, k_public=2, hidden_public=640),
}


@dataclass
class WorkloadTensors:
    x: Tensor            # [T, d] bf16
    grad_out: Tensor     # [T, d] bf16
    w_columns: Tensor    # [G, d]
    w_public: Tensor     # [P, d]
    w_private: Tensor    # [G, Q, d]
    pub: tuple[Tensor, Tensor, Tensor]   # w_up, w_gate, w_down of the public bank
    priv: tuple[Tensor, Tensor, Tensor]  # ... of the flattened private bank


def make_tensors(w: Workload, seed: int, device: torch.device | str,
                 weight_dtype: torch.dtype = torch.bfloat16) -> WorkloadTensors:
    device = torch.device(device)
    g = torch.Generator(device=device).manual_seed(seed)

    def randn(*shape: int, std: float = 1.0, dtype: torch.dtype = torch.float32) -> Tensor:
        # Drawn bank by bank so the fp32 staging buffer stays small at the 1b shape.
        if len(shape) == 3 and shape[0] * shape[1] * shape[2] > (1 << 26):
            out = torch.empty(shape, dtype=dtype, device=device)
            for i in range(shape[0]):
                out[i] = (torch.randn(shape[1:], generator=g, device=device) * std).to(dtype)
            return out
        return (torch.randn(shape, generator=g, device=device) * std).to(dtype)

    def bank(n: int, hidden: int) -> tuple[Tensor, Tensor, Tensor]:
        return (
            randn(n, w.d_model, hidden, std=w.weight_std, dtype=weight_dtype),
            randn(n, w.d_model, hidden, std=w.weight_std, dtype=weight_dtype),
            randn(n, hidden, w.d_model, std=w.weight_std, dtype=weight_dtype),
        )

    x = randn(w.tokens, w.d_model, dtype=torch.bfloat16)
    grad_out = randn(w.tokens, w.d_model, dtype=torch.bfloat16)
    w_columns = randn(w.columns, w.d_model, std=w.router_std)
    w_public = randn(w.public, w.d_model, std=w.router_std)
    w_private = randn(w.columns, w.private, w.d_model, std=w.router_std)
    return WorkloadTensors(x, grad_out, w_columns, w_public, w_private,
                           bank(w.public, w.h_public), bank(w.columns * w.private, w.hidden))


def build_pool(w: Workload, t: WorkloadTensors):
    """(column_router, pool) on the tensors' device, sharing storage with ``t``."""

    from nestor_amd.bank import StackedExpertBank
    from nestor_amd.pool import ExpertPoolMLP
    from nestor_amd.router import Router

    dtype = t.pub[0].dtype
    pool = ExpertPoolMLP.from_stacked(
        w.d_model, w.columns, w.k_columns,
        StackedExpertBank.from_tensors(*t.pub), StackedExpertBank.from_tensors(*t.priv),
        w.k_public, w.k_private, private_gate_mode="switch",
    )
    column_router = Router(w.d_model, w.columns, w.k_columns, [])
    with torch.no_grad():
        def install(router, weight):
            lin = router.score_mlp.layers[0]
            lin.weight = torch.nn.Parameter(weight.to(dtype))
            lin.bias = None
        install(column_router, t.w_columns)
        install(pool.public_router, t.w_public)
        for g, r in enumerate(pool.private_routers):
            install(r, t.w_private[g])
        # a non-degenerate path gate (the zero init is an exact 0.5 / 0.5 split)
        pool.path_gate.weight = torch.nn.Parameter(
            (0.02 * torch.ones_like(pool.path_gate.weight)).to(dtype)
        )
    return column_router.to(t.x.device), pool.to(t.x.device)


def expert_mlp_step(w: Workload, column_router, pool, x: Tensor, grad_out: Tensor | None):
    """One pass of the hot path over one batch: column router -> pool routers ->
    public + private bank calls -> weighted combine (+ backward when ``grad_out``
    is given).  Returns the ``[T, d]`` update."""

    x3 = x.view(1, w.tokens, w.d_model)
    valid = torch.ones(1, w.tokens, dtype=torch.bool, device=x.device)
    col = column_router(x3, valid)
    update, _pub, _priv = pool(x3, valid, col.gates, col.active_mask)
    if grad_out is not None:
        update.backward(grad_out.view_as(update))
    return update


class GraphedStep:
    """``expert_mlp_step`` (forward + backward) captured into one HIP graph and replayed.

    Nothing about the path's launches depends on the routing (static grids, device-side tile
    tables, no host read-backs), so a step is ~150 launches with fixed arguments: at the
    production widths the host spends longer issuing them than the device takes to run them,
    and a replay removes that cost.  ``x`` and ``grad_out`` are copied into buffers the graph
    owns; the update, ``x_grad`` and every parameter's ``.grad`` are graph-owned tensors that
    each replay overwrites (gradients are assigned, not accumulated: they are ``None`` when
    the capture starts).  With fp32 owners behind a bf16 shadow the replays read the copies
    that existed at capture: after every optimizer step call
    ``pool.refresh_shadow(in_place=True)`` before the next replay."""

    def __init__(self, w: Workload, column_router, pool, x: Tensor, grad_out: Tensor,
                 autocast: bool = False, warmup: int = 3) -> None:
        self.params = list(column_router.parameters()) + list(pool.parameters())
        self.x = x.detach().clone().requires_grad_(True)
        self.grad_out = grad_out.detach().clone()
        dev = x.device

        def step():
            with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
                return expert_mlp_step(w, column_router, pool, self.x, self.grad_out)

        def drop_grads():
            for p in self.params:
                p.grad = None
            self.x.grad = None

        import warnings

        main = torch.cuda.current_stream(dev)
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(main)
        with warnings.catch_warnings():
            # the parameters were made on another stream than the capture's: autograd says so
            # once; the replays are checked against eager steps bit for bit in the tests
            warnings.filterwarnings("ignore", message=".*AccumulateGrad node's stream.*")
            with torch.cuda.stream(side):
                for _ in range(warmup):
                    drop_grads()
                    step()
            main.wait_stream(side)
            torch.cuda.synchronize(dev)
            drop_grads()
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph):
                self.update = step()
        self.x_grad = self.x.grad

    def __call__(self, x: Tensor | None = None, grad_out: Tensor | None = None) -> Tensor:
        if x is not None:
            self.x.detach().copy_(x)
        if grad_out is not None:
            self.grad_out.copy_(grad_out)
        self.graph.replay()
        return self.update

