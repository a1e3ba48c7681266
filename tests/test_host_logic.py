"""Host-side pieces that need no GPU: stacked layout, width contract, flags,
and loud failure of the product path off-GPU."""

import os

import pytest
import torch

import nestor_amd as na
from nestor_amd import flags
from nestor_amd.pool import private_expert_hidden_dim, public_expert_hidden_dim


def test_width_contract_table():
    """The reference's documented widths (tests/test_expert_pools.py:186-215)."""

    assert public_expert_hidden_dim(640, 1) == 1280
    assert private_expert_hidden_dim(640, 3, 1) == 424
    assert public_expert_hidden_dim(960, 1) == 1920
    assert private_expert_hidden_dim(960, 3, 1) == 640
    assert public_expert_hidden_dim(1280, 1) == 2560
    assert private_expert_hidden_dim(1280, 3, 1) == 856
    assert public_expert_hidden_dim(640, 2) == 640
    assert private_expert_hidden_dim(640, 3, 2) == 216
    assert public_expert_hidden_dim(640, 2, active_budget=1.25) == 400
    assert private_expert_hidden_dim(640, 8, 1, active_budget=1.25) == 96
    assert private_expert_hidden_dim(640, 3, 1, with_public_pool=False) == 856
    # the measurement configs: active_budget 4 makes private == public == 2d
    assert private_expert_hidden_dim(2048, 2, 1, active_budget=4.0) == 4096
    assert public_expert_hidden_dim(2048, 1) == 4096


def test_stacked_bank_layout_and_views():
    """w_up[i].t() is expert i's up weight; per-expert params leave the module
    tree; state-dict keys are the stacked ones
    (tests/test_stacked_expert_banks.py:87-101,198-200 in the reference)."""

    torch.manual_seed(0)
    experts = [na.SwigluExpert(12, 20, 12) for _ in range(3)]
    before = [(e.layers[0].weight.detach().clone(), e.gate.weight.detach().clone(),
               e.layers[1].weight.detach().clone()) for e in experts]
    bank = na.StackedExpertBank(experts)
    assert bank.w_up.shape == (3, 12, 20) and bank.w_gate.shape == (3, 12, 20)
    assert bank.w_down.shape == (3, 20, 12) and bank.w_up.is_contiguous()
    for i, (up, gate, down) in enumerate(before):
        assert torch.equal(bank.w_up[i].t(), up) and torch.equal(bank.w_gate[i].t(), gate)
        assert torch.equal(bank.w_down[i].t(), down)
        assert experts[i].layers[0].weight.data_ptr() == bank.w_up[i].data_ptr()
    assert all(len(list(e.parameters())) == 0 for e in experts)
    x = torch.randn(5, 12)
    ref = torch.nn.functional.silu(x @ before[1][1].t()) * (x @ before[1][0].t()) @ before[1][2].t()
    torch.testing.assert_close(experts[1](x), ref)
    experts[1](x).sum().backward()
    assert bank.w_up.grad is not None and (bank.w_up.grad[0] == 0).all() and bank.w_up.grad[1].abs().sum() > 0

    pool = na.ExpertPoolMLP(16, 2, 1, 2, 1, 2, 1, [])
    assert na.consolidate_stacked_expert_banks(pool) == 0  # flag unset
    assert na.consolidate_stacked_expert_banks(pool, force=True) == 2
    keys = pool.state_dict().keys()
    for k in ("stacked_public.w_up", "stacked_public.w_gate", "stacked_public.w_down",
              "stacked_private.w_up", "stacked_private.w_down"):
        assert k in keys
    assert not any("public_experts" in k or "private_experts" in k for k in keys)
    assert pool.stacked_private.w_up.shape == (4, 16, private_expert_hidden_dim(16, 1, 1))
    moved = pool.to(torch.float64)
    first = moved._private_bank()[0]
    assert first.layers[0].weight.dtype == torch.float64
    assert first.layers[0].weight.data_ptr() == moved.stacked_private.w_up.data_ptr()


def test_non_uniform_bank_is_rejected():
    a, b = na.SwigluExpert(8, 8, 8), na.SwigluExpert(8, 8, 8, bias=True)
    with pytest.raises(ValueError):
        na.StackedExpertBank([a, b])
    with pytest.raises(ValueError):
        na.ExpertPoolMLP(16, 2, 3, 2, 1, 2, 1, [])
    with pytest.raises(ValueError):
        na.ExpertPoolMLP(16, 2, 1, 2, 1, 0, 1, [])


def test_flag_readers_follow_env():
    saved = {k: os.environ.get(k) for k in (
        "NESTOR_TRITON_INDEX_BUILD", "NESTOR_TRITON_EXPERT_DISPATCH", "NESTOR_STACKED_EXPERT_BANKS",
        "NESTOR_GROUPED_MM_FUSED_GATE", "NESTOR_TRITON_EXPERT_CATCAST", "NESTOR_BATCHED_ROUTERS")}
    try:
        for k in saved:
            os.environ.pop(k, None)
        assert not flags.triton_index_requested() and not flags.triton_expert_requested()
        assert not flags.stacked_banks_requested() and not flags.fused_gate_requested()
        assert flags.triton_cat_cast_requested() and not flags.batched_routers_enabled()
        os.environ["NESTOR_TRITON_INDEX_BUILD"] = "1"
        assert flags.triton_index_requested() and flags.triton_expert_requested()  # default follows
        os.environ["NESTOR_TRITON_EXPERT_DISPATCH"] = "0"
        assert not flags.triton_expert_requested()
        os.environ["NESTOR_STACKED_EXPERT_BANKS"] = "1"
        assert flags.stacked_banks_requested()
    finally:
        for k, v in saved.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v


def test_product_path_refuses_cpu_tensors():
    """No CPU fallback: calling the path with CPU tensors raises instead of
    silently computing somewhere else."""

    bank = na.StackedExpertBank.from_tensors(
        torch.randn(2, 8, 16).bfloat16(), torch.randn(2, 8, 16).bfloat16(), torch.randn(2, 16, 8).bfloat16())
    x = torch.randn(4, 8).bfloat16()
    ids = torch.zeros(4, 1, dtype=torch.long)
    w = torch.ones(4, 1)
    with pytest.raises((NotImplementedError, RuntimeError)):
        na.grouped_expert_combine(x, bank.expert_views(), ids, w, 1, stacked=bank, triton_fused=True)
    with pytest.raises(NotImplementedError):
        na.grouped_expert_combine(x.float(), bank.expert_views(), ids, w, 1, stacked=bank)  # fp32 GEMM dtype


def test_workload_flop_convention():
    from nestor_amd.workloads import WORKLOADS

    w = WORKLOADS["mlp_1b"]
    assert w.experts == 144 and w.assignments == 3
    assert w.gemm_flops(False) == pytest.approx(4.948e12, rel=1e-3)
    assert w.gemm_flops(True) == pytest.approx(1.4843e13, rel=1e-3)
    assert WORKLOADS["tiny_100m"].gemm_flops() == pytest.approx(3.866e10, rel=1e-3)
    assert WORKLOADS["mlp_200m"].gemm_flops(True) == pytest.approx(1.855e12, rel=1e-3)


def test_flop_counter_sees_the_expert_gemms():
    """``FlopCounterMode`` counts the custom GEMM ops as the reference counts
    ``aten._grouped_mm``: ``2 * rows * K * N`` over the rows as passed
    (nestor/train/flop_formulas.py:59-64).  Shape-only tensors: no GPU needed.  One bank
    call forward (2 launches) plus the five GEMMs of its backward = ``18 * rows_pad * d * h``,
    each op counted once."""

    from torch._subclasses.fake_tensor import FakeTensorMode
    from torch.utils.flop_counter import FlopCounterMode

    from nestor_amd import ops

    tokens, d, h, banks, slots = 1000, 256, 512, 8, 2
    rows_pad = ops.rows_pad_for(tokens * slots, banks)
    with FakeTensorMode():
        def mk(*shape):
            return torch.empty(*shape, dtype=torch.bfloat16, device="cuda")

        x_pad, w_up, w_gate, w_down = mk(rows_pad, d), mk(banks, d, h), mk(banks, d, h), mk(banks, h, d)
        table = torch.empty(ops.tile_table_ints(rows_pad, banks), dtype=torch.int32, device="cuda")
        offs = torch.empty(banks, dtype=torch.int32, device="cuda")
        with FlopCounterMode(display=False) as counter:
            up_gate, hidden = ops.upgate_swiglu_op(x_pad, w_up, w_gate, table, offs, None, None)
            y = ops.grouped_mm_op(hidden, w_down, table, offs, None, None)
            forward = counter.get_total_flops()
            ops.grouped_gemm_nt(y, w_down, table)
            ops.grouped_gemm_tn(hidden, y, offs, None, None)
            ops.grouped_gemm_nt_upgate(up_gate, w_up, w_gate, table)
            ops.grouped_gemm_tn(x_pad, up_gate[:, :h], offs, None, None)
            ops.grouped_gemm_tn(x_pad, up_gate[:, h:], offs, None, None)
        assert forward == 6 * rows_pad * d * h
        assert counter.get_total_flops() == 18 * rows_pad * d * h
        with FlopCounterMode(display=False) as counter:
            ops.score_heads_op(mk(tokens, d), mk(32, d), None)
        assert counter.get_total_flops() == 2 * tokens * d * 32


def test_router_noise_heads_are_built_and_batchable():
    """Routers take the reference's noise head (nestor/backbones/nestor.py:459-466); a pool
    hands ``router_noise_mlp_hidden_dims`` to every router, and batching needs same-shaped
    noise heads as it needs same-shaped score heads (batched_router.py:71-94)."""

    router = na.Router(16, 4, 1, [], noise_mlp_hidden_dims=[8])
    assert [tuple(l.weight.shape) for l in router.noise_mlp.layers] == [(8, 16), (4, 8)]
    assert na.Router(16, 4, 1, []).noise_mlp is None
    assert tuple(router.draw_noise(2, 3, "cpu", torch.float32).shape) == (2, 3, 4)
    pool = na.ExpertPoolMLP(16, 2, 1, 2, 1, 2, 1, [], router_noise_mlp_hidden_dims=[])
    assert pool.public_router.noise_mlp is not None
    assert all(r.noise_mlp is not None for r in pool.private_routers)
    drawn = pool.draw_router_noise(2, 3, "cpu", torch.float32)
    assert tuple(drawn["private"].shape) == (2, 3, 2, 2) and tuple(drawn["public"].shape) == (2, 3, 2)
    from nestor_amd.router import check_batchable

    with pytest.raises(ValueError):
        check_batchable([na.Router(16, 4, 1, [], noise_mlp_hidden_dims=[8]), na.Router(16, 4, 1, [])])
    # the anneal counter is a buffer only when the schedule is on
    assert not hasattr(router, "_noise_steps")


def test_oracle_exploration_formula():
    """``oracle.router.explore`` against the textbook pieces: softplus by its definition in
    fp64, the anneal factor at its corners, and linearity in the draw."""

    from oracle import router as orouter

    g = torch.Generator().manual_seed(3)
    scores, eps, head = (torch.randn(5, 7, generator=g, dtype=torch.float64) for _ in range(3))
    head[0, 0], head[0, 1] = 40.0, -40.0
    want = scores + eps * torch.log(1 + torch.exp(head))
    assert torch.allclose(orouter.explore(scores, eps, head), want, rtol=1e-12, atol=1e-12)
    assert torch.equal(orouter.explore(scores, torch.zeros_like(eps), head), scores)
    assert torch.equal(orouter.explore(scores, eps, head, 10, 10), scores)          # fully annealed
    assert torch.equal(orouter.explore(scores, eps, head, 25, 10), scores)          # clamped
    half = orouter.explore(scores, eps, head, 5, 10)
    assert torch.allclose(half - scores, 0.5 * (want - scores), rtol=1e-12, atol=1e-12)
    assert torch.allclose(orouter.explore(scores, 2 * eps, head) - scores, 2 * (want - scores))


def test_bf16_shadow_follows_data_writes():
    """The persistent bf16 copy of fp32 owners must not go stale when an owner is written
    through ``.data`` -- how the reference swaps EMA weights in and out around evaluation
    (nestor/train/trainer.py:974-999) and restores Muon masters on resume
    (nestor/scaling/muon.py:582) -- which leaves the tensor's version counter alone."""

    from nestor_amd.bank import StackedExpertBank

    g = torch.Generator().manual_seed(0)
    w3 = [torch.randn(3, a, b, generator=g) for a, b in ((8, 16), (8, 16), (16, 8))]
    bank = StackedExpertBank.from_tensors(*[t.clone() for t in w3]).enable_bf16_shadow()

    def copies():
        return bank.shadowed(torch.bfloat16)[0]

    first = copies()
    assert all(torch.equal(c, w.bfloat16()) for c, w in zip(first, w3))
    assert copies()[0] is first[0]                       # training mode, untouched owners: cached
    with torch.no_grad():
        bank.w_up.mul_(2.0)                              # optimizer-style update: version bump
    assert torch.equal(copies()[0], (w3[0] * 2).bfloat16())
    # the EMA swap: eval, .data write, eval again with no mode change, .data write back, train
    version = bank.w_down._version
    bank.eval()
    live = copies()[2].clone()
    bank.w_down.data.copy_(w3[2] * 3)
    assert bank.w_down._version == version               # invisible to the version counter ...
    assert torch.equal(copies()[2], (w3[2] * 3).bfloat16())   # ... and still picked up
    bank.w_down.data.copy_(w3[2])
    bank.train()
    assert torch.equal(copies()[2], live)
    # a .data write in training mode is the documented case for refresh_shadow()
    bank.w_gate.data.copy_(w3[1] * 5)
    bank.refresh_shadow()
    assert torch.equal(copies()[1], (w3[1] * 5).bfloat16())
    # in place: the copies keep their storage (what a captured graph of the step reads)
    before = [c.data_ptr() for c in copies()]
    with torch.no_grad():
        bank.w_up.add_(1.0)
    bank.refresh_shadow(in_place=True)
    after = copies()
    assert [c.data_ptr() for c in after] == before
    assert torch.equal(after[0], bank.w_up.detach().bfloat16())
    # loading a state dict drops the copy
    state = {k: v.clone() * 0.5 for k, v in bank.state_dict().items()}
    bank.load_state_dict(state)
    assert torch.equal(copies()[0], state["w_up"].bfloat16())
