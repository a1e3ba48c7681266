"""Router epilogue kernel and slot construction vs the oracle: indices and ids
bit-exact, probabilities / gates to fp32 or one-bf16-ulp accuracy."""

import pytest
import torch

from oracle import router as orouter
from tests.helpers import gen

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,choices,k,mode", [
    (1000, 8, 2, "renorm"), (1000, 4, 1, "renorm"), (4096, 16, 1, "switch"), (777, 15, 2, "switch"),
    (513, 32, 2, "renorm"), (100, 64, 8, "renorm"), (64, 1, 1, "renorm"), (300, 12, 3, "switch"),
])
def test_router_topk_kernel(cuda, dtype, n, choices, k, mode):
    from nestor_amd import ops

    g = gen(n + choices)
    scores = torch.randn(n, choices, generator=g).to(dtype)  # bf16 scores tie often
    bias = torch.randn(choices, generator=g) * 0.1
    mask = torch.rand(n, generator=g) > 0.1
    want = orouter.route(scores, bias, k, mode, mask, softmax_dtype=torch.float32)
    probs, topk, gates = ops.router_topk(scores.to(cuda), bias.to(cuda).view(1, -1), mask.to(cuda), k,
                                         1 if mode == "switch" else 0)
    assert torch.equal(topk.cpu(), want.topk_indices)  # ties: lowest index first on both sides
    torch.testing.assert_close(probs.cpu(), want.softmax_probs, rtol=1e-5, atol=1e-7)
    assert gates.dtype == dtype
    if dtype == torch.float32:
        torch.testing.assert_close(gates.cpu(), want.gates, rtol=1e-5, atol=1e-7)
    else:
        torch.testing.assert_close(gates.cpu().float(), want.gates.float(), rtol=2 ** -7, atol=1e-6)
    assert torch.equal(gates.cpu() > 0, want.active_mask) or dtype == torch.bfloat16
    assert (gates.cpu()[~mask] == 0).all()
    if k == 1 and mode == "renorm":
        # closed form: a renormalised top-1 gate is exactly 1 on valid tokens
        assert torch.equal(gates.cpu().float().sum(-1), mask.float())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("use_probs", [False, True])
@pytest.mark.parametrize("n,choices,k,mode", [
    (500, 8, 2, "renorm"), (500, 4, 1, "renorm"), (700, 16, 1, "switch"), (333, 15, 2, "switch"),
    (257, 32, 2, "renorm"), (100, 64, 8, "switch"),
])
def test_router_score_gradient(cuda, dtype, use_probs, n, choices, k, mode):
    """The op's score gradient (one launch) against autograd through the oracle's
    softmax / gather / scatter chain in fp64 on the same selections."""

    from nestor_amd import ops
    from tests.helpers import rel_l2

    g = gen(3 * n + choices)
    scores = torch.randn(n, choices, generator=g).to(dtype)
    bias = torch.randn(choices, generator=g) * 0.1
    mask = torch.rand(n, generator=g) > 0.2
    d_gates = torch.randn(n, choices, generator=g).to(dtype)
    d_probs = torch.randn(n, choices, generator=g)
    ts = scores.to(cuda).requires_grad_(True)
    probs, topk, gates = ops.router_topk(ts, bias.to(cuda).view(1, -1), mask.to(cuda), k,
                                         1 if mode == "switch" else 0)
    loss = (gates.float() * d_gates.to(cuda).float()).sum()
    if use_probs:
        loss = loss + (probs * d_probs.to(cuda)).sum()
    loss.backward()
    # fp64 chain on the kernel's own selections (ties are the only way they could differ)
    sd = scores.double().requires_grad_(True)
    sel = topk.cpu()
    if mode == "switch":
        tg = torch.softmax(sd, -1).gather(-1, sel)
    else:
        tg = torch.softmax(sd.gather(-1, sel), -1)
    dense = torch.zeros_like(sd).scatter_add(-1, sel, tg) * mask.unsqueeze(-1).double()
    ref = (dense * d_gates.double()).sum()
    if use_probs:
        ref = ref + (torch.softmax(sd, -1) * d_probs.double()).sum()
    ref.backward()
    assert ts.grad.dtype == dtype
    tol = 1e-5 if dtype == torch.float32 else 4e-3
    assert rel_l2(ts.grad, sd.grad) < tol
    if not use_probs:
        assert (ts.grad.cpu()[~mask] == 0).all()
        if k == 1 and mode == "renorm":
            assert (ts.grad == 0).all()  # a renormalised top-1 gate is the constant 1


def test_batched_private_routers_and_slots(cuda):
    """[T, G, Q] scores through one launch == G separate routers; slot ids are
    ``column * Q + expert`` and weights ``private_gate * column_gate``."""

    from nestor_amd import ops

    tokens, groups, q, k_a = 2000, 8, 4, 2
    g = gen(11)
    scores = torch.randn(tokens, groups, q, generator=g).bfloat16()
    bias = torch.randn(groups, q, generator=g) * 0.05
    col_scores = torch.randn(tokens, groups, generator=g).bfloat16()
    valid = torch.rand(tokens, generator=g) > 0.05
    col = orouter.route(col_scores, torch.zeros(groups), k_a, "renorm", valid)
    want = orouter.route_private_batched(
        scores.view(1, tokens, groups, q), bias, 1, "switch", valid.view(1, tokens),
        col.active_mask.view(1, tokens, groups), softmax_dtype=torch.float32,
    )
    member = (valid.unsqueeze(-1) & col.active_mask).reshape(-1)
    probs, topk, gates = ops.router_topk(
        scores.view(-1, q).to(cuda), bias.to(cuda), member.to(cuda), 1, 1)
    assert torch.equal(topk.cpu().view(1, tokens, groups, 1), want.topk_indices)
    torch.testing.assert_close(gates.cpu().float().view(1, tokens, groups, q),
                               want.gates.float(), rtol=2 ** -7, atol=1e-6)
    # per-router loop pins the batched oracle itself
    for gi in range(groups):
        one = orouter.route(scores[:, gi], bias[gi], 1, "switch", valid & col.active_mask[:, gi])
        assert torch.equal(one.topk_indices, want.topk_indices[0, :, gi])
        assert torch.equal(one.gates, want.gates[0, :, gi])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("tokens,groups,q,k_a,k_q,given", [
    (1000, 8, 4, 2, 1, False), (1000, 8, 4, 2, 1, True), (333, 32, 4, 2, 2, False),
    (64, 3, 5, 3, 3, False), (500, 64, 2, 4, 1, False), (1, 1, 1, 1, 1, False),
])
def test_private_slots_op(cuda, dtype, tokens, groups, q, k_a, k_q, given):
    """Slot ids / weights / selected columns in one launch: integer outputs and the
    rounded weights equal the oracle's gather chain bit for bit; both gate gradients
    equal autograd through that chain (single rounded products)."""

    from nestor_amd import ops

    g = gen(tokens + groups)
    col_scores = torch.randn(tokens, groups, generator=g).to(dtype)  # bf16: equal gates occur
    valid = torch.rand(tokens, generator=g) > 0.1
    col = orouter.route(col_scores, torch.zeros(groups), k_a, "renorm", valid)
    scores = torch.randn(tokens, groups, q, generator=g).to(dtype)
    priv = orouter.route(scores, torch.zeros(groups, q), k_q, "switch",
                         valid.unsqueeze(-1) & col.active_mask)
    picked = col.topk_indices if given else None
    cg = col.gates.detach().clone().requires_grad_(True)
    pg = priv.gates.detach().clone().requires_grad_(True)
    w_ids, w_weights, w_sel = orouter.private_slots(pg, priv.topk_indices, cg, k_a, picked)
    d_w = torch.randn(tokens, k_a * k_q, generator=g).to(dtype)
    w_weights.backward(d_w)
    tcg = col.gates.to(cuda).requires_grad_(True)
    tpg = priv.gates.to(cuda).requires_grad_(True)
    sel, ids, weights = ops.private_slots_op(
        tcg, tpg, priv.topk_indices.to(cuda), None if picked is None else picked.to(cuda), k_a)
    assert torch.equal(sel.cpu(), w_sel)
    assert torch.equal(ids.cpu(), w_ids)
    assert torch.equal(weights.cpu(), w_weights.detach())
    weights.backward(d_w.to(cuda))
    if k_q == 1 or dtype == torch.float32:
        torch.testing.assert_close(tcg.grad.cpu(), cg.grad, rtol=1e-6, atol=1e-7)
    else:  # a k_q-term sum: fp32 here, bf16 partial sums in the eager chain
        torch.testing.assert_close(tcg.grad.cpu().float(), cg.grad.float(), rtol=2 ** -6, atol=2e-2)
    assert torch.equal(tpg.grad.cpu(), pg.grad)


@pytest.mark.parametrize("tokens,dim,heads,bias", [
    (300, 64, 10, True), (1000, 512, 146, False), (129, 1024, 32, True), (4096, 2048, 160, False),
])
def test_score_linear_matches_linear(cuda, tokens, dim, heads, bias):
    """Skinny score heads: values are the library GEMM's; the input gradient comes
    from the grouped GEMM kernel (whole batch as one bank, head count zero-padded
    to a multiple of 32) and is held to the fp32 product of the same bf16 operands."""

    from nestor_amd.router import score_linear
    from tests.helpers import rel_l2

    x = torch.randn(tokens, dim, generator=gen(1)).bfloat16()
    w = (torch.randn(heads, dim, generator=gen(2)) / dim ** 0.5).bfloat16()
    b = torch.randn(heads, generator=gen(3)).bfloat16() if bias else None
    g = torch.randn(tokens, heads, generator=gen(4)).bfloat16()
    tx = x.to(cuda).requires_grad_(True)
    tw = w.to(cuda).requires_grad_(True)
    tb = b.to(cuda).requires_grad_(True) if bias else None
    out = score_linear(tx, tw, tb)
    ref = torch.nn.functional.linear(x.float(), w.float(), None if b is None else b.float())
    assert out.shape == ref.shape and out.dtype == torch.bfloat16
    torch.testing.assert_close(out.cpu().float(), ref, rtol=2 ** -6, atol=2e-2)
    out.backward(g.to(cuda))
    assert rel_l2(tx.grad, g.float() @ w.float()) < 4e-3
    assert rel_l2(tw.grad, g.float().t() @ x.float()) < 4e-3
    if bias:
        assert rel_l2(tb.grad, g.float().sum(0)) < 4e-3
    # without a gradient on the rows the library path runs and gives the same values
    plain = score_linear(x.to(cuda), tw, tb)
    assert torch.equal(plain, out)


@pytest.mark.parametrize("n,choices,k", [(5000, 16, 2), (100, 64, 8), (1, 3, 1), (70000, 32, 2)])
def test_balancing_counts_and_bias_update(cuda, n, choices, k):
    """Histogram of the selections of valid tokens (integer-exact) and the bias step."""

    from nestor_amd import ops
    from nestor_amd.router import Router

    g = gen(n)
    topk = torch.stack([torch.randperm(choices, generator=g)[:k] for _ in range(min(n, 512))])
    topk = topk.repeat((n + 511) // 512, 1)[:n].view(1, n, k)
    valid = (torch.rand(1, n, generator=g) > 0.25)
    counts = ops.router_choice_counts(topk.to(cuda), valid.to(cuda), choices)
    want = torch.bincount(topk[valid].reshape(-1), minlength=choices)
    assert torch.equal(counts.cpu().long(), want)
    router = Router(8, choices, k, [], loss_free_balancing=True, bias_update_rate=0.01).to(cuda)
    router.choice_bias.copy_(torch.randn(choices, generator=g))
    before = router.choice_bias.cpu().clone()
    router.update_detached_parameters(topk.to(cuda), valid.to(cuda))
    assert torch.equal(router.choice_bias.cpu(), orouter.balancing_update(before, topk, valid, 0.01))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mode,k", [("renorm", 2), ("switch", 1)])
def test_router_exploration_noise(cuda, dtype, mode, k):
    """Training-mode routers with a noise head (nestor/backbones/nestor.py:540-556): the
    scores are ``score + eps * softplus(noise head)`` for the draw handed in, the
    selection is the oracle's on those scores, evaluation mode and a router without a
    noise head ignore the draw, the noise head receives a gradient, and an own draw
    follows the RNG seed."""

    import nestor_amd as na

    torch.manual_seed(0)
    router = na.Router(48, 8, k, [], noise_mlp_hidden_dims=[], gate_mode=mode).to(cuda).to(dtype)
    with torch.no_grad():
        router.choice_bias.normal_(std=0.1)
        router.noise_mlp.layers[0].weight.normal_(std=0.3)
    g = torch.Generator(device=cuda).manual_seed(4)
    x = torch.randn(3, 50, 48, generator=g, device=cuda, dtype=dtype)
    valid = torch.rand(3, 50, generator=g, device=cuda) > 0.1
    eps = router.draw_noise(3, 50, cuda, dtype)
    router.train()
    out = router(x, valid, noise=eps)
    plain = router.score_mlp(x)
    head = router.noise_mlp(x)
    want_scores = orouter.explore(plain.cpu().double(), eps.cpu().double(), head.cpu().double())
    if dtype == torch.bfloat16:   # softplus, product and sum each round to 8 bits
        torch.testing.assert_close(out.scores.cpu().double(), want_scores, rtol=2 ** -6, atol=4e-2)
    else:
        torch.testing.assert_close(out.scores.cpu().double(), want_scores, rtol=1e-5, atol=1e-5)
    assert not torch.equal(out.scores, plain)
    want = orouter.route(out.scores.cpu(), router.choice_bias.cpu(), k, mode, valid.cpu(),
                         softmax_dtype=torch.float32)
    assert torch.equal(out.topk_indices.cpu(), want.topk_indices)
    assert torch.equal(out.active_mask.cpu(), want.active_mask) or dtype == torch.bfloat16
    # the noise head learns: its weight gets a gradient through the perturbed scores
    (out.softmax_probs.float() * torch.arange(8, device=cuda)).sum().backward()
    assert router.noise_mlp.layers[0].weight.grad.abs().sum() > 0
    # an own draw follows the seed
    torch.manual_seed(7)
    a = router(x, valid).scores
    torch.manual_seed(7)
    b = router(x, valid).scores
    assert torch.equal(a, b) and not torch.equal(a, out.scores)
    # evaluation mode, and a router without a noise head, are deterministic
    router.eval()
    assert torch.equal(router(x, valid, noise=eps).scores, plain)
    bare = na.Router(48, 8, k, [], gate_mode=mode).to(cuda).to(dtype).train()
    assert torch.equal(bare(x, valid, noise=eps).scores, bare.score_mlp(x))


def test_batched_noisy_routers_equal_one_router_at_a_time(cuda, monkeypatch):
    """``route_private_batched`` in training mode: one draw ``[B, S, G, Q]`` gives every
    router the result it gets alone on its slab, and with the anneal schedule on each
    counter advances once per forward but not inside a backward recompute
    (nestor/backbones/batched_router.py:188-208, nestor.py:548-555)."""

    import nestor_amd as na

    monkeypatch.setenv("NESTOR_ROUTER_NOISE_ANNEAL_STEPS", "4")
    torch.manual_seed(1)
    routers = [na.Router(32, 4, 1, [], noise_mlp_hidden_dims=[], gate_mode="switch").to(cuda)
               for _ in range(3)]
    for r in routers:
        with torch.no_grad():
            r.noise_mlp.layers[0].weight.normal_(std=0.5)
        r.train()
        assert int(r._noise_steps) == 0
    g = torch.Generator(device=cuda).manual_seed(2)
    x = torch.randn(2, 40, 32, generator=g, device=cuda)
    valid = torch.ones(2, 40, dtype=torch.bool, device=cuda)
    member = torch.rand(2, 40, 3, generator=g, device=cuda) > 0.3
    eps = torch.randn(2, 40, 3, 4, generator=g, device=cuda)
    outs, gates, topk = na.route_private_batched(routers, x, valid, member, training=True, noise=eps)
    assert [int(r._noise_steps) for r in routers] == [1, 1, 1]
    for r in routers:
        r._noise_steps.zero_()
    for gi, r in enumerate(routers):
        alone = r(x, valid & member[:, :, gi], noise=eps[:, :, gi])
        torch.testing.assert_close(outs[gi].scores, alone.scores, rtol=1e-5, atol=1e-6)
        assert torch.equal(outs[gi].topk_indices, alone.topk_indices)
    # step 1 of 4: three quarters of the perturbation; step 4 and later: none
    full = orouter.explore(routers[0].score_mlp(x).detach().cpu().double(), eps[:, :, 0].cpu().double(),
                           routers[0].noise_mlp(x).detach().cpu().double())
    base = routers[0].score_mlp(x).detach().cpu().double()
    step1 = routers[0](x, valid, noise=eps[:, :, 0]).scores.detach().cpu().double()
    torch.testing.assert_close(step1 - base, 0.75 * (full - base), rtol=1e-4, atol=1e-5)
    routers[0]._noise_steps.fill_(9)
    assert torch.equal(routers[0](x, valid, noise=eps[:, :, 0]).scores, routers[0].score_mlp(x))
    # a checkpoint's recompute does not advance the schedule
    from torch.utils.checkpoint import checkpoint

    routers[1]._noise_steps.zero_()
    xi = x.clone().requires_grad_(True)
    out = checkpoint(lambda a: routers[1](a, valid, noise=eps[:, :, 1]).softmax_probs, xi, use_reentrant=False)
    out.sum().backward()
    assert int(routers[1]._noise_steps) == 1
