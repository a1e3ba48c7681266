"""ExpertPoolMLP on the HIP path: the three output layouts agree with each other
and with the per-token definition of the pool equation."""

import pytest
import torch

from tests.helpers import gen, rel_l2

pytestmark = pytest.mark.gpu


def _pool(cuda, stacked: bool):
    import nestor_amd as na

    torch.manual_seed(9)
    pool = na.ExpertPoolMLP(
        dim=40, num_groups=4, num_groups_per_token=2, num_public_experts=4, public_top_k=2,
        num_private_experts=3, private_top_k=2, router_score_mlp_hidden_dims=[],
        private_gate_mode="switch",
    )
    with torch.no_grad():
        pool.path_gate.weight.normal_()
        for r in [pool.public_router, *pool.private_routers]:
            r.choice_bias.normal_(std=0.1)
    if stacked:
        assert na.consolidate_stacked_expert_banks(pool, force=True) == 2
    pool.triton_fused = pool.triton_index = pool.fused_gate = True
    return pool.to(cuda).eval()


def _inputs(cuda):
    g = gen(21)
    x = torch.randn(3, 70, 40, generator=g)
    valid = torch.ones(3, 70, dtype=torch.bool)
    valid[1, -5:] = False
    scores = torch.rand(3, 70, 4, generator=g)
    slot_groups = scores.topk(2, dim=-1).indices
    active = torch.zeros(3, 70, 4, dtype=torch.bool).scatter(-1, slot_groups, True) & valid.unsqueeze(-1)
    gates = torch.zeros(3, 70, 4).scatter(-1, slot_groups, 0.5) * valid.unsqueeze(-1)
    return tuple(t.to(cuda) for t in (x, valid, gates, active, slot_groups))


def _per_token_reference(pool, x, valid, gates, active):
    """The pool equation token by token in fp32, on the routing the pool chose
    (the slow-loop form of the reference's tests/test_expert_pools.py:126-180)."""

    out = torch.zeros_like(x)
    B, S, _ = x.shape

    def routed(router, experts, h, ok):
        if not ok:
            return torch.zeros_like(h)
        r = router(h.view(1, 1, -1), torch.ones(1, 1, dtype=torch.bool, device=h.device))
        acc = torch.zeros_like(h)
        for e in r.topk_indices.view(-1).tolist():
            acc = acc + r.gates.view(-1)[e] * experts[e](h)
        return acc

    for b in range(B):
        for s in range(S):
            h = x[b, s]
            alpha = torch.softmax(pool.path_gate(h).float(), -1)
            pub = routed(pool.public_router, pool.public_experts, h, bool(valid[b, s]))
            priv = torch.zeros_like(h)
            for g in range(pool.num_groups):
                if active[b, s, g] and valid[b, s]:
                    priv = priv + gates[b, s, g] * routed(pool.private_routers[g], pool.private_experts[g], h, True)
            out[b, s] = alpha[0] * pub + alpha[1] * priv
    return out


@pytest.mark.parametrize("stacked", [True, False])
def test_pool_layouts_and_definition(cuda, stacked):
    pool = _pool(cuda, stacked)
    x, valid, gates, active, slot_groups = _inputs(cuda)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        summed, pub_out, priv_outs = pool(x, valid, gates, active)
        p_slot, v_slot, _, _ = pool.forward_per_slot(x, valid, gates, active, slot_groups)
        p_grp, v_grp, _, _ = pool.forward_per_group(x, valid, gates, active)
    assert summed.dtype == torch.float32 and v_slot.shape == (3, 70, 2, 40) and v_grp.shape == (3, 70, 4, 40)
    assert len(priv_outs) == 4 and torch.equal(pub_out.valid_token_mask, valid)
    for gi, po in enumerate(priv_outs):
        assert torch.equal(po.valid_token_mask, valid & active[:, :, gi])
    # layouts: public + private summed over slots / groups == the summed forward
    torch.testing.assert_close(p_slot + v_slot.sum(2), summed, rtol=2 ** -6, atol=1e-2)
    torch.testing.assert_close(p_grp + v_grp.sum(2), summed, rtol=2 ** -6, atol=1e-2)
    idx = slot_groups.unsqueeze(-1).expand(-1, -1, -1, 40)
    torch.testing.assert_close(v_grp.gather(2, idx), v_slot, rtol=2 ** -6, atol=1e-2)
    # definition: per-token loop in fp32 with torch ops only
    with torch.no_grad():
        ref = _per_token_reference(pool, x, valid, gates, active)
    assert rel_l2(summed, ref) < 1e-2
    assert (summed[~valid] == 0).all()


def test_pool_grads_reach_every_parameter(cuda):
    """Every parameter ends a step with a finite gradient, including banks no
    token selected (the reference's DDP-safety property,
    tests/test_expert_pools.py:428-436)."""

    pool = _pool(cuda, True).train()
    x, valid, gates, active, slot_groups = _inputs(cuda)
    x = x.requires_grad_(True)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        pub, priv, _, _ = pool.forward_per_slot(x, valid, gates, active, slot_groups)
    (pub.float().sum() + priv.float().square().sum()).backward()
    names = [n for n, _ in pool.named_parameters()]
    assert "stacked_public.w_up" in names and "stacked_private.w_down" in names
    for n, p in pool.named_parameters():
        assert p.grad is not None and torch.isfinite(p.grad).all(), n
    assert x.grad is not None and torch.isfinite(x.grad).all()


def test_pool_on_an_empty_sequence_slice(cuda):
    """Zero tokens (the reference calls the pool on sequence slices): empty outputs of
    the right shapes from all three layouts, and a backward pass that reaches the banks."""

    pool = _pool(cuda, True).train()
    x = torch.zeros(2, 0, 40, device=cuda, dtype=torch.bfloat16, requires_grad=True)
    valid = torch.ones(2, 0, dtype=torch.bool, device=cuda)
    gates = torch.zeros(2, 0, 4, device=cuda, dtype=torch.bfloat16)
    active = torch.zeros(2, 0, 4, dtype=torch.bool, device=cuda)
    slot_groups = torch.zeros(2, 0, 2, dtype=torch.long, device=cuda)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        update, _, _ = pool(x, valid, gates, active)
        pub_s, priv_s, _, _ = pool.forward_per_slot(x, valid, gates, active, slot_groups)
        pub_g, priv_g, _, _ = pool.forward_per_group(x, valid, gates, active)
    assert update.shape == (2, 0, 40) and pub_s.shape == (2, 0, 40) and pub_g.shape == (2, 0, 40)
    assert priv_s.shape == (2, 0, 2, 40) and priv_g.shape == (2, 0, 4, 40)
    (update.sum() + priv_s.sum() + priv_g.sum()).backward()
    assert pool.stacked_private.w_up.grad is not None
    assert float(pool.stacked_private.w_up.grad.float().abs().sum()) == 0.0


def test_pool_under_checkpoint_recompute_and_on_sequence_slices(cuda):
    """The reference runs the pool under activation-checkpoint recompute and on slices of
    the sequence (nestor/backbones/nestor.py:9135-9153).  Recompute replays the forward
    in the backward pass: outputs and every gradient must be bit-identical to the plain
    run (the kernels are deterministic, no float atomics).  A call on the whole sequence
    must equal the calls on its halves put together (tokens are independent)."""

    from torch.utils.checkpoint import checkpoint

    x, valid, gates, active, _ = _inputs(cuda)

    def run(use_checkpoint):
        pool = _pool(cuda, True).train()
        xi = x.clone().requires_grad_(True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            if use_checkpoint:
                out = checkpoint(lambda a: pool(a, valid, gates, active)[0], xi, use_reentrant=False)
            else:
                out = pool(xi, valid, gates, active)[0]
        out.float().square().sum().backward()
        return out.detach(), xi.grad, {n: p.grad for n, p in pool.named_parameters()}

    out0, gx0, gp0 = run(False)
    out1, gx1, gp1 = run(True)
    assert torch.equal(out0, out1) and torch.equal(gx0, gx1)
    for n in gp0:
        assert torch.equal(gp0[n], gp1[n]), n

    pool = _pool(cuda, True)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        whole = pool(x, valid, gates, active)[0]
        parts = [pool(x[:, a:b], valid[:, a:b], gates[:, a:b], active[:, a:b])[0]
                 for a, b in ((0, 33), (33, 70))]
    assert torch.equal(torch.cat(parts, dim=1), whole)


@pytest.mark.parametrize("layout", ["summed", "per_slot", "per_group"])
def test_pool_compiles_as_one_graph(cuda, layout):
    """The reference runs the pool region inside a compiled graph
    (nestor/backbones/triton_expert.py:71-77).  Each of the three forwards traces as ONE
    graph (``fullgraph=True``: a graph break would raise) with the custom ops as nodes, and
    the compiled forward + backward gives the eager path's bits."""

    x, valid, gates, active, slot_groups = _inputs(cuda)

    def run(compiled):
        pool = _pool(cuda, True).train()

        def step(xi):
            if layout == "summed":
                return pool(xi, valid, gates, active)[0]
            if layout == "per_slot":
                pub, priv, _, _ = pool.forward_per_slot(xi, valid, gates, active, slot_groups)
                return pub.unsqueeze(2) + priv
            pub, priv, _, _ = pool.forward_per_group(xi, valid, gates, active)
            return pub.unsqueeze(2) + priv

        fn = torch.compile(step, backend="aot_eager", fullgraph=True) if compiled else step
        xi = x.clone().requires_grad_(True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out = fn(xi)
        out.float().square().sum().backward()
        return out.detach(), xi.grad, {n: p.grad for n, p in pool.named_parameters()}

    out0, gx0, gp0 = run(False)
    out1, gx1, gp1 = run(True)
    assert torch.equal(out0, out1) and torch.equal(gx0, gx1)
    for n in gp0:
        assert (gp0[n] is None) == (gp1[n] is None), n
        if gp0[n] is not None:
            assert torch.equal(gp0[n], gp1[n]), n


def test_pool_with_router_noise_under_checkpoint_recompute(cuda):
    """Exploration noise pre-drawn with ``draw_router_noise`` and passed as ``router_noise``
    (nestor/backbones/expert_pools.py:588-623): the checkpoint's recompute routes as the
    forward did, so outputs and gradients equal the run without a checkpoint bit for bit;
    without noise heads the same call is the deterministic pool."""

    import nestor_amd as na
    from torch.utils.checkpoint import checkpoint

    x, valid, gates, active, _ = _inputs(cuda)
    torch.manual_seed(5)
    pool = na.ExpertPoolMLP(40, 4, 2, 3, 1, 5, 1, [], router_noise_mlp_hidden_dims=[],
                            private_gate_mode="switch")
    with torch.no_grad():
        pool.path_gate.weight.normal_()
        for r in [pool.public_router, *pool.private_routers]:
            r.noise_mlp.layers[0].weight.normal_(std=0.5)
    assert na.consolidate_stacked_expert_banks(pool, force=True) == 2
    pool.triton_fused = pool.triton_index = pool.fused_gate = True
    pool = pool.to(cuda).train()
    noise = pool.draw_router_noise(3, 70, cuda, torch.bfloat16)

    def run(use_checkpoint, router_noise):
        for p in pool.parameters():
            p.grad = None
        xi = x.clone().requires_grad_(True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            fn = lambda a: pool(a, valid, gates, active, router_noise=router_noise)[0]
            out = checkpoint(fn, xi, use_reentrant=False) if use_checkpoint else fn(xi)
        out.float().square().sum().backward()
        return out.detach(), xi.grad, {n: p.grad.clone() for n, p in pool.named_parameters() if p.grad is not None}

    out0, gx0, gp0 = run(False, noise)
    out1, gx1, gp1 = run(True, noise)
    assert torch.equal(out0, out1) and torch.equal(gx0, gx1)
    assert gp0.keys() == gp1.keys() and all(torch.equal(gp0[n], gp1[n]) for n in gp0)
    assert any("noise_mlp" in n for n in gp0)          # the noise heads learn
    # another draw routes differently; evaluation mode ignores the draw
    other = {k: -v for k, v in noise.items()}
    assert not torch.equal(run(False, other)[0], out0)
    pool.eval()
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        assert torch.equal(pool(x, valid, gates, active, router_noise=noise)[0],
                           pool(x, valid, gates, active)[0])
