"""Pins for the oracle itself (CPU only).  Each oracle function is checked
against something that does not share its formula: brute-force loops, structural
invariants, library routines, finite differences, or a mathematically equivalent
route (per-expert dense evaluation, per-token loop).  The input cases of the
reference's own map tests are reused with their seeds."""

import pytest
import torch
import torch.nn.functional as F

from oracle import bank as obank
from oracle import plan as oplan
from oracle import router as orouter
from oracle import rows as orows
from tests.helpers import bank_weights, gen, routing, zipf_ids


def brute_force_plan(ids: list[int], num_banks: int, slots: int, capacity: int = 0):
    """O(rows * E) construction of the padded layout straight from its
    definition: walk the banks in order, give each bank's rows (in row order)
    consecutive slots from a 16-aligned start."""

    rows = len(ids)
    rows_pad = ((rows + 15) // 16) * 16 + 16 * num_banks
    row_dest = [rows_pad - 1] * rows
    pad_token, pad_src, eid_pad, valid = ([0] * rows_pad for _ in range(4))
    order, counts, raw_starts, padded_starts, offs, kept = [], [], [], [], [], [0] * rows
    cursor = 0
    for e in range(num_banks):
        members = [r for r in range(rows) if ids[r] == e]
        raw_starts.append(len(order))
        order.extend(members)
        counts.append(len(members))
        padded_starts.append(cursor)
        keep = members if capacity <= 0 else members[:capacity]
        for j, r in enumerate(keep):
            p = cursor + j
            row_dest[r], pad_token[p], pad_src[p], eid_pad[p], valid[p], kept[r] = p, r // slots, r, e, 1, 1
        cursor += ((len(keep) + 15) // 16) * 16
        offs.append(cursor)
    offs[-1] = rows_pad
    return dict(order=order, counts=counts, raw_starts=raw_starts, padded_starts=padded_starts,
                offs=offs, row_dest=row_dest, pad_token=pad_token, pad_src_row=pad_src,
                eid_pad=eid_pad, pad_valid=valid, row_kept=kept, rows_pad=rows_pad)


def _assert_plan(ids2d, num_banks, capacity=0):
    slots = ids2d.shape[1]
    flat = ids2d.reshape(-1)
    plan = oplan.dispatch_plan(flat, num_banks, slots, torch.float32, capacity)
    want = brute_force_plan(flat.tolist(), num_banks, slots, capacity)
    assert plan.rows_pad == want["rows_pad"]
    for name in ("order", "counts", "raw_starts", "padded_starts", "offs", "row_dest", "pad_token",
                 "pad_src_row", "eid_pad", "pad_valid", "row_kept"):
        assert getattr(plan, name).tolist() == want[name], name
    # structural invariants
    valid = plan.pad_valid != 0
    kept = plan.row_kept.bool()
    assert int(valid.sum()) == int(kept.sum())
    assert torch.equal(plan.pad_src_row[plan.row_dest[kept]], torch.nonzero(kept).squeeze(-1))
    assert torch.equal(plan.pad_token[valid], plan.pad_src_row[valid] // slots)
    assert (plan.padded_starts % 16 == 0).all() and int(plan.offs[-1]) == plan.rows_pad
    assert not valid[plan.rows_pad - 1]  # the drop target is always slack
    for name in ("pad_token", "pad_src_row", "eid_pad"):
        assert (getattr(plan, name)[~valid] == 0).all()


def test_plan_reference_test_inputs():
    torch.manual_seed(0)
    _assert_plan(torch.randint(0, 8, (300, 3)), 8)
    torch.manual_seed(1)
    ids = torch.randint(1, 5, (200, 2))
    ids[ids == 4] = 2
    _assert_plan(ids, 6)
    _assert_plan(torch.zeros(65, 1, dtype=torch.long), 1)
    torch.manual_seed(2)
    _assert_plan(torch.randint(0, 4, (341, 3)), 4)
    _assert_plan(torch.randint(0, 4, (342, 3)), 4)


@pytest.mark.parametrize("capacity", [0, 3, 17, 40])
def test_plan_brute_force_with_capacity(capacity):
    _assert_plan(zipf_ids(3, 150, 2, 12), 12, capacity)
    _assert_plan(torch.randint(0, 5, (97, 3), generator=gen(capacity)), 5, capacity)


def test_plan_capacity_not_binding_is_dropless():
    ids = torch.randint(0, 6, (200, 2), generator=gen(1)).reshape(-1)
    a = oplan.dispatch_plan(ids, 6, 2, torch.bfloat16, 0)
    b = oplan.dispatch_plan(ids, 6, 2, torch.bfloat16, 10_000)
    for x, y in zip(a[2:], b[2:]):
        assert torch.equal(x, y)


def test_dispatch_rows_loop():
    ids, _ = routing(1, 50, 3, 7)
    plan = oplan.dispatch_plan(ids.reshape(-1), 7, 3, torch.bfloat16)
    x = torch.randn(50, 24, generator=gen(2))
    out = orows.dispatch_rows(x, plan.pad_token, plan.pad_valid, torch.bfloat16)
    for p in range(plan.rows_pad):
        want = x[plan.pad_token[p]].bfloat16() if plan.pad_valid[p] != 0 else torch.zeros(24, dtype=torch.bfloat16)
        assert torch.equal(out[p], want)
    g = torch.randn(plan.rows_pad, 24, generator=gen(3)).bfloat16()
    gx = orows.dispatch_rows_bwd(g, plan.row_dest, 50, 3, torch.float32)
    for t in range(50):
        want = sum(g[plan.row_dest[t * 3 + j]].float() for j in range(3))
        torch.testing.assert_close(gx[t], want, rtol=1e-6, atol=1e-6)
    # the backward is the adjoint of the forward: <dispatch(x), g> == <x, dispatch_bwd(g)>
    xd, gd = x.double(), g.double()
    fwd = xd.index_select(0, plan.pad_token) * plan.pad_valid.double().unsqueeze(1)
    bwd = gd.index_select(0, plan.row_dest).view(50, 3, -1).sum(1)
    torch.testing.assert_close((fwd * gd).sum(), (xd * bwd).sum())


def test_swiglu_bwd_against_finite_differences():
    """The backward formula s(1 + g(1 - s)) and the two products, unrounded, in fp64."""

    g = gen(4)
    up = torch.randn(6, 5, generator=g, dtype=torch.float64, requires_grad=True)
    gate = torch.randn(6, 5, generator=g, dtype=torch.float64, requires_grad=True)
    assert torch.autograd.gradcheck(lambda u, ga: F.silu(ga) * u, (up, gate))
    go = torch.randn(6, 5, generator=g, dtype=torch.float64)
    (F.silu(gate) * up).backward(go)
    # fp64 in: the bf16 roundings are no-ops and only the oracle's fp32 arithmetic remains
    gup, ggate = orows.swiglu_bwd(go, up.detach(), gate.detach())
    torch.testing.assert_close(gup, up.grad, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(ggate, gate.grad, rtol=1e-5, atol=1e-6)
    # with bf16 inputs the same function stays within two bf16 ulps of the fp64 value
    ub, gb, gob = up.detach().bfloat16(), gate.detach().bfloat16(), go.bfloat16()
    rup, rgate = orows.swiglu_bwd(gob, ub, gb)
    u64, g64 = ub.double().requires_grad_(True), gb.double().requires_grad_(True)
    (F.silu(g64) * u64).backward(gob.double())
    torch.testing.assert_close(rup.double(), u64.grad, rtol=2 ** -6, atol=1e-3)
    torch.testing.assert_close(rgate.double(), g64.grad, rtol=2 ** -6, atol=1e-3)


def test_combine_rows_loop_and_backward():
    ids, weights = routing(5, 40, 4, 6)
    plan = oplan.dispatch_plan(ids.reshape(-1), 6, 4, torch.bfloat16)
    y = torch.randn(plan.rows_pad, 16, generator=gen(6)).bfloat16()
    w = weights.reshape(-1)
    for group in (1, 2, 4):
        out = orows.combine_rows(y, plan.row_dest, w, group, torch.float32)
        for o in range(160 // group):
            want = sum(y[plan.row_dest[o * group + e]].float() * w[o * group + e] for e in range(group))
            torch.testing.assert_close(out[o], want, rtol=1e-6, atol=1e-6)
        # fused kernel form == the eager chain up to the one bf16 rounding the eager form adds
        eager = orows.combine_rows_eager(y, plan.row_dest, w, group, torch.float32)
        torch.testing.assert_close(out, eager, rtol=1e-6, atol=1e-6)
    # backward vs autograd of the unrounded definition in fp64
    yd = y.double().requires_grad_(True)
    wd = w.double().requires_grad_(True)
    outd = (yd.index_select(0, plan.row_dest) * wd.unsqueeze(1)).view(80, 2, -1).sum(1)
    go = torch.randn(80, 16, generator=gen(7))
    outd.backward(go.double())
    gy, gw = orows.combine_rows_bwd(go, y, plan.pad_src_row, plan.pad_valid, w, 2)
    torch.testing.assert_close(gy.double(), yd.grad, rtol=2 ** -7, atol=1e-6)  # gy is rounded to bf16
    torch.testing.assert_close(gw.double(), wd.grad, rtol=1e-5, atol=1e-5)
    assert (gy[plan.pad_valid == 0] == 0).all()


def test_path_mix_loop_and_backward():
    """Element loop with hand-placed roundings, then fp64 autograd of the definition."""

    pub = torch.randn(7, 16, generator=gen(1)).bfloat16()
    priv = torch.randn(7, 16, generator=gen(2)).bfloat16()
    alpha = torch.softmax(torch.randn(7, 2, generator=gen(3)), -1).bfloat16()
    out = orows.path_mix(pub, priv, alpha)
    assert out.dtype == torch.bfloat16
    for t in range(7):
        for i in range(16):
            a = (alpha[t, 0].float() * pub[t, i].float()).bfloat16().float()
            b = (alpha[t, 1].float() * priv[t, i].float()).bfloat16().float()
            assert out[t, i] == (a + b).bfloat16()
    go = torch.randn(7, 16, generator=gen(4)).bfloat16()
    g_pub, g_priv, g_alpha = orows.path_mix_bwd(go, pub, priv, alpha)
    leaves = [t.double().requires_grad_(True) for t in (pub, priv, alpha)]
    (leaves[2][:, 0:1] * leaves[0] + leaves[2][:, 1:2] * leaves[1]).backward(go.double())
    for got, leaf in zip((g_pub, g_priv, g_alpha), leaves):
        torch.testing.assert_close(got.double(), leaf.grad, rtol=2 ** -6, atol=2e-2)
    assert not torch.equal(g_alpha[:, 0], g_alpha[:, 1])


def test_path_scale_loop():
    """Column scatter + path weight against an element loop (distinct columns per token,
    as top-k selection gives them)."""

    tokens, slots, cols, d = 9, 2, 5, 8
    inp = torch.randn(tokens, slots, d, generator=gen(1)).bfloat16()
    alpha = torch.softmax(torch.randn(tokens, 2, generator=gen(2)), -1).bfloat16()
    dest = torch.stack([torch.randperm(cols, generator=gen(10 + t))[:slots] for t in range(tokens)])
    out = orows.path_scale(inp, alpha, 1, dest, cols)
    assert out.shape == (tokens, cols, d)
    for t in range(tokens):
        for o in range(cols):
            hit = [s for s in range(slots) if dest[t, s] == o]
            for i in range(d):
                want = (alpha[t, 1].float() * inp[t, hit[0], i].float()).bfloat16() if hit else 0.0
                assert out[t, o, i] == want
    plain = orows.path_scale(inp, alpha, 0)
    assert torch.equal(plain, alpha[:, 0:1, None] * inp)
    go = torch.randn(tokens, cols, d, generator=gen(3)).bfloat16()
    g_in, g_alpha = orows.path_scale_bwd(go, inp, alpha, 1, dest, cols)
    assert (g_alpha[:, 0] == 0).all()
    for t in range(tokens):
        picked = go[t, dest[t]].float()
        torch.testing.assert_close(g_in[t].float(), picked * alpha[t, 1].float(), rtol=2 ** -7, atol=1e-6)
        torch.testing.assert_close(g_alpha[t, 1].float(), (picked * inp[t].float()).sum(),
                                   rtol=2 ** -6, atol=5e-2)


def test_biased_gold_per_token_modules():
    """The biased / pointwise gold against per-token evaluation with ``F.linear`` on the
    per-expert ``weight = owner[i].t()`` views, the way the reference's modules hold them
    (nestor/scaling/blocks.py:306-312, expert_bank_stack.py:72-77)."""

    import torch.nn.functional as F

    tokens, slots, banks, d, h = 12, 2, 3, 6, 5
    g = gen(5)
    x = torch.randn(tokens, d, generator=g, dtype=torch.float64)
    w_up, w_gate = (torch.randn(banks, d, h, generator=g, dtype=torch.float64) for _ in range(2))
    w_down = torch.randn(banks, h, d, generator=g, dtype=torch.float64)
    b_up = torch.randn(banks, h, generator=g, dtype=torch.float64)
    b_down = torch.randn(banks, d, generator=g, dtype=torch.float64)
    ids = torch.randint(0, banks, (tokens, slots), generator=g)
    wts = torch.rand(tokens, slots, generator=g, dtype=torch.float64)
    for gated, act in ((True, "silu"), (False, "gelu")):
        out = obank.gold_combine(x, w_up, w_gate if gated else None, w_down, ids, wts, slots,
                                 b_up=b_up, b_down=b_down, activation=act)
        fn = getattr(F, act)
        for t in range(tokens):
            want = torch.zeros(d, dtype=torch.float64)
            for s_ in range(slots):
                e = int(ids[t, s_])
                up = F.linear(x[t], w_up[e].t(), b_up[e])
                hid = fn(F.linear(x[t], w_gate[e].t())) * up if gated else fn(up)
                want += wts[t, s_] * F.linear(hid, w_down[e].t(), b_down[e])
            torch.testing.assert_close(out[t, 0], want, rtol=1e-10, atol=1e-10)


def test_gate_combine_slots_loop():
    rows, dim, groups = 12, 8, 3
    out_c = torch.randn(rows, dim, generator=gen(1)).bfloat16()
    bo = torch.randn(groups, dim, generator=gen(2))
    gid = torch.randint(0, groups, (rows,), generator=gen(3))
    gates = torch.rand(rows, generator=gen(4))
    slot_rows = torch.randperm(rows, generator=gen(5))[:9]
    for dtype in (torch.float32, torch.bfloat16):
        out = orows.gate_combine_slots(out_c, bo, gid, gates, slot_rows, dtype)
        for s_, r in enumerate(slot_rows.tolist()):
            for i in range(dim):
                val = (out_c[r, i].float() + bo[gid[r], i].bfloat16().float()).bfloat16()
                want = (val.to(dtype).float() * gates[r].to(dtype).float()).to(dtype)
                assert out[s_, i] == want
    plain = orows.gate_combine_slots(out_c, None, None, gates, slot_rows, torch.float32)
    assert torch.equal(plain, out_c.float().index_select(0, slot_rows) * gates[slot_rows, None])


def test_segment_mm_and_bank_routes_agree():
    """grouped (padded) path == per-expert dense evaluation == sparse loop ==
    per-token loop, in fp32 where only summation order differs
    (the reference's own tolerance, tests/test_expert_pools.py:225-226)."""

    tokens, d, h, banks, slots = 60, 16, 24, 5, 2
    ids, weights = routing(8, tokens, slots, banks)
    x = torch.randn(tokens, d, generator=gen(9))
    w_up, w_gate, w_down = bank_weights(10, banks, d, h, 0.3)
    grouped = obank.grouped_expert_combine(x, w_up, w_gate, w_down, ids, weights, slots, torch.float32)
    gold = obank.gold_combine(x, w_up, w_gate, w_down, ids, weights, slots)
    sparse = torch.zeros(tokens, d)
    obank.accumulate_sparse_expert_bank(sparse, x, w_up, w_gate, w_down,
                                        obank.dense_weights(ids, weights, banks))
    per_token = torch.zeros(tokens, d)
    for t in range(tokens):
        for j in range(slots):
            e = int(ids[t, j])
            hid = F.silu(x[t] @ w_gate[e]) * (x[t] @ w_up[e])
            per_token[t] += weights[t, j] * (hid @ w_down[e])
    for other in (gold.view(tokens, d), sparse, per_token):
        torch.testing.assert_close(grouped.view(tokens, d), other, rtol=1e-5, atol=1e-6)
    # per-slot layout: group == 1 keeps every (token, slot) row apart
    per_slot = obank.grouped_expert_combine(x, w_up, w_gate, w_down, ids, weights, 1, torch.float32)
    torch.testing.assert_close(per_slot.sum(1), grouped.view(tokens, d), rtol=1e-5, atol=1e-6)
    # capacity: dropped rows contribute exactly nothing
    plan = oplan.dispatch_plan(ids.reshape(-1), banks, slots, torch.float32, 10)
    assert (plan.row_kept == 0).any()
    capped = obank.grouped_expert_combine(x, w_up, w_gate, w_down, ids, weights, slots, torch.float32, 10)
    gold_c = obank.gold_combine(x, w_up, w_gate, w_down, ids, weights, slots, plan.row_kept)
    torch.testing.assert_close(capped, gold_c, rtol=1e-5, atol=1e-6)


def test_bf16_chain_within_tolerance_of_gold():
    """The rounding-point chain stays inside the 1e-2 rel-L2 bar vs fp32."""

    tokens, d, h, banks, slots = 256, 64, 128, 6, 2
    ids, weights = routing(11, tokens, slots, banks)
    x = torch.randn(tokens, d, generator=gen(12)).bfloat16()
    w3 = bank_weights(13, banks, d, h, 0.1, torch.bfloat16)
    emu = obank.grouped_expert_combine(x, *w3, ids, weights.bfloat16(), slots, torch.bfloat16)
    gold = obank.gold_combine(x.float(), *[t.float() for t in w3], ids, weights.bfloat16().float(), slots)
    assert ((emu.float() - gold).norm() / gold.norm()).item() < 1e-2


def test_router_library_routines_and_special_cases():
    g = gen(14)
    scores = torch.randn(500, 8, generator=g)  # fp32 draws: no ties
    bias = torch.randn(8, generator=g) * 0.1
    valid = torch.rand(500, generator=g) > 0.1
    out = orouter.route(scores, bias, 2, "renorm", valid)
    tk = torch.topk(scores + bias, 2, dim=-1)
    assert torch.equal(out.topk_indices, tk.indices)  # tie-free: any correct top-k agrees
    sel = scores.gather(-1, tk.indices)
    want = torch.zeros_like(scores).scatter(-1, tk.indices, torch.softmax(sel, -1)) * valid.unsqueeze(-1)
    torch.testing.assert_close(out.gates, want)
    torch.testing.assert_close(out.softmax_probs, torch.softmax(scores, -1))
    torch.testing.assert_close(out.gates.sum(-1), valid.float())
    # top-1 renorm: the gate is the constant 1 (nestor/backbones/nestor.py:426-444)
    one = orouter.route(scores, bias, 1, "renorm", valid)
    assert torch.equal(one.gates.sum(-1), valid.float())
    # switch: full-softmax probability of the winners
    sw = orouter.route(scores, bias, 1, "switch", valid)
    p = torch.softmax(scores, -1).gather(-1, sw.topk_indices).squeeze(-1) * valid
    torch.testing.assert_close(sw.gates.sum(-1), p)
    # ties resolve to the lowest index, in descending-score order
    tied = torch.tensor([[1.0, 3.0, 3.0, 0.0, 3.0]])
    assert orouter.stable_topk(tied, 2).tolist() == [[1, 2]]
    assert orouter.stable_topk(tied, 4).tolist() == [[1, 2, 4, 0]]


def test_balancing_update_loop():
    """Counting loop and the sign step: over-used choices go down by the rate, under-used up."""

    topk = torch.tensor([[[0, 1], [0, 2], [0, 1], [3, 0]]])
    valid = torch.tensor([[True, True, False, True]])
    bias = torch.tensor([0.5, 0.0, -0.25, 1.0])
    counts = [0, 0, 0, 0]
    for t in range(4):
        if valid[0, t]:
            for c in topk[0, t].tolist():
                counts[c] += 1
    assert counts == [3, 1, 1, 1]  # mean 1.5
    new = orouter.balancing_update(bias, topk, valid, 0.125)
    assert new.tolist() == [0.375, 0.125, -0.125, 1.125]


def test_private_slots_closed_form():
    tokens, groups, q, k_a, k_q = 30, 5, 3, 2, 2
    g = gen(15)
    gates = torch.rand(tokens, groups, q, generator=g)
    choices = torch.stack([torch.randperm(q, generator=g)[:k_q] for _ in range(tokens * groups)]).view(tokens, groups, k_q)
    col_scores = torch.rand(tokens, groups, generator=g)
    selected = col_scores.topk(k_a, -1).indices
    group_gates = torch.zeros(tokens, groups).scatter(-1, selected, 0.5)
    ids, weights, sel = orouter.private_slots(gates, choices, group_gates, k_a, selected)
    for t in range(tokens):
        for j in range(k_a):
            col = int(selected[t, j])
            for e in range(k_q):
                c = int(choices[t, col, e])
                assert int(ids[t, j * k_q + e]) == col * q + c
                assert float(weights[t, j * k_q + e]) == pytest.approx(float(gates[t, col, c]) * 0.5)
    assert torch.equal(sel, selected)
