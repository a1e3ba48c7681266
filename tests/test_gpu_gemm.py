"""Grouped GEMM kernels through the C ABI vs per-segment matmul (the
reference's own CPU fallback, nestor/backbones/grouped_mm.py:97-104)."""

import pytest
import torch

from oracle import bank as obank
from oracle import plan as oplan
from oracle import rows as orows
from tests.helpers import gen, rel_l2, routing, zipf_ids

pytestmark = pytest.mark.gpu


def _setup(tokens, slots, banks, cuda, skew=False, capacity=0):
    from nestor_amd.dispatch import dispatch_plan

    ids = zipf_ids(1, tokens, slots, banks) if skew else routing(tokens, tokens, slots, banks)[0]
    want = oplan.dispatch_plan(ids.reshape(-1), banks, slots, torch.bfloat16, capacity)
    got = dispatch_plan(ids.reshape(-1).to(cuda), banks, slots, torch.bfloat16, capacity)
    return want, got


def _padded_input(want, cols, seed, scale=1.0):
    a = (torch.randn(want.rows_pad, cols, generator=gen(seed)) * scale).to(torch.bfloat16)
    return a * want.pad_valid.unsqueeze(1)  # slack rows are zero in every padded tensor


SHAPES = [
    # tokens, slots, banks, K, N, skew
    (300, 2, 6, 40, 24, False),       # ragged everything (K, N multiples of 8 only)
    (64, 1, 1, 64, 128, False),       # a single bank
    (1000, 3, 20, 512, 1024, False),  # tiny config widths
    (700, 2, 16, 200, 424, True),     # production-like odd widths, empty banks
    (2048, 2, 8, 1024, 2048, False),
    # shapes the direct-to-LDS kernels take: K loops shorter than the prefetch
    # ring, output widths that end inside a tile
    (500, 2, 5, 32, 512, False),
    (500, 2, 5, 64, 520, False),
    (700, 2, 7, 96, 1000, True),
    (900, 1, 3, 512, 544, False),
    # the persistent weight-gradient kernel with tiles that overhang both of its
    # output dimensions, empty banks and segments of a few rows
    (1200, 2, 24, 264, 520, True),
    (40, 1, 12, 256, 256, True),
    # contractions that end inside a K step on the direct-to-LDS path (the production
    # widths): forward with K = 424 / 216 / 8, input gradient with K = 424 / 184
    (1500, 2, 6, 424, 1280, False),
    (1500, 2, 6, 1280, 424, True),
    (900, 3, 5, 216, 640, False),
    (640, 1, 3, 8, 512, False),
    (1100, 2, 4, 640, 184, False),
    # input gradients narrower than the 256-column tile (h = 160 / 136 of the production arms)
    (1500, 2, 6, 160, 1280, True),
    (700, 2, 5, 136, 512, False),
]


@pytest.mark.parametrize("tokens,slots,banks,K,N,skew", SHAPES)
def test_segment_mm_forward_and_grads(cuda, tokens, slots, banks, K, N, skew):
    from nestor_amd import segment_mm

    want, got = _setup(tokens, slots, banks, cuda, skew)
    a = _padded_input(want, K, 3)
    b = (torch.randn(banks, K, N, generator=gen(4)) / K ** 0.5).to(torch.bfloat16)
    ref = obank.segment_mm(a, b, want.offs)
    ta = a.to(cuda).requires_grad_(True)
    tb = b.to(cuda).requires_grad_(True)
    out = segment_mm(ta, tb, got.offs)
    assert out.shape == ref.shape and out.dtype == torch.bfloat16
    torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=2 ** -6, atol=1e-3)
    assert rel_l2(out, ref) < 2e-3
    go = _padded_input(want, N, 5)
    out.backward(go.to(cuda))
    # dA = go @ b^T per segment; dB[e] = a_seg^T @ go_seg (fp32 references)
    bounds = [0] + want.offs.tolist()
    da = torch.cat([go[bounds[i]:bounds[i + 1]].float() @ b[i].float().t() for i in range(banks)])
    db = torch.stack([a[bounds[i]:bounds[i + 1]].float().t() @ go[bounds[i]:bounds[i + 1]].float()
                      for i in range(banks)])
    assert rel_l2(ta.grad, da) < 4e-3
    assert rel_l2(tb.grad, db) < 4e-3
    empty = want.counts == 0
    if empty.any():
        assert (tb.grad.cpu()[empty] == 0).all()  # every bank gets a gradient, zeros if unused


@pytest.mark.parametrize("tokens,slots,banks,K,H,skew", [
    (300, 2, 6, 40, 24, False), (1000, 3, 20, 512, 1024, False), (700, 2, 16, 200, 424, True),
    (2048, 1, 4, 1024, 2048, False),
    (500, 2, 5, 64, 256, False), (600, 1, 4, 96, 520, False), (900, 2, 6, 512, 576, True),
    # production widths: the fused input gradient contracts over 2 x 424 / 2 x 216 columns,
    # each phase ending inside a K step
    (1500, 2, 6, 1280, 424, False), (900, 3, 5, 640, 216, True), (700, 2, 4, 200, 184, False),
])
def test_upgate_swiglu_fused_matches_unfused(cuda, tokens, slots, banks, K, H, skew):
    """The fused up|gate + SwiGLU kernel against the oracle chain with the
    reference's rounding points, values and gradients."""

    from nestor_amd import ops

    want, got = _setup(tokens, slots, banks, cuda, skew)
    x_pad = _padded_input(want, K, 6)
    w_up = (torch.randn(banks, K, H, generator=gen(7)) / K ** 0.5).to(torch.bfloat16)
    w_gate = (torch.randn(banks, K, H, generator=gen(8)) / K ** 0.5).to(torch.bfloat16)
    ug_ref = obank.segment_mm(x_pad, torch.cat([w_up, w_gate], -1), want.offs)
    hid_ref = orows.swiglu(ug_ref[:, :H], ug_ref[:, H:])
    tx = x_pad.to(cuda).requires_grad_(True)
    tu = w_up.to(cuda).requires_grad_(True)
    tg = w_gate.to(cuda).requires_grad_(True)
    up_gate, hidden = ops.upgate_swiglu_op(tx, tu, tg, got.tile_table, got.offs,
                                           got.padded_starts, got.kept_counts)
    torch.testing.assert_close(up_gate.cpu().float(), ug_ref.float(), rtol=2 ** -6, atol=1e-3)
    torch.testing.assert_close(hidden.cpu().float(), hid_ref.float(), rtol=2 ** -5, atol=2e-3)
    assert rel_l2(hidden, hid_ref) < 3e-3
    slack = want.pad_valid == 0
    assert (hidden.cpu()[slack] == 0).all() and (up_gate.cpu()[slack] == 0).all()
    gh = _padded_input(want, H, 9)
    hidden.backward(gh.to(cuda))
    # fp32 reference of the same chain from the bf16 operands
    xf = x_pad.float().requires_grad_(True)
    uf = w_up.float().requires_grad_(True)
    gf = w_gate.float().requires_grad_(True)
    bounds = [0] + want.offs.tolist()
    outs = []
    for i in range(banks):
        seg = xf[bounds[i]:bounds[i + 1]]
        outs.append(torch.nn.functional.silu(seg @ gf[i]) * (seg @ uf[i]))
    torch.cat(outs).backward(gh.float())
    assert rel_l2(tx.grad, xf.grad) < 1e-2
    assert rel_l2(tu.grad, uf.grad) < 1e-2
    assert rel_l2(tg.grad, gf.grad) < 1e-2


@pytest.mark.parametrize("tokens,slots,banks,K,H,skew", [
    (2048, 2, 8, 1024, 512, False),   # one launch: column tiles never straddle the halves
    (1200, 2, 24, 264, 256, True),    # one launch, overhanging row tiles, empty banks
    (900, 3, 5, 640, 216, True),      # widths that fall back to two launches
    (300, 2, 6, 40, 24, False),
])
@pytest.mark.parametrize("out_f32", [False, True])
def test_weight_gradient_pair_equals_two_calls(cuda, tokens, slots, banks, K, H, skew, out_f32):
    """Both weight gradients of the fused up|gate GEMM in one call: the same bits as one
    call per half, and both against an fp32 per-segment product."""

    from nestor_amd import ops

    want, got = _setup(tokens, slots, banks, cuda, skew)
    a = _padded_input(want, K, 11)
    g = _padded_input(want, 2 * H, 12)
    ta, tg = a.to(cuda), g.to(cuda)
    for starts, counts in ((None, None), (got.padded_starts, got.kept_counts)):
        pair = ops.grouped_gemm_tn_pair(ta, tg, got.offs, starts, counts, out_f32)
        one = [ops.grouped_gemm_tn(ta, tg[:, :H], got.offs, starts, counts, out_f32),
               ops.grouped_gemm_tn(ta, tg[:, H:], got.offs, starts, counts, out_f32)]
        for half in range(2):
            assert pair[half].dtype == (torch.float32 if out_f32 else torch.bfloat16)
            assert torch.equal(pair[half], one[half])
    bounds = [0] + want.offs.tolist()
    for half in range(2):
        ref = torch.stack([a[bounds[i]:bounds[i + 1]].float().t()
                           @ g[bounds[i]:bounds[i + 1], half * H:(half + 1) * H].float()
                           for i in range(banks)])
        assert rel_l2(pair[half], ref) < 4e-3


def test_slack_tail_is_zero_filled(cuda):
    """Rows behind the last segment belong to no bank: outputs there are zeros
    even when the output buffer held garbage."""

    from nestor_amd import ops

    want, got = _setup(200, 1, 30, cuda)
    a = _padded_input(want, 64, 1)
    b = torch.randn(30, 64, 128, generator=gen(2)).to(torch.bfloat16)
    out = ops.grouped_gemm_nn(a.to(cuda), b.to(cuda), got.tile_table)
    tail = int((want.padded_starts + (want.counts + 15) // 16 * 16)[-1])
    assert tail < want.rows_pad
    assert (out.cpu()[tail:] == 0).all()


def test_clock_hook_counts_workgroups_and_leaves_results_alone(cuda):
    """The instrumented GEMM build of the measurement library: the same bits as the
    product kernels, every workgroup that multiplied is counted, and outside the
    ``instrumented`` block the product library runs (it has no hook at all)."""
    from nestor_amd import ops, probes

    tokens, slots, banks, K, N = 2048, 2, 8, 1024, 2048
    want, got = _setup(tokens, slots, banks, cuda)
    a = _padded_input(want, K, 3).to(cuda)
    b = (torch.randn(banks, K, N, generator=gen(4)) / K ** 0.5).to(torch.bfloat16).to(cuda)
    g = _padded_input(want, N, 5).to(cuda)
    plain = ops.grouped_gemm_nn(a, b, got.tile_table)
    plain_w = ops.grouped_gemm_tn(a, g, got.offs, got.padded_starts, got.counts)
    sink = torch.zeros(64, 4, dtype=torch.int64, device=cuda)
    torch.cuda.synchronize()
    with probes.instrumented(sink.data_ptr()):
        hooked = ops.grouped_gemm_nn(a, b, got.tile_table)
        torch.cuda.synchronize()
        rows_total = sink.sum(0).tolist()
        sink.zero_()
        hooked_w = ops.grouped_gemm_tn(a, g, got.offs, got.padded_starts, got.counts)
        torch.cuda.synchronize()
        wgrad_total = sink.sum(0).tolist()
    assert torch.equal(plain, hooked) and torch.equal(plain_w, hooked_w)
    for cycles, ticks, groups, steps in (rows_total, wgrad_total):
        assert cycles > 0 and ticks > 0 and groups > 0 and steps >= groups
    # row-tiled launch: one workgroup per (balanced row tile, column tile of 512), K / 32 steps each
    padded = (want.counts + 15) // 16 * 16
    tiles = sum((((int(c) + 31) // 32) + 4) // 5 for c in padded.tolist())
    assert rows_total[2] == tiles * (N // 512) and rows_total[3] == rows_total[2] * (K // 32)
    sink.zero_()
    ops.grouped_gemm_nn(a, b, got.tile_table)
    torch.cuda.synchronize()
    assert int(sink.sum()) == 0


def test_mfma_clock_probe_reports_instructions_and_clocks(cuda):
    import ctypes

    from nestor_amd import probes as _lib

    khz = _lib.wall_clock_khz()
    assert khz > 0
    cus = torch.cuda.get_device_properties(cuda).multi_processor_count
    counters = torch.zeros(4, dtype=torch.int64, device=cuda)
    for random_operands in (0, 1):
        _lib.call("nestor_hip_mfma_clock_probe", random_operands, 500,
                  ctypes.c_void_p(counters.data_ptr()), torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        cycles, ticks, instructions, _ = counters.tolist()
        assert instructions == cus * 4 * 500 * 16
        # every instruction occupies its SIMD's matrix core for 32 cycles
        assert cycles >= 500 * 16 * 32 and ticks > 0
        mhz = cycles / ticks * khz / 1000.0
        assert 300 < mhz < 3000
    from nestor_amd._lib import NestorHipError

    with pytest.raises(NestorHipError):
        _lib.call("nestor_hip_mfma_clock_probe", 0, 0, ctypes.c_void_p(counters.data_ptr()), None)


def test_mfma_mix_probe_counts_and_rejects_bad_arguments(cuda):
    import ctypes

    from nestor_amd import probes as _lib
    from nestor_amd._lib import NestorHipError

    cus = torch.cuda.get_device_properties(cuda).multi_processor_count
    region = 1 << 16
    src = torch.zeros(8 * region, dtype=torch.uint8, device=cuda)
    counters = torch.zeros(4, dtype=torch.int64, device=cuda)
    stream = torch.cuda.current_stream().cuda_stream
    plain = None
    for reads, transfers in ((0, 0), (16, 0), (0, 8), (16, 8), (16, 10), (16, 12)):
        _lib.call("nestor_hip_mfma_mix_probe", reads, transfers, 300, ctypes.c_void_p(src.data_ptr()),
                  src.numel(), region, ctypes.c_void_p(counters.data_ptr()), stream)
        torch.cuda.synchronize()
        cycles, ticks, instructions, _ = counters.tolist()
        assert instructions == cus * 4 * 300 * 32 and ticks > 0
        assert cycles >= 300 * 32 * 32
        if plain is None:
            plain = cycles
    # the other instructions cost the wavefront issue cycles: never faster than the bare stream
    assert cycles >= plain
    # unsupported mix, no rounds, a region that is not whole 32 KiB steps, a buffer too small
    # for eight regions: refused on the host, nothing launched
    for bad in ((8, 8, 300, region, src.numel()), (16, 8, 0, region, src.numel()),
                (16, 8, 300, 1000, src.numel()), (16, 8, 300, 3 * 32768 + 4096, src.numel()),
                (16, 8, 300, region, 8 * region - 1)):
        with pytest.raises(NestorHipError):
            _lib.call("nestor_hip_mfma_mix_probe", bad[0], bad[1], bad[2], ctypes.c_void_p(src.data_ptr()),
                      bad[4], bad[3], ctypes.c_void_p(counters.data_ptr()), stream)
