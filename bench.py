"""Benchmark of the routed hybrid expert-MLP path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload mlp_1b]

A step is one forward + backward pass of the hot path over one batch of the
1b-like workload (T = 32768 tokens, d = 2048, h = 4096, 16 public + 32 x 4
private SwiGLU experts, top-2 columns -> top-1 private each, + top-1 public):
column router, pool routers, index build, dispatch, grouped GEMMs with SwiGLU,
weighted combine, and every gradient (inputs, routing weights, all three banks).
Inputs are resident in HBM before the timed region.  One JSON line is printed.
"""

from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

BF16_MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 MFMA, published
HBM_PEAK_GBS = 8000.0           # MI355X HBM3E, published
UPGATE_KERNEL_NAME = ("grouped_gemm_dma_kernel<DmaCfg<160,512,32,1,4,3>, kNNUpGate> "
                      "(private bank up|gate + SwiGLU)")
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "upgate_mlp_1b_hbm_counters.md")
# the sources the dominant kernel is compiled from (the kernels and their shared header)
GEMM_SOURCES = [os.path.join(ROOT, "nestor_amd", "csrc", name)
                for name in ("grouped_gemm.hip", "gemm_common.hpp")]


def gemm_source_digest() -> str:
    """sha256 over the bf16 GEMM kernels' source files, in the order above."""

    import hashlib

    h = hashlib.sha256()
    for path in GEMM_SOURCES:
        h.update(open(path, "rb").read())
    return h.hexdigest()


def measured_traffic_bytes() -> int | None:
    """HBM bytes per launch of the dominant kernel as the counter summary under
    ``profiles/`` records them (``traffic_bytes_per_launch: N`` beside the
    ``kernel_source_sha256`` of the GEMM sources the counters were collected on).  A
    summary made for another version of that source says nothing about this one:
    ``None`` then, and when the summary is absent."""

    import re

    try:
        text = open(TRAFFIC_PROFILE).read()
        digest = gemm_source_digest()
    except OSError:
        return None
    nbytes = re.search(r"traffic_bytes_per_launch:\s*(\d+)", text)
    sha = re.search(r"kernel_source_sha256:\s*([0-9a-f]{64})", text)
    if not nbytes or not sha or sha.group(1) != digest:
        return None
    return int(nbytes.group(1))


def _event_ms(fn, iters: int) -> float:
    """Average duration of ``fn`` over ``iters`` launches, from HIP events recorded
    on the stream the kernels are launched on (torch's current stream)."""

    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    fn()
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / iters


def routed_slots(w, tensors, column_router, pool):
    """The workload's own routing: ``(private ids [T, k_a * k_q], private slot weights,
    public ids [T, k_p], public slot weights)``."""

    x3 = tensors.x.view(1, w.tokens, w.d_model)
    valid = torch.ones(1, w.tokens, dtype=torch.bool, device=tensors.x.device)
    with torch.no_grad():
        col = column_router(x3, valid)
        pub, privs, stacked, _ = pool._route(x3, valid, col.active_mask)
        ids, weights, _ = pool._private_slots(privs, col.gates.view(w.tokens, -1), w.tokens,
                                              stacked=stacked)
        pub_ids, pub_w = pool._public_slots(pub, w.tokens)
    return ids, weights, pub_ids, pub_w


def bank_call_breakdown(x, grad_out, ids, weights, bank3, iters: int = 5,
                        gemms_only: bool = False) -> dict:
    """Per-kernel timings of one bank call (``ids [T, slots]`` into the stacked bank
    ``bank3 = (w_up, w_gate, w_down)``), each kernel measured alone with HIP events,
    against the roofline that bounds it.  ``gemms_only``: the grouped GEMMs alone."""

    import ctypes  # noqa: F401

    from nestor_amd import ops, probes
    from nestor_amd.dispatch import dispatch_plan

    dev = x.device
    T, d = x.shape
    slots = ids.shape[1]
    w_up, w_gate, w_down = (t.to(torch.bfloat16) for t in bank3)
    banks, _, h = w_up.shape
    rows = T * slots
    ids = ids.reshape(-1).contiguous()
    weights = weights.reshape(-1).to(torch.bfloat16).contiguous()
    out: dict = {}

    def report(name, ms, flops=None, bytes_=None):
        entry = {"ms": round(ms, 4)}
        if flops is not None:
            tf = flops / ms / 1e9
            entry.update(tflops=round(tf, 1), frac_mfma_peak=round(tf / BF16_MFMA_PEAK_TFLOPS, 4))
        if bytes_ is not None:
            gbs = bytes_ / ms / 1e6
            entry.update(gbs=round(gbs, 1), frac_hbm_peak=round(gbs / HBM_PEAK_GBS, 4))
        out[name] = entry

    wall_khz = probes.wall_clock_khz()

    def shader_clock(name, fn):
        """Shader clock the chip holds during this GEMM, from the kernel's own
        counters (cycle counter against the constant-rate wall clock, summed over
        its workgroups), and shader cycles per K step of a workgroup: three launches
        of the measurement library's instrumented build of the same kernel source
        (the product library carries no such hook)."""
        if wall_khz <= 0:
            return
        sink = torch.zeros(64, 4, dtype=torch.int64, device=dev)
        torch.cuda.synchronize()
        with probes.instrumented(sink.data_ptr()):
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
        cycles, ticks, _groups, steps = (int(v) for v in sink.sum(0).tolist())
        if ticks > 0 and steps > 0:
            out[name]["shader_mhz"] = round(cycles / ticks * wall_khz / 1000.0)
            out[name]["cycles_per_k_step"] = round(cycles / steps, 1)

    def gemm(name, fn, flops):
        report(name, _event_ms(fn, iters), flops=flops)
        shader_clock(name, fn)

    plan = dispatch_plan(ids, banks, slots, torch.bfloat16)
    rows_pad = plan.rows_pad
    if not gemms_only:
        ms = _event_ms(lambda: dispatch_plan(ids, banks, slots, torch.bfloat16), iters)
        report("index_build", ms, bytes_=rows * 8 + rows * 8 + 3 * rows_pad * 8 + rows_pad * 2 + banks * 20)

    x_pad = ops.dispatch_rows_fwd(x, plan.pad_token, plan.pad_valid, plan.row_dest, slots)
    if not gemms_only:
        ms = _event_ms(lambda: ops.dispatch_rows_fwd(x, plan.pad_token, plan.pad_valid, plan.row_dest, slots), iters)
        report("dispatch_fwd", ms, bytes_=T * d * 2 + rows * d * 2 + rows * 8)

    up_gate, hidden = ops.upgate_swiglu_fwd(x_pad, w_up, w_gate, plan.tile_table)
    gemm("gemm_upgate_swiglu", lambda: ops.upgate_swiglu_fwd(x_pad, w_up, w_gate, plan.tile_table),
         2.0 * rows * d * 2 * h)
    out["gemm_upgate_swiglu"]["flops_per_launch"] = 2.0 * rows * d * 2 * h

    y_pad = ops.grouped_gemm_nn(hidden, w_down, plan.tile_table)
    gemm("gemm_down", lambda: ops.grouped_gemm_nn(hidden, w_down, plan.tile_table), 2.0 * rows * h * d)

    if not gemms_only:
        o = ops.combine_rows_fwd(y_pad, plan.row_dest, weights, slots, torch.bfloat16, True)
        ms = _event_ms(lambda: ops.combine_rows_fwd(y_pad, plan.row_dest, weights, slots, torch.bfloat16, True), iters)
        report("combine_fwd", ms, bytes_=rows * d * 2 + rows * (8 + 2) + (rows // slots) * d * 2)
        del o
        ms = _event_ms(lambda: ops.combine_rows_bwd(grad_out, y_pad, plan.pad_src_row, plan.pad_valid, weights, slots, True, plan.row_dest), iters)
        report("combine_bwd", ms, bytes_=(rows // slots) * d * 2 + rows * d * 2 + rows * d * 2 + rows * 4)
    gy, _ = ops.combine_rows_bwd(grad_out, y_pad, plan.pad_src_row, plan.pad_valid, weights, slots, True, plan.row_dest)

    gemm("gemm_dgrad_down", lambda: ops.grouped_gemm_nt(gy, w_down, plan.tile_table), 2.0 * rows * h * d)
    gh = ops.grouped_gemm_nt(gy, w_down, plan.tile_table)

    gemm("gemm_wgrad_down", lambda: ops.grouped_gemm_tn(hidden, gy, plan.offs, plan.padded_starts, plan.counts),
         2.0 * rows * h * d)

    if not gemms_only:
        ms = _event_ms(lambda: ops.swiglu_bwd(gh, up_gate, h), iters)
        report("swiglu_bwd", ms, bytes_=rows * h * 2 * (1 + 2 + 2))
    gug = ops.swiglu_bwd(gh, up_gate, h)

    gemm("gemm_dgrad_upgate", lambda: ops.grouped_gemm_nt_upgate(gug, w_up, w_gate, plan.tile_table),
         2.0 * rows * d * 2 * h)
    gx_pad = ops.grouped_gemm_nt_upgate(gug, w_up, w_gate, plan.tile_table)

    gemm("gemm_wgrad_upgate_pair",
         lambda: ops.grouped_gemm_tn_pair(x_pad, gug, plan.offs, plan.padded_starts, plan.counts),
         2.0 * rows * d * 2 * h)
    if gemms_only:
        return out

    ms = _event_ms(lambda: ops.dispatch_rows_bwd(gx_pad, plan.row_dest, T, slots, torch.bfloat16), iters)
    report("dispatch_bwd", ms, bytes_=rows * d * 2 + T * d * 2)

    # biased banks: the bias gradient as a segmented column sum over the padded rows
    ms = _event_ms(lambda: ops.segment_colsum(gh, None, plan.padded_starts, plan.counts), iters)
    report("bias_grad_colsum", ms, bytes_=rows * h * 2)
    out["_scratch"] = gx_pad  # reused by the caller for the pool epilogue rows
    return out


def kernel_breakdown(w, tensors, routed, iters: int = 5) -> dict:
    """Per-kernel timings of one private-bank call (the larger of the two) on the
    workload's routed ids, plus the pool's epilogue kernels."""

    from nestor_amd import ops

    dev = tensors.x.device
    T, d = w.tokens, w.d_model
    x, go = tensors.x, tensors.grad_out
    out = bank_call_breakdown(x, go, routed[0], routed[1], tensors.priv, iters)
    out["gemm_upgate_swiglu"]["kernel"] = UPGATE_KERNEL_NAME
    gx_pad = out.pop("_scratch")

    def report(name, ms, bytes_):
        gbs = bytes_ / ms / 1e6
        out[name] = {"ms": round(ms, 4), "gbs": round(gbs, 1), "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}

    # pool epilogues: the summed layout's path mix and the column layout's scatter
    g = torch.Generator(device=dev).manual_seed(1)
    alpha = torch.softmax(torch.randn(T, 2, generator=g, device=dev), -1).to(torch.bfloat16)
    pub, priv = x, gx_pad[:T]
    ms = _event_ms(lambda: ops.path_mix_fwd(pub, priv, alpha), iters)
    report("path_mix_fwd", ms, bytes_=3 * T * d * 2)
    ms = _event_ms(lambda: ops.path_mix_bwd(go, pub, priv, alpha), iters)
    report("path_mix_bwd", ms, bytes_=5 * T * d * 2)
    k_a = w.k_columns
    per_slot = gx_pad[: T * k_a].view(T, k_a, d)
    columns = torch.rand(T, w.columns, generator=g, device=dev).topk(k_a, -1).indices
    ms = _event_ms(lambda: ops.path_scale_fwd(per_slot, alpha, 1, columns, w.columns), iters)
    report("column_scatter_fwd", ms, bytes_=T * k_a * d * 2 + T * w.columns * d * 2)
    g_cols = ops.path_scale_fwd(per_slot, alpha, 1, columns, w.columns)
    ms = _event_ms(lambda: ops.path_scale_bwd(g_cols, per_slot, alpha, 1, columns), iters)
    report("column_scatter_bwd", ms, bytes_=3 * T * k_a * d * 2)
    return out


def timed_steps(w, column_router, pool, x, grad_out, steps: int, warmup: int, autocast: bool) -> float:
    """ms per step of the whole path (forward + backward), host clock around ``steps``
    steps bracketed by device synchronisations."""

    from nestor_amd.workloads import expert_mlp_step

    params = list(column_router.parameters()) + list(pool.parameters())

    def step():
        for p in params:
            p.grad = None
        x.grad = None
        with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
            expert_mlp_step(w, column_router, pool, x, grad_out)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    for p in params:
        p.grad = None
    x.grad = None
    return ms


def graphed_steps(w, column_router, pool, x, grad_out, steps: int) -> float:
    """ms per step of the same pass replayed as one HIP graph (``GraphedStep``): what the
    step costs once the host's ~150 launches per step are out of the way."""

    from nestor_amd.workloads import GraphedStep

    params = list(column_router.parameters()) + list(pool.parameters())
    graphed = GraphedStep(w, column_router, pool, x, grad_out)
    graphed()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        graphed()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    del graphed
    for p in params:
        p.grad = None
    return ms


def extra_shapes(dev, seed: int) -> dict:
    """The path at the reference's production widths (registered ``nestor_*`` arms: d that
    is no power of two, private widths of 160-424, 6-16 slots per token, 120 private
    experts): ms per step and the grouped GEMMs of both bank calls against the MFMA peak.
    Not the headline: BASELINE's configuration is ``mlp_1b``."""

    from nestor_amd.workloads import WORKLOADS, build_pool, make_tensors

    out = {}
    for name in ("nestor_1b_block0", "nestor_1b_block6", "nestor_200m_block0"):
        w = WORKLOADS[name]
        t = make_tensors(w, seed, dev)
        column_router, pool = build_pool(w, t)
        x = t.x.clone().requires_grad_(True)
        ms = timed_steps(w, column_router, pool, x, t.grad_out, 5, 2, False)
        ms_graph = graphed_steps(w, column_router, pool, x, t.grad_out, 10)
        flops = w.gemm_flops()
        routed = routed_slots(w, t, column_router, pool)
        entry = {
            "shape": f"T={w.tokens} d={w.d_model} private {w.columns}x{w.private} h={w.hidden} "
                     f"top-{w.k_columns} columns x top-{w.k_private} = {w.k_columns * w.k_private} slots; "
                     f"public {w.public} h={w.h_public} top-{w.k_public}",
            "ms_per_step": round(ms, 3),
            "ms_per_step_hip_graph": round(ms_graph, 3),
            "tokens_per_s": round(w.tokens / ms * 1e3, 1),
            "tokens_per_s_hip_graph": round(w.tokens / ms_graph * 1e3, 1),
            "expert_gemm_tflops": round(flops / ms / 1e9, 1),
            "expert_gemm_frac_mfma_peak": round(flops / ms / 1e9 / BF16_MFMA_PEAK_TFLOPS, 4),
        }
        for call, ids, wts, bank3 in (("private", routed[0], routed[1], t.priv), ("public", routed[2], routed[3], t.pub)):
            rows = bank_call_breakdown(t.x, t.grad_out, ids, wts, bank3, 5, gemms_only=True)
            entry[f"{call}_gemms"] = {k: {"ms": v["ms"], "frac_mfma_peak": v["frac_mfma_peak"]} for k, v in rows.items()}
        out[name] = entry
        del t, pool, column_router, x
        torch.cuda.empty_cache()
    return out


def mfma_clock_probe(dev, iters: int = 100000) -> dict:
    """What the matrix cores sustain with no memory traffic at all (four wavefronts per
    CU issuing independent 32x32x16 bf16 MFMAs back to back), and the shader clock the
    chip holds meanwhile: with constant operands, and with random ones, whose power
    draw is that of real data.  The second is the ceiling of any bf16 GEMM here."""

    import ctypes

    from nestor_amd import probes as _lib

    wall_khz = _lib.wall_clock_khz()
    out = {"instruction": "v_mfma_f32_32x32x16_bf16, 16 independent accumulator tiles per wavefront"}
    counters = torch.zeros(4, dtype=torch.int64, device=dev)
    for name, random_operands in (("constant_operands", 0), ("random_operands", 1)):
        def run():
            _lib.call("nestor_hip_mfma_clock_probe", random_operands, iters,
                      ctypes.c_void_p(counters.data_ptr()), torch.cuda.current_stream().cuda_stream)
        ms = _event_ms(run, 3)
        cycles, ticks, instructions, _ = (int(v) for v in counters.tolist())
        tf = instructions * 2.0 * 32 * 32 * 16 / ms / 1e9
        out[name] = {"tflops": round(tf, 1), "frac_mfma_peak": round(tf / BF16_MFMA_PEAK_TFLOPS, 4),
                     "shader_mhz": round(cycles / ticks * wall_khz / 1000.0) if ticks > 0 and wall_khz > 0 else None}
    # the same stream (random operands) with a K step's other instructions between the MFMAs
    # and nothing else: no barriers, no waiting for data, no epilogue, every transfer an L2 hit
    region = 1 << 20
    src = torch.zeros(8 * region, dtype=torch.uint8, device=dev)
    out["main_loop_only"] = {
        "note": "the kernels' main loop and nothing around it (no barriers, data waits, epilogue, tile "
                "switches; transfers hit L2): per K step of 32 MFMAs and wavefront, 1 KiB fragment reads "
                "from LDS / 1 KiB LDS-DMA transfers; 16/8 = the 256x256x32 tile, 16/10 = the 128x512x32 one"}
    rounds = iters // 10
    for reads, transfers in ((16, 0), (0, 8), (16, 8), (16, 10), (16, 12)):
        def run():
            _lib.call("nestor_hip_mfma_mix_probe", reads, transfers, rounds,
                      ctypes.c_void_p(src.data_ptr()), src.numel(), region,
                      ctypes.c_void_p(counters.data_ptr()),
                      torch.cuda.current_stream().cuda_stream)
        ms = _event_ms(run, 3)
        cycles, ticks, instructions, _ = (int(v) for v in counters.tolist())
        tf = instructions * 2.0 * 32 * 32 * 16 / ms / 1e9
        out["main_loop_only"][f"reads{reads}_transfers{transfers}"] = {
            "tflops": round(tf, 1), "frac_mfma_peak": round(tf / BF16_MFMA_PEAK_TFLOPS, 4),
            "cycles_per_k_step": round(cycles / rounds, 1),
            "shader_mhz": round(cycles / ticks * wall_khz / 1000.0) if ticks > 0 and wall_khz > 0 else None}
    return out


def traffic_probe(w, tensors, routed, uniform: bool = False) -> None:
    """Yardsticks of known size for the HBM counters, then the private bank's up|gate
    kernel on the workload's routing.  Run under `rocprofv3 --pmc FETCH_SIZE` and again
    under `--pmc WRITE_SIZE`; each launch below is one dispatch in the counter output:

    1. ``dma_stream_probe_kernel`` x4 over a 2 GiB buffer (larger than every cache), each
       byte fetched once: 512-byte row pieces walking down the rows (how the kernel
       fetches its weight tiles), 64-byte pieces walking along the rows (how the
       input-gradient kernels fetch), 1 KiB contiguous, and 128-byte pieces;
    2. torch's elementwise copy of the 128 MiB activations (reads and writes 128 MiB);
    3. ``dispatch_fwd_kernel`` (16-byte lanes, 4 KiB rows: the store shape of the GEMM
       epilogues) writing ``rows_pad * d * 2`` bytes;
    4. ``grouped_gemm_dma_kernel<..., kNNUpGate>`` twice.

    ``uniform``: every bank gets the same number of rows (ids in round-robin order) instead of
    the routers' choice: whole 128-row tiles, four per bank, so that a tile order which
    keeps a bank's row tiles on one XCD is exactly aligned."""

    import ctypes

    from nestor_amd import ops
    from nestor_amd import probes as _lib
    from nestor_amd.dispatch import dispatch_plan

    dev = tensors.x.device
    slots = w.k_columns * w.k_private
    banks = w.columns * w.private
    ids = routed[0].reshape(-1).contiguous()
    if uniform:
        ids = (torch.arange(ids.numel(), device=dev, dtype=ids.dtype) % banks).contiguous()
    plan = dispatch_plan(ids, banks, slots, torch.bfloat16)
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    buf = torch.empty(1 << 30, dtype=torch.bfloat16, device=dev).normal_()   # 2 GiB
    row_bytes = 8192                                                       # a [K, 4096] bf16 weight row
    rows = buf.numel() * 2 // row_bytes
    torch.cuda.synchronize()
    for piece, along_rows in ((512, 1), (64, 0), (1024, 1), (128, 0)):
        _lib.call("nestor_hip_dma_stream_probe", ctypes.c_void_p(buf.data_ptr()), buf.numel() * 2, rows, row_bytes,
                  piece, along_rows, stream)
        torch.cuda.synchronize()
    del buf
    dst = torch.empty_like(tensors.x)
    dst.copy_(tensors.x)
    torch.cuda.synchronize()
    x_pad = ops.dispatch_rows_fwd(tensors.x, plan.pad_token, plan.pad_valid)
    torch.cuda.synchronize()
    w_up, w_gate, _ = (t.to(torch.bfloat16) for t in tensors.priv)
    for _ in range(2):
        ops.upgate_swiglu_fwd(x_pad, w_up, w_gate, plan.tile_table)
    torch.cuda.synchronize()
    _log(f"traffic probe done: DMA probes over {rows * row_bytes} bytes, copy of "
         f"{tensors.x.numel() * 2} bytes, dispatch writing {plan.rows_pad * w.d_model * 2} bytes, "
         f"rows_pad={plan.rows_pad}")


def _log(msg: str) -> None:
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def cpu_baseline(w, seed: int, target_seconds: float = 15.0) -> dict:
    """The reference's CPU eager path (per-expert sparse loop under bf16 autocast,
    forward + backward) on a bounded slice of the same workload: 1/16 of the
    tokens over 1/16 of the banks, so every expert sees as many rows as in the
    full workload and the work per token is unchanged."""

    from oracle import bank as obank
    from oracle import router as orouter

    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    shrink = 16
    columns = max(w.k_columns, w.columns // shrink)
    public = max(w.k_public, w.public // shrink)
    sample = max(64, w.tokens * columns // w.columns)
    d, h = w.d_model, w.hidden
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(sample, d, generator=g).bfloat16().float().requires_grad_(True)
    go = torch.randn(sample, d, generator=g)
    ones = torch.ones(sample, dtype=torch.bool)
    col = orouter.route(torch.randn(sample, columns, generator=g), torch.zeros(columns),
                        w.k_columns, "renorm", ones)
    pub = orouter.route(torch.randn(sample, public, generator=g), torch.zeros(public),
                        w.k_public, "renorm", ones)
    priv = orouter.route(torch.randn(sample, columns, w.private, generator=g),
                         torch.zeros(columns, w.private), w.k_private, "switch",
                         torch.ones(sample, columns, dtype=torch.bool))
    ids, wts, _ = orouter.private_slots(priv.gates, priv.topk_indices, col.gates, w.k_columns)
    pub_ids, pub_w = orouter.public_slots(pub.gates, pub.topk_indices)
    banks = []
    for n in (public, columns * w.private):
        banks.append(tuple(
            (torch.randn(n, a, b, generator=g) * w.weight_std).requires_grad_(True)
            for a, b in ((d, h), (d, h), (h, d))
        ))

    def step():
        for bank in banks:
            for t in bank:
                t.grad = None
        x.grad = None
        out = torch.zeros(sample, d)
        with torch.autocast("cpu", dtype=torch.bfloat16):
            obank.accumulate_sparse_expert_bank(
                out, x, *banks[0], obank.dense_weights(pub_ids, pub_w, public))
            obank.accumulate_sparse_expert_bank(
                out, x, *banks[1], obank.dense_weights(ids, wts, columns * w.private))
        out.backward(go)

    _log(f"cpu baseline: {sample} tokens, {public}+{columns}x{w.private} experts, {cores} threads")
    step()  # warm-up
    times = []
    t_end = time.perf_counter() + target_seconds
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 10):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
        _log(f"cpu baseline pass {len(times)}: {times[-1]:.2f} s")
    med = statistics.median(times)
    return {
        "value": round(sample / med, 1),
        "unit": "tokens/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{sample} of {w.tokens} tokens over {public}+{columns}x{w.private} of "
                  f"{w.public}+{w.columns}x{w.private} experts (same rows per expert as the full "
                  f"workload), fwd+bwd, per-expert sparse loop under cpu bf16 autocast, "
                  f"median of {len(times)} passes",
    }


def fp8_probe(w, tensors, column_router, pool, iters: int = 10) -> dict:
    """The inference regime: the workload's two banks in e4m3 with per-channel scales,
    forward only, at 64 / 256 / 1024 tokens routed by the workload's own routers (top-2
    columns -> top-1 private, top-1 public).  Most experts see 0-8 rows, so a call is
    bound by streaming the weights of the experts that got a row: bytes = 3*d*h per such
    expert (1 B per weight).  Timed over both bank calls: index build, dispatch, the
    weight-streaming GEMMs and the combine.  ``ms`` is the serving form (``Fp8PoolForward``:
    the public call on a side stream, the unit replayed as a HIP graph whose input
    buffers already hold the routed ids and weights); ``ms_with_input_copies`` the same
    with five copies into those buffers in front of each replay; ``ms_serial_launches``
    the launches issued one after the other."""

    from nestor_amd import fp8, ops
    from nestor_amd.dispatch import dispatch_plan
    from nestor_amd.expert_kernels import dispatch_rows

    dev = tensors.x.device
    d, h = w.d_model, w.hidden
    banks = {"public": fp8.quantize_bank(*tensors.pub), "private": fp8.quantize_bank(*tensors.priv)}
    out = {}
    units: dict = {}
    for tokens in (64, 256, 1024):
        x = tensors.x[:tokens].contiguous()
        x3 = x.view(1, tokens, d)
        valid = torch.ones(1, tokens, dtype=torch.bool, device=dev)
        with torch.no_grad():
            col = column_router(x3, valid)
            pub, privs, stacked, _ = pool._route(x3, valid, col.active_mask)
            priv_ids, priv_w, _ = pool._private_slots(privs, col.gates.view(tokens, -1), tokens,
                                                      stacked=stacked)
            pub_ids, pub_w = pool._public_slots(pub, tokens)
        calls = (("public", pub_ids, pub_w, 1), ("private", priv_ids, priv_w, priv_ids.shape[1]))

        def run():
            return [fp8.grouped_expert_combine_fp8(x, banks[n], i, wt, grp) for n, i, wt, grp in calls]

        ms_serial = _event_ms(run, iters)
        unit = units.setdefault("graph", fp8.Fp8PoolForward(
            banks["public"], banks["private"], 1, priv_ids.shape[1], graph=True))
        ms_copies = _event_ms(lambda: unit(x, pub_ids, pub_w, priv_ids, priv_w), iters)
        # the serving loop proper: the routers' results already sit in the graph's inputs
        static, _, replay = unit.bind(x, pub_ids, pub_w, priv_ids, priv_w)
        for dst, src in zip(static, (x, pub_ids, pub_w, priv_ids, priv_w)):
            dst.copy_(src)
        ms = _event_ms(replay, iters)
        # The four weight-streaming launches of the unit, each timed alone on its routed
        # rows (bytes = the e4m3 weights of the experts with rows that the launch reads).
        streams = {}
        for name, ids, _, _ in calls:
            bank = banks[name]
            slots = ids.shape[1]
            with torch.no_grad():
                plan = dispatch_plan(ids.reshape(-1), bank.w_up.shape[0], slots, torch.bfloat16)
                x_pad = dispatch_rows(x, plan.pad_token, plan.pad_valid, plan.row_dest, slots, torch.bfloat16)
                hid = ops.grouped_gemm_fp8w_upgate_swiglu(x_pad, bank.w_up, bank.w_gate, bank.s_up, bank.s_gate,
                                                          plan.tile_table, bank.tiled)
                n_live = int(torch.unique(ids).numel())
                t_up = _event_ms(lambda: ops.grouped_gemm_fp8w_upgate_swiglu(
                    x_pad, bank.w_up, bank.w_gate, bank.s_up, bank.s_gate, plan.tile_table, bank.tiled), iters)
                t_dn = _event_ms(lambda: ops.grouped_gemm_fp8w_nn(
                    hid, bank.w_down, bank.s_down, plan.tile_table, bank.tiled), iters)
            streams[f"{name}_upgate"] = {"us": round(t_up * 1e3, 1), "gbs": round(n_live * 2 * d * h / t_up / 1e6, 1)}
            streams[f"{name}_down"] = {"us": round(t_dn * 1e3, 1), "gbs": round(n_live * d * h / t_dn / 1e6, 1)}
        live = sum(int(torch.unique(i).numel()) for _, i, _, _ in calls)
        nbytes = live * 3 * d * h
        flops = 2.0 * 3 * d * h * sum(i.numel() for _, i, _, _ in calls)
        out[str(tokens)] = {
            "ms": round(ms, 4), "ms_with_input_copies": round(ms_copies, 4),
            "ms_serial_launches": round(ms_serial, 4),
            "experts_with_rows": live, "weight_bytes": nbytes,
            "gbs": round(nbytes / ms / 1e6, 1), "frac_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4),
            "tokens_per_s": round(tokens / ms * 1e3, 1), "tflops": round(flops / ms / 1e9, 2),
            "stream_launches_alone": streams,
        }
    return out


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="mlp_1b")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--weights", choices=("bf16", "fp32"), default="bf16",
                    help="bf16: bank tensors are bf16 leaves (the bench's headline flow); fp32: fp32 "
                         "owners under bf16 autocast, the weights narrowed on the way into the GEMMs")
    ap.add_argument("--no-shadow", action="store_true",
                    help="with --weights fp32: narrow the owners on every bank call instead of "
                         "keeping the persistent bf16 copy")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-breakdown", action="store_true")
    ap.add_argument("--no-extra", action="store_true",
                    help="skip the fp32-owner step and the production-shape figures")
    ap.add_argument("--no-fp8", action="store_true",
                    help="skip the e4m3 inference-regime figures (64 / 256 / 1024 tokens)")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="launch yardsticks of known size (LDS-DMA streams, a copy, a row kernel) and "
                         "the dominant kernel twice, then exit: the command to run under "
                         "`rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE`")
    ap.add_argument("--traffic-uniform", action="store_true",
                    help="with --traffic-probe: the same number of rows for every bank instead of the "
                         "routers' choice")
    ap.add_argument("--fp8-probe", action="store_true",
                    help="time the e4m3-weight forward at 64/256/1024 tokens and print one JSON "
                         "line (HBM GB/s over the weights of the experts that received a row)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU's share of the expert MLP: run it with --gpus 1 "
                 "(the path shards by tokens; there is no multi-GPU leg in this build)")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (the HIP kernels have no CPU fallback)")

    from nestor_amd import _lib
    from nestor_amd.workloads import WORKLOADS, build_pool, make_tensors

    _lib.load()
    _log("library loaded; building workload")
    w = WORKLOADS[args.workload]
    dev = torch.device("cuda:0")
    fp32_owners = args.weights == "fp32"
    tensors = make_tensors(w, args.seed, dev, torch.float32 if fp32_owners else torch.bfloat16)
    column_router, pool = build_pool(w, tensors)
    if fp32_owners and not args.no_shadow:
        pool.enable_bf16_shadow()
    with torch.autocast("cuda", dtype=torch.bfloat16, enabled=fp32_owners):
        routed = routed_slots(w, tensors, column_router, pool)
    if args.traffic_probe:
        traffic_probe(w, tensors, routed, args.traffic_uniform)
        return
    if args.fp8_probe:
        print(json.dumps({"workload": f"{w.name}, e4m3 weights, forward only",
                          "unit": "GB/s of weight bytes streamed",
                          "tokens": fp8_probe(w, tensors, column_router, pool)}))
        return
    x = tensors.x.clone().requires_grad_(True)
    grad_out = tensors.grad_out if w.backward else None
    _log("workload resident; warm-up and timing")
    ms_per_step = timed_steps(w, column_router, pool, x, grad_out, args.steps, args.warmup, fp32_owners)
    tokens_per_s = w.tokens / ms_per_step * 1e3
    flops = w.gemm_flops()
    step_tflops = flops / (ms_per_step * 1e-3) / 1e12

    _log(f"{ms_per_step:.3f} ms/step; per-kernel breakdown")
    breakdown = {} if args.no_breakdown else kernel_breakdown(w, tensors, routed)
    dom = breakdown.get("gemm_upgate_swiglu")
    roofline = None
    if dom:
        roofline = {
            "bound": "mfma",
            "kernel": dom.pop("kernel"),
            "achieved": dom["tflops"],
            "peak": BF16_MFMA_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": dom["frac_mfma_peak"],
            # HBM bytes per launch of this kernel: FETCH_SIZE + WRITE_SIZE from two
            # `rocprofv3 --pmc` runs of `bench.py --traffic-probe`, each scaled by the same
            # counter's reading for a stream of known size with the kernel's access pattern.
            "traffic": measured_traffic_bytes() if w.name == "mlp_1b" else None,
        }
    result = {
        "metric": "expert-MLP fwd+bwd tokens/s @1b shape, 1 GPU; % bf16 MFMA / HBM peak",
        "value": round(tokens_per_s, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"{w.name}: T={w.tokens} d={w.d_model} h={w.hidden} experts={w.public}+"
                        f"{w.columns}x{w.private}, top-{w.k_columns} columns -> top-{w.k_private} "
                        f"private + top-{w.k_public} public, fwd{'+bwd' if w.backward else ''}",
            "seed": args.seed,
            "weights": "bf16 leaves" if not fp32_owners else (
                "fp32 owners under bf16 autocast" +
                (", narrowed per call" if args.no_shadow else ", persistent bf16 copy")),
        },
        "expert_gemm_tflops": round(step_tflops, 1),
        "expert_gemm_frac_mfma_peak": round(step_tflops / BF16_MFMA_PEAK_TFLOPS, 4),
        "gemm_flops_per_step": flops,
        "roofline": roofline,
        "kernels": breakdown,
        "kernels_note": "one private-bank call (slots=2, 128 banks) on the workload's routed ids; "
                        "each kernel timed alone over 5 launches with HIP events; shader_mhz = the "
                        "kernel's own cycle counter against the constant-rate wall clock, in three "
                        "further launches (the published peak assumes 2400 MHz)",
    }
    if not args.no_breakdown:
        # the public bank call's GEMMs (slots = 1, 16 banks of ~2048 rows) beside the private ones
        result["kernels_public"] = bank_call_breakdown(
            tensors.x, tensors.grad_out, routed[2], routed[3], tensors.pub, 5, gemms_only=True)
        result["mfma_clock_probe"] = mfma_clock_probe(dev)
    if not args.no_extra and not fp32_owners:
        # the same step replayed as one HIP graph (what is left of the step once the host's
        # launches are out of the way; the headline above is launched from the host)
        try:
            result["ms_per_step_hip_graph"] = round(
                graphed_steps(w, column_router, pool, x, tensors.grad_out, args.steps), 3)
        except Exception as exc:  # noqa: BLE001 -- an extra figure must not cost the headline
            result["ms_per_step_hip_graph"] = None
            _log(f"graph replay of the step failed: {exc}")
        torch.cuda.empty_cache()
    if not args.no_extra and w.name == "mlp_1b" and not fp32_owners:
        # the production dtype flow: fp32 owners under bf16 autocast, the GEMMs reading a
        # persistent bf16 copy and the weight gradient written as fp32 into the owners' .grad
        _log("fp32-owner flow")
        t32 = make_tensors(w, args.seed, dev, torch.float32)
        router32, pool32 = build_pool(w, t32)
        pool32.enable_bf16_shadow()
        x32 = t32.x.clone().requires_grad_(True)
        result["fp32_owner_ms_per_step"] = round(
            timed_steps(w, router32, pool32, x32, t32.grad_out, 5, 2, True), 3)
        del t32, router32, pool32, x32
        torch.cuda.empty_cache()
        _log("production shapes")
        result["extra_shapes"] = extra_shapes(dev, args.seed)
    if not args.no_fp8 and w.name == "mlp_1b" and not fp32_owners:
        _log("e4m3 inference regime")
        del x
        result["fp8_inference"] = fp8_probe(w, tensors, column_router, pool)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(w, args.seed)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
