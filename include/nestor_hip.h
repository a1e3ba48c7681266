/*
 * nestor_hip.h -- C ABI of libnestor_hip.so, the gfx950 (MI355X) kernels behind
 * Nestor's routed hybrid expert-MLP path.
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer unless the name ends in _host.
 *   - Every entry point returns 0 on success or a negative NESTOR_HIP_E* code;
 *     nothing throws across the boundary and nothing allocates: outputs and
 *     workspaces are caller-owned.
 *   - `stream` is a hipStream_t passed as void*; work is enqueued, never
 *     synchronised.  No entry point reads device memory back to the host.
 *   - Index maps are int64 and segment ends (`offs`) int32, the widths the
 *     reference plan uses (nestor/backbones/grouped_mm.py:197-219,272-277).
 *   - Row-major tensors; a "bank" is one expert of a stacked weight tensor.
 *   - Index tensors are read on the device and cannot be checked by the host
 *     side of a call.  Bank ids, top-k choices and column selections are
 *     clamped into their range by the kernels that read them (a bad value
 *     gives a wrong result, not an access outside the tensors); row maps
 *     (row_dest, pad_token, slot_rows, gid, ...) are taken as produced by
 *     nestor_hip_index_build / nestor_hip_build_dispatch_maps and must index
 *     inside the tensors they address.
 *
 *   - One GPU per process: the library caches per-process facts on first use
 *     (kernel attributes such as the dynamic LDS limit, the CU count of the
 *     device, the values of its NESTOR_HIP_* environment switches).  A process
 *     that drives several different GPUs must not share one copy of the library
 *     between them; nestor_hip_index_build_static alone keeps per-device state.
 *
 * Each declaration cites the reference interface it stands in for (paths are
 * relative to the reference checkout).
 */
#ifndef NESTOR_HIP_H_
#define NESTOR_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NESTOR_HIP_ABI_VERSION 16

/* status codes */
#define NESTOR_HIP_OK 0
#define NESTOR_HIP_EINVAL (-22)   /* bad size / alignment / dtype code / null pointer */
#define NESTOR_HIP_ENOSPC (-28)   /* workspace too small */
#define NESTOR_HIP_ELAUNCH (-5)   /* the HIP runtime refused the launch */
#define NESTOR_HIP_ERANGE (-34)   /* size beyond what the kernels support */

/* element type codes */
#define NESTOR_HIP_F32 0
#define NESTOR_HIP_BF16 1

/* Row alignment of every expert segment in the padded layout
 * (GROUPED_MM_ALIGN, nestor/backbones/grouped_mm.py:61). */
#define NESTOR_HIP_ROW_ALIGN 16

/* Rows covered by one tile of the device-side tile table (see
 * nestor_hip_index_build / nestor_hip_tile_schedule). */
#define NESTOR_HIP_TILE_M 128

int nestor_hip_abi_version(void);
const char* nestor_hip_strerror(int code);

/* ------------------------------------------------------------------------
 * Dispatch index build  (nestor/backbones/grouped_mm.py:222-321, _dispatch_plan)
 *
 * From the flat token-major bank ids of the routed rows, builds in three
 * launches what the reference builds with argsort + scatter_add + two cumsums
 * + the map cascade: the stable sort permutation `order`, per-bank `counts`,
 * `raw_starts` / `padded_starts` (exclusive cumsums of counts and of counts
 * rounded up to 16), `offs` (int32 segment ends, last one == rows_pad) and the
 * five maps row_dest / pad_token / pad_src_row / eid_pad / pad_valid with slack
 * entries zero.  rows_pad must equal ceil16(rows) + 16 * num_banks.
 *
 * capacity <= 0: dropless (the reference's behaviour).  capacity > 0: a row
 * whose stable rank inside its bank is >= capacity gets no padded slot; its
 * row_dest is rows_pad - 1 (always a slack row) and row_kept (optional,
 * uint8[rows]) is 0.  counts / raw_starts / order always describe ALL rows;
 * padded_starts / offs describe the kept rows.
 *
 * tile_table (int32[nestor_hip_tile_table_ints(rows_pad, num_banks)]) receives the
 * tile tables the grouped GEMMs walk.  A table is bank[cap] | row0[cap] |
 * nrows[cap] | count: tile t covers rows [row0[t], row0[t] + nrows[t]) of bank[t],
 * never crossing a segment end; bank == -1 marks a tile that lies wholly in the
 * slack tail behind the last segment (outputs are zero-filled, no product is
 * formed).  Three tables sit back to back, each covering every row exactly once:
 * (1) every segment in tiles of up to NESTOR_HIP_TILE_M = 128 rows, cap =
 * max_tiles; (2) every segment in the fewest tiles of at most five 32-row blocks,
 * the segment's blocks dealt evenly over them (a segment of 530 rows becomes tiles
 * of 4, 4, 4 and 5 blocks instead of four full tiles and a fifth of 18 rows), cap =
 * max_tiles; (3) the same with at most ten blocks per tile, cap = rows_pad / 256 +
 * num_banks + 2.  The slack tail is cut at 128 / 160 / 320 rows.  max_tiles must
 * equal nestor_hip_max_tiles(rows_pad, num_banks).
 * ---------------------------------------------------------------------- */
size_t nestor_hip_index_build_workspace_bytes(int64_t rows, int32_t num_banks);
int64_t nestor_hip_max_tiles(int64_t rows_pad, int32_t num_banks);
int64_t nestor_hip_tile_table_ints(int64_t rows_pad, int32_t num_banks);
int nestor_hip_index_build(
    const int64_t* expert_ids, int64_t rows, int32_t num_banks, int32_t slots,
    int64_t rows_pad, int64_t capacity, int32_t valid_dtype,
    int64_t* order, int64_t* counts, int64_t* raw_starts, int64_t* padded_starts,
    int32_t* offs,
    int64_t* row_dest, int64_t* pad_token, int64_t* pad_src_row, int64_t* eid_pad,
    void* pad_valid, uint8_t* row_kept /* nullable */,
    int32_t* tile_table, int64_t max_tiles,
    void* workspace, size_t workspace_bytes, void* stream);

/* nestor_hip_index_build for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  It has no counterpart in the reference.  Same arguments and
 * results, bit for bit, minus the workspace: the per-chunk histograms live in a
 * fixed array inside the library (1 MiB per GPU the library runs on, held until
 * the process ends; nestor_hip_index_build_static_capacity_bytes() returns its
 * size).  A call whose nestor_hip_index_build_workspace_bytes(rows, num_banks)
 * exceeds that size is rejected with NESTOR_HIP_ERANGE (with the chunking used
 * here that means num_banks > 2048 once rows >= 32768).  The call allocates and
 * frees nothing; its first use on a device looks the array's address up
 * (hipGetSymbolAddress), so make one call per device outside any graph capture
 * first.  All calls on one GPU share the array: calls that overlap in time on
 * the same GPU (different streams, or threads) race; calls in stream order are
 * fine, and nothing has to be cleared between them. */
size_t nestor_hip_index_build_static_capacity_bytes(void);
int nestor_hip_index_build_static(
    const int64_t* expert_ids, int64_t rows, int32_t num_banks, int32_t slots,
    int64_t rows_pad, int64_t capacity, int32_t valid_dtype,
    int64_t* order, int64_t* counts, int64_t* raw_starts, int64_t* padded_starts,
    int32_t* offs,
    int64_t* row_dest, int64_t* pad_token, int64_t* pad_src_row, int64_t* eid_pad,
    void* pad_valid, uint8_t* row_kept /* nullable */,
    int32_t* tile_table, int64_t max_tiles, void* stream);

/* The reference's fused map kernel boundary, argument for argument
 * (nestor/backbones/triton_dispatch.py:109-160, build_dispatch_maps): order,
 * padded_starts and raw_starts come from the caller.  Slack entries of the
 * four rows_pad-long maps are written as zero by this call (the reference
 * zero-initialises them in its wrapper). */
int nestor_hip_build_dispatch_maps(
    const int64_t* expert_ids, const int64_t* order,
    const int64_t* padded_starts, const int64_t* raw_starts,
    int64_t rows, int32_t num_banks, int32_t slots, int64_t rows_pad,
    int32_t valid_dtype,
    int64_t* row_dest, int64_t* pad_token, int64_t* pad_src_row, int64_t* eid_pad,
    void* pad_valid, void* stream);

/* The tile tables from segment ends alone, for callers that only hold `offs`
 * (segment_mm's contract, nestor/backbones/grouped_mm.py:83-104).  Every row
 * up to offs[num_banks-1] belongs to a bank, so no tile is marked -1.  Same
 * buffer layout and sizes as for nestor_hip_index_build. */
int nestor_hip_tile_schedule(
    const int32_t* offs, int32_t num_banks, int64_t rows_pad,
    int32_t* tile_table, int64_t max_tiles, void* stream);

/* ------------------------------------------------------------------------
 * Row moves
 * ---------------------------------------------------------------------- */

/* x_pad[p,:] = pad_valid[p] ? bf16(x[pad_token[p],:]) : 0
 * (nestor/backbones/triton_expert.py:509-539 dispatch_rows; kernel
 * nestor/backbones/triton_packed.py:113-139).  dim % 8 == 0.
 * row_dest (nullable, [num_tokens*slots], the inverse map dispatch_rows also
 * receives) selects the source-major kernel for bf16 x: every token is read once
 * and written to the rows of its assignments; same result. */
int nestor_hip_dispatch_rows_fwd(
    const void* x, int32_t x_dtype, const int64_t* pad_token,
    const void* pad_valid, int32_t valid_dtype,
    void* x_pad /* bf16 [rows_pad, dim] */, int64_t rows_pad, int64_t dim,
    const int64_t* row_dest, int64_t num_tokens, int32_t slots,
    void* stream);

/* grad_x[t,:] = sum_{j<slots} grad_pad[row_dest[t*slots+j],:], fp32 sum,
 * written in x's dtype (nestor/backbones/triton_packed.py:142-169,444-463). */
int nestor_hip_dispatch_rows_bwd(
    const void* grad_pad /* bf16 [rows_pad, dim] */, const int64_t* row_dest,
    void* grad_x, int32_t x_dtype, int64_t num_tokens, int32_t slots, int64_t dim,
    void* stream);

/* out = bf16( f32(bf16(silu_f32(gate))) * f32(up) ), two roundings
 * (nestor/backbones/triton_expert.py:149-176).  up/gate rows have stride
 * `stride_in` elements, out rows `stride_out`; the fused up|gate layout is
 * gate = up + hidden, stride_in = 2*hidden (:391-402).  hidden % 8 == 0. */
int nestor_hip_swiglu_fwd(
    const void* up, const void* gate, void* out,
    int64_t rows, int64_t hidden, int64_t stride_in, int64_t stride_out,
    void* stream);

/* grad_up = bf16(go*act), grad_gate = bf16(f32(bf16(go*up)) * s*(1+g*(1-s)))
 * (nestor/backbones/triton_expert.py:179-217). */
int nestor_hip_swiglu_bwd(
    const void* grad_out, const void* up, const void* gate,
    void* grad_up, void* grad_gate,
    int64_t rows, int64_t hidden, int64_t stride_in, int64_t stride_out,
    int64_t stride_g, void* stream);

/* out[r, 0:h] = bf16(a[r,:]), out[r, h:2h] = bf16(b[r,:])
 * (nestor/backbones/triton_expert.py:220-243,542-559 cat_cast). */
int nestor_hip_cat_cast_fwd(
    const float* a, const float* b, void* out /* bf16 [rows, 2h] */,
    int64_t rows, int64_t hidden, void* stream);
/* ga[r,:] = f32(g[r,0:h]), gb[r,:] = f32(g[r,h:2h])  (:245-268). */
int nestor_hip_cat_cast_bwd(
    const void* g /* bf16 [rows, 2h] */, float* ga, float* gb,
    int64_t rows, int64_t hidden, void* stream);

/* out[o,:] = sum_{e<group} term(f32(y_pad[row_dest[o*group+e],:]) * w[o*group+e]),
 * fp32 accumulate; round_term != 0 rounds every term to out_dtype first
 * (nestor/backbones/triton_expert.py:271-302,456-480 combine_rows). */
int nestor_hip_combine_rows_fwd(
    const void* y_pad /* bf16 [rows_pad, dim] */, const int64_t* row_dest,
    const void* weights, int32_t w_dtype,
    void* out, int32_t out_dtype, int64_t n_out, int32_t group, int64_t dim,
    int32_t round_term, void* stream);

/* grad_y[p,:] = bf16(go[src/group,:] * w[src]) on valid rows, exact 0 on slack;
 * grad_w[src] = sum_d go*y in fp32 when grad_w != NULL
 * (nestor/backbones/triton_expert.py:304-344,482-503). grad_w entries of rows
 * that own no padded slot are left untouched.
 * row_dest (nullable, [n_out*group], the inverse map) selects, for group > 1, the
 * source-major kernel: each row of grad_out is read once for the `group` routed
 * rows that were summed into it; same result.  n_out is only read with row_dest. */
int nestor_hip_combine_rows_bwd(
    const void* grad_out, int32_t go_dtype, const void* y_pad,
    const int64_t* pad_src_row, const void* pad_valid, int32_t valid_dtype,
    const void* weights, int32_t w_dtype,
    void* grad_y /* bf16 [rows_pad, dim] */, float* grad_w /* nullable, [rows] */,
    int64_t rows_pad, int32_t group, int64_t dim,
    const int64_t* row_dest /* nullable */, int64_t n_out, void* stream);

/* ------------------------------------------------------------------------
 * Grouped GEMMs (bf16 operands, fp32 accumulate on MFMA, bf16 results).
 * All stand in for torch._grouped_mm(a, b, offs=offs) and its autograd as
 * called from segment_mm (nestor/backbones/grouped_mm.py:83-104,417-450).
 * They walk the tile tables of nestor_hip_index_build / _tile_schedule, which
 * carry the segment bounds (tile_table is that whole buffer, max_tiles ==
 * nestor_hip_max_tiles(rows_pad, num_banks)).  K % 8 == 0 and N % 8 == 0.
 * ---------------------------------------------------------------------- */

/* out[r,:] = a[r,:] @ b[bank(r)]   a [rows_pad,K], b [E,K,N], out [rows_pad,N]. */
int nestor_hip_grouped_gemm_nn(
    const void* a, const void* b, void* out,
    int64_t rows_pad, int64_t K, int64_t N, int32_t num_banks,
    const int32_t* tile_table, int64_t max_tiles, void* stream);

/* Up and gate projections as one launch over the two stacked banks
 * w_up / w_gate [E,K,H] (nestor/backbones/expert_bank_stack.py:72-77), with
 * SwiGLU in the epilogue: writes up_gate [rows_pad, 2H] (up | gate, each
 * rounded to bf16, what the reference's fused up|gate GEMM returns,
 * grouped_mm.py:409-417) when up_gate != NULL, and
 * hidden [rows_pad, H] = swiglu(up_gate) with the rounding points of
 * nestor_hip_swiglu_fwd. */
int nestor_hip_grouped_gemm_upgate_swiglu(
    const void* a, const void* w_up, const void* w_gate,
    void* up_gate /* nullable */, void* hidden,
    int64_t rows_pad, int64_t K, int64_t H, int32_t num_banks,
    const int32_t* tile_table, int64_t max_tiles, void* stream);

/* out[r,:] = a[r,:] @ b[bank(r)]^T   a [rows_pad,K], b [E,N,K], out [rows_pad,N]:
 * the input-gradient GEMM of torch._grouped_mm's autograd. */
int nestor_hip_grouped_gemm_nt(
    const void* a, const void* b, void* out,
    int64_t rows_pad, int64_t K, int64_t N, int32_t num_banks,
    const int32_t* tile_table, int64_t max_tiles, void* stream);

/* grad_x_pad = g_up_gate[:, :H] @ w_up[bank]^T + g_up_gate[:, H:] @ w_gate[bank]^T
 * g_up_gate [rows_pad, 2H], w_up / w_gate [E,K,H], out [rows_pad,K]. */
int nestor_hip_grouped_gemm_nt_upgate(
    const void* g_up_gate, const void* w_up, const void* w_gate, void* out,
    int64_t rows_pad, int64_t K, int64_t H, int32_t num_banks,
    const int32_t* tile_table, int64_t max_tiles, void* stream);

/* out[e] = a[seg(e),:]^T @ g[seg(e),:]   a [rows_pad,M] (row stride lda),
 * g [rows_pad,N] (row stride ldg), out [E,M,N] (row stride ldo, bank stride
 * bank_stride elements): the weight-gradient GEMM, contraction over the rows
 * of each segment; banks with no rows get exact zeros
 * (nestor/backbones/grouped_mm.py:477-479).  seg_start / seg_count
 * (int64[E], e.g. padded_starts / counts) bound the contraction; when NULL
 * the segments are taken from offs.  out_dtype NESTOR_HIP_BF16: out is bf16, what
 * torch._grouped_mm's autograd returns.  NESTOR_HIP_F32: out is float, the gradient of
 * a bank whose owners are fp32 (nestor/backbones/expert_bank_stack.py:197-213 narrows
 * the owners per micro-step, so autograd widens the bf16 gradient again;
 * nestor/backbones/triton_expert.py:444-453): one store instead of a bf16 store
 * plus a widening pass over the whole bank. */
int nestor_hip_grouped_gemm_tn(
    const void* a, int64_t lda, const void* g, int64_t ldg,
    void* out, int64_t ldo, int64_t bank_stride,
    int64_t rows_pad, int64_t M, int64_t N, int32_t num_banks,
    const int32_t* offs, const int64_t* seg_start, const int64_t* seg_count,
    int32_t out_dtype, void* stream);

/* The two weight gradients of the fused up|gate GEMM in one call: g [rows_pad, 2N] holds
 * the gradient of the up columns, then of the gate columns (the backward of
 * grouped_mm_fused_gate's concatenated weight, nestor/backbones/triton_expert.py:444-453
 * splits one [E,d,2h] gradient into the two owners'); out0[e] = a_seg^T @ g_seg[:, :N],
 * out1[e] = a_seg^T @ g_seg[:, N:], both [E,M,N] with the same strides and dtype.  One
 * launch when N is a multiple of 256 (the gradients share the activation panels), else
 * two nestor_hip_grouped_gemm_tn launches; the results are the same bits either way. */
int nestor_hip_grouped_gemm_tn_pair(
    const void* a, int64_t lda, const void* g, int64_t ldg,
    void* out0, void* out1, int64_t ldo, int64_t bank_stride,
    int64_t rows_pad, int64_t M, int64_t N, int32_t num_banks,
    const int32_t* offs, const int64_t* seg_start, const int64_t* seg_count,
    int32_t out_dtype, void* stream);

/* fp8 (OCP e4m3fn) weight variant of nestor_hip_grouped_gemm_nn for the
 * weight-streaming inference regime: b_q [E,K,N] e4m3, scale [E,N] fp32 per
 * output channel, out[r,n] = bf16( scale[bank,n] * sum_k a[r,k]*b_q[bank,k,n] ).
 * tiled != 0: b_q is stored [E, N/128, K, 128] -- each 128 output columns of a bank
 * one contiguous block, so that a workgroup streams contiguous memory instead of
 * 128..256-byte pieces of rows kilobytes apart (N % 128 == 0).  The e4m3 bank is
 * this library's own format (the reference has none), so its layout is free. */
int nestor_hip_grouped_gemm_fp8w_nn(
    const void* a, const void* b_q, const float* scale, void* out,
    int64_t rows_pad, int64_t K, int64_t N, int32_t num_banks,
    const int32_t* tile_table, int64_t max_tiles, int32_t tiled, void* stream);
/* The up and gate projections of an e4m3 bank and SwiGLU in one weight-streaming
 * launch: hidden[r,n] = bf16( silu(gate) * up ), up = bf16(scale_up[bank,n] * a[r,:] @
 * up_q[bank,:,n]), gate likewise, silu rounded to bf16 as in the unfused chain
 * (nestor/backbones/triton_expert.py:172-175).  Meant for a few rows per bank
 * (every 32 or 64 rows of a tile stream the weight panel once); K % 64 == 0 and
 * H % 128 == 0, else NESTOR_HIP_EINVAL. */
int nestor_hip_grouped_gemm_fp8w_upgate_swiglu(
    const void* a, const void* up_q, const void* gate_q,
    const float* scale_up, const float* scale_gate, void* hidden /* bf16 [rows_pad, H] */,
    int64_t rows_pad, int64_t K, int64_t H, int32_t num_banks,
    const int32_t* tile_table, int64_t max_tiles, int32_t tiled /* both banks */, void* stream);

/* ------------------------------------------------------------------------
 * Router epilogue (eval-mode Router.forward after the score GEMM,
 * nestor/backbones/nestor.py:558-593; batched over G routers,
 * nestor/backbones/batched_router.py:210-227).
 * scores [n, C] -> softmax_probs [n, C] (fp32; the caller narrows it when the
 * reference would), topk_indices [n, k] (int64, descending biased score, ties
 * broken towards the lower index), gates [n, C] (scores dtype, zero off the
 * top-k and on rows with mask[row] == 0).
 * gate_mode 0 = renorm, 1 = switch.  choice_bias [n_bias_rows, C] fp32 is
 * indexed by row % n_bias_rows (1 row: one router; G rows: batched routers
 * with n = T*G).  C <= 64, k <= 8.
 * ---------------------------------------------------------------------- */
int nestor_hip_router_topk(
    const void* scores, int32_t dtype, const float* choice_bias, int32_t n_bias_rows,
    const uint8_t* mask /* nullable, [n] */,
    float* softmax_probs, int64_t* topk_indices, void* gates,
    int64_t n, int32_t num_choices, int32_t top_k, int32_t gate_mode,
    void* stream);

/* Gradient of the scores through gates (and through softmax_probs when grad_probs
 * != NULL): what autograd derives from the reference's differentiable chain
 * softmax -> gather -> scatter_add -> mask (nestor/backbones/nestor.py:565-590),
 * fp32 with one rounding to the score dtype.  grad_gates [n, C] in the score
 * dtype (nullable), grad_probs [n, C] fp32 (nullable), grad_scores [n, C]. */
int nestor_hip_router_gates_bwd(
    const void* scores, int32_t dtype, const int64_t* topk_indices,
    const uint8_t* mask /* nullable */, const void* grad_gates, const float* grad_probs,
    void* grad_scores, int64_t n, int32_t num_choices, int32_t top_k, int32_t gate_mode,
    void* stream);

/* Loss-free balancing statistic (Router.update_detached_parameters,
 * nestor/backbones/nestor.py:613-615): counts[c] += number of (row, slot) pairs
 * with mask[row] != 0 and topk_indices[row, slot] == c.  counts [C] int32 must be
 * zeroed by the caller; integer sums, reproducible.  C <= 64. */
int nestor_hip_router_choice_counts(
    const int64_t* topk_indices /* [n, k] */, const uint8_t* mask /* nullable, [n] */,
    int32_t* counts, int64_t n, int32_t top_k, int32_t num_choices, void* stream);

/* Private slots of the pool (ExpertPoolMLP._private_slots,
 * nestor/backbones/expert_pools.py:422-521): the k_a columns with the largest
 * column gates per token (descending; equal gates lowest index first) -- or the
 * caller's selected_in [T, k_a] -- and per selected column g its k_q chosen
 * experts e = choices[t,g,i]: ids[t, j*k_q+i] = g*Q + e, weights = gates[t,g,e] *
 * column_gates[t,g] rounded to `dtype`.  column_gates [T, G], gates [T, G, Q],
 * choices [T, G, k_q]; G <= 64. */
int nestor_hip_private_slots_fwd(
    const void* column_gates, const void* gates, int32_t dtype, const int64_t* choices,
    const int64_t* selected_in /* nullable */, int64_t* selected /* [T, k_a] */,
    int64_t* ids /* [T, k_a*k_q] */, void* weights /* [T, k_a*k_q] */,
    int64_t num_tokens, int32_t num_columns, int32_t num_experts, int32_t k_a, int32_t k_q,
    void* stream);
/* Gradients of the slot weights w.r.t. column_gates [T, G] and gates [T, G, Q]
 * (dense, zero off the selected entries). */
int nestor_hip_private_slots_bwd(
    const void* grad_weights, const void* column_gates, const void* gates, int32_t dtype,
    const int64_t* choices, const int64_t* selected, void* grad_column_gates, void* grad_gates,
    int64_t num_tokens, int32_t num_columns, int32_t num_experts, int32_t k_a, int32_t k_q,
    void* stream);

/* ------------------------------------------------------------------------
 * Path mix of the pool's summed layout: update = alpha_public * public_update +
 * alpha_private * private_update with alpha = softmax of the 2-logit path gate
 * (nestor/backbones/expert_pools.py:1103-1114).  All tensors share `dtype`
 * (bf16 or fp32, the pool input's); each product and the sum are rounded to it,
 * as the eager expression rounds them.  alpha is [num_tokens, 2].
 * ---------------------------------------------------------------------- */
int nestor_hip_path_mix_fwd(
    const void* public_update, const void* private_update, const void* alpha,
    void* out, int32_t dtype, int64_t num_tokens, int64_t dim, void* stream);
/* grad_public = g*alpha[:,0], grad_private = g*alpha[:,1],
 * grad_alpha[t,0] = sum_d g*public, grad_alpha[t,1] = sum_d g*private (terms
 * rounded to `dtype`, fp32 sum, one final rounding): what autograd derives from
 * the expression above. */
int nestor_hip_path_mix_bwd(
    const void* grad_out, const void* public_update, const void* private_update,
    const void* alpha, void* grad_public, void* grad_private, void* grad_alpha,
    int32_t dtype, int64_t num_tokens, int64_t dim, void* stream);

/* Split layouts of the pool (nestor/backbones/expert_pools.py:943-953 per slot,
 * :1023-1041 per column): out[t,o,:] = alpha[t,which] * X[t,o,:] rounded to
 * `dtype`, where X = in ([num_tokens, slots, dim]; dest == NULL, num_out ==
 * slots) or in scattered onto num_out column streams by dest [num_tokens, slots]
 * (the zeros(...).scatter_add(1, index, per_slot) of :758-761; streams no slot
 * selects are zero).  dest entries must lie in [0, num_out).  slots <= 64. */
int nestor_hip_path_scale_fwd(
    const void* in, const void* alpha /* [num_tokens, 2] */, int32_t which,
    const int64_t* dest /* nullable */, void* out /* [num_tokens, num_out, dim] */,
    int32_t dtype, int64_t num_tokens, int32_t slots, int32_t num_out, int64_t dim,
    void* stream);
/* grad_in[t,s,:] = grad_out[t,o(s),:] * alpha[t,which] with o(s) = dest[t,s] (or s);
 * grad_alpha[t] = sum over slots and features of grad_out[t,o(s),:] * in[t,s,:]
 * (fp32): the gradient of alpha[t,which]. */
int nestor_hip_path_scale_bwd(
    const void* grad_out, const void* in, const void* alpha, int32_t which,
    const int64_t* dest /* nullable */, void* grad_in, float* grad_alpha /* [num_tokens] */,
    int32_t dtype, int64_t num_tokens, int32_t slots, int32_t num_out, int64_t dim,
    void* stream);

/* ------------------------------------------------------------------------
 * Biased banks (the reference's native MoE baselines:
 * nestor/backbones/grouped_mm.py:159-177 _IndexedBias, :426-437 up bias on the
 * padded rows, :541-554 down bias on the routed rows).
 * out[r,:] = bf16(rows[r,:] + bias[index[r],:]) where valid[r] != 0 (every row
 * when valid == NULL), rows[r,:] elsewhere.  rows/out bf16 [n_rows, dim], bias
 * bf16 [E, dim].
 * ---------------------------------------------------------------------- */
int nestor_hip_bias_rows_fwd(
    const void* rows, const void* bias, const int64_t* index,
    const void* valid /* nullable */, int32_t valid_dtype, void* out,
    int64_t n_rows, int64_t dim, void* stream);
/* The bias gradient, the reference's one-hot GEMM (onehot[E,rows] @ grad_rows,
 * :173-177) as a segmented column sum: out[e,:] = bf16( sum_{i < seg_count[e]}
 * grad[row(e,i),:] ), row(e,i) = row_index[seg_start[e]+i], or seg_start[e]+i
 * when row_index == NULL (padded rows: seg_start = padded_starts; routed rows:
 * row_index = the plan's stable order, seg_start = raw_starts).  fp32 sums in a
 * fixed order, no atomics.  splits > 1 divides every segment over that many
 * workgroups and needs partial [splits, E, dim] fp32. */
int nestor_hip_segment_colsum(
    const void* grad /* bf16 [*, dim] */, const int64_t* row_index /* nullable */,
    const int64_t* seg_start, const int64_t* seg_count,
    float* partial /* nullable when splits == 1 */, int32_t splits,
    void* out /* bf16 [E, dim] */, int32_t num_banks, int64_t dim, void* stream);

/* ------------------------------------------------------------------------
 * Packed column attention epilogue (gate_combine_slots,
 * nestor/backbones/triton_packed.py:332-412,547-640): slot-layout rows from the
 * packed output-GEMM rows.  out[s,:] = T(val) * T(gates[r]) with r = slot_rows[s],
 * val = out_c[r,:] (+ bf16(bias[gid[r],:]), sum rounded to bf16), T = out_dtype.
 * out_c bf16 [rows, dim], bias fp32 [G, dim] (nullable, then gid unused), gates
 * fp32 [rows] (exactly 0 on alignment-tail rows).  Its row gather is
 * nestor_hip_dispatch_rows_fwd (pack_rows, :650-676).
 * ---------------------------------------------------------------------- */
int nestor_hip_gate_slots_fwd(
    const void* out_c, const float* bias, const int64_t* gid, const float* gates,
    const int64_t* slot_rows, void* out, int32_t out_dtype, int64_t n_out, int64_t dim,
    void* stream);
/* grad_out_c[r,:] = bf16(gates[r] * g[slot_packed[r],:]); grad_gates[r] = sum_d g*val
 * in fp32 when grad_gates != NULL.  The bias gradient is
 * nestor_hip_segment_colsum over grad_out_c. */
int nestor_hip_gate_slots_bwd(
    const void* grad_slots, int32_t g_dtype, const void* out_c, const float* bias,
    const int64_t* gid, const float* gates, const int64_t* slot_packed,
    void* grad_out_c /* bf16 [rows, dim] */, float* grad_gates /* nullable */,
    int64_t rows, int64_t dim, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NESTOR_HIP_H_ */
