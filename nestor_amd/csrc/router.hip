// Router epilogue: softmax, biased top-k, gates -- one launch for a whole
// [rows, choices] score block (all G private routers of a layer at once when
// rows = tokens * G).  A row is spread over the smallest power-of-two group of
// lanes that holds its choices, so a 64-lane wavefront routes 64 / group rows
// and every reduction is a handful of xor-shuffles.
//
// Follows Router.forward in eval mode (nestor/backbones/nestor.py:558-593) and
// its batched form (nestor/backbones/batched_router.py:210-227).  torch.topk
// leaves the order of equal scores unspecified; here equal biased scores are
// taken lowest index first.
#include "common.hpp"

namespace nestor {
namespace {

constexpr int kRouterBlock = 256;

template <typename F>
__device__ __forceinline__ float group_reduce(float v, int group, F op) {
  for (int off = group >> 1; off > 0; off >>= 1) v = op(v, __shfl_xor(v, off, kWave));
  return v;
}

template <bool kF32>
__global__ __launch_bounds__(kRouterBlock) void router_topk_kernel(
    const void* __restrict__ scores, const float* __restrict__ choice_bias,
    int n_bias_rows, const uint8_t* __restrict__ mask, float* __restrict__ probs,
    int64_t* __restrict__ topk, void* __restrict__ gates, int64_t n, int num_choices,
    int top_k, int gate_mode, int group_shift) {
  const int group = 1 << group_shift;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * kRouterBlock + threadIdx.x;
  const int64_t row = gid >> group_shift;
  const int sub = static_cast<int>(gid & (group - 1));
  const bool live = row < n && sub < num_choices;
  const float ninf = -__builtin_inff();
  float s = ninf, biased = ninf;
  if (live) {
    s = load_scalar(scores, row * num_choices + sub, kF32 ? NESTOR_HIP_F32 : NESTOR_HIP_BF16);
    // scores (+ fp32 buffer) promote to fp32: one exact-then-rounded fp32 add.
    biased = s + choice_bias[(row % n_bias_rows) * num_choices + sub];
  }
  auto fmax_op = [](float a, float b) { return a > b ? a : b; };
  auto fadd_op = [](float a, float b) { return a + b; };
  const float m = group_reduce(s, group, fmax_op);
  const float e = live ? expf(s - m) : 0.0f;
  const float denom = group_reduce(e, group, fadd_op);
  const float prob = e / denom;
  if (live) probs[row * num_choices + sub] = prob;

  bool taken = false;
  for (int j = 0; j < top_k; ++j) {
    float best = taken ? ninf : biased;
    int best_idx = (live && !taken) ? sub : 0x7fffffff;
    for (int off = group >> 1; off > 0; off >>= 1) {
      const float ov = __shfl_xor(best, off, kWave);
      const int oi = __shfl_xor(best_idx, off, kWave);
      if (ov > best || (ov == best && oi < best_idx)) {
        best = ov;
        best_idx = oi;
      }
    }
    if (live && sub == best_idx) {
      taken = true;
      topk[row * top_k + j] = sub;
    }
  }

  float gate;
  if (gate_mode == 1) {  // switch: full-softmax probability of the selected choices
    gate = taken ? prob : 0.0f;
  } else {               // renorm: softmax over the selected raw scores
    const float m2 = group_reduce(taken ? s : ninf, group, fmax_op);
    const float e2 = taken ? expf(s - m2) : 0.0f;
    const float d2 = group_reduce(e2, group, fadd_op);
    gate = taken ? e2 / d2 : 0.0f;
  }
  if (live) {
    const bool valid = mask == nullptr || mask[row] != 0;
    if constexpr (kF32) {
      reinterpret_cast<float*>(gates)[row * num_choices + sub] = valid ? gate : 0.0f;
    } else {
      // gate is rounded to the score dtype before the validity product.
      reinterpret_cast<uint16_t*>(gates)[row * num_choices + sub] =
          valid ? static_cast<uint16_t>(f32_to_bf16_bits(gate)) : 0;
    }
  }
}


// Gradient of the scores through the gates (and, when grad_probs is given,
// through softmax_probs), in the lane layout of the forward kernel:
//   renorm: gate_j = softmax(scores[topk])_j  ->  dz_j = p_j * (dg_j - sum_i p_i dg_i)
//   switch: gate_j = softmax(scores)[topk_j]  ->  ds_c = P_c * (dP_c - sum P dP), dP = dg on the top-k
// with dg = grad_gates on the selected choices of rows the mask keeps, zero
// elsewhere.  fp32 throughout, one rounding to the score dtype at the end -- the
// eager chain (softmax backward in fp32, cast back) rounds at the same place.
template <bool kF32>
__global__ __launch_bounds__(kRouterBlock) void router_gates_bwd_kernel(
    const void* __restrict__ scores, const int64_t* __restrict__ topk,
    const uint8_t* __restrict__ mask, const void* __restrict__ grad_gates,
    const float* __restrict__ grad_probs, void* __restrict__ grad_scores, int64_t n,
    int num_choices, int top_k, int gate_mode, int group_shift) {
  const int group = 1 << group_shift;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * kRouterBlock + threadIdx.x;
  const int64_t row = gid >> group_shift;
  const int sub = static_cast<int>(gid & (group - 1));
  const bool live = row < n && sub < num_choices;
  const int dt = kF32 ? NESTOR_HIP_F32 : NESTOR_HIP_BF16;
  const float ninf = -__builtin_inff();
  float s = ninf, dg = 0.0f, dp = 0.0f;
  bool taken = false;
  if (live) {
    s = load_scalar(scores, row * num_choices + sub, dt);
    for (int j = 0; j < top_k; ++j) taken |= topk[row * top_k + j] == sub;
    const bool valid = mask == nullptr || mask[row] != 0;
    if (taken && valid && grad_gates != nullptr)
      dg = load_scalar(grad_gates, row * num_choices + sub, dt);
    if (grad_probs != nullptr) dp = grad_probs[row * num_choices + sub];
  }
  auto fmax_op = [](float a, float b) { return a > b ? a : b; };
  auto fadd_op = [](float a, float b) { return a + b; };
  const float m = group_reduce(s, group, fmax_op);
  const float e = live ? expf(s - m) : 0.0f;
  const float prob = e / group_reduce(e, group, fadd_op);
  float ds = 0.0f;
  if (gate_mode == 1) {
    dp += dg;  // both paths go through the full softmax
  } else {
    const float m2 = group_reduce(taken ? s : ninf, group, fmax_op);
    const float e2 = taken ? expf(s - m2) : 0.0f;
    const float p2 = e2 / group_reduce(e2, group, fadd_op);
    const float dot2 = group_reduce(p2 * dg, group, fadd_op);
    ds = taken ? p2 * (dg - dot2) : 0.0f;
  }
  if (gate_mode == 1 || grad_probs != nullptr) {
    const float dot = group_reduce(prob * dp, group, fadd_op);
    ds += prob * (dp - dot);
  }
  if (live) {
    if constexpr (kF32) {
      reinterpret_cast<float*>(grad_scores)[row * num_choices + sub] = ds;
    } else {
      reinterpret_cast<uint16_t*>(grad_scores)[row * num_choices + sub] =
          static_cast<uint16_t>(f32_to_bf16_bits(ds));
    }
  }
}

// Private slots of the pool (ExpertPoolMLP._private_slots,
// nestor/backbones/expert_pools.py:422-521): per token the k_a columns with the
// largest column gates (descending, equal gates lowest index first; or the
// caller's selection), and for each of them the column's k_q chosen experts:
//   ids[t, j*k_q+i]     = g*Q + e            g = selected[t,j], e = choices[t,g,i]
//   weights[t, j*k_q+i] = gates[t,g,e] * column_gates[t,g]   (rounded to the gate dtype)
// One thread per token: the whole thing is a few dozen scalar loads.
constexpr int kSlotsBlock = 128;

template <bool kF32>
__global__ __launch_bounds__(kSlotsBlock) void private_slots_fwd_kernel(
    const void* __restrict__ column_gates, const void* __restrict__ gates,
    const int64_t* __restrict__ choices, const int64_t* __restrict__ selected_in,
    int64_t* __restrict__ selected, int64_t* __restrict__ ids, void* __restrict__ weights,
    int64_t num_tokens, int num_columns, int num_experts, int k_a, int k_q) {
  const int64_t t = static_cast<int64_t>(blockIdx.x) * kSlotsBlock + threadIdx.x;
  if (t >= num_tokens) return;
  const int dt = kF32 ? NESTOR_HIP_F32 : NESTOR_HIP_BF16;
  uint64_t used = 0;
  for (int j = 0; j < k_a; ++j) {
    int g;
    if (selected_in != nullptr) {
      // indices handed in are clamped into range: a bad one reads a wrong gate, never other memory
      const int64_t given = selected_in[t * k_a + j];
      g = static_cast<int>(given < 0 ? 0 : (given >= num_columns ? num_columns - 1 : given));
    } else {
      float best = -__builtin_inff();
      g = 0;
      bool found = false;
      for (int c = 0; c < num_columns; ++c) {
        if ((used >> c) & 1) continue;
        const float v = load_scalar(column_gates, t * num_columns + c, dt);
        if (!found || v > best) {
          best = v;
          g = c;
          found = true;
        }
      }
      used |= 1ull << g;
    }
    selected[t * k_a + j] = g;
    const float cg = load_scalar(column_gates, t * num_columns + g, dt);
    for (int i = 0; i < k_q; ++i) {
      int64_t e = choices[(t * num_columns + g) * k_q + i];
      e = e < 0 ? 0 : (e >= num_experts ? num_experts - 1 : e);
      const float pg = load_scalar(gates, (t * num_columns + g) * num_experts + e, dt);
      const int64_t slot = (t * k_a + j) * k_q + i;
      ids[slot] = static_cast<int64_t>(g) * num_experts + e;
      const float w = pg * cg;
      if constexpr (kF32) {
        reinterpret_cast<float*>(weights)[slot] = w;
      } else {
        reinterpret_cast<uint16_t*>(weights)[slot] = static_cast<uint16_t>(f32_to_bf16_bits(w));
      }
    }
  }
}

// Gradients of the slot weights: grad_column_gates[t,g] = sum_i round(dW * gate),
// grad_gates[t,g,e] = round(dW * column_gate) on the selected entries, zero
// elsewhere (the thread clears its token's rows first; a token's selected
// columns are distinct, and so are a column's chosen experts).
template <bool kF32>
__global__ __launch_bounds__(kSlotsBlock) void private_slots_bwd_kernel(
    const void* __restrict__ grad_weights, const void* __restrict__ column_gates,
    const void* __restrict__ gates, const int64_t* __restrict__ choices,
    const int64_t* __restrict__ selected, void* __restrict__ grad_column_gates,
    void* __restrict__ grad_gates, int64_t num_tokens, int num_columns, int num_experts,
    int k_a, int k_q) {
  const int64_t t = static_cast<int64_t>(blockIdx.x) * kSlotsBlock + threadIdx.x;
  if (t >= num_tokens) return;
  const int dt = kF32 ? NESTOR_HIP_F32 : NESTOR_HIP_BF16;
  auto store = [&](void* base, int64_t i, float v) {
    if constexpr (kF32) {
      reinterpret_cast<float*>(base)[i] = v;
    } else {
      reinterpret_cast<uint16_t*>(base)[i] = static_cast<uint16_t>(f32_to_bf16_bits(v));
    }
  };
  for (int c = 0; c < num_columns; ++c) store(grad_column_gates, t * num_columns + c, 0.0f);
  for (int c = 0; c < num_columns * num_experts; ++c)
    store(grad_gates, t * num_columns * num_experts + c, 0.0f);
  for (int j = 0; j < k_a; ++j) {
    int64_t g = selected[t * k_a + j];
    g = g < 0 ? 0 : (g >= num_columns ? num_columns - 1 : g);  // as the forward clamps them
    const float cg = load_scalar(column_gates, t * num_columns + g, dt);
    float dcg = 0.0f;
    for (int i = 0; i < k_q; ++i) {
      int64_t e = choices[(t * num_columns + g) * k_q + i];
      e = e < 0 ? 0 : (e >= num_experts ? num_experts - 1 : e);
      const float pg = load_scalar(gates, (t * num_columns + g) * num_experts + e, dt);
      const float dw = load_scalar(grad_weights, (t * k_a + j) * k_q + i, dt);
      const float term = dw * pg;
      dcg += kF32 ? term : round_bf16(term);
      store(grad_gates, (t * num_columns + g) * num_experts + e, dw * cg);
    }
    store(grad_column_gates, t * num_columns + g, dcg);
  }
}

// Loss-free balancing statistic (Router.update_detached_parameters,
// nestor/backbones/nestor.py:613-615): counts[c] = number of (valid token, slot)
// pairs whose choice is c.  Integer LDS histogram per workgroup, one integer
// atomic per choice and workgroup into `counts` (which the caller zeroes):
// integer sums, so the result does not depend on the order.
__global__ __launch_bounds__(kRouterBlock) void choice_count_kernel(
    const int64_t* __restrict__ topk, const uint8_t* __restrict__ mask,
    int32_t* __restrict__ counts, int64_t n, int top_k, int num_choices) {
  __shared__ int hist[64];
  if (threadIdx.x < 64) hist[threadIdx.x] = 0;
  __syncthreads();
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kRouterBlock;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kRouterBlock + threadIdx.x; i < n * top_k;
       i += stride) {
    const int64_t row = i / top_k;
    if (mask != nullptr && mask[row] == 0) continue;
    const int64_t c = topk[i];
    if (c >= 0 && c < num_choices) atomicAdd(&hist[c], 1);
  }
  __syncthreads();
  if (threadIdx.x < num_choices && hist[threadIdx.x] != 0)
    atomicAdd(&counts[threadIdx.x], hist[threadIdx.x]);
}

}  // namespace
}  // namespace nestor

using namespace nestor;

extern "C" int nestor_hip_router_topk(const void* scores, int32_t dtype,
                                      const float* choice_bias, int32_t n_bias_rows,
                                      const uint8_t* mask, float* softmax_probs,
                                      int64_t* topk_indices, void* gates, int64_t n,
                                      int32_t num_choices, int32_t top_k, int32_t gate_mode,
                                      void* stream) {
  if ((dtype != NESTOR_HIP_F32 && dtype != NESTOR_HIP_BF16) || num_choices <= 0 ||
      num_choices > 64 || top_k <= 0 || top_k > num_choices || n_bias_rows <= 0 || n < 0 ||
      (gate_mode != 0 && gate_mode != 1))
    return NESTOR_HIP_EINVAL;
  if (n == 0) return NESTOR_HIP_OK;
  if (!scores || !choice_bias || !softmax_probs || !topk_indices || !gates)
    return NESTOR_HIP_EINVAL;
  int shift = 0;
  while ((1 << shift) < num_choices) ++shift;
  const int64_t threads = n << shift;
  const unsigned blocks = static_cast<unsigned>(ceil_div(threads, kRouterBlock));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == NESTOR_HIP_F32)
    hipLaunchKernelGGL(router_topk_kernel<true>, dim3(blocks), dim3(kRouterBlock), 0, s,
                       scores, choice_bias, n_bias_rows, mask, softmax_probs, topk_indices,
                       gates, n, num_choices, top_k, gate_mode, shift);
  else
    hipLaunchKernelGGL(router_topk_kernel<false>, dim3(blocks), dim3(kRouterBlock), 0, s,
                       scores, choice_bias, n_bias_rows, mask, softmax_probs, topk_indices,
                       gates, n, num_choices, top_k, gate_mode, shift);
  return launch_status();
}

extern "C" int nestor_hip_router_gates_bwd(const void* scores, int32_t dtype,
                                           const int64_t* topk_indices, const uint8_t* mask,
                                           const void* grad_gates, const float* grad_probs,
                                           void* grad_scores, int64_t n, int32_t num_choices,
                                           int32_t top_k, int32_t gate_mode, void* stream) {
  if ((dtype != NESTOR_HIP_F32 && dtype != NESTOR_HIP_BF16) || num_choices <= 0 ||
      num_choices > 64 || top_k <= 0 || top_k > num_choices || n < 0 ||
      (gate_mode != 0 && gate_mode != 1))
    return NESTOR_HIP_EINVAL;
  if (n == 0) return NESTOR_HIP_OK;
  if (!scores || !topk_indices || !grad_scores) return NESTOR_HIP_EINVAL;
  int shift = 0;
  while ((1 << shift) < num_choices) ++shift;
  const unsigned blocks = static_cast<unsigned>(ceil_div(n << shift, kRouterBlock));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == NESTOR_HIP_F32)
    hipLaunchKernelGGL(router_gates_bwd_kernel<true>, dim3(blocks), dim3(kRouterBlock), 0, s,
                       scores, topk_indices, mask, grad_gates, grad_probs, grad_scores, n,
                       num_choices, top_k, gate_mode, shift);
  else
    hipLaunchKernelGGL(router_gates_bwd_kernel<false>, dim3(blocks), dim3(kRouterBlock), 0, s,
                       scores, topk_indices, mask, grad_gates, grad_probs, grad_scores, n,
                       num_choices, top_k, gate_mode, shift);
  return launch_status();
}

extern "C" int nestor_hip_private_slots_fwd(const void* column_gates, const void* gates,
                                            int32_t dtype, const int64_t* choices,
                                            const int64_t* selected_in, int64_t* selected,
                                            int64_t* ids, void* weights, int64_t num_tokens,
                                            int32_t num_columns, int32_t num_experts,
                                            int32_t k_a, int32_t k_q, void* stream) {
  if ((dtype != NESTOR_HIP_F32 && dtype != NESTOR_HIP_BF16) || num_columns <= 0 ||
      num_columns > 64 || num_experts <= 0 || k_a <= 0 || k_a > num_columns || k_q <= 0 ||
      k_q > num_experts || num_tokens < 0)
    return NESTOR_HIP_EINVAL;
  if (num_tokens == 0) return NESTOR_HIP_OK;
  if (!column_gates || !gates || !choices || !selected || !ids || !weights)
    return NESTOR_HIP_EINVAL;
  const unsigned blocks = static_cast<unsigned>(ceil_div(num_tokens, kSlotsBlock));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == NESTOR_HIP_F32)
    hipLaunchKernelGGL(private_slots_fwd_kernel<true>, dim3(blocks), dim3(kSlotsBlock), 0, s,
                       column_gates, gates, choices, selected_in, selected, ids, weights,
                       num_tokens, num_columns, num_experts, k_a, k_q);
  else
    hipLaunchKernelGGL(private_slots_fwd_kernel<false>, dim3(blocks), dim3(kSlotsBlock), 0, s,
                       column_gates, gates, choices, selected_in, selected, ids, weights,
                       num_tokens, num_columns, num_experts, k_a, k_q);
  return launch_status();
}

extern "C" int nestor_hip_private_slots_bwd(const void* grad_weights, const void* column_gates,
                                            const void* gates, int32_t dtype,
                                            const int64_t* choices, const int64_t* selected,
                                            void* grad_column_gates, void* grad_gates,
                                            int64_t num_tokens, int32_t num_columns,
                                            int32_t num_experts, int32_t k_a, int32_t k_q,
                                            void* stream) {
  if ((dtype != NESTOR_HIP_F32 && dtype != NESTOR_HIP_BF16) || num_columns <= 0 ||
      num_columns > 64 || num_experts <= 0 || k_a <= 0 || k_a > num_columns || k_q <= 0 ||
      k_q > num_experts || num_tokens < 0)
    return NESTOR_HIP_EINVAL;
  if (num_tokens == 0) return NESTOR_HIP_OK;
  if (!grad_weights || !column_gates || !gates || !choices || !selected || !grad_column_gates ||
      !grad_gates)
    return NESTOR_HIP_EINVAL;
  const unsigned blocks = static_cast<unsigned>(ceil_div(num_tokens, kSlotsBlock));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == NESTOR_HIP_F32)
    hipLaunchKernelGGL(private_slots_bwd_kernel<true>, dim3(blocks), dim3(kSlotsBlock), 0, s,
                       grad_weights, column_gates, gates, choices, selected, grad_column_gates,
                       grad_gates, num_tokens, num_columns, num_experts, k_a, k_q);
  else
    hipLaunchKernelGGL(private_slots_bwd_kernel<false>, dim3(blocks), dim3(kSlotsBlock), 0, s,
                       grad_weights, column_gates, gates, choices, selected, grad_column_gates,
                       grad_gates, num_tokens, num_columns, num_experts, k_a, k_q);
  return launch_status();
}

extern "C" int nestor_hip_router_choice_counts(const int64_t* topk_indices, const uint8_t* mask,
                                               int32_t* counts, int64_t n, int32_t top_k,
                                               int32_t num_choices, void* stream) {
  if (num_choices <= 0 || num_choices > 64 || top_k <= 0 || n < 0) return NESTOR_HIP_EINVAL;
  if (n == 0) return NESTOR_HIP_OK;
  if (!topk_indices || !counts) return NESTOR_HIP_EINVAL;
  const int64_t want = ceil_div(n * top_k, kRouterBlock * 8);
  const unsigned blocks = static_cast<unsigned>(want < 1 ? 1 : want > 1024 ? 1024 : want);
  hipLaunchKernelGGL(choice_count_kernel, dim3(blocks), dim3(kRouterBlock), 0,
                     static_cast<hipStream_t>(stream), topk_indices, mask, counts, n, top_k,
                     num_choices);
  return launch_status();
}

extern "C" int nestor_hip_abi_version(void) { return NESTOR_HIP_ABI_VERSION; }

extern "C" const char* nestor_hip_strerror(int code) {
  switch (code) {
    case NESTOR_HIP_OK: return "ok";
    case NESTOR_HIP_EINVAL: return "invalid argument (size, alignment, dtype code or null pointer)";
    case NESTOR_HIP_ENOSPC: return "workspace too small";
    case NESTOR_HIP_ELAUNCH: return "HIP kernel launch failed";
    case NESTOR_HIP_ERANGE: return "size beyond what the kernels support";
    default: return "unknown nestor_hip status";
  }
}
