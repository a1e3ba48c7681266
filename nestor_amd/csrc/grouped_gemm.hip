// Grouped expert GEMMs on the gfx950 matrix cores.
//
// A workgroup of 4 wavefronts owns a BM x BN output tile and walks the
// contraction in steps of BK through double-buffered LDS; each wavefront keeps
// a (BM / WGM) x (BN / WGN) accumulator as v_mfma_f32_32x32x16_bf16 tiles.
// Which rows form a tile and which bank multiplies them comes from the
// device-side tile table written by the index build, so no launch parameter
// depends on the routing and the host never reads a count.
//
// Operand tiles sit in LDS in the layout they have in HBM.  An operand whose
// contraction index is contiguous in memory (activations in the forward and
// input-gradient GEMMs, W^T in the input-gradient GEMM) is fetched for the MFMA
// with one 128-bit LDS read per lane.  An operand whose contraction index is
// the row index (W[K,N] in the forward GEMM, both operands of the
// weight-gradient GEMM) is fetched with ds_read_b64_tr_b16: in each group of 16
// lanes, lane j points at row j/4, columns 4*(j%4)..+3 of a 4 x 16 block and
// lane i receives column i of that block, i.e. four consecutive contraction
// indices for one output index -- the MFMA operand layout, with no transpose
// pass over the weights or activations in HBM.
//
// Three kernel families share the building blocks of gemm_common.hpp (in file order):
//  * grouped_gemm_kernel -- register-staged: global -> registers -> padded LDS.
//    Per K step the tile for step t+1 goes from registers to the idle LDS
//    buffer, the global loads for step t+2 are issued, then step t is computed
//    from the other buffer with MFMA operand fragments double-buffered in
//    registers.  Takes any K that is a multiple of 8 and narrow outputs; the
//    general fallback.
//  * grouped_gemm_dma_kernel -- the row-tiled modes on the direct-to-LDS path
//    (global_load_lds_dwordx4 into a three-stage unpadded ring, conflicts avoided
//    by swizzling which 16-byte piece each lane fetches): the default at the
//    measured shapes.
//  * wgrad_persistent_kernel -- the weight gradient: one workgroup per CU walks a
//    list of output tiles with the ring running across tile boundaries.
// (The e4m3 weight-streaming kernels are in fp8_stream.hip.)
//
// The MFMA is issued with its operands swapped (B fragment first), which
// produces the transposed 32 x 32 tile: every lane then holds four consecutive
// output columns of one row and the epilogue can stage the bf16 tile through
// LDS with 64-bit writes and leave through 128-bit coalesced stores.
#include "gemm_common.hpp"

namespace nestor {
namespace {

template <typename C, int kMode>
__global__ __launch_bounds__(kThreads) void grouped_gemm_kernel(GemmParams p) {
  extern __shared__ __align__(16) uint16_t lds[];
  constexpr int BM = C::BM, BN = C::BN, BK = C::BK;
  constexpr bool kUpGateFwd = kMode == kNNUpGate;
  constexpr bool kAContig = kMode != kTN;                         // a is [rows, K]
  constexpr bool kBContig = kMode == kNT || kMode == kNTUpGate;   // b is [N, K]
  constexpr int kOutCols = kUpGateFwd ? BN / 2 : BN;              // output columns per tile
  constexpr int A_LD = kAContig ? C::KC_LD : BM + 32;
  constexpr int B_LD = kBContig ? C::KC_LD : BN + 32;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wavefront-uniform: keep it scalar
  const int wm = wave / C::WGN;
  const int wn = wave % C::WGN;

  // ---- which tile -------------------------------------------------------
  int bank, row0 = 0, nrows = BM;
  int64_t n0, m0 = 0;
  int64_t seg_begin = 0, seg_end = 0;
  if constexpr (kMode == kTN) {
    bank = blockIdx.z;
    m0 = static_cast<int64_t>(blockIdx.y) * BM;
    n0 = static_cast<int64_t>(blockIdx.x) * BN;
    if (p.seg_start != nullptr) {
      seg_begin = p.seg_start[bank];
      seg_end = seg_begin + p.seg_count[bank];
    } else {
      seg_begin = bank == 0 ? 0 : p.offs[bank - 1];
      seg_end = p.offs[bank];
    }
    if (seg_end > p.rows_pad) seg_end = p.rows_pad;
  } else {
    const int tile = blockIdx.x / p.n_tiles;
    const int nt = blockIdx.x % p.n_tiles;
    const int32_t* tt = p.tile_table;
    if (tile >= tt[3 * p.max_tiles]) return;
    bank = tt[tile];
    row0 = tt[p.max_tiles + tile];
    nrows = tt[2 * p.max_tiles + tile];
    n0 = static_cast<int64_t>(nt) * kOutCols;
    if (bank < 0) {
      // Slack tail: every padded tensor holds zeros there.
      const u32x4 zero = {0, 0, 0, 0};
      for (int c = tid; c < BM * (kOutCols / 8); c += kThreads) {
        const int row = c / (kOutCols / 8);
        const int64_t n = n0 + (c % (kOutCols / 8)) * 8;
        if (row < nrows && n < p.N) {
          const int64_t r = row0 + row;
          if constexpr (kUpGateFwd) {
            if (p.out != nullptr) {
              st16o(p.out + r * p.ldo + n, zero);
              st16o(p.out + r * p.ldo + p.N + n, zero);
            }
            st16o(p.out2 + r * p.ldo2 + n, zero);
          } else {
            st16o(p.out + r * p.ldo + n, zero);
          }
        }
      }
      return;
    }
  }

  int num_kt, kt_per_phase = 1;
  if constexpr (kMode == kTN) {
    num_kt = seg_end > seg_begin ? static_cast<int>((seg_end - seg_begin + BK - 1) / BK) : 0;
  } else {
    kt_per_phase = static_cast<int>((p.K + BK - 1) / BK);
    num_kt = kMode == kNTUpGate ? 2 * kt_per_phase : kt_per_phase;
  }
  const uint16_t* a_rows = p.a + static_cast<int64_t>(row0) * p.lda;

  u32x4 ra[C::A_CHUNKS], rb[C::B_CHUNKS];
  const u32x4 zero4 = {0, 0, 0, 0};

  // Global -> register tile loads.  Every load is unconditional: indices that
  // fall outside the tile are clamped to a valid element (their products only
  // reach output rows / columns that are never stored), and only the partial
  // last step of the contraction (kTail) zeroes what it must not sum.
  bool has_tail;
  if constexpr (kMode == kTN)
    has_tail = ((seg_end - seg_begin) % BK) != 0;
  else
    has_tail = (p.K % BK) != 0;
  const int last_row = nrows - 1;

  auto load_a = [&](int kt, auto tail_tag) {
    constexpr bool kTail = decltype(tail_tag)::value;
    if constexpr (kAContig) {
      const int phase = kMode == kNTUpGate ? kt / kt_per_phase : 0;
      const int64_t k0 = static_cast<int64_t>(kt - phase * kt_per_phase) * BK;
      const int64_t col0 = kMode == kNTUpGate ? phase * p.K : 0;
#pragma unroll
      for (int i = 0; i < C::A_CHUNKS; ++i) {
        const int c = tid + kThreads * i;
        int row = c / (BK / 8);
        row = row < last_row ? row : last_row;
        const int64_t k = k0 + (c % (BK / 8)) * 8;
        if constexpr (kTail) {
          const bool ok = k < p.K;
          const u32x4 v = ld16(a_rows + row * p.lda + col0 + (ok ? k : 0));
          ra[i] = ok ? v : zero4;
        } else {
          ra[i] = ld16(a_rows + row * p.lda + col0 + k);
        }
      }
    } else {
      const int64_t r0 = seg_begin + static_cast<int64_t>(kt) * BK;
#pragma unroll
      for (int i = 0; i < C::A_CHUNKS; ++i) {
        const int c = tid + kThreads * i;
        const int64_t r = r0 + c / (BM / 8);
        int64_t m = m0 + (c % (BM / 8)) * 8;
        m = m < p.M ? m : p.M - 8;
        if constexpr (kTail) {
          const bool ok = r < seg_end;
          const u32x4 v = ld16(p.a + (ok ? r : seg_begin) * p.lda + m);
          ra[i] = ok ? v : zero4;
        } else {
          ra[i] = ld16(p.a + r * p.lda + m);
        }
      }
    }
  };
  auto load_b = [&](int kt, auto tail_tag) {
    constexpr bool kTail = decltype(tail_tag)::value;
    if constexpr (kMode == kTN) {
      const int64_t r0 = seg_begin + static_cast<int64_t>(kt) * BK;
      const uint16_t* g = reinterpret_cast<const uint16_t*>(p.b0);
#pragma unroll
      for (int i = 0; i < C::B_CHUNKS; ++i) {
        const int c = tid + kThreads * i;
        const int64_t r = r0 + c / (BN / 8);
        int64_t n = n0 + (c % (BN / 8)) * 8;
        n = n < p.N ? n : p.N - 8;
        if constexpr (kTail) {
          const bool ok = r < seg_end;
          const u32x4 v = ld16(g + (ok ? r : seg_begin) * p.ldb + n);
          rb[i] = ok ? v : zero4;
        } else {
          rb[i] = ld16(g + r * p.ldb + n);
        }
      }
    } else if constexpr (kBContig) {
      const int phase = kMode == kNTUpGate ? kt / kt_per_phase : 0;
      const int64_t k0 = static_cast<int64_t>(kt - phase * kt_per_phase) * BK;
      const uint16_t* b = reinterpret_cast<const uint16_t*>(phase == 0 ? p.b0 : p.b1) +
                          bank * p.bank_stride;
#pragma unroll
      for (int i = 0; i < C::B_CHUNKS; ++i) {
        const int c = tid + kThreads * i;
        int64_t n = n0 + c / (BK / 8);
        n = n < p.N ? n : p.N - 1;
        const int64_t k = k0 + (c % (BK / 8)) * 8;
        if constexpr (kTail) {
          const bool ok = k < p.K;
          const u32x4 v = ld16(b + n * p.ldb + (ok ? k : 0));
          rb[i] = ok ? v : zero4;
        } else {
          rb[i] = ld16(b + n * p.ldb + k);
        }
      }
    } else {
      const int64_t k0 = static_cast<int64_t>(kt) * BK;
#pragma unroll
      for (int i = 0; i < C::B_CHUNKS; ++i) {
        const int c = tid + kThreads * i;
        const int64_t k = k0 + c / (BN / 8);
        const int nc = c % (BN / 8);
        const bool ok = !kTail || k < p.K;
        const int64_t kr = ok ? k : 0;
        u32x4 v;
        if constexpr (kMode == kNNUpGate) {
          constexpr int kHalf = BN / 16;  // chunks of the up half
          const uint16_t* b = reinterpret_cast<const uint16_t*>(nc < kHalf ? p.b0 : p.b1) +
                              bank * p.bank_stride;
          int64_t n = n0 + (nc % kHalf) * 8;
          n = n < p.N ? n : p.N - 8;
          v = ld16(b + kr * p.ldb + n);
        } else if constexpr (kMode == kNNFp8W) {
          const uint8_t* b = reinterpret_cast<const uint8_t*>(p.b0) + bank * p.bank_stride;
          int64_t n = n0 + nc * 8;
          n = n < p.N ? n : p.N - 8;
          const int64_t at = p.tile_stride != 0 ? (n >> 7) * p.tile_stride + kr * 128 + (n & 127)
                                                : kr * p.ldb + n;
          v = fp8x8_to_bf16x8(*reinterpret_cast<const u32x2*>(b + at));
        } else {
          const uint16_t* b = reinterpret_cast<const uint16_t*>(p.b0) + bank * p.bank_stride;
          int64_t n = n0 + nc * 8;
          n = n < p.N ? n : p.N - 8;
          v = ld16(b + kr * p.ldb + n);
        }
        rb[i] = ok ? v : zero4;
      }
    }
  };
  auto load_full = [&](int kt) {  // a step known not to be the partial last one
    load_a(kt, std::false_type{});
    load_b(kt, std::false_type{});
  };
  // The partial step closes the contraction -- of each of the two phases when
  // the contraction runs over the up and the gate half in turn.
  auto is_tail = [&](int kt) {
    if (!has_tail) return false;
    if constexpr (kMode == kNTUpGate) return (kt % kt_per_phase) == kt_per_phase - 1;
    return kt == num_kt - 1;
  };
  auto load_tiles = [&](int kt) {
    if (is_tail(kt)) {
      load_a(kt, std::true_type{});
      load_b(kt, std::true_type{});
    } else {
      load_full(kt);
    }
  };
  auto store_tiles = [&](int stage) {
    uint16_t* sa = lds + stage * (C::A_ELEMS + C::B_ELEMS);
    uint16_t* sb = sa + C::A_ELEMS;
#pragma unroll
    for (int i = 0; i < C::A_CHUNKS; ++i) {
      const int c = tid + kThreads * i;
      if constexpr (kAContig)
        *reinterpret_cast<u32x4*>(sa + (c / (BK / 8)) * A_LD + (c % (BK / 8)) * 8) = ra[i];
      else
        *reinterpret_cast<u32x4*>(sa + (c / (BM / 8)) * A_LD + (c % (BM / 8)) * 8) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < C::B_CHUNKS; ++i) {
      const int c = tid + kThreads * i;
      if constexpr (kBContig)
        *reinterpret_cast<u32x4*>(sb + (c / (BK / 8)) * B_LD + (c % (BK / 8)) * 8) = rb[i];
      else
        *reinterpret_cast<u32x4*>(sb + (c / (BN / 8)) * B_LD + (c % (BN / 8)) * 8) = rb[i];
    }
  };

  f32x16 acc[C::MI][C::NJ];
#pragma unroll
  for (int i = 0; i < C::MI; ++i)
#pragma unroll
    for (int j = 0; j < C::NJ; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  // Fragment addressing (per lane).
  const int kc_row = lane & 31, kc_k = 8 * (lane >> 5);
  const int tr_krow = 8 * (lane >> 5) + ((lane & 15) >> 2);
  const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  auto read_frags = [&](const uint16_t* sa, const uint16_t* sb, int kk, bf16x8* fa, bf16x8* fb) {
#pragma unroll
    for (int i = 0; i < C::MI; ++i) {
      if constexpr (kAContig)
        fa[i] = lds_read_kc<A_LD>(sa, C::WTM * wm + 32 * i + kc_row, 16 * kk + kc_k);
      else
        fa[i] = lds_read_tr<A_LD>(sa, 16 * kk + tr_krow, C::WTM * wm + 32 * i + tr_col);
    }
#pragma unroll
    for (int j = 0; j < C::NJ; ++j) {
      if constexpr (kBContig)
        fb[j] = lds_read_kc<B_LD>(sb, C::WTN * wn + 32 * j + kc_row, 16 * kk + kc_k);
      else
        fb[j] = lds_read_tr<B_LD>(sb, 16 * kk + tr_krow, C::WTN * wn + 32 * j + tr_col);
    }
  };

  // Fragment registers persist across K steps: the first fragment of step t+1
  // is read behind the last MFMAs of step t.
  bf16x8 fa[2][C::MI], fb[2][C::NJ];
  static_assert(C::KK % 2 == 0, "fragment double-buffer parity");
  constexpr int kReads = (kAContig ? C::MI : 2 * C::MI) + (kBContig ? C::NJ : 2 * C::NJ);
  constexpr int kWrites = C::A_CHUNKS + C::B_CHUNKS;
  constexpr int kMfma = C::MI * C::NJ;
  using MfmaSeq = std::make_integer_sequence<int, kMfma>;

  // One K step.  kStore: the tile of step kt+1 (already in registers) goes to
  // the idle LDS buffer.  kLoad: 0 = nothing left to fetch, 1 = fetch step kt+2
  // (a full step), 2 = fetch step kt+2 (possibly the partial last one).
  auto k_step = [&](int kt, auto store_tag, auto load_tag) {
    constexpr bool kStore = decltype(store_tag)::value;
    constexpr int kLoad = decltype(load_tag)::value;
    const int cur = kt & 1;
    const uint16_t* sa = lds + cur * (C::A_ELEMS + C::B_ELEMS);
    const uint16_t* sb = sa + C::A_ELEMS;
    const uint16_t* na = lds + (cur ^ 1) * (C::A_ELEMS + C::B_ELEMS);
    const uint16_t* nb = na + C::A_ELEMS;
    if constexpr (kStore) store_tiles(cur ^ 1);
    if constexpr (kLoad == 1) load_full(kt + 2);
    if constexpr (kLoad == 2) load_tiles(kt + 2);
#pragma unroll
    for (int kk = 0; kk < C::KK; ++kk) {
      if (kk + 1 < C::KK) {
        read_frags(sa, sb, kk + 1, fa[(kk + 1) & 1], fb[(kk + 1) & 1]);
      } else {
        // Everyone has written the next buffer and read its last fragment of
        // this one; the only barrier of the step.
        __syncthreads();
        if constexpr (kStore) read_frags(na, nb, 0, fa[0], fb[0]);
      }
#pragma unroll
      for (int i = 0; i < C::MI; ++i)
#pragma unroll
        for (int j = 0; j < C::NJ; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[kk & 1][j], fa[kk & 1][i],
                                                               acc[i][j], 0, 0, 0);
      if (kk == 0)
        interleave_memory<kReads, kStore ? kWrites : 0, 0, kMfma>(MfmaSeq{});
      else if (kk + 1 < C::KK)
        interleave_memory<kReads, 0, 0, kMfma>(MfmaSeq{});
      else
        interleave_memory<kStore ? kReads : 0, 0, kLoad == 1 ? kWrites : 0, kMfma>(MfmaSeq{});
    }
  };

  if (num_kt > 0) {
    load_tiles(0);
    store_tiles(0);
    if (num_kt > 1) load_tiles(1);
    __syncthreads();
    read_frags(lds, lds + C::A_ELEMS, 0, fa[0], fb[0]);
    using Store = std::true_type;
    using NoStore = std::false_type;
    int kt = 0;
    // Steady state: the fetched step kt+2 is never a partial one (a two-phase
    // contraction with a partial step per phase takes the checking variant).
    if (kMode == kNTUpGate && has_tail) {
      for (; kt + 3 < num_kt; ++kt) k_step(kt, Store{}, std::integral_constant<int, 2>{});
    } else {
      for (; kt + 3 < num_kt; ++kt) k_step(kt, Store{}, std::integral_constant<int, 1>{});
    }
    if (kt + 2 < num_kt) {
      k_step(kt, Store{}, std::integral_constant<int, 2>{});
      ++kt;
    }
    if (kt + 1 < num_kt) {
      k_step(kt, Store{}, std::integral_constant<int, 0>{});
      ++kt;
    }
    k_step(kt, NoStore{}, std::integral_constant<int, 0>{});
  } else {
    __syncthreads();
  }

  // ---- epilogue: bf16 tile through LDS, then coalesced 128-bit stores -----
  uint16_t* stage = lds;
  const float* col_scale = kMode == kNNFp8W ? p.scale + bank * p.N : nullptr;
#pragma unroll
  for (int i = 0; i < C::MI; ++i)
#pragma unroll
    for (int j = 0; j < C::NJ; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int m = C::WTM * wm + 32 * i + (lane & 31);
        const int n = C::WTN * wn + 32 * j + 8 * q + 4 * (lane >> 5);
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if constexpr (C::MI * C::NJ == 16) {
            // 256 accumulator registers live in AGPRs; reading them where they
            // are used keeps the compiler from hoisting every read and spilling.
            asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v[e]) : "a"(acc[i][j][4 * q + e]));
          } else {
            v[e] = acc[i][j][4 * q + e];
          }
        }
        if constexpr (kMode == kNNFp8W) {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] *= (n0 + n + e < p.N) ? col_scale[n0 + n + e] : 0.0f;
        }
        u32x2 packed = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
        *reinterpret_cast<u32x2*>(stage + m * C::STAGE_LD + n) = packed;
      }
  __syncthreads();
  if constexpr (kUpGateFwd) {
    constexpr int kHalfChunks = BN / 16;
    for (int c = tid; c < BM * kHalfChunks; c += kThreads) {
      const int row = c / kHalfChunks;
      const int hc = c % kHalfChunks;
      const int64_t n = n0 + hc * 8;
      if (row < nrows && n < p.N) {
        const int64_t r = row0 + row;
        const u32x4 up = *reinterpret_cast<const u32x4*>(stage + row * C::STAGE_LD + hc * 8);
        const u32x4 gate =
            *reinterpret_cast<const u32x4*>(stage + row * C::STAGE_LD + BN / 2 + hc * 8);
        if (p.out != nullptr) {
          st16o(p.out + r * p.ldo + n, up);
          st16o(p.out + r * p.ldo + p.N + n, gate);
        }
        float u[8], g[8], h[8];
        unpack8(up, u);
        unpack8(gate, g);
#pragma unroll
        for (int e = 0; e < 8; ++e) h[e] = silu_rounded(g[e]) * u[e];
        st16o(p.out2 + r * p.ldo2 + n, pack8(h));
      }
    }
  } else if constexpr (kMode == kTN) {
    for (int c = tid; c < BM * (BN / 8); c += kThreads) {
      const int64_t m = m0 + c / (BN / 8);
      const int64_t n = n0 + (c % (BN / 8)) * 8;
      if (m < p.M && n < p.N) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(stage + (c / (BN / 8)) * C::STAGE_LD +
                                                        (c % (BN / 8)) * 8);
        if (p.out_f32) {
          // this general kernel rounds to bf16 on the way through LDS; widened here
          float f[8];
          unpack8(v, f);
          store8_from_f32<true>(reinterpret_cast<float*>(p.out) + bank * p.bank_stride,
                                m * p.ldo + n, f);
        } else {
          st16o(p.out + bank * p.bank_stride + m * p.ldo + n, v);
        }
      }
    }
  } else {
    for (int c = tid; c < BM * (BN / 8); c += kThreads) {
      const int row = c / (BN / 8);
      const int64_t n = n0 + (c % (BN / 8)) * 8;
      if (row < nrows && n < p.N)
        st16o(p.out + (row0 + row) * p.ldo + n,
             *reinterpret_cast<const u32x4*>(stage + row * C::STAGE_LD + (c % (BN / 8)) * 8));
    }
  }
}

// ---------------------------------------------------------------------------
// Direct-to-LDS variant.  Operand tiles go HBM -> LDS with
// global_load_lds_dwordx4 (no staging registers, no LDS write instructions)
// into a ring of three unpadded LDS stages, so the fetch of step t+2 is in
// flight during the whole of steps t and t+1.  A wavefront instruction deposits
// 64 lanes x 16 bytes as one contiguous KiB, so bank conflicts are avoided not
// by padding rows but by choosing WHICH 16-byte piece of the tile each lane
// fetches: position (row, c) of a contraction-contiguous tile holds logical
// piece c ^ f(row); a contraction-major tile XORs the 32-byte column block with
// the low bits of its row.  Fragment reads apply the same XOR.
//
// Tiles are as tall as their table entry says, up to C::BM rows: a wavefront
// multiplies mi = ceil(ceil(rows / 32) / WGM) of its C::MI row blocks (the same
// count in every wavefront row) and the wavefront rows sit 32 * mi rows apart, so
// a tile of 96 or of 160 rows costs its own blocks and nothing else.  The balanced
// tile tables use that: a segment's 32-row blocks are dealt evenly over the fewest
// tiles instead of leaving a short last tile that would stream a whole weight panel
// for a few rows.  Four row blocks accumulate in the accumulation registers; a
// fifth (C::MI == 5) accumulates in ordinary vector registers through the
// vector-register form of the MFMA, issued as inline assembly (the compiler
// only ever picks one register class for all of a kernel's MFMAs).
//
// Requirement checked by the launcher: the contraction length is a multiple of
// BK.  Row-tiled modes only; the weight gradient has its own kernel below.
// A-stage transfer instructions per lane that a tile of mi row blocks per wavefront row
// needs: its 32 * mi * WGM rows, in whole instructions.
template <typename C>
constexpr int a_chunks_needed(int mi) {
  return (32 * mi * C::WGM + C::A_ROW_UNIT - 1) / C::A_ROW_UNIT;
}

__device__ __forceinline__ void mfma_vgpr(f32x16& c, bf16x8 a, bf16x8 b) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
}

// kRagK: the contraction length is not a multiple of BK (any multiple of 8 goes).  The
// last K step of each phase then fetches, in place of the pieces behind the
// contraction's end, pieces in front of it (finite values from inside the operand) and
// multiplies them with A fragments zeroed in registers; the per-transfer offset
// correction costs two vector instructions per transfer, which is why contractions
// that are multiples of BK keep the variant without it.
template <typename C, int kMode, bool kRagK>
__global__ __launch_bounds__(C::THREADS, C::OCC) void grouped_gemm_dma_kernel(GemmParams p) {
  static_assert(kMode != kTN && kMode != kNNFp8W, "row-tiled bf16 modes");
  constexpr int kThreads = C::THREADS, kWaves = C::WAVES;
  extern __shared__ __align__(16) uint16_t lds[];
  constexpr int BM = C::BM, BN = C::BN, BK = C::BK;
  constexpr bool kUpGateFwd = kMode == kNNUpGate;
  constexpr bool kBContig = kMode == kNT || kMode == kNTUpGate;
  constexpr int kOutCols = kUpGateFwd ? BN / 2 : BN;
  // The forward up|gate tile is two contraction-major sub-tiles side by side
  // (up columns, gate columns) so that one DMA instruction reads one bank.  A
  // wavefront multiplies WTN / 2 columns of the up sub-tile and the same columns of
  // the gate sub-tile, so each lane ends up with matching up and gate values.
  constexpr int kSub = kUpGateFwd ? 2 : 1;
  constexpr int BW = BN / kSub;
  static_assert(!kUpGateFwd || (C::NJ % 2 == 0), "half of a wavefront's column blocks are up, half gate");
  constexpr int kStageElems = C::A_ELEMS + C::B_ELEMS;
  constexpr int kAccMi = C::MI < 4 ? C::MI : 4;  // row blocks held in accumulation registers
  constexpr bool kAgprReads = kAccMi * C::NJ == 16;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wavefront-uniform: keep it scalar
  const int wm = wave / C::WGN;
  const int wn = wave % C::WGN;

  // Workgroup b runs on XCD b % 8.  For the GEMMs with few column tiles and a
  // long contraction (down projection, fused up|gate input gradient) each XCD
  // takes groups of consecutive row tiles with all their column tiles, so the
  // tiles that share an activation panel and the tiles that share a weight panel
  // meet in the same L2.  The GEMMs that stream wide weight panels once do as well
  // when all XCDs walk the same expert at the same time, each on its own column
  // tiles (plain order, column tile fastest).
  int tile, nt;
  if (p.tile_group > 0) {
    const int xcd = blockIdx.x & 7;
    const int local = blockIdx.x >> 3;
    const int per_group = p.tile_group * p.n_tiles;
    const int group = local / per_group;
    const int within = local - group * per_group;
    if (p.tile_order == 0) {
      tile = (group * 8 + xcd) * p.tile_group + within / p.n_tiles;
      nt = within % p.n_tiles;
    } else {
      // row tile fastest: the row tiles of a group that share a column tile (and its
      // weight panel) are consecutive workgroups of one XCD
      tile = (group * 8 + xcd) * p.tile_group + within % p.tile_group;
      nt = within / p.tile_group;
    }
  } else {
    tile = blockIdx.x / p.n_tiles;
    nt = blockIdx.x % p.n_tiles;
  }
  const int32_t* tt = p.tile_table;
  if (tile >= tt[3 * p.max_tiles]) return;
  const int bank = tt[tile];
  const int row0 = tt[p.max_tiles + tile];
  int nrows = tt[2 * p.max_tiles + tile];
  nrows = nrows < BM ? nrows : BM;  // the launcher pairs every configuration with a table it covers
  const int64_t n0 = static_cast<int64_t>(nt) * kOutCols;
  if (bank < 0) {
    const u32x4 zero = {0, 0, 0, 0};
    for (int c = tid; c < BM * (kOutCols / 8); c += kThreads) {
      const int row = c / (kOutCols / 8);
      const int64_t n = n0 + (c % (kOutCols / 8)) * 8;
      if (row < nrows && n < p.N) {
        const int64_t r = row0 + row;
        if constexpr (kUpGateFwd) {
          if (p.out != nullptr) {
            st16o(p.out + r * p.ldo + n, zero);
            st16o(p.out + r * p.ldo + p.N + n, zero);
          }
          st16o(p.out2 + r * p.ldo2 + n, zero);
        } else {
          st16o(p.out + r * p.ldo + n, zero);
        }
      }
    }
    return;
  }

  const int kt_per_phase = static_cast<int>((p.K + BK - 1) / BK);
  const int num_kt = kMode == kNTUpGate ? 2 * kt_per_phase : kt_per_phase;
  const int k_rem = static_cast<int>(p.K % BK);  // kRagK: valid contraction indices of a phase's last step
#if NESTOR_GEMM_CLOCK_HOOK
  unsigned long long clk_c0 = 0, clk_w0 = 0;
  if (p.clock_sink != nullptr) {
    clk_c0 = clock64();
    clk_w0 = wall_clock64();
  }
#endif

  // Row blocks per wavefront in this tile, and where this wavefront's rows start.
  int mi_eff = (((nrows + 31) >> 5) + C::WGM - 1) / C::WGM;
  mi_eff = mi_eff < 1 ? 1 : (mi_eff > C::MI ? C::MI : mi_eff);
  mi_eff = __builtin_amdgcn_readfirstlane(mi_eff);
  const int wave_row0 = 32 * mi_eff * wm;

  // Per-lane byte offsets of every DMA instruction relative to a wavefront-uniform
  // base that advances with the K step (and carries the row / bank origin).  Rows
  // behind the tile's last one (also the rows that only round the A stage up to
  // whole instructions) fetch the last row again: what they feed is never stored.
  uint32_t offa[C::A_CHUNKS], offb[C::B_CHUNKS];
  const int last_row = nrows - 1;
#pragma unroll
  for (int i = 0; i < C::A_CHUNKS; ++i)
    offa[i] = dma::a_lane_offset<BK>((wave + kWaves * i) * 64 + lane, last_row, p.lda);
  // Column origin of the tile: part of the scalar base; the last column tile of a ragged
  // width is clamped per lane.
#pragma unroll
  for (int i = 0; i < C::B_CHUNKS; ++i) {
    const int ci = (wave + kWaves * i) * 64 + lane;
    if constexpr (kBContig) offb[i] = dma::b_contig_lane_offset<BK>(ci, n0, p.N, p.ldb);
    else offb[i] = dma::b_major_lane_offset<BK, BW>(ci, n0, p.N, p.ldb);
  }
  // kRagK: what a phase's last K step subtracts from those offsets
  uint32_t adja[kRagK ? C::A_CHUNKS : 1], adjb[kRagK ? C::B_CHUNKS : 1];
  if constexpr (kRagK) {
#pragma unroll
    for (int i = 0; i < C::A_CHUNKS; ++i)
      adja[i] = dma::kc_partial_adjust<BK>((wave + kWaves * i) * 64 + lane, k_rem);
#pragma unroll
    for (int i = 0; i < C::B_CHUNKS; ++i) {
      const int ci = (wave + kWaves * i) * 64 + lane;
      if constexpr (kBContig) adjb[i] = dma::kc_partial_adjust<BK>(ci, k_rem);
      else adjb[i] = dma::b_major_partial_adjust<BK, BW>(ci, k_rem, p.ldb);
    }
  }
  const uint16_t* a_origin = p.a + static_cast<int64_t>(row0) * p.lda;
  const int64_t b_origin = bank * p.bank_stride + (kBContig ? n0 * p.ldb : n0);

  // DMA instruction q (A pieces first, then B pieces) of K step kt into ring
  // stage `stage`.  Steps past the end re-fetch the last step: the extra tile
  // lands in a stage nobody reads again, and every step then issues the same
  // number of instructions, which keeps the vmcnt bookkeeping uniform.
  // Byte offsets of a K step fit 32 bits (checked on the host): the step's scalar
  // base is one 32-bit multiply and a 64-bit add, shared by the step's instructions.
  const uint32_t a_step = BK * 2;
  const uint32_t b_step = static_cast<uint32_t>(kBContig ? BK * 2 : BK * 2 * p.ldb);
  const char* a_bytes = reinterpret_cast<const char*>(a_origin);
  const char* b0_bytes = reinterpret_cast<const char*>(reinterpret_cast<const uint16_t*>(p.b0) + b_origin);
  const char* b1_bytes = reinterpret_cast<const char*>(reinterpret_cast<const uint16_t*>(p.b1) + b_origin);
  const uint32_t wave_lds = lds_byte_addr(lds) + wave * 1024;
  // a_tag: how many A instructions per lane the tile's height needs (the rows behind
  // 32 * mi * WGM are never read, so a short tile does not fetch them).
  auto issue_one = [&](int kt, int stage, auto a_tag, auto q_tag) __attribute__((always_inline)) {
    constexpr int kA = decltype(a_tag)::value;
    constexpr int q = decltype(q_tag)::value;
    kt = kt < num_kt ? kt : num_kt - 1;
    const uint32_t stage_lds = wave_lds + stage * (kStageElems * 2);
    // all ones in a phase's last (partial) K step, else zero: wavefront-uniform
    uint32_t part = 0;
    uint32_t a_col_bytes = static_cast<uint32_t>(kt) * a_step;
    if constexpr (kRagK) {
      const int phase = (kMode == kNTUpGate && kt >= kt_per_phase) ? 1 : 0;
      const int in_phase = kt - phase * kt_per_phase;
      part = in_phase == kt_per_phase - 1 ? 0xffffffffu : 0u;
      // the second phase's columns start at K, which is not a whole number of K steps here
      a_col_bytes = static_cast<uint32_t>(phase) * static_cast<uint32_t>(p.K * 2) +
                    static_cast<uint32_t>(in_phase) * a_step;
    }
    if constexpr (q < kA) {
      uint32_t off = offa[q];
      if constexpr (kRagK) off -= adja[q] & part;
      dma16s<q * kWaves * 1024>(a_bytes + a_col_bytes, off, stage_lds);
    } else {
      constexpr int i = q - kA;
      constexpr int kLdsOff = C::A_ELEMS * 2 + i * kWaves * 1024;
      const char* base;
      if constexpr (kBContig) {
        const int phase = (kMode == kNTUpGate && kt >= kt_per_phase) ? 1 : 0;
        base = (phase == 0 ? b0_bytes : b1_bytes) +
               static_cast<uint32_t>(kt - phase * kt_per_phase) * b_step;
      } else {
        // blocks of the second sub-tile (the gate bank) are the upper half of the
        // instructions: wave + kWaves * i >= kBlkPerSub for every wavefront
        constexpr int kBlkPerSub = BK * BW / 8 / 64;
        static_assert(kSub == 1 || kBlkPerSub % kWaves == 0, "a sub-tile is whole instructions");
        constexpr bool kSecond = kSub == 2 && i * kWaves >= kBlkPerSub;
        base = (kSecond ? b1_bytes : b0_bytes) + static_cast<uint32_t>(kt) * b_step;
      }
      uint32_t off = offb[i];
      if constexpr (kRagK) off -= adjb[i] & part;
      dma16s<kLdsOff>(base, off, stage_lds);
    }
  };

  f32x16 acc[kAccMi][C::NJ];
  f32x16 accv[C::NJ];  // the fifth row block (C::MI == 5 only)
#pragma unroll
  for (int i = 0; i < kAccMi; ++i)
#pragma unroll
    for (int j = 0; j < C::NJ; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  const int kc_row = lane & 31, kc_piece = lane >> 5;
  const int tr_krow = 8 * (lane >> 5) + ((lane & 15) >> 2);
  const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  const int a_wave_elems = wave_row0 * BK;  // this wavefront's first row inside an A stage
  // Fragment read r of a fragment set into the registers of parity `par`, in
  // the order the MFMAs consume them: B fragment 0, the A fragments, then the
  // remaining B fragments.
  bf16x8 fa[2][C::MI], fb[2][C::NJ];
  auto read_one = [&](const uint16_t* sa, const uint16_t* sb, int kk, int r, int par, int mi_n) __attribute__((always_inline)) {
    if (r >= 1 && r <= mi_n) {
      const int i = r - 1;
      // wave_row0 is a multiple of 32 rows: the swizzle of a row depends on its low bits only
      fa[par][i] = *reinterpret_cast<const bf16x8*>(sa + a_wave_elems +
                                                    kc_offset<BK>(32 * i + kc_row, 2 * kk + kc_piece));
    } else {
      const int j = r == 0 ? 0 : r - mi_n;
      if constexpr (kBContig) {
        const int row = C::WTN * wn + 32 * j + kc_row;
        fb[par][j] = *reinterpret_cast<const bf16x8*>(sb + kc_offset<BK>(row, 2 * kk + kc_piece));
      } else {
        // column inside the B tile: its sub-tile, and the column inside that
        const int half = kUpGateFwd ? j / (C::NJ / 2) : 0;
        const int col = kUpGateFwd ? (C::WTN / 2) * wn + 32 * (j % (C::NJ / 2)) : C::WTN * wn + 32 * j;
        const uint16_t* sub = sb + (kUpGateFwd ? half : col / BW) * (BK * BW);
        const int k = 16 * kk + tr_krow;
        const int n = (col % BW) + tr_col;
        fb[par][j] = lds_read_tr_pair<BW>(sub + nc_offset<BW>(k, n));
      }
    }
  };

  constexpr int S = C::kStages;

  // One block of MFMAs on the fragment set of parity `par`, with this block's
  // share of the memory instructions placed between them in program order:
  // the reads of the next fragment set (into parity par ^ 1) and share `share_tag`
  // of the DMA instructions of K step lt (a step's instructions are dealt over its KK
  // blocks: share s is [s * kLoads / KK, (s + 1) * kLoads / KK)).  The scheduling barriers pin that order:
  // memory instructions issued in a burst back up the address path and stall the
  // wavefront's matrix instructions behind them.
  // mi_tag: how many of the wavefront's 32-row blocks hold rows of the tile; the
  // MFMAs and A fragments of the others are skipped.
  // ckk: the K sub-step (of 16) whose fragments this block multiplies when its K step is a
  // phase's partial last one, else -1 (kRagK only).
  auto mfma_block = [&](auto mi_tag, int par, auto reads_tag, const uint16_t* ra, const uint16_t* rb,
                        int rkk, int lt, int ls, auto share_tag, int ckk) __attribute__((always_inline)) {
    constexpr int kMi = decltype(mi_tag)::value;
    constexpr bool kDoReads = decltype(reads_tag)::value;
    constexpr int kMfmaEff = kMi * C::NJ, kReadsEff = kMi + C::NJ;
    using ATag = std::integral_constant<int, a_chunks_needed<C>(kMi)>;
    constexpr int kLoads = ATag::value + C::B_CHUNKS;
    constexpr int kShare = decltype(share_tag)::value;
    constexpr int kL0 = kShare * kLoads / C::KK;
    constexpr int kLn = (kShare + 1) * kLoads / C::KK - kL0;
    if constexpr (kRagK) {
      // a phase's last K step: the A fragments of contraction indices behind its end are zero
      if (ckk >= 0) {
        const bool dead = 16 * ckk + 8 * kc_piece >= k_rem;
        const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < kMi; ++i) fa[par][i] = dead ? zero : fa[par][i];
      }
    }
    static_for<kMfmaEff>([&](auto mc) __attribute__((always_inline)) {
      constexpr int m = decltype(mc)::value;
      if constexpr (kDoReads) {
#pragma unroll
        for (int r = m * kReadsEff / kMfmaEff; r < (m + 1) * kReadsEff / kMfmaEff; ++r)
          read_one(ra, rb, rkk, r, par ^ 1, kMi);
      }
      constexpr int kQ0 = m * kLn / kMfmaEff, kQ1 = (m + 1) * kLn / kMfmaEff;
      static_for<kQ1 - kQ0>([&](auto qc) __attribute__((always_inline)) {
        issue_one(lt, ls, ATag{}, std::integral_constant<int, kL0 + kQ0 + decltype(qc)::value>{});
      });
      constexpr int j = m / kMi, i = m % kMi;
      if constexpr (i < 4) {
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[par][j], fa[par][i], acc[i][j], 0, 0, 0);
      } else {
        mfma_vgpr(accv[j], fb[par][j], fa[par][i]);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  // K step kt on ring stage cur.  Ring invariant: behind the barrier of step kt
  // every wavefront has finished reading stage cur, so step kt+S is fetched
  // into it, one share of its DMA instructions per MFMA block: the first share
  // behind the barrier, the others in the leading blocks of step kt+1 (where
  // that stage is `prv`).
  auto k_step = [&](auto mi_tag, int kt, int cur, auto next_tag) __attribute__((always_inline)) {
    constexpr bool kNext = decltype(next_tag)::value;
    const int nxt = cur == S - 1 ? 0 : cur + 1;
    const int prv = cur == 0 ? S - 1 : cur - 1;
    const uint16_t* sa = lds + cur * kStageElems;
    const uint16_t* sb = sa + C::A_ELEMS;
    const uint16_t* na = lds + nxt * kStageElems;
    const uint16_t* nb = na + C::A_ELEMS;
    constexpr int kLoads = a_chunks_needed<C>(decltype(mi_tag)::value) + C::B_CHUNKS;
    bool partial = false;
    if constexpr (kRagK) {
      const int in_phase = (kMode == kNTUpGate && kt >= kt_per_phase) ? kt - kt_per_phase : kt;
      partial = in_phase == kt_per_phase - 1;
    }
    static_for<C::KK - 1>([&](auto kc) __attribute__((always_inline)) {
      constexpr int kk = decltype(kc)::value;
      mfma_block(mi_tag, kk & 1, std::true_type{}, sa, sb, kk + 1, kt + S - 1, prv,
                 std::integral_constant<int, kk + 1>{}, partial ? kk : -1);
    });
    if constexpr (kNext) {
      // Step kt+1 has landed once only the later steps' instructions are
      // outstanding: steps kt+2 .. kt+S-1, all issued in full by now.
      wait_vmcnt<(S - 2) * kLoads>();
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      mfma_block(mi_tag, (C::KK - 1) & 1, std::true_type{}, na, nb, 0, kt + S, cur,
                 std::integral_constant<int, 0>{}, partial ? C::KK - 1 : -1);
    } else {
      mfma_block(mi_tag, (C::KK - 1) & 1, std::false_type{}, na, nb, 0, kt + S, cur,
                 std::integral_constant<int, 0>{}, partial ? C::KK - 1 : -1);
    }
  };

  auto k_loop = [&](auto mi_tag) __attribute__((always_inline)) {
    constexpr int kMi = decltype(mi_tag)::value;
    using ATag = std::integral_constant<int, a_chunks_needed<C>(kMi)>;
    constexpr int kLoads = ATag::value + C::B_CHUNKS;
#pragma unroll
    for (int t = 0; t < S; ++t)
      static_for<kLoads>([&](auto qc) __attribute__((always_inline)) { issue_one(t, t, ATag{}, qc); });
    if constexpr (kMi == 5) {
#pragma unroll
      for (int j = 0; j < C::NJ; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) accv[j][e] = 0.0f;
    }
    wait_vmcnt<(S - 1) * kLoads>();
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int r = 0; r < kMi + C::NJ; ++r) read_one(lds, lds + C::A_ELEMS, 0, r, 0, kMi);
    int cur = 0;
    for (int kt = 0; kt + 1 < num_kt; ++kt) {
      k_step(mi_tag, kt, cur, std::true_type{});
      cur = cur == S - 1 ? 0 : cur + 1;
    }
    k_step(mi_tag, num_kt - 1, cur, std::false_type{});
    if constexpr (kMi == 5) {
      // The fifth block's MFMAs are opaque to the compiler's hazard bookkeeping: keep the
      // epilogue's first read of their results behind the matrix pipe's write-back.
      asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory");
    }
  };

  if (num_kt > 0) {
    switch (mi_eff) {
      case 1: k_loop(std::integral_constant<int, 1>{}); break;
      case 2:
        if constexpr (C::MI >= 2) k_loop(std::integral_constant<int, 2>{});
        break;
      case 3:
        if constexpr (C::MI >= 3) k_loop(std::integral_constant<int, 3>{});
        break;
      case 4:
        if constexpr (C::MI >= 4) k_loop(std::integral_constant<int, 4>{});
        break;
      default:
        if constexpr (C::MI >= 5) k_loop(std::integral_constant<int, 5>{});
        break;
    }
  }
  wait_vmcnt<0>();
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();

  // ---- epilogue, per wavefront ----------------------------------------------
  // The ring is drained and nobody reads it again: each wavefront takes a slab of
  // 32 rows x WTN columns in it, writes one row block of its accumulators there as
  // bf16, reads the block back row by row and stores whole 128- or 256-byte row
  // pieces.  No workgroup barrier: the same wavefront wrote and reads, in program
  // order.  Up and gate of a column sit in the same lane (see kSub above), so the
  // fused SwiGLU needs nothing from another wavefront.
  constexpr int kEpiLd = C::EPI_LD;
  uint16_t* slab = lds + wave * (32 * kEpiLd);
  const int col0 = kUpGateFwd ? (C::WTN / 2) * wn : C::WTN * wn;  // first output column in the tile
  static_for<C::MI>([&](auto ic) __attribute__((always_inline)) {
    constexpr int i = decltype(ic)::value;
    const int rbase = wave_row0 + 32 * i;  // tile row of the block's first row
    if (i < mi_eff && rbase < nrows) {
      __builtin_amdgcn_sched_barrier(0);  // one slab's worth of registers at a time
#pragma unroll
      for (int j = 0; j < C::NJ; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = 32 * j + 8 * q + 4 * (lane >> 5);
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if constexpr (i >= 4) {
              v[e] = accv[j][4 * q + e];
            } else if constexpr (kAgprReads) {
              // 256 accumulator registers live in AGPRs; reading them where they
              // are used keeps the compiler from hoisting every read and spilling.
              asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v[e]) : "a"(acc[i][j][4 * q + e]));
            } else {
              v[e] = acc[i][j][4 * q + e];
            }
          }
          u32x2 packed = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
          *reinterpret_cast<u32x2*>(slab + (lane & 31) * kEpiLd + n) = packed;
        }
      if constexpr (kUpGateFwd) {
        constexpr int kHalf = C::WTN / 2;   // up columns of the slab, then the same gate columns
        constexpr int kCpr = kHalf / 8;     // 16-byte pieces per row of either
        constexpr int kPieces = 32 * kCpr / 64;
        u32x4 up[kPieces], gate[kPieces];
#pragma unroll
        for (int t = 0; t < kPieces; ++t) {
          const int c = lane + 64 * t;
          up[t] = *reinterpret_cast<const u32x4*>(slab + (c / kCpr) * kEpiLd + (c % kCpr) * 8);
          gate[t] = *reinterpret_cast<const u32x4*>(slab + (c / kCpr) * kEpiLd + kHalf + (c % kCpr) * 8);
        }
#pragma unroll
        for (int t = 0; t < kPieces; ++t) {
          const int c = lane + 64 * t;
          const int row = rbase + c / kCpr;
          const int64_t n = n0 + col0 + (c % kCpr) * 8;
          if (row < nrows && n < p.N) {
            const int64_t r = row0 + row;
            if (p.out != nullptr) {
              st16o(p.out + r * p.ldo + n, up[t]);
              st16o(p.out + r * p.ldo + p.N + n, gate[t]);
            }
            float u[8], g[8], h[8];
            unpack8(up[t], u);
            unpack8(gate[t], g);
#pragma unroll
            for (int e = 0; e < 8; ++e) h[e] = silu_rounded(g[e]) * u[e];
            st16o(p.out2 + r * p.ldo2 + n, pack8(h));
          }
        }
      } else {
        constexpr int kCpr = C::WTN / 8;
        constexpr int kPieces = 32 * kCpr / 64;
        u32x4 piece[kPieces];
#pragma unroll
        for (int t = 0; t < kPieces; ++t) {
          const int c = lane + 64 * t;
          piece[t] = *reinterpret_cast<const u32x4*>(slab + (c / kCpr) * kEpiLd + (c % kCpr) * 8);
        }
#pragma unroll
        for (int t = 0; t < kPieces; ++t) {
          const int c = lane + 64 * t;
          const int row = rbase + c / kCpr;
          const int64_t n = n0 + col0 + (c % kCpr) * 8;
          if (row < nrows && n < p.N) st16o(p.out + (row0 + row) * p.ldo + n, piece[t]);
        }
      }
    }
  });
#if NESTOR_GEMM_CLOCK_HOOK
  if (p.clock_sink != nullptr && tid == 0) clock_sink_add(p.clock_sink, clk_c0, clk_w0, num_kt);
#endif
}

// ---------------------------------------------------------------------------
// Persistent weight-gradient kernel: out[bank] = a[seg]^T @ g[seg].  A bank's
// contraction is only as long as its segment (a few hundred rows), so a
// one-tile workgroup spends as long filling its pipeline and storing its
// 256 x 256 result as it does multiplying.  Here one workgroup per CU walks a
// list of output tiles with the LDS ring running across tile boundaries: the
// first K steps of the next tile are in flight during the last K steps and the
// epilogue of the current one.
//
// Both operands are contraction-major ([row, column] with the segment row as
// the contraction index), fetched with transposing LDS reads.  The transfers go
// through buffer descriptors that end with the segment's last row: pieces of rows
// behind it arrive as zeros, so no K step needs masking and nothing is assumed
// about rows outside the segments.
// Tile (bank, mt, nt) descriptors of a workgroup's list sit in LDS, filled once
// at start.
template <typename C>
struct WgradLayout {
  static constexpr int kMaxItems = 1024;
  static constexpr int kRingElems = C::kStages * (C::A_ELEMS + C::B_ELEMS);
  static constexpr int kEpiCols = C::WTN;  // bf16 columns of a slab
  static constexpr int kEpiLd = kEpiCols + 8;
  static constexpr int kEpiElems = 32 * kEpiLd;  // one 32-row slab per wavefront
  static constexpr int kTableOffset = kRingElems + C::WAVES * kEpiElems;  // in uint16 units
  static constexpr size_t LDS_BYTES = sizeof(uint16_t) * kTableOffset + 16 * kMaxItems;
  static_assert(LDS_BYTES <= 160 * 1024, "LDS of one CU");
};

// kOutF32: the gradient tile leaves as fp32 straight from the accumulators (no bf16
// rounding): what a bank with fp32 owners wants, instead of a bf16 result that the
// caller widens in another pass over the whole bank.
template <typename C, bool kOutF32>
__global__ __launch_bounds__(C::THREADS, 1) void wgrad_persistent_kernel(GemmParams p, int num_banks) {
  constexpr int kWaves = C::WAVES, kThreads = C::THREADS;
  extern __shared__ __align__(16) uint16_t lds[];
  constexpr int BM = C::BM, BN = C::BN, BK = C::BK, S = C::kStages;
  constexpr int kStageElems = C::A_ELEMS + C::B_ELEMS;
  constexpr int kLoads = C::A_CHUNKS + C::B_CHUNKS;
  constexpr int kLoadsPerBlock = kLoads / C::KK;
  constexpr int kReads = C::MI + C::NJ;
  constexpr int kMfma = C::MI * C::NJ;
  using L = WgradLayout<C>;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / C::WGN;
  const int wn = wave % C::WGN;

  // ---- work list -----------------------------------------------------------
  // Output tiles are numbered so that 32 consecutive numbers form a rectangle of
  // 4 row tiles x 8 column tiles of one bank, and consecutive groups of 32 go to
  // consecutive XCDs (workgroup b runs on XCD b % 8): the CUs of an XCD share
  // the rectangle's operand panels through that XCD's L2.
  const int m_tiles = static_cast<int>((p.M + BM - 1) / BM);
  const int n_tiles = static_cast<int>((p.N + BN - 1) / BN);
  const int num_rt = num_banks * m_tiles;  // row tiles over all banks
  const int per_xcd = gridDim.x >> 3;
  const int xcd = blockIdx.x & 7;
  const int slot = blockIdx.x >> 3;
  const bool rect = per_xcd == 32 && (n_tiles & 7) == 0 && (m_tiles & 3) == 0;
  const int band_items = 4 * n_tiles;
  const int w_end = num_rt * n_tiles;
  auto decode = [&](int i, int& rt, int& nt) __attribute__((always_inline)) -> bool {
    const int w = (i * 8 + xcd) * per_xcd + slot;
    if (w >= w_end) return false;
    if (rect) {
      const int band = w / band_items;
      const int r = w - band * band_items;
      rt = band * 4 + ((r & 31) >> 3);
      nt = (r >> 5) * 8 + (r & 7);
    } else {
      rt = w / n_tiles;
      nt = w - rt * n_tiles;
    }
    return true;
  };
  int4* table = reinterpret_cast<int4*>(lds + L::kTableOffset);
  int count = 0;
  {
    int rt, nt;
    while (count < L::kMaxItems && decode(count, rt, nt)) ++count;
  }
  for (int i = tid; i < count; i += kThreads) {
    int rt, nt;
    decode(i, rt, nt);
    const int bank = rt / m_tiles;
    int64_t beg, end;
    if (p.seg_start != nullptr) {
      beg = p.seg_start[bank];
      end = beg + p.seg_count[bank];
    } else {
      beg = bank == 0 ? 0 : p.offs[bank - 1];
      end = p.offs[bank];
    }
    if (end > p.rows_pad) end = p.rows_pad;
    if (end < beg) end = beg;
    table[i] = make_int4(static_cast<int>(beg), static_cast<int>(end), rt, nt);
  }
  __syncthreads();
  if (count == 0) return;
#if NESTOR_GEMM_CLOCK_HOOK
  unsigned long long clk_c0 = 0, clk_w0 = 0, clk_steps = 0;
  if (p.clock_sink != nullptr) {
    clk_c0 = clock64();
    clk_w0 = wall_clock64();
  }
#endif
  auto steps_of = [&](int i) __attribute__((always_inline)) -> int {
    const int4 t = table[i];
    return __builtin_amdgcn_readfirstlane((t.y - t.x + BK - 1) / BK);
  };

  // ---- load cursor -----------------------------------------------------------
  // Each lane fetches the same pieces (contraction row krow of the tile, a fixed
  // group of 8 columns) in every K step of every tile: one 32-bit byte offset per
  // DMA instruction, computed once, into a buffer descriptor per operand that
  // starts at the K step's first segment row and the tile's column origin and ends
  // with the tile's columns of the segment's last row.  Pieces of rows behind the
  // segment end lie beyond the descriptor's num_records and arrive as zeros, so
  // the segment's last, partial K step runs the same instructions as every other
  // and nothing is assumed about rows outside the segments.  A tile that overhangs
  // the operand's width reads on into the next columns of the same rows (inside
  // the operand: the last row's are cut off by num_records); what that
  // contributes goes to output rows / columns that are never stored.  A K step
  // moves the descriptors on by BK rows with scalar arithmetic.
  static_assert(BM / 8 == 32 && BN / 8 == 32, "one DMA instruction covers two contraction rows");
  uint32_t offa[C::A_CHUNKS], offb[C::B_CHUNKS];
#pragma unroll
  for (int c = 0; c < C::A_CHUNKS; ++c) offa[c] = dma::wgrad_lane_offset(wave, kWaves, c, lane, p.lda, BM);
#pragma unroll
  for (int c = 0; c < C::B_CHUNKS; ++c) offb[c] = dma::wgrad_lane_offset(wave, kWaves, c, lane, p.ldb, BN);
  i32x4 desc_a = buffer_descriptor(p.a, 0), desc_b = buffer_descriptor(p.b0, 0);
  // bytes per K step; the launcher checks that a whole operand spans less than 4 GiB
  const uint32_t step_a = static_cast<uint32_t>(BK * p.lda * 2), step_b = static_cast<uint32_t>(BK * p.ldb * 2);
  const uint32_t wave_lds = lds_byte_addr(lds) + wave * 1024;
  int l_item = -1, l_kt = 0, l_steps = 0, l_stage = 0;
  auto move_on = [&](i32x4& d, uint32_t bytes) __attribute__((always_inline)) {
    const uint32_t lo = static_cast<uint32_t>(d[0]) + bytes;
    d[1] += lo < bytes ? 1 : 0;
    d[0] = static_cast<int>(lo);
    d[2] -= static_cast<int>(bytes);
  };
  // Moves the cursor to the first K step of the next tile that has one; false
  // when the list is exhausted (the cursor then stays where it is).
  auto next_load_item = [&]() __attribute__((always_inline)) -> bool {
    int i = l_item + 1;
    while (i < count && steps_of(i) == 0) ++i;
    if (i >= count) return false;
    l_item = i;
    const int4 t = table[i];
    const int beg = __builtin_amdgcn_readfirstlane(t.x);
    const int end = __builtin_amdgcn_readfirstlane(t.y);
    const int rt = __builtin_amdgcn_readfirstlane(t.z);
    const int nt = __builtin_amdgcn_readfirstlane(t.w);
    const int seg_rows = end - beg;
    l_steps = (seg_rows + BK - 1) / BK;
    l_kt = 0;
    const int m0 = (rt % m_tiles) * BM;
    const int n0 = nt * BN;
    // valid bytes from the descriptor's base: whole rows up to the segment's last
    // one, of which the tile's own columns
    desc_a = buffer_descriptor(p.a + static_cast<int64_t>(beg) * p.lda + m0,
                               dma::wgrad_num_records(seg_rows, p.lda, p.M, m0, BM));
    desc_b = buffer_descriptor(
        reinterpret_cast<const uint16_t*>(p.b0) + static_cast<int64_t>(beg) * p.ldb + n0,
        dma::wgrad_num_records(seg_rows, p.ldb, p.N, n0, BN));
    return true;
  };
  // DMA instruction q of the cursor's K step.
  auto issue_one = [&](auto q_tag) __attribute__((always_inline)) {
    constexpr int q = decltype(q_tag)::value;
    constexpr bool kIsA = q < C::A_CHUNKS;
    constexpr int c = kIsA ? q : q - C::A_CHUNKS;
    constexpr int kLdsOff = (kIsA ? 0 : C::A_ELEMS * 2) + c * kWaves * 1024;
    const uint32_t stage_lds = wave_lds + l_stage * (kStageElems * 2);
    if constexpr (kIsA) dma16b<kLdsOff>(desc_a, offa[c], stage_lds);
    else dma16b<kLdsOff>(desc_b, offb[c], stage_lds);
  };
  // Next K step of the work list; past the end the last step is fetched again
  // (into a stage nobody reads), which keeps the vmcnt bookkeeping uniform.
  auto advance = [&]() __attribute__((always_inline)) {
    l_stage = l_stage == S - 1 ? 0 : l_stage + 1;
    if (l_kt + 1 < l_steps) {
      ++l_kt;
      move_on(desc_a, step_a);
      move_on(desc_b, step_b);
    } else {
      next_load_item();
    }
  };

  // ---- fragments -------------------------------------------------------------
  f32x16 acc[C::MI][C::NJ];
  const int tr_krow = 8 * (lane >> 5) + ((lane & 15) >> 2);
  const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  bf16x8 fa[2][C::MI], fb[2][C::NJ];
  // Element offset of each fragment's first transposing read inside a ring
  // stage; the second K half of the stage and the upper four contraction rows of
  // a fragment are constant offsets from it.
  int frag_a[C::MI], frag_b[C::NJ];
#pragma unroll
  for (int i = 0; i < C::MI; ++i) frag_a[i] = nc_offset<BM>(tr_krow, C::WTM * wm + 32 * i + tr_col);
#pragma unroll
  for (int j = 0; j < C::NJ; ++j)
    frag_b[j] = C::A_ELEMS + nc_offset<BN>(tr_krow, C::WTN * wn + 32 * j + tr_col);
  auto read_one = [&](int stage, auto kk_tag, int r, int par) __attribute__((always_inline)) {
    constexpr int kk = decltype(kk_tag)::value;
    const uint16_t* base = lds + stage * kStageElems;
    if (r >= 1 && r <= C::MI) {
      const int i = r - 1;
      fa[par][i] = lds_read_tr_pair<BM>(base + frag_a[i] + kk * 16 * BM);
    } else {
      const int j = r == 0 ? 0 : r - C::MI;
      fb[par][j] = lds_read_tr_pair<BN>(base + frag_b[j] + kk * 16 * BN);
    }
  };
  // first_tag: the block opens a tile's contraction.  Its products start from a zero
  // constant instead of the accumulator registers, which spares writing 256 zeros
  // per tile (a tile here has only ~16 K steps).
  auto mfma_block = [&](auto first_tag, int par, int rstage, auto rkk_tag, auto l0_tag) __attribute__((always_inline)) {
    constexpr bool kFirst = decltype(first_tag)::value;
    constexpr int l0 = decltype(l0_tag)::value;
    static_for<kMfma>([&](auto mc) __attribute__((always_inline)) {
      constexpr int m = decltype(mc)::value;
#pragma unroll
      for (int r = m * kReads / kMfma; r < (m + 1) * kReads / kMfma; ++r)
        read_one(rstage, rkk_tag, r, par ^ 1);
      constexpr int q_lo = m * kLoadsPerBlock / kMfma, q_hi = (m + 1) * kLoadsPerBlock / kMfma;
      static_for<q_hi - q_lo>([&](auto qc) __attribute__((always_inline)) {
        issue_one(std::integral_constant<int, l0 + q_lo + decltype(qc)::value>{});
      });
      constexpr int j = m / C::MI, i = m % C::MI;
      if constexpr (kFirst) {
        const f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[par][j], fa[par][i], zero, 0, 0, 0);
      } else {
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[par][j], fa[par][i], acc[i][j], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  // ---- epilogue of one output tile, per wavefront -----------------------------
  uint16_t* epi = lds + L::kRingElems + wave * L::kEpiElems;
  auto epilogue = [&](int item) __attribute__((always_inline)) {
    const int4 t = table[item];
    const int rt = __builtin_amdgcn_readfirstlane(t.z);
    const int nt = __builtin_amdgcn_readfirstlane(t.w);
    const int bank = rt / m_tiles;
    const int m0 = (rt - bank * m_tiles) * BM;
    // a pair launch (p.split > 0, a multiple of BN): the column tiles from `split` on belong
    // to the second output
    const bool second = p.split > 0 && static_cast<int64_t>(nt) * BN >= p.split;
    const int n0 = nt * BN - (second ? static_cast<int>(p.split) : 0);
    const int64_t n_end = p.split > 0 ? p.split : p.N;   // columns of one output
    uint16_t* const out_base = second ? p.out2 : p.out;
    if constexpr (kOutF32) {
      // fp32 results through the same per-wavefront slab, half as many columns at a
      // time (32 rows x 64 columns of fp32 fill the space of 32 x 128 of bf16), so that
      // every store instruction still writes whole 256-byte row segments.  (Storing
      // each lane's four columns directly writes 32-byte pieces: 2.7x slower.)
      float* out32 = reinterpret_cast<float*>(out_base) + bank * p.bank_stride;
      float* epi32 = reinterpret_cast<float*>(epi);
      constexpr int kCols32 = L::kEpiCols / 2;  // fp32 columns per pass
      constexpr int kBlk32 = kCols32 / 32;      // column blocks per pass
      constexpr int kLd32 = L::kEpiLd / 2;      // floats per slab row: kCols32 + 4 of padding
      static_assert(L::kEpiLd % 2 == 0 && kLd32 >= kCols32 + 4, "slab row holds a pass's floats");
      static_assert(C::NJ % kBlk32 == 0, "whole passes");
#pragma unroll
      for (int i = 0; i < C::MI; ++i)
#pragma unroll
        for (int jp = 0; jp < C::NJ / kBlk32; ++jp) {
          __builtin_amdgcn_sched_barrier(0);  // one slab's worth of registers at a time
#pragma unroll
          for (int jj = 0; jj < kBlk32; ++jj)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              f32x4 v;
#pragma unroll
              for (int e = 0; e < 4; ++e)
                asm volatile("v_accvgpr_read_b32 %0, %1"
                             : "=v"(v[e])
                             : "a"(acc[i][kBlk32 * jp + jj][4 * q + e]));
              *reinterpret_cast<f32x4*>(epi32 + (lane & 31) * kLd32 + 32 * jj + 8 * q +
                                        4 * (lane >> 5)) = v;
            }
          constexpr int kCpr32 = kCols32 / 4;         // 16-byte pieces per slab row
          constexpr int kPieces32 = 32 * kCpr32 / 64;  // per lane
          f32x4 piece[kPieces32];
#pragma unroll
          for (int t = 0; t < kPieces32; ++t) {
            const int c = lane + 64 * t;
            piece[t] = *reinterpret_cast<const f32x4*>(epi32 + (c / kCpr32) * kLd32 + (c % kCpr32) * 4);
          }
#pragma unroll
          for (int t = 0; t < kPieces32; ++t) {
            const int c = lane + 64 * t;
            const int64_t m = m0 + C::WTM * wm + 32 * i + c / kCpr32;
            const int64_t n = n0 + C::WTN * wn + kCols32 * jp + (c % kCpr32) * 4;
            if (m < p.M && n < n_end)
              __builtin_nontemporal_store(piece[t], reinterpret_cast<f32x4*>(out32 + m * p.ldo + n));
          }
        }
      return;
    }
    uint16_t* out = out_base + bank * p.bank_stride;
    constexpr int kBlk = L::kEpiCols / 32;  // column blocks per pass
#pragma unroll
    for (int i = 0; i < C::MI; ++i)
#pragma unroll
      for (int jg = 0; jg < C::NJ / kBlk; ++jg) {
        __builtin_amdgcn_sched_barrier(0);  // one slab's worth of registers at a time
#pragma unroll
        for (int jj = 0; jj < kBlk; ++jj)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int n = 32 * jj + 8 * q + 4 * (lane >> 5);
            // Read the accumulators where they are used: left to the compiler, all
            // 256 reads move to the top of the epilogue and spill.
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e)
              asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v[e]) : "a"(acc[i][kBlk * jg + jj][4 * q + e]));
            u32x2 packed = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
            *reinterpret_cast<u32x2*>(epi + (lane & 31) * L::kEpiLd + n) = packed;
          }
        // The same wavefront wrote and reads: program order is enough.  All reads
        // go out before the first store so that their latencies overlap.
        constexpr int kCpr = L::kEpiCols / 8;
        constexpr int kPieces = 32 * kCpr / 64;
        u32x4 piece[kPieces];
#pragma unroll
        for (int t = 0; t < kPieces; ++t) {
          const int c = lane + 64 * t;
          piece[t] = *reinterpret_cast<const u32x4*>(epi + (c / kCpr) * L::kEpiLd + (c % kCpr) * 8);
        }
#pragma unroll
        for (int t = 0; t < kPieces; ++t) {
          const int c = lane + 64 * t;
          const int64_t m = m0 + C::WTM * wm + 32 * i + c / kCpr;
          const int64_t n = n0 + C::WTN * wn + L::kEpiCols * jg + (c % kCpr) * 8;
          if (m < p.M && n < n_end) st16o(out + m * p.ldo + n, piece[t]);
        }
      }
  };
  // This wavefront's part of an output tile whose bank has no rows.
  auto store_zero_tile = [&](int item) __attribute__((always_inline)) {
    const int4 t = table[item];
    const int rt = __builtin_amdgcn_readfirstlane(t.z);
    const int nt = __builtin_amdgcn_readfirstlane(t.w);
    const int bank = rt / m_tiles;
    const int m0 = (rt - bank * m_tiles) * BM;
    const bool second = p.split > 0 && static_cast<int64_t>(nt) * BN >= p.split;
    const int n0 = nt * BN - (second ? static_cast<int>(p.split) : 0);
    const int64_t n_end = p.split > 0 ? p.split : p.N;
    uint16_t* const out_base = second ? p.out2 : p.out;
    constexpr int kCpr = C::WTN / 8;
    const u32x4 zero = {0, 0, 0, 0};
    for (int c = lane; c < C::WTM * kCpr; c += 64) {
      const int64_t m = m0 + C::WTM * wm + c / kCpr;
      const int64_t n = n0 + C::WTN * wn + (c % kCpr) * 8;
      if (m < p.M && n < n_end) {
        if constexpr (kOutF32) {
          float* o = reinterpret_cast<float*>(out_base) + bank * p.bank_stride + m * p.ldo + n;
          st16o(o, zero);
          st16o(o + 4, zero);
        } else {
          st16o(out_base + bank * p.bank_stride + m * p.ldo + n, zero);
        }
      }
    }
  };

  // ---- pipeline ----------------------------------------------------------------
  if (!next_load_item()) {
    // every bank of this workgroup's tiles is empty: the gradients are zero
    for (int item = 0; item < count; ++item) store_zero_tile(item);
    return;
  }
#pragma unroll
  for (int t = 0; t + 1 < S; ++t) {
    static_for<kLoads>([&](auto qc) __attribute__((always_inline)) { issue_one(qc); });
    advance();
  }
  static_for<kLoadsPerBlock>([&](auto qc) __attribute__((always_inline)) { issue_one(qc); });
  wait_vmcnt<(S - 2) * kLoads + kLoadsPerBlock>();
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int r = 0; r < kReads; ++r) read_one(0, std::integral_constant<int, 0>{}, r, 0);

  // One K step of the current tile on ring stage cur.
  int cur = 0;
  // inside_tag: the load cursor, S - 1 steps ahead, is known to stay inside its tile,
  // so it moves on without looking at the work list.
  auto k_step = [&](auto first_tag, auto inside_tag) __attribute__((always_inline)) {
    const int nxt = cur == S - 1 ? 0 : cur + 1;
    using K0 = std::integral_constant<int, 0>;
    using K1 = std::integral_constant<int, 1>;
    mfma_block(first_tag, 0, cur, K1{}, std::integral_constant<int, kLoadsPerBlock>{});
    if constexpr (decltype(inside_tag)::value) {
      l_stage = l_stage == S - 1 ? 0 : l_stage + 1;
      ++l_kt;
      move_on(desc_a, step_a);
      move_on(desc_b, step_b);
    } else {
      advance();
    }
    // The next K step has landed once only the later steps' transfers are
    // outstanding.
    wait_vmcnt<(S - 2) * kLoads>();
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    mfma_block(std::false_type{}, 1, nxt, K0{}, K0{});
    cur = nxt;
  };
  for (int item = 0; item < count; ++item) {
    const int num_kt = __builtin_amdgcn_readfirstlane(steps_of(item));
    if (num_kt == 0) {
      // an empty bank: its gradient tile is zero, and nothing of the ring is consumed
      store_zero_tile(item);
      continue;
    }
    // While step kt is multiplied the cursor moves from step kt + S - 1 to step
    // kt + S: inside this tile as long as kt + S < num_kt, behind that into the
    // following tiles.
    if (num_kt > S) {
      k_step(std::true_type{}, std::true_type{});
      for (int kt = 1; kt < num_kt - S; ++kt) k_step(std::false_type{}, std::true_type{});
      for (int kt = num_kt - S < 1 ? 1 : num_kt - S; kt < num_kt; ++kt)
        k_step(std::false_type{}, std::false_type{});
    } else {
      k_step(std::true_type{}, std::false_type{});
      for (int kt = 1; kt < num_kt; ++kt) k_step(std::false_type{}, std::false_type{});
    }
    epilogue(item);
#if NESTOR_GEMM_CLOCK_HOOK
    clk_steps += num_kt;
#endif
  }
  wait_vmcnt<0>();
#if NESTOR_GEMM_CLOCK_HOOK
  if (p.clock_sink != nullptr && tid == 0) clock_sink_add(p.clock_sink, clk_c0, clk_w0, clk_steps);
#endif
}

// Tile configurations.  Row-tiled modes need BM == NESTOR_HIP_TILE_M.
using CfgSmall = Cfg<128, 128, 64, 2, 2>;   // wavefront tile 64 x 64
using CfgWide = Cfg<128, 256, 64, 2, 2>;    // wavefront tile 64 x 128
using CfgXWide = Cfg<128, 512, 32, 1, 4>;   // wavefront tile 128 x 128
using CfgSquare = Cfg<256, 256, 64, 2, 2>;  // wavefront tile 128 x 128 (weight gradient)
static_assert(NESTOR_HIP_TILE_M == 128, "tile table granularity");

template <typename C, int kMode>
int launch_rows(GemmParams p, void* stream) {
  constexpr int out_cols = kMode == kNNUpGate ? C::BN / 2 : C::BN;
  p.n_tiles = static_cast<int>(ceil_div(p.N, out_cols));
  const int64_t blocks = p.max_tiles * p.n_tiles;
  if (blocks > INT32_MAX) return NESTOR_HIP_ERANGE;
  static const bool configured = allow_dynamic_lds(
      reinterpret_cast<const void*>(grouped_gemm_kernel<C, kMode>), C::LDS_BYTES);
  (void)configured;
  hipLaunchKernelGGL((grouped_gemm_kernel<C, kMode>), dim3(static_cast<unsigned>(blocks)),
                     dim3(kThreads), C::LDS_BYTES, static_cast<hipStream_t>(stream), p);
  return launch_status();
}

// Each configuration walks the tile table whose tiles it covers.
using DmaXWide = DmaCfg<160, 512, 32, 1, 4, 3>;   // up to 5 row blocks x (128 x 128 per wavefront); balanced 160-row table
using DmaSquare = DmaCfg<320, 256, 32, 2, 2, 3>;  // 2 x 2 wavefronts of up to 5 blocks x 128 columns; balanced 320-row table
using DmaWide = DmaCfg<128, 256, 64, 2, 2, 3>;    // wavefront tile 64 x 128; 128-row table
using WgradPers = DmaCfg<256, 256, 32, 2, 2, 3>;  // persistent weight gradient

#if NESTOR_GEMM_CLOCK_HOOK
// Measurement hook (instrumented build only): where the direct-to-LDS kernels add their
// cycle and wall-clock counts (see GemmParams::clock_sink); null unless
// nestor_hip_gemm_clock_sink set it.
unsigned long long* g_clock_sink = nullptr;
#endif

template <typename C, int kMode, bool kRagK = false>
int launch_rows_dma(GemmParams p, int table_kind, int64_t rows_pad, int32_t num_banks, void* stream) {
  if constexpr (!kRagK) {
    // a contraction that ends inside a K step takes the variant that handles it
    if (p.K % C::BK != 0) return launch_rows_dma<C, kMode, true>(p, table_kind, rows_pad, num_banks, stream);
  }
  static_assert(C::BM == 128 || C::BM == 160 || C::BM == 320, "a tile table exists for these heights");
  if (32 * tile_blocks_cap(table_kind) > C::BM) return NESTOR_HIP_EINVAL;
  p.tile_table += table_offset(table_kind, rows_pad, num_banks);
  p.max_tiles = table_cap(table_kind, rows_pad, num_banks);
  constexpr int out_cols = kMode == kNNUpGate ? C::BN / 2 : C::BN;
  p.n_tiles = static_cast<int>(ceil_div(p.N, out_cols));
#if NESTOR_GEMM_CLOCK_HOOK
  p.clock_sink = g_clock_sink;
#endif
  static const int forced_group = config_choice("NESTOR_HIP_TILE_GROUP", -1);
  // Measured at the 1b-like shapes: the down projection runs best (and fetches least)
  // with a bank's row tiles per XCD group walked row tile first (four tiles for banks of
  // ~512 rows: 1.33 -> 1.27 ms against groups of eight; eight for banks of thousands of
  // rows); the fused input gradient with four, column tile first; the others in plain
  // order.  The spread is 2-6 %.
  const int64_t tiles_per_bank = rows_pad / num_banks / 128;
  p.tile_group = forced_group >= 0 ? forced_group
                                   : (kMode == kNN ? (tiles_per_bank <= 5 ? 4 : 8) : kMode == kNTUpGate ? 4 : 0);
  static const int forced_order = config_choice("NESTOR_HIP_TILE_ORDER", -1);
  p.tile_order = forced_order >= 0 ? forced_order : (kMode == kNN ? 1 : 0);
  // whole groups of row tiles per XCD (see the kernel's tile mapping)
  const int64_t gran = p.tile_group > 0 ? 8 * p.tile_group : 1;
  const int64_t blocks = ceil_div(p.max_tiles, gran) * gran * p.n_tiles;
  if (blocks > INT32_MAX) return NESTOR_HIP_ERANGE;
  static const bool configured = allow_dynamic_lds(
      reinterpret_cast<const void*>(grouped_gemm_dma_kernel<C, kMode, kRagK>), C::LDS_BYTES);
  (void)configured;
  hipLaunchKernelGGL((grouped_gemm_dma_kernel<C, kMode, kRagK>), dim3(static_cast<unsigned>(blocks)),
                     dim3(C::THREADS), C::LDS_BYTES, static_cast<hipStream_t>(stream), p);
  return launch_status();
}

// Row-tiled modes: which kernel walks which of the buffer's tile tables.
template <int kMode>
int dispatch_rows_gemm(const GemmParams& p, int64_t rows_pad, int32_t num_banks, void* stream) {
  static const int forced = config_choice("NESTOR_HIP_GEMM_CFG", -1);
  int cfg = forced;
  const int64_t width = kMode == kNNUpGate ? 2 * p.N : p.N;
  constexpr bool kBContigMode = kMode == kNT || kMode == kNTUpGate;
  if (cfg < 0) {
    // Measured on the 1b-like shapes: the direct-to-LDS variants win in every
    // mode.  The forward GEMMs (weights contraction-major) prefer the x512x32 tile
    // with one row of wavefronts (cfg 3).  The input-gradient GEMMs (both operands
    // contraction-contiguous, so every transfer is made of 64-byte row pieces) prefer
    // x256x32 with 2 x 2 wavefronts (cfg 7), which moves 20 % fewer pieces per MFMA.
    // Narrower outputs take the x256x64 tile (cfg 4).  The register-staged kernels
    // (cfg 2 and below) remain for outputs narrower than 256 and operands of 4 GiB.
    cfg = kBContigMode ? 7 : 3;
    // The fused up|gate tile holds 256 up and 256 gate columns: from 129 columns of each on
    // it beats two passes of the 128 + 128 tile over the activations (measured at h = 160,
    // 184, 216: 15-24 % faster), although up to half of its weight panel is padding.
    if (cfg == 3 && width < (kMode == kNNUpGate ? 264 : 512)) cfg = 4;
  }
  if constexpr (kMode != kNNFp8W) {
    // Direct-to-LDS variants: whole K steps only, and byte offsets inside one bank's
    // operand (and inside a tile's rows of activations) that fit 32 bits.
    const int64_t b_span = (kBContigMode ? p.N : p.K) * p.ldb * 2;
    const bool spans_fit = b_span < (int64_t{1} << 32) && 512 * p.lda * 2 < (int64_t{1} << 32);
    // An input gradient narrower than the 256-column tile still runs faster on it than on the
    // register-staged kernel (rows of the weight tile behind the last output column re-read
    // that column): 136 / 160 / 216 / 248 columns 0.295 -> 0.221, 0.297 -> 0.224,
    // 0.064 -> 0.056, 0.140 -> 0.106 ms.
    if (spans_fit && cfg == 7 && width >= (kBContigMode ? 136 : 256))
      return launch_rows_dma<DmaSquare, kMode>(p, kTilesBal320, rows_pad, num_banks, stream);
    if (spans_fit && (cfg == 3 || cfg == 7) && width >= 264)
      return launch_rows_dma<DmaXWide, kMode>(p, kTilesBal160, rows_pad, num_banks, stream);
    if (spans_fit && cfg >= 3 && width >= 256)
      return launch_rows_dma<DmaWide, kMode>(p, kTiles128, rows_pad, num_banks, stream);
  }
  if (cfg >= 3) cfg = 2;
  if (cfg == 2 && width < 512) cfg = 1;
  if (cfg == 1 && width < 256) cfg = 0;
  switch (cfg) {
    case 2: return launch_rows<CfgXWide, kMode>(p, stream);
    case 1: return launch_rows<CfgWide, kMode>(p, stream);
    default: return launch_rows<CfgSmall, kMode>(p, stream);
  }
}

template <typename C>
int launch_wgrad(const GemmParams& p, int32_t num_banks, void* stream) {
  static const bool configured = allow_dynamic_lds(
      reinterpret_cast<const void*>(grouped_gemm_kernel<C, kTN>), C::LDS_BYTES);
  (void)configured;
  const int64_t my = ceil_div(p.M, C::BM);
  if (my > 65535) return NESTOR_HIP_ERANGE;
  hipLaunchKernelGGL((grouped_gemm_kernel<C, kTN>),
                     dim3(static_cast<unsigned>(ceil_div(p.N, C::BN)), static_cast<unsigned>(my),
                          static_cast<unsigned>(num_banks)),
                     dim3(kThreads), C::LDS_BYTES, static_cast<hipStream_t>(stream), p);
  return launch_status();
}

}  // namespace

int launch_fp8_staged(const GemmParams& p, void* stream) {
  return launch_rows<CfgSmall, kNNFp8W>(p, stream);
}

}  // namespace nestor

using namespace nestor;

extern "C" int nestor_hip_grouped_gemm_nn(const void* a, const void* b, void* out,
                                          int64_t rows_pad, int64_t K, int64_t N,
                                          int32_t num_banks, const int32_t* tile_table,
                                          int64_t max_tiles, void* stream) {
  if (!dims_ok(rows_pad, K, N, num_banks, max_tiles)) return NESTOR_HIP_EINVAL;
  if (rows_pad == 0) return NESTOR_HIP_OK;
  if (!a || !b || !out || !tile_table) return NESTOR_HIP_EINVAL;
  GemmParams p = {};
  p.a = static_cast<const uint16_t*>(a);
  p.lda = K;
  p.b0 = b;
  p.bank_stride = K * N;
  p.ldb = N;
  p.out = static_cast<uint16_t*>(out);
  p.ldo = N;
  p.K = K;
  p.N = N;
  p.tile_table = tile_table;
  p.max_tiles = max_tiles;
  return dispatch_rows_gemm<kNN>(p, rows_pad, num_banks, stream);
}

extern "C" int nestor_hip_grouped_gemm_upgate_swiglu(
    const void* a, const void* w_up, const void* w_gate, void* up_gate, void* hidden,
    int64_t rows_pad, int64_t K, int64_t H, int32_t num_banks, const int32_t* tile_table,
    int64_t max_tiles, void* stream) {
  if (!dims_ok(rows_pad, K, H, num_banks, max_tiles)) return NESTOR_HIP_EINVAL;
  if (rows_pad == 0) return NESTOR_HIP_OK;
  if (!a || !w_up || !w_gate || !hidden || !tile_table) return NESTOR_HIP_EINVAL;
  GemmParams p = {};
  p.a = static_cast<const uint16_t*>(a);
  p.lda = K;
  p.b0 = w_up;
  p.b1 = w_gate;
  p.bank_stride = K * H;
  p.ldb = H;
  p.out = static_cast<uint16_t*>(up_gate);
  p.ldo = 2 * H;
  p.out2 = static_cast<uint16_t*>(hidden);
  p.ldo2 = H;
  p.K = K;
  p.N = H;
  p.tile_table = tile_table;
  p.max_tiles = max_tiles;
  return dispatch_rows_gemm<kNNUpGate>(p, rows_pad, num_banks, stream);
}

extern "C" int nestor_hip_grouped_gemm_nt(const void* a, const void* b, void* out,
                                          int64_t rows_pad, int64_t K, int64_t N,
                                          int32_t num_banks, const int32_t* tile_table,
                                          int64_t max_tiles, void* stream) {
  if (!dims_ok(rows_pad, K, N, num_banks, max_tiles)) return NESTOR_HIP_EINVAL;
  if (rows_pad == 0) return NESTOR_HIP_OK;
  if (!a || !b || !out || !tile_table) return NESTOR_HIP_EINVAL;
  GemmParams p = {};
  p.a = static_cast<const uint16_t*>(a);
  p.lda = K;
  p.b0 = b;
  p.bank_stride = K * N;
  p.ldb = K;
  p.out = static_cast<uint16_t*>(out);
  p.ldo = N;
  p.K = K;
  p.N = N;
  p.tile_table = tile_table;
  p.max_tiles = max_tiles;
  return dispatch_rows_gemm<kNT>(p, rows_pad, num_banks, stream);
}

extern "C" int nestor_hip_grouped_gemm_nt_upgate(
    const void* g_up_gate, const void* w_up, const void* w_gate, void* out,
    int64_t rows_pad, int64_t K, int64_t H, int32_t num_banks, const int32_t* tile_table,
    int64_t max_tiles, void* stream) {
  // Output width is K (the model dim); the contraction runs over H twice.
  if (!dims_ok(rows_pad, H, K, num_banks, max_tiles)) return NESTOR_HIP_EINVAL;
  if (rows_pad == 0) return NESTOR_HIP_OK;
  if (!g_up_gate || !w_up || !w_gate || !out || !tile_table) return NESTOR_HIP_EINVAL;
  GemmParams p = {};
  p.a = static_cast<const uint16_t*>(g_up_gate);
  p.lda = 2 * H;
  p.b0 = w_up;
  p.b1 = w_gate;
  p.bank_stride = K * H;
  p.ldb = H;
  p.out = static_cast<uint16_t*>(out);
  p.ldo = K;
  p.K = H;
  p.N = K;
  p.tile_table = tile_table;
  p.max_tiles = max_tiles;
  return dispatch_rows_gemm<kNTUpGate>(p, rows_pad, num_banks, stream);
}

namespace nestor {
namespace {

bool tn_args_ok(const void* a, int64_t lda, const void* g, int64_t ldg, const void* out, int64_t ldo,
                int64_t rows_pad, int64_t M, int64_t N, int64_t g_cols, int32_t num_banks,
                const int32_t* offs, const int64_t* seg_start, const int64_t* seg_count,
                int32_t out_dtype) {
  if (rows_pad < 0 || M <= 0 || N <= 0 || M % 8 != 0 || N % 8 != 0 || lda % 8 != 0 ||
      ldg % 8 != 0 || ldo % 8 != 0 || lda < M || ldg < g_cols || ldo < N || num_banks <= 0 ||
      num_banks > 65535)
    return false;
  if (!out || (!offs && !(seg_start && seg_count)) || (rows_pad > 0 && (!a || !g))) return false;
  if ((seg_start == nullptr) != (seg_count == nullptr)) return false;
  return out_dtype == NESTOR_HIP_BF16 || out_dtype == NESTOR_HIP_F32;
}

// The persistent kernel when the shape allows it (returns 1 when it does not), else a status.
int launch_wgrad_persistent(GemmParams p, int32_t num_banks, void* stream) {
  using C = WgradPers;
  // its buffer descriptors count an operand's bytes in 32 bits
  const bool spans_fit =
      p.rows_pad * p.lda * 2 < (int64_t{1} << 32) && p.rows_pad * p.ldb * 2 < (int64_t{1} << 32);
  if (p.rows_pad > INT32_MAX || !spans_fit) return 1;
  static const bool configured =
      allow_dynamic_lds(reinterpret_cast<const void*>(wgrad_persistent_kernel<C, false>),
                        WgradLayout<C>::LDS_BYTES) &&
      allow_dynamic_lds(reinterpret_cast<const void*>(wgrad_persistent_kernel<C, true>),
                        WgradLayout<C>::LDS_BYTES);
  (void)configured;
  const int num_cus = cu_count() / 8 * 8;
  const int64_t items = ceil_div(p.M, C::BM) * ceil_div(p.N, C::BN) * num_banks;
  if (num_cus < 8 || items / num_cus + 2 > WgradLayout<C>::kMaxItems) return 1;
#if NESTOR_GEMM_CLOCK_HOOK
  p.clock_sink = g_clock_sink;
#endif
  if (p.out_f32)
    hipLaunchKernelGGL((wgrad_persistent_kernel<C, true>), dim3(static_cast<unsigned>(num_cus)),
                       dim3(C::THREADS), WgradLayout<C>::LDS_BYTES,
                       static_cast<hipStream_t>(stream), p, num_banks);
  else
    hipLaunchKernelGGL((wgrad_persistent_kernel<C, false>), dim3(static_cast<unsigned>(num_cus)),
                       dim3(C::THREADS), WgradLayout<C>::LDS_BYTES,
                       static_cast<hipStream_t>(stream), p, num_banks);
  return launch_status();
}

// One weight gradient: which kernel takes it.
int launch_tn(const GemmParams& p, int32_t num_banks, void* stream) {
  static const int forced = config_choice("NESTOR_HIP_WGRAD_CFG", -1);
  // The persistent kernel's 256 x 256 tiles may overhang the outputs: it wins from 128
  // columns on (1280 x 160 outputs: 0.31 -> 0.21 ms; its descriptors cut the overhang off).
  static const int pers_min = config_choice("NESTOR_HIP_WGRAD_MIN", 128);
  int cfg = forced >= 0 ? forced : ((p.M >= pers_min && p.N >= pers_min) ? 5 : 0);
  if (cfg == 5 && p.M >= pers_min && p.N >= pers_min) {
    const int rc = launch_wgrad_persistent(p, num_banks, stream);
    if (rc <= 0) return rc;
  }
  if (cfg == 5) cfg = 3;
  switch (cfg) {
    case 3: return launch_wgrad<CfgSquare>(p, num_banks, stream);
    case 1: return launch_wgrad<CfgWide>(p, num_banks, stream);
    default: return launch_wgrad<CfgSmall>(p, num_banks, stream);
  }
}

GemmParams tn_params(const void* a, int64_t lda, const void* g, int64_t ldg, void* out, int64_t ldo,
                     int64_t bank_stride, int64_t rows_pad, int64_t M, int64_t N,
                     const int32_t* offs, const int64_t* seg_start, const int64_t* seg_count,
                     int32_t out_dtype) {
  GemmParams p = {};
  p.out_f32 = out_dtype == NESTOR_HIP_F32;
  p.a = static_cast<const uint16_t*>(a);
  p.lda = lda;
  p.b0 = g;
  p.ldb = ldg;
  p.out = static_cast<uint16_t*>(out);
  p.ldo = ldo;
  p.bank_stride = bank_stride;
  p.M = M;
  p.N = N;
  p.rows_pad = rows_pad;
  p.offs = offs;
  p.seg_start = seg_start;
  p.seg_count = seg_count;
  return p;
}

}  // namespace
}  // namespace nestor

extern "C" int nestor_hip_grouped_gemm_tn(const void* a, int64_t lda, const void* g,
                                          int64_t ldg, void* out, int64_t ldo,
                                          int64_t bank_stride, int64_t rows_pad, int64_t M,
                                          int64_t N, int32_t num_banks, const int32_t* offs,
                                          const int64_t* seg_start, const int64_t* seg_count,
                                          int32_t out_dtype, void* stream) {
  if (!tn_args_ok(a, lda, g, ldg, out, ldo, rows_pad, M, N, N, num_banks, offs, seg_start, seg_count,
                  out_dtype))
    return NESTOR_HIP_EINVAL;
  return launch_tn(tn_params(a, lda, g, ldg, out, ldo, bank_stride, rows_pad, M, N, offs, seg_start,
                             seg_count, out_dtype),
                   num_banks, stream);
}

extern "C" int nestor_hip_grouped_gemm_tn_pair(const void* a, int64_t lda, const void* g,
                                               int64_t ldg, void* out0, void* out1, int64_t ldo,
                                               int64_t bank_stride, int64_t rows_pad, int64_t M,
                                               int64_t N, int32_t num_banks, const int32_t* offs,
                                               const int64_t* seg_start, const int64_t* seg_count,
                                               int32_t out_dtype, void* stream) {
  if (!tn_args_ok(a, lda, g, ldg, out0, ldo, rows_pad, M, N, 2 * N, num_banks, offs, seg_start,
                  seg_count, out_dtype) || !out1)
    return NESTOR_HIP_EINVAL;
  GemmParams p = tn_params(a, lda, g, ldg, out0, ldo, bank_stride, rows_pad, M, N, offs, seg_start,
                           seg_count, out_dtype);
  static const int forced = config_choice("NESTOR_HIP_WGRAD_CFG", -1);
  static const bool pair_off = config_choice("NESTOR_HIP_WGRAD_PAIR", 1) == 0;
  // One launch over both halves of g when a column tile never straddles them: the two
  // gradients share the activation panels and one launch's ramp and tail.
  if ((forced < 0 || forced == 5) && !pair_off && N % WgradPers::BN == 0 && M >= 128) {
    GemmParams both = p;
    both.N = 2 * N;
    both.split = N;
    both.out2 = static_cast<uint16_t*>(out1);
    const int rc = launch_wgrad_persistent(both, num_banks, stream);
    if (rc <= 0) return rc;
  }
  const int rc = launch_tn(p, num_banks, stream);
  if (rc != NESTOR_HIP_OK) return rc;
  p.b0 = static_cast<const uint16_t*>(g) + N;
  p.out = static_cast<uint16_t*>(out1);
  return launch_tn(p, num_banks, stream);
}

#if NESTOR_GEMM_CLOCK_HOOK
extern "C" int nestor_hip_gemm_clock_sink(uint64_t* sink) {
  g_clock_sink = reinterpret_cast<unsigned long long*>(sink);
  return NESTOR_HIP_OK;
}
#endif
