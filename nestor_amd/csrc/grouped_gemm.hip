// Grouped expert GEMMs on the gfx950 matrix cores.
//
// One workgroup (4 wavefronts, 2 x 2) owns a 128 x 128 output tile and walks K
// in steps of 64 through double-buffered LDS; each wavefront keeps a 64 x 64
// accumulator as 2 x 2 v_mfma_f32_32x32x16_bf16 tiles.  Which rows form a tile
// and which bank multiplies them comes from the device-side tile table written
// by the index build, so no launch parameter depends on the routing and the
// host never reads a count.
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
// The MFMA is issued with its operands swapped (B fragment first), which
// produces the transposed 32 x 32 tile: every lane then holds four consecutive
// output columns of one row and the epilogue can stage the bf16 tile through
// LDS with 64-bit writes and leave through 128-bit coalesced stores.
#include "common.hpp"

namespace nestor {
namespace {

constexpr int BM = 128;
constexpr int BN = 128;
constexpr int BK = 64;
constexpr int kThreads = 256;
constexpr int KC_LD = BK + 8;    // row stride (elements) of a contraction-contiguous tile
constexpr int NC_LD = BN + 16;   // row stride of a contraction-major tile
constexpr int TILE_ELEMS = BM * KC_LD;  // == BK * NC_LD == 9216
static_assert(BM * KC_LD == BK * NC_LD, "both tile layouts share one buffer size");
constexpr int STAGE_LD = BN + 8;
constexpr size_t kGemmLds = 4 * TILE_ELEMS * sizeof(uint16_t);  // 2 stages x (A, B)
static_assert(BM * STAGE_LD <= 2 * TILE_ELEMS, "epilogue staging reuses the A buffers");
static_assert(NESTOR_HIP_TILE_M == BM, "tile table granularity");

#define NESTOR_LDS __attribute__((address_space(3)))
typedef short s16x4 __attribute__((ext_vector_type(4)));

enum GemmMode {
  kNN = 0,        // out = a @ b[bank]            b [E,K,N]
  kNNUpGate = 1,  // up|gate = a @ [w_up | w_gate], swiglu epilogue
  kNT = 2,        // out = a @ b[bank]^T          b [E,N,K]
  kNTUpGate = 3,  // out = g[:, :H] @ w_up^T + g[:, H:] @ w_gate^T
  kNNFp8W = 4,    // kNN with e4m3 weights and per-column scales
};

struct GemmParams {
  const uint16_t* a;
  int64_t lda;
  const void* b0;
  const void* b1;
  int64_t bank_stride;  // elements between banks of b0 / b1
  int64_t ldb;
  const float* scale;   // [E, N] (kNNFp8W)
  uint16_t* out;
  int64_t ldo;
  uint16_t* out2;       // hidden (kNNUpGate)
  int64_t ldo2;
  int64_t K;            // contraction length (per phase)
  int64_t N;            // output columns (kNNUpGate: H)
  const int32_t* tile_table;
  int64_t max_tiles;
  int n_tiles;
};

__device__ __forceinline__ bf16x8 lds_read_kc(const uint16_t* tile, int row, int k) {
  return *reinterpret_cast<const bf16x8*>(tile + row * KC_LD + k);
}

// Eight consecutive contraction indices (k .. k+7) of output index `col`, from
// a contraction-major tile, as two transposing 64-bit LDS reads.
__device__ __forceinline__ bf16x8 lds_read_tr(const uint16_t* tile, int krow, int col) {
  typedef __attribute__((__vector_size__(4 * sizeof(short)))) short v4s;
  const uint16_t* p0 = tile + krow * NC_LD + col;
  const uint16_t* p1 = p0 + 4 * NC_LD;
  v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NESTOR_LDS v4s*)(p0));
  v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NESTOR_LDS v4s*)(p1));
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  return __builtin_bit_cast(bf16x8, v);
}

__device__ __forceinline__ u32x4 fp8x8_to_bf16x8(u32x2 raw) {
  float f[8];
#pragma unroll
  for (int w = 0; w < 2; ++w) {
    auto lo = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(raw[w]), false);
    auto hi = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(raw[w]), true);
    f[4 * w + 0] = lo[0];
    f[4 * w + 1] = lo[1];
    f[4 * w + 2] = hi[0];
    f[4 * w + 3] = hi[1];
  }
  return pack8(f);
}

struct TileRef {
  int bank;
  int row0;
  int nrows;
};

__device__ __forceinline__ bool fetch_tile(const int32_t* tt, int64_t max_tiles, int tile,
                                           TileRef* t) {
  if (tile >= tt[3 * max_tiles]) return false;
  t->bank = tt[tile];
  t->row0 = tt[max_tiles + tile];
  t->nrows = tt[2 * max_tiles + tile];
  return true;
}

// Accumulators -> bf16 staging tile [BM][STAGE_LD] (optionally scaled per column).
template <bool kScale>
__device__ __forceinline__ void stage_accumulators(uint16_t* stage, const f32x16 (&acc)[2][2],
                                                   int wm, int wn, int lane,
                                                   const float* col_scale, int64_t n0,
                                                   int64_t n_limit) {
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int m = 64 * wm + 32 * i + (lane & 31);
        const int n = 64 * wn + 32 * j + 8 * q + 4 * (lane >> 5);
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[i][j][4 * q + e];
        if constexpr (kScale) {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            v[e] *= (n0 + n + e < n_limit) ? col_scale[n0 + n + e] : 0.0f;
        }
        u32x2 packed = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
        *reinterpret_cast<u32x2*>(stage + m * STAGE_LD + n) = packed;
      }
}

template <int kMode>
__global__ __launch_bounds__(kThreads) void grouped_gemm_kernel(GemmParams p) {
  extern __shared__ __align__(16) uint16_t lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1;
  const int wn = wave & 1;
  const int tile = blockIdx.x / p.n_tiles;
  const int nt = blockIdx.x % p.n_tiles;
  TileRef t;
  if (!fetch_tile(p.tile_table, p.max_tiles, tile, &t)) return;

  constexpr bool kUpGateFwd = kMode == kNNUpGate;
  constexpr bool kBContig = kMode == kNT || kMode == kNTUpGate;  // b is [N, K]
  constexpr int kOutCols = kUpGateFwd ? BN / 2 : BN;  // output columns per tile
  const int64_t n0 = static_cast<int64_t>(nt) * kOutCols;

  if (t.bank < 0) {
    // Slack tail: every padded tensor holds zeros there.
    const u32x4 zero = {0, 0, 0, 0};
    for (int c = tid; c < BM * (kOutCols / 8); c += kThreads) {
      const int row = c / (kOutCols / 8);
      const int64_t n = n0 + (c % (kOutCols / 8)) * 8;
      if (row < t.nrows && n < p.N) {
        const int64_t r = t.row0 + row;
        if constexpr (kUpGateFwd) {
          if (p.out != nullptr) {
            st16(p.out + r * p.ldo + n, zero);
            st16(p.out + r * p.ldo + p.N + n, zero);
          }
          st16(p.out2 + r * p.ldo2 + n, zero);
        } else {
          st16(p.out + r * p.ldo + n, zero);
        }
      }
    }
    return;
  }

  const int kt_per_phase = static_cast<int>((p.K + BK - 1) / BK);
  const int num_kt = kMode == kNTUpGate ? 2 * kt_per_phase : kt_per_phase;
  const uint16_t* a_rows = p.a + static_cast<int64_t>(t.row0) * p.lda;

  u32x4 ra[4], rb[4];
  const u32x4 zero4 = {0, 0, 0, 0};

  auto load_a = [&](int kt) {
    const int phase = kMode == kNTUpGate ? kt / kt_per_phase : 0;
    const int64_t k0 = static_cast<int64_t>(kt - phase * kt_per_phase) * BK;
    const int64_t col0 = kMode == kNTUpGate ? phase * p.K : 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + kThreads * i;
      const int row = c >> 3;
      const int64_t k = k0 + (c & 7) * 8;
      ra[i] = (row < t.nrows && k < p.K) ? ld16(a_rows + row * p.lda + col0 + k) : zero4;
    }
  };
  auto load_b = [&](int kt) {
    if constexpr (kBContig) {
      const int phase = kMode == kNTUpGate ? kt / kt_per_phase : 0;
      const int64_t k0 = static_cast<int64_t>(kt - phase * kt_per_phase) * BK;
      const uint16_t* b = reinterpret_cast<const uint16_t*>(phase == 0 ? p.b0 : p.b1) +
                          t.bank * p.bank_stride;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = tid + kThreads * i;
        const int64_t n = n0 + (c >> 3);
        const int64_t k = k0 + (c & 7) * 8;
        rb[i] = (n < p.N && k < p.K) ? ld16(b + n * p.ldb + k) : zero4;
      }
    } else {
      const int64_t k0 = static_cast<int64_t>(kt) * BK;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = tid + kThreads * i;
        const int64_t k = k0 + (c >> 4);
        const int nc = c & 15;
        if constexpr (kMode == kNNUpGate) {
          const uint16_t* b = reinterpret_cast<const uint16_t*>(nc < 8 ? p.b0 : p.b1) +
                              t.bank * p.bank_stride;
          const int64_t n = n0 + (nc & 7) * 8;
          rb[i] = (k < p.K && n < p.N) ? ld16(b + k * p.ldb + n) : zero4;
        } else if constexpr (kMode == kNNFp8W) {
          const uint8_t* b = reinterpret_cast<const uint8_t*>(p.b0) + t.bank * p.bank_stride;
          const int64_t n = n0 + nc * 8;
          rb[i] = (k < p.K && n < p.N)
                      ? fp8x8_to_bf16x8(*reinterpret_cast<const u32x2*>(b + k * p.ldb + n))
                      : zero4;
        } else {
          const uint16_t* b = reinterpret_cast<const uint16_t*>(p.b0) + t.bank * p.bank_stride;
          const int64_t n = n0 + nc * 8;
          rb[i] = (k < p.K && n < p.N) ? ld16(b + k * p.ldb + n) : zero4;
        }
      }
    }
  };
  auto store_tiles = [&](int stage) {
    uint16_t* sa = lds + stage * 2 * TILE_ELEMS;
    uint16_t* sb = sa + TILE_ELEMS;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + kThreads * i;
      *reinterpret_cast<u32x4*>(sa + (c >> 3) * KC_LD + (c & 7) * 8) = ra[i];
      if constexpr (kBContig)
        *reinterpret_cast<u32x4*>(sb + (c >> 3) * KC_LD + (c & 7) * 8) = rb[i];
      else
        *reinterpret_cast<u32x4*>(sb + (c >> 4) * NC_LD + (c & 15) * 8) = rb[i];
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  load_a(0);
  load_b(0);
  store_tiles(0);
  __syncthreads();

  for (int kt = 0; kt < num_kt; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < num_kt) {
      load_a(kt + 1);
      load_b(kt + 1);
    }
    const uint16_t* sa = lds + cur * 2 * TILE_ELEMS;
    const uint16_t* sb = sa + TILE_ELEMS;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      bf16x8 fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
        fa[i] = lds_read_kc(sa, 64 * wm + 32 * i + (lane & 31), 16 * kk + 8 * (lane >> 5));
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        if constexpr (kBContig)
          fb[j] = lds_read_kc(sb, 64 * wn + 32 * j + (lane & 31), 16 * kk + 8 * (lane >> 5));
        else
          fb[j] = lds_read_tr(sb, 16 * kk + 8 * (lane >> 5) + ((lane & 15) >> 2),
                              64 * wn + 32 * j + 16 * ((lane >> 4) & 1) + 4 * (lane & 3));
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < num_kt) store_tiles(cur ^ 1);
    __syncthreads();
  }

  // Epilogue: bf16 tile through LDS, then coalesced 128-bit stores.
  uint16_t* stage = lds;
  if constexpr (kMode == kNNFp8W)
    stage_accumulators<true>(stage, acc, wm, wn, lane, p.scale + t.bank * p.N, n0, p.N);
  else
    stage_accumulators<false>(stage, acc, wm, wn, lane, nullptr, 0, 0);
  __syncthreads();
  if constexpr (kUpGateFwd) {
    for (int c = tid; c < BM * 8; c += kThreads) {
      const int row = c >> 3;
      const int hc = c & 7;
      const int64_t n = n0 + hc * 8;
      if (row < t.nrows && n < p.N) {
        const int64_t r = t.row0 + row;
        const u32x4 up = *reinterpret_cast<const u32x4*>(stage + row * STAGE_LD + hc * 8);
        const u32x4 gate =
            *reinterpret_cast<const u32x4*>(stage + row * STAGE_LD + 64 + hc * 8);
        if (p.out != nullptr) {
          st16(p.out + r * p.ldo + n, up);
          st16(p.out + r * p.ldo + p.N + n, gate);
        }
        float u[8], g[8], h[8];
        unpack8(up, u);
        unpack8(gate, g);
#pragma unroll
        for (int e = 0; e < 8; ++e) h[e] = round_bf16(g[e] / (1.0f + __expf(-g[e]))) * u[e];
        st16(p.out2 + r * p.ldo2 + n, pack8(h));
      }
    }
  } else {
    for (int c = tid; c < BM * 16; c += kThreads) {
      const int row = c >> 4;
      const int64_t n = n0 + (c & 15) * 8;
      if (row < t.nrows && n < p.N)
        st16(p.out + (t.row0 + row) * p.ldo + n,
             *reinterpret_cast<const u32x4*>(stage + row * STAGE_LD + (c & 15) * 8));
    }
  }
}

struct WgradParams {
  const uint16_t* a;
  int64_t lda;
  const uint16_t* g;
  int64_t ldg;
  uint16_t* out;
  int64_t ldo;
  int64_t bank_stride;
  int64_t M;
  int64_t N;
  int64_t rows_pad;
  const int32_t* offs;
  const int64_t* seg_start;
  const int64_t* seg_count;
};

// out[e] = a[seg(e)]^T @ g[seg(e)]: both operands are contraction-major.
__global__ __launch_bounds__(kThreads) void grouped_wgrad_kernel(WgradParams p) {
  extern __shared__ __align__(16) uint16_t lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1;
  const int wn = wave & 1;
  const int bank = blockIdx.z;
  const int64_t m0 = static_cast<int64_t>(blockIdx.y) * BM;
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * BN;
  int64_t seg_begin, seg_end;
  if (p.seg_start != nullptr) {
    seg_begin = p.seg_start[bank];
    seg_end = seg_begin + p.seg_count[bank];
  } else {
    seg_begin = bank == 0 ? 0 : p.offs[bank - 1];
    seg_end = p.offs[bank];
  }
  if (seg_end > p.rows_pad) seg_end = p.rows_pad;
  const int num_kt = seg_end > seg_begin ? static_cast<int>((seg_end - seg_begin + BK - 1) / BK) : 0;

  u32x4 ra[4], rb[4];
  const u32x4 zero4 = {0, 0, 0, 0};
  auto load_tiles = [&](int kt) {
    const int64_t r0 = seg_begin + static_cast<int64_t>(kt) * BK;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + kThreads * i;
      const int64_t r = r0 + (c >> 4);
      const int cc = (c & 15) * 8;
      ra[i] = (r < seg_end && m0 + cc < p.M) ? ld16(p.a + r * p.lda + m0 + cc) : zero4;
      rb[i] = (r < seg_end && n0 + cc < p.N) ? ld16(p.g + r * p.ldg + n0 + cc) : zero4;
    }
  };
  auto store_tiles = [&](int stage) {
    uint16_t* sa = lds + stage * 2 * TILE_ELEMS;
    uint16_t* sb = sa + TILE_ELEMS;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + kThreads * i;
      *reinterpret_cast<u32x4*>(sa + (c >> 4) * NC_LD + (c & 15) * 8) = ra[i];
      *reinterpret_cast<u32x4*>(sb + (c >> 4) * NC_LD + (c & 15) * 8) = rb[i];
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  if (num_kt > 0) {
    load_tiles(0);
    store_tiles(0);
  }
  __syncthreads();
  for (int kt = 0; kt < num_kt; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < num_kt) load_tiles(kt + 1);
    const uint16_t* sa = lds + cur * 2 * TILE_ELEMS;
    const uint16_t* sb = sa + TILE_ELEMS;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      bf16x8 fa[2], fb[2];
      const int krow = 16 * kk + 8 * (lane >> 5) + ((lane & 15) >> 2);
      const int cofs = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
#pragma unroll
      for (int i = 0; i < 2; ++i) fa[i] = lds_read_tr(sa, krow, 64 * wm + 32 * i + cofs);
#pragma unroll
      for (int j = 0; j < 2; ++j) fb[j] = lds_read_tr(sb, krow, 64 * wn + 32 * j + cofs);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < num_kt) store_tiles(cur ^ 1);
    __syncthreads();
  }

  uint16_t* stage = lds;
  stage_accumulators<false>(stage, acc, wm, wn, lane, nullptr, 0, 0);
  __syncthreads();
  uint16_t* out = p.out + bank * p.bank_stride;
  for (int c = tid; c < BM * 16; c += kThreads) {
    const int64_t m = m0 + (c >> 4);
    const int64_t n = n0 + (c & 15) * 8;
    if (m < p.M && n < p.N)
      st16(out + m * p.ldo + n,
           *reinterpret_cast<const u32x4*>(stage + (c >> 4) * STAGE_LD + (c & 15) * 8));
  }
}

bool dims_ok(int64_t rows_pad, int64_t K, int64_t N, int32_t num_banks, int64_t max_tiles) {
  return rows_pad >= 0 && rows_pad <= INT32_MAX && K > 0 && N > 0 && K % 8 == 0 &&
         N % 8 == 0 && num_banks > 0 && max_tiles > 0;
}

template <int kMode>
int launch_gemm(const GemmParams& p, int64_t max_tiles, void* stream) {
  const int64_t blocks = max_tiles * p.n_tiles;
  if (blocks > INT32_MAX) return NESTOR_HIP_ERANGE;
  static bool configured = false;
  if (!configured) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(grouped_gemm_kernel<kMode>),
                              hipFuncAttributeMaxDynamicSharedMemorySize,
                              static_cast<int>(kGemmLds));
    configured = true;
  }
  hipLaunchKernelGGL(grouped_gemm_kernel<kMode>, dim3(static_cast<unsigned>(blocks)),
                     dim3(kThreads), kGemmLds, static_cast<hipStream_t>(stream), p);
  return launch_status();
}

}  // namespace
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
  p.n_tiles = static_cast<int>(ceil_div(N, BN));
  return launch_gemm<kNN>(p, max_tiles, stream);
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
  p.n_tiles = static_cast<int>(ceil_div(H, BN / 2));
  return launch_gemm<kNNUpGate>(p, max_tiles, stream);
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
  p.n_tiles = static_cast<int>(ceil_div(N, BN));
  return launch_gemm<kNT>(p, max_tiles, stream);
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
  p.n_tiles = static_cast<int>(ceil_div(K, BN));
  return launch_gemm<kNTUpGate>(p, max_tiles, stream);
}

extern "C" int nestor_hip_grouped_gemm_fp8w_nn(const void* a, const void* b_q,
                                               const float* scale, void* out,
                                               int64_t rows_pad, int64_t K, int64_t N,
                                               int32_t num_banks, const int32_t* tile_table,
                                               int64_t max_tiles, void* stream) {
  if (!dims_ok(rows_pad, K, N, num_banks, max_tiles)) return NESTOR_HIP_EINVAL;
  if (rows_pad == 0) return NESTOR_HIP_OK;
  if (!a || !b_q || !scale || !out || !tile_table) return NESTOR_HIP_EINVAL;
  GemmParams p = {};
  p.a = static_cast<const uint16_t*>(a);
  p.lda = K;
  p.b0 = b_q;
  p.bank_stride = K * N;
  p.ldb = N;
  p.scale = scale;
  p.out = static_cast<uint16_t*>(out);
  p.ldo = N;
  p.K = K;
  p.N = N;
  p.tile_table = tile_table;
  p.max_tiles = max_tiles;
  p.n_tiles = static_cast<int>(ceil_div(N, BN));
  return launch_gemm<kNNFp8W>(p, max_tiles, stream);
}

extern "C" int nestor_hip_grouped_gemm_tn(const void* a, int64_t lda, const void* g,
                                          int64_t ldg, void* out, int64_t ldo,
                                          int64_t bank_stride, int64_t rows_pad, int64_t M,
                                          int64_t N, int32_t num_banks, const int32_t* offs,
                                          const int64_t* seg_start, const int64_t* seg_count,
                                          void* stream) {
  if (rows_pad < 0 || M <= 0 || N <= 0 || M % 8 != 0 || N % 8 != 0 || lda % 8 != 0 ||
      ldg % 8 != 0 || ldo % 8 != 0 || lda < M || ldg < N || ldo < N || num_banks <= 0 ||
      num_banks > 65535)
    return NESTOR_HIP_EINVAL;
  if (!out || (!offs && !(seg_start && seg_count)) || (rows_pad > 0 && (!a || !g)))
    return NESTOR_HIP_EINVAL;
  if ((seg_start == nullptr) != (seg_count == nullptr)) return NESTOR_HIP_EINVAL;
  WgradParams p = {};
  p.a = static_cast<const uint16_t*>(a);
  p.lda = lda;
  p.g = static_cast<const uint16_t*>(g);
  p.ldg = ldg;
  p.out = static_cast<uint16_t*>(out);
  p.ldo = ldo;
  p.bank_stride = bank_stride;
  p.M = M;
  p.N = N;
  p.rows_pad = rows_pad;
  p.offs = offs;
  p.seg_start = seg_start;
  p.seg_count = seg_count;
  static bool configured = false;
  if (!configured) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(grouped_wgrad_kernel),
                              hipFuncAttributeMaxDynamicSharedMemorySize,
                              static_cast<int>(kGemmLds));
    configured = true;
  }
  const int64_t my = ceil_div(M, BM);
  if (my > 65535) return NESTOR_HIP_ERANGE;
  hipLaunchKernelGGL(grouped_wgrad_kernel,
                     dim3(static_cast<unsigned>(ceil_div(N, BN)), static_cast<unsigned>(my),
                          static_cast<unsigned>(num_banks)),
                     dim3(kThreads), kGemmLds, static_cast<hipStream_t>(stream), p);
  return launch_status();
}
