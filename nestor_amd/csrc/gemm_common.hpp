// Building blocks shared by the grouped-GEMM translation units (grouped_gemm.hip: the
// bf16 kernels; fp8_stream.hip: the e4m3 weight-streaming kernels): launch parameters,
// tile configurations, LDS / LDS-DMA / MFMA helpers and the host-side switches.
#pragma once

#include <cstdlib>
#include <type_traits>
#include <utility>

#include "common.hpp"
#include "dma_addressing.hpp"

namespace nestor {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;

#define NESTOR_LDS __attribute__((address_space(3)))

// Instrumented build (the measurement library only): the direct-to-LDS kernels add their
// cycle and wall-clock counts to a caller-provided sink.  Compiled out of the product.
#ifndef NESTOR_GEMM_CLOCK_HOOK
#define NESTOR_GEMM_CLOCK_HOOK 0
#endif

// Output tiles are written once and read by a later kernel.
#ifndef NESTOR_GEMM_NT_STORES
#define NESTOR_GEMM_NT_STORES 1
#endif
__device__ __forceinline__ void st16o(void* p, u32x4 v) {
#if NESTOR_GEMM_NT_STORES
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
#else
  st16(p, v);
#endif
}

template <int BM_, int BN_, int BK_, int WGM_, int WGN_>
struct Cfg {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WGM = WGM_, WGN = WGN_;
  static_assert(WGM * WGN == kWaves, "4 wavefronts per workgroup");
  static constexpr int WTM = BM / WGM, WTN = BN / WGN;  // wavefront tile
  static constexpr int MI = WTM / 32, NJ = WTN / 32;    // MFMA tiles per wavefront
  static constexpr int KK = BK / 16;
  static constexpr int KC_LD = BK + 8;       // row stride of a contraction-contiguous tile
  static constexpr int STAGE_LD = BN + 8;    // epilogue staging row stride
  // Tile sizes in elements for the two layouts of each operand.
  static constexpr int A_KC = BM * KC_LD, A_MC = BK * (BM + 32);
  static constexpr int B_KC = BN * KC_LD, B_NC = BK * (BN + 32);
  static constexpr int A_ELEMS = A_KC > A_MC ? A_KC : A_MC;
  static constexpr int B_ELEMS = B_KC > B_NC ? B_KC : B_NC;
  static constexpr int STAGE_ELEMS = BM * STAGE_LD;
  static constexpr int PIPE_ELEMS = 2 * (A_ELEMS + B_ELEMS);
  static constexpr size_t LDS_BYTES =
      sizeof(uint16_t) * (PIPE_ELEMS > STAGE_ELEMS ? PIPE_ELEMS : STAGE_ELEMS);
  static constexpr int A_CHUNKS = BM * BK / 8 / kThreads;  // 16-byte chunks per thread
  static constexpr int B_CHUNKS = BN * BK / 8 / kThreads;
  static_assert(BM * BK / 8 % kThreads == 0 && BN * BK / 8 % kThreads == 0, "chunking");
};

enum GemmMode {
  kNN = 0,        // out = a @ b[bank]            b [E,K,N]
  kNNUpGate = 1,  // up|gate = a @ [w_up | w_gate], swiglu epilogue
  kNT = 2,        // out = a @ b[bank]^T          b [E,N,K]
  kNTUpGate = 3,  // out = g[:, :H] @ w_up^T + g[:, H:] @ w_gate^T
  kNNFp8W = 4,    // kNN with e4m3 weights and per-column scales
  kTN = 5,        // out[bank] = a[seg]^T @ g[seg]   (weight gradient)
};

struct GemmParams {
  const uint16_t* a;
  int64_t lda;
  const void* b0;
  const void* b1;
  int64_t bank_stride;  // elements between banks of b0 / b1 (kTN: of out)
  int64_t ldb;
  const float* scale;   // [E, N] (kNNFp8W)
  const float* scale2;  // [E, N] of the gate bank (fused e4m3 up|gate)
  uint16_t* out;
  int64_t ldo;
  uint16_t* out2;       // hidden (kNNUpGate)
  int64_t ldo2;
  int64_t K;            // contraction length (per phase); kTN: unused
  int64_t N;            // output columns (kNNUpGate: H)
  int64_t M;            // kTN: output rows
  const int32_t* tile_table;
  int64_t max_tiles;
  int n_tiles;
  int tile_group;       // row tiles per XCD group in the grouped tile order (0: plain order)
  int tile_order;       // inside a group: 0 = column tile fastest, 1 = row tile fastest
  int64_t tile_stride;  // e4m3 stream kernels: bytes per [K][128] column block of a tiled bank, or 0
  // kTN segment description
  int64_t rows_pad;
  const int32_t* offs;
  const int64_t* seg_start;
  const int64_t* seg_count;
  int out_f32;          // kTN: out is float* (fp32 results), not bf16
  int64_t split;        // kTN pair: output columns from `split` on go to out2 (column - split); 0: one output
  // Measurement hook of the direct-to-LDS kernels (null in normal use): 64 slots of
  // {shader cycles, wall-clock ticks, workgroups, K steps}, summed over the
  // workgroups of a launch (slot = workgroup index % 64).
  unsigned long long* clock_sink;
};

// Adds one workgroup's figures to its slot of the measurement hook.
__device__ __forceinline__ void clock_sink_add(unsigned long long* sink, unsigned long long c0,
                                               unsigned long long w0, unsigned long long steps) {
  unsigned long long* slot = sink + 4 * (blockIdx.x & 63);
  atomicAdd(slot + 0, clock64() - c0);
  atomicAdd(slot + 1, wall_clock64() - w0);
  atomicAdd(slot + 2, 1ull);
  atomicAdd(slot + 3, steps);
}

template <int LD>
__device__ __forceinline__ bf16x8 lds_read_kc(const uint16_t* tile, int row, int k) {
  return *reinterpret_cast<const bf16x8*>(tile + row * LD + k);
}

// Eight consecutive contraction indices (krow .. krow+7 of this lane's half) of
// output index `col`, from a contraction-major tile, as two transposing reads.
template <int LD>
__device__ __forceinline__ bf16x8 lds_read_tr(const uint16_t* tile, int krow, int col) {
  typedef __attribute__((__vector_size__(4 * sizeof(short)))) short v4s;
  const uint16_t* p0 = tile + krow * LD + col;
  const uint16_t* p1 = p0 + 4 * LD;
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

// The same widening through the packed convert instruction (an e4m3 value is
// exactly representable in bf16, so no rounding happens).
__device__ __forceinline__ u32x4 fp8x8_to_bf16x8_exact(u32x2 raw) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  u32x4 out;
#pragma unroll
  for (int w = 0; w < 2; ++w) {
    const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(raw[w]), false);
    const f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(raw[w]), true);
    out[2 * w] = __builtin_bit_cast(uint32_t, __builtin_convertvector(lo, bf16x2));
    out[2 * w + 1] = __builtin_bit_cast(uint32_t, __builtin_convertvector(hi, bf16x2));
  }
  return out;
}

// Scheduling recipe for one fragment's worth of MFMAs: before MFMA m, let
// through this MFMA's share of the LDS reads (0x100), LDS writes (0x200) and
// global loads (0x010, any VMEM) that sit in the same scheduling region, so each memory
// latency hides behind the matrix pipe (0x008) instead of in front of it.
template <int kReads, int kWrites, int kVmem, int kMfma, int... Ms>
__device__ __forceinline__ void interleave_memory(std::integer_sequence<int, Ms...>) {
  (([] {
     constexpr int m = Ms;
     constexpr int r = ((m + 1) * kReads) / kMfma - (m * kReads) / kMfma;
     constexpr int w = ((m + 1) * kWrites) / kMfma - (m * kWrites) / kMfma;
     constexpr int v = ((m + 1) * kVmem) / kMfma - (m * kVmem) / kMfma;
     if constexpr (r > 0) __builtin_amdgcn_sched_group_barrier(0x100, r, 0);
     if constexpr (w > 0) __builtin_amdgcn_sched_group_barrier(0x200, w, 0);
     if constexpr (v > 0) __builtin_amdgcn_sched_group_barrier(0x010, v, 0);
     __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
   }()),
   ...);
}

// Tile configuration of the direct-to-LDS kernels (ring of STAGES_ unpadded stages).
// BM is the tallest tile the configuration takes; a wavefront holds up to MI = BM / WGM /
// 32 row blocks of 32 x WTN accumulators (the fifth block, where there is one, in
// ordinary vector registers: the accumulation registers hold four).
template <int BM_, int BN_, int BK_, int WGM_, int WGN_, int STAGES_, int OCC_ = 1>
struct DmaCfg {
  static constexpr int OCC = OCC_;  // workgroups resident per CU the register budget is sized for
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WGM = WGM_, WGN = WGN_;
  static constexpr int WAVES = WGM * WGN, THREADS = 64 * WAVES;
  static_assert(WAVES == 4 || WAVES == 8, "one or two wavefronts per SIMD");
  static constexpr int WTM = BM / WGM, WTN = BN / WGN;
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "whole MFMA tiles");
  static constexpr int MI = WTM / 32, NJ = WTN / 32;
  static_assert(MI >= 1 && MI <= 5, "four row blocks in accumulation registers, a fifth in vector registers");
  static constexpr int KK = BK / 16;
  // Rows of the A stage: BM rounded up to whole transfer instructions per wavefront.
  static constexpr int A_ROW_UNIT = THREADS * 8 / BK;
  static constexpr int A_ROWS = (BM + A_ROW_UNIT - 1) / A_ROW_UNIT * A_ROW_UNIT;
  static constexpr int A_ELEMS = A_ROWS * BK, B_ELEMS = BN * BK;
  static constexpr int kStages = STAGES_;
  static constexpr int PIPE_ELEMS = kStages * (A_ELEMS + B_ELEMS);
  // Epilogue: one slab of 32 rows x WTN columns per wavefront, inside the drained ring.
  static constexpr int EPI_LD = WTN + 8;
  static constexpr int EPI_ELEMS = WAVES * 32 * EPI_LD;
  static constexpr size_t LDS_BYTES =
      sizeof(uint16_t) * (PIPE_ELEMS > EPI_ELEMS ? PIPE_ELEMS : EPI_ELEMS);
  static_assert(LDS_BYTES <= 160 * 1024, "LDS of one CU");
  static constexpr int A_CHUNKS = A_ROWS * BK / 8 / THREADS;  // DMA instructions per lane
  static constexpr int B_CHUNKS = BN * BK / 8 / THREADS;
  static_assert(BN * BK / 8 % THREADS == 0, "chunking");
  static_assert(KK % 2 == 0, "fragment double-buffer parity");
};

// One LDS-DMA instruction: 64 lanes x 16 bytes from per-lane global addresses to
// the KiB of LDS starting at lds_addr (wavefront-uniform).  Issued as inline
// assembly on purpose: when the compiler knows that LDS-DMA transfers are in
// flight it makes LDS reads it cannot disambiguate from them (every transposing
// read) wait for vmcnt(0), which drains the whole prefetch ring.  Completion is
// tracked by hand with wait_vmcnt; LDS reads stay ordinary compiler-tracked
// instructions.
__device__ __forceinline__ void dma16(const void* src, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
               :
               : "s"(lds_addr), "v"(src)
               : "memory", "m0");
}
// The same with the source split into a wavefront-uniform base (scalar registers)
// and a per-lane 32-bit byte offset: one address register per lane instead of
// two, and the base advances with scalar arithmetic shared by all of a K step's
// instructions instead of a 64-bit vector add per instruction.
// The LDS destination is lds_base (scalar register) + kLdsOff (immediate), formed
// in m0 by the one scalar add.
template <int kLdsOff>
__device__ __forceinline__ void dma16s(const void* base, uint32_t byte_off, uint32_t lds_base) {
  asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_base), "v"(byte_off), "s"(base), "n"(kLdsOff)
               : "memory", "m0", "scc");
}
// The same through a buffer descriptor (four scalar registers: base address, zero
// stride, num_records bytes, raw-buffer format word): the hardware checks every dword
// of the transfer against num_records and deposits zeros for those at or beyond it,
// so a K step that ends inside its tile needs neither a branch nor a per-lane select.
// The range check covers the lane offset only, which is why a K step advances the
// descriptor (base up, num_records down) instead of passing a scalar offset.
typedef int i32x4 __attribute__((ext_vector_type(4)));
constexpr int kRawBufferWord3 = 0x00020000;
__device__ __forceinline__ i32x4 buffer_descriptor(const void* base, uint32_t num_records) {
  const uint64_t a = reinterpret_cast<uint64_t>(base);
  i32x4 r;
  r[0] = static_cast<int>(static_cast<uint32_t>(a));
  r[1] = static_cast<int>(static_cast<uint32_t>(a >> 32) & 0xffffu);
  r[2] = static_cast<int>(num_records);
  r[3] = kRawBufferWord3;
  return r;
}
template <int kLdsOff>
__device__ __forceinline__ void dma16b(i32x4 rsrc, uint32_t byte_off, uint32_t lds_base) {
  asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
               :
               : "s"(lds_base), "v"(byte_off), "s"(rsrc), "n"(kLdsOff)
               : "memory", "m0", "scc");
}
__device__ __forceinline__ uint32_t lds_byte_addr(const void* p) {
  return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((NESTOR_LDS const void*)p));
}
// Eight consecutive contraction indices of one output index from a swizzled
// contraction-major tile: two transposing reads kRowElems * 4 elements apart.
template <int kRowElems>
__device__ __forceinline__ bf16x8 lds_read_tr_pair(const uint16_t* p0) {
  typedef __attribute__((__vector_size__(4 * sizeof(short)))) short v4s;
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NESTOR_LDS v4s*)(p0));
  v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NESTOR_LDS v4s*)(p0 + 4 * kRowElems));
  s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  return __builtin_bit_cast(bf16x8, v);
}

template <typename F, int... Is>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, Is...>) {
  (f(std::integral_constant<int, Is>{}), ...);
}
// f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N - 1>{})
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Swizzled element offset of (row, logical 16-byte piece c) in a
// contraction-contiguous tile with BK elements per row.
template <int BK>
__device__ __forceinline__ int kc_offset(int row, int c) {
  constexpr int cpr = BK / 8;            // pieces per row
  constexpr int rp = 256 / (BK * 2);     // rows per 256 bytes
  return row * BK + ((c ^ ((row / rp) % cpr)) * 8);
}
// Swizzled element offset of (contraction row k, column n) in a
// contraction-major tile with W elements per row (n a multiple of 4).
template <int W>
__device__ __forceinline__ int nc_offset(int k, int n) {
  return k * W + ((((n >> 3) ^ (4 * (k & 3))) << 3) | (n & 7));
}

inline int config_choice(const char* name, int fallback) {
  const char* v = std::getenv(name);
  return v != nullptr ? std::atoi(v) : fallback;
}

inline bool dims_ok(int64_t rows_pad, int64_t K, int64_t N, int32_t num_banks, int64_t max_tiles) {
  return rows_pad >= 0 && rows_pad <= INT32_MAX && K > 0 && N > 0 && K % 8 == 0 &&
         N % 8 == 0 && num_banks > 0 &&
         max_tiles == table_cap(kTiles128, rows_pad, num_banks);
}

// Compute units of the current device (0 if the query fails).  Initialised once, by
// whichever thread comes first (function-local statics are thread-safe).
inline int cu_count() {
  static const int cus = [] {
    int dev = 0;
    hipDeviceProp_t prop;
    return (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
               ? prop.multiProcessorCount
               : 0;
  }();
  return cus;
}

// Raises a kernel's dynamic LDS limit; meant as the initialiser of a function-local
// static of each launcher, so that it runs once per kernel and is safe to race into.
inline bool allow_dynamic_lds(const void* kernel, size_t bytes) {
  (void)hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes));
  return true;
}

// The register-staged e4m3-weight kernel (128-row tiles, weights widened on the way into
// LDS): the fallback of the streaming kernels for many rows per bank or odd widths.
// Defined beside the register-staged kernel.
int launch_fp8_staged(const GemmParams& p, void* stream);

}  // namespace nestor
