// Measurement aid: a stream of LDS-DMA transfers (global_load_lds_dwordx4) over a
// buffer of known size with the access patterns of the grouped GEMMs' operand
// fetches.  It exists so that hardware counters of HBM traffic (rocprofv3 --pmc
// FETCH_SIZE) can be read against a launch whose true byte count is known exactly
// and whose requests look like the GEMMs': the counters price requests of different
// widths differently, so a plain copy kernel is the wrong yardstick for them.
//
// The buffer is taken as `rows` rows of `row_bytes`.  One transfer instruction moves
// 1 KiB: 1024 / piece_bytes consecutive rows, piece_bytes contiguous bytes of each
// (piece_bytes = 64: sixteen 64-byte row pieces, the fetch of a contraction-contiguous
// operand at a K step of 32; piece_bytes = 512: two 512-byte row pieces, the fetch
// of a contraction-major weight tile).  A wavefront owns a strip of rows (along_rows
// = 0: walks along its rows, the next piece of the same rows each time, like K steps
// over a contraction-contiguous operand) or a strip of columns (along_rows = 1:
// walks down the rows, like K steps over a contraction-major one).  Every byte of
// the buffer is fetched exactly once.
#include "common.hpp"
#include "nestor_hip_probes.h"

namespace nestor {
namespace {

constexpr int kProbeThreads = 256;
constexpr int kSlots = 4;  // transfers in flight per wavefront

__global__ __launch_bounds__(kProbeThreads) void dma_stream_probe_kernel(
    const char* __restrict__ src, int64_t rows, int64_t row_bytes, int piece_bytes,
    int along_rows) {
  __shared__ __align__(16) char ring[kProbeThreads / kWave][kSlots][1024];
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int64_t gwave = static_cast<int64_t>(blockIdx.x) * (kProbeThreads / kWave) + wave;
  const int64_t nwaves = static_cast<int64_t>(gridDim.x) * (kProbeThreads / kWave);
  const int lanes_per_row = piece_bytes / 16;
  const int rows_per_instr = kWave / lanes_per_row;
  const int64_t row_blocks = rows / rows_per_instr;
  const int64_t col_blocks = row_bytes / piece_bytes;
  // strips: along_rows == 0 -> one strip per row block, col_blocks steps;
  //         along_rows == 1 -> one strip per column block, row_blocks steps
  const int64_t strips = along_rows ? col_blocks : row_blocks;
  const int64_t steps = along_rows ? row_blocks : col_blocks;
  const int64_t lane_off = static_cast<int64_t>(lane / lanes_per_row) * row_bytes +
                           (lane % lanes_per_row) * 16;
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
      (__attribute__((address_space(3))) const void*)&ring[wave][0][0]));
  int slot = 0;
  for (int64_t strip = gwave; strip < strips; strip += nwaves) {
    for (int64_t step = 0; step < steps; ++step) {
      const int64_t rb = along_rows ? step : strip;
      const int64_t cb = along_rows ? strip : step;
      const char* p = src + rb * rows_per_instr * row_bytes + cb * piece_bytes + lane_off;
      const uint32_t dst = lds0 + slot * 1024;
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\t"
                   "s_waitcnt vmcnt(3)"
                   :
                   : "s"(dst), "v"(p)
                   : "memory", "m0");
      slot = slot == kSlots - 1 ? 0 : slot + 1;
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// Measurement aid: what the matrix cores sustain on their own.  Every wavefront
// (four per CU, one per SIMD) issues v_mfma_f32_32x32x16_bf16 back to back on 16
// independent accumulator tiles, with no memory traffic at all, and workgroup 0
// reads the shader cycle counter and the constant-rate wall clock around its loop:
// their ratio is the shader clock the chip held under that load.  With constant
// operands the multipliers barely toggle; with random operands (4 x 4 different
// register sets, every product different) the power drawn is that of real data, and
// the clock the power management settles at is the ceiling of any bf16 GEMM.
typedef __attribute__((ext_vector_type(8))) __bf16 probe_bf16x8;
typedef __attribute__((ext_vector_type(16))) float probe_f32x16;

template <bool kRandom>
__global__ __launch_bounds__(kProbeThreads) void mfma_clock_probe_kernel(
    int iters, float* sink, unsigned long long* counters) {
  constexpr int kAcc = 16;
  probe_f32x16 acc[kAcc];
#pragma unroll
  for (int i = 0; i < kAcc; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
  probe_bf16x8 a[4], b[4];
  uint32_t h = (blockIdx.x * kProbeThreads + threadIdx.x) * 2654435761u + 17u;
#pragma unroll
  for (int k = 0; k < 4; ++k)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if constexpr (kRandom) {
        h = h * 1664525u + 1013904223u;
        a[k][e] = static_cast<__bf16>((static_cast<int>(h >> 16) - 32768) / 32768.0f);
        h = h * 1664525u + 1013904223u;
        b[k][e] = static_cast<__bf16>((static_cast<int>(h >> 16) - 32768) / 32768.0f * 0.05f);
      } else {
        a[k][e] = static_cast<__bf16>(static_cast<float>(threadIdx.x & 3));
        b[k][e] = static_cast<__bf16>(1.0f);
      }
    }
  const unsigned long long c0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < kAcc; ++i)
      acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i % 4], b[(i / 4) % 4], acc[i], 0, 0, 0);
  }
  const unsigned long long c1 = clock64(), w1 = wall_clock64();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < kAcc; ++i) s += acc[i][0] + acc[i][15];
  // keeps the products alive; the value is never a NaN pattern the test below matches
  if (s == -12345.678f) sink[0] = s;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    counters[0] = c1 - c0;
    counters[1] = w1 - w0;
    counters[2] = static_cast<unsigned long long>(gridDim.x) * (kProbeThreads / kWave) * iters * kAcc;
  }
}

// Measurement aid: the main loop of the GEMM kernels and nothing around it.  A
// wavefront multiplies a 128 x 128 accumulator tile (16 tiles of 32 x 32) in blocks of
// 16 MFMAs on fragments it read from LDS during the block before (two register sets,
// as in the kernels), reading the next block's kReads fragments (1 KiB each, one
// ds_read_b128) and issuing kDma LDS-DMA transfers of 1 KiB between the MFMAs at the
// kernels' spacing -- and has no barriers, no waiting for the transfers' data (they
// land in a ring nobody reads), no epilogue and no tile switches.  The transfers
// walk a region of region_bytes per XCD that the XCD's workgroups share (workgroup b
// runs on XCD b % 8), each from its own starting point: L2 hits after the first pass.
// The fragments are random bf16 values in (-1, 1) that change from block to block,
// so the matrix cores draw the power of real data.
template <int kReads, int kDma>
__global__ __launch_bounds__(kProbeThreads) void mfma_mix_probe_kernel(
    int iters, const char* __restrict__ src, long long region_bytes, float* sink,
    unsigned long long* counters) {
  __shared__ __align__(16) char lds[65536];
  static_assert(kReads == 0 || kReads == 8, "fragment reads per block of 16 MFMAs");
  static_assert(kDma >= 0 && kDma <= 8, "transfers per block of 16 MFMAs");
  probe_f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  // 32 KiB of fragments: random bf16 in (-1, 1)
  uint32_t h = (blockIdx.x * kProbeThreads + threadIdx.x) * 2654435761u + 17u;
  for (int i = threadIdx.x; i < 16384; i += kProbeThreads) {
    h = h * 1664525u + 1013904223u;
    const float v = (static_cast<int>(h >> 16) - 32768) / 32768.0f;
    reinterpret_cast<__bf16*>(lds)[i] = static_cast<__bf16>(v);
  }
  __syncthreads();
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  typedef __attribute__((address_space(3))) char LdsChar;
  typedef const __attribute__((address_space(3))) probe_bf16x8 LdsFrag;
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((LdsChar*)lds));
  // fragment f of register set p: 1 KiB at (8 * p + f) KiB of the first 16 KiB, shifted
  // by 4 KiB per wavefront inside 32 KiB; transfer ring: 8 KiB per wavefront behind it
  const uint32_t frag_addr = lds0 + lane * 16 + wave * 4096;
  const uint32_t ring = lds0 + 32768 + wave * 8192;
  const char* base = src + static_cast<long long>(blockIdx.x & 7) * region_bytes;
  long long pos = __builtin_amdgcn_readfirstlane(
      static_cast<int>(wave * 1024 + static_cast<long long>(blockIdx.x >> 3) * 32768 % region_bytes));
  uint32_t slot = 0;
  const uint32_t lane_off = lane * 16;
  probe_bf16x8 fa[2][4], fb[2][4];
  auto read_frag = [&](int set, int f) __attribute__((always_inline)) -> probe_bf16x8 {
    return *reinterpret_cast<LdsFrag*>(
        (LdsChar*)static_cast<uintptr_t>(frag_addr + (8 * set + f) * 1024));
  };
#pragma unroll
  for (int f = 0; f < 4; ++f) {
    fa[0][f] = read_frag(0, f);
    fb[0][f] = read_frag(0, 4 + f);
    fa[1][f] = read_frag(1, f);
    fb[1][f] = read_frag(1, 4 + f);
  }
  const unsigned long long c0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int par = 0; par < 2; ++par) {   // one block of 16 MFMAs on register set `par`
#pragma unroll
      for (int m = 0; m < 16; ++m) {
        // this block's share of the memory instructions, in front of MFMA m
        if (kReads == 8 && (m & 1) == 0) {
          const int f = m >> 1;  // B fragment 0, the A fragments, the other B fragments
          if (f == 0) fb[par ^ 1][0] = read_frag(par ^ 1, 4);
          else if (f <= 4) fa[par ^ 1][f - 1] = read_frag(par ^ 1, f - 1);
          else fb[par ^ 1][f - 4] = read_frag(par ^ 1, f);
        }
        if ((m * kDma) / 16 != ((m + 1) * kDma) / 16) {
          // scalar base + 32-bit lane offset, the kernels' addressing
          asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                       :
                       : "s"(ring + slot * 1024), "v"(lane_off), "s"(base + pos)
                       : "memory", "m0");
          slot = (slot + 1) & 7;
          pos += 4096;
          pos = pos >= region_bytes ? pos - region_bytes : pos;
        }
        const int j = m / 4, i = m % 4;
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[par][j], fa[par][i], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      // at most one block's transfers stay in flight, as behind the kernels' barrier
      if (kDma > 0) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kDma) : "memory");
      asm volatile("" ::: "memory");  // LDS counts as changed: the fragments are read again
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  const unsigned long long c1 = clock64(), w1 = wall_clock64();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) s += acc[i][j][0] + acc[i][j][15];
  if (s == -12345.678f) sink[0] = s;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    counters[0] = c1 - c0;
    counters[1] = w1 - w0;
    counters[2] = static_cast<unsigned long long>(gridDim.x) * (kProbeThreads / kWave) * iters * 32;
  }
}

}  // namespace
}  // namespace nestor

using namespace nestor;

extern "C" int nestor_hip_mfma_clock_probe(int32_t random_operands, int32_t iters,
                                           uint64_t* counters, void* stream) {
  if (!counters || iters <= 0) return NESTOR_HIP_EINVAL;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    return NESTOR_HIP_ELAUNCH;
  // the fourth counter is scratch for the kernel's never-taken store
  float* sink = reinterpret_cast<float*>(counters + 3);
  auto* c = reinterpret_cast<unsigned long long*>(counters);
  if (random_operands)
    hipLaunchKernelGGL(mfma_clock_probe_kernel<true>, dim3(cus), dim3(kProbeThreads), 0,
                       static_cast<hipStream_t>(stream), iters, sink, c);
  else
    hipLaunchKernelGGL(mfma_clock_probe_kernel<false>, dim3(cus), dim3(kProbeThreads), 0,
                       static_cast<hipStream_t>(stream), iters, sink, c);
  return launch_status();
}

extern "C" int nestor_hip_wall_clock_khz(void) {
  int dev = 0, khz = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess || khz <= 0)
    return -1;
  return khz;
}

extern "C" int nestor_hip_dma_stream_probe(const void* src, int64_t src_bytes, int64_t rows,
                                           int64_t row_bytes, int32_t piece_bytes,
                                           int32_t along_rows, void* stream) {
  if (!src || rows <= 0 || row_bytes <= 0) return NESTOR_HIP_EINVAL;
  // the walk touches exactly rows * row_bytes bytes from src on
  if (rows > INT64_MAX / row_bytes || rows * row_bytes > src_bytes) return NESTOR_HIP_EINVAL;
  if (piece_bytes != 64 && piece_bytes != 128 && piece_bytes != 256 && piece_bytes != 512 &&
      piece_bytes != 1024)
    return NESTOR_HIP_EINVAL;
  if (row_bytes % piece_bytes != 0 || rows % (1024 / piece_bytes) != 0) return NESTOR_HIP_EINVAL;
  hipLaunchKernelGGL(dma_stream_probe_kernel, dim3(2048), dim3(kProbeThreads), 0,
                     static_cast<hipStream_t>(stream), static_cast<const char*>(src), rows,
                     row_bytes, piece_bytes, along_rows);
  return launch_status();
}

extern "C" int nestor_hip_mfma_mix_probe(int32_t reads_per_step, int32_t transfers_per_step,
                                         int32_t iters, const void* src, int64_t src_bytes,
                                         int64_t region_bytes, uint64_t* counters, void* stream) {
  if (!counters || !src || iters <= 0) return NESTOR_HIP_EINVAL;
  // every workgroup's walk stays inside its XCD's region: whole 4 KiB steps, 32 KiB starts;
  // the eight regions lie back to back from src on
  if (region_bytes < 65536 || region_bytes % 32768 != 0) return NESTOR_HIP_EINVAL;
  if (region_bytes > INT64_MAX / 8 || 8 * region_bytes > src_bytes) return NESTOR_HIP_EINVAL;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    return NESTOR_HIP_ELAUNCH;
  float* sink = reinterpret_cast<float*>(counters + 3);
  auto* c = reinterpret_cast<unsigned long long*>(counters);
  const char* s = static_cast<const char*>(src);
  const dim3 grid(static_cast<unsigned>(cus)), block(kProbeThreads);
  auto st = static_cast<hipStream_t>(stream);
  const long long rb = region_bytes;
#define NESTOR_MIX(R, D)                                                                      \
  if (reads_per_step == 2 * (R) && transfers_per_step == 2 * (D)) {                           \
    hipLaunchKernelGGL((mfma_mix_probe_kernel<R, D>), grid, block, 0, st, iters, s, rb, sink, c); \
    return launch_status();                                                                   \
  }
  NESTOR_MIX(0, 0)
  NESTOR_MIX(8, 0)
  NESTOR_MIX(0, 4)
  NESTOR_MIX(8, 4)
  NESTOR_MIX(8, 5)
  NESTOR_MIX(8, 6)
#undef NESTOR_MIX
  return NESTOR_HIP_EINVAL;
}
