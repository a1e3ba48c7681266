// Shared device/host helpers for the gfx950 expert-path kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "nestor_hip.h"

namespace nestor {

constexpr int kWave = 64;

typedef __bf16 bf16_t;
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// 16-byte global load/store of 8 bf16 values.
__device__ __forceinline__ u32x4 ld16(const void* p) {
  return *reinterpret_cast<const u32x4*>(p);
}
__device__ __forceinline__ void st16(void* p, u32x4 v) {
  *reinterpret_cast<u32x4*>(p) = v;
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) {
  return __builtin_bit_cast(float, bits16 << 16);
}
// Round-to-nearest-even fp32 -> bf16 (the hardware conversion on gfx950).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  bf16_t b = static_cast<bf16_t>(f);
  return static_cast<uint32_t>(__builtin_bit_cast(uint16_t, b));
}
__device__ __forceinline__ float round_bf16(float f) {
  return bf16_bits_to_f32(f32_to_bf16_bits(f));
}
// silu(g) = g / (1 + exp(-g)) in fp32, rounded to bf16 (the activation's rounding
// point in the reference chain).  The quotient goes through the hardware
// reciprocal (1 ulp): the ten-instruction IEEE division sequence is a measurable
// share of the fused up|gate epilogue, and the bf16 rounding that follows hides
// the difference except on rounding ties.  Every kernel takes it from here, so the
// fused and the unfused paths agree bit for bit.
__device__ __forceinline__ float silu_rounded(float g) {
  return round_bf16(g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)));
}
// Two values through one v_cvt_pk_bf16_f32 (converted one by one the compiler
// spends four instructions per pair: two converts with a dead half, a shift, an or).
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef bf16_t bf16x2_t __attribute__((ext_vector_type(2)));
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
// Unpack 8 bf16 (one 16-byte chunk) to fp32.
__device__ __forceinline__ void unpack8(u32x4 v, float* f) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = bf16_bits_to_f32(v[i] & 0xffffu);
    f[2 * i + 1] = bf16_bits_to_f32(v[i] >> 16);
  }
}
__device__ __forceinline__ u32x4 pack8(const float* f) {
  u32x4 v;
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = pack_bf16x2(f[2 * i], f[2 * i + 1]);
  return v;
}

// Load 8 consecutive elements of a bf16 or fp32 row as fp32.
template <bool kF32>
__device__ __forceinline__ void load8_as_f32(const void* base, int64_t elem, float* f) {
  if constexpr (kF32) {
    const float* p = reinterpret_cast<const float*>(base) + elem;
    f32x4 a = *reinterpret_cast<const f32x4*>(p);
    f32x4 b = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[i] = a[i];
      f[4 + i] = b[i];
    }
  } else {
    const uint16_t* p = reinterpret_cast<const uint16_t*>(base) + elem;
    unpack8(ld16(p), f);
  }
}
template <bool kF32>
__device__ __forceinline__ void store8_from_f32(void* base, int64_t elem, const float* f) {
  if constexpr (kF32) {
    float* p = reinterpret_cast<float*>(base) + elem;
    f32x4 a, b;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a[i] = f[i];
      b[i] = f[4 + i];
    }
    *reinterpret_cast<f32x4*>(p) = a;
    *reinterpret_cast<f32x4*>(p + 4) = b;
  } else {
    uint16_t* p = reinterpret_cast<uint16_t*>(base) + elem;
    st16(p, pack8(f));
  }
}

// A scalar of a bf16 / fp32 vector as fp32.
__device__ __forceinline__ float load_scalar(const void* base, int64_t i, int dtype) {
  if (dtype == NESTOR_HIP_F32) return reinterpret_cast<const float*>(base)[i];
  return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(base)[i]);
}
// pad_valid is exactly 1 or 0 in either dtype: any non-zero magnitude is "real".
__device__ __forceinline__ bool load_valid(const void* base, int64_t i, int dtype) {
  if (dtype == NESTOR_HIP_F32)
    return (reinterpret_cast<const uint32_t*>(base)[i] & 0x7fffffffu) != 0;
  return (reinterpret_cast<const uint16_t*>(base)[i] & 0x7fffu) != 0;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

inline int launch_status() {
  return hipGetLastError() == hipSuccess ? NESTOR_HIP_OK : NESTOR_HIP_ELAUNCH;
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// The three tile tables of a tile_table buffer (written by the index build, walked by
// the grouped GEMMs): their capacities depend on the static sizes only.
//   kTiles128     every segment cut into tiles of up to 128 rows;
//   kTilesBal160  every segment cut into the fewest tiles of up to five 32-row blocks,
//                 the blocks dealt evenly over a segment's tiles;
//   kTilesBal320  the same with up to ten 32-row blocks per tile.
enum TileKind { kTiles128 = 0, kTilesBal160 = 1, kTilesBal320 = 2, kTileKinds = 3 };

// 32-row blocks a tile of this kind holds at most.
__host__ __device__ inline int tile_blocks_cap(int kind) {
  return kind == kTiles128 ? 4 : kind == kTilesBal160 ? 5 : 10;
}
// A balanced table never holds more tiles than cutting at 128 (256) rows would.
__host__ __device__ inline int64_t table_cap(int kind, int64_t rows_pad, int num_banks) {
  if (kind == kTilesBal320) return rows_pad / 256 + num_banks + 2;
  return rows_pad / 128 + num_banks + 2;
}
__host__ __device__ inline int64_t table_offset(int kind, int64_t rows_pad, int num_banks) {
  int64_t off = 0;
  for (int k = 0; k < kind; ++k) off += 3 * table_cap(k, rows_pad, num_banks) + 1;
  return off;
}

}  // namespace nestor
