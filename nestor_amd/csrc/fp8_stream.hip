// e4m3 weight-streaming grouped GEMMs (the inference regime: a few rows per bank, a
// bank call is bound by reading the weights of the banks that got a row).
#include "gemm_common.hpp"

namespace nestor {
namespace {

// ---------------------------------------------------------------------------
// Weight-streaming kernel for e4m3 weights at a few rows per bank (the inference
// regime: a bank call is bound by reading the weights of the banks that got a
// row).  The register-staged kernel keeps one K step of 8 KiB of weights in
// flight per workgroup, which is latency times occupancy = a quarter of the HBM
// rate.  Here the e4m3 bytes go HBM -> LDS with the DMA path into a ring of
// kStages K steps of 64 x 256 bytes (48 KiB of weights in flight per workgroup;
// 16 KiB per CU already saturate the stream).  Weights are widened to bf16 in registers after a
// transposing 8-bit LDS read (ds_read_b64_tr_b8: lanes 2r, 2r+1 of a 16-lane group
// address 16 bytes of row r; lane j receives column j of the 8 x 16 byte block),
// and the MFMA runs in bf16 as in the other kernels.
//
// An item is (tile, 256 weight columns); its rows are walked in blocks of
// 32 * kMi rows, streaming the weight panel once per block: meant for tiles that
// fit one block.
// ---------------------------------------------------------------------------
// kW wavefronts per workgroup: 4 (each accumulates 64 weight columns; two workgroups
// per CU) or 8 (each 32 columns; one workgroup per CU whose ring may then take most of
// the LDS: the 96-row blocks, which with four wavefronts would leave a CU with one
// wavefront per SIMD and nothing to cover its waits).
// kBN weight columns (bytes of a K row) per item: 256, or 128 for a down projection
// with so few items that 256-column ones would leave CUs without work.
template <int kMi, int kStages, int kW, int kBN = 256>
struct Fp8StreamCfg {
  static constexpr int BN = kBN, BK = 64;
  static constexpr int WAVES = kW, THREADS = kW * kWave;
  static constexpr int NJ = kBN / 32 / kW;        // 32-column fragments per wavefront
  static_assert(kBN == 256 || (kBN == 128 && kW == 4), "256 columns, or 128 with four wavefronts");
  static constexpr int ROWS = 32 * kMi;
  static constexpr int A_BYTES = ROWS * BK * 2;   // bf16 activations, K-contiguous rows of 128 B
  static constexpr int B_BYTES = BK * BN;         // e4m3 weights, rows of BN bytes
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int A_WAVES = 4;                          // wavefronts 0..3 fetch the activations
  static constexpr int A_LOADS = A_BYTES / 1024 / A_WAVES;   // DMA instructions per such wavefront and K step
  static constexpr int B_LOADS = B_BYTES / 1024 / kW;        // ... per wavefront (all of them)
  static constexpr size_t LDS_BYTES = static_cast<size_t>(kStages) * STAGE_BYTES;
  static_assert(kW == 4 || kW == 8, "4 or 8 wavefronts");
  static_assert(A_BYTES % (1024 * A_WAVES) == 0, "whole DMA instructions per wavefront");
};

// kUpGate: the 256 weight columns of a K row are 128 of w_up and the same 128 of
// w_gate; a wavefront accumulates 32 columns of each and the epilogue writes
// hidden = silu(gate) * up with the bf16 rounding points of the unfused chain.
//
// The kernel is persistent: workgroup w walks the items (tile, column block)
// w, w + gridDim.x, ... and the ring runs across item boundaries -- while an item's
// last K steps are multiplied and its result is stored, the first steps of the
// workgroup's next item are already in flight, so a workgroup never restarts its
// stream.  Two state machines walk the same item list: the producer (which K step of
// which row block of which item the next transfer belongs to) runs kStages - 1 steps
// ahead of the consumer.  Everything the loop reads besides the ring comes through
// scalar loads from constant address space (tile table, column scales): a vector load
// there would make the compiler wait for vmcnt, i.e. for the whole ring.
#define NESTOR_CONST __attribute__((address_space(4)))
template <int kMi, int kStages, bool kUpGate, int kW, int kBN>
__global__ __launch_bounds__(kW * kWave, kW == 4 ? 2 : 1) void fp8w_stream_kernel(GemmParams p) {
  using C = Fp8StreamCfg<kMi, kStages, kW, kBN>;
  static_assert(!kUpGate || kBN == 256, "up|gate items are 128 + 128 columns");
  extern __shared__ __align__(16) uint16_t lds[];
  uint8_t* ring = reinterpret_cast<uint8_t*>(lds);
  constexpr int BN = C::BN, BK = C::BK, S = kStages, NJ = C::NJ, KK = BK / 16;
  constexpr int kThreads = C::THREADS;   // (shadows the file-wide four-wavefront constant)
  constexpr int kOutCols = kUpGate ? BN / 2 : BN;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  const NESTOR_CONST int32_t* tt = (const NESTOR_CONST int32_t*)p.tile_table;
  const int max_tiles = static_cast<int>(p.max_tiles);
  const int total = tt[3 * max_tiles] * p.n_tiles;   // items of this launch
  const int stride = static_cast<int>(gridDim.x);
  if (static_cast<int>(blockIdx.x) >= total) return;
  const int num_kt = static_cast<int>(p.K / BK);
  const int64_t b_kstep = static_cast<int64_t>(BK) * (p.tile_stride != 0 ? 128 : p.ldb);

  struct Item { int bank, row0, nrows, nt; };   // bank -1: slack rows to clear; -2: past the end
  auto load_item = [&](int it) __attribute__((always_inline)) {
    Item d = {-2, 0, 0, 0};
    if (it < total) {
      const int tile = it / p.n_tiles;
      d.nt = it - tile * p.n_tiles;
      d.bank = tt[tile];
      d.row0 = tt[max_tiles + tile];
      d.nrows = tt[2 * max_tiles + tile];
    }
    return d;
  };

  // ---- producer --------------------------------------------------------------
  int p_it = static_cast<int>(blockIdx.x);
  Item pi = load_item(p_it);
  while (pi.bank == -1) { p_it += stride; pi = load_item(p_it); }
  int p_rb = 0, p_kt = 0;
  const uint16_t* a_src[C::A_LOADS] = {};
  const uint8_t* b_src = nullptr;
  // Per-lane source addresses of this wavefront's DMA instructions for the
  // producer's (item, row block).
  // A: instruction i moves rows 8*(wave + 4i) .. +7, lane -> (row, position); the
  // position holds global piece (position ^ ((row >> 1) & 7)): conflict-free 128-bit
  // fragment reads.  Rows past the tile re-read its last row.
  // B: instruction i moves K rows 4*(wave + 4i) .. +3 of 256 bytes; position holds
  // global piece (position ^ (2 * (k & 7))): conflict-free transposing reads.
  // Tiled banks (p.tile_stride != 0) hold each 128 columns of a bank as one
  // contiguous [K][128] block: a workgroup then streams whole contiguous blocks (two
  // per item) instead of 128- or 256-byte pieces of rows 2-4 KiB apart.
  auto set_sources = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < C::A_LOADS; ++i) {
      const int row = 8 * ((wave & 3) + C::A_WAVES * i) + (lane >> 3);
      const int piece = (lane & 7) ^ ((row >> 1) & 7);
      const int r = p_rb + row < pi.nrows ? p_rb + row : pi.nrows - 1;
      a_src[i] = p.a + static_cast<int64_t>(pi.row0 + r) * p.lda + piece * 8;
    }
    const uint8_t* wq = static_cast<const uint8_t*>(p.b0) + static_cast<int64_t>(pi.bank) * p.bank_stride;
    const uint8_t* wq2 =
        kUpGate ? static_cast<const uint8_t*>(p.b1) + static_cast<int64_t>(pi.bank) * p.bank_stride : wq;
    const int64_t n0 = static_cast<int64_t>(pi.nt) * kOutCols;
    if constexpr (kBN == 256) {
      // Instruction i fetches K rows 4 * kW * i further down with the same swizzle
      // (a multiple of 8 rows): one per-lane address, uniform offsets.
      const int k = 4 * wave + (lane >> 4);
      const int piece = (lane & 15) ^ (2 * (k & 7));
      if constexpr (kUpGate) {
        const int64_t origin = p.tile_stride != 0
                                   ? static_cast<int64_t>(pi.nt) * p.tile_stride + static_cast<int64_t>(k) * 128
                                   : static_cast<int64_t>(k) * p.ldb + n0;
        b_src = (piece < 8 ? wq : wq2) + origin + (piece & 7) * 16;
      } else {
        const int64_t origin =
            p.tile_stride != 0
                ? static_cast<int64_t>(2 * pi.nt + (piece >> 3)) * p.tile_stride +
                      static_cast<int64_t>(k) * 128 + (piece & 7) * 16
                : static_cast<int64_t>(k) * p.ldb + n0 + piece * 16;
        b_src = wq + origin;
      }
    } else {
      // 128-byte rows: an instruction moves 8 K rows; position holds global piece
      // (position ^ (2 * ((k >> 1) & 3))).  Instruction i: 8 * kW rows further down.
      const int k = 8 * wave + (lane >> 3);
      const int piece = (lane & 7) ^ (2 * ((k >> 1) & 3));
      const int64_t origin = p.tile_stride != 0
                                 ? static_cast<int64_t>(pi.nt) * p.tile_stride + static_cast<int64_t>(k) * 128
                                 : static_cast<int64_t>(k) * p.ldb + n0;
      b_src = wq + origin + piece * 16;
    }
  };
  // Issues the producer's K step into `stage` and moves the producer on.  Behind the
  // last item it keeps re-fetching the last step it issued, so that every step of
  // the consumer sees the same number of transfers (uniform vmcnt bookkeeping).
  auto produce = [&](int stage) __attribute__((always_inline)) {
    uint8_t* sa = ring + stage * C::STAGE_BYTES;
    uint8_t* sb = sa + C::A_BYTES;
    if (kW == 4 || wave < C::A_WAVES) {
#pragma unroll
      for (int i = 0; i < C::A_LOADS; ++i)
        dma16(a_src[i] + static_cast<int64_t>(p_kt) * BK,
              lds_byte_addr(sa + (wave + C::A_WAVES * i) * 1024));
    }
#pragma unroll
    for (int i = 0; i < C::B_LOADS; ++i)
      dma16(b_src + static_cast<int64_t>(p_kt) * b_kstep + i * (b_kstep / (BK / (1024 / BN * kW))),
            lds_byte_addr(sb + (wave + kW * i) * 1024));
    if (pi.bank < 0) return;            // past the end: stay on the last step issued
    if (++p_kt < num_kt) return;
    p_rb += C::ROWS;
    if (p_rb >= pi.nrows) {
      p_rb = 0;
      do { p_it += stride; pi = load_item(p_it); } while (pi.bank == -1);
    }
    if (pi.bank >= 0) {
      p_kt = 0;
      set_sources();
    } else {
      p_kt = num_kt - 1;
    }
  };
  const bool streams = pi.bank >= 0;   // this workgroup has at least one item with weights
  if (streams) {
    set_sources();
#pragma unroll
    for (int t = 0; t + 1 < S; ++t) produce(t);
  }

  // ---- consumer --------------------------------------------------------------
  const int a_row = lane & 31, a_half = lane >> 5;
  const int grp = lane >> 4, gi = lane & 15;
  int cur = 0;
  for (int it = static_cast<int>(blockIdx.x); it < total; it += stride) {
    const Item ci = load_item(it);
    const int64_t n0 = static_cast<int64_t>(ci.nt) * kOutCols;
    if (ci.bank < 0) {
      const u32x4 zero = {0, 0, 0, 0};
      for (int c = tid; c < ci.nrows * (kOutCols / 8); c += kThreads) {
        const int row = c / (kOutCols / 8);
        st16o(p.out + static_cast<int64_t>(ci.row0 + row) * p.ldo + n0 + (c % (kOutCols / 8)) * 8, zero);
      }
      continue;
    }
    // Column scales of this wavefront's output columns (32 of each bank, or 64).
    typedef float f32x16s __attribute__((ext_vector_type(16)));
    // Four wavefronts: 32 columns of each bank (or 64 of the one); eight: 16 (or 32).
    constexpr int kColsPerWave = (kUpGate ? 128 : BN) / kW;
    const NESTOR_CONST float* sc_base =
        (const NESTOR_CONST float*)p.scale + static_cast<int64_t>(ci.bank) * p.N + n0 +
        kColsPerWave * wave;
    const NESTOR_CONST float* sc_base2 =
        kUpGate ? (const NESTOR_CONST float*)p.scale2 + static_cast<int64_t>(ci.bank) * p.N + n0 +
                      kColsPerWave * wave
                : sc_base + 32;
    f32x16s sc[2][2];
    sc[0][0] = *reinterpret_cast<const NESTOR_CONST f32x16s*>(sc_base);
    sc[1][0] = *reinterpret_cast<const NESTOR_CONST f32x16s*>(NJ == 1 && !kUpGate ? sc_base + 16 : sc_base2);
    if constexpr (NJ == 2) {
      sc[0][1] = *reinterpret_cast<const NESTOR_CONST f32x16s*>(sc_base + 16);
      sc[1][1] = *reinterpret_cast<const NESTOR_CONST f32x16s*>(sc_base2 + 16);
    }

    for (int rb = 0; rb < ci.nrows; rb += C::ROWS) {
      f32x16 acc[kMi][NJ];
#pragma unroll
      for (int i = 0; i < kMi; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
          for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

      // One pass over the weight panel.  A K step is "opened" (its transfers waited
      // for, the barrier, the producer's next step issued, its fragments read from
      // LDS into one of two register buffers) one step before its MFMAs run: the LDS
      // reads of step kt + 1 are in flight under the MFMAs of step kt.  With every
      // wavefront of a workgroup in step behind the barrier, reads and MFMAs would
      // otherwise alternate instead of overlapping.  kLive: row blocks of 32 that hold
      // rows of the tile; the ones behind them are skipped.
      auto run_pass = [&](auto live_tag) __attribute__((always_inline)) {
        constexpr int kLive = decltype(live_tag)::value;
        bf16x8 fa[2][KK][kLive];
        u32x2 raw[2][KK][NJ];
        auto open_step = [&](auto buf_tag) __attribute__((always_inline)) {
          constexpr int buf = decltype(buf_tag)::value;
          // this step has landed (for this wavefront's transfers) ...
          if (kW == 4 || wave < C::A_WAVES) wait_vmcnt<(S - 2) * (C::A_LOADS + C::B_LOADS)>();
          else wait_vmcnt<(S - 2) * C::B_LOADS>();
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
          __builtin_amdgcn_s_barrier();   // ... for everyone's, and the previous step's reads are done
          produce(cur == 0 ? S - 1 : cur - 1);
          const uint8_t* sa = ring + cur * C::STAGE_BYTES;
          const uint8_t* sb = sa + C::A_BYTES;
#pragma unroll
          for (int kk = 0; kk < KK; ++kk) {
#pragma unroll
            for (int i = 0; i < kLive; ++i) {
              const int row = 32 * i + a_row;
              const int piece = (2 * kk + a_half) ^ ((row >> 1) & 7);
              fa[buf][kk][i] = *reinterpret_cast<const bf16x8*>(sa + row * 128 + piece * 16);
            }
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
              const int k = 16 * kk + 8 * (grp >> 1) + (gi >> 1);
              // Four wavefronts: fragment j is 32 columns of up (j = 0) / gate (j = 1),
              // or of the one bank.  Eight: the one fragment is 16 columns of up beside
              // the same 16 of gate (an accumulator lane then holds matching pairs), or
              // 32 columns of the one bank.
              const int col_piece =
                  NJ == 2 ? (kUpGate ? 8 * j + 2 * wave + (grp & 1) : 4 * wave + 2 * j + (grp & 1))
                          : (kUpGate ? 8 * (grp & 1) + wave : 2 * wave + (grp & 1));
              const int piece = col_piece ^ (kBN == 256 ? 2 * (k & 7) : 2 * ((k >> 1) & 3));
              typedef int v2i __attribute__((ext_vector_type(2)));
              const v2i r = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                  (NESTOR_LDS v2i*)(sb + k * BN + piece * 16 + 8 * (gi & 1)));
              raw[buf][kk][j] = u32x2{static_cast<uint32_t>(r[0]), static_cast<uint32_t>(r[1])};
            }
          }
          cur = cur == S - 1 ? 0 : cur + 1;
        };
        auto multiply = [&](auto buf_tag) __attribute__((always_inline)) {
          constexpr int buf = decltype(buf_tag)::value;
#pragma unroll
          for (int kk = 0; kk < KK; ++kk) {
            bf16x8 fb[NJ];
#pragma unroll
            for (int j = 0; j < NJ; ++j)
              fb[j] = __builtin_bit_cast(bf16x8, fp8x8_to_bf16x8_exact(raw[buf][kk][j]));
#pragma unroll
            for (int i = 0; i < kLive; ++i)
#pragma unroll
              for (int j = 0; j < NJ; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[buf][kk][i], acc[i][j], 0, 0, 0);
          }
        };
        using B0 = std::integral_constant<int, 0>;
        using B1 = std::integral_constant<int, 1>;
        open_step(B0{});
        int kt = 1;
        for (; kt + 1 < num_kt; kt += 2) {
          open_step(B1{});
          multiply(B0{});
          open_step(B0{});
          multiply(B1{});
        }
        if (kt < num_kt) {
          open_step(B1{});
          multiply(B0{});
          multiply(B1{});
        } else {
          multiply(B0{});
        }
      };
      if constexpr (kMi == 1) {
        run_pass(std::integral_constant<int, 1>{});
      } else {
        const int live_blocks = (ci.nrows - rb + 31) >> 5;   // wave-uniform
        if (live_blocks >= kMi) run_pass(std::integral_constant<int, kMi>{});
        else if (kMi == 3 && live_blocks == 2) run_pass(std::integral_constant<int, 2>{});
        else run_pass(std::integral_constant<int, 1>{});
      }

      // ---- epilogue: scale per output column, round, store the block's rows ----
      // Accumulator entry 4q + e of a lane is weight column 8q + 4*(lane >> 5) + e of the fragment; with
      // four wavefronts its scale is sc[j][q >> 1][8 * (q & 1) + 4 * (lane >> 5) + e].
      // (The lane index goes through an empty asm so that the per-lane selection of
      // scale values below is not hoisted out of the loops, where it would hold 64
      // registers across the main loop.)
      int lane_here = lane;
      asm volatile("" : "+v"(lane_here));
      const bool upper = lane_here >= 32;
#pragma unroll
      for (int i = 0; i < kMi; ++i) {
        const int row = rb + 32 * i + (lane & 31);
        uint16_t* dst = p.out + static_cast<int64_t>(ci.row0 + row) * p.ldo;
        if constexpr (kUpGate && kW == 8) {
          // One fragment: accumulator entries 0..7 are 8 of this wavefront's 16 up
          // columns, entries 8..15 the same columns of gate.
#pragma unroll
          for (int q = 0; q < 2; ++q) {
            const int64_t n = n0 + 16 * wave + 8 * q + 4 * (lane >> 5);
            float h[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int s = 8 * q + e;
              const float su = upper ? sc[0][0][s + 4] : sc[0][0][s];
              const float sg = upper ? sc[1][0][s + 4] : sc[1][0][s];
              const float u = round_bf16(acc[i][0][4 * q + e] * su);
              const float g = round_bf16(acc[i][0][8 + 4 * q + e] * sg);
              h[e] = silu_rounded(g) * u;
            }
            const u32x2 packed = {pack_bf16x2(h[0], h[1]), pack_bf16x2(h[2], h[3])};
            if (row < ci.nrows) *reinterpret_cast<u32x2*>(dst + n) = packed;
          }
        } else if constexpr (kUpGate) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int64_t n = n0 + 32 * wave + 8 * q + 4 * (lane >> 5);
            float h[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int s = 8 * (q & 1) + e;
              const float su = upper ? sc[0][q >> 1][s + 4] : sc[0][q >> 1][s];
              const float sg = upper ? sc[1][q >> 1][s + 4] : sc[1][q >> 1][s];
              const float u = round_bf16(acc[i][0][4 * q + e] * su);
              const float g = round_bf16(acc[i][1][4 * q + e] * sg);
              h[e] = silu_rounded(g) * u;
            }
            const u32x2 packed = {pack_bf16x2(h[0], h[1]), pack_bf16x2(h[2], h[3])};
            if (row < ci.nrows) *reinterpret_cast<u32x2*>(dst + n) = packed;
          }
        } else {
#pragma unroll
          for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int64_t n = n0 + 32 * NJ * wave + 32 * j + 8 * q + 4 * (lane >> 5);
              float v[4];
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const int s = 8 * (q & 1) + e;
                // (a wavefront with one fragment keeps its second 16 scales in sc[1][0])
                const f32x16s& part = NJ == 1 ? sc[q >> 1][0] : sc[j][q >> 1];
                v[e] = acc[i][j][4 * q + e] * (upper ? part[s + 4] : part[s]);
              }
              const u32x2 packed = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
              if (row < ci.nrows) *reinterpret_cast<u32x2*>(dst + n) = packed;
            }
        }
      }
    }
  }
  wait_vmcnt<0>();   // the steps the producer issued past the end
}

// Rows a workgroup of the e4m3 stream kernels covers per pass over its weight panel:
// 32 (cfg 1: four wavefronts, two workgroups per CU), 64 (cfg 2) or 96 (cfg 3; both
// eight wavefronts, one workgroup per CU).  A bank with more rows than that streams its
// weights once per pass, so the choice follows the average bank with a margin for the
// spread of the counts (which the host cannot read): at 64 rows per bank on average
// half of the banks would take two passes with 64-row blocks.  0: many rows per bank,
// the register-staged kernel.
int fp8_stream_config(int64_t avg_rows) {
  if (avg_rows <= 20) return 1;
  if (avg_rows <= 44) return 2;
  if (avg_rows <= 80) return 3;
  return 0;
}

template <int kMi, int kStages, bool kUpGate, int kW = 4, int kBN = 256>
int launch_fp8_stream(GemmParams p, void* stream) {
  using C = Fp8StreamCfg<kMi, kStages, kW, kBN>;
  p.n_tiles = static_cast<int>(p.N / (kUpGate ? C::BN / 2 : C::BN));
  int64_t blocks = p.max_tiles * p.n_tiles;
  if (blocks > INT32_MAX) return NESTOR_HIP_ERANGE;
  static const bool configured = allow_dynamic_lds(
      reinterpret_cast<const void*>(fp8w_stream_kernel<kMi, kStages, kUpGate, kW, kBN>), C::LDS_BYTES);
  (void)configured;
  // Persistent workgroups, as many per CU as the ring's LDS allows; fewer when the
  // launch cannot have that many items.
  const int cus = cu_count();
  if (cus <= 0) return NESTOR_HIP_ELAUNCH;
  constexpr int kPerCu = kW == 4 ? 2 : 1;
  if (blocks > kPerCu * cus) blocks = kPerCu * cus;
  hipLaunchKernelGGL((fp8w_stream_kernel<kMi, kStages, kUpGate, kW, kBN>),
                     dim3(static_cast<unsigned>(blocks)), dim3(C::THREADS), C::LDS_BYTES,
                     static_cast<hipStream_t>(stream), p);
  return launch_status();
}

}  // namespace
}  // namespace nestor

using namespace nestor;

extern "C" int nestor_hip_grouped_gemm_fp8w_nn(const void* a, const void* b_q,
                                               const float* scale, void* out,
                                               int64_t rows_pad, int64_t K, int64_t N,
                                               int32_t num_banks, const int32_t* tile_table,
                                               int64_t max_tiles, int32_t tiled, void* stream) {
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
  // A few rows per bank: the call is bound by streaming the weights.  Average
  // rows per bank from the static sizes (rows_pad holds 16 slack rows per bank).
  if (tiled != 0) {
    if (N % 128 != 0) return NESTOR_HIP_EINVAL;
    p.tile_stride = K * 128;
  }
  const int64_t avg_rows = (rows_pad - 16 * static_cast<int64_t>(num_banks)) / num_banks;
  int cfg = config_choice("NESTOR_HIP_FP8_CFG", fp8_stream_config(avg_rows));
  if (K % 64 != 0 || N % 256 != 0) cfg = 0;
  // A bank with few experts and a narrow output (the public bank's down projection:
  // 16 experts x 8 items of 256 columns) cannot fill the device with 256-column
  // items: 128-column ones, two workgroups per CU.
  const int narrow_forced = config_choice("NESTOR_HIP_FP8_NARROW", -1);
  const bool narrow = narrow_forced >= 0 ? narrow_forced != 0
                                         : static_cast<int64_t>(num_banks) * (N / 256) < 3 * cu_count() / 2;
  if (narrow) {
    if (cfg == 1) return launch_fp8_stream<1, 4, false, 4, 128>(p, stream);
    if (cfg == 2) return launch_fp8_stream<2, 4, false, 4, 128>(p, stream);
    if (cfg == 3) return launch_fp8_stream<3, 4, false, 4, 128>(p, stream);
  }
  if (cfg == 1) return launch_fp8_stream<1, 4, false>(p, stream);
  if (cfg == 2) return launch_fp8_stream<2, 4, false, 8>(p, stream);
  if (cfg == 3) return launch_fp8_stream<3, 4, false, 8>(p, stream);
  return launch_fp8_staged(p, stream);
}

extern "C" int nestor_hip_grouped_gemm_fp8w_upgate_swiglu(
    const void* a, const void* up_q, const void* gate_q, const float* scale_up,
    const float* scale_gate, void* hidden, int64_t rows_pad, int64_t K, int64_t H,
    int32_t num_banks, const int32_t* tile_table, int64_t max_tiles, int32_t tiled,
    void* stream) {
  if (!dims_ok(rows_pad, K, H, num_banks, max_tiles) || K % 64 != 0 || H % 128 != 0)
    return NESTOR_HIP_EINVAL;
  if (rows_pad == 0) return NESTOR_HIP_OK;
  if (!a || !up_q || !gate_q || !scale_up || !scale_gate || !hidden || !tile_table)
    return NESTOR_HIP_EINVAL;
  GemmParams p = {};
  p.a = static_cast<const uint16_t*>(a);
  p.lda = K;
  p.b0 = up_q;
  p.b1 = gate_q;
  p.bank_stride = K * H;
  p.ldb = H;
  p.scale = scale_up;
  p.scale2 = scale_gate;
  p.out = static_cast<uint16_t*>(hidden);
  p.ldo = H;
  p.K = K;
  p.N = H;
  p.tile_table = tile_table;
  p.max_tiles = max_tiles;
  if (tiled != 0) p.tile_stride = K * 128;  // H % 128 == 0 was checked above
  const int64_t avg_rows = (rows_pad - 16 * static_cast<int64_t>(num_banks)) / num_banks;
  int cfg = config_choice("NESTOR_HIP_FP8_CFG", fp8_stream_config(avg_rows));
  if (cfg == 1) return launch_fp8_stream<1, 4, true>(p, stream);
  if (cfg == 3 || cfg == 0) return launch_fp8_stream<3, 4, true, 8>(p, stream);
  return launch_fp8_stream<2, 4, true, 8>(p, stream);
}
