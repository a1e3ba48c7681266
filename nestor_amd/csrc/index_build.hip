// Dispatch index build: stable counting sort of routed rows by bank, the
// 16-row-aligned padded layout, the five dispatch maps and the GEMM tile table.
//
// Three launches (one for a batch of a few thousand rows: index_build_small), no
// atomics, no host reads:
//   1. wave_histogram   every wavefront counts the banks of its own contiguous
//                       chunk of rows into a private LDS histogram (ballot
//                       match-any, one LDS add per distinct bank per 64 rows).
//   2. plan_scan        one workgroup turns the per-chunk histograms into
//                       exclusive per-chunk bases, builds counts / raw_starts /
//                       padded_starts / offs and the tile table, and zeroes the
//                       slack entries of the maps.
//   3. scatter_maps     every wavefront replays its chunk in row order and
//                       hands each row its stable rank (chunk base + running
//                       LDS counter + rank among equal banks in the ballot),
//                       then writes order and the five maps.
// Results follow nestor/backbones/grouped_mm.py:253-318 bit for bit.
#include <mutex>

#include "common.hpp"

namespace nestor {
namespace {

constexpr int kMaxBanks = 4096;
constexpr int kHistBlock = 256;                   // 4 wavefronts, one chunk each
constexpr int kWavesPerBlock = kHistBlock / kWave;
constexpr int kScanBlock = 1024;
constexpr int kMaxChunks = 128;
constexpr int kIdBatch = 4;   // rounds of 64 rows whose ids a wavefront loads together

// Per-wavefront counters in LDS, updated by one lane at a time between wavefront
// barriers: volatile so every access is made, and typed as LDS so they are ds_
// instructions (a volatile access through a generic pointer stays a flat_ one).
typedef __attribute__((address_space(3))) volatile int32_t* LdsCounters;

__host__ __device__ inline int64_t chunk_rows_for(int64_t rows) {
  int64_t per = (rows + kMaxChunks - 1) / kMaxChunks;
  per = ((per + kWave - 1) / kWave) * kWave;
  return per < 256 ? 256 : per;
}

__device__ __forceinline__ int clamp_bank(int64_t id, int num_banks) {
  // Out-of-range ids are a caller error with undefined results in the
  // reference; clamping keeps every access in bounds.
  if (id < 0) return 0;
  if (id >= num_banks) return num_banks - 1;
  return static_cast<int>(id);
}

// Lanes of this wavefront that are valid and hold the same key.
__device__ __forceinline__ uint64_t match_any(int key, bool valid, int nbits) {
  uint64_t mask = __ballot(valid);
  for (int b = 0; b < nbits; ++b) {
    const bool bit = (key >> b) & 1;
    const uint64_t vote = __ballot(bit);
    mask &= bit ? vote : ~vote;
  }
  return mask;
}

// One wavefront counts the banks of rows [begin, end) into its histogram in LDS.
__device__ __forceinline__ void histogram_chunk(const int64_t* __restrict__ ids, int64_t begin,
                                                int64_t end, int num_banks, int nbits,
                                                LdsCounters hist) {
  const int lane = threadIdx.x % kWave;
  for (int e = lane; e < num_banks; e += kWave) hist[e] = 0;
  __builtin_amdgcn_wave_barrier();
  // Four rounds of 64 rows at a time: their ids are loaded together (one memory
  // latency per four rounds), then counted round by round.
  for (int64_t base = begin; base < end; base += kIdBatch * kWave) {
    int key[kIdBatch];
    bool valid[kIdBatch];
#pragma unroll
    for (int j = 0; j < kIdBatch; ++j) {
      const int64_t r = base + j * kWave + lane;
      valid[j] = r < end;
      key[j] = valid[j] ? clamp_bank(ids[r], num_banks) : 0;
    }
#pragma unroll
    for (int j = 0; j < kIdBatch; ++j) {
      if (base + j * kWave >= end) break;   // wave-uniform
      const uint64_t same = match_any(key[j], valid[j], nbits);
      if (valid[j] && lane == __ffsll(static_cast<unsigned long long>(same)) - 1)
        hist[key[j]] = hist[key[j]] + __popcll(same);
      __builtin_amdgcn_wave_barrier();
    }
  }
}

__global__ __launch_bounds__(kHistBlock) void wave_histogram(
    const int64_t* __restrict__ ids, int64_t rows, int num_banks, int nbits,
    int64_t chunk_rows, int num_chunks, int32_t* __restrict__ chunk_counts) {
  extern __shared__ int32_t lds_hist[];  // [kWavesPerBlock][num_banks]
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int chunk = blockIdx.x * kWavesPerBlock + wave;
  LdsCounters hist = (LdsCounters)(lds_hist + wave * num_banks);
  if (chunk < num_chunks) {
    const int64_t begin = chunk * chunk_rows;
    int64_t end = begin + chunk_rows;
    if (end > rows) end = rows;
    histogram_chunk(ids, begin, end, num_banks, nbits, hist);
    for (int e = lane; e < num_banks; e += kWave)
      chunk_counts[static_cast<int64_t>(chunk) * num_banks + e] = hist[e];
  }
}

// In-place exclusive scan of n int32 values in LDS by the whole workgroup;
// returns the total. scratch holds kScanBlock / kWave + 1 ints.
__device__ __forceinline__ int block_exclusive_scan(int32_t* vals, int n, int32_t* scratch) {
  const int tid = threadIdx.x;
  const int items = (n + kScanBlock - 1) / kScanBlock;
  const int begin = tid * items;
  int local = 0;
  for (int i = 0; i < items; ++i)
    if (begin + i < n) local += vals[begin + i];
  int incl = local;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const int up = __shfl_up(incl, off, kWave);
    if ((tid % kWave) >= off) incl += up;
  }
  const int wave = tid / kWave;
  if (tid % kWave == kWave - 1) scratch[wave] = incl;
  __syncthreads();
  // the wavefront totals, scanned by the first wavefront (kScanBlock / kWave <= kWave)
  static_assert(kScanBlock / kWave <= kWave, "one wavefront scans the wavefront totals");
  if (tid < kWave) {
    const int t = tid < kScanBlock / kWave ? scratch[tid] : 0;
    int run = t;
#pragma unroll
    for (int off = 1; off < kScanBlock / kWave; off <<= 1) {
      const int up = __shfl_up(run, off, kWave);
      if (tid >= off) run += up;
    }
    if (tid < kScanBlock / kWave) scratch[tid] = run - t;
    if (tid == kScanBlock / kWave - 1) scratch[kScanBlock / kWave] = run;
  }
  __syncthreads();
  int run = scratch[wave] + incl - local;
  for (int i = 0; i < items; ++i) {
    if (begin + i < n) {
      const int v = vals[begin + i];
      vals[begin + i] = run;
      run += v;
    }
  }
  const int total = scratch[kScanBlock / kWave];
  __syncthreads();
  return total;
}

template <typename T>
__device__ __forceinline__ void store_one(void* base, int64_t i);
template <>
__device__ __forceinline__ void store_one<float>(void* base, int64_t i) {
  reinterpret_cast<float*>(base)[i] = 1.0f;
}
template <>
__device__ __forceinline__ void store_one<uint16_t>(void* base, int64_t i) {
  reinterpret_cast<uint16_t*>(base)[i] = 0x3f80u;  // bf16 1.0
}

__device__ __forceinline__ void zero_slot(int64_t p, int64_t* pad_token,
                                          int64_t* pad_src_row, int64_t* eid_pad,
                                          void* pad_valid, int valid_dtype) {
  pad_token[p] = 0;
  pad_src_row[p] = 0;
  eid_pad[p] = 0;
  if (valid_dtype == NESTOR_HIP_F32)
    reinterpret_cast<float*>(pad_valid)[p] = 0.0f;
  else
    reinterpret_cast<uint16_t*>(pad_valid)[p] = 0;
}

// Tile tables.  A table is bank[cap] | row0[cap] | nrows[cap] | count for a capacity
// `cap` fixed by the static sizes; three of them sit back to back in the tile_table
// buffer:
//   kTiles128     every segment cut into tiles of up to 128 rows, then the slack tail
//                 behind the last segment as bank == -1 tiles;
//   kTilesBal160  every segment cut into the fewest tiles of at most five 32-row
//                 blocks, its blocks dealt evenly over them (530 rows = 17 blocks ->
//                 tiles of 4, 4, 4 and 5 blocks, not four full tiles and a fifth of 18
//                 rows that streams a whole weight panel for them), then the slack tail;
//   kTilesBal320  the same with at most ten blocks per tile (the 2 x 2 wavefront tiles).
// Every table covers every padded row exactly once.
__device__ __forceinline__ int tiles_of(int kind, int len) {
  if (kind == kTiles128) return (len + 127) / 128;
  const int cap = tile_blocks_cap(kind);
  return ((len + 31) / 32 + cap - 1) / cap;
}

// Writes one table for segments [start[e], start[e] + len[e]) held in LDS.
__device__ __forceinline__ void emit_tiles(int kind, const int32_t* seg_start, const int32_t* seg_len,
                           int32_t* tile_first, int32_t* scratch, int num_banks,
                           int64_t tail_begin, int64_t tail_end, int32_t* tile_table,
                           int64_t max_tiles) {
  const int tid = threadIdx.x;
  const int tile_rows = 32 * tile_blocks_cap(kind);
  for (int e = tid; e < num_banks; e += kScanBlock) tile_first[e] = tiles_of(kind, seg_len[e]);
  __syncthreads();
  const int bank_tiles = block_exclusive_scan(tile_first, num_banks, scratch);
  int32_t* t_bank = tile_table;
  int32_t* t_row0 = tile_table + max_tiles;
  int32_t* t_rows = tile_table + 2 * max_tiles;
  // a wavefront per bank, a lane per tile: a single bank with hundreds of tiles (a whole
  // batch as one segment) and hundreds of banks with a few tiles each both stay short
  for (int e = tid / kWave; e < num_banks; e += kScanBlock / kWave) {
    const int len = seg_len[e];
    const int n = tiles_of(kind, len);
    const int64_t blocks = (len + 31) / 32;
    for (int j = tid % kWave; j < n; j += kWave) {
      const int64_t t = tile_first[e] + j;
      if (t < max_tiles) {
        // tile j of n takes blocks [j * blocks / n, (j + 1) * blocks / n); cutting at 128
        // rows is the same rule with the blocks dealt four at a time
        int first, rows;
        if (kind == kTiles128) {
          first = j * 128;
          rows = 128;
        } else {
          const int b0 = static_cast<int>(j * blocks / n), b1 = static_cast<int>((j + 1) * blocks / n);
          first = 32 * b0;
          rows = 32 * (b1 - b0);
        }
        const int left = len - first;
        t_bank[t] = e;
        t_row0[t] = seg_start[e] + first;
        t_rows[t] = left < rows ? left : rows;
      }
    }
  }
  const int64_t tail_tiles = (tail_end - tail_begin + tile_rows - 1) / tile_rows;
  for (int64_t j = tid; j < tail_tiles; j += kScanBlock) {
    const int64_t t = bank_tiles + j;
    if (t < max_tiles) {
      const int64_t r0 = tail_begin + j * tile_rows;
      const int64_t left = tail_end - r0;
      t_bank[t] = -1;
      t_row0[t] = static_cast<int32_t>(r0);
      t_rows[t] = static_cast<int32_t>(left < tile_rows ? left : tile_rows);
    }
  }
  if (tid == 0) {
    int64_t total = bank_tiles + tail_tiles;
    if (total > max_tiles) total = max_tiles;
    tile_table[3 * max_tiles] = static_cast<int32_t>(total);
  }
  __syncthreads();  // tile_first / scratch are reused by the next table
}

// All three tables, back to back.
__device__ __forceinline__ void emit_all_tiles(const int32_t* seg_start, const int32_t* seg_len,
                               int32_t* tile_first, int32_t* scratch, int num_banks,
                               int64_t tail_begin, int64_t tail_end, int64_t rows_pad,
                               int32_t* tile_table) {
  for (int kind = 0; kind < kTileKinds; ++kind)
    emit_tiles(kind, seg_start, seg_len, tile_first, scratch, num_banks, tail_begin, tail_end,
               tile_table + table_offset(kind, rows_pad, num_banks),
               table_cap(kind, rows_pad, num_banks));
}

// The plan of a whole workgroup of kScanBlock threads over per-chunk histograms
// (global memory or LDS): see the file header.  `lds` holds 6 * num_banks +
// kScanBlock / kWave + 1 ints; on return s_raw = lds + num_banks and s_pstart =
// lds + 3 * num_banks hold the raw and the padded start of every bank.
__device__ __forceinline__ void plan_body(
    int32_t* chunk_counts, int num_chunks, int num_banks,
    int64_t rows_pad, int64_t capacity, int valid_dtype,
    int64_t* __restrict__ counts, int64_t* __restrict__ raw_starts,
    int64_t* __restrict__ padded_starts, int32_t* __restrict__ offs,
    int64_t* __restrict__ pad_token, int64_t* __restrict__ pad_src_row,
    int64_t* __restrict__ eid_pad, void* __restrict__ pad_valid,
    int32_t* __restrict__ tile_table, int32_t* lds) {
  int32_t* s_count = lds;                    // all rows of the bank
  int32_t* s_raw = s_count + num_banks;      // exclusive cumsum of counts
  int32_t* s_kept = s_raw + num_banks;       // rows that keep a padded slot
  int32_t* s_pstart = s_kept + num_banks;    // exclusive cumsum of ceil16(kept)
  int32_t* s_tiles = s_pstart + num_banks;
  int32_t* s_plen = s_tiles + num_banks;     // ceil16(kept)
  int32_t* scratch = s_plen + num_banks;     // kScanBlock / kWave + 1
  const int tid = threadIdx.x;

  // Per bank: exclusive prefix over the chunks (in place) and the total.
  for (int e = tid; e < num_banks; e += kScanBlock) {
    int total = 0;
    for (int c0 = 0; c0 < num_chunks; c0 += 8) {
      int v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j)  // independent loads first, then the serial adds
        v[j] = c0 + j < num_chunks
                   ? chunk_counts[static_cast<int64_t>(c0 + j) * num_banks + e]
                   : 0;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (c0 + j < num_chunks)
          chunk_counts[static_cast<int64_t>(c0 + j) * num_banks + e] = total;
        total += v[j];
      }
    }
    int kept = total;
    if (capacity > 0 && kept > capacity) kept = static_cast<int>(capacity);
    s_count[e] = total;
    s_raw[e] = total;
    s_kept[e] = kept;
    const int padded = (kept + NESTOR_HIP_ROW_ALIGN - 1) / NESTOR_HIP_ROW_ALIGN *
                       NESTOR_HIP_ROW_ALIGN;
    s_plen[e] = padded;
    s_pstart[e] = padded;
  }
  __syncthreads();
  block_exclusive_scan(s_raw, num_banks, scratch);
  const int padded_total = block_exclusive_scan(s_pstart, num_banks, scratch);

  for (int e = tid; e < num_banks; e += kScanBlock) {
    counts[e] = s_count[e];
    raw_starts[e] = s_raw[e];
    padded_starts[e] = s_pstart[e];
    // The last segment absorbs the slack so offs[-1] == rows_pad.
    offs[e] = e + 1 < num_banks ? s_pstart[e] + s_plen[e]
                                : static_cast<int32_t>(rows_pad);
  }
  // Slack inside the segments: at most 15 slots per bank.
  for (int i = tid; i < num_banks * NESTOR_HIP_ROW_ALIGN; i += kScanBlock) {
    const int e = i / NESTOR_HIP_ROW_ALIGN;
    const int j = i % NESTOR_HIP_ROW_ALIGN;
    if (s_kept[e] + j < s_plen[e])
      zero_slot(static_cast<int64_t>(s_pstart[e]) + s_kept[e] + j, pad_token,
                pad_src_row, eid_pad, pad_valid, valid_dtype);
  }
  // Slack tail behind the last segment.
  for (int64_t p = padded_total + tid; p < rows_pad; p += kScanBlock)
    zero_slot(p, pad_token, pad_src_row, eid_pad, pad_valid, valid_dtype);

  emit_all_tiles(s_pstart, s_plen, s_tiles, scratch, num_banks, padded_total, rows_pad, rows_pad,
                 tile_table);
}

__global__ __launch_bounds__(kScanBlock) void plan_scan(
    int32_t* __restrict__ chunk_counts, int num_chunks, int num_banks,
    int64_t rows_pad, int64_t capacity, int valid_dtype,
    int64_t* __restrict__ counts, int64_t* __restrict__ raw_starts,
    int64_t* __restrict__ padded_starts, int32_t* __restrict__ offs,
    int64_t* __restrict__ pad_token, int64_t* __restrict__ pad_src_row,
    int64_t* __restrict__ eid_pad, void* __restrict__ pad_valid,
    int32_t* __restrict__ tile_table) {
  extern __shared__ int32_t lds[];
  plan_body(chunk_counts, num_chunks, num_banks, rows_pad, capacity, valid_dtype, counts,
            raw_starts, padded_starts, offs, pad_token, pad_src_row, eid_pad, pad_valid,
            tile_table, lds);
}

// One wavefront replays rows [begin, end) in order.  next[e] holds the rank (within
// bank e) of the first row of e in this range and is advanced as rows are placed.
// kStart: int64 (global arrays) or int32 (the plan's LDS copies).
template <typename kStart>
__device__ __forceinline__ void scatter_chunk(
    const int64_t* __restrict__ ids, int64_t begin, int64_t end, int num_banks, int nbits,
    int slots, int64_t rows_pad, int64_t capacity, int valid_dtype, LdsCounters next,
    const kStart* raw_starts, const kStart* padded_starts, int64_t* __restrict__ order,
    int64_t* __restrict__ row_dest, int64_t* __restrict__ pad_token,
    int64_t* __restrict__ pad_src_row, int64_t* __restrict__ eid_pad,
    void* __restrict__ pad_valid, uint8_t* __restrict__ row_kept) {
  const int lane = threadIdx.x % kWave;
  const uint64_t lower = (1ull << lane) - 1ull;
  for (int64_t base0 = begin; base0 < end; base0 += kIdBatch * kWave) {
    int keys[kIdBatch];
#pragma unroll
    for (int j = 0; j < kIdBatch; ++j) {  // the ids of four rounds, loaded together
      const int64_t r = base0 + j * kWave + lane;
      keys[j] = r < end ? clamp_bank(ids[r], num_banks) : 0;
    }
#pragma unroll
    for (int j = 0; j < kIdBatch; ++j) {
      const int64_t base = base0 + j * kWave;
      if (base >= end) break;  // wave-uniform
      const int64_t r = base + lane;
      const bool valid = r < end;
      const int key = keys[j];
      const uint64_t same = match_any(key, valid, nbits);
      int rank = 0;
      if (valid) rank = next[key] + __popcll(same & lower);
      __builtin_amdgcn_wave_barrier();
      if (valid && lane == __ffsll(static_cast<unsigned long long>(same)) - 1)
        next[key] = next[key] + __popcll(same);
      __builtin_amdgcn_wave_barrier();
      if (!valid) continue;
      order[static_cast<int64_t>(raw_starts[key]) + rank] = r;
      const bool kept = capacity <= 0 || rank < capacity;
      if (row_kept != nullptr) row_kept[r] = kept ? 1 : 0;
      if (kept) {
        const int64_t dest = static_cast<int64_t>(padded_starts[key]) + rank;
        row_dest[r] = dest;
        pad_token[dest] = r / slots;
        pad_src_row[dest] = r;
        eid_pad[dest] = key;
        if (valid_dtype == NESTOR_HIP_F32)
          store_one<float>(pad_valid, dest);
        else
          store_one<uint16_t>(pad_valid, dest);
      } else {
        row_dest[r] = rows_pad - 1;  // always a slack row
      }
    }
  }
}

__global__ __launch_bounds__(kHistBlock) void scatter_maps(
    const int64_t* __restrict__ ids, int64_t rows, int num_banks, int nbits,
    int slots, int64_t rows_pad, int64_t capacity, int valid_dtype,
    int64_t chunk_rows, int num_chunks,
    const int32_t* __restrict__ chunk_bases, const int64_t* __restrict__ raw_starts,
    const int64_t* __restrict__ padded_starts, int64_t* __restrict__ order,
    int64_t* __restrict__ row_dest, int64_t* __restrict__ pad_token,
    int64_t* __restrict__ pad_src_row, int64_t* __restrict__ eid_pad,
    void* __restrict__ pad_valid, uint8_t* __restrict__ row_kept) {
  extern __shared__ int32_t lds_base[];  // [kWavesPerBlock][num_banks]
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int chunk = blockIdx.x * kWavesPerBlock + wave;
  if (chunk >= num_chunks) return;
  LdsCounters next = (LdsCounters)(lds_base + wave * num_banks);
  // Rank (within its bank) of the first row this chunk holds of each bank.
  for (int e = lane; e < num_banks; e += kWave)
    next[e] = chunk_bases[static_cast<int64_t>(chunk) * num_banks + e];
  __builtin_amdgcn_wave_barrier();
  const int64_t begin = chunk * chunk_rows;
  int64_t end = begin + chunk_rows;
  if (end > rows) end = rows;
  scatter_chunk<int64_t>(ids, begin, end, num_banks, nbits, slots, rows_pad, capacity, valid_dtype,
                         next, raw_starts, padded_starts, order, row_dest, pad_token, pad_src_row,
                         eid_pad, pad_valid, row_kept);
}

// The whole index build of a small batch as one workgroup: its kScanBlock / kWave
// wavefronts take one chunk of rows each, the chunk histograms never leave LDS, and
// the three phases are separated by workgroup barriers instead of launches (at a
// few thousand rows the three launches are mostly launch latency).
constexpr int kSmallWaves = kScanBlock / kWave;
constexpr int64_t kSmallChunkRows = 256;
constexpr int64_t kSmallMaxRows = kSmallWaves * kSmallChunkRows;
constexpr int kSmallMaxBanks = 512;

__global__ __launch_bounds__(kScanBlock) void index_build_small(
    const int64_t* __restrict__ ids, int64_t rows, int num_banks, int nbits, int slots,
    int64_t rows_pad, int64_t capacity, int valid_dtype, int64_t* __restrict__ order,
    int64_t* __restrict__ counts, int64_t* __restrict__ raw_starts,
    int64_t* __restrict__ padded_starts, int32_t* __restrict__ offs,
    int64_t* __restrict__ row_dest, int64_t* __restrict__ pad_token,
    int64_t* __restrict__ pad_src_row, int64_t* __restrict__ eid_pad,
    void* __restrict__ pad_valid, uint8_t* __restrict__ row_kept,
    int32_t* __restrict__ tile_table) {
  extern __shared__ int32_t lds_all[];
  int32_t* hists = lds_all;                             // [kSmallWaves][num_banks]
  int32_t* plan_lds = lds_all + kSmallWaves * num_banks;
  const int wave = threadIdx.x / kWave;
  const int64_t begin = wave * kSmallChunkRows < rows ? wave * kSmallChunkRows : rows;
  const int64_t end = begin + kSmallChunkRows < rows ? begin + kSmallChunkRows : rows;
  LdsCounters mine = (LdsCounters)(hists + wave * num_banks);
  histogram_chunk(ids, begin, end, num_banks, nbits, mine);
  __syncthreads();
  plan_body(hists, kSmallWaves, num_banks, rows_pad, capacity, valid_dtype, counts, raw_starts,
            padded_starts, offs, pad_token, pad_src_row, eid_pad, pad_valid, tile_table, plan_lds);
  __syncthreads();
  // The histograms now hold each chunk's first rank per bank; the plan's LDS copies
  // of the starts serve instead of the global arrays it has just written.
  scatter_chunk<int32_t>(ids, begin, end, num_banks, nbits, slots, rows_pad, capacity, valid_dtype,
                         mine, plan_lds + num_banks, plan_lds + 3 * num_banks, order, row_dest,
                         pad_token, pad_src_row, eid_pad, pad_valid, row_kept);
}

// The reference's map kernel boundary: order / starts come from the caller.
__global__ __launch_bounds__(256) void maps_from_order(
    const int64_t* __restrict__ ids, const int64_t* __restrict__ order,
    const int64_t* __restrict__ padded_starts, const int64_t* __restrict__ raw_starts,
    int64_t rows, int num_banks, int slots, int valid_dtype,
    int64_t* __restrict__ row_dest, int64_t* __restrict__ pad_token,
    int64_t* __restrict__ pad_src_row, int64_t* __restrict__ eid_pad,
    void* __restrict__ pad_valid) {
  const int64_t p = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (p >= rows) return;
  const int64_t orig = order[p];
  const int eid = clamp_bank(ids[orig], num_banks);
  const int64_t dest = padded_starts[eid] - raw_starts[eid] + p;
  row_dest[orig] = dest;
  pad_token[dest] = orig / slots;
  pad_src_row[dest] = orig;
  eid_pad[dest] = eid;
  if (valid_dtype == NESTOR_HIP_F32)
    store_one<float>(pad_valid, dest);
  else
    store_one<uint16_t>(pad_valid, dest);
}

__global__ __launch_bounds__(256) void slack_from_starts(
    const int64_t* __restrict__ padded_starts, const int64_t* __restrict__ raw_starts,
    int64_t rows, int num_banks, int64_t rows_pad, int valid_dtype,
    int64_t* __restrict__ pad_token, int64_t* __restrict__ pad_src_row,
    int64_t* __restrict__ eid_pad, void* __restrict__ pad_valid) {
  const int e = blockIdx.x;
  const int64_t count = (e + 1 < num_banks ? raw_starts[e + 1] : rows) - raw_starts[e];
  const int64_t begin = padded_starts[e] + count;
  const int64_t end = e + 1 < num_banks ? padded_starts[e + 1] : rows_pad;
  for (int64_t p = begin + threadIdx.x; p < end; p += blockDim.x)
    zero_slot(p, pad_token, pad_src_row, eid_pad, pad_valid, valid_dtype);
}

__global__ __launch_bounds__(kScanBlock) void tiles_from_offs(
    const int32_t* __restrict__ offs, int num_banks, int64_t rows_pad,
    int32_t* __restrict__ tile_table) {
  extern __shared__ int32_t lds[];
  int32_t* s_start = lds;
  int32_t* s_len = s_start + num_banks;
  int32_t* s_tiles = s_len + num_banks;
  int32_t* scratch = s_tiles + num_banks;
  for (int e = threadIdx.x; e < num_banks; e += kScanBlock) {
    const int32_t b = e == 0 ? 0 : offs[e - 1];
    s_start[e] = b;
    s_len[e] = offs[e] - b;
  }
  __syncthreads();
  emit_all_tiles(s_start, s_len, s_tiles, scratch, num_banks, 0, 0, rows_pad, tile_table);
}

int bits_for(int num_banks) {
  int nbits = 0;
  while ((1 << nbits) < num_banks) ++nbits;
  return nbits;
}

}  // namespace
}  // namespace nestor

using namespace nestor;

extern "C" size_t nestor_hip_index_build_workspace_bytes(int64_t rows, int32_t num_banks) {
  if (rows < 0 || num_banks <= 0) return 0;
  const int64_t cr = chunk_rows_for(rows);
  int64_t chunks = ceil_div(rows, cr);
  if (chunks < 1) chunks = 1;
  return static_cast<size_t>(chunks) * num_banks * sizeof(int32_t);
}

extern "C" int64_t nestor_hip_max_tiles(int64_t rows_pad, int32_t num_banks) {
  return table_cap(kTiles128, rows_pad, num_banks);
}

extern "C" int64_t nestor_hip_tile_table_ints(int64_t rows_pad, int32_t num_banks) {
  return table_offset(kTileKinds, rows_pad, num_banks);
}

namespace nestor {
namespace {

// Argument checks shared by the two index-build entry points (everything but
// the chunk-histogram buffer).
int index_build_check(const int64_t* expert_ids, int64_t rows, int32_t num_banks, int32_t slots,
                      int64_t rows_pad, int32_t valid_dtype, const int64_t* order,
                      const int64_t* counts, const int64_t* raw_starts,
                      const int64_t* padded_starts, const int32_t* offs, const int64_t* row_dest,
                      const int64_t* pad_token, const int64_t* pad_src_row, const int64_t* eid_pad,
                      const void* pad_valid, const int32_t* tile_table, int64_t max_tiles) {
  if (rows < 0 || num_banks <= 0 || slots <= 0) return NESTOR_HIP_EINVAL;
  if (num_banks > kMaxBanks) return NESTOR_HIP_ERANGE;
  if (valid_dtype != NESTOR_HIP_F32 && valid_dtype != NESTOR_HIP_BF16)
    return NESTOR_HIP_EINVAL;
  const int64_t want_pad = ceil_div(rows, NESTOR_HIP_ROW_ALIGN) * NESTOR_HIP_ROW_ALIGN +
                           static_cast<int64_t>(NESTOR_HIP_ROW_ALIGN) * num_banks;
  if (rows_pad != want_pad || rows_pad > INT32_MAX) return NESTOR_HIP_EINVAL;
  if (max_tiles != nestor_hip_max_tiles(rows_pad, num_banks)) return NESTOR_HIP_EINVAL;
  // the per-row arrays of an empty batch are empty: their pointers may be null
  if (!counts || !raw_starts || !padded_starts || !offs || !pad_token || !pad_src_row ||
      !eid_pad || !pad_valid || !tile_table ||
      (rows > 0 && (!expert_ids || !order || !row_dest)))
    return NESTOR_HIP_EINVAL;
  return NESTOR_HIP_OK;
}

// The three launches; chunk_counts holds num_chunks * num_banks int32 and is
// written in full by the first launch before anything reads it.
int index_build_launch(const int64_t* expert_ids, int64_t rows, int32_t num_banks, int32_t slots,
                       int64_t rows_pad, int64_t capacity, int32_t valid_dtype, int64_t* order,
                       int64_t* counts, int64_t* raw_starts, int64_t* padded_starts,
                       int32_t* offs, int64_t* row_dest, int64_t* pad_token,
                       int64_t* pad_src_row, int64_t* eid_pad, void* pad_valid,
                       uint8_t* row_kept, int32_t* tile_table, int64_t max_tiles,
                       int32_t* chunk_counts, hipStream_t s) {
  const int nbits = bits_for(num_banks);
  if (rows <= kSmallMaxRows && num_banks <= kSmallMaxBanks) {
    const size_t lds = sizeof(int32_t) * (static_cast<size_t>(kSmallWaves + 6) * num_banks +
                                          kScanBlock / kWave + 1);   // <= 46 KiB
    hipLaunchKernelGGL(index_build_small, dim3(1), dim3(kScanBlock), lds, s, expert_ids, rows,
                       num_banks, nbits, slots, rows_pad, capacity, valid_dtype, order, counts,
                       raw_starts, padded_starts, offs, row_dest, pad_token, pad_src_row,
                       eid_pad, pad_valid, row_kept, tile_table);
    return launch_status();
  }
  const int64_t cr = chunk_rows_for(rows);
  int num_chunks = static_cast<int>(ceil_div(rows, cr));
  if (num_chunks < 1) num_chunks = 1;
  const int blocks = static_cast<int>(ceil_div(num_chunks, kWavesPerBlock));
  const size_t wave_lds = sizeof(int32_t) * kWavesPerBlock * num_banks;
  hipLaunchKernelGGL(wave_histogram, dim3(blocks), dim3(kHistBlock), wave_lds, s,
                     expert_ids, rows, num_banks, nbits, cr, num_chunks, chunk_counts);
  const size_t scan_lds = sizeof(int32_t) * (6 * num_banks + kScanBlock / kWave + 1);
  // Beyond 64 KiB of dynamic LDS (more than ~2700 banks) a kernel has to be told so;
  // set on the current device each time, the case is rare.
  if (scan_lds > 65536 &&
      hipFuncSetAttribute(reinterpret_cast<const void*>(plan_scan),
                          hipFuncAttributeMaxDynamicSharedMemorySize,
                          static_cast<int>(scan_lds)) != hipSuccess) {
    (void)hipGetLastError();
    return NESTOR_HIP_ERANGE;
  }
  hipLaunchKernelGGL(plan_scan, dim3(1), dim3(kScanBlock), scan_lds, s, chunk_counts,
                     num_chunks, num_banks, rows_pad, capacity, valid_dtype, counts,
                     raw_starts, padded_starts, offs, pad_token, pad_src_row, eid_pad,
                     pad_valid, tile_table);
  if (rows > 0)
    hipLaunchKernelGGL(scatter_maps, dim3(blocks), dim3(kHistBlock), wave_lds, s,
                       expert_ids, rows, num_banks, nbits, slots, rows_pad, capacity,
                       valid_dtype, cr, num_chunks, chunk_counts, raw_starts,
                       padded_starts, order, row_dest, pad_token, pad_src_row, eid_pad,
                       pad_valid, row_kept);
  return launch_status();
}

}  // namespace
}  // namespace nestor

extern "C" int nestor_hip_index_build(
    const int64_t* expert_ids, int64_t rows, int32_t num_banks, int32_t slots,
    int64_t rows_pad, int64_t capacity, int32_t valid_dtype, int64_t* order,
    int64_t* counts, int64_t* raw_starts, int64_t* padded_starts, int32_t* offs,
    int64_t* row_dest, int64_t* pad_token, int64_t* pad_src_row, int64_t* eid_pad,
    void* pad_valid, uint8_t* row_kept, int32_t* tile_table, int64_t max_tiles,
    void* workspace, size_t workspace_bytes, void* stream) {
  const int bad = index_build_check(expert_ids, rows, num_banks, slots, rows_pad, valid_dtype,
                                    order, counts, raw_starts, padded_starts, offs, row_dest,
                                    pad_token, pad_src_row, eid_pad, pad_valid, tile_table,
                                    max_tiles);
  if (bad != NESTOR_HIP_OK) return bad;
  if (!workspace) return NESTOR_HIP_EINVAL;
  if (workspace_bytes < nestor_hip_index_build_workspace_bytes(rows, num_banks))
    return NESTOR_HIP_ENOSPC;
  return index_build_launch(expert_ids, rows, num_banks, slots, rows_pad, capacity, valid_dtype,
                            order, counts, raw_starts, padded_starts, offs, row_dest, pad_token,
                            pad_src_row, eid_pad, pad_valid, row_kept, tile_table, max_tiles,
                            static_cast<int32_t*>(workspace), static_cast<hipStream_t>(stream));
}

// ---------------------------------------------------------------------------
// The index build for callers that cannot allocate.  The chunk histograms live
// in a file-scope device array instead of a caller workspace.  Every GPU holds
// its own copy of the array at its own address: the address is looked up once
// per device (with that device current) and only that pointer is ever handed to
// a kernel -- in host code the array's name is a host-side stand-in, not a
// device address.
// ---------------------------------------------------------------------------
namespace nestor {
namespace {

constexpr int64_t kStaticHistInts = int64_t{kMaxChunks} * 2048;  // 1 MiB

}  // namespace
}  // namespace nestor

static __device__ __align__(256) int32_t scratch[nestor::kStaticHistInts];

namespace nestor {
namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
int32_t* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device; nullptr on failure.
int32_t* static_hist_buffer() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) {
      (void)hipGetLastError();
      return nullptr;
    }
    g_scratch_ptr[dev] = static_cast<int32_t*>(ptr);
  }
  return g_scratch_ptr[dev];
}

}  // namespace
}  // namespace nestor

extern "C" size_t nestor_hip_index_build_static_capacity_bytes(void) {
  return static_cast<size_t>(kStaticHistInts) * sizeof(int32_t);
}

extern "C" int nestor_hip_index_build_static(
    const int64_t* expert_ids, int64_t rows, int32_t num_banks, int32_t slots,
    int64_t rows_pad, int64_t capacity, int32_t valid_dtype, int64_t* order,
    int64_t* counts, int64_t* raw_starts, int64_t* padded_starts, int32_t* offs,
    int64_t* row_dest, int64_t* pad_token, int64_t* pad_src_row, int64_t* eid_pad,
    void* pad_valid, uint8_t* row_kept, int32_t* tile_table, int64_t max_tiles,
    void* stream) {
  const int bad = index_build_check(expert_ids, rows, num_banks, slots, rows_pad, valid_dtype,
                                    order, counts, raw_starts, padded_starts, offs, row_dest,
                                    pad_token, pad_src_row, eid_pad, pad_valid, tile_table,
                                    max_tiles);
  if (bad != NESTOR_HIP_OK) return bad;
  // The histograms of this call must fit the fixed array.
  if (nestor_hip_index_build_workspace_bytes(rows, num_banks) >
      nestor_hip_index_build_static_capacity_bytes())
    return NESTOR_HIP_ERANGE;
  int32_t* hist = static_hist_buffer();
  if (hist == nullptr) return NESTOR_HIP_ELAUNCH;
  // Nothing in the array has to start at zero: the first launch writes every
  // entry the later launches read.
  return index_build_launch(expert_ids, rows, num_banks, slots, rows_pad, capacity, valid_dtype,
                            order, counts, raw_starts, padded_starts, offs, row_dest, pad_token,
                            pad_src_row, eid_pad, pad_valid, row_kept, tile_table, max_tiles,
                            hist, static_cast<hipStream_t>(stream));
}

extern "C" int nestor_hip_build_dispatch_maps(
    const int64_t* expert_ids, const int64_t* order, const int64_t* padded_starts,
    const int64_t* raw_starts, int64_t rows, int32_t num_banks, int32_t slots,
    int64_t rows_pad, int32_t valid_dtype, int64_t* row_dest, int64_t* pad_token,
    int64_t* pad_src_row, int64_t* eid_pad, void* pad_valid, void* stream) {
  if (rows < 0 || num_banks <= 0 || slots <= 0 || rows_pad < rows) return NESTOR_HIP_EINVAL;
  if (valid_dtype != NESTOR_HIP_F32 && valid_dtype != NESTOR_HIP_BF16)
    return NESTOR_HIP_EINVAL;
  if (!padded_starts || !raw_starts || !row_dest || !pad_token || !pad_src_row ||
      !eid_pad || !pad_valid || (rows > 0 && (!expert_ids || !order)))
    return NESTOR_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(slack_from_starts, dim3(num_banks), dim3(256), 0, s, padded_starts,
                     raw_starts, rows, num_banks, rows_pad, valid_dtype, pad_token,
                     pad_src_row, eid_pad, pad_valid);
  if (rows > 0)
    hipLaunchKernelGGL(maps_from_order, dim3(static_cast<unsigned>(ceil_div(rows, 256))),
                       dim3(256), 0, s, expert_ids, order, padded_starts, raw_starts, rows,
                       num_banks, slots, valid_dtype, row_dest, pad_token, pad_src_row,
                       eid_pad, pad_valid);
  return launch_status();
}

extern "C" int nestor_hip_tile_schedule(const int32_t* offs, int32_t num_banks, int64_t rows_pad,
                                        int32_t* tile_table, int64_t max_tiles,
                                        void* stream) {
  if (!offs || !tile_table || num_banks <= 0 || rows_pad < 0) return NESTOR_HIP_EINVAL;
  if (num_banks > kMaxBanks) return NESTOR_HIP_ERANGE;
  if (max_tiles != nestor_hip_max_tiles(rows_pad, num_banks)) return NESTOR_HIP_EINVAL;
  const size_t lds = sizeof(int32_t) * (3 * num_banks + kScanBlock / kWave + 1);
  hipLaunchKernelGGL(tiles_from_offs, dim3(1), dim3(kScanBlock), lds,
                     static_cast<hipStream_t>(stream), offs, num_banks, rows_pad, tile_table);
  return launch_status();
}
