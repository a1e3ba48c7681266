// Host check of the direct-to-LDS transfers' address arithmetic (built and run by
// tests/test_dma_addressing.py; no GPU).  It calls the functions the kernels call
// (nestor_amd/csrc/dma_addressing.hpp) for every wavefront, lane, transfer and K step of
// ragged shapes and asserts that each 16-byte piece lies inside the rows / columns it may
// touch, that the weight-gradient descriptors never reach past their operand and never
// underflow while a K loop moves them on, and that each transfer fills its KiB of the
// LDS stage exactly once.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "dma_addressing.hpp"

using namespace nestor::dma;

static long checks = 0;
#define REQUIRE(cond, ...)                                   \
  do {                                                       \
    ++checks;                                                \
    if (!(cond)) {                                           \
      std::printf("FAILED %s:%d %s: ", __FILE__, __LINE__, #cond); \
      std::printf(__VA_ARGS__);                              \
      std::printf("\n");                                     \
      std::exit(1);                                          \
    }                                                        \
  } while (0)

// One row-tiled configuration: tile heights up to BM, A stage of A_ROWS rows.
template <int BM, int BN, int BK, int WAVES, bool kBContig, int kSub>
void check_rows(int64_t K, int64_t N, int64_t lda, int64_t ldb, int nrows, int64_t n0, int phases) {
  constexpr int THREADS = 64 * WAVES;
  constexpr int A_UNIT = THREADS * 8 / BK;
  constexpr int A_ROWS = (BM + A_UNIT - 1) / A_UNIT * A_UNIT;
  constexpr int A_CHUNKS = A_ROWS * BK / 8 / THREADS, B_CHUNKS = BN * BK / 8 / THREADS;
  constexpr int BW = BN / kSub;
  const int last_row = nrows - 1;
  const int num_kt = static_cast<int>((K + BK - 1) / BK);  // per phase; the last one may be partial
  const int k_rem = static_cast<int>(K % BK);              // valid contraction indices of a partial last step
  std::vector<int> filled(A_ROWS * BK / 8 + BN * BK / 8, 0);
  for (int wave = 0; wave < WAVES; ++wave)
    for (int lane = 0; lane < 64; ++lane) {
      for (int i = 0; i < A_CHUNKS; ++i) {
        const int ci = (wave + WAVES * i) * 64 + lane;
        REQUIRE(ci < A_ROWS * BK / 8, "A stage position %d", ci);
        ++filled[ci];
        const uint32_t off = a_lane_offset<BK>(ci, last_row, lda);
        const uint32_t adj = k_rem ? kc_partial_adjust<BK>(ci, k_rem) : 0u;
        REQUIRE(adj <= off, "A adjustment %u beyond the offset %u", adj, off);
        for (int phase = 0; phase < phases; ++phase)
          for (int kt = 0; kt < num_kt; ++kt) {
            const bool part = k_rem != 0 && kt == num_kt - 1;
            // bytes from the tile's first row: the piece must lie in rows [0, nrows) and in the
            // phase's own K columns (the phases sit side by side in a row)
            const int64_t b0 = static_cast<int64_t>(phase) * K * 2 + static_cast<int64_t>(kt) * BK * 2 + off - (part ? adj : 0);
            const int64_t row = b0 / (lda * 2), col = (b0 % (lda * 2)) / 2;
            REQUIRE(row >= 0 && row < nrows, "A row %ld of %d (wave %d lane %d i %d)", (long)row, nrows, wave, lane, i);
            REQUIRE(col >= phase * K && col + 8 <= (phase + 1) * K, "A columns %ld..+8 of phase %d, K %ld", (long)col, phase, (long)K);
          }
      }
      for (int i = 0; i < B_CHUNKS; ++i) {
        const int ci = (wave + WAVES * i) * 64 + lane;
        REQUIRE(ci < BN * BK / 8, "B stage position %d", ci);
        ++filled[A_ROWS * BK / 8 + ci];
        for (int kt = 0; kt < num_kt; ++kt) {
          const bool part = k_rem != 0 && kt == num_kt - 1;
          if (kBContig) {
            // b is [N, K] (ldb elements per row): rows n0 .. N - 1, columns of K step kt
            const uint32_t off = b_contig_lane_offset<BK>(ci, n0, N, ldb);
            const uint32_t adj = part ? kc_partial_adjust<BK>(ci, k_rem) : 0u;
            REQUIRE(adj <= off, "B adjustment beyond the offset");
            const int64_t b0 = n0 * ldb * 2 + static_cast<int64_t>(kt) * BK * 2 + off - adj;
            const int64_t row = b0 / (ldb * 2), col = (b0 % (ldb * 2)) / 2;
            REQUIRE(row >= n0 && row < N, "B row %ld of [%ld, %ld)", (long)row, (long)n0, (long)N);
            REQUIRE(col + 8 <= K, "B columns %ld..+8 of %ld", (long)col, (long)K);
          } else {
            // b is [K, N]: contraction rows of K step kt, columns n0 .. N - 1
            const uint32_t off = b_major_lane_offset<BK, BW>(ci, n0, N, ldb);
            const uint32_t adj = part ? b_major_partial_adjust<BK, BW>(ci, k_rem, ldb) : 0u;
            REQUIRE(adj <= off, "B adjustment beyond the offset");
            const int64_t b0 = n0 * 2 + static_cast<int64_t>(kt) * BK * ldb * 2 + off - adj;
            const int64_t row = b0 / (ldb * 2), col = (b0 % (ldb * 2)) / 2;
            REQUIRE(row >= static_cast<int64_t>(kt) * BK && row < static_cast<int64_t>(kt + 1) * BK && row < K,
                    "B contraction row %ld in step %d of K %ld", (long)row, kt, (long)K);
            REQUIRE(col >= 0 && col + 8 <= N, "B columns %ld..+8 of %ld (n0 %ld)", (long)col, (long)N, (long)n0);
          }
        }
      }
    }
  for (size_t c = 0; c < filled.size(); ++c) REQUIRE(filled[c] == 1, "stage piece %zu written %d times", c, filled[c]);
}

// The persistent weight gradient's descriptors over one segment and one tile.
template <int TILE>
void check_wgrad(int64_t rows_total, int64_t beg, int seg_rows, int64_t ld, int64_t cols, int m0) {
  constexpr int BK = 32, WAVES = 4, CHUNKS = TILE * BK / 8 / (64 * WAVES);
  if (ld >= TILE) {  // (a narrower row does not tell a piece's row from its byte offset)
    // a K step's transfers fetch every 16-byte piece of its BK rows x TILE columns exactly once
    std::vector<int> seen(BK * (TILE / 8), 0);
    for (int wave = 0; wave < WAVES; ++wave)
      for (int c = 0; c < CHUNKS; ++c)
        for (int lane = 0; lane < 64; ++lane) {
          const uint32_t off = wgrad_lane_offset(wave, WAVES, c, lane, ld, TILE);
          const int64_t krow = off / (ld * 2), piece = off % (ld * 2) / 16;
          REQUIRE(krow < BK && piece < TILE / 8, "wgrad piece (%ld, %ld) outside the K step", (long)krow, (long)piece);
          // where the transfer puts it: lanes fill the instruction's KiB in order, which must be
          // the swizzled slot that the transposing reads expect
          const int slot = ((wave + WAVES * c) * 64 + lane);
          const int want = static_cast<int>(krow) * (TILE / 8) + (static_cast<int>(piece) ^ (4 * (static_cast<int>(krow) & 3)));
          REQUIRE(slot == want, "wgrad piece (%ld, %ld) lands in slot %d, read from %d", (long)krow, (long)piece, slot, want);
          ++seen[krow * (TILE / 8) + piece];
        }
    for (size_t i = 0; i < seen.size(); ++i) REQUIRE(seen[i] == 1, "wgrad piece %zu fetched %d times", i, seen[i]);
  }
  const int64_t operand_bytes = rows_total * ld * 2;
  int64_t base = (beg * ld + m0) * 2;  // bytes from the operand's start
  int64_t records = wgrad_num_records(seg_rows, ld, cols, m0, TILE);
  REQUIRE(records > 0 && records < (int64_t{1} << 32), "num_records %ld", (long)records);
  const int steps = (seg_rows + BK - 1) / BK;
  const int64_t seg_end_bytes = ((beg + seg_rows - 1) * ld + cols) * 2;  // end of the segment's last row
  for (int kt = 0; kt < steps; ++kt) {
    REQUIRE(records > 0, "num_records underflow at step %d of %d", kt, steps);
    REQUIRE(base + records <= operand_bytes, "descriptor ends %ld past the operand", (long)(base + records - operand_bytes));
    REQUIRE(base + records <= seg_end_bytes, "descriptor ends behind the segment's last row");
    for (int wave = 0; wave < WAVES; ++wave)
      for (int c = 0; c < CHUNKS; ++c)
        for (int lane = 0; lane < 64; ++lane) {
          const uint32_t off = wgrad_lane_offset(wave, WAVES, c, lane, ld, TILE);
          // the hardware drops what lies at or behind num_records; what it lets through
          // must be rows of this segment
          if (static_cast<int64_t>(off) + 16 <= records) {
            const int64_t b0 = base + off;
            const int64_t row = b0 / (ld * 2);
            REQUIRE(row >= beg && row < beg + seg_rows, "wgrad row %ld of [%ld, %ld)", (long)row, (long)beg,
                    (long)(beg + seg_rows));
          }
        }
    if (kt + 1 < steps) {  // the kernel's move_on
      base += static_cast<int64_t>(BK) * ld * 2;
      records -= static_cast<int64_t>(BK) * ld * 2;
    }
  }
}

int main() {
  // row-tiled configurations x (K, N, nrows, column tile origin); ragged widths and short tiles
  const int heights160[] = {1, 16, 31, 32, 33, 96, 128, 144, 159, 160};
  for (int nrows : heights160)
    for (int64_t N : {512, 520, 1000, 4096})
      for (int64_t n0 = 0; n0 < N; n0 += 512) {
        check_rows<160, 512, 32, 4, false, 1>(2048, N, 2048, N, nrows, n0, 1);          // down projection
      }
  for (int nrows : heights160)
    for (int64_t H : {256, 424, 4096})
      for (int64_t n0 = 0; n0 < H; n0 += 256)
        check_rows<160, 512, 32, 4, false, 2>(1280, H, 1280, H, nrows, n0, 1);            // up|gate, sub-tiles of 256
  const int heights320[] = {1, 16, 64, 65, 255, 256, 272, 304, 319, 320};
  for (int nrows : heights320)
    for (int64_t N : {256, 264, 2048})
      for (int64_t n0 = 0; n0 < N; n0 += 256) {
        check_rows<320, 256, 32, 4, true, 1>(4096, N, 4096, 4096, nrows, n0, 1);          // input gradient of down
        check_rows<320, 256, 32, 4, true, 1>(4096, N, 8192, 4096, nrows, n0, 2);          // fused up|gate input gradient
      }
  for (int nrows : {1, 17, 64, 100, 128})
    for (int64_t N : {256, 320, 848})
      for (int64_t n0 = 0; n0 < N; n0 += 256) {
        check_rows<128, 256, 64, 4, true, 1>(1280, N, 1280, 1280, nrows, n0, 1);
        check_rows<128, 256, 64, 4, false, 1>(1280, N, 1280, N, nrows, n0, 1);
      }
  // input gradients narrower than a column tile (h = 136 .. 248): rows of the weight tile
  // behind the last output column are re-reads of that column
  for (int nrows : {1, 100, 320})
    for (int64_t N : {136, 160, 216, 248}) {
      check_rows<320, 256, 32, 4, true, 1>(1280, N, 1280, 1280, nrows, 0, 1);
      check_rows<320, 256, 32, 4, true, 1>(424, N, 848, 424, nrows, 0, 2);   // fused, narrow model width
    }
  // contractions that end inside a K step (the production widths 424, 216, 184; the shortest ones)
  for (int64_t K : {8, 24, 40, 184, 216, 424})
    for (int nrows : {1, 100, 160}) {
      check_rows<160, 512, 32, 4, false, 1>(K, 1280, K, 1280, nrows, 0, 1);       // down projection, K = h
      check_rows<160, 512, 32, 4, false, 1>(K, 1280, K, 1280, nrows, 1024, 1);
      check_rows<320, 256, 32, 4, true, 1>(K, 1280, 2 * K, K, nrows, 1024, 2);    // fused up|gate input gradient, K = h
      check_rows<320, 256, 32, 4, true, 1>(K, 424, K, K, nrows, 256, 1);
      check_rows<128, 256, 64, 4, true, 1>(K, 320, 2 * K, K, nrows, 256, 2);
      check_rows<128, 256, 64, 4, false, 2>(K, 160, K, 160, nrows, 128, 1);
    }
  // weight gradient: segments whose length is not a multiple of the K step, operands narrower
  // than a tile, overhanging column tiles, the last segment ending with the operand
  for (int seg_rows : {1, 2, 16, 31, 32, 33, 100, 512, 530})
    for (int64_t cols : {64, 160, 216, 256, 264, 424, 2048})
      for (int64_t ld : {cols, cols + 8, 2 * cols})
      {
        for (int m0 = 0; m0 < cols; m0 += 256) {
          check_wgrad<256>(seg_rows, 0, seg_rows, ld, cols, m0);            // the operand is this segment
          check_wgrad<256>(600 + seg_rows, 600, seg_rows, ld, cols, m0);    // the last segment of a longer operand
          check_wgrad<256>(2000, 48, seg_rows, ld, cols, m0);
        }
        for (int m0 = 0; m0 < cols; m0 += 128) {                            // the 128-column tile
          check_wgrad<128>(seg_rows, 0, seg_rows, ld, cols, m0);
          check_wgrad<128>(600 + seg_rows, 600, seg_rows, ld, cols, m0);
          check_wgrad<128>(2000, 48, seg_rows, ld, cols, m0);
        }
      }
  std::printf("ok: %ld checks\n", checks);
  return 0;
}
