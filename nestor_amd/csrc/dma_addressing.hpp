// Address arithmetic of the direct-to-LDS transfers, as plain integer functions that
// compile for the host as well as for the device.  The kernels take every per-lane
// offset, every buffer-descriptor size and every LDS destination from here, and a
// host program (tests/dma_addressing_check.cpp) runs the same functions over every
// wavefront, lane, transfer and K step of ragged shapes and checks each byte range
// against the operand it must stay inside -- the check that has to pass before a
// change to this arithmetic reaches a GPU, where an address out of range is a fault.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__) || defined(__CUDACC__)
#define NESTOR_HD __host__ __device__ inline
#else
#define NESTOR_HD inline
#endif

namespace nestor {
namespace dma {

// ---- row-tiled kernels ------------------------------------------------------
// Swizzled 16-byte piece of a contraction-contiguous tile (BK elements per row) that
// position ci of the LDS stage holds: its row and its logical piece.
template <int BK>
NESTOR_HD void kc_piece_of(int ci, int& row, int& piece) {
  constexpr int cpr = BK / 8, rp = 256 / (BK * 2);
  row = ci / cpr;
  piece = (ci % cpr) ^ ((row / rp) % cpr);
}
// Byte offset (from the tile's first row, first column of the K step) of the piece an
// A transfer's lane fetches.  Rows behind last_row fetch last_row again.
template <int BK>
NESTOR_HD uint32_t a_lane_offset(int ci, int last_row, int64_t lda) {
  int row, c;
  kc_piece_of<BK>(ci, row, c);
  row = row < last_row ? row : last_row;
  return static_cast<uint32_t>((static_cast<int64_t>(row) * lda + c * 8) * 2);
}
// The same for a contraction-contiguous B tile ([N, K] weights): row = output column
// n0 + row, clamped to the operand's last column N - 1.
template <int BK>
NESTOR_HD uint32_t b_contig_lane_offset(int ci, int64_t n0, int64_t N, int64_t ldb) {
  int row, c;
  kc_piece_of<BK>(ci, row, c);
  int64_t n = n0 + row;
  n = n < N ? n : N - 1;
  return static_cast<uint32_t>(((n - n0) * ldb + c * 8) * 2);
}
// A contraction-major B tile ([K, N] weights): sub-tiles of BK rows x BW columns; piece
// ci covers contraction row k of its sub-tile and eight columns from n0 + 8 * c on,
// clamped to the operand's last eight columns.
template <int BK, int BW>
NESTOR_HD uint32_t b_major_lane_offset(int ci, int64_t n0, int64_t N, int64_t ldb) {
  constexpr int kPerSub = BK * BW / 8;
  const int cs = ci % kPerSub;
  const int k = cs / (BW / 8);
  const int c = (cs % (BW / 8)) ^ (4 * (k & 3));
  int64_t n = n0 + c * 8;
  n = n < N ? n : N - 8;
  return static_cast<uint32_t>((static_cast<int64_t>(k) * ldb + (n - n0)) * 2);
}

// ---- the last K step of a contraction that is not a multiple of BK -------------
// k_rem = K % BK valid contraction indices (a multiple of 8, > 0).  Every lane still
// fetches 16 bytes that lie inside the operand (and hold finite values): a piece
// behind k_rem is replaced by one in front of it, and what the replaced pieces feed is
// cancelled by zeroing the A fragments of those contraction indices in registers.
// Each function returns how many bytes to SUBTRACT from the regular lane offset.
template <int BK>
NESTOR_HD uint32_t kc_partial_adjust(int ci, int k_rem) {
  int row, c;
  kc_piece_of<BK>(ci, row, c);
  return c * 8 < k_rem ? 0u : static_cast<uint32_t>(c * 16);  // piece 0 of the same row
}
template <int BK, int BW>
NESTOR_HD uint32_t b_major_partial_adjust(int ci, int k_rem, int64_t ldb) {
  constexpr int kPerSub = BK * BW / 8;
  const int k = (ci % kPerSub) / (BW / 8);
  return k < k_rem ? 0u : static_cast<uint32_t>(static_cast<int64_t>(k - (k_rem - 1)) * ldb * 2);  // row k_rem - 1
}

// ---- persistent weight gradient ----------------------------------------------
// Both operands are [segment row, column] with tiles of 256 or 128 columns: one transfer
// covers two contraction rows x 32 pieces, or four x 16.
NESTOR_HD uint32_t wgrad_lane_offset(int wave, int waves, int chunk, int lane, int64_t ld,
                                     int tile_cols = 256) {
  const int ppr = tile_cols / 8;  // pieces per contraction row of the tile
  const int krow = (64 / ppr) * (wave + waves * chunk) + lane / ppr;
  const int pc = (lane % ppr) ^ (4 * (krow & 3));
  return static_cast<uint32_t>((static_cast<int64_t>(krow) * ld + pc * 8) * 2);
}
// num_records of the descriptor that starts at (segment row 0, column m0) of an
// operand with `cols` columns: whole rows up to the segment's last one, of which the
// tile's own columns (tile_cols wide, cut at the operand's width).
NESTOR_HD uint32_t wgrad_num_records(int seg_rows, int64_t ld, int64_t cols, int m0, int tile_cols) {
  const int64_t own = cols - m0 < tile_cols ? cols - m0 : tile_cols;
  return static_cast<uint32_t>((static_cast<int64_t>(seg_rows - 1) * ld + own) * 2);
}

}  // namespace dma
}  // namespace nestor
