// K-tiled bf16 matrix layout shared by the row movers, the weight packer and the MFMA kernels.
//
// A matrix [rows, cols] (cols a multiple of 32, rows padded to a multiple of 16) is cut into blocks of 16 rows x
// 32 columns = 1 KiB.  Blocks are stored contiguously and ordered [column block][row block], so the 256 rows x 32
// columns a workgroup consumes per K step are ONE contiguous 16 KiB run: every global->LDS load instruction moves
// a full contiguous KiB, the access pattern the memory pipeline sustains at its highest rate.
// Inside a block, row r occupies 64 bytes and its 16-byte chunk c is stored in slot c ^ ((r >> 2) & 3): this is
// the bank swizzle the MFMA fragment reads use, so blocks are copied to LDS verbatim.
#pragma once
#include <stdint.h>

namespace wx {

constexpr int kBlkRows = 16;
constexpr int kBlkCols = 32;
constexpr int kBlkBytes = kBlkRows * kBlkCols * 2;

__host__ __device__ inline int64_t tiled_row_blocks(int64_t rows) { return (rows + kBlkRows - 1) / kBlkRows; }
__host__ __device__ inline int64_t tiled_bytes(int64_t rows, int64_t cols) {
  return tiled_row_blocks(rows) * (cols / kBlkCols) * kBlkBytes;
}

// Byte offset of the 16-byte chunk holding columns [col, col + 8) of `row` (col a multiple of 8).
__host__ __device__ inline int64_t tiled_chunk_offset(int64_t row, int64_t col, int64_t row_blocks) {
  const int64_t rb = row >> 4, kb = col >> 5;
  const int r = static_cast<int>(row & 15), c = static_cast<int>((col >> 3) & 3);
  return ((kb * row_blocks + rb) << 10) + (r << 6) + ((c ^ ((r >> 2) & 3)) << 4);
}

// Rows of the expert-sorted space as the MFMA kernels see it: each expert's rows start at a multiple of 256, so
// every 256-row tile is 16 whole row blocks of one expert.
__host__ __device__ inline int64_t round_up_256(int64_t v) { return (v + 255) / 256 * 256; }
// Upper bound of the padded row count for `rows` tokens split over two experts.
__host__ __device__ inline int64_t padded_sorted_rows(int64_t rows) { return round_up_256(rows) + 256; }

}  // namespace wx
