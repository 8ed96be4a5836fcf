// The 2:4 record layout that the sparse-MFMA kernel streams, and the host functions that make it.
//
// The reference splits a weight into a part with at most two kept values in every group of four
// (for NVIDIA's sparse tensor cores) and a residual that stays in Tiled-CSL
// (kernel_benchmark/spmm_decompose.h:12-51); its own device form of the first part
// (csrc/SpMM_API.cu:1127-1553: InitSparseMatrixA1_Vec_Sparse_Load, inspect_metadata) follows
// mma.sp's operand and metadata order.  Here the first part is stored in the operand order of
// gfx950's v_smfmac_f32_16x16x32_f16, so that a wave loads its registers straight from memory:
//
//   record = 16 rows x 128 columns, 2304 bytes.  Records are ordered by group of eight 16-row blocks
//   (128 rows), then by 128-column unit, then by block within the group: the eight records that a
//   128-row workgroup needs for one unit are 18 KiB of contiguous memory, and its units follow one
//   another (measured: 7 to 17 % faster than one stream per 16-row block).  The record of block rb
//   and unit u is number ((rb / 8) * (K / 128) + u) * 8 + rb % 8.
//   For lane L in 0..63 (row L % 16 of the block, column group g = L / 16), step s in 0..3 (one
//   sparse MFMA, 32 columns) and slot j in 0..3:
//     value  fp16 at byte (s / 2) * 1024 + L * 16 + ((s % 2) * 4 + j) * 2
//     column s * 32 + g * 8 + (j / 2) * 4 + q of the unit, q = the 2-bit field at bit 8 * s + 2 * j
//            of the 32-bit word at byte 2048 + L * 4 (byte s of that word is the index operand the
//            instruction selects with ABID = s).
//   Slots 0,1 serve the first group of four of the lane's eight columns, slots 2,3 the second; the
//   two positions of a group are different and ascending.  A group with fewer than two kept values
//   is filled with zero values at free positions.
//   1.125 bytes per dense element whatever the sparsity.
#pragma once
#include <cstdint>

namespace a24 {

constexpr int kRows = 16;          // rows of one record
constexpr int kGroupBlocks = 8;    // 16-row blocks whose records of one unit are stored together
constexpr int kUnitCols = 128;     // columns of one record
constexpr int kRecordBytes = 2304; // 2048 bytes of values + 256 bytes of positions
constexpr int kIndexOffset = 2048;

constexpr int kErrBadShape = -1;
constexpr int kErrNoMemory = -2;
constexpr int kErrNullPointer = -3;
constexpr int kErrNotTwoOfFour = -6;  // a group of four holds more than two kept values

// kernel_benchmark/spmm_decompose.h:12-51, bit for bit (without its printed statistics).
void decompose(const uint16_t* A, uint16_t* A1, uint16_t* A2, long length);
// Packs a row-major M x K matrix with at most two kept values per group of four into records.
// M % 128 == 0, K % 128 == 0; packed must hold bytes(M, K).  Returns 0 or a negative code.
int pack(const uint16_t* A1, int M, int K, uint8_t* packed);
inline long record_index(long row_block, int unit, int units)
{
    return ((row_block / kGroupBlocks) * units + unit) * kGroupBlocks + row_block % kGroupBlocks;
}
inline long bytes(int M, int K)
{
    return static_cast<long>(M / kRows) * (K / kUnitCols) * kRecordBytes;
}

}  // namespace a24
