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
//
// The residual (what a group of four holds beyond its first two kept values) for the launch that
// multiplies both parts at once: one list of 32-bit words per record, numbered like the records
// (record_index), lists stored one after the other in that order, so that the lists of a group of
// eight row blocks for one unit are neighbours, like their records.
//   word    = fp16 value | address << 16
//   address = byte address of element (row r, column c) of the record's 16 x 128 block in the dense
//             image the kernel keeps in LDS: r * 256 + (((c / 8) ^ r) << 4) + (c % 8) * 2  (the 16-byte
//             granules of a row are permuted by the row number, so that the sixteen rows' granules
//             of one column group fall into sixteen different bank groups)
//   Offsets[i] .. Offsets[i + 1] are list i's words (records + 1 entries, 32-bit).  The words of a
//   list are read 64 at a time, one per lane; they are ordered so that each such round spreads
//   over the LDS banks (words that share a bank are dealt to different rounds).  The array of
//   words is followed by 64 words of padding.
// 4 bytes per kept residual value.
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
// Residual lists of a row-major M x K matrix (the A2 of decompose; any matrix with at most 1024
// kept values per 16 x 128 block works).  *words and *offsets are malloc'ed (caller frees);
// *longest = the longest list's length.  Returns the number of offsets or a negative code.
int pack_residual(const uint16_t* A2, int M, int K, uint32_t** words, int** offsets, int* longest);
constexpr int kListPadWords = 64;
inline uint32_t residual_address(int row, int col)
{
    return static_cast<uint32_t>(row * 256 + ((((col >> 3) ^ row) & 15) << 4) + (col & 7) * 2);
}
inline long bytes(int M, int K)
{
    return static_cast<long>(M / kRows) * (K / kUnitCols) * kRecordBytes;
}

}  // namespace a24
