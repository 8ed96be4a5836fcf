// Constants and small helpers of the Tiled-CSL format shared by the host code.
// The values are fixed by the reference's encoder and tile configuration
// (csrc/SpMM_API.cu:249-251, csrc/TilingConfig.h:22-29,91-95); changing any of
// them changes the on-disk and in-memory format.
#pragma once
#include <cstdint>

namespace tcsl {

constexpr int kTileRows = 128;      // rows of one encoded tile
constexpr int kTileCols = 64;       // columns of one encoded tile
constexpr int kBanks = 32;          // 4-byte LDS banks the encoder balances over
constexpr int kVec = 4;             // words per 16-byte vector; tiles are padded to it
constexpr int kGroup = 32;          // lanes per interleave group of the encoder
constexpr int kOffsetPadding = 2;   // TileOffsets holds tiles + 2 entries

// Error codes of the host entry points (all negative; the reference exits or asserts instead).
constexpr int kErrBadShape = -1;
constexpr int kErrNoMemory = -2;
constexpr int kErrNullPointer = -3;
constexpr int kErrFile = -4;
constexpr int kErrTooLarge = -5;

// word = fp16 bits | (row * 64 + (col ^ ((row % 8) << 3))) << 16   (csrc/SpMM_API.cu:336-339)
inline uint32_t pack_item(uint16_t value_bits, int position)
{
    return static_cast<uint32_t>(value_bits) | (static_cast<uint32_t>(position & 0xffff) << 16);
}

int encode(const uint16_t* A, int M, int K, uint32_t** items_out, int** offsets_out);
int encode_noreorder(const uint16_t* A, int M, int K, uint32_t** items_out, int** offsets_out);
int encode_file(const char* dense, int M, int K, const char* nz_path, const char* off_path, const char* sizes_path);

// Deterministic synthetic inputs (counter based, identical on every host).
void synth_weights(uint16_t* A, int M, int K, double sparsity, int row_skewed, uint64_t seed);
void synth_activations(uint16_t* B, long count, uint64_t seed);
// The same keep decisions with the value pattern of the reference's harness: weights 1.0, activations in {-5, -3, -1, 1, 3}.
void synth_harness_weights(uint16_t* A, int M, int K, double sparsity, int row_skewed, uint64_t seed);
void synth_harness_activations(uint16_t* B, long count, uint64_t seed);

}  // namespace tcsl
