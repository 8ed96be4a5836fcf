// Host-side Tiled-CSL encoder: dense row-major fp16 weight -> packed
// (value,index) words + TileOffsets, bit-exact with the reference's
// InitSparseMatrixA_API (csrc/SpMM_API.cu:241-438) but organised differently:
//
//   * The reference simulates 32 stacks and runs a 32-way arg-max for every
//     word it emits.  Its pop order has a closed form: with bank sizes s[b],
//     the sequence of pops is "for level = max(s) down to 1, for bank b = 0..31
//     in order, if s[b] >= level take element level-1 of bank b" (the largest
//     stack with the lowest id always wins, so equal-height stacks are drained
//     in id order, one layer at a time).  The emission order (tail drawn first,
//     main part after, both written last-in first-out) is then pure index
//     arithmetic on that sequence; see emit_tile().
//   * Tiles are independent once their output offsets are known, so the work is
//     two passes (count -> prefix sum -> encode) spread over a small thread pool
//     by tile row.  The reference is single threaded.
//
// Plain C++: no HIP here.
#include <algorithm>
#include <atomic>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <new>
#include <thread>
#include <vector>

#include "tiled_csl_format.h"

namespace tcsl {

namespace {

// The reference keeps an element when fabs(float(v)) > 0 (csrc/SpMM_API.cu:262):
// +-0 and NaN are dropped, subnormals and infinities are kept.
inline bool kept(uint16_t h)
{
    const uint16_t mag = h & 0x7fffu;
    return mag != 0 && mag <= 0x7c00u;
}

int pool_size(long work_items)
{
    int n = 0;
    if (const char* e = std::getenv("SPMM_ENCODE_THREADS"))
        n = std::atoi(e);
    if (n <= 0) {
        n = static_cast<int>(std::thread::hardware_concurrency());
        if (n <= 0)
            n = 1;
        if (n > 16)
            n = 16;
    }
    if (n > work_items)
        n = static_cast<int>(work_items);
    return n < 1 ? 1 : n;
}

// Runs fn(i) for i in [0, count) on the pool; dynamic distribution.
template<typename F>
void parallel_for(long count, F fn)
{
    const int nt = pool_size(count);
    if (nt == 1) {
        for (long i = 0; i < count; i++)
            fn(i);
        return;
    }
    std::atomic<long> next{0};
    std::vector<std::thread> pool;
    pool.reserve(nt);
    for (int t = 0; t < nt; t++)
        pool.emplace_back([&] {
            for (;;) {
                long i = next.fetch_add(1);
                if (i >= count)
                    return;
                fn(i);
            }
        });
    for (auto& th : pool)
        th.join();
}

int count_tile(const uint16_t* tile, int ld)
{
    int nz = 0;
    for (int m = 0; m < kTileRows; m++) {
        const uint16_t* row = tile + static_cast<size_t>(m) * ld;
        for (int n = 0; n < kTileCols; n++)
            nz += kept(row[n]);
    }
    return nz;
}

struct TileScratch {
    uint32_t bank[kBanks][kTileRows * kTileCols / kBanks + kVec];  // 256 positions per bank + pads
    int size[kBanks];
    uint32_t seq[kTileRows * kTileCols];  // pop sequence
};

// Encodes one tile into dst; returns the number of words written (a multiple of 4).
int emit_tile(const uint16_t* tile, int ld, uint32_t* dst, TileScratch& ws)
{
    int first_zero[kBanks];
    for (int b = 0; b < kBanks; b++) {
        ws.size[b] = 0;
        first_zero[b] = -1;
    }
    int count = 0;
    for (int m = 0; m < kTileRows; m++) {
        const uint16_t* row = tile + static_cast<size_t>(m) * ld;
        const int flip = (m & 7) << 3;
        for (int n = 0; n < kTileCols; n++) {
            const int swz = n ^ flip;          // swizzled column (csrc/SpMM_API.cu:332-333)
            const int b = (swz >> 1) & 31;     // 4-byte LDS bank of that position (:334)
            const int pos = m * kTileCols + swz;
            const uint16_t v = row[n];
            if (kept(v)) {
                ws.bank[b][ws.size[b]++] = pack_item(v, pos);
                count++;
            } else if (first_zero[b] < 0) {
                first_zero[b] = pos;
            }
        }
    }
    if (count == 0)
        return 0;
    // zero padding to a multiple of 4, each pad on the currently smallest bank (:352-365)
    const int pad = (kVec - count % kVec) % kVec;
    for (int p = 0; p < pad; p++) {
        int b = 0;
        for (int i = 1; i < kBanks; i++)
            if (ws.size[i] < ws.size[b])
                b = i;
        // the smallest bank of a tile that needs padding always has a zero position
        ws.bank[b][ws.size[b]++] = pack_item(0, first_zero[b]);
        count++;
    }
    // pop sequence, closed form
    int top = 0;
    for (int b = 0; b < kBanks; b++)
        top = std::max(top, ws.size[b]);
    int qn = 0;
    for (int level = top; level >= 1; level--)
        for (int b = 0; b < kBanks; b++)
            if (ws.size[b] >= level)
                ws.seq[qn++] = ws.bank[b][level - 1];
    // emission (:379-424).  V vectors = R full groups of 32 lanes + `rem` lanes.
    // The first 4*rem pops fill the tail, lane b receiving pops v*rem + b; the
    // rest fill the main part, lane b receiving pops 4*rem + k*32 + b, k = 0..4R-1.
    // Both are written out in reverse arrival order, main part first.
    const int vecs = count / kVec;
    const int R = vecs / kGroup, rem = vecs % kGroup;
    const uint32_t* mainq = ws.seq + kVec * rem;
    for (int r = 0; r < R; r++)
        for (int b = 0; b < kGroup; b++)
            for (int v = 0; v < kVec; v++)
                dst[(r * kGroup + b) * kVec + v] = mainq[(kVec * R - 1 - (kVec * r + v)) * kGroup + b];
    uint32_t* tail = dst + R * kGroup * kVec;
    for (int b = 0; b < rem; b++)
        for (int v = 0; v < kVec; v++)
            tail[b * kVec + v] = ws.seq[(kVec - 1 - v) * rem + b];
    return count;
}

// One tile without reordering (csrc/SpMM_API.cu:514-551): kept elements in scan order, and the
// first `pads` elements of the scan that are not kept, with whatever bits they hold.
int emit_tile_noreorder(const uint16_t* tile, int ld, uint32_t* dst, int pads)
{
    int w = 0;
    for (int m = 0; m < kTileRows; m++) {
        const uint16_t* row = tile + static_cast<size_t>(m) * ld;
        const int flip = (m & 7) << 3;
        for (int n = 0; n < kTileCols; n++) {
            const uint16_t v = row[n];
            if (kept(v)) {
                dst[w++] = pack_item(v, m * kTileCols + (n ^ flip));
            } else if (pads > 0) {
                pads--;
                dst[w++] = pack_item(v, m * kTileCols + (n ^ flip));
            }
        }
    }
    return w;
}

int encode_impl(const uint16_t* A, int M, int K, uint32_t** items_out, int** offsets_out, bool reorder);

}  // namespace

int encode(const uint16_t* A, int M, int K, uint32_t** items_out, int** offsets_out)
{
    return encode_impl(A, M, K, items_out, offsets_out, true);
}

int encode_noreorder(const uint16_t* A, int M, int K, uint32_t** items_out, int** offsets_out)
{
    return encode_impl(A, M, K, items_out, offsets_out, false);
}

namespace {

int encode_impl(const uint16_t* A, int M, int K, uint32_t** items_out, int** offsets_out, bool reorder)
{
    if (!A || !items_out || !offsets_out)
        return kErrNullPointer;
    if (M <= 0 || K <= 0 || M % kTileRows != 0 || K % kTileCols != 0)
        return kErrBadShape;
    const int tr = M / kTileRows, tc = K / kTileCols;
    const long ntiles = static_cast<long>(tr) * tc;

    int* offs = static_cast<int*>(std::malloc((ntiles + kOffsetPadding) * sizeof(int)));
    if (!offs)
        return kErrNoMemory;

    // pass 1: padded word count of every tile, stored in offs[t + 1]
    parallel_for(tr, [&](long i) {
        for (int j = 0; j < tc; j++) {
            const int nz = count_tile(A + static_cast<size_t>(i) * kTileRows * K + static_cast<size_t>(j) * kTileCols, K);
            offs[i * tc + j + 1] = (nz + kVec - 1) / kVec;
        }
    });
    offs[0] = 0;
    long total_vecs = 0;
    for (long t = 0; t < ntiles; t++) {
        total_vecs += offs[t + 1];
        if (total_vecs > INT32_MAX) {
            std::free(offs);
            return kErrTooLarge;
        }
        offs[t + 1] = static_cast<int>(total_vecs);
    }
    offs[ntiles + 1] = static_cast<int>(total_vecs);  // trailing empty tile (:433-435)

    uint32_t* items = static_cast<uint32_t*>(std::malloc(std::max<size_t>(total_vecs * kVec, 1) * sizeof(uint32_t)));
    if (!items) {
        std::free(offs);
        return kErrNoMemory;
    }

    // pass 2: every tile row into its slot
    std::atomic<bool> ok{true};
    parallel_for(tr, [&](long i) {
        TileScratch* ws = new (std::nothrow) TileScratch;
        if (!ws) {
            ok = false;
            return;
        }
        for (int j = 0; j < tc; j++) {
            const long t = i * tc + j;
            const uint16_t* tile = A + static_cast<size_t>(i) * kTileRows * K + static_cast<size_t>(j) * kTileCols;
            uint32_t* dst = items + static_cast<size_t>(offs[t]) * kVec;
            int n;
            if (reorder) {
                n = emit_tile(tile, K, dst, *ws);
            } else {
                const int nz = count_tile(tile, K);
                n = emit_tile_noreorder(tile, K, dst, (kVec - nz % kVec) % kVec);
            }
            if (n != (offs[t + 1] - offs[t]) * kVec)
                ok = false;
        }
        delete ws;
    });
    if (!ok) {
        std::free(items);
        std::free(offs);
        return kErrNoMemory;
    }
    *items_out = items;
    *offsets_out = offs;
    return static_cast<int>(ntiles + kOffsetPadding);
}

}  // namespace

int encode_file(const char* dense, int M, int K, const char* nz_path, const char* off_path, const char* sizes_path)
{
    if (!dense || !nz_path || !off_path || !sizes_path)
        return kErrNullPointer;
    if (M <= 0 || K <= 0 || M % kTileRows != 0 || K % kTileCols != 0)
        return kErrBadShape;
    const size_t bytes = static_cast<size_t>(M) * K * sizeof(uint16_t);
    std::vector<uint16_t> host(static_cast<size_t>(M) * K);
    std::ifstream in(dense, std::ios::in | std::ios::binary);
    if (!in.is_open()) {
        std::fprintf(stderr, "file %s cannot be opened, loadDataArrayFromBin fails. \n", dense);
        return kErrFile;
    }
    in.read(reinterpret_cast<char*>(host.data()), static_cast<std::streamsize>(bytes));
    const size_t got = static_cast<size_t>(in.gcount());
    if (got != bytes) {
        std::fprintf(stderr, "file %s only has %zu, but request %zu, loading DenseMatrix fails! \n", dense, got, bytes);
        return kErrFile;
    }
    in.close();

    uint32_t* items = nullptr;
    int* offs = nullptr;
    const int num_offsets = encode(host.data(), M, K, &items, &offs);
    if (num_offsets < 0)
        return num_offsets;
    const int nnz = offs[num_offsets - 1] * kVec;

    std::ofstream out_sizes(sizes_path, std::ios::out | std::ios::binary);
    std::ofstream out_nz(nz_path, std::ios::out | std::ios::binary);
    std::ofstream out_off(off_path, std::ios::out | std::ios::binary);
    int rc = 0;
    if (!out_sizes.is_open() || !out_nz.is_open() || !out_off.is_open()) {
        std::fprintf(stderr, "GenSparseMatrixBinFile() ERROR: file %s, %s, or %s cannot be opened or created. \n",
                     sizes_path, nz_path, off_path);
        rc = kErrFile;
    } else {
        // int32 NNZ then int32 NumOffsets (csrc/SpMM_API.cu:1613-1615)
        out_sizes.write(reinterpret_cast<const char*>(&nnz), sizeof(int));
        out_sizes.write(reinterpret_cast<const char*>(&num_offsets), sizeof(int));
        out_nz.write(reinterpret_cast<const char*>(items), static_cast<std::streamsize>(sizeof(uint32_t)) * nnz);
        out_off.write(reinterpret_cast<const char*>(offs), static_cast<std::streamsize>(sizeof(int)) * num_offsets);
        // a short write may only show when the buffers are flushed: close first, then look
        out_sizes.close();
        out_nz.close();
        out_off.close();
        if (out_sizes.fail() || out_nz.fail() || out_off.fail())
            rc = kErrFile;
    }
    std::free(items);
    std::free(offs);
    return rc;
}

}  // namespace tcsl
