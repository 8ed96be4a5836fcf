// Tiled-CSL encoder on the GPU, bit-identical to the reference's host encoder
// InitSparseMatrixA_API (csrc/SpMM_API.cu:241-438) and to tiled_csl_encode.cpp.
//
// The reference simulates 32 per-bank stacks with repeated arg-max pops.  Two facts make
// the same output computable in parallel, one workgroup per 128x64 tile:
//   * row m contributes exactly one pair of adjacent columns to every bank: swizzled column
//     c ^ ((m & 7) << 3) has bank (swizzled >> 1), so bank b of row m holds swizzled
//     positions 2b and 2b+1 (csrc/SpMM_API.cu:330-334).  A bank's list is therefore the kept
//     elements among 256 candidates in a fixed order, and an element's place in it is a
//     prefix count;
//   * the pop order is "level = tallest stack down to 1, banks in id order, every bank at
//     least that tall" (the largest stack with the lowest id wins each arg-max,
//     csrc/SpMM_API.cu:223-234), and the emission order (:379-424) is index arithmetic on it.
// So every element computes its own final position.  Three kernels: count per tile, scan,
// emit.  No counterpart in the reference, which encodes on one host thread.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

constexpr int kTileRows = 128, kTileCols = 64, kBanks = 32, kThreads = 256;
constexpr int kRowsPerThread = kTileRows / (kThreads / kBanks);  // 16
constexpr int kMaxLevel = 2 * kTileRows + 4;                      // 256 per bank + up to 3 pads, rounded up

// csrc/SpMM_API.cu:262: kept when fabs(float(v)) > 0, i.e. not +-0 and not NaN
__device__ __forceinline__ bool kept(uint32_t h)
{
    const uint32_t mag = h & 0x7fffu;
    return mag != 0 && mag <= 0x7c00u;
}

// The pair of adjacent columns that row m gives to bank b, as one 32-bit load.
__device__ __forceinline__ uint32_t load_pair(const uint16_t* tile, int ld, int m, int b)
{
    const int x = b ^ ((m & 7) << 2);  // the unswizzled column pair
    return *reinterpret_cast<const uint32_t*>(tile + (size_t)m * ld + 2 * x);
}

__global__ __launch_bounds__(kThreads) void tcsl_count_tiles(const uint16_t* __restrict__ A, int K, int tiles_k,
                                                            int* __restrict__ offsets)
{
    const int t = blockIdx.x;
    const uint16_t* tile = A + (size_t)(t / tiles_k) * kTileRows * K + (size_t)(t % tiles_k) * kTileCols;
    const int b = threadIdx.x & 31, rg = threadIdx.x >> 5;
    int c = 0;
#pragma unroll
    for (int i = 0; i < kRowsPerThread; i++) {
        const uint32_t p = load_pair(tile, K, rg * kRowsPerThread + i, b);
        c += kept(p & 0xffffu) + kept(p >> 16);
    }
    __shared__ int part[kThreads / 64];
    for (int o = 32; o > 0; o >>= 1)
        c += __shfl_down(c, o);
    if ((threadIdx.x & 63) == 0)
        part[threadIdx.x >> 6] = c;
    __syncthreads();
    if (threadIdx.x == 0) {
        int nz = 0;
        for (int i = 0; i < kThreads / 64; i++)
            nz += part[i];
        offsets[t + 1] = (nz + 3) / 4;  // vectors of four words, zero padded (:289)
    }
}

// offsets[1..tiles] hold per-tile vector counts; turn them into the running total
// (offsets[0] = 0, offsets[tiles + 1] = total, :426-435).  One workgroup.  If the total does
// not fit an int, offsets[tiles + 1] is set to -1.
__global__ __launch_bounds__(1024) void tcsl_scan_offsets(int* __restrict__ offsets, long tiles)
{
    __shared__ long long sums[1024];
    const long chunk = (tiles + 1023) / 1024;
    const long lo = threadIdx.x * chunk, hi = lo + chunk < tiles ? lo + chunk : tiles;
    long long s = 0;
    for (long i = lo; i < hi; i++)
        s += offsets[i + 1];
    sums[threadIdx.x] = s;
    __syncthreads();
    for (int o = 1; o < 1024; o <<= 1) {  // inclusive scan of the chunk sums
        const long long v = threadIdx.x >= o ? sums[threadIdx.x - o] : 0;
        __syncthreads();
        sums[threadIdx.x] += v;
        __syncthreads();
    }
    long long run = threadIdx.x ? sums[threadIdx.x - 1] : 0;
    const bool fits = sums[1023] <= 0x7fffffffLL;
    for (long i = lo; i < hi; i++) {
        run += offsets[i + 1];
        offsets[i + 1] = fits ? static_cast<int>(run) : 0;
    }
    if (threadIdx.x == 0) {
        offsets[0] = 0;
        offsets[tiles + 1] = fits ? static_cast<int>(sums[1023]) : -1;
    }
}

__global__ __launch_bounds__(kThreads) void tcsl_emit_tiles(const uint16_t* __restrict__ A, int K, int tiles_k,
                                                           const int* __restrict__ offsets,
                                                           uint32_t* __restrict__ items)
{
    __shared__ uint32_t bank[kBanks][kMaxLevel];      // the per-bank lists ("stacks" of the reference)
    __shared__ int grp_count[kThreads / kBanks][kBanks];
    __shared__ int grp_zero[kThreads / kBanks][kBanks];
    __shared__ int size[kBanks];
    __shared__ uint32_t level_mask[kMaxLevel + 2];    // banks at least l tall
    __shared__ int level_first[kMaxLevel + 2];        // pops made before level l starts
    __shared__ int total_words;

    const int t = blockIdx.x;
    const int words = (offsets[t + 1] - offsets[t]) * 4;
    if (words == 0)
        return;  // an all-zero tile emits nothing (uniform for the workgroup)
    const uint16_t* tile = A + (size_t)(t / tiles_k) * kTileRows * K + (size_t)(t % tiles_k) * kTileCols;
    uint32_t* out = items + (size_t)offsets[t] * 4;
    const int b = threadIdx.x & 31, rg = threadIdx.x >> 5;

    // 1. this thread's 16 rows of bank b: count the kept elements, note the first zero position
    uint32_t pairs[kRowsPerThread];
    int c = 0, zero = -1;
#pragma unroll
    for (int i = 0; i < kRowsPerThread; i++) {
        const int m = rg * kRowsPerThread + i;
        pairs[i] = load_pair(tile, K, m, b);
        const bool k0 = kept(pairs[i] & 0xffffu), k1 = kept(pairs[i] >> 16);
        c += k0 + k1;
        if (zero < 0 && !k0)
            zero = m * kTileCols + 2 * b;       // position = row * 64 + swizzled column (:330-339)
        if (zero < 0 && !k1)
            zero = m * kTileCols + 2 * b + 1;
    }
    grp_count[rg][b] = c;
    grp_zero[rg][b] = zero;
    __syncthreads();

    // 2. place in the bank's list = kept elements of the bank in earlier rows; write the words
    int rank = 0;
    for (int g = 0; g < rg; g++)
        rank += grp_count[g][b];
#pragma unroll
    for (int i = 0; i < kRowsPerThread; i++) {
        const int m = rg * kRowsPerThread + i;
        const uint32_t lo = pairs[i] & 0xffffu, hi = pairs[i] >> 16;
        if (kept(lo))
            bank[b][rank++] = lo | (uint32_t)(m * kTileCols + 2 * b) << 16;
        if (kept(hi))
            bank[b][rank++] = hi | (uint32_t)(m * kTileCols + 2 * b + 1) << 16;
    }
    if (rg == kThreads / kBanks - 1)
        size[b] = rank;
    __syncthreads();

    // 3. zero padding to a multiple of four, each pad on the currently smallest bank (lowest id
    //    on ties), pointing at that bank's first zero position (:352-365)
    if (threadIdx.x == 0) {
        int count = 0;
        for (int i = 0; i < kBanks; i++)
            count += size[i];
        const int pad = (4 - count % 4) % 4;
        for (int p = 0; p < pad; p++) {
            int s = 0;
            for (int i = 1; i < kBanks; i++)
                if (size[i] < size[s])
                    s = i;
            int z = -1;
            for (int g = 0; g < kThreads / kBanks && z < 0; g++)
                z = grp_zero[g][s];
            bank[s][size[s]++] = (uint32_t)z << 16;
        }
        total_words = count + pad;
    }
    __syncthreads();

    // 4. pop order: level = tallest down to 1, banks by id.  level_first[l] = pops before level l.
    for (int l = threadIdx.x + 1; l <= kMaxLevel; l += kThreads) {
        uint32_t mask = 0;
        for (int i = 0; i < kBanks; i++)
            mask |= (uint32_t)(size[i] >= l) << i;
        level_mask[l] = mask;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int run = 0;
        for (int l = kMaxLevel; l >= 1; l--) {
            level_first[l] = run;
            run += __popc(level_mask[l]);
        }
    }
    __syncthreads();

    // 5. emission (:379-424): V vectors = R groups of 32 lanes + rem lanes.  The first 4*rem pops
    //    fill the tail (lane = pop % rem, slot 3 - pop / rem), the rest the main part (lane =
    //    pop' % 32, arrival kk = pop' / 32 written at reverse position 4R-1-kk).
    const int vecs = total_words / 4, R = vecs / 32, rem = vecs % 32;
    for (int j = rg; j < size[b]; j += kThreads / kBanks) {
        const int l = j + 1;
        const int pop = level_first[l] + __popc(level_mask[l] & ((1u << b) - 1u));
        int idx;
        if (pop < 4 * rem) {
            idx = R * 128 + (pop % rem) * 4 + (3 - pop / rem);
        } else {
            const int q = pop - 4 * rem, kk = q >> 5, lane = q & 31;
            const int pos = 4 * R - 1 - kk;  // = 4 * r + v
            idx = ((pos >> 2) * 32 + lane) * 4 + (pos & 3);
        }
        out[idx] = bank[b][j];
    }
}

}  // namespace

// TileOffsets (tiles + 2 ints, device memory) of the dense row-major fp16 matrix A (device memory).
extern "C" int tcsl_launch_encode_offsets(void* stream, const void* A, int M, int K, int* offsets)
{
    const long tiles_k = K / kTileCols, tiles = (long)(M / kTileRows) * tiles_k;
    if (tiles < 1 || tiles > 0x7fffffffL)
        return static_cast<int>(hipErrorInvalidValue);
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(tcsl_count_tiles, dim3((unsigned)tiles), dim3(kThreads), 0, s, static_cast<const uint16_t*>(A), K,
                       (int)tiles_k, offsets);
    hipLaunchKernelGGL(tcsl_scan_offsets, dim3(1), dim3(1024), 0, s, offsets, tiles);
    return static_cast<int>(hipGetLastError());
}

// The packed words, 4 * offsets[tiles + 1] of them, given the offsets computed above.
extern "C" int tcsl_launch_encode_items(void* stream, const void* A, int M, int K, const int* offsets, void* items)
{
    const long tiles_k = K / kTileCols, tiles = (long)(M / kTileRows) * tiles_k;
    if (tiles < 1 || tiles > 0x7fffffffL)
        return static_cast<int>(hipErrorInvalidValue);
    hipLaunchKernelGGL(tcsl_emit_tiles, dim3((unsigned)tiles), dim3(kThreads), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t*>(A), K, (int)tiles_k, offsets, static_cast<uint32_t*>(items));
    return static_cast<int>(hipGetLastError());
}
