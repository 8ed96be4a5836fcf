// gfx950 device code for the Tiled-CSL SpMM and the only translation unit of
// the library that talks to the HIP runtime.  The host logic (spmm_api.cpp)
// reaches it through the few extern "C" tcsl_* launchers at the bottom.
//
// Replaces, with a different design, the reference's SpMM_Kernel
// (csrc/SpMM_Kernel.cuh:293-735) and SplitK_Reduction
// (csrc/Reduction_Kernel.cuh:24-47).
//
// Design: "load as sparse, compute as dense", one wavefront per work unit.
//   * A work unit is one 128-row tile row of A times a run of 64-column tiles, and one
//     wave64 owns it from start to finish: LDS operations of one wave execute in issue
//     order, which is all the scatter -> read-back -> clear chain needs, so the loop has
//     no barrier.
//   * A workgroup is W such waves, in one of two layouts the host chooses between:
//       rows  (KSPLIT = false)  W consecutive tile rows of the same split-K batch; they
//             can share the batch's activation slice, staged once into LDS (BLDS);
//       runs  (KSPLIT = true)   the W contiguous runs that one tile row's batch is cut
//             into; the waves add their accumulators up in LDS at the end, so with
//             Split_K == 1 the kernel writes C itself.
//   * The packed (value,index) words of a tile are streamed from HBM with non-temporal
//     128-bit buffer loads into a ring of two register slots, a full tile ahead of their
//     use.  The loads are inline assembly and their completion is awaited with hand-placed
//     s_waitcnt vmcnt(N): every issue puts a fixed number of loads in flight, so N is a
//     compile-time constant.  A wave keeps 8 KiB of words in flight (16 KiB where at most four
//     waves work on a compute unit): more only lengthens the memory system's queues.  The
//     loop is instantiated for 2, 4, 8 and 10 vectors per lane and issue, and a run takes the
//     one that fits its tiles' size.
//   * A private 16 KiB LDS tile holds the dense 128x64 fp16 image.  It is cleared once; per
//     tile the wave scatters the values with ds_write_b16 at byte address 2*index (the index
//     already carries the XOR swizzle that makes the read-back conflict free), reads the tile
//     back as MFMA operands with ds_read_b128, issues v_mfma_f32_16x16x32_f16 against the
//     activation fragments (from the staged slice, or fetched from global memory, where they
//     are L2 resident), and then restores the zeros by writing 0 to the same addresses (kept
//     in registers: a wave is busy 0.8 to 1 us per tile, which four or five waves per compute
//     unit only just turn into more than the memory delivers, so every instruction saved
//     shows).  Undoing ~26 scatter instructions is cheaper than re-clearing 16 KiB, which costs
//     as much LDS bandwidth as reading the tile.  The words of a tile may come in any order
//     (the reference's encoder orders them to spread LDS banks, which is worth 3 % here).
//   * TileOffsets of the unit sit in one VGPR (lane i = offset i) and are read with
//     v_readlane, so the steady-state loop performs no scalar memory reads.
//   * fp32 accumulators stay in registers over the whole run; the epilogue rounds to fp16
//     once.  In the runs layout the host launches eight waves and each workgroup decides from
//     its own tile row's density how many of them stream (the plan's number on dense rows,
//     six on sparse ones); all eight share the final sum.
//   * Split_K > 1 writes slabs of partial sums; in the runs layout the last workgroup
//     to finish a tile row then adds the slabs up itself (arrival counters in a static device
//     array, slabs written through and read at system scope), otherwise a second kernel does.
//   * ROWMAJ takes B as [K][N] and writes [M][N]; strides (ldb, ldo, ldc) and a fused clamp
//     at zero serve callers that chain layers.
//
// Rule for the asynchronous loads: the compiler does not know that the outputs of
// the load asm statements arrive later.  On every path, each destination register
// of a load must therefore stay live until after a wait that covers the load:
// land() waits and then names all registers of the slot as inputs of an (empty)
// asm statement.  Without that, the register allocator could hand a register with
// a load still in flight to some other value, which the landing load would then
// overwrite.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <mutex>
#include <utility>

#include "split_k_in_launch.h"

namespace {

using inlaunch::fused_reduction_tail;
using inlaunch::load_through;
using inlaunch::store_through;

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int kTileRows = 128;  // rows of one encoded tile
constexpr int kTileCols = 64;   // columns of one encoded tile
constexpr int kTileBytes = kTileRows * kTileCols * 2;
constexpr int kWave = 64;
constexpr int kVecPerLane = 8;       // 16-byte vectors per lane and ring slot: 512 vectors, i.e. tiles up to 25 % dense in one go
// ... and for runs whose tiles are mostly larger or much smaller, picked by the run's average
// vectors per tile: 10 per lane (640 vectors, 31 % dense) from 498 up to 640, 4 (256) up to 232,
// 2 (128) up to 112.
constexpr int kVecPerLaneLong = 10, kVecPerLaneShort = 4, kVecPerLaneTiny = 2;
constexpr int kLongTileVectors = 498, kShortTileVectors = 232, kTinyTileVectors = 112;
__device__ __forceinline__ int segment_choice(int vectors, int tiles)  // 0 tiny, 1 short, 2 regular, 3 long
{
    if (tiles <= 0)
        return 2;
    if (vectors <= kTinyTileVectors * tiles)
        return 0;
    if (vectors <= kShortTileVectors * tiles)
        return 1;
    return vectors >= kLongTileVectors * tiles && vectors <= kVecPerLaneLong * kWave * tiles ? 3 : 2;
}
constexpr int kRing = 2;        // ring slots: one tile being consumed, one in flight
constexpr unsigned kMaxLdsBytes = 160 * 1024;  // LDS of one gfx950 compute unit
constexpr int kDenseTileVectors = 340;         // average vectors per tile from which a unit counts as dense (about 83 % sparsity)
constexpr int kSparseWaves = 6;                // waves that work on a sparse unit when the launch shape is adaptive

// Arrival counters of the fused split-K reduction: pages of one counter per group of output
// rows, handed out by the host (one page per caller stream, or per graph capture and stream).
// Zero when the module is loaded; the workgroup that brings a counter to Split_K sets it back to
// zero, so every call finds them at zero.  Kernels receive a page's address as an argument.
constexpr int kCounterPages = 256;
constexpr int kCountersPerPage = 4096;
static __device__ __align__(256) unsigned int tcsl_arrivals[kCounterPages][kCountersPerPage];

// Workspace of the entry point that allocates nothing (SpMM_SplitK_API_StaticWorkspace): one
// page of arrival counters, then room for the slabs of partial sums.  Every device the library
// runs on holds its own copy for as long as the process lives.  In host code the name is only a
// handle for hipGetSymbolAddress; kernels and launchers use the per-device address that call returns.
constexpr int kScratchPage = 1 << 20;  // "page number" of the scratch's own counters
constexpr size_t kScratchCounterBytes = kCountersPerPage * sizeof(unsigned int);
constexpr size_t kScratchSlabBytes = size_t(32) << 20;
static __device__ __align__(256) unsigned char scratch[kScratchCounterBytes + kScratchSlabBytes];

template<int... Is, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, Is...>, F&& f)
{
    (f(std::integral_constant<int, Is>{}), ...);
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>), fully unrolled
template<int N, typename F>
__device__ __forceinline__ void static_for(F&& f)
{
    static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F&&>(f));
}

// 16 bytes per lane through a buffer descriptor; lanes at or past the descriptor's
// size read zero and cause no memory traffic.  Non-temporal: the stream is read once.
template<int IMM>
__device__ __forceinline__ u32x4 load_words(i32x4 rsrc, int voff)
{
    u32x4 r;
    asm volatile("buffer_load_dwordx4 %0, %1, %2, 0 offen offset:%3 nt" : "=v"(r) : "v"(voff), "s"(rsrc), "n"(IMM));
    return r;
}

__device__ __forceinline__ half8 load_activations(const _Float16* p)
{
    half8 r;
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(r) : "v"(p));
    return r;
}

// One tile offset per lane, asynchronous like the loads above (to be waited for by hand).
__device__ __forceinline__ int load_offset(const int* p)
{
    int r;
    asm volatile("global_load_dword %0, %1, off" : "=v"(r) : "v"(p));
    return r;
}

// 16 bytes per lane at base + voff (uniform 64-bit base, per-lane 32-bit byte offset)
__device__ __forceinline__ half8 load_activations_at(const _Float16* base, uint32_t voff)
{
    half8 r;
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(r) : "v"(voff), "s"(base));
    return r;
}

// Wait until at most N vector-memory loads are outstanding (they complete in order).
template<int N>
__device__ __forceinline__ void wait_loads()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N < 63 ? N : 63));
}

// Ties a register to the preceding wait: later uses cannot be scheduled above it.
template<typename T>
__device__ __forceinline__ void settle(T& x)
{
    asm volatile("" : "+v"(x));
}

// A use of the register at this point and nothing else: keeps it reserved up to here
// without creating a new value (which could make the compiler copy it elsewhere).
template<typename T>
__device__ __forceinline__ void pin(const T& x)
{
    asm volatile("" ::"v"(x));
}

// Four packed words -> four 16-bit LDS writes of the value at byte address
// base + 2 * (word >> 16).  One v_mad_u32_u16 on the word's high half forms each address;
// all four are formed first so the writes issue back to back.  The addresses are kept for
// clear_words, which writes zero to them after the tile has been multiplied.
#define TCSL_ADDR(d, s) "v_mad_u32_u16 " d ", " s ", %9, %8 op_sel:[1,0,0,0]\n"
__device__ __forceinline__ void scatter_words_keep(u32x4 w, uint32_t base, uint32_t two, uint32_t (&a)[4])
{
    asm volatile(TCSL_ADDR("%0", "%4") TCSL_ADDR("%1", "%5") TCSL_ADDR("%2", "%6") TCSL_ADDR("%3", "%7")
                 "ds_write_b16 %0, %4\n ds_write_b16 %1, %5\n ds_write_b16 %2, %6\n ds_write_b16 %3, %7\n"
                 : "=&v"(a[0]), "=&v"(a[1]), "=&v"(a[2]), "=&v"(a[3])
                 : "v"(w.x), "v"(w.y), "v"(w.z), "v"(w.w), "v"(base), "v"(two)
                 : "memory");
}
__device__ __forceinline__ void clear_words(const uint32_t (&a)[4], uint32_t zero)
{
    asm volatile("ds_write_b16 %0, %4\n ds_write_b16 %1, %4\n ds_write_b16 %2, %4\n ds_write_b16 %3, %4\n"
                 :
                 : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(zero)
                 : "memory");
}
#undef TCSL_ADDR

__device__ __forceinline__ void clear_tile(uint8_t* tile, int lane)
{
    typedef uint64_t __attribute__((may_alias)) u64_a;
#pragma unroll
    for (int u = 0; u < kTileBytes / (kWave * 8); u++)
        *reinterpret_cast<u64_a*>(tile + u * (kWave * 8) + lane * 8) = 0;
}

// ldb = elements between two tokens' vectors in B, ldo = the same for the output (column-major
// only; the slabs of partial sums use M); relu != 0 clamps the output at zero (final results only).
// arrivals != nullptr (KSPLIT, Split_K > 1): `out` receives the slabs of partial sums
// as usual, and the last workgroup to finish a tile row adds the slabs up into fused_out (token
// stride ldc, clamped if relu) itself; arrivals are counted in arrivals[blockIdx.x] (device memory,
// zero before the launch and after it).  The row-sharing layout always leaves the sum to the
// reduction kernel (one workgroup would be left with W x 128 rows of every slab: measured slower).
// blockDim.x = W * 64, grid = (groups of tile rows, Split_K).  Wave w of workgroup (g, b) owns
// tile row g * W + w of batch b; with KSPLIT the workgroup owns tile row g and its waves share
// the batch.  avg = tiles per batch = ceil((K / 64) / Split_K).  NB = number of 16-token column blocks;
// ROWMAJ = B is [K][N] and the output [M][N].  HALF = N is 8 (the upper eight columns of the single block are computed on duplicates
// and dropped); BLDS = the batch's activation slice is staged in LDS; MAXW bounds W and
// with it the registers a wave may use.
// BSW > 0 (row-sharing layout, 32 or 64 tokens): the W = BSW waves of the workgroup walk their tile
// rows in step and share each 64-column activation tile through LDS: every wave fetches its
// 1/BSW of the tile's tokens with full-line loads (together with its own words of that tile,
// two tiles ahead), writes it into one of two tile buffers, and after one barrier per tile all
// read their MFMA operands from there.  That cuts the activation bytes a compute unit pulls
// through its vector memory path by BSW, which is what bounds 32 and 64 tokens otherwise (the
// fragments of one tile are 4 or 8 KiB against 6.5 KiB of weight words, and they cost about half
// as much per byte although they come from the L2).
// Dynamic LDS: W tiles of 16 KiB, then tokens * 128 bytes times tiles_per_batch (BLDS), times W
// (ROWMAJ) or times two (BSW); with KSPLIT at least 8 * W * NB KiB in all (the waves' accumulators meet there).
template<int NB, bool HALF, bool BLDS, bool KSPLIT, bool ROWMAJ, int MAXW, int BSW = 0>
__global__ __launch_bounds__(MAXW* kWave) void tcsl_spmm_kernel(const int* __restrict__ offsets,
                                                                const u32x4* __restrict__ items,
                                                                const _Float16* __restrict__ B,
                                                                _Float16* __restrict__ out, int K, int avg,
                                                                int wave_counts, int ldb, int M, int ldo,
                                                                _Float16* __restrict__ fused_out,
                                                                unsigned int* __restrict__ arrivals, int ldc,
                                                                int relu, int split_k)
{
    // (Argument order: the first 14 dwords are preloaded into scalar registers when a wave starts
    // (-amdgpu-kernarg-preload-count); they are what the way to the first tile's loads needs.
    // wave_counts = W | dense_waves << 8, W = waves per workgroup = blockDim.x / 64, passed so
    // that it is among them; the number of tokens is the template's.)
    const int W = wave_counts & 0xff, dense_waves = wave_counts >> 8;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int D = kRing;
    constexpr int NTOK = HALF ? 8 : NB * 16;      // tokens
    // activation loads per issue: two fragments per column block, or (ROWMAJ) the tile's
    // 64 x N block as 1 KiB pieces, or (BSW) this wave's share of the tile's tokens, eight
    // tokens' 128-byte lines per load
    constexpr int kShareTokens = BSW > 0 ? NTOK / BSW : 0;  // tokens this wave fetches per tile
    constexpr int BL = BLDS ? 0 : BSW > 0 ? (kShareTokens + 7) / 8 : (ROWMAJ ? NTOK / 8 : 2 * NB);

    static_assert(!(KSPLIT && BLDS), "a workgroup that splits K shares no activation slice");
    static_assert(!(ROWMAJ && BLDS), "row-major activations are not staged");
    static_assert(BSW == 0 || (!KSPLIT && !BLDS && !ROWMAJ && !HALF && NB >= 2 && NTOK % BSW == 0 && BSW <= MAXW),
                  "activation tiles are streamed through LDS in the row-sharing layout only");

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // uniform, and known to be
    // grid: x = group of tile rows (one tile row in the K-splitting layout), y = split-K batch
    const int row_tiles = M / kTileRows;
    const int batch = blockIdx.y;
    const int rt = KSPLIT ? blockIdx.x : blockIdx.x * W + wave;
    const bool active = rt < row_tiles;
    // split-K bookkeeping of the reference (csrc/SpMM_Kernel.cuh:312-320), clamped to the matrix;
    // avg = ceil((K / 64) / split_k), from the host
    const int nkb = K / kTileCols;
    int kb0 = batch * avg;
    kb0 = kb0 < nkb ? kb0 : nkb;
    int kb1 = kb0 + avg;
    kb1 = kb1 < nkb ? kb1 : nkb;
    int Wk = W;    // waves that work in a K-splitting workgroup
    int segments = 2;  // segment_choice of this run
    int wreg = 0;  // offsets window: lane l holds the offset of tile wbase + l of this wave's run
    bool cleared = false;
    uint8_t* const tile = lds + wave * kTileBytes;
    if (KSPLIT) {
        const int n = kb1 - kb0;
        const int* u = offsets + (size_t)rt * nkb;  // this tile row's offsets
        // The batch's tiles are dealt to the working waves in contiguous runs.  (Dealing them
        // round robin, so that the workgroup reads one contiguous stretch at a time, measured
        // slower.)  Waves 4.. share a SIMD with waves 0..3 and issue behind them (the older wave
        // wins the arbitration; per-wave time stamps show the fifth wave of five about 10 %
        // slower per tile and the first unaffected), so their runs are 7/8 as long: with
        // share(w) = 8 w for w <= 4, 32 + 7 (w - 4) above, wave w's run starts at tile
        // round(n share(w) / share(waves)).  The quotient is taken in floating point; x + 1/2 is
        // never within 1 / (2 * 60) of a multiple of the divisor, far more than the error (and
        // beyond 2^24 / 60 tiles per batch, where it is not, neighbours still compute the same cuts).
        auto run = [&](int waves, int& b0, int& b1) {
            const int shares = waves <= 4 ? 8 * waves : 4 + 7 * waves;
            const float inv = __builtin_amdgcn_rcpf(static_cast<float>(shares));
            auto cut = [&](int w) {  // cut(0) = 0, cut(waves) = n whatever the rounding does
                const int x = n * (w <= 4 ? 8 * w : 4 + 7 * w) + shares / 2;
                const int c = static_cast<int>((static_cast<float>(x) + 0.5f) * inv);
                return w >= waves ? n : (c < n ? c : n);
            };
            b0 = kb0 + cut(wave);
            b1 = kb0 + cut(wave + 1);
        };
        // The host launches eight waves and says how many of them dense tiles want; sparse tiles
        // want kSparseWaves (small tiles: a wave's turnaround per tile, not the memory system, is
        // the limit, so more waves help, up to a point); the unit's own density decides.  The
        // others stream nothing and wait at the barrier of the final sum, of which they take
        // their share.  The offsets windows of both
        // outcomes travel with the two offsets that give the density, so the decision costs no
        // memory round trip of its own.  (All four loads are issued on every path, adaptive or
        // not, and waited for in one place: a value that is still on its way must not meet
        // another at a join, where the compiler would copy it.)
        const bool adaptive = dense_waves > 0 && dense_waves < W && n > 0;
        const int sparse_waves = adaptive && W > kSparseWaves ? kSparseWaves : W;
        int b0 = kb0, b1 = kb0;
        if (wave < sparse_waves)
            run(sparse_waves, b0, b1);
        Wk = sparse_waves;
        int d0 = kb0, d1 = kb0;
        if (adaptive && wave < dense_waves)
            run(dense_waves, d0, d1);
        int wd = load_offset(u + (d0 + lane <= d1 ? d0 + lane : d1));
        wreg = load_offset(u + (b0 + lane <= b1 ? b0 + lane : b1));
        int e0 = load_offset(u + kb0), e1 = load_offset(u + kb1);
        clear_tile(tile, lane);
        cleared = true;
        // (the arguments that are not preloaded are fetched while the offsets are on their way)
        asm volatile("" ::"s"(relu), "s"(arrivals), "s"(ldc), "s"(split_k), "s"(fused_out));
        wait_loads<0>();
        settle(wd);
        settle(wreg);
        settle(e0);
        settle(e1);
        const int unit_vectors = __builtin_amdgcn_readfirstlane(e1 - e0);
        segments = segment_choice(unit_vectors, n);
        if (adaptive && unit_vectors >= kDenseTileVectors * n) {
            Wk = dense_waves;
            b0 = d0;
            b1 = d1;
            wreg = wd;
        }
        kb0 = b0;
        kb1 = b1;
    }
    // tiles of this wave (BSW: a wave past the last tile row walks along with empty tiles, for its
    // share of the activation tiles and for the barriers)
    const int ntile = active || BSW > 0 ? kb1 - kb0 : 0;
    // Activations in LDS, per tile [token][8 granules of 16 B at position g ^ (token & 7)]: the
    // batch's slice, staged once and shared (BLDS), or (ROWMAJ) a one-tile buffer per wave in
    // which the tile's k-major block is turned into token-major MFMA operands.
    uint8_t* const bslice = lds + W * kTileBytes + (ROWMAJ ? wave * (NTOK * 128) : 0);

    // Offsets window: lane l holds toff[wbase + l]; toff[i] = first vector of tile i,
    // toff[ntile] = end.  Issued first so its latency overlaps the staging below.
    const int* toff = offsets + (size_t)(active ? rt : 0) * nkb + kb0;
    int wbase = 0;
    if (!KSPLIT)
        wreg = active ? toff[lane <= ntile ? lane : ntile] : 0;

    if (BLDS) {
        const int ngran = (kb1 - kb0) * NTOK * 8;  // the whole batch, whatever this wave's own share
        for (int id = threadIdx.x; id < ngran; id += W * kWave) {
            const int j = id / (NTOK * 8), t = (id >> 3) % NTOK, g = id & 7;
            const half8 v = *reinterpret_cast<const half8*>(B + (size_t)t * ldb + (size_t)(kb0 + j) * kTileCols + g * 8);
            *reinterpret_cast<half8*>(bslice + (size_t)j * (NTOK * 128) + t * 128 + ((g ^ (t & 7)) << 4)) = v;
        }
    }
    if (active && !cleared)
        clear_tile(tile, lane);
    if (BLDS)
        __syncthreads();  // the only barrier: every wave of the workgroup reaches it
    if (!KSPLIT && !active && BSW == 0)
        return;
    const bool clamp = relu && !(KSPLIT && arrivals);  // partial sums are never clamped

    auto tile_range = [&](int i, int& begin, int& end) __attribute__((always_inline)) {  // 0 <= i < ntile
        if (i + 1 - wbase >= kWave) {  // slide the window (more than 63 tiles per wave only)
            wbase = i;
            const int idx = i + lane;
            wreg = active ? toff[idx <= ntile ? idx : ntile] : 0;
            settle(wreg);  // makes the compiler wait for this load here, on the rare path, not at the join below
        }
        begin = __builtin_amdgcn_readlane(wreg, i - wbase);
        end = __builtin_amdgcn_readlane(wreg, i + 1 - wbase);
    };

    f32x4 acc[NB][8];
#pragma unroll
    for (int c = 0; c < NB; c++)
#pragma unroll
        for (int r = 0; r < 8; r++)
            acc[c][r] = f32x4{0.f, 0.f, 0.f, 0.f};

    // MFMA operand geometry (v_mfma_f32_16x16x32_f16): lane l supplies row (l & 15) of a
    // 16-row weight block and column (l & 15) of a 16-token activation block, both for the
    // eight k values 8*(l >> 4) .. +7 of the 32-wide step.
    const int l15 = lane & 15, q = lane >> 4;
    // LDS byte offset of this lane's 16-byte granule for k-step s in row block 0; row blocks
    // are 16 rows * 128 B apart.  Granule g of row r sits at position g ^ (r & 7) (the
    // encoder's swizzle, csrc/SpMM_API.cu:330-339), and (r & 7) == (lane & 7).
    int a_off[2];
#pragma unroll
    for (int s = 0; s < 2; s++)
        a_off[s] = l15 * 128 + (((s * 4 + q) ^ (lane & 7)) << 4);

    // Activations: one contiguous K vector per token in global memory; in the staged
    // slice the same granule swizzle as the weight tile keeps the reads conflict free.
    const _Float16* bptr[NB];
    int b_off[NB][2];
#pragma unroll
    for (int c = 0; c < NB; c++) {
        int tok = c * 16 + l15;
        if (HALF)
            tok &= 7;
        bptr[c] = ROWMAJ ? B : B + (size_t)tok * ldb + (size_t)kb0 * kTileCols + q * 8;
#pragma unroll
        for (int s = 0; s < 2; s++)
            b_off[c][s] = tok * 128 + (((s * 4 + q) ^ (tok & 7)) << 4);
    }
    // ROWMAJ: the tile's 64 x N block sits in the wave's buffer as it sits in memory, row k at
    // byte k * 2 N (with 64 tokens the four 32-byte column chunks of a row are permuted by
    // (k >> 1) & 3, so that the four rows one transposing read touches fall into different
    // banks).  ds_read_b64_tr_b16 hands lane i of a group of sixteen the i-th column of a 4 x 16
    // block whose rows the sixteen lanes address four to a row: lane j points at row j / 4,
    // columns 4 (j % 4) .. + 3.  Two such reads give a lane its eight consecutive k of one token.
    auto rowmaj_byte = [](int k, int n) {
        return NTOK == 64 ? k * 128 + ((((n >> 4) ^ (k >> 1)) & 3) << 5) + (n & 15) * 2 : (k * NTOK + n) * 2;
    };
    int tr_off[NB][2][2];
    if (ROWMAJ) {
#pragma unroll
        for (int c = 0; c < NB; c++)
#pragma unroll
            for (int s = 0; s < 2; s++)
#pragma unroll
                for (int hh = 0; hh < 2; hh++)
                    tr_off[c][s][hh] = rowmaj_byte(32 * s + 8 * q + 4 * hh + (l15 >> 2), (16 * c + 4 * (l15 & 3)) % NTOK);
    }
    // BSW: load i of this wave's share of a tile covers tokens share0 + 8 i + (lane >> 3), lane & 7
    // being the 16-byte granule of the token's 128-byte line; lanes beyond the share (a share of
    // four tokens fills half a load) repeat a token and write nothing.
    const _Float16* sh_ptr[BL > 0 ? BL : 1];
    int sh_off[BL > 0 ? BL : 1];
    bool sh_ok[BL > 0 ? BL : 1];
    if (BSW > 0) {
#pragma unroll
        for (int i = 0; i < BL; i++) {
            const int t = 8 * i + (lane >> 3);
            sh_ok[i] = t < kShareTokens;
            const int tok = wave * kShareTokens + t % (kShareTokens > 0 ? kShareTokens : 1);
            sh_ptr[i] = B + (size_t)tok * ldb + (size_t)kb0 * kTileCols + (lane & 7) * 8;
            sh_off[i] = tok * 128 + (((lane & 7) ^ (tok & 7)) << 4);
        }
    }
    // Per-lane byte offsets of the word loads: chunk u sits at lane*16 + u*1024 and the
    // instruction's immediate offset reaches 4095.
    const int voff_lo = lane * 16, voff_hi = lane * 16 + 4096, voff_top = lane * 16 + 8192;
    // constants the scatter asm wants in VGPRs
    uint32_t vzero = 0, vtwo = 2, vbase = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(tile));
    asm volatile("" : "+v"(vzero), "+v"(vtwo), "+v"(vbase));

    // Everything from here to the end of the run is written once for any number VPL of 16-byte
    // vectors per lane and segment (ring slot), and instantiated for four: kVecPerLane (8: tiles
    // up to 25 % dense in one segment), kVecPerLaneLong (10), kVecPerLaneShort (4) and
    // kVecPerLaneTiny (2).  A tile that does not fit one segment costs a full clear of the image
    // instead of an un-scatter, about 14 % of the time per tile; ten vectors per lane cost 1.3 %
    // on tiles that fit eight; and every issue is VPL load instructions however little a tile
    // holds, which on small tiles (90 % sparsity and up) is 5 to 14 % of the time.  So a
    // workgroup (or, in the row-sharing layout, a wave) picks by its own run's density
    // (`segments`, set where the density is read).
    auto stream_run = [&](auto vpl_c) __attribute__((always_inline)) {
        constexpr int VPL = decltype(vpl_c)::value;
        constexpr int L = VPL + BL;        // loads per issue: word loads (+ activation loads)
        constexpr int kSeg = VPL * kWave;  // vectors per segment
        // Vectors a wave may have in flight.  One regular segment's worth (8 KiB): beyond that the
        // memory system only queues (about 4 % slower on a 165 MB stream at 80 % sparsity with
        // five and more waves per compute unit, where two tiles would be 13 KiB).  Two segments'
        // worth where at most four waves work on a compute unit (one per SIMD: fewer requesters,
        // -0.7 %), except at N = 64.  Two small tiles together (90 % sparsity and up) may always
        // both be in flight, or a wave's 3 KiB at a time would leave it latency bound.
        const int flight = (NB <= 2 && (KSPLIT ? Wk : W) <= 4 ? 2 : 1) * kVecPerLane * kWave;
        // The unit's stream is cut into segments of up to kSeg vectors that never cross a tile:
        // a tile of n vectors is ceil(n / kSeg) segments, an empty tile one empty segment.
        struct Seg {
            int tile;     // index within the unit; ntile = past the end
            int begin;    // first vector, absolute
            int n;        // vectors in this segment
            bool first;   // first segment of its tile
            bool last;    // last segment of its tile
        };
        struct Cur {
            int tile, off;
        };
        auto make_seg = [&](Cur c, Seg& s, Cur& nxt) __attribute__((always_inline)) {
            if (c.tile >= ntile) {
                s = Seg{ntile, 0, 0, true, true};
                nxt = c;
                return;
            }
            int b, e;
            tile_range(c.tile, b, e);
            const int rest = e - b - c.off;
            s.tile = c.tile;
            s.begin = b + c.off;
            s.n = rest < kSeg ? rest : kSeg;
            s.first = c.off == 0;
            s.last = rest <= kSeg;
            nxt = s.last ? Cur{c.tile + 1, 0} : Cur{c.tile, c.off + kSeg};
        };

        u32x4 regs[D][VPL];
        half8 bfrag[D][BL > 0 ? BL : 1];  // only used when the activations come from global memory
        Seg held[D] = {};

        // Always exactly L loads, whatever the segment holds, so the wait counts are static.
        auto issue = [&](int slot, const Seg& s) __attribute__((always_inline)) {
            if (held[slot ^ 1].n + s.n > flight)
                wait_loads<0>();
            const bool live = s.tile < ntile;
            const uint64_t base = reinterpret_cast<uint64_t>(items + s.begin);
            // descriptor over exactly this segment (nothing at all past the end of the unit)
            i32x4 rs = {(int)(uint32_t)base, (int)((uint32_t)(base >> 32) & 0xffff), live ? s.n * 16 : 0, 0x00020000};
            // Activation loads go first: they hit in L2 and return quickly, and loads return in order,
            // so behind the weight loads they would hold their slots for a full HBM round trip (1-3 %).
            if (!BLDS) {
                const int bt = live ? s.tile : ntile - 1;
                if (BSW > 0) {
    #pragma unroll
                    for (int h = 0; h < BL; h++)
                        bfrag[slot][h] = load_activations(sh_ptr[h] + bt * kTileCols);
                } else if (ROWMAJ) {
                    // B[k][n]: the tile's 64 x N block is contiguous; piece h = bytes [1024 h, 1024 h + 1024)
                    const _Float16* blk = B + (size_t)(kb0 + bt) * (kTileCols * NTOK);
    #pragma unroll
                    for (int h = 0; h < BL; h++)
                        bfrag[slot][h] = load_activations_at(blk + h * 512, lane * 16);
                } else {
    #pragma unroll
                    for (int cb = 0; cb < NB; cb++)
    #pragma unroll
                        for (int k = 0; k < 2; k++)
                            bfrag[slot][cb * 2 + k] = load_activations(bptr[cb] + bt * kTileCols + k * 32);
                }
            }
            static_for<VPL>([&](auto uc) {
                constexpr int u = decltype(uc)::value;
                if constexpr (u < 4)
                    regs[slot][u] = load_words<u * 1024>(rs, voff_lo);
                else if constexpr (u < 8)
                    regs[slot][u] = load_words<(u - 4) * 1024>(rs, voff_hi);
                else
                    regs[slot][u] = load_words<(u - 8) * 1024>(rs, voff_top);
            });
        };

        // Waits for every load of `slot` (at most Y younger ones may stay in flight) and keeps the
        // slot's registers live up to that point, so none of them can be reused while a load into
        // it is still on its way.
        auto land = [&](int slot, auto younger) __attribute__((always_inline)) {
            constexpr int Y = decltype(younger)::value;
            wait_loads<Y>();
            static_for<VPL>([&](auto uc) { pin(regs[slot][decltype(uc)::value]); });
            if (!BLDS) {
    #pragma unroll
                for (int h = 0; h < BL; h++)
                    settle(bfrag[slot][h]);
            }
        };

        // Y = loads issued after this slot's that may stay in flight.  The slot's loads were issued
        // a whole tile ago, so waiting for all of them up front costs nothing in steady state and
        // keeps one unconditional wait on every path through the loop.
        auto consume = [&](int slot, const Seg& s, auto younger) __attribute__((always_inline)) {
            land(slot, younger);
            if (BSW > 0 && s.tile < ntile) {
                // This wave's share of the tile's activations goes into the tile's buffer with the
                // tile's first segment; one barrier per tile, ahead of its last segment (every tile
                // has one, an empty tile too: the other waves count on it).  Before the barrier every
                // wave has written its share and has finished reading the previous tile's activations
                // from the other buffer, so after it this tile's buffer is complete and the other one
                // may be written for the next tile.
                if (s.first) {
    #pragma unroll
                    for (int h = 0; h < BL; h++)
                        if (sh_ok[h])
                            *reinterpret_cast<half8*>(bslice + (s.tile & 1) * (NTOK * 128) + sh_off[h]) = bfrag[slot][h];
                }
                if (s.last)
                    __syncthreads();
            }
            if (s.n == 0)
                return;  // empty tile or past the end
            uint32_t kept[VPL][4];  // the scatter's LDS addresses, for the un-scatter
            // One code path per number of full 64-vector chunks (a uniform switch): those run
            // unguarded, the one partial chunk under a lane mask, the rest not at all.  (A lane mask
            // per chunk costs a compare and three scalar instructions each, twice per tile.)
            const int full = s.n >> 6;
            const bool in_part = (full << 6) + lane < s.n;  // this lane's vector of the partial chunk exists
            auto by_chunks = [&](auto&& op) {
                auto run = [&](auto pc) {
                    constexpr int P = decltype(pc)::value;
                    static_for<P>([&](auto uc) { op(uc); });
                    if constexpr (P < VPL) {
                        if (in_part)
                            op(pc);
                    }
                };
                bool done = false;
                static_for<VPL + 1>([&](auto pc) {
                    if (!done && full == decltype(pc)::value) {
                        run(pc);
                        done = true;
                    }
                });
            };
            by_chunks([&](auto uc) {
                constexpr int u = decltype(uc)::value;
                scatter_words_keep(regs[slot][u], vbase, vtwo, kept[u]);
            });
            if (!s.last)
                return;  // more segments of this tile follow
            half8 bf[NB][2];
            if (BLDS || ROWMAJ || BSW > 0) {
                const uint8_t* bt = bslice + (BLDS ? (size_t)s.tile * (NTOK * 128) : BSW > 0 ? (s.tile & 1) * (NTOK * 128) : 0);
                if (ROWMAJ) {
                    // lane l of piece h holds tokens n0 .. n0+7 of row k, (k, n0) = divmod(512 h + 8 l, N)
    #pragma unroll
                    for (int h = 0; h < BL; h++) {
                        const int e0 = h * 512 + lane * 8;
                        *reinterpret_cast<half8*>(bslice + rowmaj_byte(e0 / NTOK, e0 % NTOK)) = bfrag[slot][h];
                    }
                    asm volatile("" ::: "memory");  // other lanes' reads below come after these writes
                    typedef short short4v __attribute__((ext_vector_type(4)));
                    typedef short short8v __attribute__((ext_vector_type(8)));
                    typedef __attribute__((address_space(3))) short4v lds_short4v;
    #pragma unroll
                    for (int cb = 0; cb < NB; cb++)
    #pragma unroll
                        for (int k = 0; k < 2; k++) {
                            const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4v*)(bt + tr_off[cb][k][0]));
                            const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4v*)(bt + tr_off[cb][k][1]));
                            const short8v both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                            bf[cb][k] = __builtin_bit_cast(half8, both);
                        }
                } else {
    #pragma unroll
                    for (int cb = 0; cb < NB; cb++)
    #pragma unroll
                        for (int k = 0; k < 2; k++)
                            bf[cb][k] = *reinterpret_cast<const half8*>(bt + b_off[cb][k]);
                }
            } else {
    #pragma unroll
                for (int cb = 0; cb < NB; cb++)
    #pragma unroll
                    for (int k = 0; k < 2; k++)
                        bf[cb][k] = bfrag[slot][cb * 2 + k];
            }
            // read the dense tile back and multiply; all reads of a pass are issued before its MFMAs
            constexpr int kPasses = NB == 1 ? 1 : 2;
            constexpr int kStepsPerPass = 2 / kPasses;
    #pragma unroll
            for (int p = 0; p < kPasses; p++) {
                half8 afrag[kStepsPerPass][8];
    #pragma unroll
                for (int k = 0; k < kStepsPerPass; k++)
    #pragma unroll
                    for (int r = 0; r < 8; r++)
                        afrag[k][r] = *reinterpret_cast<const half8*>(tile + a_off[p * kStepsPerPass + k] + r * 2048);
                __builtin_amdgcn_sched_barrier(0);
    #pragma unroll
                for (int k = 0; k < kStepsPerPass; k++)
    #pragma unroll
                    for (int r = 0; r < 8; r++)
    #pragma unroll
                        for (int cb = 0; cb < NB; cb++)
                            acc[cb][r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(afrag[k][r], bf[cb][p * kStepsPerPass + k],
                                                                                acc[cb][r], 0, 0, 0);
            }
            // restore the all-zero tile: undo this segment's writes, or clear everything when
            // earlier segments (whose words are gone) wrote into it as well
            if (!s.first) {
                clear_tile(tile, lane);
            } else {
                by_chunks([&](auto uc) {
                    constexpr int u = decltype(uc)::value;
                    clear_words(kept[u], vzero);
                });
            }
        };

        if (ntile > 0) {
            Cur ci{0, 0};
    #pragma unroll
            for (int s = 0; s < D; s++) {
                Cur nx;
                make_seg(ci, held[s], nx);
                ci = nx;
                issue(s, held[s]);
            }
            for (;;) {
    #pragma unroll
                for (int s = 0; s < D; s++) {
                    consume(s, held[s], std::integral_constant<int, (D - 1) * L>{});
                    Cur nx;
                    make_seg(ci, held[s], nx);
                    ci = nx;
                    issue(s, held[s]);
                }
                if (held[0].tile >= ntile)
                    break;  // every later slot is past the end as well
            }
            // the loads of the last (empty) issues are still in flight: let them land while their
            // destination registers are still reserved
    #pragma unroll
            for (int s = 0; s < D; s++)
                land(s, std::integral_constant<int, 0>{});
        }

    };
    if (!KSPLIT && ntile > 0) {
        // a wave of the row-sharing layout owns its run alone and judges it by its offsets window
        const int nw = ntile < kWave - 1 ? ntile : kWave - 1;
        const int run_vectors = __builtin_amdgcn_readlane(wreg, nw) - __builtin_amdgcn_readlane(wreg, 0);
        segments = segment_choice(run_vectors, nw);
    }
    if (segments == 3)
        stream_run(std::integral_constant<int, kVecPerLaneLong>{});
    else if (segments == 1)
        stream_run(std::integral_constant<int, kVecPerLaneShort>{});
    else if (segments == 0)
        stream_run(std::integral_constant<int, kVecPerLaneTiny>{});
    else
        stream_run(std::integral_constant<int, kVecPerLane>{});

    auto write_out = [&]() {
    // Epilogue.  acc[c][r][i] is output row r*16 + 4*q + i of this tile row for token
    // c*16 + l15; the output keeps one contiguous M vector per token.  The block goes through
    // the wave's LDS tile as [token][128 rows] (token stride padded to 272 B) so that the
    // global stores are 16 bytes per lane with 16 lanes covering a token's 256 bytes.
    // column-major: C[token][M], this wave's 128 rows start at rt * 128 of every token's vector;
    // row-major: C[M][N], this wave's rows are one contiguous block of 128 * N values
    _Float16* oslab = out + (size_t)batch * M * NTOK + (size_t)rt * kTileRows * (ROWMAJ ? NTOK : 1);
    if (KSPLIT) {
        // Sum the working waves' accumulators through LDS, in wave order.  Each parks its own in
        // its own tile, [row block r][column block c][lane] x 16 bytes (two tiles' worth at
        // N = 64, which then takes a barrier before as well); every launched wave w, working or
        // not, then owns the (r, c) cells w, w + W, ...  The sum is specialised by the number of
        // working waves: a vector instruction takes four cycles, so selects or a loop would cost
        // more than the additions themselves.
        constexpr int kCells = 8 * NB;
        constexpr bool kOwnTile = kCells * kWave * 16 <= kTileBytes;
        f32x4* const red = reinterpret_cast<f32x4*>(lds);
        const int wave_stride = kOwnTile ? kTileBytes / 16 : kCells * kWave;  // in f32x4
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // this wave's last clearing writes
        if (!kOwnTile)
            __syncthreads();                                  // every wave is done with its tile
        if (wave < Wk) {
#pragma unroll
            for (int r = 0; r < 8; r++)
#pragma unroll
                for (int c = 0; c < NB; c++)
                    red[wave * wave_stride + (r * NB + c) * kWave + lane] = acc[c][r];
        }
        __syncthreads();
        for (int cell = wave; cell < kCells; cell += W) {
            const int r = cell / NB, c = cell % NB;
            const f32x4* const src = red + cell * kWave + lane;
            f32x4 sum = src[0];
            static_for<MAXW - 1>([&](auto wc) {
                constexpr int WK = decltype(wc)::value + 2;  // 2 .. MAXW working waves
                if (Wk == WK) {
                    f32x4 part[WK];
#pragma unroll
                    for (int w = 1; w < WK; w++)
                        part[w] = src[w * wave_stride];
#pragma unroll
                    for (int w = 1; w < WK; w++)
#pragma unroll
                        for (int i = 0; i < 4; i++)
                            sum[i] += part[w][i];
                }
            });
            half4 h;
#pragma unroll
            for (int i = 0; i < 4; i++)
                h[i] = static_cast<_Float16>(clamp ? fmaxf(sum[i], 0.f) : sum[i]);
            // rows r*16 + 4*q .. +3 of token c*16 + l15
            if (!(HALF && l15 >= 8)) {
                if (ROWMAJ) {
#pragma unroll
                    for (int i = 0; i < 4; i++) {  // the 16 tokens of a row are adjacent
                        _Float16* dst = oslab + (r * 16 + q * 4 + i) * NTOK + c * 16 + l15;
                        if (arrivals)
                            store_through(dst, h[i]);
                        else
                            *dst = h[i];
                    }
                } else {  // the four q-lanes of a token cover 32 bytes
                    _Float16* dst = oslab + (size_t)(c * 16 + l15) * ldo + r * 16 + q * 4;
                    if (arrivals)
                        store_through(dst, h);
                    else
                        *reinterpret_cast<half4*>(dst) = h;
                }
            }
        }
        return;
    }
    if (ROWMAJ) {
        // the wave's 128 x N block through its LDS tile in memory order, then 16 bytes per lane
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the last tile's clearing writes
        if (!(HALF && l15 >= 8)) {
#pragma unroll
            for (int c = 0; c < NB; c++)
#pragma unroll
                for (int r = 0; r < 8; r++)
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        *reinterpret_cast<_Float16*>(tile + ((r * 16 + q * 4 + i) * NTOK + c * 16 + l15) * 2) =
                            static_cast<_Float16>(clamp ? fmaxf(acc[c][r][i], 0.f) : acc[c][r][i]);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // other lanes read what this lane wrote
#pragma unroll
        for (int i = 0; i < kTileRows * NTOK * 2 / (kWave * 16); i++) {
            const half8 v = *reinterpret_cast<const half8*>(tile + (i * kWave + lane) * 16);
            *reinterpret_cast<half8*>(oslab + (i * kWave + lane) * 8) = v;
        }
        return;
    }
    constexpr int kTokStride = 272;
    constexpr int kTok = HALF ? 8 : 16;
#pragma unroll
    for (int c = 0; c < NB; c++) {
        // the clearing writes of the last tile (inline asm, unknown to the compiler's own
        // LDS bookkeeping) and the previous block's reads must be done before the tile is reused
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (!(HALF && l15 >= 8)) {
#pragma unroll
            for (int r = 0; r < 8; r++) {
                half4 h;
#pragma unroll
                for (int i = 0; i < 4; i++)
                    h[i] = static_cast<_Float16>(clamp ? fmaxf(acc[c][r][i], 0.f) : acc[c][r][i]);
                *reinterpret_cast<half4*>(tile + l15 * kTokStride + (r * 16 + q * 4) * 2) = h;
            }
        }
        // other lanes read what this lane wrote: the compiler must not move the reads above
        // the writes (it reasons per lane), and the writes must have landed
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int i = 0; i < kTok / 4; i++) {
            const int e = i * kWave + lane;
            const int tok = e >> 4, part = e & 15;
            const half8 v = *reinterpret_cast<const half8*>(tile + tok * kTokStride + part * 16);
            *reinterpret_cast<half8*>(oslab + (size_t)(c * 16 + tok) * ldo + part * 8) = v;
        }
    }
    };
    if (KSPLIT || active)
        write_out();
    if (!KSPLIT || !arrivals)
        return;
    fused_reduction_tail(out, fused_out, M, NTOK, ldc, split_k, relu, blockIdx.x * kTileRows, kTileRows,
                         arrivals + blockIdx.x, reinterpret_cast<unsigned int*>(lds), W * kWave, ROWMAJ);
}

// C[n][m] = fp16(sum over slabs of float(W[s][n][m])) (csrc/Reduction_Kernel.cuh:36-46), 8 elements
// per thread; rows8 = vector length / 8, ldc = elements between two vectors of C (slabs are
// dense).  The slab loads of a thread are independent; they are issued eight at a time so
// their latencies overlap (the reduction is latency bound: a few MB in all).
__global__ __launch_bounds__(64) void tcsl_reduce_kernel(_Float16* __restrict__ C, const _Float16* __restrict__ W,
                                                        long mn8, long mn, int rows8, long ldc, int split_k, int relu)
{
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= mn8)
        return;
    const _Float16* w0 = W + i * 8;
    float sum[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    int s = 0;
    for (; s + 8 <= split_k; s += 8) {
        half8 w[8];
#pragma unroll
        for (int u = 0; u < 8; u++)
            w[u] = __builtin_nontemporal_load(reinterpret_cast<const half8*>(w0 + (size_t)(s + u) * mn));
#pragma unroll
        for (int u = 0; u < 8; u++)  // summed in slab order, as the reference does
#pragma unroll
            for (int j = 0; j < 8; j++)
                sum[j] += static_cast<float>(w[u][j]);
    }
    for (; s < split_k; s++) {
        const half8 w = __builtin_nontemporal_load(reinterpret_cast<const half8*>(w0 + (size_t)s * mn));
#pragma unroll
        for (int j = 0; j < 8; j++)
            sum[j] += static_cast<float>(w[j]);
    }
    half8 o;
#pragma unroll
    for (int j = 0; j < 8; j++)
        o[j] = static_cast<_Float16>(relu ? fmaxf(sum[j], 0.f) : sum[j]);
    const long n = i / rows8, m8 = i - n * rows8;
    *reinterpret_cast<half8*>(C + n * ldc + m8 * 8) = o;
}

// Plain streaming copy, used only to calibrate hardware counters against a
// transfer of known size.
__global__ __launch_bounds__(256) void tcsl_copy_kernel(u32x4* __restrict__ dst, const u32x4* __restrict__ src, long n16)
{
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (long)gridDim.x * blockDim.x)
        dst[i] = src[i];
}

// Device addresses of the two static arrays above on the current device.  A __device__ array's
// name in host code is a handle, not an address, and every device holds its own copy: the
// address is asked for once per device (with that device current) and kept.
struct DeviceArrays {
    unsigned int* arrivals;      // tcsl_arrivals
    unsigned char* scratch;      // scratch
};
constexpr int kMaxDevices = 64;
int device_arrays(DeviceArrays* out)
{
    static std::mutex mu;
    static DeviceArrays table[kMaxDevices];
    static std::atomic<bool> known[kMaxDevices];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess)
        return static_cast<int>(e);
    if (dev < 0 || dev >= kMaxDevices)
        return static_cast<int>(hipErrorInvalidDevice);
    if (!known[dev].load(std::memory_order_acquire)) {
        std::lock_guard<std::mutex> lock(mu);
        if (!known[dev].load(std::memory_order_relaxed)) {
            DeviceArrays a{nullptr, nullptr};
            if ((e = hipGetSymbolAddress(reinterpret_cast<void**>(&a.arrivals), HIP_SYMBOL(tcsl_arrivals))) != hipSuccess)
                return static_cast<int>(e);
            if ((e = hipGetSymbolAddress(reinterpret_cast<void**>(&a.scratch), HIP_SYMBOL(scratch))) != hipSuccess)
                return static_cast<int>(e);
            if (!a.arrivals || !a.scratch)
                return static_cast<int>(hipErrorInvalidSymbol);
            table[dev] = a;
            known[dev].store(true, std::memory_order_release);
        }
    }
    *out = table[dev];
    return 0;
}

template<int NB, bool HALF, bool BLDS, bool KSPLIT, bool ROWMAJ, int MAXW, int BSW = 0>
int launch_spmm(hipStream_t stream, const void* items, const int* offsets, const void* B, void* out, int M, int N,
                int K, int split_k, int waves, unsigned lds_bytes, int ldb, int ldo, int relu, void* fused_out,
                int ldc, unsigned int* arrivals, int dense_waves)
{
    if (waves < 1 || waves > MAXW || lds_bytes > kMaxLdsBytes)
        return static_cast<int>(hipErrorInvalidValue);
    if (BSW > 0 && waves != BSW)
        return static_cast<int>(hipErrorInvalidValue);
    auto kernel = tcsl_spmm_kernel<NB, HALF, BLDS, KSPLIT, ROWMAJ, MAXW, BSW>;
    // more than 64 KiB of dynamic LDS has to be allowed once per kernel (per device, re-armed lazily)
    static std::atomic<int> armed_device{-1};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess)
        return static_cast<int>(e);
    if (armed_device.load(std::memory_order_acquire) != dev) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                kMaxLdsBytes);
        if (e != hipSuccess)
            return static_cast<int>(e);
        armed_device.store(dev, std::memory_order_release);
    }
    const int row_tiles = M / kTileRows;
    const int groups = KSPLIT ? row_tiles : (row_tiles + waves - 1) / waves;
    const int nkb = K / kTileCols;
    if (split_k > 65535)
        return static_cast<int>(hipErrorInvalidValue);
    hipLaunchKernelGGL(kernel, dim3(groups, split_k), dim3(waves * kWave), lds_bytes, stream,
                       offsets, static_cast<const u32x4*>(items), static_cast<const _Float16*>(B),
                       static_cast<_Float16*>(out), K, (nkb - 1) / split_k + 1, waves | dense_waves << 8, ldb, M, ldo,
                       static_cast<_Float16*>(fused_out), arrivals, ldc, relu, split_k);
    return static_cast<int>(hipGetLastError());
}

}  // namespace

// ---------------------------------------------------------------------------
// Launchers called by the host logic.  Shapes are validated by the caller; all
// pointers are device memory; everything is asynchronous on `stream`.

// mode 0: the W waves of a workgroup take W consecutive tile rows of one batch; with stage_b = 1
//         (N <= 16) they share the batch's activation slice, staged once in LDS; with stage_b = 2
//         (N = 32: 4 or 8 waves, N = 64: 4 waves) they walk the batch in step and share each
//         activation tile through LDS;
// mode 1: the W waves of a workgroup split the batch of one tile row among themselves and
//         add their results up in LDS (stage_b must be 0).
// row_major: B is [K][N] and the output [M][N] instead of [N][K] and [N][M] (stage_b must be 0).
// waves = 1..8 for N <= 32, 1..4 for N = 64; lds_bytes = what the shape needs (the host plans it).
// ldb, ldo: token strides of B and of the output in elements (column-major; multiples of 8).
// fuse_page >= 0: out = Split_K dense slabs, and the kernel itself reduces them into fused_out
// (token stride ldc), counting arrivals on that page of counters (0 .. 255: the library's pages;
// kScratchPage: the counters of the static workspace); at most 4096 row groups.
// relu: bit 0 clamps final results at zero; with fuse_page >= 0, bits 8 and up = number of further
// slabs behind the Split_K of this launch that the fused reduction adds as well.
// dense_waves (mode 1; 0 = off): of the `waves` launched, only this many work on a unit whose
// tiles average 340 vectors or more (six on sparser units); the kernel looks at each unit's own offsets.
extern "C" int tcsl_launch_spmm(void* stream, const void* items, const int* offsets, const void* B, void* out, int M,
                                int N, int K, int split_k, int mode, int waves, int stage_b, int row_major,
                                unsigned lds_bytes, int ldb, int ldo, int relu, void* fused_out, int ldc,
                                int fuse_page, int dense_waves)
{
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (mode != 0 && mode != 1)
        return static_cast<int>(hipErrorInvalidValue);
    if (stage_b == 1 && (mode == 1 || row_major || N > 16))
        return static_cast<int>(hipErrorInvalidValue);
    if (stage_b == 2 && (mode == 1 || row_major || !((N == 32 && (waves == 4 || waves == 8)) || (N == 64 && waves == 4))))
        return static_cast<int>(hipErrorInvalidValue);
    if (stage_b < 0 || stage_b > 2)
        return static_cast<int>(hipErrorInvalidValue);
    unsigned int* arrivals = nullptr;
    if (fuse_page >= 0) {
        const long groups = mode ? M / kTileRows : (M / kTileRows + waves - 1) / waves;
        if ((fuse_page >= kCounterPages && fuse_page != kScratchPage) || groups > kCountersPerPage || mode != 1 || M % 8 != 0 ||
            split_k + (relu >> 8) < 2 || !fused_out)
            return static_cast<int>(hipErrorInvalidValue);
        DeviceArrays a;
        if (const int rc = device_arrays(&a))
            return rc;
        arrivals = fuse_page == kScratchPage ? reinterpret_cast<unsigned int*>(a.scratch)
                                             : a.arrivals + static_cast<size_t>(fuse_page) * kCountersPerPage;
    }
#define TCSL_GO(NB, HALF, BLDS, KS, RM, MAXW, ...) \
    launch_spmm<NB, HALF, BLDS, KS, RM, MAXW, ##__VA_ARGS__>(s, items, offsets, B, out, M, N, K, split_k, waves, lds_bytes, ldb, ldo, relu, \
                                              fused_out, ldc, arrivals, dense_waves)
#define TCSL_PICK(NB, HALF, MAXW)                                                                     \
    (row_major ? (mode ? TCSL_GO(NB, HALF, false, true, true, MAXW) : TCSL_GO(NB, HALF, false, false, true, MAXW)) \
               : (mode ? TCSL_GO(NB, HALF, false, true, false, MAXW) : TCSL_GO(NB, HALF, false, false, false, MAXW)))
    switch (N) {
        case 8:
            return stage_b ? TCSL_GO(1, true, true, false, false, 8) : TCSL_PICK(1, true, 8);
        case 16:
            return stage_b ? TCSL_GO(1, false, true, false, false, 8) : TCSL_PICK(1, false, 8);
        case 32:
            if (stage_b == 2)
                return waves == 8 ? TCSL_GO(2, false, false, false, false, 8, 8) : TCSL_GO(2, false, false, false, false, 8, 4);
            return TCSL_PICK(2, false, 8);
        case 64:
            if (stage_b == 2)
                return TCSL_GO(4, false, false, false, false, 4, 4);
            return TCSL_PICK(4, false, 4);
        default:
            return static_cast<int>(hipErrorInvalidValue);
    }
#undef TCSL_PICK
#undef TCSL_GO
}

// C[n*ldc + m] = sum over slabs of W[s][n*rows + m], n < vectors, m < rows (rows % 8 == 0, ldc % 8 == 0)
extern "C" int tcsl_launch_reduce(void* stream, void* C, const void* W, long rows, long vectors, long ldc, int split_k,
                                  int relu)
{
    const long mn = rows * vectors;
    const long mn8 = mn / 8;
    const long blocks = (mn8 + 63) / 64;
    if (blocks < 1 || blocks > 0x7fffffffL || rows / 8 > 0x7fffffffL)
        return static_cast<int>(hipErrorInvalidValue);
    hipLaunchKernelGGL(tcsl_reduce_kernel, dim3((unsigned)blocks), dim3(64), 0, static_cast<hipStream_t>(stream),
                       static_cast<_Float16*>(C), static_cast<const _Float16*>(W), mn8, mn, static_cast<int>(rows / 8),
                       ldc, split_k, relu);
    return static_cast<int>(hipGetLastError());
}

extern "C" int tcsl_launch_copy(void* stream, void* dst, const void* src, long bytes)
{
    hipLaunchKernelGGL(tcsl_copy_kernel, dim3(256 * 16), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<u32x4*>(dst), static_cast<const u32x4*>(src), bytes / 16);
    return static_cast<int>(hipGetLastError());
}

// Address of page `page` (0 .. 255) of the arrival counters on the current device, for the other
// kernels of the library that sum their split-K slabs inside the launch.
extern "C" int tcsl_counter_page_address(int page, unsigned int** address)
{
    if (page < 0 || page >= kCounterPages || !address)
        return static_cast<int>(hipErrorInvalidValue);
    DeviceArrays a;
    if (const int rc = device_arrays(&a))
        return rc;
    *address = a.arrivals + static_cast<size_t>(page) * kCountersPerPage;
    return 0;
}

// The slab part of the static workspace on the current device: its address and size in bytes.
// Asks the runtime for the array's address on the first call on a device; allocates nothing.
extern "C" int tcsl_static_workspace(void** slabs, long* bytes)
{
    DeviceArrays a;
    if (const int rc = device_arrays(&a))
        return rc;
    *slabs = a.scratch + kScratchCounterBytes;
    *bytes = static_cast<long>(kScratchSlabBytes);
    return 0;
}

// 1 and *id = the capture's id while `stream` is recording into a graph, 0 while it is not,
// -1 when the runtime cannot say (treated by the caller like a capture it knows nothing about).
extern "C" int tcsl_stream_capture(void* stream, unsigned long long* id)
{
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    unsigned long long cid = 0;
    if (hipStreamGetCaptureInfo(static_cast<hipStream_t>(stream), &st, &cid) != hipSuccess) {
        (void)hipGetLastError();
        return -1;
    }
    if (st == hipStreamCaptureStatusNone)
        return 0;
    if (st != hipStreamCaptureStatusActive)
        return -1;
    *id = cid;
    return 1;
}

// Events behind the launches that count on a recycled counter page (the host's page table says
// which pages those are): one event per page, made on first use, asked when the page is wanted
// for another stream.  Only ever called with the page table's lock held.
namespace {
constexpr int kGuardedPages = 64;
struct PageGuard {
    hipEvent_t event;
    int device;
};
PageGuard page_guards[kGuardedPages] = {};
}  // namespace

// Makes sure `page` has an event on the current device; 0 or a hipError_t value.
extern "C" int tcsl_page_prepare(int page)
{
    if (page < 0 || page >= kGuardedPages)
        return static_cast<int>(hipErrorInvalidValue);
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess)
        return static_cast<int>(e);
    PageGuard& g = page_guards[page];
    if (g.event && g.device == dev)
        return 0;
    if (g.event) {  // the page moved to a stream of another device (its last launch there has finished)
        (void)hipEventDestroy(g.event);
        g.event = nullptr;
    }
    if ((e = hipEventCreateWithFlags(&g.event, hipEventDisableTiming)) != hipSuccess) {
        g.event = nullptr;
        (void)hipGetLastError();
        return static_cast<int>(e);
    }
    g.device = dev;
    return 0;
}

// Records the page's event behind what `stream` holds so far.
extern "C" int tcsl_page_mark(int page, void* stream)
{
    if (page < 0 || page >= kGuardedPages || !page_guards[page].event)
        return static_cast<int>(hipErrorInvalidValue);
    return static_cast<int>(hipEventRecord(page_guards[page].event, static_cast<hipStream_t>(stream)));
}

// 1 when the last launch marked on the page has finished (or none ever was), 0 while it has not
// or the runtime cannot say.
extern "C" int tcsl_page_idle(int page)
{
    if (page < 0 || page >= kGuardedPages)
        return 0;
    if (!page_guards[page].event)
        return 1;
    // Asking an event is a call that the runtime forbids while any thread records a graph in the
    // global capture mode (it would invalidate that capture), unless the asking thread's own mode
    // is the relaxed one: switch to it for the one call.
    hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
    if (hipThreadExchangeStreamCaptureMode(&mode) != hipSuccess) {
        (void)hipGetLastError();
        return 0;  // cannot ask safely: the page counts as busy
    }
    const hipError_t e = hipEventQuery(page_guards[page].event);
    if (e != hipSuccess)
        (void)hipGetLastError();
    (void)hipThreadExchangeStreamCaptureMode(&mode);  // back to what it was
    return e == hipSuccess ? 1 : 0;
}

// Timing events for benchmarks (the host logic never includes HIP headers).
extern "C" void* tcsl_event_create(void)
{
    hipEvent_t e = nullptr;
    return hipEventCreate(&e) == hipSuccess ? static_cast<void*>(e) : nullptr;
}

extern "C" void tcsl_event_destroy(void* e)
{
    if (e)
        (void)hipEventDestroy(static_cast<hipEvent_t>(e));
}

extern "C" int tcsl_event_record(void* e, void* stream)
{
    return static_cast<int>(hipEventRecord(static_cast<hipEvent_t>(e), static_cast<hipStream_t>(stream)));
}

// Waits for `stop`, then returns stop - start in milliseconds (negative on error).
extern "C" float tcsl_event_elapsed_ms(void* start, void* stop)
{
    float ms = -1.f;
    if (hipEventSynchronize(static_cast<hipEvent_t>(stop)) != hipSuccess)
        return -1.f;
    if (hipEventElapsedTime(&ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)) != hipSuccess)
        return -1.f;
    return ms;
}

extern "C" const char* tcsl_error_string(int code)
{
    return hipGetErrorString(static_cast<hipError_t>(code));
}

extern "C" int tcsl_error_unknown(void)
{
    return static_cast<int>(hipErrorUnknown);
}

extern "C" int tcsl_error_invalid_value(void)
{
    return static_cast<int>(hipErrorInvalidValue);
}
