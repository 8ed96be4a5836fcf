// gfx950 device code for the Tiled-CSL SpMM and the only translation unit of
// the library that talks to the HIP runtime.  The host logic (spmm_api.cpp)
// reaches it through the few extern "C" tcsl_* launchers at the bottom.
//
// Replaces, with a different design, the reference's SpMM_Kernel
// (csrc/SpMM_Kernel.cuh:293-735) and SplitK_Reduction
// (csrc/Reduction_Kernel.cuh:24-47).
//
// Design: "load as sparse, compute as dense", one wavefront per work unit.
//   * A work unit is one 128-row tile row of A times one split-K batch of
//     64-column tiles.  A workgroup is a single wave64, so there is no
//     workgroup barrier anywhere: LDS operations of one wave execute in issue
//     order, which is all the scatter -> read-back -> clear chain needs.
//   * The packed (value,index) words of a tile are streamed from HBM with
//     non-temporal 128-bit buffer loads into a ring of register slots, a full
//     tile ahead of their use.  The loads are inline assembly and their
//     completion is awaited with hand-placed s_waitcnt vmcnt(N): every issue
//     puts a fixed number of loads in flight, so N is a compile-time constant
//     and the loads of the next tile stay in flight while this one is consumed.
//   * A private 16 KiB LDS tile holds the dense 128x64 fp16 image.  It is
//     cleared once; per tile the wave scatters the values with ds_write_b16 at
//     byte address 2*index (the index already carries the XOR swizzle that makes
//     the read-back conflict free), reads the tile back as MFMA operands with
//     ds_read_b128, issues v_mfma_f32_16x16x32_f16 against activation fragments
//     fetched straight from global memory (L2 resident), and then restores the
//     zeros by writing 0 to the same addresses.  On gfx950 an LDS write costs
//     about the same whatever its width, so undoing ~26 scatter instructions is
//     cheaper than re-clearing 16 KiB.
//   * TileOffsets of the unit sit in one VGPR (lane i = offset i) and are read
//     with v_readlane, so the steady-state loop performs no scalar memory reads.
//   * fp32 accumulators stay in registers over the whole batch; the epilogue
//     rounds to fp16 and stores one slab of partial sums (or C itself when
//     Split_K == 1).
//
// Rule for the asynchronous loads: the compiler does not know that the outputs of
// the load asm statements arrive later.  A slot's registers may therefore only
// become dead after a wait that covers the slot's loads -- consume() performs such
// a wait on every path -- otherwise the register allocator could hand a register
// with a load still in flight to an address computation.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <utility>

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int kTileRows = 128;  // rows of one encoded tile
constexpr int kTileCols = 64;   // columns of one encoded tile
constexpr int kTileBytes = kTileRows * kTileCols * 2;
constexpr int kWave = 64;
constexpr int kVecPerLane = 8;  // 16-byte vectors per lane and ring slot: 512 vectors, i.e. tiles up to 25 % dense in one go
constexpr int kRing = 2;        // ring slots: one tile being consumed, one in flight

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

// Four packed words -> four 16-bit LDS writes of the value (or of zero) at byte
// address 2 * (word >> 16).  One SDWA shift forms each address; all four are formed
// first so the writes issue back to back.  Addresses are absolute LDS addresses: the
// tile is the kernel's only LDS object and sits at address 0 (checked at entry).
#define TCSL_ADDR(d, s) \
    "v_lshlrev_b32_sdwa " d ", 1, " s " dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_1\n"
template<bool CLEAR>
__device__ __forceinline__ void scatter_words(u32x4 w, uint32_t zero)
{
    uint32_t a0, a1, a2, a3;
    if (!CLEAR)
        asm volatile(TCSL_ADDR("%0", "%4") TCSL_ADDR("%1", "%5") TCSL_ADDR("%2", "%6") TCSL_ADDR("%3", "%7")
                     "ds_write_b16 %0, %4\n ds_write_b16 %1, %5\n ds_write_b16 %2, %6\n ds_write_b16 %3, %7\n"
                     : "=&v"(a0), "=&v"(a1), "=&v"(a2), "=&v"(a3)
                     : "v"(w.x), "v"(w.y), "v"(w.z), "v"(w.w)
                     : "memory");
    else
        asm volatile(TCSL_ADDR("%0", "%4") TCSL_ADDR("%1", "%5") TCSL_ADDR("%2", "%6") TCSL_ADDR("%3", "%7")
                     "ds_write_b16 %0, %8\n ds_write_b16 %1, %8\n ds_write_b16 %2, %8\n ds_write_b16 %3, %8\n"
                     : "=&v"(a0), "=&v"(a1), "=&v"(a2), "=&v"(a3)
                     : "v"(w.x), "v"(w.y), "v"(w.z), "v"(w.w), "v"(zero)
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

// One work unit.  NB = number of 16-token column blocks; HALF = N is 8 (the upper
// eight columns of the single block are computed on duplicates and dropped).
template<int NB, bool HALF>
__global__ __launch_bounds__(kWave) void tcsl_spmm_kernel(const u32x4* __restrict__ items,
                                                         const int* __restrict__ offsets,
                                                         const _Float16* __restrict__ B, _Float16* __restrict__ out,
                                                         int M, int N, int K, int split_k)
{
    __shared__ __attribute__((aligned(16))) uint8_t tile[kTileBytes];
    constexpr int VPL = kVecPerLane;
    constexpr int D = kRing;
    constexpr int L = VPL + 2 * NB;     // loads per issue: VPL word loads + 2 activation loads per column block
    constexpr int kSeg = VPL * kWave;   // vectors per segment
    if (static_cast<uint32_t>(reinterpret_cast<uintptr_t>(tile)) != 0u)
        return;  // scatter_words() assumes the tile starts at LDS address 0

    const int lane = threadIdx.x;
    const int row_tiles = M / kTileRows;
    const int rt = blockIdx.x % row_tiles;
    const int batch = blockIdx.x / row_tiles;
    // split-K bookkeeping of the reference (csrc/SpMM_Kernel.cuh:312-320), clamped to the matrix
    const int nkb = K / kTileCols;
    const int avg = (nkb - 1) / split_k + 1;
    int kb0 = batch * avg;
    kb0 = kb0 < nkb ? kb0 : nkb;
    int kb1 = kb0 + avg;
    kb1 = kb1 < nkb ? kb1 : nkb;
    const int ntile = kb1 - kb0;                          // tiles of this unit
    const int* toff = offsets + (size_t)rt * nkb + kb0;   // toff[i] = first vector of tile i, toff[ntile] = end

    // Offsets window: lane l holds toff[wbase + l].
    int wbase = 0;
    int wreg = toff[lane <= ntile ? lane : ntile];
    auto tile_range = [&](int i, int& begin, int& end) {  // 0 <= i < ntile
        if (i + 1 - wbase >= kWave) {  // slide the window (units longer than 63 tiles only)
            wbase = i;
            const int idx = i + lane;
            wreg = toff[idx <= ntile ? idx : ntile];
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

    // Activations: one contiguous K vector per token.
    const _Float16* bptr[NB];
#pragma unroll
    for (int c = 0; c < NB; c++) {
        int tok = c * 16 + l15;
        if (HALF)
            tok &= 7;
        bptr[c] = B + (size_t)tok * K + (size_t)kb0 * kTileCols + q * 8;
    }
    // Per-lane byte offsets of the word loads: chunk u sits at lane*16 + u*1024 and the
    // instruction's immediate offset reaches 4095.
    const int voff_lo = lane * 16, voff_hi = lane * 16 + 4096;
    uint32_t vzero = 0;
    asm volatile("" : "+v"(vzero));  // a zero that stays in a VGPR for the clearing writes

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
    auto make_seg = [&](Cur c, Seg& s, Cur& nxt) {
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
    half8 bfrag[D][NB][2];
    Seg held[D];

    // Always exactly L loads, whatever the segment holds, so the wait counts are static.
    auto issue = [&](int slot, const Seg& s) {
        const bool live = s.tile < ntile;
        const uint64_t base = reinterpret_cast<uint64_t>(items + s.begin);
        // descriptor over exactly this segment (nothing at all past the end of the unit)
        i32x4 rs = {(int)(uint32_t)base, (int)((uint32_t)(base >> 32) & 0xffff), live ? s.n * 16 : 0, 0x00020000};
        static_for<VPL>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            if constexpr (u < 4)
                regs[slot][u] = load_words<u * 1024>(rs, voff_lo);
            else
                regs[slot][u] = load_words<(u - 4) * 1024>(rs, voff_hi);
        });
        const int bt = live ? s.tile : ntile - 1;
#pragma unroll
        for (int cb = 0; cb < NB; cb++)
#pragma unroll
            for (int k = 0; k < 2; k++)
                bfrag[slot][cb][k] = load_activations(bptr[cb] + bt * kTileCols + k * 32);
    };

    // Y = loads issued after this slot's that may stay in flight.
    auto consume = [&](int slot, const Seg& s, auto younger) {
        constexpr int Y = decltype(younger)::value;
        if (s.n == 0) {  // empty tile or past the end: only let the slot's loads land
            wait_loads<Y>();
            return;
        }
        static_for<VPL>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            if (u * kWave < s.n) {
                wait_loads<Y + (L - 1 - u)>();
                settle(regs[slot][u]);
                if ((u + 1) * kWave <= s.n)
                    scatter_words<false>(regs[slot][u], vzero);
                else if (u * kWave + lane < s.n)  // the segment's last, partial chunk
                    scatter_words<false>(regs[slot][u], vzero);
            }
        });
        wait_loads<Y>();
        if (!s.last)
            return;  // more segments of this tile follow
#pragma unroll
        for (int cb = 0; cb < NB; cb++)
#pragma unroll
            for (int k = 0; k < 2; k++)
                settle(bfrag[slot][cb][k]);
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
                        acc[cb][r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                            afrag[k][r], bfrag[slot][cb][p * kStepsPerPass + k], acc[cb][r], 0, 0, 0);
        }
        // restore the all-zero tile: undo this segment's writes, or clear everything when
        // earlier segments (whose words are gone) wrote into it as well
        if (!s.first) {
            clear_tile(tile, lane);
        } else {
            static_for<VPL>([&](auto uc) {
                constexpr int u = decltype(uc)::value;
                if (u * kWave < s.n) {
                    if ((u + 1) * kWave <= s.n)
                        scatter_words<true>(regs[slot][u], vzero);
                    else if (u * kWave + lane < s.n)
                        scatter_words<true>(regs[slot][u], vzero);
                }
            });
        }
    };

    if (ntile > 0) {
        clear_tile(tile, lane);
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
        wait_loads<0>();
    }

    // Epilogue.  acc[c][r][i] is output row r*16 + 4*q + i of this tile row for token
    // c*16 + l15; the output keeps one contiguous M vector per token.
    _Float16* obase = out + (size_t)batch * M * N + (size_t)rt * kTileRows + q * 4;
#pragma unroll
    for (int c = 0; c < NB; c++) {
        if (HALF && l15 >= 8)
            continue;
        _Float16* o = obase + (size_t)(c * 16 + l15) * M;
#pragma unroll
        for (int r = 0; r < 8; r++) {
            half4 h;
#pragma unroll
            for (int i = 0; i < 4; i++)
                h[i] = static_cast<_Float16>(acc[c][r][i]);
            *reinterpret_cast<half4*>(o + r * 16) = h;
        }
    }
}

// C[e] = fp16(sum over slabs of float(W[s][e])), 8 elements per thread.
__global__ __launch_bounds__(256) void tcsl_reduce_kernel(_Float16* __restrict__ C, const _Float16* __restrict__ W,
                                                         long mn8, long mn, int split_k)
{
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < mn8; i += (long)gridDim.x * blockDim.x) {
        float sum[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        for (int s = 0; s < split_k; s++) {
            half8 w = *reinterpret_cast<const half8*>(W + (size_t)s * mn + i * 8);
#pragma unroll
            for (int j = 0; j < 8; j++)
                sum[j] += static_cast<float>(w[j]);
        }
        half8 o;
#pragma unroll
        for (int j = 0; j < 8; j++)
            o[j] = static_cast<_Float16>(sum[j]);
        *reinterpret_cast<half8*>(C + i * 8) = o;
    }
}

// Plain streaming copy, used only to calibrate hardware counters against a
// transfer of known size.
__global__ __launch_bounds__(256) void tcsl_copy_kernel(u32x4* __restrict__ dst, const u32x4* __restrict__ src, long n16)
{
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (long)gridDim.x * blockDim.x)
        dst[i] = src[i];
}

template<int NB, bool HALF>
int launch_spmm(hipStream_t stream, const void* items, const int* offsets, const void* B, void* out, int M, int N,
                int K, int split_k)
{
    const int units = (M / kTileRows) * split_k;
    hipLaunchKernelGGL((tcsl_spmm_kernel<NB, HALF>), dim3(units), dim3(kWave), 0, stream,
                       static_cast<const u32x4*>(items), offsets, static_cast<const _Float16*>(B),
                       static_cast<_Float16*>(out), M, N, K, split_k);
    return static_cast<int>(hipGetLastError());
}

}  // namespace

// ---------------------------------------------------------------------------
// Launchers called by the host logic.  Shapes are validated by the caller; all
// pointers are device memory; everything is asynchronous on `stream`.

extern "C" int tcsl_launch_spmm(void* stream, const void* items, const int* offsets, const void* B, void* out, int M,
                                int N, int K, int split_k)
{
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (N) {
        case 8:
            return launch_spmm<1, true>(s, items, offsets, B, out, M, N, K, split_k);
        case 16:
            return launch_spmm<1, false>(s, items, offsets, B, out, M, N, K, split_k);
        case 32:
            return launch_spmm<2, false>(s, items, offsets, B, out, M, N, K, split_k);
        case 64:
            return launch_spmm<4, false>(s, items, offsets, B, out, M, N, K, split_k);
        default:
            return static_cast<int>(hipErrorInvalidValue);
    }
}

extern "C" int tcsl_launch_reduce(void* stream, void* C, const void* W, long mn, int split_k)
{
    const long mn8 = mn / 8;
    long blocks = (mn8 + 255) / 256;
    if (blocks > 4096)
        blocks = 4096;
    if (blocks < 1)
        blocks = 1;
    hipLaunchKernelGGL(tcsl_reduce_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<_Float16*>(C), static_cast<const _Float16*>(W), mn8, mn, split_k);
    return static_cast<int>(hipGetLastError());
}

extern "C" int tcsl_launch_copy(void* stream, void* dst, const void* src, long bytes)
{
    hipLaunchKernelGGL(tcsl_copy_kernel, dim3(256 * 16), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<u32x4*>(dst), static_cast<const u32x4*>(src), bytes / 16);
    return static_cast<int>(hipGetLastError());
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
