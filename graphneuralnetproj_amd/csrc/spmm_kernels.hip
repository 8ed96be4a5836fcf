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
//     64-column tiles.  A workgroup is a single wave64, so no workgroup
//     barrier exists anywhere: LDS operations of one wave execute in issue
//     order, which is all the zero-fill -> scatter -> read-back chain needs.
//   * Per 128x64 tile the wave streams the tile's packed (value,index) words
//     from HBM with 128-bit buffer loads into registers (one tile ahead of
//     use), clears a private 16 KiB LDS tile, scatters the fp16 values with
//     ds_write_b16 at byte address 2*index (the index already carries the
//     XOR swizzle that makes the read-back conflict free), reads the dense
//     tile back as MFMA operands with ds_read_b128 and issues
//     v_mfma_f32_16x16x32_f16 against the activation fragments, which come
//     straight from global memory (they are L2 resident).
//   * fp32 accumulators stay in registers over the whole batch; the epilogue
//     rounds to fp16 and stores one slab of partial sums (or C itself when
//     Split_K == 1).
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 __attribute__((may_alias)) u32x4_a;
typedef uint16_t __attribute__((may_alias)) u16_a;

constexpr int kTileRows = 128;                      // rows of one encoded tile
constexpr int kTileCols = 64;                       // columns of one encoded tile
constexpr int kTileBytes = kTileRows * kTileCols * 2;
constexpr int kWave = 64;

// Packed words of one tile, register resident: VPL 16-byte vectors per lane.
template<int VPL>
struct TileRegs {
    u32x4 v[VPL];
};

// Issue the loads of one segment: up to VPL*64 consecutive vectors of one tile,
// starting `rel` vectors into the unit's slice, of which `n` (> 0) belong to the
// tile.  Always exactly VPL loads per lane, whatever n is, so that the
// compiler's vmcnt bookkeeping is exact and the loads of the following segment
// can stay in flight while this one is consumed.  Lanes past the end re-read the
// last vector (scattering it twice is idempotent, and it is only scattered for
// chunks that hold at least one real vector).  With the null descriptor nothing
// is fetched at all.
template<int VPL>
__device__ __forceinline__ void load_segment(TileRegs<VPL>& r, __amdgpu_buffer_rsrc_t rsrc, int rel, int n, int lane)
{
    const int last = rel + (n > 0 ? n - 1 : 0);
#pragma unroll
    for (int u = 0; u < VPL; u++) {
        int v = rel + u * kWave + lane;
        v = v < last ? v : last;
        r.v[u] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, v * 16, 0, 0);
    }
}

__device__ __forceinline__ void scatter_vec(uint8_t* tile, u32x4 w)
{
    // word = fp16 value | index << 16; byte address in the tile = 2 * index.
    // The mask keeps a corrupt index inside the tile.
#pragma unroll
    for (int e = 0; e < 4; e++) {
        uint32_t it = w[e];
        *reinterpret_cast<u16_a*>(tile + ((it >> 15) & (kTileBytes - 2))) = static_cast<uint16_t>(it);
    }
}

// One work unit.  NB = number of 16-token column blocks (N = 8 uses one block
// with the upper 8 tokens masked to zero).
template<int NB, int VPL>
__global__ __launch_bounds__(kWave) void tcsl_spmm_kernel(const u32x4* __restrict__ items,
                                                         const int* __restrict__ offsets,
                                                         const _Float16* __restrict__ B, _Float16* __restrict__ out,
                                                         int M, int N, int K, int split_k)
{
    __shared__ __attribute__((aligned(16))) uint8_t tile[kTileBytes];

    const int lane = threadIdx.x;
    const int row_tiles = M / kTileRows;
    const int rt = blockIdx.x % row_tiles;
    const int batch = blockIdx.x / row_tiles;
    const int nkb = K / kTileCols;
    const int avg = (nkb - 1) / split_k + 1;
    int kb0 = batch * avg;
    kb0 = kb0 < nkb ? kb0 : nkb;
    int kb1 = kb0 + avg;
    kb1 = kb1 < nkb ? kb1 : nkb;

    const int* toff = offsets + (size_t)rt * nkb;  // offsets of this tile row, in vectors
    const int unit_begin = toff[kb0];
    const int unit_end = toff[kb1];
    // Buffer descriptors cover this unit's slice only (see issue()): offsets stay
    // below 4 GiB whatever the matrix size, and reads past the slice return zero.

    f32x4 acc[NB][8];
#pragma unroll
    for (int c = 0; c < NB; c++)
#pragma unroll
        for (int r = 0; r < 8; r++)
            acc[c][r] = f32x4{0.f, 0.f, 0.f, 0.f};

    // MFMA operand geometry (v_mfma_f32_16x16x32_f16): lane l supplies row
    // (l & 15) of the weight block and column (l & 15) of the activation
    // block, both for the eight k values 8*(l >> 4) .. +7 of the 32-wide step.
    const int l15 = lane & 15, q = lane >> 4;
    // LDS byte offset of this lane's 16-byte granule for k-step s in row block 0;
    // row blocks are 16 rows * 128 B = 2048 B apart.  Granule g of row r sits at
    // position g ^ (r & 7) (the encoder's swizzle), and (r & 7) == (lane & 7).
    int a_off[2];
#pragma unroll
    for (int s = 0; s < 2; s++)
        a_off[s] = l15 * 128 + (((s * 4 + q) ^ (lane & 7)) << 4);

    // Activation fragment pointers: token-major B, one contiguous K vector per token.
    const _Float16* bptr[NB];
    bool btok[NB];
#pragma unroll
    for (int c = 0; c < NB; c++) {
        int tok = c * 16 + l15;
        btok[c] = tok < N;
        bptr[c] = B + (size_t)(btok[c] ? tok : 0) * K + q * 8;
    }

    // The stream of this unit is cut into segments: a tile of n vectors is
    // ceil(n / (VPL*64)) segments (an empty tile is one empty segment).  The
    // first segment of a tile clears the LDS tile, the last one multiplies.
    constexpr int kSeg = VPL * kWave;
    struct Cursor {
        int kb;   // 64-column tile index within the tile row
        int off;  // vectors of this tile covered by earlier segments
    };
    auto next = [&](Cursor c) {
        const int n = c.kb < kb1 ? toff[c.kb + 1] - toff[c.kb] : 0;
        return (c.off + kSeg >= n) ? Cursor{c.kb + 1, 0} : Cursor{c.kb, c.off + kSeg};
    };

    TileRegs<VPL> regs[2];
    half8 bfrag[2][NB][2];

    // Loads are issued unconditionally (a cursor past the end reads through a
    // null descriptor and a clamped activation pointer), again to keep the
    // number of outstanding loads static.
    auto issue = [&](int slot, Cursor c) {
        const bool live = c.kb < kb1;
        const int kb = live ? c.kb : kb1 - 1;
        const int n = toff[kb + 1] - toff[kb] - c.off;
        __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<u32x4*>(items + unit_begin), 0, live ? (unit_end - unit_begin) * 16 : 0, 0x00020000);
        load_segment<VPL>(regs[slot], rs, toff[kb] - unit_begin + c.off, n < kSeg ? n : kSeg, lane);
#pragma unroll
        for (int cb = 0; cb < NB; cb++)
#pragma unroll
            for (int s = 0; s < 2; s++)
                bfrag[slot][cb][s] = *reinterpret_cast<const half8*>(bptr[cb] + kb * kTileCols + s * 32);
    };

    auto consume = [&](int slot, Cursor c) {
        const int n = toff[c.kb + 1] - toff[c.kb];
        const int here = n - c.off;  // vectors from this segment's start to the tile's end
        if (c.off == 0 && n > 0) {
#pragma unroll
            for (int u = 0; u < kTileBytes / (kWave * 16); u++)
                *reinterpret_cast<u32x4_a*>(tile + u * (kWave * 16) + lane * 16) = u32x4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int u = 0; u < VPL; u++)
            if (u * kWave < here)
                scatter_vec(tile, regs[slot].v[u]);
        // the last segment of a non-empty tile: read back as dense operands and multiply
        if (n > 0 && here <= kSeg) {
#pragma unroll
            for (int s = 0; s < 2; s++) {
#pragma unroll
                for (int r = 0; r < 8; r++) {
                    half8 a = *reinterpret_cast<const half8*>(tile + a_off[s] + r * 2048);
#pragma unroll
                    for (int cb = 0; cb < NB; cb++) {
                        half8 bv = bfrag[slot][cb][s];
                        if (!btok[cb])
                            bv = half8{0, 0, 0, 0, 0, 0, 0, 0};
                        acc[cb][r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bv, acc[cb][r], 0, 0, 0);
                    }
                }
            }
        }
    };

    if (kb0 < kb1) {
        Cursor c0{kb0, 0};
        issue(0, c0);
        for (;;) {
            Cursor c1 = next(c0);
            issue(1, c1);
            consume(0, c0);
            if (c1.kb >= kb1)
                break;
            c0 = next(c1);
            issue(0, c0);
            consume(1, c1);
            if (c0.kb >= kb1)
                break;
        }
    }

    // Epilogue.  acc[c][r][i] is output row r*16 + 4*q + i of this tile row for
    // token c*16 + l15; the output keeps one contiguous M vector per token.
    _Float16* obase = out + (size_t)batch * M * N + (size_t)rt * kTileRows + q * 4;
#pragma unroll
    for (int c = 0; c < NB; c++) {
        if (!btok[c])
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

template<int NB, int VPL>
int launch_spmm(hipStream_t stream, const void* items, const int* offsets, const void* B, void* out, int M, int N,
                int K, int split_k)
{
    const int units = (M / kTileRows) * split_k;
    hipLaunchKernelGGL((tcsl_spmm_kernel<NB, VPL>), dim3(units), dim3(kWave), 0, stream,
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
        case 16:
            return launch_spmm<1, 8>(s, items, offsets, B, out, M, N, K, split_k);
        case 32:
            return launch_spmm<2, 8>(s, items, offsets, B, out, M, N, K, split_k);
        case 64:
            return launch_spmm<4, 8>(s, items, offsets, B, out, M, N, K, split_k);
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
