// gfx950 kernels for the 2:4 part of a weight: C[n][m] (+ split-K slabs) = A1 * B with A1 held as
// records in sparse-MFMA operand order (layout: a24_format.h).  The reference runs this part on
// NVIDIA's mma.sp (csrc/SpMM_Kernel.cuh:293-735 with csrc/MMA_PTX.cuh:195-210); nothing of that
// is reused.  Here a wave loads values and positions straight into the registers that
// v_smfmac_f32_16x16x32_f16 reads: no LDS staging of the weights, no scatter.
//
// Two work splits.  a24_spmm_kernel: a workgroup owns RB consecutive 16-row blocks of one split-K
// batch; its W waves cut the batch's 128-column units among themselves, keep RB x N/16
// accumulator tiles each, fetch their activation fragments from the L2 in operand order, and add
// up through LDS in wave order at the end (fp32, one rounding to fp16).
// a24_spmm_shared_b_kernel (the default launch): the waves own rows instead and share each unit's
// activation tile through LDS.  Also here: the split + pack on the GPU, and the second stream
// that the two-stream form of the hybrid call uses.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>
#include <type_traits>

#include "split_k_in_launch.h"

extern "C" int tcsl_counter_page_address(int page, unsigned int** address);  // spmm_kernels.hip

namespace {

typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
constexpr int kRecordBytes = 2304;
constexpr int kGroupBlocks = 8;                             // records of eight row blocks are stored together, unit by unit
constexpr int kUnitStride = kGroupBlocks * kRecordBytes;    // bytes between a row block's records of two consecutive units

// First record (unit 0) of 16-row block rb.
__device__ __forceinline__ const uint8_t* block_records(const uint8_t* packed, int rb, int units)
{
    return packed + ((size_t)(rb / kGroupBlocks) * units * kGroupBlocks + rb % kGroupBlocks) * kRecordBytes;
}

struct AFrag {      // one record's share of a lane
    u32x4 v[2];     // steps 0,1 and steps 2,3: four fp16 values each
    unsigned idx;   // byte s = positions for step s
};

template<int NT>
struct BFrag {
    half8 b[NT][4];  // token block x step: eight consecutive columns of one token
};

__device__ __forceinline__ AFrag load_a(const uint8_t* rec, int lane)
{
    AFrag a;
    a.v[0] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(rec + lane * 16));
    a.v[1] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(rec + 1024 + lane * 16));
    a.idx = __builtin_nontemporal_load(reinterpret_cast<const unsigned*>(rec + 2048 + lane * 4));
    return a;
}

// The shared-tile kernel issues its loads from inline assembly and waits for them by hand: left
// to itself the compiler sinks a prefetch to the block that first uses it and waits for every
// load at the loop's joins, so no unit's loads ever overlap another unit's multiplication.  The
// compiler does not know that these registers are written later; the source keeps every register
// of a load untouched until the wait that covers it (the build checks that on the generated code).
__device__ __forceinline__ AFrag issue_a(const uint8_t* rec_lane, const uint8_t* idx_lane)
{
    AFrag a;
    asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(a.v[0]) : "v"(rec_lane));
    asm volatile("global_load_dwordx4 %0, %1, off offset:1024 nt" : "=v"(a.v[1]) : "v"(rec_lane));
    asm volatile("global_load_dword %0, %1, off offset:2048 nt" : "=v"(a.idx) : "v"(idx_lane));
    return a;
}
__device__ __forceinline__ u32x4 issue_b(const _Float16* p)
{
    u32x4 r;
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(r) : "v"(p));
    return r;
}
template<int N>
__device__ __forceinline__ void wait_loads()  // at most N loads stay in flight (they complete in order)
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N < 63 ? N : 63) : "memory");
}
template<typename T>
__device__ __forceinline__ void settle(T& x)  // the register's value is the one that landed, from here on
{
    asm volatile("" : "+v"(x));
}

template<int NT>
__device__ __forceinline__ void load_b(BFrag<NT>& f, const _Float16* const (&tok)[NT], int unit)
{
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int s = 0; s < 4; s++)
            f.b[t][s] = *reinterpret_cast<const half8*>(tok[t] + (size_t)unit * 128 + s * 32);
}

__device__ __forceinline__ half4 step_values(const AFrag& a, int s)
{
    union {
        u32x4 u;
        half4 h[2];
    } x;
    x.u = a.v[s >> 1];
    return x.h[s & 1];
}

template<int NT, int RB>
__device__ __forceinline__ void multiply(float4v (&acc)[RB][NT], const AFrag (&a)[RB], const BFrag<NT>& f)
{
#pragma unroll
    for (int t = 0; t < NT; t++) {
#pragma unroll
        for (int r = 0; r < RB; r++) {
            acc[r][t] = __builtin_amdgcn_smfmac_f32_16x16x32_f16(step_values(a[r], 0), f.b[t][0], acc[r][t], (int)a[r].idx, 0, 0);
            acc[r][t] = __builtin_amdgcn_smfmac_f32_16x16x32_f16(step_values(a[r], 1), f.b[t][1], acc[r][t], (int)a[r].idx, 0, 1);
            acc[r][t] = __builtin_amdgcn_smfmac_f32_16x16x32_f16(step_values(a[r], 2), f.b[t][2], acc[r][t], (int)a[r].idx, 0, 2);
            acc[r][t] = __builtin_amdgcn_smfmac_f32_16x16x32_f16(step_values(a[r], 3), f.b[t][3], acc[r][t], (int)a[r].idx, 0, 3);
        }
    }
}

// grid (M / (16 * RB), Split_K), block W * 64.  out + batch * slab is the batch's fp16 [N][ldo]
// result.  n_tokens may be 8 with NT = 1: tokens 8..15 then read token 7 again and are not stored.
template<int NT, int RB, int W>
__global__ __launch_bounds__(W* kWave) void a24_spmm_kernel(const uint8_t* __restrict__ packed,
                                                            const _Float16* __restrict__ B, _Float16* __restrict__ out,
                                                            int units, int units_per_batch, long ldb, long ldo,
                                                            long slab, int n_tokens)
{
    extern __shared__ float4v lds[];  // [W][RB][NT][64]
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int batch = blockIdx.y;
    // this wave's units of the batch
    const int b0 = batch * units_per_batch;
    const int bcnt = min(units_per_batch, units - b0);
    const int base = bcnt / W, rem = bcnt % W;
    const int u0 = b0 + wave * base + min(wave, rem);
    const int u1 = u0 + base + (wave < rem ? 1 : 0);

    const uint8_t* rec[RB];
#pragma unroll
    for (int r = 0; r < RB; r++)
        rec[r] = block_records(packed, blockIdx.x * RB + r, units);
    const _Float16* tok[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        int n = t * 16 + (lane & 15);
        n = n < n_tokens ? n : n_tokens - 1;
        tok[t] = B + (size_t)n * ldb + (lane >> 4) * 8;
    }

    float4v acc[RB][NT];
#pragma unroll
    for (int r = 0; r < RB; r++)
#pragma unroll
        for (int t = 0; t < NT; t++)
            acc[r][t] = float4v{0.f, 0.f, 0.f, 0.f};

    AFrag a0[RB], a1[RB];
    BFrag<NT> f0, f1;
    int u = u0;
    if (u < u1) {
        load_b<NT>(f0, tok, u);
#pragma unroll
        for (int r = 0; r < RB; r++)
            a0[r] = load_a(rec[r] + (size_t)u * kUnitStride, lane);
        while (true) {
            if (u + 1 < u1) {
                load_b<NT>(f1, tok, u + 1);
#pragma unroll
                for (int r = 0; r < RB; r++)
                    a1[r] = load_a(rec[r] + (size_t)(u + 1) * kUnitStride, lane);
            }
            multiply<NT, RB>(acc, a0, f0);
            if (++u >= u1)
                break;
            if (u + 1 < u1) {
                load_b<NT>(f0, tok, u + 1);
#pragma unroll
                for (int r = 0; r < RB; r++)
                    a0[r] = load_a(rec[r] + (size_t)(u + 1) * kUnitStride, lane);
            }
            multiply<NT, RB>(acc, a1, f1);
            if (++u >= u1)
                break;
        }
    }

    // sum over the workgroup's waves, in wave order
    if constexpr (W > 1) {
#pragma unroll
        for (int r = 0; r < RB; r++)
#pragma unroll
            for (int t = 0; t < NT; t++)
                lds[((wave * RB + r) * NT + t) * kWave + lane] = acc[r][t];
        __syncthreads();
    }
    _Float16* dst = out + (size_t)batch * slab;
    const int row0 = blockIdx.x * RB * 16 + (lane >> 4) * 4;
    for (int p = wave; p < RB * NT; p += W) {
        const int r = p / NT, t = p % NT;
        float4v s;
        if constexpr (W > 1) {
            s = lds[(r * NT + t) * kWave + lane];
            for (int w = 1; w < W; w++) {
                const float4v x = lds[((w * RB + r) * NT + t) * kWave + lane];
                s += x;
            }
        } else {
            // with one wave the loop index is compile-time only through this unrolled search
            s = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int rr = 0; rr < RB; rr++)
#pragma unroll
                for (int tt = 0; tt < NT; tt++)
                    if (rr == r && tt == t)
                        s = acc[rr][tt];
        }
        const int n = t * 16 + (lane & 15);
        if (n < n_tokens) {
            half4 h = {static_cast<_Float16>(s[0]), static_cast<_Float16>(s[1]), static_cast<_Float16>(s[2]),
                       static_cast<_Float16>(s[3])};
            *reinterpret_cast<half4*>(dst + (size_t)n * ldo + row0 + r * 16) = h;
        }
    }
}

// The other work split, the library's default: the W waves of a workgroup own RB row blocks each
// (16 * RB * W rows per workgroup) and walk the batch's units together.  The unit's activation
// tile (n_tokens x 128 fp16) is fetched once per workgroup with full-line loads, kept in LDS
// (two buffers, rows padded to 272 bytes so that the sixteen lanes of a quarter wave read sixteen
// different bank groups) and read back by every wave in operand order: a wave's fragments come
// from LDS instead of the L2, and no sum across waves is needed at the end.
constexpr int kRowBytes = 272;

// With RL > 0 the same launch also multiplies the residual (what the split leaves beyond two kept
// values per group of four), so that C = A1*B + A2*B costs one pass over the activations instead of
// two kernels and a sum.  The residual comes as one list of words per record (a24_format.h:
// fp16 value | byte address in a 16 x 128 image << 16); RL rounds of 64 words travel with the unit's
// records, and what a longer list holds beyond them is fetched inside the unit's multiplication.  A wave
// scatters a list into its own 4 KiB LDS image (ds_write_b16; lanes past the end repeat the last
// word), reads the image back as dense MFMA operands, writes zeros where it wrote values, and runs
// v_mfma_f32_16x16x32_f16 on the same activation fragments and accumulators as the sparse
// instruction.  The lists' offsets travel one unit ahead of the words, on the vector path like
// everything else, so that every unit issues the same number of loads.
constexpr int kImageBytes = 4096;

// RM: the operands are row-major, this fork's own layout (csrc/SpMM_Kernel.cuh:372-374 for B,
// :731-734 for the output): B[k][n] (K x n_tokens, dense), out / fused_out and the slabs [m][n]
// (M x n_tokens, dense; ldb, ldo and ldc are not used).  A unit's 128 x n_tokens activation block is
// then one contiguous run: it is staged in LDS as it sits in memory (with 64 tokens the four
// 32-byte column chunks of a row are permuted by (k >> 1) & 3, so that the four rows one read touches
// fall into different banks) and read back with the transposing LDS read ds_read_b64_tr_b16, which
// hands lane i of a group of sixteen the i-th column of a 4 x 16 block whose rows the sixteen lanes
// address four to a row: two such reads give a lane the eight consecutive k of its token that the
// matrix instructions want.
template<int NT, int RB, int W, int RL, bool RM = false>
__global__ __launch_bounds__(W* kWave) void a24_spmm_shared_b_kernel(const uint8_t* __restrict__ packed,
                                                                     const _Float16* __restrict__ B,
                                                                     _Float16* __restrict__ out, int units,
                                                                     int units_per_batch, long ldb, long ldo, long slab,
                                                                     int n_tokens, const unsigned* __restrict__ words,
                                                                     const int* __restrict__ offsets, int relu, int M,
                                                                     _Float16* __restrict__ fused_out,
                                                                     unsigned int* __restrict__ arrivals, long ldc)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char tile[];  // [2][NT * 16][kRowBytes], then [W][kImageBytes]
    constexpr int kBuf = NT * 16 * kRowBytes;
    constexpr int RLA = RL > 0 ? RL : 1;
    constexpr int kThreads = W * kWave;
    constexpr int CH = (NT * 256 + kThreads - 1) / kThreads;  // 16-byte chunks of a tile per thread
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int batch = blockIdx.y;
    const int u0 = batch * units_per_batch;
    const int u1 = min(units, u0 + units_per_batch);
    const int block0 = (blockIdx.x * W + wave) * RB;

    const uint8_t* rec[RB];
#pragma unroll
    for (int r = 0; r < RB; r++)
        rec[r] = block_records(packed, block0 + r, units);
    // this thread's chunks of the activation tile: token c / 16, columns (c % 16) * 8 .. + 8
    // (RM: chunk c of the unit's contiguous block, i.e. tokens 8 (c % (n_tokens / 8)) .. + 7 of row
    // c / (n_tokens / 8), kept where it sits in memory)
    auto rm_byte = [&](int k, int n) __attribute__((always_inline)) {  // LDS byte of B[unit's row k][token n], RM only
        return n_tokens == 64 ? k * 128 + ((((n >> 4) ^ (k >> 1)) & 3) << 5) + (n & 15) * 2 : (k * n_tokens + n) * 2;
    };
    const _Float16* src[CH];
    int dst[CH];
    const size_t unit_step = RM ? (size_t)128 * n_tokens : 128;  // elements between a chunk's places in two consecutive units
#pragma unroll
    for (int i = 0; i < CH; i++) {
        const int c = tid + i * kThreads;
        if constexpr (RM) {
            const int cc = c < n_tokens * 16 ? c : 0;
            const int per_row_log2 = __builtin_ctz(n_tokens >> 3);
            src[i] = B + (size_t)cc * 8;
            dst[i] = rm_byte(cc >> per_row_log2, 8 * (cc & ((1 << per_row_log2) - 1)));
        } else {
            const int n = c < n_tokens * 16 ? c >> 4 : 0;
            src[i] = B + (size_t)n * ldb + (c & 15) * 8;
            dst[i] = n * kRowBytes + (c & 15) * 16;
        }
    }
    // where this lane's fragments sit in a buffer (with more than 16 tokens every token block is
    // full, so the blocks are a constant apart: one register instead of NT)
    int frag[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        int n = t * 16 + (lane & 15);
        if (NT == 1)
            n = n < n_tokens ? n : n_tokens - 1;
        frag[t] = n * kRowBytes + (lane >> 4) * 16;
    }
    // RM: where the two transposing reads (hh = 0, 1) of step 0 for token block t start: lane j of a
    // group of sixteen points at row 8 (lane / 16) + 4 hh + j / 4, tokens 16 t + 4 (j % 4) .. + 3 (with
    // 8 tokens the upper half repeats the lower); a step further is 32 rows further.  Everything
    // but the lane's own part is a constant of (t, hh): with 64 tokens the permuted chunk is
    // t ^ (2 hh + j / 8), whose bit 1 is constant and whose bit 0 is j / 8 for even t and its
    // complement for odd t, so two registers serve all blocks.
    int tr_lane[2] = {0, 0};
    const int rm_row_bytes = NT == 4 ? 128 : 2 * n_tokens;
    if constexpr (RM) {
        const int l15 = lane & 15;
        const int base0 = (8 * (lane >> 4) + (l15 >> 2)) * rm_row_bytes + ((4 * (l15 & 3)) & (n_tokens - 1)) * 2;
        tr_lane[0] = NT == 4 ? base0 + 32 * (l15 >> 3) : base0;
        tr_lane[1] = NT == 4 ? base0 + 32 - 32 * (l15 >> 3) : base0;
    }
    auto tr_at = [&](int t, int hh) __attribute__((always_inline)) {
        return NT == 4 ? tr_lane[t & 1] + 512 * hh + 64 * ((t >> 1) ^ hh) : tr_lane[0] + 4 * hh * rm_row_bytes + 32 * t;
    };
    const int tr_step = 32 * rm_row_bytes;

    // The residual's dense products get accumulators of their own, added to the others at the end:
    // a dense MFMA that takes the sparse instruction's result as its addend directly behind it read
    // the last two of the four registers before they were written (the compiler places no wait
    // between the two kinds; chains of one kind are fine).
    float4v acc[RB][NT], accd[RL > 0 ? RB : 1][NT];
#pragma unroll
    for (int r = 0; r < RB; r++)
#pragma unroll
        for (int t = 0; t < NT; t++) {
            acc[r][t] = float4v{0.f, 0.f, 0.f, 0.f};
            if constexpr (RL > 0)
                accd[r][t] = float4v{0.f, 0.f, 0.f, 0.f};
        }

    // Three rotating sets of "unit registers": the records of RB row blocks and this thread's chunks
    // of the activation tile.  (A thread beyond the tile's last chunk repeats one of token 0's: the
    // same bytes to the same place, so that every thread issues the same number of loads.)
    struct UnitRegs {
        AFrag a[RB];
        u32x4 stage[CH];
        unsigned w[RB][RLA];  // residual words of the unit's RB lists
        int next;             // lane j <= RB: offsets[first record of the unit after this one + j]
        int count[RB];        // words in each list (the same in every lane)
        int start[RB];        // where each list starts in `words`
    };
    constexpr int kLoadsA = (3 + RL) * RB;      // loads of one unit's records and lists per lane
    constexpr int kLoadsHead = RL > 0 ? 1 : 0;  // the offsets load that leads a unit's loads
    // A launch with the most rounds (five, 320 words) may meet lists that are longer still (blocks
    // of a row-skewed or nearly dense weight; a residual block holds up to 1024 words).  EX further
    // rounds of such a list are fetched when the unit's turn comes, ahead of the loads that the
    // same phase issues for the unit two further on, and awaited with the count of just those
    // loads; whatever a list holds beyond that comes through ordinary loads inside the
    // multiplication, which wait for everything in flight.  Extra loads never invalidate the
    // constant waits elsewhere: a wait that allows N loads to stay outstanding covers the loads it
    // is meant for however many younger ones there are.
    constexpr bool kLong = RL == 5;
    constexpr int EX = 3;
    constexpr int kLoadsUnit = kLoadsHead + CH + kLoadsA;  // what issue_unit puts in flight
    unsigned ex[RB][EX] = {};
    auto any_longer = [&](const UnitRegs& x) __attribute__((always_inline)) {
        bool any = false;
#pragma unroll
        for (int r = 0; r < RB; r++)
            any = any || x.count[r] > RL * kWave;
        return any;
    };
    auto issue_extras = [&](const UnitRegs& x) __attribute__((always_inline)) {
        if constexpr (kLong) {
            if (any_longer(x)) {  // all RB * EX loads or none: lanes and rounds past a list's end repeat its last word
#pragma unroll
                for (int r = 0; r < RB; r++) {
                    const int last = x.count[r] > 0 ? x.count[r] - 1 : 0;
#pragma unroll
                    for (int i = 0; i < EX; i++) {
                        const int at = lane + (RL + i) * kWave;
                        const unsigned* p = words + x.start[r] + (at < last ? at : last);
                        asm volatile("global_load_dword %0, %1, off nt" : "=v"(ex[r][i]) : "v"(p));
                    }
                }
            }
        }
    };
    // lists are numbered like records: this wave's RB lists of a unit are neighbours
    const long list0 = ((long)(block0 / kGroupBlocks) * units) * kGroupBlocks + block0 % kGroupBlocks;
    const int* const off_lane = offsets + list0 + (lane <= RB ? lane : RB);
    unsigned char* const image = tile + 2 * kBuf + wave * kImageBytes;
    // A unit's loads: the offsets of the unit after it, its activation chunks (needed first), its
    // records, and (issue_words; o[0..RB] = the offsets of the unit's lists, the same in every lane)
    // its residual words.
    auto issue_head = [&](UnitRegs& x, int unit, int unit_after) __attribute__((always_inline)) {
        if constexpr (RL > 0)
            asm volatile("global_load_dword %0, %1, off" : "=v"(x.next) : "v"(off_lane + (size_t)unit_after * kGroupBlocks));
#pragma unroll
        for (int i = 0; i < CH; i++)
            x.stage[i] = issue_b(src[i] + (size_t)unit * unit_step);
#pragma unroll
        for (int r = 0; r < RB; r++)
            x.a[r] = issue_a(rec[r] + (size_t)unit * kUnitStride + lane * 16, rec[r] + (size_t)unit * kUnitStride + lane * 4);
    };
    auto issue_words = [&](UnitRegs& x, const int (&o)[RB + 1]) __attribute__((always_inline)) {
        if constexpr (RL > 0) {
#pragma unroll
            for (int r = 0; r < RB; r++) {
                const int n = o[r + 1] - o[r];
                x.count[r] = n;
                x.start[r] = o[r];
                const int last = n > 0 ? n - 1 : 0;
#pragma unroll
                for (int i = 0; i < RL; i++) {
                    const int at = lane + i * kWave;
                    const unsigned* p = words + o[r] + (at < last ? at : last);
                    asm volatile("global_load_dword %0, %1, off nt" : "=v"(x.w[r][i]) : "v"(p));
                }
            }
        }
    };
    auto issue_unit = [&](UnitRegs& x, int unit, int unit_after, const int (&o)[RB + 1]) __attribute__((always_inline)) {
        issue_head(x, unit, unit_after);
        issue_words(x, o);
    };
    // The offsets that a unit's `next` load brought, once it has landed.
    auto offsets_from = [&](UnitRegs& x, int (&o)[RB + 1]) __attribute__((always_inline)) {
        if constexpr (RL > 0) {
            settle(x.next);
#pragma unroll
            for (int j = 0; j <= RB; j++)
                o[j] = __builtin_amdgcn_readlane(x.next, j);
        }
    };
    auto store_b = [&](UnitRegs& x, int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < CH; i++) {
            settle(x.stage[i]);
            *reinterpret_cast<u32x4*>(tile + buf * kBuf + dst[i]) = x.stage[i];
        }
    };
    auto landed = [&](UnitRegs& x) __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < RB; r++) {
            settle(x.a[r].v[0]);
            settle(x.a[r].v[1]);
            settle(x.a[r].idx);
            if constexpr (RL > 0) {
#pragma unroll
                for (int i = 0; i < RL; i++)
                    settle(x.w[r][i]);
            }
        }
    };
    // where this lane's dense operands sit in the image: row lane % 16, granule (4 s + lane / 16) ^ row
    const int img_row = (lane & 15) * 256;
    auto multiply_from = [&](UnitRegs& x, int buf) __attribute__((always_inline)) {
        const AFrag(&a)[RB] = x.a;
        half8 dense[RB][4];
        if constexpr (kLong) {
            if (any_longer(x)) {  // the extra rounds were issued just before this phase's issue_unit
                wait_loads<kLoadsUnit>();
#pragma unroll
                for (int r = 0; r < RB; r++)
#pragma unroll
                    for (int i = 0; i < EX; i++)
                        settle(ex[r][i]);
            }
        }
        if constexpr (RL > 0) {
            // One list after the other through the wave's image: LDS operations of a wave run in
            // order, so values, read-back and zeros need no barrier.
#pragma unroll
            for (int r = 0; r < RB; r++) {
                const int n = x.count[r];
                if (n > 0) {
#pragma unroll
                    for (int i = 0; i < RL; i++)
                        if (i == 0 || n > i * kWave)
                            *reinterpret_cast<unsigned short*>(image + (x.w[r][i] >> 16)) = static_cast<unsigned short>(x.w[r][i]);
                    // A list longer than the RL rounds that travel with the unit: EX more rounds
                    // have just landed (above); the rest is fetched here, with ordinary loads,
                    // which wait for everything this wave has in flight (a stall per round, for
                    // lists of more than 512 words only).
                    const bool longer = kLong && n > RL * kWave;
                    if constexpr (kLong) {
                        if (longer) {
                            // (already waited for at the top on every real path: repeated here so
                            // that wait and use sit under one condition, which is what the build's
                            // checker of in-flight registers can follow)
                            wait_loads<kLoadsUnit>();
#pragma unroll
                            for (int i = 0; i < EX; i++)
                                settle(ex[r][i]);
#pragma unroll
                            for (int i = 0; i < EX; i++)
                                if (n > (RL + i) * kWave)
                                    *reinterpret_cast<unsigned short*>(image + (ex[r][i] >> 16)) = static_cast<unsigned short>(ex[r][i]);
                            for (int at0 = (RL + EX) * kWave; at0 < n; at0 += kWave) {
                                const int at = at0 + lane;
                                const unsigned w = words[x.start[r] + (at < n ? at : n - 1)];
                                *reinterpret_cast<unsigned short*>(image + (w >> 16)) = static_cast<unsigned short>(w);
                            }
                        }
                    }
#pragma unroll
                    for (int s = 0; s < 4; s++)
                        dense[r][s] = *reinterpret_cast<const half8*>(image + img_row + (((s * 4 + (lane >> 4)) ^ (lane & 15)) << 4));
                    if (longer) {  // the extra words are gone: clear the whole image (as much LDS traffic as four rounds)
#pragma unroll
                        for (int i = 0; i < kImageBytes / (kWave * 16); i++)
                            *reinterpret_cast<u32x4*>(image + (i * kWave + lane) * 16) = u32x4{0u, 0u, 0u, 0u};
                    } else {
#pragma unroll
                        for (int i = 0; i < RL; i++)
                            if (i == 0 || n > i * kWave)
                                *reinterpret_cast<unsigned short*>(image + (x.w[r][i] >> 16)) = 0;
                    }
                }
            }
        }
#pragma unroll
        for (int t = 0; t < NT; t++) {
            half8 f[4];
#pragma unroll
            for (int s = 0; s < 4; s++) {
                if constexpr (RM) {
                    typedef short short4v __attribute__((ext_vector_type(4)));
                    typedef short short8v __attribute__((ext_vector_type(8)));
                    typedef __attribute__((address_space(3))) short4v lds_short4v;
                    const unsigned char* const at = tile + buf * kBuf + s * tr_step;
                    const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4v*)(at + tr_at(t, 0)));
                    const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4v*)(at + tr_at(t, 1)));
                    const short8v both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    f[s] = __builtin_bit_cast(half8, both);
                } else {
                    f[s] = *reinterpret_cast<const half8*>(tile + buf * kBuf + frag[t] + s * 64);
                }
            }
#pragma unroll
            for (int r = 0; r < RB; r++) {
                acc[r][t] = __builtin_amdgcn_smfmac_f32_16x16x32_f16(step_values(a[r], 0), f[0], acc[r][t], (int)a[r].idx, 0, 0);
                acc[r][t] = __builtin_amdgcn_smfmac_f32_16x16x32_f16(step_values(a[r], 1), f[1], acc[r][t], (int)a[r].idx, 0, 1);
                acc[r][t] = __builtin_amdgcn_smfmac_f32_16x16x32_f16(step_values(a[r], 2), f[2], acc[r][t], (int)a[r].idx, 0, 2);
                acc[r][t] = __builtin_amdgcn_smfmac_f32_16x16x32_f16(step_values(a[r], 3), f[3], acc[r][t], (int)a[r].idx, 0, 3);
                if constexpr (RL > 0) {
                    if (x.count[r] > 0) {
#pragma unroll
                        for (int s = 0; s < 4; s++)
                            accd[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(dense[r][s], f[s], accd[r][t], 0, 0, 0);
                    }
                }
            }
        }
    };

    // Pipeline, per unit u (records two units ahead, the tile one buffer ahead; queue oldest first;
    // with the residual, "records" stands for records + words, and every unit's loads are led by
    // the offsets of the unit after it):
    //   in flight at the top        records(u), [offsets(u+2),] tile(u+1), records(u+1)
    //   wait until only kLoadsA stay   -> records(u), offsets(u+2) and tile(u+1) have landed
    //   tile(u+1) -> the other LDS buffer; issue [offsets(u+3),] tile(u+2), records(u+2); multiply unit u; barrier
    // Loads past the batch's end repeat its last unit, so every path issues the same loads and the
    // wait count is a constant.  A buffer is written only after the barrier that follows its last reader.
    UnitRegs x[3];
    int u = u0;  // every wave of the workgroup walks the same units: the barriers below are uniform
    if (u < u1) {
        const int last = u1 - 1;
        auto ahead = [&](int d) __attribute__((always_inline)) { return u + d < last ? u + d : last; };
        int o[RB + 1] = {};
        if constexpr (RL > 0) {
            // The first two units' offsets are fetched by themselves, and their records and
            // activation chunks go out before those offsets are back; their words follow.  The
            // queue of the first phase is therefore: records(u), unit u + 1's head, words(u), words(u + 1).
            int first, second;
            asm volatile("global_load_dword %0, %1, off" : "=v"(first) : "v"(off_lane + (size_t)u * kGroupBlocks));
            asm volatile("global_load_dword %0, %1, off" : "=v"(second) : "v"(off_lane + (size_t)ahead(1) * kGroupBlocks));
            issue_head(x[0], u, ahead(1));
            issue_head(x[1], ahead(1), ahead(2));
            for (int i = lane * 16; i < kImageBytes; i += kWave * 16)  // the image starts out clear
                *reinterpret_cast<u32x4*>(image + i) = u32x4{0u, 0u, 0u, 0u};
            wait_loads<2 * (kLoadsHead + CH + 3 * RB)>();
            settle(first);
            settle(second);
#pragma unroll
            for (int j = 0; j <= RB; j++)
                o[j] = __builtin_amdgcn_readlane(first, j);
            issue_words(x[0], o);
#pragma unroll
            for (int j = 0; j <= RB; j++)
                o[j] = __builtin_amdgcn_readlane(second, j);
            issue_words(x[1], o);
        } else {
            issue_unit(x[0], u, u, o);
            issue_unit(x[1], ahead(1), u, o);
        }
        wait_loads<kLoadsA + kLoadsHead + CH + kLoadsA>();  // the first tile
        store_b(x[0], 0);
        __syncthreads();
        auto phase = [&](auto kc, auto is_first) __attribute__((always_inline)) {  // unit u, whose registers are set kc
            constexpr int k = decltype(kc)::value;
            const int buf = (u - u0) & 1;
            if constexpr (RL > 0 && decltype(is_first)::value)
                wait_loads<RL * RB>();  // only words(u + 1) are younger than what the first phase needs
            else
                wait_loads<kLoadsA>();
            landed(x[k]);
            issue_extras(x[k]);
            store_b(x[(k + 1) % 3], buf ^ 1);
            int o2[RB + 1] = {};
            offsets_from(x[(k + 1) % 3], o2);  // unit u + 1 brought the offsets of unit u + 2
            issue_unit(x[(k + 2) % 3], ahead(2), ahead(3), o2);
            multiply_from(x[k], buf);
            __syncthreads();
            ++u;
        };
        // Whole rounds of three units, then the rest: no exit from inside a round, so that every
        // path through the loop carries the same loads in the same registers.
        using std::integral_constant;
        const int units_after_first = u1 - u0 - 1;
        phase(integral_constant<int, 0>{}, integral_constant<bool, true>{});
        for (int round = units_after_first / 3; round > 0; round--) {
            phase(integral_constant<int, 1>{}, integral_constant<bool, false>{});
            phase(integral_constant<int, 2>{}, integral_constant<bool, false>{});
            phase(integral_constant<int, 0>{}, integral_constant<bool, false>{});
        }
        const int rest = units_after_first % 3;
        if (rest >= 1) {
            phase(integral_constant<int, 1>{}, integral_constant<bool, false>{});
            if (rest >= 2)
                phase(integral_constant<int, 2>{}, integral_constant<bool, false>{});
        }
        // the repeated loads of the last phases are still on their way into registers that the
        // stores below may reuse
        wait_loads<0>();
#pragma unroll
        for (int k = 0; k < 3; k++) {
            landed(x[k]);
#pragma unroll
            for (int i = 0; i < CH; i++)
                settle(x[k].stage[i]);
            if constexpr (RL > 0)
                settle(x[k].next);
        }
#pragma unroll
        for (int r = 0; r < RB; r++)
#pragma unroll
            for (int i = 0; i < EX; i++)
                settle(ex[r][i]);
    }

    _Float16* dstc = out + (size_t)batch * slab;
#pragma unroll
    for (int r = 0; r < RB; r++) {
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const int n = t * 16 + (lane & 15);
            if (n < n_tokens) {
                float4v s = acc[r][t];
                if constexpr (RL > 0)
                    s += accd[r][t];
                if (relu && !arrivals)  // partial sums are never clamped
                    s = float4v{fmaxf(s[0], 0.f), fmaxf(s[1], 0.f), fmaxf(s[2], 0.f), fmaxf(s[3], 0.f)};
                half4 h = {static_cast<_Float16>(s[0]), static_cast<_Float16>(s[1]), static_cast<_Float16>(s[2]),
                           static_cast<_Float16>(s[3])};
                if constexpr (RM) {  // [m][n]: the sixteen tokens of a row are adjacent (sixteen lanes to a 32-byte segment)
                    _Float16* const to = dstc + ((size_t)(block0 + r) * 16 + (lane >> 4) * 4) * n_tokens + n;
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        if (arrivals)
                            inlaunch::store_through(to + (size_t)i * n_tokens, h[i]);
                        else
                            to[(size_t)i * n_tokens] = h[i];
                    }
                } else {
                    _Float16* const to = dstc + (size_t)n * ldo + (block0 + r) * 16 + (lane >> 4) * 4;
                    if (arrivals)
                        inlaunch::store_through(to, h);
                    else
                        *reinterpret_cast<half4*>(to) = h;
                }
            }
        }
    }
    // arrivals != nullptr (more than one batch): `out` holds the batches' slabs ([N][M] each, M * N
    // apart), and the last workgroup to finish this group of rows adds them up into fused_out (token
    // stride ldc, clamped if relu), like the main kernel's K-splitting layout and with the same bits
    // as the reduction kernel.
    if (arrivals)
        inlaunch::fused_reduction_tail(out, fused_out, M, n_tokens, static_cast<int>(ldc), gridDim.y, relu,
                                       blockIdx.x * (16 * RB * W), 16 * RB * W, arrivals + blockIdx.x,
                                       reinterpret_cast<unsigned int*>(tile), W * kWave, RM);
}

template<int NT, int RB, int W, int RL, bool RM>
int launch_shared_b(hipStream_t stream, const void* packed, const void* B, void* out, int M, int N, int K, int split_k,
                    long ldb, long ldo, long slab, const void* words, const void* offsets, int relu, void* fused_out,
                    unsigned int* arrivals, long ldc)
{
    const int units = K / 128;
    const int per_batch = (units + split_k - 1) / split_k;
    if (M % (16 * RB * W) != 0)
        return static_cast<int>(hipErrorInvalidValue);
    const unsigned lds = 2 * NT * 16 * kRowBytes + (RL > 0 ? W * kImageBytes : 0);
    auto kern = a24_spmm_shared_b_kernel<NT, RB, W, RL, RM>;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess)
            return static_cast<int>(e);
    }
    hipLaunchKernelGGL(kern, dim3(M / (16 * RB * W), split_k), dim3(W * kWave), lds, stream,
                       static_cast<const uint8_t*>(packed), static_cast<const _Float16*>(B), static_cast<_Float16*>(out), units,
                       per_batch, ldb, ldo, slab, N, static_cast<const unsigned*>(words), static_cast<const int*>(offsets), relu, M,
                       static_cast<_Float16*>(fused_out), arrivals, ldc);
    return static_cast<int>(hipGetLastError());
}

// rl: loads per residual list (0 = no residual).  The fused form has the library's own launch
// shapes only: two row blocks per wave, four or eight waves.
template<int NT>
int launch_shared_b_nt(hipStream_t s, const void* packed, const void* B, void* out, int M, int N, int K, int split_k, int rb,
                       int waves, long ldb, long ldo, long slab, int rl, const void* words, const void* offsets, int relu,
                       void* fused_out, unsigned int* arrivals, long ldc, bool row_major)
{
#define A24_GO(RB_, W_, RL_, RM_) \
    launch_shared_b<NT, RB_, W_, RL_, RM_>(s, packed, B, out, M, N, K, split_k, ldb, ldo, slab, words, offsets, relu, fused_out, arrivals, ldc)
    // the library's own launch shapes (two row blocks per wave) take either operand layout
#define A24_CASE(RB_, W_, RL_)                   \
    if (rb == RB_ && waves == W_ && rl == RL_) \
        return row_major ? A24_GO(RB_, W_, RL_, true) : A24_GO(RB_, W_, RL_, false);
#define A24_CASE_COLUMN_MAJOR(RB_, W_, RL_)                     \
    if (rb == RB_ && waves == W_ && rl == RL_ && !row_major) \
        return A24_GO(RB_, W_, RL_, false);
    A24_CASE(2, 4, 0) A24_CASE(2, 8, 0)
    A24_CASE(2, 4, 1) A24_CASE(2, 8, 1) A24_CASE(2, 4, 2) A24_CASE(2, 8, 2) A24_CASE(2, 4, 3) A24_CASE(2, 8, 3)
    A24_CASE(2, 4, 4) A24_CASE(2, 4, 5)
    if constexpr (NT > 2) {
        A24_CASE_COLUMN_MAJOR(2, 8, 4)  // (row-major with 64 tokens: one register too many for eight waves)
    }
    if constexpr (NT <= 2) {
        A24_CASE(2, 8, 4)
        A24_CASE(2, 8, 5)  // with 64 tokens it would not fit 256 registers
        // (three record sets of four row blocks do not fit the registers beside 64 tokens)
        A24_CASE_COLUMN_MAJOR(4, 2, 0) A24_CASE_COLUMN_MAJOR(4, 4, 0) A24_CASE_COLUMN_MAJOR(4, 8, 0)
    }
#undef A24_CASE_COLUMN_MAJOR
#undef A24_CASE
#undef A24_GO
    return static_cast<int>(hipErrorInvalidValue);
}

template<int NT, int RB, int W>
int launch(hipStream_t stream, const void* packed, const void* B, void* out, int M, int N, int K, int split_k, long ldb,
           long ldo, long slab)
{
    const int units = K / 128;
    const int per_batch = (units + split_k - 1) / split_k;
    const unsigned lds = W > 1 ? W * RB * NT * kWave * sizeof(float4v) : 0;
    auto kern = a24_spmm_kernel<NT, RB, W>;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess)
            return static_cast<int>(e);
    }
    hipLaunchKernelGGL(kern, dim3(M / (16 * RB), split_k), dim3(W * kWave), lds, stream,
                       static_cast<const uint8_t*>(packed), static_cast<const _Float16*>(B), static_cast<_Float16*>(out),
                       units, per_batch, ldb, ldo, slab, N);
    return static_cast<int>(hipGetLastError());
}

template<int NT>
int launch_nt(hipStream_t s, const void* packed, const void* B, void* out, int M, int N, int K, int split_k, int rb, int waves,
              long ldb, long ldo, long slab)
{
#define A24_CASE(RB_, W_)                  \
    if (rb == RB_ && waves == W_)          \
        return launch<NT, RB_, W_>(s, packed, B, out, M, N, K, split_k, ldb, ldo, slab);
    A24_CASE(1, 4) A24_CASE(1, 8) A24_CASE(2, 2) A24_CASE(2, 4) A24_CASE(2, 8) A24_CASE(4, 1) A24_CASE(4, 2) A24_CASE(4, 4)
    if constexpr (NT <= 2) {  // larger accumulator sets would not fit the register file
        A24_CASE(4, 8) A24_CASE(8, 1) A24_CASE(8, 2) A24_CASE(8, 4)
    }
#undef A24_CASE
    return static_cast<int>(hipErrorInvalidValue);
}

}  // namespace

// Batch b of ceil((K/128)/split_k) units writes fp16 [N][ldo] to out + b * slab.  The caller has
// checked: M % (16 * rb) == 0 (share_b: M % (16 * rb * waves) == 0), K % 128 == 0, N in {8, 16, 32, 64}, no batch empty, pointers set.
// residual_loads > 0 (share_b with rb == 2 only): the launch also multiplies the residual lists
// words / offsets; residual_loads rounds of 64 words travel with the records, a longer list's rest is
// fetched where it is needed.  relu (share_b only): negative
// results are written as zero (for a launch that writes the finished result).
// fuse_page >= 0 (share_b, split_k > 1, ldo == M, slab == M * N): the launch adds its slabs up into
// fused_out (token stride ldc) itself, counting arrivals on that page of the library's counters.
// row_major (share_b with rb == 2 only): B is [K][N] and out, the slabs and fused_out [M][N], all
// dense (ldb, ldo and ldc are not used; slab == M * N).
extern "C" int a24_launch_spmm(void* stream, const void* packed, const void* B, void* out, int M, int N, int K,
                               int split_k, int rb, int waves, int share_b, long ldb, long ldo, long slab,
                               int residual_loads, const void* words, const void* offsets, int relu, int fuse_page,
                               void* fused_out, long ldc, int row_major)
{
    hipStream_t s = static_cast<hipStream_t>(stream);
    unsigned int* arrivals = nullptr;
    if (fuse_page >= 0) {
        if (!share_b || split_k < 2 || !fused_out || (ldo != M && !row_major) || slab != static_cast<long>(M) * N || rb < 1 || waves < 1
            || M / (16 * rb * waves) > 4096 || M % 8 != 0)
            return static_cast<int>(hipErrorInvalidValue);
        if (const int rc = tcsl_counter_page_address(fuse_page, &arrivals))
            return rc;
    }
    if (share_b) {  // waves own rows and share the activation tile through LDS
        switch (N) {
            case 8:
            case 16: return launch_shared_b_nt<1>(s, packed, B, out, M, N, K, split_k, rb, waves, ldb, ldo, slab, residual_loads, words, offsets, relu,
                                                     fused_out, arrivals, ldc, row_major != 0);
            case 32: return launch_shared_b_nt<2>(s, packed, B, out, M, N, K, split_k, rb, waves, ldb, ldo, slab, residual_loads, words, offsets, relu,
                                                     fused_out, arrivals, ldc, row_major != 0);
            case 64: return launch_shared_b_nt<4>(s, packed, B, out, M, N, K, split_k, rb, waves, ldb, ldo, slab, residual_loads, words, offsets, relu,
                                                     fused_out, arrivals, ldc, row_major != 0);
            default: return static_cast<int>(hipErrorInvalidValue);
        }
    }
    if (residual_loads != 0 || relu || row_major)
        return static_cast<int>(hipErrorInvalidValue);
    switch (N) {
        case 8:
        case 16: return launch_nt<1>(s, packed, B, out, M, N, K, split_k, rb, waves, ldb, ldo, slab);
        case 32: return launch_nt<2>(s, packed, B, out, M, N, K, split_k, rb, waves, ldb, ldo, slab);
        case 64: return launch_nt<4>(s, packed, B, out, M, N, K, split_k, rb, waves, ldb, ldo, slab);
        default: return static_cast<int>(hipErrorInvalidValue);
    }
}

// Split and pack on the GPU: the same bits as the host's decompose + pack (a24_pack.cpp), for
// weights that are already in device memory.  One thread per lane of a record: it reads its row's
// 4 x 8 columns of the unit, keeps the first two kept values of every group of four
// (kernel_benchmark/spmm_decompose.h:12-51) in the record and writes the others to the dense
// residual (when asked for one), zero elsewhere.
__global__ __launch_bounds__(256) void a24_split_pack_kernel(const uint16_t* __restrict__ A, uint8_t* __restrict__ packed,
                                                             uint16_t* __restrict__ residual, int K, int units,
                                                             long records)
{
    const long id = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long record = id >> 6;
    if (record >= records)
        return;
    const int L = static_cast<int>(id & 63);
    // records are numbered ((rb / 8) * units + u) * 8 + rb % 8
    const long group = record / (static_cast<long>(units) * kGroupBlocks);
    const int within = static_cast<int>(record - group * units * kGroupBlocks);
    const int u = within / kGroupBlocks;
    const long rb = group * kGroupBlocks + within % kGroupBlocks;
    const size_t row = (size_t)(rb * 16 + (L & 15)) * K + (size_t)u * 128 + (L >> 4) * 8;
    uint8_t* rec = packed + (size_t)record * kRecordBytes;
    typedef unsigned short u16x8 __attribute__((ext_vector_type(8)));
    unsigned word = 0;
#pragma unroll
    for (int s = 0; s < 4; s++) {
        const u16x8 in = *reinterpret_cast<const u16x8*>(A + row + s * 32);
        u16x8 rest = {0, 0, 0, 0, 0, 0, 0, 0};
        unsigned short val[4];
#pragma unroll
        for (int half = 0; half < 2; half++) {
            int pos[2] = {0, 1}, n = 0;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const unsigned short v = in[half * 4 + e];
                if ((v & 0x7fffu) != 0) {  // compares unequal to zero as a float: NaN counts, -0 does not
                    if (n < 2)
                        pos[n] = e;
                    else
                        rest[half * 4 + e] = v;
                    n++;
                }
            }
            unsigned short v0 = 0, v1 = 0;
            if (n >= 2) {
                v0 = in[half * 4 + pos[0]];
                v1 = in[half * 4 + pos[1]];
            } else if (n == 1) {
                if (pos[0] == 3) {  // the free slot goes before it
                    v1 = in[half * 4 + 3];
                    pos[0] = 2;
                    pos[1] = 3;
                } else {
                    v0 = in[half * 4 + pos[0]];
                    pos[1] = 3;
                }
            } else {
                pos[0] = 0;
                pos[1] = 1;
            }
            val[half * 2] = v0;
            val[half * 2 + 1] = v1;
            word |= static_cast<unsigned>(pos[0]) << (8 * s + 4 * half) | static_cast<unsigned>(pos[1]) << (8 * s + 4 * half + 2);
        }
        typedef unsigned short u16x4 __attribute__((ext_vector_type(4)));
        const u16x4 out = {val[0], val[1], val[2], val[3]};
        *reinterpret_cast<u16x4*>(rec + (s >> 1) * 1024 + L * 16 + (s & 1) * 8) = out;
        if (residual)
            *reinterpret_cast<u16x8*>(residual + row + s * 32) = rest;
    }
    *reinterpret_cast<unsigned*>(rec + 2048 + L * 4) = word;
}

// A: row-major M x K fp16 in device memory (M % 16 == 0, K % 128 == 0, checked by the caller);
// residual may be null.
extern "C" int a24_launch_split_pack(void* stream, const void* A, void* packed, void* residual, int M, int K)
{
    const int units = K / 128;
    const long records = static_cast<long>(M / 16) * units;
    const long blocks = (records * 64 + 255) / 256;
    if (blocks < 1 || blocks > 0x7fffffffL)
        return static_cast<int>(hipErrorInvalidValue);
    hipLaunchKernelGGL(a24_split_pack_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t*>(A), static_cast<uint8_t*>(packed), static_cast<uint16_t*>(residual), K,
                       units, records);
    return static_cast<int>(hipGetLastError());
}

// The residual lists (a24_format.h) on the GPU, from the dense residual that the split above
// leaves in device memory: the same words in the same order as the host's pack_residual
// (a24_pack.cpp).  Three kernels: count per record, scan, emit.  One wave per record: lane L
// reads columns 32 * (L % 4) .. + 31 of row L / 4, so lane order is the row-major order that the
// host collects a list in.
namespace {

constexpr int kMaxListWords = 16 * 128 / 2;  // a residual holds at most two of every four

__device__ __forceinline__ bool residual_kept(unsigned v)
{
    return (v & 0x7fffu) != 0;
}

__device__ __forceinline__ void record_of_list(long list, int units, long& rb, int& u)
{
    const long group = list / (static_cast<long>(units) * kGroupBlocks);
    const int within = static_cast<int>(list - group * units * kGroupBlocks);
    u = within / kGroupBlocks;
    rb = group * kGroupBlocks + within % kGroupBlocks;
}

typedef unsigned short u16x8v __attribute__((ext_vector_type(8)));

__global__ __launch_bounds__(256) void a24_residual_count_kernel(const uint16_t* __restrict__ A2, int K, int units,
                                                                 long lists, int* __restrict__ offsets)
{
    const long list = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (list >= lists)
        return;
    const int L = threadIdx.x & 63;
    long rb;
    int u;
    record_of_list(list, units, rb, u);
    const uint16_t* src = A2 + (size_t)(rb * 16 + (L >> 2)) * K + (size_t)u * 128 + (L & 3) * 32;
    int n = 0;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const u16x8v v = *reinterpret_cast<const u16x8v*>(src + q * 8);
#pragma unroll
        for (int e = 0; e < 8; e++)
            n += residual_kept(v[e]) ? 1 : 0;
    }
    for (int o = 32; o > 0; o >>= 1)
        n += __shfl_down(n, o);
    if (L == 0)
        offsets[list + 1] = n;
}

// offsets[1..lists] hold the lists' lengths; turn them into running totals (offsets[0] = 0) and
// report the longest.  One workgroup.  A total beyond what an int holds gives offsets[lists] = -1.
__global__ __launch_bounds__(1024) void a24_residual_scan_kernel(int* __restrict__ offsets, long lists,
                                                                 int* __restrict__ longest)
{
    __shared__ long long sums[1024];
    __shared__ int most[1024];
    const long chunk = (lists + 1023) / 1024;
    const long lo = threadIdx.x * chunk, hi = lo + chunk < lists ? lo + chunk : lists;
    long long s = 0;
    int m = 0;
    for (long i = lo; i < hi; i++) {
        const int n = offsets[i + 1];
        s += n;
        m = n > m ? n : m;
    }
    sums[threadIdx.x] = s;
    most[threadIdx.x] = m;
    __syncthreads();
    for (int o = 1; o < 1024; o <<= 1) {
        const long long v = threadIdx.x >= o ? sums[threadIdx.x - o] : 0;
        const int w = threadIdx.x >= o ? most[threadIdx.x - o] : 0;
        __syncthreads();
        sums[threadIdx.x] += v;
        most[threadIdx.x] = w > most[threadIdx.x] ? w : most[threadIdx.x];
        __syncthreads();
    }
    const bool fits = sums[1023] <= 0x7fffffffLL - 64;
    long long run = threadIdx.x ? sums[threadIdx.x - 1] : 0;
    for (long i = lo; i < hi; i++) {
        run += offsets[i + 1];
        offsets[i + 1] = fits ? static_cast<int>(run) : (i + 1 == lists ? -1 : 0);
    }
    if (threadIdx.x == 0) {
        offsets[0] = 0;
        *longest = most[1023];
    }
}

// One wave (= one workgroup) per list.
__global__ __launch_bounds__(64) void a24_residual_emit_kernel(const uint16_t* __restrict__ A2, int K, int units, long lists,
                                                               const int* __restrict__ offsets, uint32_t* __restrict__ words)
{
    __shared__ uint32_t natural[kMaxListWords];  // the list in row-major order, later in its final order
    __shared__ uint32_t by_bank[kMaxListWords];  // grouped by bank, fullest bank first
    __shared__ int order[64], count_of[64], start_of[64], used[16], mine[16];
    const long list = blockIdx.x;
    const int L = threadIdx.x;
    long rb;
    int u;
    record_of_list(list, units, rb, u);
    const int row = L >> 2, c0 = (L & 3) * 32;
    const uint16_t* src = A2 + (size_t)(rb * 16 + row) * K + (size_t)u * 128 + c0;
    u16x8v v[4];
    int mine_n = 0;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        v[q] = *reinterpret_cast<const u16x8v*>(src + q * 8);
#pragma unroll
        for (int e = 0; e < 8; e++)
            mine_n += residual_kept(v[q][e]) ? 1 : 0;
    }
    int incl = mine_n;  // inclusive scan over the lanes
    for (int o = 1; o < 64; o <<= 1) {
        const int t = __shfl_up(incl, o);
        if (L >= o)
            incl += t;
    }
    const int n = __shfl(incl, 63);
    const int begin = offsets[list];
    const int total = offsets[lists];
    if (total < 0)  // the word count did not fit an int: no offset of this table means anything, nothing is written
        return;
    if (list == lists - 1)  // the padding behind the last list
        words[(size_t)total + L] = 0;
    if (n == 0 || n > kMaxListWords)  // (more than a residual can hold: not this format's input; nothing is written)
        return;
    int at = incl - mine_n;
    const bool in_order = n <= 64;  // one round: the host leaves such a list as collected
#pragma unroll
    for (int q = 0; q < 4; q++)
#pragma unroll
        for (int e = 0; e < 8; e++)
            if (residual_kept(v[q][e])) {
                const int c = c0 + q * 8 + e;
                const uint32_t address = row * 256 + ((((c >> 3) ^ row) & 15) << 4) + (c & 7) * 2;
                const uint32_t w = v[q][e] | address << 16;
                if (in_order)
                    words[(size_t)begin + at] = w;
                else
                    natural[at] = w;
                at++;
            }
    if (in_order)
        return;
    __syncthreads();
    // lane b looks after bank b: how many words, where they start among the banks sorted by
    // (count descending, bank ascending), and its words in collected order
    auto bank_of = [](uint32_t w) { return static_cast<int>(((w >> 16) >> 2) & 63); };
    int cnt = 0;
    for (int i = 0; i < n; i++)
        cnt += bank_of(natural[i]) == L ? 1 : 0;
    int rank = 0, start = 0;
    for (int b = 0; b < 64; b++) {
        const int other = __shfl(cnt, b);
        const bool before = other > cnt || (other == cnt && b < L);
        rank += before ? 1 : 0;
        start += before ? other : 0;
    }
    order[rank] = L;
    count_of[L] = cnt;
    start_of[L] = start;
    for (int i = 0, k = start; i < n; i++) {
        const uint32_t w = natural[i];
        if (bank_of(w) == L)
            by_bank[k++] = w;
    }
    __syncthreads();
    // the host's dealing, word by word (a24_pack.cpp: order_by_bank), on one lane
    if (L == 0) {
        const int rounds = (n + 63) / 64;
        for (int r = 0; r < rounds; r++)
            used[r] = 0;
        for (int i = 0; i < 64; i++) {
            const int b = order[i];
            const int c = count_of[b];
            if (c == 0)
                break;
            for (int r = 0; r < rounds; r++)
                mine[r] = 0;
            for (int j = 0; j < c; j++) {
                int best = -1, best_free = 0;
                for (int r = 0; r < rounds; r++) {
                    const int free = (r == rounds - 1 ? n - 64 * (rounds - 1) : 64) - used[r];
                    if (free > 0 && (best < 0 || mine[r] < mine[best] || (mine[r] == mine[best] && free > best_free))) {
                        best = r;
                        best_free = free;
                    }
                }
                natural[best * 64 + used[best]++] = by_bank[start_of[b] + j];
                mine[best]++;
            }
        }
    }
    __syncthreads();
    for (int i = L; i < n; i += 64)
        words[(size_t)begin + i] = natural[i];
}

}  // namespace

// A2: row-major M x K fp16 in device memory (M % 128 == 0, K % 128 == 0, checked by the caller).
// offsets: (M / 16) * (K / 128) + 1 ints; *longest: the longest list's length.
extern "C" int a24_launch_residual_offsets(void* stream, const void* A2, int M, int K, int* offsets, int* longest)
{
    const int units = K / 128;
    const long lists = static_cast<long>(M / 16) * units;
    if (lists < 1 || lists > 0x7ffffff0L)
        return static_cast<int>(hipErrorInvalidValue);
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(a24_residual_count_kernel, dim3((unsigned)((lists + 3) / 4)), dim3(256), 0, s,
                       static_cast<const uint16_t*>(A2), K, units, lists, offsets);
    hipLaunchKernelGGL(a24_residual_scan_kernel, dim3(1), dim3(1024), 0, s, offsets, lists, longest);
    return static_cast<int>(hipGetLastError());
}

// words: offsets[last] + 64 of them (the last 64 are zeroed).
extern "C" int a24_launch_residual_words(void* stream, const void* A2, int M, int K, const int* offsets, void* words)
{
    const int units = K / 128;
    const long lists = static_cast<long>(M / 16) * units;
    if (lists < 1 || lists > 0x7ffffff0L)
        return static_cast<int>(hipErrorInvalidValue);
    hipLaunchKernelGGL(a24_residual_emit_kernel, dim3((unsigned)lists), dim3(64), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t*>(A2), K, units, lists, offsets, static_cast<uint32_t*>(words));
    return static_cast<int>(hipGetLastError());
}

// A second stream per caller stream, so that the residual's Tiled-CSL kernel can run beside the 2:4
// kernel (the reference gives them two streams as well, kernel_benchmark/spmm_test.cu:459-461).
// Default priority, created on first use, kept until the process ends; at most 32 caller
// streams get one, further ones run everything on the caller's stream (*side = stream).
namespace {
struct SideStream {
    hipStream_t owner, side;
    hipEvent_t fork, join;
};
std::mutex side_mu;
SideStream side_table[32];
int side_used = 0;
}  // namespace

// Everything enqueued on `stream` so far happens before what is then enqueued on *side.
extern "C" int a24_side_begin(void* stream, void** side)
{
    hipStream_t s = static_cast<hipStream_t>(stream);
    SideStream* e = nullptr;
    {
        std::lock_guard<std::mutex> lock(side_mu);
        for (int i = 0; i < side_used && !e; i++)
            if (side_table[i].owner == s)
                e = &side_table[i];
        // Streams and events are not created while the caller's stream is being captured into a
        // graph (not a call a capture allows): such a call runs on the caller's stream alone unless
        // an earlier, eager call has already made the pair.
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (!e && hipStreamIsCapturing(s, &capturing) != hipSuccess) {
            (void)hipGetLastError();
            capturing = hipStreamCaptureStatusActive;
        }
        if (!e && side_used < 32 && capturing == hipStreamCaptureStatusNone) {
            SideStream n{s, nullptr, nullptr, nullptr};
            if (hipStreamCreateWithFlags(&n.side, hipStreamNonBlocking) != hipSuccess
                || hipEventCreateWithFlags(&n.fork, hipEventDisableTiming) != hipSuccess
                || hipEventCreateWithFlags(&n.join, hipEventDisableTiming) != hipSuccess) {
                (void)hipGetLastError();
                // whatever was made before the failure goes back: the next call tries afresh
                if (n.join)
                    (void)hipEventDestroy(n.join);
                if (n.fork)
                    (void)hipEventDestroy(n.fork);
                if (n.side)
                    (void)hipStreamDestroy(n.side);
            } else {
                side_table[side_used] = n;
                e = &side_table[side_used++];
            }
        }
    }
    if (!e) {
        *side = stream;
        return 0;
    }
    hipError_t rc = hipEventRecord(e->fork, s);
    if (rc == hipSuccess)
        rc = hipStreamWaitEvent(e->side, e->fork, 0);
    *side = e->side;
    return static_cast<int>(rc);
}

// Everything enqueued on `side` so far happens before what is then enqueued on `stream`.
extern "C" int a24_side_end(void* stream, void* side)
{
    if (side == stream)
        return 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    std::lock_guard<std::mutex> lock(side_mu);
    for (int i = 0; i < side_used; i++) {
        if (side_table[i].owner == s) {
            hipError_t rc = hipEventRecord(side_table[i].join, side_table[i].side);
            if (rc == hipSuccess)
                rc = hipStreamWaitEvent(s, side_table[i].join, 0);
            return static_cast<int>(rc);
        }
    }
    return static_cast<int>(hipErrorInvalidValue);
}
