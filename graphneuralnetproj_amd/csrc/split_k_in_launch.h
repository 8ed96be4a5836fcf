// The split-K reduction inside a launch, shared by the Tiled-CSL kernel (spmm_kernels.hip) and the
// 2:4 kernel (a24_kernels.hip): the write-through stores and memory-served loads that carry slabs
// of partial sums between workgroups, and the tail in which the last workgroup to finish a group
// of rows adds that group's slabs up.  Stands in for csrc/Reduction_Kernel.cuh:24-47 where a launch
// can do the sum itself; same order of additions, hence the same bits.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace inlaunch {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));

// Stores and loads at system scope (write through every cache level / served from memory):
// how the slabs of partial sums travel between workgroups of one launch without cache
// maintenance.  A device-wide fence would write back and invalidate the whole L2 of the XCD,
// which the weight stream lives in.  Relaxed 64-bit atomics rather than inline assembly: the
// compiler then also keeps the store data registers untouched for as long as the hardware
// needs them (an assembly store's data was seen overwritten by the next VALU instruction).
__device__ __forceinline__ void store_through(_Float16* p, half4 v)
{
    __hip_atomic_store(reinterpret_cast<uint64_t*>(p), __builtin_bit_cast(uint64_t, v), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_SYSTEM);
}
__device__ __forceinline__ void store_through(_Float16* p, _Float16 v)
{
    __hip_atomic_store(reinterpret_cast<uint16_t*>(p), __builtin_bit_cast(uint16_t, v), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_SYSTEM);
}
__device__ __forceinline__ half8 load_through(const _Float16* p)
{
    typedef uint64_t u64x2 __attribute__((ext_vector_type(2)));
    u64x2 w;
    w[0] = __hip_atomic_load(reinterpret_cast<const uint64_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    w[1] = __hip_atomic_load(reinterpret_cast<const uint64_t*>(p) + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    return __builtin_bit_cast(half8, w);
}

// Fused split-K reduction, called by every thread of a workgroup that has just written its slab
// of partial sums (through to memory) for rows [row0, row0 + nrows): the last of the Split_K
// workgroups that share those rows adds the slabs up, in slab order like the separate kernel
// (csrc/Reduction_Kernel.cuh:36-46), so both paths give the same bits.  `counter` is the rows'
// arrival count in device memory (zero between calls), `flag` one free LDS word, nthreads the
// number of threads of the workgroup that are still there (the first nthreads).
// Bits 8 and up of `relu` count further slabs that an earlier launch on the same stream left right
// behind this launch's own Split_K (the 2:4 part's partial sums); they are added after them.
// row_major: slabs and C are [M][N] (the rows' block is one contiguous run of nrows * N values;
// ldc is not used) instead of one M vector per token.
// The sum moves eight rows at a time: nrows, M and row0 must be multiples of 8 (the launchers check M).
__device__ __forceinline__ void fused_reduction_tail(const _Float16* __restrict__ slabs, _Float16* __restrict__ C, int M,
                                                     int N, int ldc, int split_k, int relu, int row0, int nrows,
                                                     unsigned int* counter, unsigned int* flag, int nthreads,
                                                     bool row_major)
{
    // This workgroup's partial sums have reached memory before it is counted.  The hardware side
    // of that is the wait (the write-through stores are acknowledged at the coherence point); the
    // two workgroup-scope fences say the same to the compiler, which may then move neither the
    // slab stores below the counting nor the slab loads above it.  At workgroup scope a fence is
    // waits only: no cache is written back or invalidated (a wider fence would flush the L2 that
    // the weight stream lives in).
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0), on top of what the compiler tracks itself
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    if (threadIdx.x == 0)
        *flag = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    if (*flag != static_cast<unsigned int>(split_k - 1))
        return;
    split_k += relu >> 8;
    relu &= 0xff;
    nrows = nrows < M - row0 ? nrows : M - row0;
    const int per_tok = nrows / 8;
    const int total = per_tok * N;  // runs of eight rows to sum
    const size_t slab = (size_t)M * N;
    // Every load is served from memory, and a thread can only add what has arrived.  A thread with
    // several runs of eight rows (64 tokens: four per thread) keeps four slabs of four runs in flight,
    // sixteen 16-byte loads, so that its trips to memory are ceil(split_k / 4) in all rather than per
    // run (9216 x 9216, 64 tokens, three batches: 28.9 -> 26.2 us).  Each element's slabs are still
    // added in slab order.  (Sixteen slabs of one run at a time, for the threads that have a single
    // run, measured 2 to 3 % slower than four even where there are only four.)
    auto sum_runs = [&](auto it_c, auto g_c) __attribute__((always_inline)) {
        constexpr int IT = decltype(it_c)::value, G = decltype(g_c)::value;
        for (int c0 = threadIdx.x; c0 < total; c0 += nthreads * IT) {
            size_t at[IT];
            float sum[IT][8];
#pragma unroll
            for (int i = 0; i < IT; i++) {
                const int c = c0 + i * nthreads < total ? c0 + i * nthreads : c0;  // a run past the end repeats the first
                const int tok = c / per_tok, m8 = c - tok * per_tok;
                at[i] = row_major ? (size_t)row0 * N + (size_t)c * 8 : (size_t)tok * M + row0 + m8 * 8;
#pragma unroll
                for (int j = 0; j < 8; j++)
                    sum[i][j] = 0.f;
            }
            int sidx = 0;
            for (; sidx + G <= split_k; sidx += G) {
                half8 w[IT][G];
#pragma unroll
                for (int u = 0; u < G; u++)
#pragma unroll
                    for (int i = 0; i < IT; i++)
                        w[i][u] = load_through(slabs + at[i] + (size_t)(sidx + u) * slab);
#pragma unroll
                for (int u = 0; u < G; u++)
#pragma unroll
                    for (int i = 0; i < IT; i++)
#pragma unroll
                        for (int j = 0; j < 8; j++)
                            sum[i][j] += static_cast<float>(w[i][u][j]);
            }
            for (; sidx < split_k; sidx++) {
                half8 w[IT];
#pragma unroll
                for (int i = 0; i < IT; i++)
                    w[i] = load_through(slabs + at[i] + (size_t)sidx * slab);
#pragma unroll
                for (int i = 0; i < IT; i++)
#pragma unroll
                    for (int j = 0; j < 8; j++)
                        sum[i][j] += static_cast<float>(w[i][j]);
            }
#pragma unroll
            for (int i = 0; i < IT; i++) {
                const int c = c0 + i * nthreads;
                if (c >= total)
                    break;
                half8 o;
#pragma unroll
                for (int j = 0; j < 8; j++)
                    o[j] = static_cast<_Float16>(relu ? fmaxf(sum[i][j], 0.f) : sum[i][j]);
                const int tok = c / per_tok, m8 = c - tok * per_tok;
                *reinterpret_cast<half8*>(C + (row_major ? at[i] : (size_t)tok * ldc + row0 + m8 * 8)) = o;
            }
        }
    };
    if (total <= nthreads)
        sum_runs(std::integral_constant<int, 1>{}, std::integral_constant<int, 4>{});
    else
        sum_runs(std::integral_constant<int, 4>{}, std::integral_constant<int, 4>{});
    if (threadIdx.x == 0)
        *counter = 0;  // ready for the next call
}

}  // namespace inlaunch
