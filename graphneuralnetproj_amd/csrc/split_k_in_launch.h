// The split-K reduction inside a launch, shared by the Tiled-CSL kernel (spmm_kernels.hip) and the
// 2:4 kernel (a24_kernels.hip): the write-through stores and memory-served loads that carry slabs
// of partial sums between workgroups, and the tail in which the last workgroup to finish a group
// of rows adds that group's slabs up.  Stands in for csrc/Reduction_Kernel.cuh:24-47 where a launch
// can do the sum itself; same order of additions, hence the same bits.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

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
    const size_t slab = (size_t)M * N;
    for (int c = threadIdx.x; c < per_tok * N; c += nthreads) {
        const int tok = c / per_tok, m8 = c - tok * per_tok;
        const size_t at = row_major ? (size_t)row0 * N + (size_t)c * 8 : (size_t)tok * M + row0 + m8 * 8;
        const _Float16* w0 = slabs + at;
        float sum[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        int sidx = 0;
        for (; sidx + 4 <= split_k; sidx += 4) {
            half8 w[4];
#pragma unroll
            for (int u = 0; u < 4; u++)
                w[u] = load_through(w0 + (size_t)(sidx + u) * slab);
#pragma unroll
            for (int u = 0; u < 4; u++)
#pragma unroll
                for (int j = 0; j < 8; j++)
                    sum[j] += static_cast<float>(w[u][j]);
        }
        for (; sidx < split_k; sidx++) {
            const half8 w = load_through(w0 + (size_t)sidx * slab);
#pragma unroll
            for (int j = 0; j < 8; j++)
                sum[j] += static_cast<float>(w[j]);
        }
        half8 o;
#pragma unroll
        for (int j = 0; j < 8; j++)
            o[j] = static_cast<_Float16>(relu ? fmaxf(sum[j], 0.f) : sum[j]);
        *reinterpret_cast<half8*>(C + (row_major ? at : (size_t)tok * ldc + row0 + m8 * 8)) = o;
    }
    if (threadIdx.x == 0)
        *counter = 0;  // ready for the next call
}

}  // namespace inlaunch
