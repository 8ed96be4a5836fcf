// Host side of the 2:4 + residual path: the reference's split of a weight into a part for
// sparse matrix cores and a Tiled-CSL residual, and the packer of the first part's records.
#include <atomic>
#include <cstring>
#include <thread>
#include <vector>

#include "a24_format.h"

namespace a24 {
namespace {

// binary16 -> "compares unequal to zero as a float": everything but +0 and -0 (NaN included),
// which is what `__half2float(x) != 0.0f` gives (kernel_benchmark/spmm_decompose.h:26).
inline bool kept(uint16_t h)
{
    return (h & 0x7fffu) != 0;
}

int host_threads(long work_items)
{
    unsigned hw = std::thread::hardware_concurrency();
    long t = hw ? hw : 1;
    if (t > 16)
        t = 16;
    if (t > work_items)
        t = work_items;
    return t < 1 ? 1 : static_cast<int>(t);
}

template<typename F>
void parallel_for(long n, F body)
{
    const int t = host_threads(n);
    if (t <= 1) {
        body(0L, n);
        return;
    }
    std::vector<std::thread> pool;
    for (int i = 0; i < t; i++)
        pool.emplace_back([=] { body(n * i / t, n * (i + 1) / t); });
    for (auto& th : pool)
        th.join();
}

}  // namespace

void decompose(const uint16_t* A, uint16_t* A1, uint16_t* A2, long length)
{
    const long groups = length / 4;
    parallel_for(groups, [=](long g0, long g1) {
        for (long g = g0; g < g1; g++) {
            int taken = 0;
            for (int e = 0; e < 4; e++) {
                const uint16_t v = A[g * 4 + e];
                const bool k = kept(v);
                A1[g * 4 + e] = (k && taken < 2) ? v : 0;
                A2[g * 4 + e] = (k && taken >= 2) ? v : 0;
                taken += k ? 1 : 0;
            }
        }
    });
    for (long i = groups * 4; i < length; i++)  // the reference asserts length % 4 == 0
        A1[i] = A2[i] = 0;
}

int pack(const uint16_t* A1, int M, int K, uint8_t* packed)
{
    if (!A1 || !packed)
        return kErrNullPointer;
    if (M <= 0 || K <= 0 || M % (kRows * kGroupBlocks) != 0 || K % kUnitCols != 0)
        return kErrBadShape;
    const int units = K / kUnitCols;
    const long blocks = M / kRows;
    std::atomic<int> bad{0};
    std::atomic<int>* bad_flag = &bad;
    parallel_for(blocks, [=](long b0, long b1) {
        for (long rb = b0; rb < b1; rb++) {
            for (int u = 0; u < units; u++) {
                uint8_t* rec = packed + record_index(rb, u, units) * kRecordBytes;
                for (int L = 0; L < 64; L++) {
                    const uint16_t* row = A1 + (rb * kRows + L % 16) * static_cast<long>(K) + static_cast<long>(u) * kUnitCols;
                    uint32_t word = 0;
                    for (int s = 0; s < 4; s++) {
                        for (int half = 0; half < 2; half++) {  // the lane's two groups of four in this step
                            const uint16_t* grp = row + s * 32 + (L / 16) * 8 + half * 4;
                            int pos[2], n = 0;
                            for (int e = 0; e < 4; e++) {
                                if (kept(grp[e])) {
                                    if (n < 2)
                                        pos[n] = e;
                                    n++;
                                }
                            }
                            if (n > 2) {
                                bad_flag->store(1, std::memory_order_relaxed);
                                n = 2;
                            }
                            uint16_t val[2] = {0, 0};
                            if (n == 2) {
                                val[0] = grp[pos[0]];
                                val[1] = grp[pos[1]];
                            } else if (n == 1) {
                                if (pos[0] == 3) {  // the free slot goes before it
                                    val[1] = grp[3];
                                    pos[0] = 2;
                                    pos[1] = 3;
                                } else {
                                    val[0] = grp[pos[0]];
                                    pos[1] = 3;
                                }
                            } else {
                                pos[0] = 0;
                                pos[1] = 1;
                            }
                            for (int t = 0; t < 2; t++) {
                                const int j = half * 2 + t;
                                std::memcpy(rec + (s / 2) * 1024 + L * 16 + ((s % 2) * 4 + j) * 2, &val[t], 2);
                                word |= static_cast<uint32_t>(pos[t]) << (8 * s + 2 * j);
                            }
                        }
                    }
                    std::memcpy(rec + kIndexOffset + L * 4, &word, 4);
                }
            }
        }
    });
    return bad.load() ? kErrNotTwoOfFour : 0;
}

}  // namespace a24
