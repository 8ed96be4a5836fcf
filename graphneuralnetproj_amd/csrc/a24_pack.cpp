// Host side of the 2:4 + residual path: the reference's split of a weight into a part for
// sparse matrix cores and a Tiled-CSL residual, and the packer of the first part's records.
#include <algorithm>
#include <atomic>
#include <cstdlib>
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

namespace {

// Orders one list's words so that every round of 64 (one word per lane; the last round may be
// partial) spreads over the 64 LDS banks: banks are taken fullest first, and each of a bank's
// words goes to the round that holds the fewest words of that bank so far and still has room
// (the emptier round on a tie).
void order_by_bank(std::vector<uint32_t>& list, std::vector<uint32_t>& tmp)
{
    const int n = static_cast<int>(list.size());
    const int rounds = (n + 63) / 64;
    if (rounds <= 1)
        return;
    auto bank_of = [](uint32_t w) { return static_cast<int>(((w >> 16) >> 2) & 63); };
    int count[64] = {};
    for (uint32_t w : list)
        count[bank_of(w)]++;
    int order[64];
    for (int b = 0; b < 64; b++)
        order[b] = b;
    std::stable_sort(order, order + 64, [&](int a, int b) { return count[a] > count[b]; });
    int start[64], at = 0;  // where each bank's words begin in the bank-sorted sequence
    for (int i = 0; i < 64; i++) {
        start[order[i]] = at;
        at += count[order[i]];
    }
    tmp.assign(n, 0);
    int fill[64];
    for (int b = 0; b < 64; b++)
        fill[b] = start[b];
    for (uint32_t w : list)
        tmp[fill[bank_of(w)]++] = w;
    std::vector<int> used(rounds, 0), mine(rounds);
    for (int i = 0; i < 64; i++) {
        const int b = order[i];
        std::fill(mine.begin(), mine.end(), 0);
        for (int j = 0; j < count[b]; j++) {
            int best = -1, best_free = 0;
            for (int r = 0; r < rounds; r++) {
                const int free = (r == rounds - 1 ? n - 64 * (rounds - 1) : 64) - used[r];
                if (free > 0 && (best < 0 || mine[r] < mine[best] || (mine[r] == mine[best] && free > best_free))) {
                    best = r;
                    best_free = free;
                }
            }
            list[best * 64 + used[best]++] = tmp[start[b] + j];
            mine[best]++;
        }
    }
}

}  // namespace

int pack_residual(const uint16_t* A2, int M, int K, uint32_t** words, int** offsets, int* longest)
{
    if (!A2 || !words || !offsets || !longest)
        return kErrNullPointer;
    if (M <= 0 || K <= 0 || M % (kRows * kGroupBlocks) != 0 || K % kUnitCols != 0)
        return kErrBadShape;
    const int units = K / kUnitCols;
    const long blocks = M / kRows;
    const long records = blocks * units;
    if (records + 1 > 0x7fffffffL)
        return kErrBadShape;
    int* off = static_cast<int*>(std::malloc((records + 1) * sizeof(int)));
    if (!off)
        return kErrNoMemory;
    // pass 1: list lengths, by list number
    parallel_for(blocks, [=](long b0, long b1) {
        for (long rb = b0; rb < b1; rb++)
            for (int u = 0; u < units; u++) {
                int n = 0;
                for (int r = 0; r < kRows; r++) {
                    const uint16_t* row = A2 + (rb * kRows + r) * static_cast<long>(K) + static_cast<long>(u) * kUnitCols;
                    for (int c = 0; c < kUnitCols; c++)
                        n += kept(row[c]) ? 1 : 0;
                }
                off[record_index(rb, u, units) + 1] = n;
            }
    });
    off[0] = 0;
    int most = 0;
    long total = 0;
    for (long i = 1; i <= records; i++) {
        most = off[i] > most ? off[i] : most;
        total += off[i];
        if (total > 0x7fffffffL - kListPadWords) {
            std::free(off);
            return kErrBadShape;
        }
        off[i] = static_cast<int>(total);
    }
    uint32_t* out = static_cast<uint32_t*>(std::malloc((total + kListPadWords) * sizeof(uint32_t)));
    if (!out) {
        std::free(off);
        return kErrNoMemory;
    }
    std::memset(out + total, 0, kListPadWords * sizeof(uint32_t));
    // pass 2: the words
    parallel_for(blocks, [=](long b0, long b1) {
        std::vector<uint32_t> list, tmp;
        for (long rb = b0; rb < b1; rb++)
            for (int u = 0; u < units; u++) {
                list.clear();
                for (int r = 0; r < kRows; r++) {
                    const uint16_t* row = A2 + (rb * kRows + r) * static_cast<long>(K) + static_cast<long>(u) * kUnitCols;
                    for (int c = 0; c < kUnitCols; c++)
                        if (kept(row[c]))
                            list.push_back(row[c] | residual_address(r, c) << 16);
                }
                order_by_bank(list, tmp);
                if (!list.empty())  // (an empty vector's data() may be null, which memcpy must not be given)
                    std::memcpy(out + off[record_index(rb, u, units)], list.data(), list.size() * sizeof(uint32_t));
            }
    });
    *words = out;
    *offsets = off;
    *longest = most;
    return static_cast<int>(records + 1);
}

}  // namespace a24
