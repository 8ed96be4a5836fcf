// Deterministic synthetic inputs for tests and benchmarks.  Every element is a
// pure function of (seed, stream, element index), so any host produces the same
// bits regardless of thread count or evaluation order.
//
//   weights     element (m,k) is kept with probability p_row(m); a kept value is
//               fp16_rn(0.02 * z), z standard normal (Box-Muller).  Uniform
//               sparsity: p_row = 1 - sparsity.  Row skewed: p_row =
//               min(1, (1 - sparsity) * beta / 0.2), beta ~ Beta(2, 8) (mean 0.2)
//               drawn per row as X / (X + Y) with X ~ Gamma(2), Y ~ Gamma(8).
//   activations fp16_rn(z).
//
// This mirrors the shape of the reference's test data (fake Bernoulli sparsity,
// end2end_inference/ft_tools/huggingface_opt_convert_Phase2.py:68-71) with
// normally distributed magnitudes instead of its constant 1.0 weights
// (kernel_benchmark/spmm_test_utils.h:108-141).
//
// The harness's own value pattern is there as well (synth_harness_*): every kept
// weight exactly 1.0 and every activation one of -5, -3, -1, 1, 3
// (kernel_benchmark/spmm_test_utils.h:111-141), with the keep decisions of the
// generator above.  Every product and every partial sum is then a small integer,
// exact in fp32, so a whole output can be checked bit for bit.
#include <atomic>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <thread>
#include <vector>

#include "tiled_csl_format.h"

namespace tcsl {

namespace {

inline uint64_t mix(uint64_t x)
{
    x += 0x9e3779b97f4a7c15ull;
    x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ull;
    x = (x ^ (x >> 27)) * 0x94d049bb133111ebull;
    return x ^ (x >> 31);
}

// uniform in (0, 1), 53 bits
inline double unit(uint64_t seed, uint64_t stream, uint64_t index)
{
    const uint64_t r = mix(mix(seed ^ (stream * 0xd1342543de82ef95ull)) + index);
    return (static_cast<double>(r >> 11) + 0.5) * (1.0 / 9007199254740992.0);
}

inline float normal(uint64_t seed, uint64_t stream, uint64_t index)
{
    const double u1 = unit(seed, stream, index), u2 = unit(seed, stream + 1, index);
    return static_cast<float>(std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2));
}

// binary32 -> binary16, round to nearest even
inline uint16_t to_half(float f)
{
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint16_t sign = static_cast<uint16_t>((x >> 16) & 0x8000u);
    x &= 0x7fffffffu;
    if (x > 0x7f800000u)
        return sign | 0x7e00u;
    if (x >= 0x47800000u)
        return sign | 0x7c00u;
    if (x < 0x33000000u)
        return sign;
    const int e = static_cast<int>(x >> 23) - 127;
    const uint32_t m = (x & 0x7fffffu) | 0x800000u;
    const int drop = e < -14 ? 13 + (-14 - e) : 13;
    uint32_t keep = m >> drop;
    const uint32_t rest = m & ((1u << drop) - 1u), mid = 1u << (drop - 1);
    if (rest > mid || (rest == mid && (keep & 1u)))
        keep++;
    uint32_t out = e < -14 ? keep : (static_cast<uint32_t>(e + 14) << 10) + keep;
    if (out > 0x7c00u)
        out = 0x7c00u;
    return sign | static_cast<uint16_t>(out);
}

template<typename F>
void for_rows(long rows, F fn)
{
    int nt = static_cast<int>(std::thread::hardware_concurrency());
    nt = nt < 1 ? 1 : (nt > 16 ? 16 : nt);
    if (rows < nt)
        nt = static_cast<int>(rows < 1 ? 1 : rows);
    std::atomic<long> next{0};
    std::vector<std::thread> pool;
    for (int t = 0; t < nt; t++)
        pool.emplace_back([&] {
            for (;;) {
                const long r = next.fetch_add(1);
                if (r >= rows)
                    return;
                fn(r);
            }
        });
    for (auto& th : pool)
        th.join();
}

}  // namespace

namespace {
void weights(uint16_t* A, int M, int K, double sparsity, int row_skewed, uint64_t seed, bool ones);
}

void synth_weights(uint16_t* A, int M, int K, double sparsity, int row_skewed, uint64_t seed)
{
    weights(A, M, K, sparsity, row_skewed, seed, false);
}

void synth_harness_weights(uint16_t* A, int M, int K, double sparsity, int row_skewed, uint64_t seed)
{
    weights(A, M, K, sparsity, row_skewed, seed, true);
}

void synth_harness_activations(uint16_t* B, long count, uint64_t seed)
{
    // (rand() % 5) / 5 - 0.5) * 10 of the reference: -5, -3, -1, 1, 3 as fp16 bit patterns
    static const uint16_t kValues[5] = {0xc500, 0xc200, 0xbc00, 0x3c00, 0x4200};
    const long chunk = 4096;
    for_rows((count + chunk - 1) / chunk, [&](long c) {
        const long end = (c + 1) * chunk < count ? (c + 1) * chunk : count;
        for (long i = c * chunk; i < end; i++)
            B[i] = kValues[mix(mix(seed ^ (5 * 0xd1342543de82ef95ull)) + static_cast<uint64_t>(i)) % 5];
    });
}

namespace {
void weights(uint16_t* A, int M, int K, double sparsity, int row_skewed, uint64_t seed, bool ones)
{
    const double keep_mean = 1.0 - sparsity;
    for_rows(M, [&](long m) {
        double p = keep_mean;
        if (row_skewed) {
            double x = 0.0, y = 0.0;  // Gamma(k) = -ln(product of k uniforms)
            for (int i = 0; i < 2; i++)
                x -= std::log(unit(seed, 10, static_cast<uint64_t>(m) * 16 + i));
            for (int i = 0; i < 8; i++)
                y -= std::log(unit(seed, 10, static_cast<uint64_t>(m) * 16 + 2 + i));
            p = keep_mean * (x / (x + y)) / 0.2;
            if (p > 1.0)
                p = 1.0;
        }
        uint16_t* row = A + static_cast<size_t>(m) * K;
        for (int k = 0; k < K; k++) {
            const uint64_t idx = static_cast<uint64_t>(m) * static_cast<uint64_t>(K) + k;
            row[k] = unit(seed, 1, idx) < p ? (ones ? uint16_t(0x3c00) : to_half(0.02f * normal(seed, 2, idx))) : 0;
        }
    });
}
}  // namespace

void synth_activations(uint16_t* B, long count, uint64_t seed)
{
    const long chunk = 4096;
    for_rows((count + chunk - 1) / chunk, [&](long c) {
        const long end = (c + 1) * chunk < count ? (c + 1) * chunk : count;
        for (long i = c * chunk; i < end; i++)
            B[i] = to_half(normal(seed, 4, static_cast<uint64_t>(i)));
    });
}

}  // namespace tcsl
