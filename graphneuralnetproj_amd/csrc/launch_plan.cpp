// Picks the launch shape of the main kernel: which of its two workgroup layouts, how many
// waves per workgroup, and (for SpMM_SuggestSplitK) how many split-K batches.
//
// The reference fixes one block shape and tunes Split_K per matrix by hand
// (kernel_benchmark/benchmark.sh:15, end2end_inference/ft_tools/huggingface_opt_convert_Phase2.py:20).
// Here the choice is made by a small analytic model of an MI355X (256 compute units, one
// workgroup slot set per unit limited by LDS and registers), fitted to the tuner's logs
// (graphneuralnetproj_amd/tune_plans.py) on OPT-30B/66B/175B layer shapes at 80 % sparsity,
// backed by a table of the measured optimum for those shapes themselves.
#include "launch_plan.h"

#include <cmath>

#include "tiled_csl_format.h"

namespace tcsl {

namespace {

constexpr long kLdsPerCu = 160 * 1024;
constexpr long kTileLds = 16384;   // dense fp16 image of one 128x64 tile
constexpr int kCUs = 256;

// Fitted constants (microseconds, bytes per microsecond): least squares on the logarithm of
// estimate / measurement over every plan within 30 % of its shape's best in the tuner's logs
// (24 shapes x 4 token counts at 80 % sparsity) and over the same grid, with the reduction kernel behind
// the K-splitting launches as well, on ten small matrices of 8 to 96 tile rows (4632 points in all),
// checked on ten shapes the fit never saw.
constexpr double kLaunchUs = 2.985;         // fixed cost of the main kernel
constexpr double kTileBytes = kTileBytesAt80;  // one tile at 80 % sparsity: what the constants below were fitted on
constexpr double kChipBytesPerUs = 10.95e6; // whole-chip stream rate
constexpr double kCuBytesPerUs = 65.79e3;   // what one compute unit's vector memory path can pull
constexpr double kFragWeight = 0.494;       // weight of a tile's activation fragments (2 KiB per 16 tokens) on that path ...
constexpr double kFragUnshared = 0.284;     // ... of which the row-sharing waves of a workgroup share the rest through the L1
constexpr double kMfmaTileUs = 0.201;       // serial MFMA + LDS time per tile and 16-token block
constexpr double kRoundUs = 2.885;          // start-up and drain of one round of workgroups
constexpr double kNorm = 1.386;             // exponent that blends the three bounds (close to a sum)
constexpr double kCrowdPenalty = 0.0593;    // per resident wave above kCrowdWaves on a unit
constexpr double kCrowdWaves = 4.0;
constexpr double kModeKPenalty = 0.0474;    // mode 1: no sharing of fragments, reduction in LDS
constexpr double kReduceUs = 2.566;         // fixed cost of the reduction as a second kernel
constexpr double kFusedReduceUs = 0.712;    // ... and inside the main kernel (mode 1), where the last workgroup of a
constexpr double kFusedSlabUs = 0.028;      //     tile row pulls Split_K slabs of 128 x N values alone: a term per slab
constexpr double kFusedSlabTokenUs = 0.00694;  //  and one per slab and token
constexpr double kReduceBytesPerUs = 5.989e6;

int column_blocks(int N)
{
    return N <= 16 ? 1 : N / 16;
}

int max_waves(int N)
{
    return N <= 32 ? 8 : 4;  // registers: two waves per SIMD up to N = 32, one at N = 64
}

// Measured optima for the layer shapes of OPT-30B and OPT-66B, {M, K, N, Split_K, mode, waves,
// stage_b}: one table per sparsity the benchmark names.  A caller that knows the weight's bytes
// gets its Split_K from the table of the nearest density; a call, which knows only (M, N, K,
// Split_K), takes the launch shape of whichever table holds that Split_K for the shape (80 %
// first), so the Split_K that a converter stored carries the choice to the run.  A shape's first
// row is its measured best; further rows of the same (M, K, N) hold the best launch shape for
// other Split_K values a caller may fix (the benchmark's sweep of 1, 2, 4, 7 on the attention
// projections; tune_plans.py --split-k).
struct Tuned {
    int M, K, N, split_k, mode, waves, stage_b;
    int separate_reduction = 0;  // an eighth value in a row: mode 1 with the reduction kernel
};
constexpr Tuned kTuned80[] = {
#include "tuned_plans.inc"
};
constexpr Tuned kTuned70[] = {
#include "tuned_plans_70.inc"
};
constexpr Tuned kTuned90[] = {
#include "tuned_plans_90.inc"
};

// 0: the 80 % table (also for an unknown density), 1: 70 %, 2: 90 %; boundaries at 75 % and 85 % sparsity
int density_table(double tile_bytes)
{
    if (!(tile_bytes > 0.0))
        return 0;
    return tile_bytes > 1.25 * kTileBytes ? 1 : tile_bytes < 0.75 * kTileBytes ? 2 : 0;
}

template<int Rows>
const Tuned* find_in(const Tuned (&table)[Rows], int M, int N, int K, int split_k)
{
    for (const Tuned& t : table)
        if (t.M == M && t.K == K && t.N == N && (split_k == 0 || t.split_k == split_k))
            return &t;
    return nullptr;
}

// split_k == 0: any.  which = 0, 1, 2 as density_table(); -1: every table, the 80 % one first, then 70 %, then 90 %
const Tuned* find_tuned(int M, int N, int K, int split_k, int which)
{
    const Tuned* t = nullptr;
    // (The 90 % table comes last: a K-splitting launch of a sparse weight picks its number of
    // streaming waves per tile row in the kernel, so that table's wave counts say little, while
    // the denser tables' counts are what dense tile rows run with.)
    if (which == 0 || which < 0)
        t = find_in(kTuned80, M, N, K, split_k);
    if (!t && (which == 1 || which < 0))
        t = find_in(kTuned70, M, N, K, split_k);
    if (!t && (which == 2 || which < 0))
        t = find_in(kTuned90, M, N, K, split_k);
    return t;
}

}  // namespace

bool complete_plan(int N, int K, int split_k, bool row_major, LaunchPlan& p)
{
    if (N != 8 && N != 16 && N != 32 && N != 64)
        return false;
    if (split_k < 1 || p.waves < 1 || p.waves > max_waves(N))
        return false;
    const int nb = column_blocks(N);
    const long nkb = K / kTileCols;
    const long tiles = (nkb - 1) / split_k + 1;  // tiles of the longest batch
    long lds = p.waves * kTileLds;
    if (row_major) {
        if (p.stage_b)
            return false;
        lds += static_cast<long>(p.waves) * N * 128;  // one tile's activations per wave, being transposed
    }
    if (p.mode == 0) {
        if (p.stage_b == 1) {  // the batch's whole slice, up to 16 tokens
            if (nb != 1)
                return false;
            lds += tiles * (N == 8 ? 8 : 16) * 128;
        } else if (p.stage_b == 2) {  // one tile at a time through two buffers, 32 and 64 tokens
            if (row_major || !((N == 32 && (p.waves == 4 || p.waves == 8)) || (N == 64 && p.waves == 4)))
                return false;
            lds += 2L * N * 128;
        } else if (p.stage_b != 0) {
            return false;
        }
    } else if (p.mode == 1) {
        if (p.stage_b)
            return false;
        const long red = 8L * p.waves * nb * 1024;  // fp32 accumulators of all waves
        if (red > lds)
            lds = red;
    } else {
        return false;
    }
    if (lds > kLdsPerCu)
        return false;
    p.lds_bytes = static_cast<unsigned>(lds);
    return true;
}

double plan_cost_us(int M, int N, int K, int split_k, const LaunchPlan& p, double tile_bytes)
{
    if (!(tile_bytes > 0.0))
        tile_bytes = kTileBytes;
    const long row_tiles = M / kTileRows;
    const long nkb = K / kTileCols;
    const int nb = column_blocks(N);
    const int W = p.waves;
    const long batch_tiles = (nkb - 1) / split_k + 1;
    long wgs, t;  // workgroups; tiles per wave
    if (p.mode == 0) {
        wgs = (row_tiles + W - 1) / W * split_k;
        t = batch_tiles;
    } else {
        wgs = row_tiles * split_k;
        t = (batch_tiles + W - 1) / W;
    }
    long fit = kLdsPerCu / (p.lds_bytes ? p.lds_bytes : 1);
    if (fit > max_waves(N) / W)
        fit = max_waves(N) / W;
    if (fit < 1 || (p.mode == 1 && N <= 32))
        fit = 1;  // (a K-splitting plan is launched with eight waves: one workgroup per compute unit)
    const long slots = kCUs * fit;
    // activation fragments of one tile as the unit's vector memory path sees them: from the L2 per wave
    // in the K-splitting layout, partly shared between the waves of a row-sharing workgroup, half as
    // heavy when the waves hand each other the tile through LDS, absent with the staged slice
    double frag = kFragWeight * 2048.0 * nb * (N == 8 ? 0.5 : 1.0);
    if (p.mode == 0)
        frag *= kFragUnshared + (1.0 - kFragUnshared) / W;
    if (p.stage_b == 1)
        frag = 0.0;
    else if (p.stage_b == 2)
        frag *= 0.5;
    const double tau_chip = tile_bytes / kChipBytesPerUs;
    const double tau_cu = (tile_bytes + frag) / kCuBytesPerUs;
    const double tau_wave = kMfmaTileUs * nb;
    double total = kLaunchUs;
    for (long left = wgs; left > 0;) {
        const long n = left < slots ? left : slots;
        left -= n;
        const long per_cu = (n + kCUs - 1) / kCUs;
        const double crowd = static_cast<double>(per_cu * W) - kCrowdWaves;
        const double chip = static_cast<double>(n) * W * t * tau_chip * (1.0 + (crowd > 0 ? kCrowdPenalty * crowd : 0.0));
        const double lat = kRoundUs + t * tau_wave;
        const double cu = static_cast<double>(per_cu) * W * t * tau_cu;
        total += std::pow(std::pow(chip, kNorm) + std::pow(lat, kNorm) + std::pow(cu, kNorm), 1.0 / kNorm);
    }
    if (p.mode == 1)
        total *= 1.0 + kModeKPenalty;
    if (split_k > 1) {
        const bool in_launch = p.mode == 1 && !p.separate_reduction;
        total += (in_launch ? kFusedReduceUs + split_k * (kFusedSlabUs + kFusedSlabTokenUs * N) : kReduceUs) +
                 (2.0 * split_k + 1.0) * M * N * 2.0 / kReduceBytesPerUs;
    }
    return total;
}

LaunchPlan plan_launch(int M, int N, int K, int split_k, bool row_major, double* cost_us, double tile_bytes)
{
    // a measured optimum with this Split_K: of the weight's own density if the caller gave it, else of any
    if (const Tuned* t = find_tuned(M, N, K, split_k, tile_bytes > 0.0 ? density_table(tile_bytes) : -1)) {
        // (row-major activations are not staged per batch: every wave keeps its own tile of them in
        // LDS, and the row-sharing shapes measure as fast that way as the staged column-major ones)
        LaunchPlan p{t->mode, t->waves, row_major ? 0 : t->stage_b, 0};
        p.separate_reduction = t->separate_reduction != 0;
        if (complete_plan(N, K, split_k, row_major, p)) {
            if (cost_us)
                *cost_us = plan_cost_us(M, N, K, split_k, p, tile_bytes);
            return p;
        }
    }
    LaunchPlan best{0, 1, 0, static_cast<unsigned>(kTileLds)};
    double best_cost = -1.0;
    for (int mode = 0; mode <= 1; mode++)
        for (int w = 1; w <= max_waves(N); w++)
            for (int stage = 0; stage <= (mode == 0 ? 1 : 0); stage++) {
                // Measured on 24 shapes x 4 token counts: where the K-splitting layout wins it
                // does so with four streaming waves, one per SIMD, or within 2 % of that; the
                // cost model's own preference among wave counts is not that sharp.
                if (mode == 1 && w != 4)
                    continue;
                // The row-sharing layout is only considered in the shapes the tuner measures and
                // the constants were fitted on: 5..8 waves up to 16 tokens, the batch's activation
                // slice staged in LDS or its fragments from the L2 (tried first); fragments from
                // the L2 above, with 4 waves at 32 tokens and 1 to 4 at 64 (the model cannot rank the
                // other wave counts of 32 tokens: with them allowed it picks worse).
                if (mode == 0 && (N <= 16 ? w < 5 : (stage || (N == 32 && w != 4))))
                    continue;
                LaunchPlan p{mode, w, row_major ? 0 : stage, 0};
                if (!complete_plan(N, K, split_k, row_major, p))
                    continue;
                // the K-splitting layout adds its slabs up inside the launch or leaves them to the
                // reduction kernel, whichever the model prices lower (many batches, many tokens: the kernel)
                for (int separate = 0; separate <= (mode == 1 && split_k > 1 ? 1 : 0); separate++) {
                    p.separate_reduction = separate != 0;
                    const double c = plan_cost_us(M, N, K, split_k, p, tile_bytes);
                    if (best_cost < 0 || c < best_cost) {
                        best = p;
                        best_cost = c;
                    }
                }
            }
    if (cost_us)
        *cost_us = best_cost;
    return best;
}

int suggest_split_k(int M, int N, int K, LaunchPlan* plan, double tile_bytes)
{
    if (const Tuned* t = find_tuned(M, N, K, 0, density_table(tile_bytes))) {
        LaunchPlan p{t->mode, t->waves, t->stage_b, 0};
        p.separate_reduction = t->separate_reduction != 0;
        if (complete_plan(N, K, t->split_k, false, p)) {
            if (plan)
                *plan = p;
            return t->split_k;
        }
    }
    const long nkb = K / kTileCols > 0 ? K / kTileCols : 1;
    int best = 1;
    double best_cost = -1.0;
    LaunchPlan best_plan{0, 1, 0, static_cast<unsigned>(kTileLds)};
    for (long s = 1; s <= 32 && s <= nkb; s++) {
        const long tiles = (nkb + s - 1) / s;
        if (s > 1 && tiles * (s - 1) >= nkb)
            continue;  // a split that leaves the last batch empty
        double c = 0.0;
        const LaunchPlan p = plan_launch(M, N, K, static_cast<int>(s), false, &c, tile_bytes);
        if (best_cost < 0 || c < best_cost - 1e-9) {
            best = static_cast<int>(s);
            best_cost = c;
            best_plan = p;
        }
    }
    if (plan)
        *plan = best_plan;
    return best;
}

}  // namespace tcsl
