// Launch shape of the main kernel and the cost model that picks it.  Host only.
#pragma once

namespace tcsl {

// mode 0: the W waves of a workgroup take W consecutive 128-row tile rows of one split-K
//         batch (stage_b: the batch's activation slice is staged in LDS and shared);
// mode 1: the W waves of a workgroup split the batch of one tile row among themselves and
//         add their accumulators up in LDS.
// separate_reduction (mode 1, Split_K > 1): the slabs of partial sums are added up by the reduction
//         kernel instead of by the last workgroup of each tile row inside the launch (mode 0 always
//         uses the reduction kernel).
struct LaunchPlan {
    int mode;
    int waves;
    int stage_b;
    unsigned lds_bytes;
    bool separate_reduction = false;
};

// True (and lds_bytes filled in) when the kernels can run this shape.
bool complete_plan(int N, int K, int split_k, bool row_major, LaunchPlan& p);

// Estimated time in microseconds of SpMM_SplitK_API (main kernel + reduction) with this plan.
// tile_bytes: average compressed bytes per 128 x 64 tile of the weight (16 * vectors / tiles);
// 0 = not known, taken as 80 % sparsity.
constexpr double kTileBytesAt80 = 6558.0;
double plan_cost_us(int M, int N, int K, int split_k, const LaunchPlan& p, double tile_bytes = 0.0);

// Best plan for a given Split_K; *cost_us (optional) receives its estimate.
// row_major: B is [K][N] and C [M][N]; such calls cannot stage the activation slice.
LaunchPlan plan_launch(int M, int N, int K, int split_k, bool row_major, double* cost_us, double tile_bytes = 0.0);

// Best Split_K in 1..32 (with its plan) for the shape.
int suggest_split_k(int M, int N, int K, LaunchPlan* plan, double tile_bytes = 0.0);

}  // namespace tcsl
