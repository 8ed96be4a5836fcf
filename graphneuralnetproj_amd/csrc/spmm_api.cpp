// Host logic behind the C ABI declared in include/SpMM_API.h: argument
// checking, the split-K plan and the order of launches.  Plain C++; the GPU is
// reached only through the tcsl_* launchers of spmm_kernels.hip.
#include <cstdint>
#include <cstdio>
#include <cstdlib>

#include "../../include/SpMM_API.h"
#include "tiled_csl_format.h"

extern "C" {
int tcsl_launch_spmm(void* stream, const void* items, const int* offsets, const void* B, void* out, int M, int N,
                     int K, int split_k, int waves, int stage_b, unsigned lds_bytes);
int tcsl_launch_reduce(void* stream, void* C, const void* W, long mn, int split_k);
int tcsl_launch_copy(void* stream, void* dst, const void* src, long bytes);
void* tcsl_event_create(void);
void tcsl_event_destroy(void* e);
int tcsl_event_record(void* e, void* stream);
float tcsl_event_elapsed_ms(void* start, void* stop);
const char* tcsl_error_string(int code);
int tcsl_error_unknown(void);
int tcsl_error_invalid_value(void);
}

extern "C" int InitSparseMatrixA_API(const uint16_t* A_h, int M, int N, int K, uint32_t** Compressed_A,
                                     int** TileOffsets)
{
    (void)N;  // unused by the reference too (csrc/SpMM_API.cu:241-246)
    return tcsl::encode(A_h, M, K, Compressed_A, TileOffsets);
}

extern "C" int GenSparseMatrixBinFile(char* DenseMatrixFileName, int M, int K, char* NZWeightsFileName,
                                      char* TileOffsetsFileName, char* OutputSizesFileName)
{
    return tcsl::encode_file(DenseMatrixFileName, M, K, NZWeightsFileName, TileOffsetsFileName, OutputSizesFileName);
}

extern "C" void SpMM_FreeHost(void* p)
{
    std::free(p);
}

extern "C" const char* SpMM_GetErrorString(int code)
{
    return tcsl_error_string(code);
}

namespace {

// Launch shape of the main kernel: W waves per workgroup (each wave owns one 128-row tile
// row of one batch), and whether the batch's activation slice is staged in LDS.
struct LaunchPlan {
    int waves;
    int stage_b;
    unsigned lds_bytes;
};

LaunchPlan plan_launch(int M, int N, int K, int Split_K)
{
    constexpr long kLds = 160 * 1024, kTile = 16384, kCUs = 256;
    const long row_tiles = M / tcsl::kTileRows;
    const long nkb = K / tcsl::kTileCols;
    const long tiles = (nkb - 1) / Split_K + 1;  // tiles of the longest batch
    if (N > 16)  // wide accumulators: one wave per workgroup, activations from global memory
        return LaunchPlan{1, 0, static_cast<unsigned>(kTile)};
    const long slice = tiles * (N == 8 ? 8 : 16) * 128;  // staged activation bytes
    // Pick W: the busiest compute unit runs ceil(workgroups / 256) workgroups of W waves of
    // `tiles` tiles each, and pulls its stream at full rate only with about seven waves
    // resident.  Ties go to the larger W (more waves share one staged slice).
    LaunchPlan best{1, 0, static_cast<unsigned>(kTile)};
    double best_cost = 0.0;
    for (int w = 1; w <= 8; w++) {
        for (int stage = 0; stage <= 1; stage++) {
            const long lds = w * kTile + (stage ? slice : 0);
            if (lds > kLds)
                continue;
            const long wgs = (row_tiles + w - 1) / w * Split_K;
            long fit = kLds / lds;  // workgroups resident per compute unit
            if (fit > 8 / w)
                fit = 8 / w;        // eight waves per compute unit at this kernel's register use
            const long per_cu = (wgs + kCUs - 1) / kCUs;
            const long resident = (per_cu < fit ? per_cu : fit) * w;
            double cost = static_cast<double>(per_cu) * w * tiles * (resident < 7 ? 7.0 / resident : 1.0);
            if (!stage)
                cost *= 1.03;  // activations re-fetched through L2 for every tile
            if (best_cost == 0.0 || cost <= best_cost * (1.0 + 1e-9)) {
                best = LaunchPlan{w, stage, static_cast<unsigned>(lds)};
                best_cost = cost;
            }
        }
    }
    return best;
}

int launch_main(void* stream, const void* Compressed_A, const int* TileOffsets, const void* B, void* out, int M, int N,
                int K, int Split_K)
{
    const LaunchPlan p = plan_launch(M, N, K, Split_K);
    return tcsl_launch_spmm(stream, Compressed_A, TileOffsets, B, out, M, N, K, Split_K, p.waves, p.stage_b,
                            p.lds_bytes);
}

int spmm_splitk(void* stream, const void* Compressed_A, const int* TileOffsets, const void* B, void* C, int M, int N,
                int K, void* Reduction_Workspace, int Split_K, void* ev_begin, void* ev_end);
}

extern "C" int SpMM_SplitK_API(void* stream, const void* A, const void* Compressed_A, const int* TileOffsets,
                               const void* B, void* C, int M, int N, int K, void* Reduction_Workspace, int Split_K)
{
    (void)A;
    return spmm_splitk(stream, Compressed_A, TileOffsets, B, C, M, N, K, Reduction_Workspace, Split_K, nullptr,
                       nullptr);
}

extern "C" int SpMM_SplitK_API_Events(void* stream, const void* A, const void* Compressed_A, const int* TileOffsets,
                                      const void* B, void* C, int M, int N, int K, void* Reduction_Workspace,
                                      int Split_K, void* KernelBegin, void* KernelEnd)
{
    (void)A;
    return spmm_splitk(stream, Compressed_A, TileOffsets, B, C, M, N, K, Reduction_Workspace, Split_K, KernelBegin,
                       KernelEnd);
}

extern "C" int SpMM_SplitK_Partials(void* stream, const void* Compressed_A, const int* TileOffsets, const void* B,
                                    void* Partials, int M, int N, int K, int Split_K)
{
    if (N != 8 && N != 16 && N != 32 && N != 64)
        return tcsl_error_unknown();
    if (M <= 0 || K <= 0 || M % tcsl::kTileRows != 0 || K % tcsl::kTileCols != 0 || Split_K < 1 ||
        static_cast<long>(M / tcsl::kTileRows) * Split_K > 0x7fffffffL)
        return tcsl_error_invalid_value();
    if (!Compressed_A || !TileOffsets || !B || !Partials)
        return tcsl_error_invalid_value();
    return launch_main(stream, Compressed_A, TileOffsets, B, Partials, M, N, K, Split_K);
}

extern "C" void* SpMM_EventCreate(void)
{
    return tcsl_event_create();
}

extern "C" void SpMM_EventDestroy(void* event)
{
    tcsl_event_destroy(event);
}

extern "C" int SpMM_EventRecord(void* event, void* stream)
{
    return event ? tcsl_event_record(event, stream) : tcsl_error_invalid_value();
}

extern "C" float SpMM_EventElapsedMs(void* start, void* stop)
{
    return (start && stop) ? tcsl_event_elapsed_ms(start, stop) : -1.f;
}

namespace {

int spmm_splitk(void* stream, const void* Compressed_A, const int* TileOffsets, const void* B, void* C, int M, int N,
                int K, void* Reduction_Workspace, int Split_K, void* ev_begin, void* ev_end)
{
    if (N != 8 && N != 16 && N != 32 && N != 64) {
        std::printf("MM_Sparse_API Error: Unsupported N dimension %d!\n", N);
        return tcsl_error_unknown();
    }
    if (M <= 0 || K <= 0 || M % tcsl::kTileRows != 0 || K % tcsl::kTileCols != 0 || Split_K < 1) {
        std::fprintf(stderr, "SpMM_SplitK_API: unsupported shape M=%d K=%d Split_K=%d (need M %% 128 == 0, K %% 64 == 0, Split_K >= 1)\n",
                     M, K, Split_K);
        return tcsl_error_invalid_value();
    }
    if (!Compressed_A || !TileOffsets || !B || !C || (Split_K > 1 && !Reduction_Workspace)) {
        std::fprintf(stderr, "SpMM_SplitK_API: null device pointer\n");
        return tcsl_error_invalid_value();
    }
    // the launch grid is (M/128) * Split_K single-wave workgroups
    if (static_cast<long>(M / tcsl::kTileRows) * Split_K > 0x7fffffffL) {
        std::fprintf(stderr, "SpMM_SplitK_API: Split_K=%d too large for M=%d\n", Split_K, M);
        return tcsl_error_invalid_value();
    }
    // optional events bracket the main kernel only (not the reduction)
    int rc = 0;
    if (ev_begin && (rc = tcsl_event_record(ev_begin, stream)) != 0)
        return rc;
    rc = launch_main(stream, Compressed_A, TileOffsets, B, Split_K == 1 ? C : Reduction_Workspace, M, N, K, Split_K);
    if (rc != 0)
        return rc;
    if (ev_end && (rc = tcsl_event_record(ev_end, stream)) != 0)
        return rc;
    if (Split_K == 1)
        return 0;
    return tcsl_launch_reduce(stream, C, Reduction_Workspace, static_cast<long>(M) * N, Split_K);
}
}  // namespace

extern "C" int SpMM_SuggestSplitK(int M, int N, int K)
{
    if (M <= 0 || K <= 0 || N <= 0)
        return 1;
    // One wave per (128-row tile row, batch), spread over 256 compute units.  The stream a
    // compute unit has to pull is the sum of its waves' tiles, and it needs about seven
    // resident waves to pull at full rate, so the estimate to minimise is
    //   max(ceil(units / 256), 7) * tiles_per_unit    busiest unit's share of the weight stream
    // + units / 256 * slab_cost                       partial sums written, then read by the reduction
    // in units of one 80 %-sparse tile (about 6.5 KB); ties go to the smaller split.
    const long row_tiles = (M + tcsl::kTileRows - 1) / tcsl::kTileRows;
    const long nkb = K / tcsl::kTileCols > 0 ? K / tcsl::kTileCols : 1;
    const double slab_cost = 2.0 * tcsl::kTileRows * N * 2.0 / 6554.0;
    int best = 1;
    double best_cost = 0.0;
    for (long s = 1; s <= 32 && s <= nkb; s++) {
        const long tiles = (nkb + s - 1) / s;
        if (s > 1 && (tiles < 2 || tiles * (s - 1) >= nkb))
            continue;  // batches of one tile, or a split that leaves the last batch empty
        const long units = row_tiles * s;
        const long waves_per_cu = (units + 255) / 256;
        const double cost = static_cast<double>(waves_per_cu > 7 ? waves_per_cu : 7) * tiles +
                            (s > 1 ? units / 256.0 * slab_cost : 0.0);
        if (s == 1 || cost < best_cost - 1e-9) {
            best = static_cast<int>(s);
            best_cost = cost;
        }
    }
    return best;
}

extern "C" void SpMM_SynthWeights(uint16_t* A_h, int M, int K, double sparsity, int row_skewed, uint64_t seed)
{
    tcsl::synth_weights(A_h, M, K, sparsity, row_skewed, seed);
}

extern "C" void SpMM_SynthActivations(uint16_t* B_h, long count, uint64_t seed)
{
    tcsl::synth_activations(B_h, count, seed);
}

extern "C" int SpMM_CalibrationCopy(void* stream, void* dst, const void* src, long bytes)
{
    if (!dst || !src || bytes < 0 || bytes % 16 != 0)
        return tcsl_error_invalid_value();
    return tcsl_launch_copy(stream, dst, src, bytes);
}
