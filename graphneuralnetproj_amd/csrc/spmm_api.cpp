// Host logic behind the C ABI declared in include/SpMM_API.h: argument
// checking, the split-K plan and the order of launches.  Plain C++; the GPU is
// reached only through the tcsl_* launchers of spmm_kernels.hip and
// tiled_csl_encode_device.hip and the a24_* launchers of a24_kernels.hip.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <mutex>

#include "../../include/SpMM_API.h"
#include "a24_format.h"
#include "counter_pages.h"
#include "launch_plan.h"
#include "tiled_csl_format.h"

extern "C" {
int tcsl_launch_spmm(void* stream, const void* items, const int* offsets, const void* B, void* out, int M, int N,
                     int K, int split_k, int mode, int waves, int stage_b, int row_major, unsigned lds_bytes, int ldb,
                     int ldo, int relu, void* fused_out, int ldc, int fuse_page, int dense_waves);
int tcsl_launch_reduce(void* stream, void* C, const void* W, long rows, long vectors, long ldc, int split_k, int relu);
int tcsl_launch_copy(void* stream, void* dst, const void* src, long bytes);
int tcsl_launch_encode_offsets(void* stream, const void* A, int M, int K, int* offsets);
int tcsl_launch_encode_items(void* stream, const void* A, int M, int K, const int* offsets, void* items);
int a24_launch_spmm(void* stream, const void* packed, const void* B, void* out, int M, int N, int K, int split_k, int rb,
                    int waves, int share_b, long ldb, long ldo, long slab, int residual_loads = 0,
                    const void* words = nullptr, const void* offsets = nullptr, int relu = 0, int fuse_page = -1,
                    void* fused_out = nullptr, long ldc = 0, int row_major = 0);
int a24_launch_split_pack(void* stream, const void* A, void* packed, void* residual, int M, int K);
int a24_launch_residual_offsets(void* stream, const void* A2, int M, int K, int* offsets, int* longest);
int a24_launch_residual_words(void* stream, const void* A2, int M, int K, const int* offsets, void* words);
int a24_side_begin(void* stream, void** side);
int a24_side_end(void* stream, void* side);
int tcsl_static_workspace(void** slabs, long* bytes);
int tcsl_stream_capture(void* stream, unsigned long long* id);
int tcsl_page_prepare(int page);
int tcsl_page_mark(int page, void* stream);
int tcsl_page_idle(int page);
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

extern "C" int InitSparseMatrixA_API_NoReorder(const uint16_t* A_h, int M, int N, int K, uint32_t** Compressed_A,
                                               int** TileOffsets)
{
    (void)N;
    return tcsl::encode_noreorder(A_h, M, K, Compressed_A, TileOffsets);
}

extern "C" int GenSparseMatrixBinFile(char* DenseMatrixFileName, int M, int K, char* NZWeightsFileName,
                                      char* TileOffsetsFileName, char* OutputSizesFileName)
{
    return tcsl::encode_file(DenseMatrixFileName, M, K, NZWeightsFileName, TileOffsetsFileName, OutputSizesFileName);
}

extern "C" int SpMM_DeviceEncodeOffsets(void* stream, const void* A_d, int M, int K, int* TileOffsets_d)
{
    if (M <= 0 || K <= 0 || M % tcsl::kTileRows != 0 || K % tcsl::kTileCols != 0 || !A_d || !TileOffsets_d)
        return tcsl_error_invalid_value();
    return tcsl_launch_encode_offsets(stream, A_d, M, K, TileOffsets_d);
}

extern "C" int SpMM_DeviceEncodeItems(void* stream, const void* A_d, int M, int K, const int* TileOffsets_d,
                                      void* Compressed_A_d)
{
    if (M <= 0 || K <= 0 || M % tcsl::kTileRows != 0 || K % tcsl::kTileCols != 0 || !A_d || !TileOffsets_d ||
        !Compressed_A_d)
        return tcsl_error_invalid_value();
    return tcsl_launch_encode_items(stream, A_d, M, K, TileOffsets_d, Compressed_A_d);
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

// Plans are a pure function of the shape; the last few are remembered per thread so that a
// decode loop cycling over a handful of layer shapes never re-runs the model.
tcsl::LaunchPlan cached_plan(int M, int N, int K, int Split_K, bool row_major)
{
    struct Entry {
        int M, N, K, S;
        bool row_major;
        tcsl::LaunchPlan plan;
    };
    constexpr int kEntries = 16;
    thread_local Entry cache[kEntries] = {};
    thread_local int next = 0;
    for (const Entry& e : cache)
        if (e.M == M && e.N == N && e.K == K && e.S == Split_K && e.row_major == row_major)
            return e.plan;
    const tcsl::LaunchPlan p = tcsl::plan_launch(M, N, K, Split_K, row_major, nullptr);
    cache[next] = Entry{M, N, K, Split_K, row_major, p};
    next = (next + 1) % kEntries;
    return p;
}

// The fused split-K reduction counts arrivals in a page of device counters that no launch
// which might overlap this one may use (counter_pages.h has the rules).  -1 when no page can be
// had: the call then runs the reduction as a second kernel.  The caller holds pages.mutex().
tcsl::CounterPages& counter_pages()
{
    static tcsl::CounterPages pages;
    return pages;
}

int counter_page(void* stream)
{
    unsigned long long capture_id = 0;
    const int capturing = tcsl_stream_capture(stream, &capture_id);
    if (capturing < 0)
        return -1;
    const int page = counter_pages().acquire(tcsl::CounterPages::stream_key(stream), capturing == 1, capture_id, [](int p) { return tcsl_page_idle(p) == 1; });
    // a page that changes hands is guarded by an event behind each of its launches; without one, no page
    if (page >= 0 && tcsl::CounterPages::recycled(page) && tcsl_page_prepare(page) != 0)
        return -1;
    return page;
}

constexpr int kStaticWorkspacePage = 1 << 20;  // the counters inside the static workspace (spmm_kernels.hip: kScratchPage)

// What varies between the entry points that end in the same two launches.
struct CallOptions {
    bool row_major = false;   // B is [K][N], C and the slabs [M][N]
    long ldb = 0;             // elements between two tokens' vectors in B (0 = K); column-major only
    long ldc = 0;             // the same for C (0 = M)
    bool relu = false;        // clamp C at zero
    bool separate_reduction = false;  // never fuse the reduction into the main kernel
    void* ev_begin = nullptr; // events recorded around the main kernel
    void* ev_end = nullptr;
    const tcsl::LaunchPlan* forced = nullptr;
    bool adaptive_waves = false;  // with `forced`: launch it the way a planned call would be
    int extra_slabs = 0;      // fused reduction only: slabs of an earlier launch, right behind this one's, to add as well
    bool static_workspace = false;  // the slabs are the library's static workspace: count arrivals there too
};

// fused_out != nullptr asks for the fused reduction; *fused says whether it was possible.
int launch_main(void* stream, const void* Compressed_A, const int* TileOffsets, const void* B, void* out, int M, int N,
                int K, int Split_K, const CallOptions& o, int ldb, int ldo, bool relu, void* fused_out, long ldc,
                bool* fused)
{
    const tcsl::LaunchPlan p = o.forced ? *o.forced : cached_plan(M, N, K, Split_K, o.row_major);
    int page = -1;
    // Only the layout whose workgroup owns a single tile row fuses the reduction: its last arriver
    // adds up 128 rows.  In the row-sharing layout one workgroup would be left with W x 128 rows of
    // every slab while the rest of the chip idles, which measured slower than the second kernel.
    // A page from the pool stays this call's until the launch is enqueued (the lock): from then
    // on its stream counts as busy and the page cannot change hands.
    std::unique_lock<std::mutex> page_lock;
    if (fused_out && p.mode == 1 && !p.separate_reduction && M / tcsl::kTileRows <= 4096) {
        if (o.static_workspace) {
            page = kStaticWorkspacePage;
        } else {
            page_lock = std::unique_lock<std::mutex>(counter_pages().mutex());
            page = counter_page(stream);
        }
    }
    if (fused)
        *fused = page >= 0;
    // The plan's wave count is tuned on 80 % sparse weights.  Sparser ones want every wave the
    // registers allow (a wave's turnaround per tile becomes the limit), which the host cannot see:
    // in the K-splitting layout it launches them all and lets each workgroup look at its own tiles.
    tcsl::LaunchPlan run = p;
    int dense_waves = 0;
    if ((!o.forced || o.adaptive_waves) && p.mode == 1 && N <= 32 && p.waves < 8) {
        tcsl::LaunchPlan all{1, 8, 0, 0};
        if (tcsl::complete_plan(N, K, Split_K, o.row_major, all)) {
            run = all;
            dense_waves = p.waves;
        }
    }
    int rc = tcsl_launch_spmm(stream, Compressed_A, TileOffsets, B, out, M, N, K, Split_K, run.mode, run.waves, run.stage_b,
                              o.row_major ? 1 : 0, run.lds_bytes, ldb, ldo,
                              (relu && (Split_K == 1 || page >= 0) ? 1 : 0)  // slabs of partial sums are never clamped
                                  | (page >= 0 ? o.extra_slabs << 8 : 0),
                              page >= 0 ? fused_out : nullptr, static_cast<int>(ldc), page, dense_waves);
    if (rc == 0 && tcsl::CounterPages::recycled(page))
        rc = tcsl_page_mark(page, stream);
    return rc;
}

int check_call(const void* Compressed_A, const int* TileOffsets, const void* B, const void* C, int M, int N, int K,
               bool have_workspace, int Split_K);
int spmm_splitk(void* stream, const void* Compressed_A, const int* TileOffsets, const void* B, void* C, int M, int N,
                int K, void* Reduction_Workspace, int Split_K, const CallOptions& o);
}  // namespace

extern "C" int SpMM_SplitK_API(void* stream, const void* A, const void* Compressed_A, const int* TileOffsets,
                               const void* B, void* C, int M, int N, int K, void* Reduction_Workspace, int Split_K)
{
    (void)A;
    return spmm_splitk(stream, Compressed_A, TileOffsets, B, C, M, N, K, Reduction_Workspace, Split_K, CallOptions{});
}

extern "C" int SpMM_SplitK_API_StaticWorkspace(void* stream, const void* A, const void* Compressed_A,
                                               const int* TileOffsets, const void* B, void* C, int M, int N, int K,
                                               int Split_K)
{
    (void)A;
    void* slabs = nullptr;
    long room = 0;
    if (const int rc = check_call(Compressed_A, TileOffsets, B, C, M, N, K, true, Split_K))
        return rc;
    if (Split_K > 1) {
        if (const int rc = tcsl_static_workspace(&slabs, &room))
            return rc;
        const long need = static_cast<long>(Split_K) * M * N * 2;
        if (need > room) {
            std::fprintf(stderr,
                         "SpMM_SplitK_API_StaticWorkspace: Split_K=%d x M=%d x N=%d fp16 partial sums need %ld bytes, the "
                         "static workspace holds %ld; use a smaller Split_K or SpMM_SplitK_API with a workspace of your own\n",
                         Split_K, M, N, need, room);
            return tcsl_error_invalid_value();
        }
    }
    CallOptions o;
    o.static_workspace = true;
    return spmm_splitk(stream, Compressed_A, TileOffsets, B, C, M, N, K, slabs, Split_K, o);
}

extern "C" int SpMM_SplitK_API_RowMajor(void* stream, const void* A, const void* Compressed_A, const int* TileOffsets,
                                        const void* B, void* C, int M, int N, int K, void* Reduction_Workspace,
                                        int Split_K)
{
    (void)A;
    CallOptions o;
    o.row_major = true;
    return spmm_splitk(stream, Compressed_A, TileOffsets, B, C, M, N, K, Reduction_Workspace, Split_K, o);
}

extern "C" int SpMM_SplitK_API_Strided(void* stream, const void* Compressed_A, const int* TileOffsets, const void* B,
                                       long ldb, void* C, long ldc, int M, int N, int K, void* Reduction_Workspace,
                                       int Split_K, int Flags)
{
    if (ldb < K || ldc < M || ldb % 8 != 0 || ldc % 8 != 0 || ldb > 0x7fffffffL || ldc > 0x7fffffffL ||
        (Flags & ~(SPMM_FLAG_RELU | SPMM_FLAG_SEPARATE_REDUCTION)) != 0)
        return tcsl_error_invalid_value();
    CallOptions o;
    o.ldb = ldb;
    o.ldc = ldc;
    o.relu = (Flags & SPMM_FLAG_RELU) != 0;
    o.separate_reduction = (Flags & SPMM_FLAG_SEPARATE_REDUCTION) != 0;
    return spmm_splitk(stream, Compressed_A, TileOffsets, B, C, M, N, K, Reduction_Workspace, Split_K, o);
}

extern "C" int SpMM_SplitK_API_RowMajor_Flags(void* stream, const void* Compressed_A, const int* TileOffsets, const void* B,
                                              void* C, int M, int N, int K, void* Reduction_Workspace, int Split_K, int Flags)
{
    if ((Flags & ~(SPMM_FLAG_RELU | SPMM_FLAG_SEPARATE_REDUCTION)) != 0)
        return tcsl_error_invalid_value();
    CallOptions o;
    o.row_major = true;
    o.relu = (Flags & SPMM_FLAG_RELU) != 0;
    o.separate_reduction = (Flags & SPMM_FLAG_SEPARATE_REDUCTION) != 0;
    return spmm_splitk(stream, Compressed_A, TileOffsets, B, C, M, N, K, Reduction_Workspace, Split_K, o);
}

extern "C" int SpMM_SplitK_API_Planned(void* stream, const void* Compressed_A, const int* TileOffsets, const void* B,
                                       void* C, int M, int N, int K, void* Reduction_Workspace, int Split_K, int Mode,
                                       int Waves, int StageB, int RowMajor, int Flags)
{
    tcsl::LaunchPlan p{Mode, Waves, StageB, 0};
    if (!tcsl::complete_plan(N, K > 0 ? K : 64, Split_K, RowMajor != 0, p) ||
        (Flags & ~(SPMM_FLAG_RELU | SPMM_FLAG_SEPARATE_REDUCTION | SPMM_FLAG_ADAPTIVE_WAVES)) != 0)
        return tcsl_error_invalid_value();
    CallOptions o;
    o.relu = (Flags & SPMM_FLAG_RELU) != 0;
    o.separate_reduction = (Flags & SPMM_FLAG_SEPARATE_REDUCTION) != 0;
    o.adaptive_waves = (Flags & SPMM_FLAG_ADAPTIVE_WAVES) != 0;
    o.row_major = RowMajor != 0;
    o.forced = &p;
    return spmm_splitk(stream, Compressed_A, TileOffsets, B, C, M, N, K, Reduction_Workspace, Split_K, o);
}

extern "C" int SpMM_PlanLaunch(int M, int N, int K, int Split_K, int* Mode, int* Waves, int* StageB, int* LdsBytes,
                               double* EstimatedUs)
{
    if ((N != 8 && N != 16 && N != 32 && N != 64) || M <= 0 || K <= 0 || M % tcsl::kTileRows != 0 ||
        K % tcsl::kTileCols != 0 || Split_K < 1)
        return -1;
    double cost = 0.0;
    const tcsl::LaunchPlan p = tcsl::plan_launch(M, N, K, Split_K, false, &cost);
    if (Mode)
        *Mode = p.mode;
    if (Waves)
        *Waves = p.waves;
    if (StageB)
        *StageB = p.stage_b;
    if (LdsBytes)
        *LdsBytes = static_cast<int>(p.lds_bytes);
    if (EstimatedUs)
        *EstimatedUs = cost;
    return 0;
}

extern "C" int SpMM_PlanReductionInLaunch(int M, int N, int K, int Split_K)
{
    if ((N != 8 && N != 16 && N != 32 && N != 64) || M <= 0 || K <= 0 || M % tcsl::kTileRows != 0 ||
        K % tcsl::kTileCols != 0 || Split_K < 1)
        return -1;
    if (Split_K == 1)
        return 0;
    const tcsl::LaunchPlan p = tcsl::plan_launch(M, N, K, Split_K, false, nullptr);
    return p.mode == 1 && !p.separate_reduction && M / tcsl::kTileRows <= 4096 ? 1 : 0;
}

extern "C" int SpMM_SplitK_API_Events(void* stream, const void* A, const void* Compressed_A, const int* TileOffsets,
                                      const void* B, void* C, int M, int N, int K, void* Reduction_Workspace,
                                      int Split_K, void* KernelBegin, void* KernelEnd)
{
    (void)A;
    CallOptions o;
    o.ev_begin = KernelBegin;
    o.ev_end = KernelEnd;
    return spmm_splitk(stream, Compressed_A, TileOffsets, B, C, M, N, K, Reduction_Workspace, Split_K, o);
}

extern "C" int SpMM_SplitK_Partials(void* stream, const void* Compressed_A, const int* TileOffsets, const void* B,
                                    void* Partials, int M, int N, int K, int Split_K)
{
    if (N != 8 && N != 16 && N != 32 && N != 64)
        return tcsl_error_unknown();
    if (M <= 0 || K <= 0 || M % tcsl::kTileRows != 0 || K % tcsl::kTileCols != 0 || Split_K < 1 ||
        Split_K > 65535)
        return tcsl_error_invalid_value();
    if (!Compressed_A || !TileOffsets || !B || !Partials)
        return tcsl_error_invalid_value();
    return launch_main(stream, Compressed_A, TileOffsets, B, Partials, M, N, K, Split_K, CallOptions{}, K, M, false,
                       nullptr, 0, nullptr);
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

// The checks every product entry point makes before anything is launched; 0 = fine.
int check_call(const void* Compressed_A, const int* TileOffsets, const void* B, const void* C, int M, int N, int K,
               bool have_workspace, int Split_K)
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
    if (!Compressed_A || !TileOffsets || !B || !C || (Split_K > 1 && !have_workspace)) {
        std::fprintf(stderr, "SpMM_SplitK_API: null device pointer\n");
        return tcsl_error_invalid_value();
    }
    // the launch grid is (groups of tile rows) x Split_K workgroups, and a grid's second dimension ends at 65535
    if (Split_K > 65535) {
        std::fprintf(stderr, "SpMM_SplitK_API: Split_K=%d too large for M=%d\n", Split_K, M);
        return tcsl_error_invalid_value();
    }
    return 0;
}

int spmm_splitk(void* stream, const void* Compressed_A, const int* TileOffsets, const void* B, void* C, int M, int N,
                int K, void* Reduction_Workspace, int Split_K, const CallOptions& o)
{
    if (const int bad = check_call(Compressed_A, TileOffsets, B, C, M, N, K, Reduction_Workspace != nullptr, Split_K))
        return bad;
    const int ldb = o.ldb ? static_cast<int>(o.ldb) : K;
    const long ldc = o.ldc ? o.ldc : M;
    // optional events bracket the main kernel only (not the reduction)
    int rc = 0;
    if (o.ev_begin && (rc = tcsl_event_record(o.ev_begin, stream)) != 0)
        return rc;
    bool fused = false;
    if (Split_K == 1) {  // the kernel writes C itself, with C's stride and the clamp
        rc = launch_main(stream, Compressed_A, TileOffsets, B, C, M, N, K, 1, o, ldb, static_cast<int>(ldc), o.relu,
                         nullptr, 0, nullptr);
    } else {
        // Dense slabs of partial sums; stride and clamp are applied by the reduction, which the
        // main kernel does itself (its last workgroup per group of rows) unless the caller wants
        // the main kernel timed alone or no counters are free.
        const bool want_fused = !o.separate_reduction && !o.ev_begin && !o.ev_end;
        rc = launch_main(stream, Compressed_A, TileOffsets, B, Reduction_Workspace, M, N, K, Split_K, o, ldb, M, o.relu,
                         want_fused ? C : nullptr, ldc, &fused);
    }
    if (rc != 0)
        return rc;
    if (o.ev_end && (rc = tcsl_event_record(o.ev_end, stream)) != 0)
        return rc;
    if (Split_K == 1 || fused)
        return 0;
    if (o.row_major || ldc == M)  // C is as dense as the slabs: one flat vector
        return tcsl_launch_reduce(stream, C, Reduction_Workspace, static_cast<long>(M) * N, 1, static_cast<long>(M) * N,
                                  Split_K, o.relu ? 1 : 0);
    return tcsl_launch_reduce(stream, C, Reduction_Workspace, M, N, ldc, Split_K, o.relu ? 1 : 0);
}
}  // namespace

extern "C" int SpMM_SuggestSplitK(int M, int N, int K)
{
    if (M <= 0 || K <= 0 || (N != 8 && N != 16 && N != 32 && N != 64))
        return 1;
    return tcsl::suggest_split_k(M - M % tcsl::kTileRows > 0 ? M - M % tcsl::kTileRows : tcsl::kTileRows, N,
                                 K - K % tcsl::kTileCols > 0 ? K - K % tcsl::kTileCols : tcsl::kTileCols, nullptr);
}

extern "C" int SpMM_SuggestSplitK_Bytes(int M, int N, int K, long Vectors)
{
    if (M <= 0 || K <= 0 || (N != 8 && N != 16 && N != 32 && N != 64) || M % tcsl::kTileRows != 0 || K % tcsl::kTileCols != 0)
        return 1;
    const double tiles = static_cast<double>(M / tcsl::kTileRows) * (K / tcsl::kTileCols);
    return tcsl::suggest_split_k(M, N, K, nullptr, Vectors > 0 ? 16.0 * static_cast<double>(Vectors) / tiles : 0.0);
}

extern "C" void SpMM_SynthWeights(uint16_t* A_h, int M, int K, double sparsity, int row_skewed, uint64_t seed)
{
    tcsl::synth_weights(A_h, M, K, sparsity, row_skewed, seed);
}

extern "C" void SpMM_SynthActivations(uint16_t* B_h, long count, uint64_t seed)
{
    tcsl::synth_activations(B_h, count, seed);
}

extern "C" void SpMM_SynthHarnessWeights(uint16_t* A_h, int M, int K, double sparsity, int row_skewed, uint64_t seed)
{
    tcsl::synth_harness_weights(A_h, M, K, sparsity, row_skewed, seed);
}

extern "C" void SpMM_SynthHarnessActivations(uint16_t* B_h, long count, uint64_t seed)
{
    tcsl::synth_harness_activations(B_h, count, seed);
}

extern "C" int SpMM_CalibrationCopy(void* stream, void* dst, const void* src, long bytes)
{
    if (!dst || !src || bytes < 0 || bytes % 16 != 0)
        return tcsl_error_invalid_value();
    return tcsl_launch_copy(stream, dst, src, bytes);
}

// ---------------------------------------------------------------------------------------------
// 2:4 part on the sparse matrix cores + Tiled-CSL residual

extern "C" int HeteroSparse_Decompose(const uint16_t* A_h, uint16_t* A1_h, uint16_t* A2_h, long Length)
{
    if (!A_h || !A1_h || !A2_h)
        return a24::kErrNullPointer;
    if (Length < 0 || Length % 4 != 0)  // the reference asserts this (kernel_benchmark/spmm_decompose.h:17)
        return a24::kErrBadShape;
    a24::decompose(A_h, A1_h, A2_h, Length);
    return 0;
}

extern "C" long HeteroSparse_PackedBytes(int M, int K)
{
    if (M <= 0 || K <= 0 || M % (a24::kRows * a24::kGroupBlocks) != 0 || K % a24::kUnitCols != 0)
        return a24::kErrBadShape;
    return a24::bytes(M, K);
}

extern "C" int HeteroSparse_PackA1(const uint16_t* A1_h, int M, int K, void* Packed_h)
{
    return a24::pack(A1_h, M, K, static_cast<uint8_t*>(Packed_h));
}

extern "C" int HeteroSparse_DeviceSplitPack(void* stream, const void* A_d, int M, int K, void* Packed_A1_d, void* A2_d)
{
    if (!A_d || !Packed_A1_d || M <= 0 || K <= 0 || M % (a24::kRows * a24::kGroupBlocks) != 0 || K % a24::kUnitCols != 0) {
        std::fprintf(stderr, "HeteroSparse_DeviceSplitPack: need M %% 128 == 0, K %% 128 == 0 and non-null pointers (M=%d K=%d)\n", M, K);
        return tcsl_error_invalid_value();
    }
    return a24_launch_split_pack(stream, A_d, Packed_A1_d, A2_d, M, K);
}

namespace {

// Launch shape of the 2:4 kernel: row blocks per workgroup, waves per workgroup, split-K.
struct A24Plan {
    int row_blocks, waves, split_k;
    int share_b = 0;  // 0: the waves of a workgroup split K and add up; 1: they split rows and share the activation tile in LDS
};

// Waves per workgroup for a given split: eight (256 rows) where that many workgroups still fill
// the chip, else four (two such workgroups share a compute unit).
int a24_waves_for(int M, int split_k)
{
    return (M % 256 == 0 && static_cast<long>(M / 256) * split_k > 160) ? 8 : 4;
}

A24Plan a24_default_plan(int M, int N, int K)
{
    // From sweeps over the OPT-30B and OPT-66B shapes (N = 16 and 64, with and without the residual):
    // waves that own two row blocks each and share the activation tile through LDS, and the split-K
    // with the least estimated time for the finished result: rounds of workgroups (256 of eight
    // waves or 512 of four at a time), each compute unit streaming its share of the records at one
    // unit's rate plus a fixed cost per round, and the reduction kernel plus a cost per slab once
    // there is more than one batch.  That picks what the sweeps found fastest: just under 256
    // workgroups of eight waves or as many of four with half the slabs (FFN1 28672x7168, N = 16:
    // four waves, one batch, no reduction: 36.0 us against 35.2 + 3 us), else e.g. 432 rather than
    // 144 or 288.  With 64 tokens eight waves hide the matrix cores' and the LDS's latencies better
    // (FFN1: 41 us + reduction against 46).
    A24Plan p{2, 4, 1, 1};
    const int units = K / a24::kUnitCols;
    const double bytes = static_cast<double>(a24::bytes(M, K));
    constexpr double kUnitBytesPerUs = 25.4e3, kRoundUs = 6.0, kReduceUs = 3.0, kSlabUs = 0.8, kFourWaves64 = 1.15;
    double best = 0.0;
    for (int s = 1; s <= 32 && s <= units; s++) {
        const int per = (units + s - 1) / s;
        if ((s > 1 && per < 2) || static_cast<long>(per) * (s - 1) >= units)
            continue;  // batches of one unit, or an empty last batch
        const int waves = a24_waves_for(M, s);
        const long n = static_cast<long>(M / (16 * p.row_blocks * waves)) * s;
        const long at_once = waves == 8 ? 256 : 512;
        const long rounds = (n + at_once - 1) / at_once;
        const long per_unit = ((n < at_once ? n : at_once) + 255) / 256;  // workgroups that share a compute unit
        const double stream = bytes / n * per_unit / kUnitBytesPerUs * (N == 64 && waves == 4 ? kFourWaves64 : 1.0);
        const double cost = rounds * (stream + kRoundUs) + (s > 1 ? kReduceUs + kSlabUs * s : 0.0);
        if (best == 0.0 || cost < best * 0.999) {
            best = cost;
            p.split_k = s;
            p.waves = waves;
        }
    }
    return p;
}

bool a24_shape_ok(int M, int N, int K, int split_k, int row_blocks, int waves, int share_b = 0)
{
    if (N != 8 && N != 16 && N != 32 && N != 64)
        return false;
    if (M <= 0 || K <= 0 || M % 128 != 0 || K % a24::kUnitCols != 0 || split_k < 1 || split_k > 65535)
        return false;
    const int units = K / a24::kUnitCols;
    const int per_batch = (units + split_k - 1) / split_k;
    if (static_cast<long>(per_batch) * (split_k - 1) >= units)  // the last batch would be empty
        return false;
    if (row_blocks < 1 || row_blocks > 8 || (row_blocks & (row_blocks - 1)) || waves < 1 || waves > 8)
        return false;
    if (share_b) {  // the kernel table of this layout, and whole workgroups only
        if (row_blocks < 2 || waves < 2 || row_blocks * waves < 8 || M % (16 * row_blocks * waves) != 0)
            return false;
        if (row_blocks > (N == 64 ? 2 : 4))  // three sets of record registers: what fits beside the accumulators
            return false;
        return true;
    }
    if (N == 64 && (row_blocks == 8 || (row_blocks == 4 && waves == 8)))  // accumulators would not fit the registers
        return false;
    return true;
}

}  // namespace

namespace {
int a24_split_call(void* stream, const void* Packed_A1, const void* B, long ldb, void* C, long ldc, int M, int N, int K,
                   void* Reduction_Workspace, int Split_K, int row_blocks, int waves, int loads, const void* words,
                   const void* offsets, int relu, bool separate_reduction, bool row_major = false);
int hybrid_call(const char* who, void* stream, const void* Packed_A1, const void* Compressed_A2, const int* TileOffsets_A2,
                const void* B, void* C, int M, int N, int K, void* Reduction_Workspace, int Split_K_A1, int Split_K_A2,
                int Flags, bool row_major);
}

extern "C" int HeteroSparse_A1_Partials(void* stream, const void* Packed_A1, const void* B, void* Partials, int M, int N,
                                        int K, int Split_K, int RowBlocks, int Waves, int ShareB)
{
    A24Plan p{RowBlocks, Waves, Split_K, ShareB ? 1 : 0};
    if (RowBlocks == 0 || Waves == 0) {
        const A24Plan d = a24_default_plan(M > 0 ? M : 128, N, K > 0 ? K : 128);
        p.row_blocks = d.row_blocks;
        p.waves = a24_waves_for(M > 0 ? M : 128, Split_K);
        p.share_b = d.share_b;
    }
    if (!Packed_A1 || !B || !Partials || !a24_shape_ok(M, N, K, p.split_k, p.row_blocks, p.waves, p.share_b)) {
        std::fprintf(stderr, "HeteroSparse_A1_Partials: unsupported call M=%d N=%d K=%d Split_K=%d (need M %% 128 == 0, K %% 128 == 0, N in {8,16,32,64}, no empty batch)\n",
                     M, N, K, Split_K);
        return tcsl_error_invalid_value();
    }
    return a24_launch_spmm(stream, Packed_A1, B, Partials, M, N, K, p.split_k, p.row_blocks, p.waves, p.share_b, K, M,
                           static_cast<long>(M) * N);
}

extern "C" int HeteroSparse_SuggestSplitK(int M, int N, int K)
{
    if (!a24_shape_ok(M, N, K, 1, 1, 1))
        return 1;
    return a24_default_plan(M, N, K).split_k;
}

extern "C" int HeteroSparse_SpMM_API(void* stream, const void* Packed_A1, const void* Compressed_A2,
                                     const int* TileOffsets_A2, const void* B, void* C, int M, int N, int K,
                                     void* Reduction_Workspace, int Split_K_A1, int Split_K_A2, int Flags)
{
    return hybrid_call("HeteroSparse_SpMM_API", stream, Packed_A1, Compressed_A2, TileOffsets_A2, B, C, M, N, K,
                       Reduction_Workspace, Split_K_A1, Split_K_A2, Flags, false);
}

extern "C" int HeteroSparse_SpMM_API_RowMajor(void* stream, const void* Packed_A1, const void* Compressed_A2,
                                              const int* TileOffsets_A2, const void* B, void* C, int M, int N, int K,
                                              void* Reduction_Workspace, int Split_K_A1, int Split_K_A2, int Flags)
{
    return hybrid_call("HeteroSparse_SpMM_API_RowMajor", stream, Packed_A1, Compressed_A2, TileOffsets_A2, B, C, M, N, K,
                       Reduction_Workspace, Split_K_A1, Split_K_A2, Flags, true);
}

namespace {
// row_major: B is [K][N], C and every slab [M][N] (this fork's layout) instead of [N][K] and [N][M].
int hybrid_call(const char* who, void* stream, const void* Packed_A1, const void* Compressed_A2, const int* TileOffsets_A2,
                const void* B, void* C, int M, int N, int K, void* Reduction_Workspace, int Split_K_A1, int Split_K_A2,
                int Flags, bool row_major)
{
    const bool residual = Compressed_A2 != nullptr;
    if (N != 8 && N != 16 && N != 32 && N != 64) {
        std::printf("MM_Sparse_API Error: Unsupported N dimension %d!\n", N);  // csrc/SpMM_API.cu:192-193
        return tcsl_error_unknown();
    }
    A24Plan d = a24_shape_ok(M, N, K, Split_K_A1, 1, 1) ? a24_default_plan(M, N, K) : A24Plan{1, 1, 1};
    if (d.share_b)
        d.waves = a24_waves_for(M, Split_K_A1);
    if (!Packed_A1 || !B || !C || (residual && !TileOffsets_A2) || !a24_shape_ok(M, N, K, Split_K_A1, d.row_blocks, d.waves, d.share_b)
        || (residual && (Split_K_A2 < 1 || Split_K_A2 > 65535)) || ((residual || Split_K_A1 > 1) && !Reduction_Workspace)
        || (Flags & ~HETERO_FLAG_TWO_STREAMS)) {
        std::fprintf(stderr, "%s: unsupported call M=%d N=%d K=%d Split_K=%d/%d (need M %% 128 == 0, K %% 128 == 0, no empty batch, non-null pointers)\n",
                     who, M, N, K, Split_K_A1, Split_K_A2);
        return tcsl_error_invalid_value();
    }
    if (row_major && !d.share_b)  // (the library's plans all share the activation tile; the other kernel takes column-major only)
        return tcsl_error_invalid_value();
    const long mn = static_cast<long>(M) * N;
    if (!residual && Split_K_A1 == 1)  // the 2:4 kernel writes C itself
        return a24_launch_spmm(stream, Packed_A1, B, C, M, N, K, 1, d.row_blocks, d.waves, d.share_b, K, M, mn, 0, nullptr, nullptr, 0,
                               -1, nullptr, 0, row_major ? 1 : 0);
    int rc = 0;
    uint16_t* ws = static_cast<uint16_t*>(Reduction_Workspace);
    if (!residual) {
        if (d.share_b)
            return a24_split_call(stream, Packed_A1, B, K, C, M, M, N, K, ws, Split_K_A1, d.row_blocks, d.waves, 0, nullptr, nullptr,
                                  0, false, row_major);
        rc = a24_launch_spmm(stream, Packed_A1, B, ws, M, N, K, Split_K_A1, d.row_blocks, d.waves, d.share_b, K, M, mn);
        return rc != 0 ? rc : tcsl_launch_reduce(stream, C, ws, mn, 1, mn, Split_K_A1, 0);
    }
    // Slabs: the residual's Split_K_A2 first, the 2:4 part's Split_K_A1 behind them.
    uint16_t* ws_a1 = ws + Split_K_A2 * mn;
    bool fused = false;
    if (Flags & HETERO_FLAG_TWO_STREAMS) {
        // On request the residual's kernel goes to a second stream, beside the 2:4 kernel.  Measured
        // slower than one stream (the two kernels compete, and two event waits cost more than the
        // overlap gains), hence optional.
        void* side = stream;
        if ((rc = a24_side_begin(stream, &side)) != 0)
            return rc;
        CallOptions o;
        o.separate_reduction = true;
        o.row_major = row_major;
        rc = launch_main(side, Compressed_A2, TileOffsets_A2, B, ws, M, N, K, Split_K_A2, o, K, M, false, nullptr, 0,
                         nullptr);
        if (rc == 0)
            rc = a24_launch_spmm(stream, Packed_A1, B, ws_a1, M, N, K, Split_K_A1, d.row_blocks, d.waves, d.share_b, K, M,
                                 mn, 0, nullptr, nullptr, 0, -1, nullptr, 0, row_major ? 1 : 0);
        // the side stream joins the caller's whatever happened in between: a fork left open would
        // leave the two streams unordered (and invalidate a graph capture that includes this call)
        const int joined = a24_side_end(stream, side);
        if (rc != 0 || (rc = joined) != 0)
            return rc;
    } else {
        // One stream: the 2:4 kernel first; the residual's kernel then adds everything up itself where
        // its launch shape has the in-launch reduction (the last workgroup of a tile row sums that
        // row's slabs, the 2:4 part's included), which saves the separate reduction kernel.
        if ((rc = a24_launch_spmm(stream, Packed_A1, B, ws_a1, M, N, K, Split_K_A1, d.row_blocks, d.waves, d.share_b, K, M,
                                  mn, 0, nullptr, nullptr, 0, -1, nullptr, 0, row_major ? 1 : 0)) != 0)
            return rc;
        CallOptions o;
        o.row_major = row_major;
        o.extra_slabs = Split_K_A1;
        if ((rc = launch_main(stream, Compressed_A2, TileOffsets_A2, B, ws, M, N, K, Split_K_A2, o, K, M, false, C, M,
                              &fused)) != 0)
            return rc;
    }
    if (fused)
        return 0;
    return tcsl_launch_reduce(stream, C, ws, mn, 1, mn, Split_K_A1 + Split_K_A2, 0);
}
}  // namespace

extern "C" int HeteroSparse_PackA2(const uint16_t* A2_h, int M, int K, uint32_t** Words, int** Offsets, int* LongestList)
{
    return a24::pack_residual(A2_h, M, K, Words, Offsets, LongestList);
}

extern "C" int HeteroSparse_DevicePackA2_Offsets(void* stream, const void* A2_d, int M, int K, int* Offsets_d, int* LongestList_d)
{
    if (!A2_d || !Offsets_d || !LongestList_d || M <= 0 || K <= 0 || M % (a24::kRows * a24::kGroupBlocks) != 0
        || K % a24::kUnitCols != 0) {
        std::fprintf(stderr, "HeteroSparse_DevicePackA2_Offsets: need M %% 128 == 0, K %% 128 == 0 and non-null pointers (M=%d K=%d)\n", M, K);
        return tcsl_error_invalid_value();
    }
    return a24_launch_residual_offsets(stream, A2_d, M, K, Offsets_d, LongestList_d);
}

extern "C" int HeteroSparse_DevicePackA2_Words(void* stream, const void* A2_d, int M, int K, const int* Offsets_d, void* Words_d)
{
    if (!A2_d || !Offsets_d || !Words_d || M <= 0 || K <= 0 || M % (a24::kRows * a24::kGroupBlocks) != 0
        || K % a24::kUnitCols != 0) {
        std::fprintf(stderr, "HeteroSparse_DevicePackA2_Words: need M %% 128 == 0, K %% 128 == 0 and non-null pointers (M=%d K=%d)\n", M, K);
        return tcsl_error_invalid_value();
    }
    return a24_launch_residual_words(stream, A2_d, M, K, Offsets_d, Words_d);
}

namespace {

// The 2:4 kernel in its shared-tile layout with more than one batch, through to the finished C:
// the launch sums its own slabs where a page of arrival counters can be had (and the caller does
// not ask for the second kernel), else the reduction kernel follows.
int a24_split_call(void* stream, const void* Packed_A1, const void* B, long ldb, void* C, long ldc, int M, int N, int K,
                   void* Reduction_Workspace, int Split_K, int row_blocks, int waves, int loads, const void* words,
                   const void* offsets, int relu, bool separate_reduction, bool row_major)
{
    const long mn = static_cast<long>(M) * N;
    int page = -1;
    std::unique_lock<std::mutex> page_lock;
    // (up to 16 tokens: with more, the slabs' trip through memory inside the launch costs more than
    // the second kernel: 9216 x 9216 at 60 % sparsity and N = 64 39.8 us against 35.2)
    if (!separate_reduction && N <= 16 && M / (16 * row_blocks * waves) <= 4096) {
        page_lock = std::unique_lock<std::mutex>(counter_pages().mutex());
        page = counter_page(stream);
    }
    int rc = a24_launch_spmm(stream, Packed_A1, B, Reduction_Workspace, M, N, K, Split_K, row_blocks, waves, 1, ldb, M, mn, loads,
                             words, offsets, page >= 0 ? relu : 0, page, page >= 0 ? C : nullptr, ldc, row_major ? 1 : 0);
    if (rc == 0 && tcsl::CounterPages::recycled(page))
        rc = tcsl_page_mark(page, stream);
    if (page_lock.owns_lock())
        page_lock.unlock();
    if (rc != 0 || page >= 0)
        return rc;
    if (row_major)  // C is as dense as the slabs: one flat vector
        return tcsl_launch_reduce(stream, C, static_cast<uint16_t*>(Reduction_Workspace), mn, 1, mn, Split_K, relu);
    return tcsl_launch_reduce(stream, C, static_cast<uint16_t*>(Reduction_Workspace), M, N, ldc, Split_K, relu);
}

int fused_call(const char* who, void* stream, const void* Packed_A1, const void* A2_Words, const int* A2_Offsets, int LongestList,
               const void* B, long ldb, void* C, long ldc, int M, int N, int K, void* Reduction_Workspace, int Split_K, int Flags,
               bool row_major = false)
{
    if (N != 8 && N != 16 && N != 32 && N != 64) {
        std::printf("MM_Sparse_API Error: Unsupported N dimension %d!\n", N);  // csrc/SpMM_API.cu:192-193
        return tcsl_error_unknown();
    }
    // two row blocks per wave, activation tile shared through LDS: the one layout that takes the residual along
    // up to five rounds of 64 words travel with a unit's records; what a longer list holds beyond them
    // is fetched where it is needed (a24_kernels.hip)
    const int rounds = (LongestList + 63) / 64;
    const int loads = rounds < HETERO_FUSED_PIPELINED_ROUNDS ? rounds : HETERO_FUSED_PIPELINED_ROUNDS;
    // (four waves for the longest lists at 64 tokens: what fits the registers)
    const int waves = (N == 64 && loads >= (row_major ? 4 : 5)) ? 4 : a24_waves_for(M > 0 ? M : 128, Split_K);
    if (!Packed_A1 || !A2_Words || !A2_Offsets || !B || !C || LongestList < 0 || LongestList > HETERO_FUSED_MAX_LIST
        || !a24_shape_ok(M, N, K, Split_K, 2, waves, 1) || (Split_K > 1 && !Reduction_Workspace) || ldb < K || ldc < M
        || ldb % 8 != 0 || ldc % 8 != 0 || (Flags & ~(SPMM_FLAG_RELU | SPMM_FLAG_SEPARATE_REDUCTION))) {
        std::fprintf(stderr, "%s: unsupported call M=%d N=%d K=%d Split_K=%d LongestList=%d ldb=%ld ldc=%ld (need M %% 128 == 0, K %% 128 == 0, no empty batch, lists of at most %d words, strides that are multiples of 8 and hold a vector, non-null pointers)\n",
                     who, M, N, K, Split_K, LongestList, ldb, ldc, HETERO_FUSED_MAX_LIST);
        return tcsl_error_invalid_value();
    }
    const int relu = (Flags & SPMM_FLAG_RELU) ? 1 : 0;
    const long mn = static_cast<long>(M) * N;
    if (Split_K == 1)
        return a24_launch_spmm(stream, Packed_A1, B, C, M, N, K, 1, 2, waves, 1, ldb, ldc, mn, loads, A2_Words, A2_Offsets, relu, -1,
                               nullptr, 0, row_major ? 1 : 0);
    return a24_split_call(stream, Packed_A1, B, ldb, C, ldc, M, N, K, Reduction_Workspace, Split_K, 2, waves, loads, A2_Words,
                          A2_Offsets, relu, (Flags & SPMM_FLAG_SEPARATE_REDUCTION) != 0, row_major);
}

}  // namespace

extern "C" int HeteroSparse_Fused_SpMM_API(void* stream, const void* Packed_A1, const void* A2_Words, const int* A2_Offsets,
                                           int LongestList, const void* B, void* C, int M, int N, int K,
                                           void* Reduction_Workspace, int Split_K)
{
    return fused_call("HeteroSparse_Fused_SpMM_API", stream, Packed_A1, A2_Words, A2_Offsets, LongestList, B, K, C, M, M, N, K,
                      Reduction_Workspace, Split_K, 0);
}

extern "C" int HeteroSparse_Fused_SpMM_API_Strided(void* stream, const void* Packed_A1, const void* A2_Words,
                                                   const int* A2_Offsets, int LongestList, const void* B, long ldb, void* C,
                                                   long ldc, int M, int N, int K, void* Reduction_Workspace, int Split_K,
                                                   int Flags)
{
    return fused_call("HeteroSparse_Fused_SpMM_API_Strided", stream, Packed_A1, A2_Words, A2_Offsets, LongestList, B, ldb, C, ldc,
                      M, N, K, Reduction_Workspace, Split_K, Flags);
}

extern "C" int HeteroSparse_Fused_SpMM_API_RowMajor(void* stream, const void* Packed_A1, const void* A2_Words,
                                                    const int* A2_Offsets, int LongestList, const void* B, void* C, int M,
                                                    int N, int K, void* Reduction_Workspace, int Split_K, int Flags)
{
    return fused_call("HeteroSparse_Fused_SpMM_API_RowMajor", stream, Packed_A1, A2_Words, A2_Offsets, LongestList, B, K, C, M, M, N,
                      K, Reduction_Workspace, Split_K, Flags, true);
}
