/*
 * libSpMM_API.so -- MI355X (gfx950) implementation of the Tiled-CSL sparse
 * weight x dense activation product.  Plain C ABI: every symbol is extern "C",
 * arguments are raw pointers and ints, no HIP or torch types appear.
 *
 * Each entry point names the reference interface it stands in for (paths are
 * relative to the reference checkout).  The reference's own symbols are C++
 * (mangled) except GenSparseMatrixBinFile; here all of them are C symbols with
 * the same names and the same argument order.
 *
 * Data layout
 *   A            row-major M x K fp16 (A[m*K + k]); only read by the encoder.
 *   Compressed_A packed words, one per kept element plus zero padding to a
 *                multiple of 4 per 128x64 tile: bits 0-15 fp16 value, bits 16-31
 *                row*64 + (col ^ ((row % 8) << 3)) within the tile.
 *   TileOffsets  (M/128)*(K/64) + 2 ints, in units of 4 words; tile t (row-major
 *                over tiles) owns words [4*TileOffsets[t], 4*TileOffsets[t+1]);
 *                the last two entries are equal.
 *   B            activations, one contiguous K vector per token:  B[n*K + k].
 *   C            result, one contiguous M vector per token:       C[n*M + m].
 *                (the column-major convention of csrc/MatMulUtilities.cuh:15-18,
 *                the one the FasterTransformer caller uses, third_party/ft.patch:2823-2846)
 */
#ifndef TILED_CSL_SPMM_API_H
#define TILED_CSL_SPMM_API_H

#include <stdint.h>

#define SPMM_EXPORT __attribute__((visibility("default")))

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Host encoder.  Stands in for
 *   int InitSparseMatrixA_API(half* A_h, int M, int N, int K, uint32_t** Compressed_A, int** TileOffsets)
 *   (declared build/SpMM_API.cuh:55, defined csrc/SpMM_API.cu:241-438).
 * A_h holds fp16 bit patterns; N is ignored, as in the reference.  On success
 * *Compressed_A and *TileOffsets are malloc()ed (the caller frees them, with
 * free() or SpMM_FreeHost) and the number of TileOffsets entries is returned;
 * the word count is 4 * (*TileOffsets)[ret - 1].  Output is bit-identical to the
 * reference's.  Where the reference asserts or exits, a negative code comes back
 * and nothing is allocated:  -1 M % 128 or K % 64 != 0 (or not positive),
 * -2 out of memory, -3 null pointer, -5 more than 2^31-1 vectors.
 * Re-entrant.  Uses up to 16 host threads (SPMM_ENCODE_THREADS overrides).
 */
SPMM_EXPORT int InitSparseMatrixA_API(const uint16_t* A_h, int M, int N, int K, uint32_t** Compressed_A, int** TileOffsets);

/*
 * The encoder without its bank-aware reordering.  Stands in for
 *   int InitSparseMatrixA_API_NoReorder(half* A_h, int M, int N, int K, uint32_t** Compressed_A, int** TileOffsets)
 *   (declared build/SpMM_API.cuh:57-62, defined csrc/SpMM_API.cu:441-567), the reference's
 *   ablation of "ahead of time sparse data reordering".
 * Same conventions and return codes as InitSparseMatrixA_API, same TileOffsets; the words of a
 * tile come in scan order.  Bit-identical to the reference's, including that a padding word
 * carries the bits of the element it points at (+0 normally, but -0 or a NaN pattern if that is
 * what the matrix holds there).  Every SpMM entry point accepts either encoding: a word carries
 * its own position.
 */
SPMM_EXPORT int InitSparseMatrixA_API_NoReorder(const uint16_t* A_h, int M, int N, int K, uint32_t** Compressed_A,
                                                int** TileOffsets);

/*
 * The product C = A * B on the GPU.  Stands in for
 *   cudaError_t SpMM_SplitK_API(cudaStream_t stream, const half* A, const uint4* Compressed_A,
 *                               const int* TileOffsets, const half* B, half* C,
 *                               int M_Global, int N_Global, int K_Global,
 *                               half* Reduction_Workspace, int Split_K)
 *   in the 11-argument form its caller uses (third_party/ft.patch:2833-2843; this
 *   checkout's declaration, build/SpMM_API.cuh:40-52, carries two extra operands of
 *   an unrelated format; dispatch and semantics csrc/SpMM_API.cu:79-208).
 * stream is a hipStream_t (NULL = the default stream).  A is unused and may be
 * NULL.  All other pointers are device memory owned by the caller.  The call
 * only enqueues work on `stream`; it never synchronises.
 *   Split_K == 1: C is written directly, the workspace is not touched.
 *   Split_K  > 1: batch b of ceil((K/64)/Split_K) column tiles writes fp16 partial
 *                 sums to Reduction_Workspace[b*M*N ..), then C = fp16(sum in fp32), added
 *                 up in batch order either by the last workgroup of the same launch to
 *                 finish a tile row (launch shape "mode 1" with few batches, M <= 524288) or
 *                 by a second kernel (same bits either way; the planner takes the cheaper,
 *                 SpMM_PlanReductionInLaunch tells which).
 *                 Reduction_Workspace must hold Split_K*M*N fp16 values and may be
 *                 shared by successive calls on one stream.
 * Accumulation is fp32.  Returns the hipError_t value: 0 on success;
 * hipErrorUnknown, after printing the reference's message, for N outside
 * {8, 16, 32, 64} (csrc/SpMM_API.cu:192-193); hipErrorInvalidValue for M % 128,
 * K % 64, Split_K < 1, Split_K > 65535 or a null pointer (the reference checks these only in
 * debug builds, :93-98, and requires M % 256).  Nothing is launched on error.
 * Thread safe.  The in-launch reduction counts arrivals in a static device array of counter
 * pages (4 MiB per GPU), and two launches that might overlap never count on the same page:
 * an eager call uses the page of its stream handle (the first 32 handles keep theirs for good;
 * later ones share 32 pages, each guarded by an event that the call records behind its launch,
 * and when all have owners the least recently used one whose last launch has finished changes
 * hands; if none has, this call runs the second kernel instead), a call recorded into a HIP graph
 * the page of its (capture, stream) (192 pages, kept until the process ends, because the graph
 * may be replayed at any time; beyond them captured calls run the second kernel).  The per-thread
 * default stream (hipStreamPerThread: one handle value, a different stream in every host thread)
 * counts per calling thread.  What remains the caller's duty: two executable graphs instantiated
 * from the same capture must not run at the same time, and a stream must have finished its work
 * (hipStreamSynchronize) before it is destroyed: the runtime may hand the next stream the same
 * handle, and launches on it would then count where the old stream's last launch still does.
 */
SPMM_EXPORT int SpMM_SplitK_API(void* stream, const void* A, const void* Compressed_A, const int* TileOffsets, const void* B,
                    void* C, int M_Global, int N_Global, int K_Global, void* Reduction_Workspace, int Split_K);

/*
 * SpMM_SplitK_API for callers that must not allocate and have no workspace to pass: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the
 * reference, whose caller allocates 128 MiB once (third_party/ft.patch:2762-2765).  Same
 * arguments without Reduction_Workspace, same checks, same results bit for bit: the slabs of
 * partial sums and the arrival counters of the in-launch reduction live in a static device array
 * of 32 MiB + 16 KiB that every GPU the library runs on holds until the process ends.  The call
 * allocates and frees nothing (neither does SpMM_SplitK_API itself; here the caller need not
 * either).  hipErrorInvalidValue, with a message, when Split_K*M*N*2 exceeds 32 MiB (every
 * OPT-30B/66B/175B layer shape fits with the planner's Split_K up to 64 tokens).  All calls on a
 * GPU share that one array: calls of this entry point that may overlap on one GPU (different
 * streams, concurrent graph launches) race and must be ordered by the caller; calls on one
 * stream are ordered already.
 */
SPMM_EXPORT int SpMM_SplitK_API_StaticWorkspace(void* stream, const void* A, const void* Compressed_A,
                                                const int* TileOffsets, const void* B, void* C, int M_Global,
                                                int N_Global, int K_Global, int Split_K);

/*
 * SpMM_SplitK_API for row-major operands: B[k*N + n] (K x N) and C[m*N + n] (M x N), with
 * the split-K slabs in the same M x N layout.  This is the convention of this checkout's
 * kernel (csrc/SpMM_Kernel.cuh:372-374 for B, :731-734 for the output; its benchmark passes a
 * transposed B and transposes C back, kernel_benchmark/spmm_test.cu:137-141,474,569-576),
 * whereas SpMM_SplitK_API keeps the column-major one of the original interface and of the
 * FasterTransformer caller.  Same arguments, checks and return codes.  The activation
 * block of every tile is contiguous in this layout; the kernel stages it in LDS as it sits in
 * memory and reads it back transposed, which makes this entry as fast as the column-major one
 * (2 % faster on OPT-30B FFN1 at 16 tokens, 4 % slower at 64).
 */
SPMM_EXPORT int SpMM_SplitK_API_RowMajor(void* stream, const void* A, const void* Compressed_A, const int* TileOffsets,
                                         const void* B, void* C, int M_Global, int N_Global, int K_Global,
                                         void* Reduction_Workspace, int Split_K);

/*
 * SpMM_SplitK_API (column-major operands) for activations and results that sit inside
 * wider per-token buffers, with an optional fused clamp: B[n*ldb + k], C[n*ldc + m],
 * ldb >= K, ldc >= M, both multiples of 8 elements; Flags = 0 or a sum of SPMM_FLAG_RELU
 * (C = max(A*B, 0)) and SPMM_FLAG_SEPARATE_REDUCTION.  This is what chaining the layers of a decoder block needs without
 * copies: the attention output projection reads a slice of the fused QKV result, and the
 * first feed-forward product is followed by ReLU (third_party/ft.patch:513-632 runs that
 * activation as a separate kernel).  hipErrorInvalidValue for strides that do not fit.
 * Fastest when B and ldb keep every token vector on a 128-byte boundary (ldb a multiple of 64
 * elements): a vector that straddles cache lines costs 7 % (N = 16) to 14 % (N = 64).
 */
#define SPMM_FLAG_RELU 1
#define SPMM_FLAG_SEPARATE_REDUCTION 2 /* Split_K > 1: always run the reduction as its own kernel */
#define SPMM_FLAG_ADAPTIVE_WAVES 4     /* SpMM_SplitK_API_Planned only: treat Waves (Mode 1, N <= 32) the way a planned
                                          call does, as the count for dense tile rows, and launch eight */
SPMM_EXPORT int SpMM_SplitK_API_Strided(void* stream, const void* Compressed_A, const int* TileOffsets, const void* B,
                                        long ldb, void* C, long ldc, int M_Global, int N_Global, int K_Global,
                                        void* Reduction_Workspace, int Split_K, int Flags);

/*
 * SpMM_SplitK_API_RowMajor with the flags of SpMM_SplitK_API_Strided (the clamp, the reduction as a
 * kernel of its own).  A chain of layers in this fork's layout needs no strides: a product's
 * result C[M][N] is the next product's B[K][N] as it stands, and the output projection's input, the
 * first third of the fused QKV result, is that result's first K rows.
 */
SPMM_EXPORT int SpMM_SplitK_API_RowMajor_Flags(void* stream, const void* Compressed_A, const int* TileOffsets, const void* B,
                                               void* C, int M_Global, int N_Global, int K_Global, void* Reduction_Workspace,
                                               int Split_K, int Flags);

/*
 * SpMM_SplitK_API with two hipEvent_t recorded on `stream` immediately before and
 * after the main kernel (the split-K reduction, if any, follows KernelEnd), so a
 * benchmark can time that kernel alone inside its own loop.  Either event may be
 * NULL.  The SpMM_Event* helpers create and read such events without HIP headers.
 * No counterpart in the reference, whose harness times whole calls with cudaEvents
 * (kernel_benchmark/spmm_test.cu:467-561).
 */
SPMM_EXPORT int SpMM_SplitK_API_Events(void* stream, const void* A, const void* Compressed_A, const int* TileOffsets,
                                       const void* B, void* C, int M_Global, int N_Global, int K_Global,
                                       void* Reduction_Workspace, int Split_K, void* KernelBegin, void* KernelEnd);
/*
 * The first half of SpMM_SplitK_API alone: batch b's fp16 partial sums go to
 * Partials[b*M*N ..) (Split_K*M*N values; with Split_K == 1 that is the product itself)
 * and no reduction follows.  Lets a caller fuse its own reduction, and lets a benchmark
 * time the main kernel back to back.  Same checks and return codes as SpMM_SplitK_API
 * (nothing is printed).  The reference has no such entry point; its kernel writes the
 * same slabs (csrc/SpMM_Kernel.cuh:731-734).
 */
SPMM_EXPORT int SpMM_SplitK_Partials(void* stream, const void* Compressed_A, const int* TileOffsets, const void* B,
                                     void* Partials, int M_Global, int N_Global, int K_Global, int Split_K);
SPMM_EXPORT void* SpMM_EventCreate(void);
SPMM_EXPORT void SpMM_EventDestroy(void* event);
SPMM_EXPORT int SpMM_EventRecord(void* event, void* stream);
/* Waits for `stop`; milliseconds between the two events, negative on error. */
SPMM_EXPORT float SpMM_EventElapsedMs(void* start, void* stop);

/*
 * File-to-file encoder used by model converters.  Stands in for
 *   extern "C" void GenSparseMatrixBinFile(char* DenseMatrixFileName, int M, int K,
 *                                          char* NZWeightsFileName, char* TileOffsetsFileName,
 *                                          char* OutputSizesFileName)
 *   (defined csrc/SpMM_API.cu:1565-1620; called through ctypes by
 *   end2end_inference/ft_tools/huggingface_opt_convert_Phase2.py:36-59).
 * Reads M*K fp16 values, writes the packed words (uint32), the offsets (int32)
 * and two int32 {word count, number of offsets}.  Returns 0, or a negative code
 * (-4 file error, otherwise as InitSparseMatrixA_API) where the reference exits.
 */
SPMM_EXPORT int GenSparseMatrixBinFile(char* DenseMatrixFileName, int M, int K, char* NZWeightsFileName,
                           char* TileOffsetsFileName, char* OutputSizesFileName);

/*
 * The encoder on the GPU, for weights that are already in device memory (row-major M x K
 * fp16 at A_d): same bits as InitSparseMatrixA_API.  Two steps, because the caller owns
 * the output buffers and their size depends on the data:
 *   SpMM_DeviceEncodeOffsets  fills TileOffsets_d ((M/128)*(K/64) + 2 ints);
 *                             the last entry, V, is the number of 16-byte vectors
 *                             (-1 if it would not fit an int);
 *   SpMM_DeviceEncodeItems    fills Compressed_A_d (16 * V bytes) from A_d and those offsets.
 * Both only enqueue kernels on `stream`; read V back (after synchronising) to size the
 * second buffer, or allocate the worst case M*K*4 + 16*tiles bytes up front.  Return a
 * hipError_t value; hipErrorInvalidValue for M % 128, K % 64 or null pointers.  The
 * reference encodes on one host thread only (csrc/SpMM_API.cu:241-438).
 */
SPMM_EXPORT int SpMM_DeviceEncodeOffsets(void* stream, const void* A_d, int M, int K, int* TileOffsets_d);
SPMM_EXPORT int SpMM_DeviceEncodeItems(void* stream, const void* A_d, int M, int K, const int* TileOffsets_d,
                                       void* Compressed_A_d);

/* free() for buffers returned by InitSparseMatrixA_API (for callers without a C runtime at hand). */
SPMM_EXPORT void SpMM_FreeHost(void* p);

/* Text for a code returned by SpMM_SplitK_API. */
SPMM_EXPORT const char* SpMM_GetErrorString(int code);

/*
 * The Split_K that the library's launch planner expects to be fastest for this shape
 * on an MI355X (256 compute units); the counterpart of the reference's hand-tuned
 * per-shape table (kernel_benchmark/benchmark.sh:15, huggingface_opt_convert_Phase2.py:20).
 * Measured optima are built in for the OPT-30B and OPT-66B layer shapes; other shapes
 * go through an analytic cost model.  Returns 1 for shapes the kernels do not take.
 */
SPMM_EXPORT int SpMM_SuggestSplitK(int M_Global, int N_Global, int K_Global);

/*
 * SpMM_SuggestSplitK for a caller that knows how much the weight holds: Vectors = the last entry of
 * its TileOffsets (16-byte vectors of packed words; a converter has it at hand when it writes
 * SplitK_List, huggingface_opt_convert_Phase2.py:189-195).  Optima measured at 70, 80 and 90 %
 * sparsity are built in for the OPT-30B and OPT-66B shapes; the weight's bytes per tile pick the
 * table (boundaries at 75 and 85 %), other shapes go through the cost model with their real bytes
 * per tile.  A later SpMM_SplitK_API call with that Split_K finds the matching launch shape again
 * (it searches every table for the shape and Split_K).  Vectors <= 0 = not known (same as
 * SpMM_SuggestSplitK).  Returns 1 for shapes the kernels do not take.
 */
SPMM_EXPORT int SpMM_SuggestSplitK_Bytes(int M_Global, int N_Global, int K_Global, long Vectors);

/*
 * The launch shape SpMM_SplitK_API uses for (M, N, K, Split_K):
 *   Mode 0  the Waves waves of a workgroup take consecutive 128-row tile rows of one
 *           split-K batch (StageB = 1, up to 16 tokens: they share the batch's activation slice,
 *           staged once in LDS; StageB = 2, 32 tokens with 4 or 8 waves and 64 tokens with 4:
 *           they walk the batch in step and share each 64-column activation tile through LDS);
 *   Mode 1  the Waves waves of a workgroup split the batch of one tile row among
 *           themselves and add their accumulators up in LDS.
 * Any output pointer may be NULL.  EstimatedUs is the cost model's figure for the whole
 * call.  Returns 0, or -1 for a shape the kernels do not take.  The reference has one
 * fixed block shape (csrc/SpMM_API.cu:25-71) and nothing like this.
 */
SPMM_EXPORT int SpMM_PlanLaunch(int M_Global, int N_Global, int K_Global, int Split_K, int* Mode, int* Waves, int* StageB,
                                int* LdsBytes, double* EstimatedUs);

/*
 * Where SpMM_SplitK_API adds the Split_K slabs of partial sums up for (M, N, K, Split_K): 1 = inside the
 * main kernel's launch (Mode 1: the last workgroup to finish a tile row sums that row's slabs; what
 * the planner picks for few batches), 0 = with the reduction kernel, the counterpart of the
 * reference's SplitK_Reduction (csrc/Reduction_Kernel.cuh:24-47; Mode 0 always, Mode 1 with many
 * batches or many tokens, where one workgroup pulling every slab of its rows costs more than a
 * second kernel), or Split_K == 1.  Same bits either way.  -1 for a shape the kernels do not take.
 * A call may still fall back to the reduction kernel (SPMM_FLAG_SEPARATE_REDUCTION, no free counters).
 */
SPMM_EXPORT int SpMM_PlanReductionInLaunch(int M_Global, int N_Global, int K_Global, int Split_K);

/*
 * SpMM_SplitK_API with the launch shape given by the caller instead of the planner
 * (for tuning a table of plans on the target machine, and for tests).  Returns
 * hipErrorInvalidValue when the shape does not fit (Waves above 8, or 4 for N = 64;
 * StageB with Mode 1 or RowMajor, StageB = 1 with N > 16, StageB = 2 outside the shapes above;
 * more than 160 KiB of LDS).  RowMajor != 0 selects
 * the operand layout of SpMM_SplitK_API_RowMajor; Flags as for SpMM_SplitK_API_Strided.  No
 * counterpart in the reference.
 */
SPMM_EXPORT int SpMM_SplitK_API_Planned(void* stream, const void* Compressed_A, const int* TileOffsets, const void* B,
                                        void* C, int M_Global, int N_Global, int K_Global, void* Reduction_Workspace,
                                        int Split_K, int Mode, int Waves, int StageB, int RowMajor, int Flags);

/*
 * Deterministic synthetic inputs for tests and benchmarks (host memory, fp16 bit
 * patterns): Bernoulli or Beta(2,8)-row-skewed sparsity with N(0, 0.02) weights,
 * N(0, 1) activations.  No counterpart in the reference, whose harness uses
 * unseeded rand() (kernel_benchmark/spmm_test_utils.h:108-141).
 */
SPMM_EXPORT void SpMM_SynthWeights(uint16_t* A_h, int M, int K, double sparsity, int row_skewed, uint64_t seed);
SPMM_EXPORT void SpMM_SynthActivations(uint16_t* B_h, long count, uint64_t seed);
/*
 * The value pattern of the reference's own harness, init_host_matrices
 * (kernel_benchmark/spmm_test_utils.h:111-141): every kept weight is exactly 1.0 and every
 * activation one of -5, -3, -1, 1, 3, here with the seeded keep decisions of SpMM_SynthWeights
 * (a weight drawn with the same arguments has its non-zeros in the same places) instead of rand().
 * All products and partial sums are small integers, exact in fp32: the whole output of a product
 * can be compared bit for bit.
 */
SPMM_EXPORT void SpMM_SynthHarnessWeights(uint16_t* A_h, int M, int K, double sparsity, int row_skewed, uint64_t seed);
SPMM_EXPORT void SpMM_SynthHarnessActivations(uint16_t* B_h, long count, uint64_t seed);

/*
 * Device-to-device streaming copy of `bytes` (multiple of 16) on `stream`; a
 * transfer of known size against which hardware byte counters are calibrated.
 * No counterpart in the reference.
 */
SPMM_EXPORT int SpMM_CalibrationCopy(void* stream, void* dst, const void* src, long bytes);

/*
 * ---- 2:4 part on the sparse matrix cores + Tiled-CSL residual ------------------------------
 * This checkout's own line of work: a weight is split into A1, with at most two kept values in
 * every group of four along K (the shape sparse matrix cores take), and the residual A2, which
 * stays in Tiled-CSL; C = A1*B + A2*B.  The reference builds A1's device form for NVIDIA's mma.sp
 * (csrc/SpMM_API.cu:1127-1553) and passes it through two extra operands of SpMM_SplitK_API
 * (build/SpMM_API.cuh:40-52), with A2 going to a second kernel on another stream
 * (kernel_benchmark/spmm_test.cu:285-330,462-560).  Here A1 is stored as records in the operand
 * order of gfx950's v_smfmac_f32_16x16x32_f16 (16 rows x 128 columns, 2304 bytes: 2048 bytes of
 * fp16 values, 256 bytes of 2-bit positions; 1.125 bytes per dense element at any sparsity), the
 * records of eight consecutive 16-row blocks stored together unit by unit.
 */

/*
 * Stands in for  void decompose(half* A, half* A1, half* A2, int length)
 * (kernel_benchmark/spmm_decompose.h:12-51), bit for bit: in each group of four consecutive
 * elements the first two that compare unequal to zero (NaN counts, -0 does not) go to A1, the
 * others to A2; everything else is +0.  Host memory, fp16 bit patterns, Length % 4 == 0.
 * Returns 0, -1 (bad length) or -3 (null pointer) where the reference asserts; prints nothing.
 */
SPMM_EXPORT int HeteroSparse_Decompose(const uint16_t* A_h, uint16_t* A1_h, uint16_t* A2_h, long Length);

/*
 * Stand in for InitSparseMatrixA1_Vec_Sparse_Load and inspect_metadata (csrc/SpMM_API.cu:1127-1553),
 * which produce mma.sp's value and metadata arrays; the bytes differ by design (other hardware).
 * HeteroSparse_PackedBytes: size of the records of an M x K matrix (M % 128 == 0, K % 128 == 0), or -1.
 * HeteroSparse_PackA1: fills Packed_h (host memory of that size) from row-major A1_h.  Returns 0,
 * -1 bad shape, -3 null pointer, -6 if some group of four holds more than two kept values.
 */
SPMM_EXPORT long HeteroSparse_PackedBytes(int M, int K);
SPMM_EXPORT int HeteroSparse_PackA1(const uint16_t* A1_h, int M, int K, void* Packed_h);

/*
 * Split and pack on the GPU, for a weight that is already in device memory (row-major M x K fp16 at
 * A_d, M % 128 == 0, K % 128 == 0): Packed_A1_d receives the records (HeteroSparse_PackedBytes bytes),
 * A2_d, if not NULL, the dense residual (M*K fp16, zero where nothing is left), ready for
 * SpMM_DeviceEncodeOffsets / SpMM_DeviceEncodeItems.  Same bits as HeteroSparse_Decompose followed by
 * HeteroSparse_PackA1.  Only enqueues a kernel on `stream`; returns a hipError_t value.  The reference
 * does both steps on one host thread (kernel_benchmark/spmm_test.cu:285-330).
 */
SPMM_EXPORT int HeteroSparse_DeviceSplitPack(void* stream, const void* A_d, int M, int K, void* Packed_A1_d, void* A2_d);

/*
 * C = A1*B + A2*B on the GPU; the counterpart of this checkout's 13-argument SpMM_SplitK_API call
 * followed by its residual kernel and reduction (kernel_benchmark/spmm_test.cu:462-560).
 * Packed_A1: device copy of the records; Compressed_A2 / TileOffsets_A2: device Tiled-CSL of the
 * residual (InitSparseMatrixA_API on A2), or both NULL when there is none.  B[N][K], C[N][M] as
 * for SpMM_SplitK_API.  The 2:4 kernel writes Split_K_A1 slabs of fp16 partial sums, the
 * Tiled-CSL kernel Split_K_A2 more, and one reduction adds them up in fp32: Reduction_Workspace
 * must hold (Split_K_A1 + Split_K_A2)*M*N fp16 values.  With no residual and Split_K_A1 == 1 the
 * workspace is not touched.  HeteroSparse_SuggestSplitK gives a Split_K_A1 that fills the chip.
 * The kernels run one after the other on `stream`.  Flags = HETERO_FLAG_TWO_STREAMS sends the
 * residual's kernel to a second stream that the library keeps per caller stream (default priority,
 * made on first use; the reference gives the two parts their own streams,
 * kernel_benchmark/spmm_test.cu:459-461), ordered after what `stream` held before the call, with
 * the reduction on `stream` waiting for both; on an MI355X that measured slower than one stream.
 * Returns a hipError_t value: hipErrorUnknown for N outside {8, 16, 32, 64};
 * hipErrorInvalidValue for M % 128, K % 128, a split that leaves a batch of 128-column units
 * empty, or a missing pointer.  Only enqueues work on `stream`.  Thread safe.
 */
#define HETERO_FLAG_TWO_STREAMS 1
SPMM_EXPORT int HeteroSparse_SpMM_API(void* stream, const void* Packed_A1, const void* Compressed_A2,
                                      const int* TileOffsets_A2, const void* B, void* C, int M_Global, int N_Global,
                                      int K_Global, void* Reduction_Workspace, int Split_K_A1, int Split_K_A2, int Flags);
SPMM_EXPORT int HeteroSparse_SuggestSplitK(int M_Global, int N_Global, int K_Global);

/*
 * The 2:4 kernel alone: batch b of ceil((K/128)/Split_K) units writes fp16 A1*B partial sums to
 * Partials[b*M*N ..).  RowBlocks, Waves and ShareB choose the launch shape; 0, 0 = the library's
 * choice (ShareB is then ignored).
 *   ShareB = 1  each of the Waves (2, 4, 8) waves of a workgroup owns RowBlocks (2 or 4; 2 for N = 64)
 *               16-row blocks and all share the activation tile through LDS; RowBlocks * Waves >= 8 and
 *               M % (16 * RowBlocks * Waves) == 0.  The library's own launches are of this kind.
 *   ShareB = 0  a workgroup owns RowBlocks (1, 2, 4, 8) blocks; its Waves (1, 2, 4, 8) waves split the
 *               batch's columns and add their sums up.
 * hipErrorInvalidValue for shapes the kernel tables do not hold.  For tuning and tests.
 */
SPMM_EXPORT int HeteroSparse_A1_Partials(void* stream, const void* Packed_A1, const void* B, void* Partials, int M_Global,
                                         int N_Global, int K_Global, int Split_K, int RowBlocks, int Waves, int ShareB);

/*
 * Both parts in one launch.  The reference multiplies the residual with a kernel of its own on a
 * second stream (kernel_benchmark/FSP_Batch8.h:129-206, launched at
 * kernel_benchmark/spmm_test.cu:462-560); here the 2:4 kernel can take the residual along: every
 * wave scatters the residual values of its 16 x 128 blocks into a dense image in LDS and multiplies
 * that on the ordinary matrix cores, against the activation tile and into the accumulators that the
 * 2:4 part uses, so the activations are read once and nothing is added up afterwards.
 *
 * HeteroSparse_PackA2: the residual in the form that launch reads, from row-major A2_h (M x K fp16
 * bit patterns in host memory, M % 128 == 0, K % 128 == 0): *Words (fp16 value | position << 16, one
 * list per 16 x 128 block, 4 bytes per kept value) and *Offsets (list i = words Offsets[i] ..
 * Offsets[i + 1]), both malloc'ed, caller frees; *LongestList = the longest list's length.  *Words
 * holds Offsets[last] + 64 words (copy them all to the device).  Returns the number of offsets,
 * (M / 16) * (K / 128) + 1, or -1 bad shape, -2 out of memory, -3 null pointer.
 *
 * HeteroSparse_Fused_SpMM_API: C = A1*B + A2*B, one kernel (plus the reduction kernel when
 * Split_K > 1: Reduction_Workspace then holds Split_K*M*N fp16 values; HeteroSparse_SuggestSplitK).
 * Device pointers; B[N][K], C[N][M] as for SpMM_SplitK_API.  LongestList as HeteroSparse_PackA2 gave
 * it, at most HETERO_FUSED_MAX_LIST = 1024, which is what a block of a residual can hold, so every
 * residual is accepted.  Lists of up to 320 words (uniform sparsity of 50 % and more stays below) travel
 * with the records' own loads; the words of a longer list (a matrix with some dense rows, e.g.
 * Beta(2,8)-skewed row densities) beyond the 320th are fetched where they are needed, which stalls that
 * wave once per such list: correct at any length, fastest when long lists are rare.  Returns a
 * hipError_t value: hipErrorUnknown for N outside {8, 16, 32, 64}; hipErrorInvalidValue for M % 128,
 * K % 128, an empty batch, a list too long, a missing pointer.  Only enqueues work on `stream`.
 */
/*
 * HeteroSparse_PackA2 on the GPU, for a residual that is already in device memory (the A2_d that
 * HeteroSparse_DeviceSplitPack wrote): the same words in the same order.  Two steps, because the
 * caller owns the buffers and their size depends on the data:
 *   HeteroSparse_DevicePackA2_Offsets  fills Offsets_d ((M/16)*(K/128) + 1 ints; the last one, T, is
 *                                      the number of words, -1 if it would not fit an int) and
 *                                      *LongestList_d (one int);
 *   HeteroSparse_DevicePackA2_Words    fills Words_d (T + 64 words, the last 64 zero) from A2_d and
 *                                      those offsets.
 * Both only enqueue kernels on `stream`; read T and the longest list back (after synchronising) to
 * size the second buffer, or allocate the worst case M*K/2 + 64 words up front.  A2_d must be a
 * residual: at most two kept values in every group of four, hence at most 1024 per 16 x 128 block
 * (a block that holds more gets no words; *LongestList_d shows it).  With T = -1 the second
 * step writes nothing at all: check T before trusting Words_d.  Return a hipError_t value;
 * hipErrorInvalidValue for M % 128, K % 128 or null pointers.
 */
SPMM_EXPORT int HeteroSparse_DevicePackA2_Offsets(void* stream, const void* A2_d, int M_Global, int K_Global, int* Offsets_d,
                                                  int* LongestList_d);
SPMM_EXPORT int HeteroSparse_DevicePackA2_Words(void* stream, const void* A2_d, int M_Global, int K_Global,
                                                const int* Offsets_d, void* Words_d);

#define HETERO_FUSED_MAX_LIST 1024       /* what a 16 x 128 block of a residual can hold: two of every four */
#define HETERO_FUSED_PIPELINED_ROUNDS 5  /* rounds of 64 words that travel with a unit's records */
SPMM_EXPORT int HeteroSparse_PackA2(const uint16_t* A2_h, int M_Global, int K_Global, uint32_t** Words, int** Offsets,
                                    int* LongestList);
SPMM_EXPORT int HeteroSparse_Fused_SpMM_API(void* stream, const void* Packed_A1, const void* A2_Words, const int* A2_Offsets,
                                            int LongestList, const void* B, void* C, int M_Global, int N_Global,
                                            int K_Global, void* Reduction_Workspace, int Split_K);

/*
 * HeteroSparse_Fused_SpMM_API for activations and results inside wider per-token buffers
 * (B[n*ldb + k], C[n*ldc + m], ldb >= K, ldc >= M, multiples of 8 elements) with an optional clamp
 * (Flags = 0 or a sum of SPMM_FLAG_RELU and SPMM_FLAG_SEPARATE_REDUCTION), like SpMM_SplitK_API_Strided:
 * what a chain of decoder layers needs.  With Split_K > 1 and up to 16 tokens the launch adds its
 * slabs up itself (same bits as the reduction kernel, which SPMM_FLAG_SEPARATE_REDUCTION asks for).
 */
SPMM_EXPORT int HeteroSparse_Fused_SpMM_API_Strided(void* stream, const void* Packed_A1, const void* A2_Words,
                                                    const int* A2_Offsets, int LongestList, const void* B, long ldb, void* C,
                                                    long ldc, int M_Global, int N_Global, int K_Global,
                                                    void* Reduction_Workspace, int Split_K, int Flags);

/*
 * The two calls above for row-major operands, the layout of this checkout's own hybrid kernel and
 * benchmark (csrc/SpMM_Kernel.cuh:372-374 for B, :731-734 for the output;
 * kernel_benchmark/spmm_test.cu:137-141,474,569-576): B[k*N + n] (K x N), C[m*N + n] (M x N), both
 * dense, and every slab of partial sums in the workspace M x N as well.  The weight operands are the
 * same records, Tiled-CSL residual or residual lists as for the column-major calls.
 *   HeteroSparse_SpMM_API_RowMajor        arguments, checks and return codes of HeteroSparse_SpMM_API;
 *   HeteroSparse_Fused_SpMM_API_RowMajor  those of HeteroSparse_Fused_SpMM_API plus Flags (0 or a sum of
 *                                         SPMM_FLAG_RELU and SPMM_FLAG_SEPARATE_REDUCTION).  A chain of
 *                                         layers needs no strides in this layout: a result is the next
 *                                         product's B as it stands.
 * The 2:4 kernel stages each unit's 128 x N activation block in LDS as it sits in memory and reads it
 * back with the transposing LDS read, as the Tiled-CSL kernel does for SpMM_SplitK_API_RowMajor.
 */
SPMM_EXPORT int HeteroSparse_SpMM_API_RowMajor(void* stream, const void* Packed_A1, const void* Compressed_A2,
                                               const int* TileOffsets_A2, const void* B, void* C, int M_Global,
                                               int N_Global, int K_Global, void* Reduction_Workspace, int Split_K_A1,
                                               int Split_K_A2, int Flags);
SPMM_EXPORT int HeteroSparse_Fused_SpMM_API_RowMajor(void* stream, const void* Packed_A1, const void* A2_Words,
                                                     const int* A2_Offsets, int LongestList, const void* B, void* C,
                                                     int M_Global, int N_Global, int K_Global, void* Reduction_Workspace,
                                                     int Split_K, int Flags);

#ifdef __cplusplus
}
#endif
#endif
