/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the Tiled-CSL SpMM path.
 *
 * A plain-C restatement of what the reference computes on this path, used as
 * the checker by tests/, by __graft_entry__.smoke() and by the cpu_baseline
 * leg of bench.py.  Nothing in the product (the HIP library or its Python
 * mirror) links, imports or calls this file.
 *
 * Each function cites the reference lines it restates (paths relative to the
 * reference checkout).  How each function is pinned:
 *   oracle_encode        - bit-compared with the reference's own encoder
 *                          compiled from csrc/SpMM_API.cu:210-438 (oracle/_ref)
 *                          and with committed golden vectors made by it;
 *                          hand-derived micro cases; format invariants.
 *   oracle_encode_noreorder - bit-compared with the reference's own
 *                          InitSparseMatrixA_API_NoReorder compiled from
 *                          csrc/SpMM_API.cu:441-567 (oracle/_ref) and with committed
 *                          golden vectors made by it; decode(encode) == A.
 *   oracle_decode        - closed-form inverse of the index packing
 *                          (csrc/SpMM_API.cu:330-339); decode(encode(A)) == A.
 *   oracle_gemm_f32      - textbook fp32-accumulate product; checked against
 *                          numpy float64 on exactly representable inputs and
 *                          one-hot / identity special cases.
 *   oracle_splitk_range  - closed form of csrc/SpMM_Kernel.cuh:312-320;
 *                          partition property checked by brute force.
 *   oracle_reduce        - closed form of csrc/Reduction_Kernel.cuh:36-46.
 *   oracle_spmm_splitk   - composition of the above; sum of slabs equals the
 *                          full product.
 *   half conversions     - exhaustive comparison with numpy float16.
 *   oracle_decompose     - bit-compared with the reference's own decompose()
 *                          compiled from kernel_benchmark/spmm_decompose.h:12-51
 *                          (oracle/_ref) and with committed golden vectors made by it; A1 + A2 == A with disjoint supports; at
 *                          most two kept values per group of four in A1; hand cases.
 *   oracle_a24_unpack    - reader of this build's 2:4 record layout (the reference's
 *                          own on-device form, csrc/SpMM_API.cu:1127-1553, is made for
 *                          NVIDIA's mma.sp and has no meaning here); pinned by
 *                          hand-built records and by unpack(pack(A1)) == A1.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_TILE_ROWS 128 /* csrc/SpMM_API.cu:249  (_TILE_M)            */
#define ORACLE_TILE_COLS 64  /* csrc/TilingConfig.h:29 (TILE_K = 16 * 4)   */
#define ORACLE_BANKS 32      /* csrc/SpMM_API.cu:320                       */
#define ORACLE_VEC 4         /* csrc/SpMM_API.cu:250  (VECTOR_SIZE)        */
#define ORACLE_GROUP 32      /* csrc/TilingConfig.h:25 (WARP_SIZE)         */

/* ---------------------------------------------------------------- fp16 -- */

/* IEEE binary16 -> binary32, exact (what __half2float does). */
float oracle_half_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: renormalise */
            int shift = 0;
            while (!(man & 0x400u)) {
                man <<= 1;
                shift++;
            }
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* binary32 -> binary16, round to nearest even (what __float2half_rn does). */
uint16_t oracle_float_to_half_rn(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t absx = x & 0x7fffffffu;
    if (absx > 0x7f800000u) /* NaN: keep it a quiet NaN */
        return (uint16_t)(sign | 0x7e00u);
    if (absx >= 0x47800000u) /* >= 65536: inf (65520..65536 handled below)   */
        return (uint16_t)(sign | 0x7c00u);
    if (absx < 0x33000000u) /* < 2^-25: rounds to zero                      */
        return sign;
    int e = (int)(absx >> 23) - 127;
    uint32_t m = (absx & 0x7fffffu) | 0x800000u; /* 24-bit significand */
    int drop; /* bits dropped from the 24-bit significand */
    int he;   /* biased half exponent field before carry  */
    if (e < -14) { /* subnormal half */
        drop = 13 + (-14 - e);
        he = 0;
    } else {
        drop = 13;
        he = e + 15;
    }
    uint32_t kept = m >> drop;
    uint32_t rem = m & ((1u << drop) - 1u);
    uint32_t halfway = 1u << (drop - 1);
    if (rem > halfway || (rem == halfway && (kept & 1u)))
        kept++;
    uint32_t out;
    if (he == 0)
        out = kept; /* carry into exponent field is the right result */
    else
        out = ((uint32_t)(he - 1) << 10) + kept; /* kept includes the hidden bit */
    if (out >= 0x7c00u)
        out = 0x7c00u;
    return (uint16_t)(sign | out);
}

/* The reference's non-zero test `fabs(__half2float(v)) > 0.0f`
 * (csrc/SpMM_API.cu:262,285,335): +-0 and NaN are "zero", subnormals and
 * infinities are non-zero. */
static int is_kept(uint16_t h)
{
    float f = oracle_half_to_float(h);
    if (f < 0)
        f = -f;
    return f > 0.0f;
}

/* ------------------------------------------------------------- encoder -- */

typedef struct {
    uint32_t *v;
    int n, cap;
} stack_t;

static void st_push(stack_t *s, uint32_t x)
{
    if (s->n == s->cap) {
        s->cap = s->cap ? 2 * s->cap : 64;
        s->v = (uint32_t *)realloc(s->v, (size_t)s->cap * sizeof(uint32_t));
    }
    s->v[s->n++] = x;
}
static uint32_t st_pop(stack_t *s) { return s->v[--s->n]; }

/* Smallest stack, lowest id on ties (csrc/SpMM_API.cu:210-221). */
static int smallest(const stack_t *b)
{
    int id = 0;
    for (int i = 1; i < ORACLE_BANKS; i++)
        if (b[i].n < b[id].n)
            id = i;
    return id;
}
/* Largest stack, lowest id on ties (csrc/SpMM_API.cu:223-234). */
static int largest(const stack_t *b)
{
    int id = 0;
    for (int i = 1; i < ORACLE_BANKS; i++)
        if (b[i].n > b[id].n)
            id = i;
    return id;
}

/* Tiled-CSL encode (csrc/SpMM_API.cu:241-438).  A is row-major M x K fp16
 * bits.  On success *items (4*offsets[last] words) and *offsets
 * ((M/128)*(K/64)+2 ints) are malloc'd and the number of offsets is
 * returned; -1 for a shape the reference asserts on (:310), -2 for
 * allocation failure. */
int oracle_encode(const uint16_t *A, int M, int K, uint32_t **items, int **offsets)
{
    if (M <= 0 || K <= 0 || M % ORACLE_TILE_ROWS || K % ORACLE_TILE_COLS)
        return -1;
    const int tr = M / ORACLE_TILE_ROWS, tc = K / ORACLE_TILE_COLS;
    const long ntiles = (long)tr * tc;

    /* pass 1: padded length (:278-294) */
    long total = 0;
    for (int i = 0; i < tr; i++)
        for (int j = 0; j < tc; j++) {
            int nz = 0;
            for (int m = 0; m < ORACLE_TILE_ROWS; m++)
                for (int n = 0; n < ORACLE_TILE_COLS; n++)
                    nz += is_kept(A[(size_t)(i * ORACLE_TILE_ROWS + m) * K + j * ORACLE_TILE_COLS + n]);
            total += nz + (ORACLE_VEC - nz % ORACLE_VEC) % ORACLE_VEC;
        }

    uint32_t *out = (uint32_t *)malloc((total ? total : 1) * sizeof(uint32_t));
    int *offs = (int *)malloc((ntiles + 2) * sizeof(int));
    if (!out || !offs) {
        free(out);
        free(offs);
        return -2;
    }

    stack_t bank[ORACLE_BANKS], mainp[ORACLE_GROUP], tailp[ORACLE_GROUP];
    memset(bank, 0, sizeof bank);
    memset(mainp, 0, sizeof mainp);
    memset(tailp, 0, sizeof tailp);

    long written = 0;
    uint32_t *dst = out;
    offs[0] = 0; /* :432 */
    for (int i = 0; i < tr; i++) {
        for (int j = 0; j < tc; j++) {
            int first_zero[ORACLE_BANKS];
            for (int b = 0; b < ORACLE_BANKS; b++) {
                bank[b].n = 0;
                mainp[b].n = 0;
                tailp[b].n = 0;
                first_zero[b] = -1;
            }
            int count = 0;
            /* scan the tile row-major, bucket by LDS bank of the swizzled
             * position (:326-349) */
            for (int m = 0; m < ORACLE_TILE_ROWS; m++)
                for (int n = 0; n < ORACLE_TILE_COLS; n++) {
                    uint16_t v = A[(size_t)(i * ORACLE_TILE_ROWS + m) * K + j * ORACLE_TILE_COLS + n];
                    int swz = n ^ ((m % 8) << 3);
                    int b = (swz / 2) % ORACLE_BANKS;
                    int pos = m * ORACLE_TILE_COLS + swz;
                    if (is_kept(v)) {
                        st_push(&bank[b], (uint32_t)v | ((uint32_t)(uint16_t)(int16_t)pos << 16));
                        count++;
                    } else if (first_zero[b] < 0) {
                        first_zero[b] = pos;
                    }
                }
            /* pad to a multiple of 4 with +0.0 items at a known-zero
             * position of the currently smallest bank (:352-365) */
            int pad = (ORACLE_VEC - count % ORACLE_VEC) % ORACLE_VEC;
            for (int p = 0; p < pad; p++) {
                int b = smallest(bank);
                if (first_zero[b] < 0) { /* reference asserts (:356) */
                    free(out);
                    free(offs);
                    return -3;
                }
                st_push(&bank[b], (uint32_t)(uint16_t)(int16_t)first_zero[b] << 16);
                count++;
            }
            int vecs = count / ORACLE_VEC;
            int rounds = vecs / ORACLE_GROUP, rem = vecs % ORACLE_GROUP;
            /* tail is drawn first (:384-391), then the main part (:394-403) */
            for (int v = 0; v < ORACLE_VEC; v++)
                for (int b = 0; b < rem; b++)
                    st_push(&tailp[b], st_pop(&bank[largest(bank)]));
            for (int r = 0; r < rounds; r++)
                for (int v = 0; v < ORACLE_VEC; v++)
                    for (int b = 0; b < ORACLE_GROUP; b++)
                        st_push(&mainp[b], st_pop(&bank[largest(bank)]));
            /* emission, last-in first-out (:406-424) */
            for (int r = 0; r < rounds; r++)
                for (int v = 0; v < ORACLE_VEC; v++)
                    for (int b = 0; b < ORACLE_GROUP; b++)
                        dst[r * ORACLE_VEC * ORACLE_GROUP + b * ORACLE_VEC + v] = st_pop(&mainp[b]);
            dst += rounds * ORACLE_VEC * ORACLE_GROUP;
            for (int v = 0; v < ORACLE_VEC; v++)
                for (int b = 0; b < rem; b++)
                    dst[b * ORACLE_VEC + v] = st_pop(&tailp[b]);
            dst += rem * ORACLE_VEC;
            written += count;
            offs[(long)i * tc + j + 1] = (int)(written / ORACLE_VEC); /* :427 */
        }
    }
    offs[ntiles + 1] = (int)(written / ORACLE_VEC); /* :433-434 */
    for (int b = 0; b < ORACLE_BANKS; b++) {
        free(bank[b].v);
        free(mainp[b].v);
        free(tailp[b].v);
    }
    if (written != total) {
        free(out);
        free(offs);
        return -4;
    }
    *items = out;
    *offsets = offs;
    return (int)(ntiles + 2);
}

/* Tiled-CSL encode without the bank-aware reordering (csrc/SpMM_API.cu:441-567): the kept
 * elements of a tile in scan order, and, interleaved with them, the first `pad` elements of
 * the scan that are not kept, carrying their own bits as the value (:533-546; normally +0,
 * but -0 and NaN bit patterns are copied as they are).  Same return convention as
 * oracle_encode. */
int oracle_encode_noreorder(const uint16_t *A, int M, int K, uint32_t **items, int **offsets)
{
    if (M <= 0 || K <= 0 || M % ORACLE_TILE_ROWS || K % ORACLE_TILE_COLS)
        return -1;
    const int tr = M / ORACLE_TILE_ROWS, tc = K / ORACLE_TILE_COLS;
    const long ntiles = (long)tr * tc;
    long total = 0;
    for (int i = 0; i < tr; i++)
        for (int j = 0; j < tc; j++) {
            int nz = 0;
            for (int m = 0; m < ORACLE_TILE_ROWS; m++)
                for (int n = 0; n < ORACLE_TILE_COLS; n++)
                    nz += is_kept(A[(size_t)(i * ORACLE_TILE_ROWS + m) * K + j * ORACLE_TILE_COLS + n]);
            total += nz + (ORACLE_VEC - nz % ORACLE_VEC) % ORACLE_VEC;
        }
    uint32_t *out = (uint32_t *)malloc((total ? total : 1) * sizeof(uint32_t));
    int *offs = (int *)malloc((ntiles + 2) * sizeof(int));
    if (!out || !offs) {
        free(out);
        free(offs);
        return -2;
    }
    long w = 0;
    for (int i = 0; i < tr; i++)
        for (int j = 0; j < tc; j++) {
            const uint16_t *tile = A + (size_t)i * ORACLE_TILE_ROWS * K + (size_t)j * ORACLE_TILE_COLS;
            int nz = 0;
            for (int m = 0; m < ORACLE_TILE_ROWS; m++)
                for (int n = 0; n < ORACLE_TILE_COLS; n++)
                    nz += is_kept(tile[(size_t)m * K + n]);
            int pads = (ORACLE_VEC - nz % ORACLE_VEC) % ORACLE_VEC;
            for (int m = 0; m < ORACLE_TILE_ROWS; m++)
                for (int n = 0; n < ORACLE_TILE_COLS; n++) {
                    const uint16_t v = tile[(size_t)m * K + n];
                    const uint32_t pos = (uint32_t)(m * ORACLE_TILE_COLS + (n ^ ((m % 8) << 3)));
                    if (is_kept(v)) {
                        out[w++] = (uint32_t)v | pos << 16;
                    } else if (pads > 0) {
                        pads--;
                        out[w++] = (uint32_t)v | pos << 16;
                    }
                }
            offs[(long)i * tc + j + 1] = (int)(w / ORACLE_VEC);
        }
    offs[0] = 0;
    offs[ntiles + 1] = (int)(w / ORACLE_VEC);
    *items = out;
    *offsets = offs;
    return (int)(ntiles + 2);
}

void oracle_free(void *p) { free(p); }

/* ------------------------------------------------------------- decoder -- */

/* Inverse of the packing at csrc/SpMM_API.cu:330-339: item = value |
 * (row*64 + (col ^ ((row%8)<<3))) << 16.  Rebuilds the dense row-major
 * M x K matrix (zero-filled first, so -0 and NaN inputs come back as +0). */
void oracle_decode(const uint32_t *items, const int *offsets, int M, int K, uint16_t *A_out)
{
    const int tr = M / ORACLE_TILE_ROWS, tc = K / ORACLE_TILE_COLS;
    memset(A_out, 0, (size_t)M * K * sizeof(uint16_t));
    for (int i = 0; i < tr; i++)
        for (int j = 0; j < tc; j++) {
            long t = (long)i * tc + j;
            for (long e = (long)offsets[t] * ORACLE_VEC; e < (long)offsets[t + 1] * ORACLE_VEC; e++) {
                uint32_t it = items[e];
                uint16_t val = (uint16_t)(it & 0xffffu);
                int pos = (int)(it >> 16);
                int r = pos >> 6;
                int c = (pos & 63) ^ ((r & 7) << 3);
                if (val) /* pads carry +0.0 and may share a position */
                    A_out[(size_t)(i * ORACLE_TILE_ROWS + r) * K + j * ORACLE_TILE_COLS + c] = val;
            }
        }
}

/* ---------------------------------------------------------------- GEMM -- */

/* C[n][m] = sum_k float(A[m][k]) * float(B[n][k]), fp32 accumulate in
 * increasing k (the fp32-compute dense product the reference harness uses as
 * truth, kernel_benchmark/spmm_test.cu:170-188).  A row-major M x K;
 * B and C in the library's default layout: one contiguous K-vector (resp.
 * M-vector) per token (csrc/MatMulUtilities.cuh:15-18).  Only k in
 * [k_begin, k_end) is summed, so split-K slabs can be formed. */
void oracle_gemm_f32(const uint16_t *A, const uint16_t *B, float *C, int M, int N, int K, int k_begin, int k_end)
{
    float *brow = (float *)malloc((size_t)K * sizeof(float));
    for (int n = 0; n < N; n++) {
        for (int k = 0; k < K; k++)
            brow[k] = oracle_half_to_float(B[(size_t)n * K + k]);
        for (int m = 0; m < M; m++) {
            float acc = 0.0f;
            const uint16_t *a = A + (size_t)m * K;
            for (int k = k_begin; k < k_end; k++)
                acc += oracle_half_to_float(a[k]) * brow[k];
            C[(size_t)n * M + m] = acc;
        }
    }
    free(brow);
}

/* ------------------------------------------------------------- split-K -- */

/* k-block range of batch b (csrc/SpMM_Kernel.cuh:312-320): blocks of 64
 * columns, ceil(NumKBlock/Split_K) per batch, the last batch takes what is
 * left.  Where the reference's arithmetic would run past the matrix (its
 * last batch count goes negative) the range is clamped to the matrix. */
void oracle_splitk_range(int K, int Split_K, int b, int *kb_begin, int *kb_end)
{
    int nkb = K / ORACLE_TILE_COLS;
    int avg = (nkb - 1) / Split_K + 1;
    long s = (long)b * avg, e = s + avg;
    if (s > nkb)
        s = nkb;
    if (e > nkb)
        e = nkb;
    *kb_begin = (int)s;
    *kb_end = (int)e;
}

/* C[e] = fp16_rn(sum_s float(W[s*MN + e])) (csrc/Reduction_Kernel.cuh:36-46). */
void oracle_reduce(uint16_t *C, const uint16_t *W, long MN, int Split_K)
{
    for (long e = 0; e < MN; e++) {
        float acc = 0.0f;
        for (int s = 0; s < Split_K; s++)
            acc += oracle_half_to_float(W[(size_t)s * MN + e]);
        C[e] = oracle_float_to_half_rn(acc);
    }
}

/* Whole call, original library semantics (csrc/SpMM_API.cu:99-103,198-206):
 * Split_K == 1 writes fp16 C directly; otherwise each batch's fp32 partial is
 * rounded to fp16 into slab b of the workspace and the slabs are reduced.
 * A is taken in compressed form and decoded first.  Returns 0, or -1 on a
 * bad shape. */
int oracle_spmm_splitk(const uint32_t *items, const int *offsets, const uint16_t *B, uint16_t *C, int M, int N, int K,
                       uint16_t *workspace, int Split_K)
{
    if (M % ORACLE_TILE_ROWS || K % ORACLE_TILE_COLS || Split_K < 1 || N < 1)
        return -1;
    uint16_t *A = (uint16_t *)malloc((size_t)M * K * sizeof(uint16_t));
    float *acc = (float *)malloc((size_t)M * N * sizeof(float));
    oracle_decode(items, offsets, M, K, A);
    const long MN = (long)M * N;
    for (int b = 0; b < Split_K; b++) {
        int s, e;
        oracle_splitk_range(K, Split_K, b, &s, &e);
        oracle_gemm_f32(A, B, acc, M, N, K, s * ORACLE_TILE_COLS, e * ORACLE_TILE_COLS);
        uint16_t *dst = (Split_K == 1) ? C : workspace + (size_t)b * MN;
        for (long x = 0; x < MN; x++)
            dst[x] = oracle_float_to_half_rn(acc[x]);
    }
    if (Split_K > 1)
        oracle_reduce(C, workspace, MN, Split_K);
    free(A);
    free(acc);
    return 0;
}


/* ------------------------------------------------- 2:4 + residual split -- */

/*
 * kernel_benchmark/spmm_decompose.h:12-51.  The flat array is cut into groups of
 * four consecutive elements; in each group the first two values that compare
 * unequal to zero as floats (so NaN counts, -0 does not) go to A1 at their own
 * positions, every further one goes to A2.  Both outputs are zero-filled first.
 */
void oracle_decompose(const uint16_t *A, uint16_t *A1, uint16_t *A2, long length)
{
    memset(A1, 0, sizeof(uint16_t) * (size_t)length);
    memset(A2, 0, sizeof(uint16_t) * (size_t)length);
    for (long i = 0; i + 3 < length; i += 4) {
        int taken = 0;
        for (int e = 0; e < 4; e++) {
            if (oracle_half_to_float(A[i + e]) != 0.0f) {
                if (taken < 2)
                    A1[i + e] = A[i + e];
                else
                    A2[i + e] = A[i + e];
                taken++;
            }
        }
    }
}

/*
 * Reader of the 2:4 records that the sparse-MFMA kernel streams.  One record covers
 * 16 rows x 128 columns and is 2304 bytes: for lane L in 0..63 (row L % 16, column
 * group g = L / 16), step s in 0..3 and slot j in 0..3, the fp16 value at byte
 * (s / 2) * 1024 + L * 16 + ((s % 2) * 4 + j) * 2 belongs to column
 * s * 32 + g * 8 + (j / 2) * 4 + q of the record, where q is the 2-bit field at bit
 * 8 * s + 2 * j of the 32-bit word at byte 2048 + L * 4.  Records are ordered by group
 * of eight 16-row blocks, then by 128-column unit, then by block within the group:
 * block rb, unit u is record ((rb / 8) * (K / 128) + u) * 8 + rb % 8 (M % 128 == 0).  Returns 0, or -1 if two slots of one group
 * of four name the same column or come in descending order.
 */
int oracle_a24_unpack(const uint8_t *packed, int M, int K, uint16_t *A_out)
{
    const int units = K / 128;
    memset(A_out, 0, sizeof(uint16_t) * (size_t)M * (size_t)K);
    for (int rb = 0; rb < M / 16; rb++) {
        for (int u = 0; u < units; u++) {
            const uint8_t *rec = packed + (((size_t)(rb / 8) * units + u) * 8 + (size_t)(rb % 8)) * 2304;
            for (int L = 0; L < 64; L++) {
                uint32_t word;
                memcpy(&word, rec + 2048 + L * 4, 4);
                for (int s = 0; s < 4; s++) {
                    for (int j = 0; j < 4; j++) {
                        uint16_t v;
                        memcpy(&v, rec + (s / 2) * 1024 + L * 16 + ((s % 2) * 4 + j) * 2, 2);
                        int q = (int)((word >> (8 * s + 2 * j)) & 3u);
                        if (j % 2 == 1) {
                            int q_prev = (int)((word >> (8 * s + 2 * (j - 1))) & 3u);
                            if (q_prev >= q)
                                return -1;
                        }
                        size_t row = (size_t)rb * 16 + (size_t)(L % 16);
                        size_t col = (size_t)u * 128 + (size_t)(s * 32 + (L / 16) * 8 + (j / 2) * 4 + q);
                        A_out[row * (size_t)K + col] = v;
                    }
                }
            }
        }
    }
    return 0;
}
