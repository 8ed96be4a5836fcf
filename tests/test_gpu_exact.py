"""Every element of full-size products, bit for bit, on the value pattern of the reference's own
harness (kernel_benchmark/spmm_test_utils.h:111-141): every kept weight is exactly 1.0 and every
activation one of -5, -3, -1, 1, 3.

With such data every product and every partial sum is a small integer, exact in fp32 in any order
of summation, so the expected result has a closed form that numpy evaluates exactly:

    Split_K == 1:  C = fp16_rn(sum over all k)
    Split_K  > 1:  C = fp16_rn(sum over batches b of fp16_rn(sum over the k of batch b))

(a slab holds fp16 partial sums, csrc/SpMM_Kernel.cuh:731-734; the reduction adds them in fp32 and
rounds once, csrc/Reduction_Kernel.cuh:36-46; a sum of fp16 values below 2^24 is exact in fp32).
The batches are the oracle's (oracle_splitk_range; for the 2:4 kernel ceil(units / Split_K) units
of 128 columns).  A dropped or doubled tile, a wrong batch boundary, a lost slab or a row written
to the wrong place changes some element by at least 1 and fails the comparison; tolerances play
no part.  The expected values come from numpy alone (float32 matrix products of integers).

Covered: the attention projections with every Split_K of the sweep in both operand layouts, the
feed-forward matrices at 70 / 80 / 90 % Bernoulli and Beta(2,8) row-skewed sparsity for 8 to 64
tokens, the OPT-66B and OPT-175B shapes of the reference's sweep (kernel_benchmark/benchmark.sh:13-14),
the entry point with the static workspace, and the 2:4 + residual calls.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

TOKENS = 64  # activations are drawn once for 64 tokens; a call with N tokens takes the first N


def _torch():
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch


def _dev(torch, a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        return torch.from_numpy(a.view(np.int16)).to("cuda:0").view(torch.float16)
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).to("cuda:0")
    return torch.from_numpy(a).to("cuda:0")


def _segment_sums(A, B, cuts):
    """out[s][n][m] = sum over columns cuts[s] <= k < cuts[s + 1] of A[m][k] * B[n][k], exact
    (integers far below 2^24 in float32).  A: M x K fp16 of zeros and ones, B: TOKENS x K fp16."""
    M, K = A.shape
    assert cuts[0] == 0 and cuts[-1] == K and list(cuts) == sorted(set(cuts))
    out = np.empty((len(cuts) - 1, TOKENS, M), dtype=np.float32)
    Bf = B.astype(np.float32)
    step = 2048
    buf = np.empty((step, K), dtype=np.float32)
    for r0 in range(0, M, step):
        r1 = min(M, r0 + step)
        np.copyto(buf[:r1 - r0], A[r0:r1])  # fp16 -> fp32 is exact
        for s in range(len(cuts) - 1):
            k0, k1 = cuts[s], cuts[s + 1]
            out[s, :, r0:r1] = Bf[:, k0:k1] @ buf[:r1 - r0, k0:k1].T
    return out


def _expected(seg, cuts, batches, N):
    """fp16 [N][M]: the closed form of the module docstring for batches = [(k0, k1), ...] (columns)."""
    at = {c: i for i, c in enumerate(cuts)}
    total = np.zeros((N, seg.shape[2]), dtype=np.float32)
    for k0, k1 in batches:
        part = seg[at[k0]:at[k1], :N].sum(axis=0, dtype=np.float32)
        if len(batches) > 1:  # a slab of partial sums is fp16
            part = part.astype(np.float16).astype(np.float32)
        total += part
    return total.astype(np.float16)


def _csl_batches(oracle, K, split_k):
    return [tuple(64 * kb for kb in oracle.splitk_range(K, split_k, b)) for b in range(split_k)]


def _unit_batches(K, split_k):
    units = K // 128
    per = -(-units // split_k)
    return [(128 * min(b * per, units), 128 * min((b + 1) * per, units)) for b in range(split_k)]


def _cuts(K, batch_lists):
    return sorted({0, K} | {c for batches in batch_lists for pair in batches for c in pair})


def _assert_identical(got, want, what):
    got = np.asarray(got)
    assert got.shape == want.shape, what
    g, w = got.astype(np.float32), want.astype(np.float32)
    assert np.isfinite(g).all(), f"{what}: non-finite output (unwritten or corrupt)"
    bad = g != w  # (+0 and -0 compare equal: an empty row may be either)
    if bad.any():
        n, m = np.argwhere(bad)[0]
        raise AssertionError(f"{what}: {int(bad.sum())} of {bad.size} elements differ, first at token {n} row {m}: "
                             f"got {g[n, m]}, want {w[n, m]}")


class _Weight:
    """One harness-pattern weight, encoded by the product and resident on the GPU, with the
    activations and everything the expected values need."""

    def __init__(self, spmm, torch, M, K, sparsity, skew, seed):
        self.M, self.K = M, K
        self.A = spmm.synth_harness_weights(M, K, sparsity, skew, seed=seed)
        self.B = spmm.synth_harness_activations(TOKENS, K, seed=seed + 1)
        self.items, self.offsets = spmm.InitSparseMatrixA_API(self.A)
        self.vectors = int(self.offsets[-1])
        self.d_items, self.d_offs = _dev(torch, self.items), _dev(torch, self.offsets)
        self.d_B = _dev(torch, self.B)  # [64][K]: the first N rows are a call's B[N][K]


def _run(spmm, torch, w, N, split_k, entry="column_major"):
    """C as fp16 [N][M] from the named entry point."""
    M, K = w.M, w.K
    stream = torch.cuda.current_stream()
    d_W = torch.full((max(split_k, 1), N, M), float("nan"), dtype=torch.float16, device="cuda:0")
    print(f"[gpu case] exact {entry} M={M} K={K} N={N} split_k={split_k}", flush=True)
    if entry == "row_major":
        d_Bt = w.d_B[:N].t().contiguous()
        d_Ct = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda:0")
        spmm.SpMM_SplitK_API_RowMajor(stream, None, w.d_items, w.d_offs, d_Bt, d_Ct, M, N, K, d_W, split_k)
        torch.cuda.synchronize()
        return d_Ct.t().contiguous().cpu().numpy()
    d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device="cuda:0")
    if entry == "static_workspace":
        spmm.SpMM_SplitK_API_StaticWorkspace(stream, None, w.d_items, w.d_offs, w.d_B[:N], d_C, M, N, K, split_k)
    else:
        spmm.SpMM_SplitK_API(stream, None, w.d_items, w.d_offs, w.d_B[:N], d_C, M, N, K, d_W, split_k)
    torch.cuda.synchronize()
    return d_C.cpu().numpy()


@pytest.mark.parametrize("M,K", [(21504, 7168), (7168, 7168)])
def test_exact_attention_projections_every_split_both_layouts(spmm, oracle, M, K):
    """OPT-30B QKV and output projection at 80 %: N in {8, 16, 32} x Split_K in {1, 2, 4, 7}, through
    the column-major and the row-major entry; the split calls also through the static workspace."""
    torch = _torch()
    w = _Weight(spmm, torch, M, K, 0.8, False, seed=M + K)
    splits = (1, 2, 4, 7)
    batches = {s: _csl_batches(oracle, K, s) for s in splits}
    cuts = _cuts(K, batches.values())
    seg = _segment_sums(w.A, w.B, cuts)
    for N in (8, 16, 32):
        for s in splits:
            want = _expected(seg, cuts, batches[s], N)
            for entry in ("column_major", "row_major") + (("static_workspace",) if N == 16 else ()):
                _assert_identical(_run(spmm, torch, w, N, s, entry), want, f"{entry} {M}x{K} N={N} Split_K={s}")


@pytest.mark.parametrize("skew", [False, True])
@pytest.mark.parametrize("sparsity", [0.7, 0.8, 0.9])
@pytest.mark.parametrize("M,K", [(28672, 7168), (7168, 28672)])
def test_exact_feed_forward_sparsity_and_skew(spmm, oracle, M, K, sparsity, skew):
    """OPT-30B FFN1 and FFN2 at 70 / 80 / 90 % sparsity, Bernoulli and Beta(2,8) row-skewed, N in
    {8, 16, 32, 64} with the planner's Split_K; the row-major entry at 16 and 64 tokens."""
    torch = _torch()
    w = _Weight(spmm, torch, M, K, sparsity, skew, seed=M // 64 + K + int(sparsity * 100) + skew)
    if skew:  # the skew is real: rows differ several times in what they hold, and tile rows (128 of them each) still visibly
        per_row = np.count_nonzero(w.A.view(np.uint16), axis=1)
        assert per_row.max() > 4 * max(int(per_row.min()), 1)
        per_tile_row = np.diff(w.offsets[:-1].astype(np.int64)[::K // 64])
        assert per_tile_row.max() > 1.2 * per_tile_row.min()
    split = {N: spmm.SpMM_SuggestSplitK_Bytes(M, N, K, w.vectors) for N in (8, 16, 32, 64)}
    batches = {s: _csl_batches(oracle, K, s) for s in set(split.values())}
    cuts = _cuts(K, batches.values())
    seg = _segment_sums(w.A, w.B, cuts)
    for N in (8, 16, 32, 64):
        want = _expected(seg, cuts, batches[split[N]], N)
        what = f"{M}x{K} {sparsity:.0%}{' skewed' if skew else ''} N={N} Split_K={split[N]}"
        _assert_identical(_run(spmm, torch, w, N, split[N]), want, "column_major " + what)
        if N in (16, 64):
            _assert_identical(_run(spmm, torch, w, N, split[N], "row_major"), want, "row_major " + what)


@pytest.mark.parametrize("M,K", [(27648, 9216), (9216, 9216), (36864, 9216), (9216, 36864)])
def test_exact_opt66b_shapes(spmm, oracle, M, K):
    """The four OPT-66B products at 80 %, N in {8, 16, 32}, the planner's Split_K and Split_K = 1."""
    torch = _torch()
    w = _Weight(spmm, torch, M, K, 0.8, False, seed=M // 128 + K)
    split = {N: spmm.SpMM_SuggestSplitK_Bytes(M, N, K, w.vectors) for N in (8, 16, 32)}
    batches = {s: _csl_batches(oracle, K, s) for s in set(split.values()) | {1}}
    cuts = _cuts(K, batches.values())
    seg = _segment_sums(w.A, w.B, cuts)
    for N in (8, 16, 32):
        for s in sorted({split[N], 1}):
            want = _expected(seg, cuts, batches[s], N)
            _assert_identical(_run(spmm, torch, w, N, s), want, f"column_major {M}x{K} N={N} Split_K={s}")
        _assert_identical(_run(spmm, torch, w, N, split[N], "row_major"), _expected(seg, cuts, batches[split[N]], N),
                          f"row_major {M}x{K} N={N} Split_K={split[N]}")


@pytest.mark.parametrize("M,K", [(36864, 12288), (12288, 12288), (49152, 12288), (12288, 49152)])
def test_exact_opt175b_shapes(spmm, oracle, M, K):
    """The four OPT-175B products of the reference's sweep (kernel_benchmark/benchmark.sh:13-14) at
    80 %, N in {8, 16, 32, 64}, the planner's Split_K."""
    torch = _torch()
    w = _Weight(spmm, torch, M, K, 0.8, False, seed=M // 128 + K + 1)
    split = {N: spmm.SpMM_SuggestSplitK_Bytes(M, N, K, w.vectors) for N in (8, 16, 32, 64)}
    batches = {s: _csl_batches(oracle, K, s) for s in set(split.values())}
    cuts = _cuts(K, batches.values())
    seg = _segment_sums(w.A, w.B, cuts)
    for N in (8, 16, 32, 64):
        want = _expected(seg, cuts, batches[split[N]], N)
        _assert_identical(_run(spmm, torch, w, N, split[N]), want, f"column_major {M}x{K} N={N} Split_K={split[N]}")
    _assert_identical(_run(spmm, torch, w, 16, split[16], "row_major"), _expected(seg, cuts, batches[split[16]], 16),
                      f"row_major {M}x{K} N=16 Split_K={split[16]}")


@pytest.mark.parametrize("M,K,sparsity", [(28672, 7168, 0.6), (7168, 28672, 0.7), (9216, 9216, 0.5)])
def test_exact_two_to_four_part_and_residual(spmm, oracle, M, K, sparsity):
    """The fork's split of a weight (kernel_benchmark/spmm_decompose.h:12-51) through both hybrid
    calls, N = 16 and 64: the two-kernel call sums the residual's Tiled-CSL slabs and the 2:4
    part's slabs (each batch rounded to fp16 by itself), the one-launch call one slab per batch of
    128-column units that holds both parts' sum."""
    torch = _torch()
    A = spmm.synth_harness_weights(M, K, sparsity, False, seed=M + K + 7)
    B = spmm.synth_harness_activations(TOKENS, K, seed=M + K + 8)
    A1, A2 = oracle.decompose(A)              # the checker's split, for the expected values
    p1, p2 = spmm.HeteroSparse_Decompose(A)   # the product's, for what the GPU is given
    assert np.array_equal(A1.view(np.uint16), p1.view(np.uint16)) and np.array_equal(A2.view(np.uint16), p2.view(np.uint16))
    del p1, p2
    d_packed = _dev(torch, spmm.HeteroSparse_PackA1(A1))
    items2, offsets2 = spmm.InitSparseMatrixA_API(A2)
    words, list_offsets, longest = spmm.HeteroSparse_PackA2(A2)
    d_items2, d_offs2, d_words, d_lists = (_dev(torch, x) for x in (items2, offsets2, words, list_offsets))
    d_B = _dev(torch, B)
    stream = torch.cuda.current_stream()
    s1 = {N: spmm.HeteroSparse_SuggestSplitK(M, N, K) for N in (16, 64)}
    s2 = {N: spmm.SpMM_SuggestSplitK(M, N, K) for N in (16, 64)}
    unit_batches = {s: _unit_batches(K, s) for s in set(s1.values())}
    csl_batches = {s: _csl_batches(oracle, K, s) for s in set(s2.values())}
    cuts = _cuts(K, list(unit_batches.values()) + list(csl_batches.values()))
    seg1 = _segment_sums(A1, B, cuts)
    seg2 = _segment_sums(A2, B, cuts)
    at = {c: i for i, c in enumerate(cuts)}
    for N in (16, 64):
        ub, cb = unit_batches[s1[N]], csl_batches[s2[N]]
        # two kernels: Split_K_A2 slabs of the residual, then Split_K_A1 slabs of the 2:4 part
        total = np.zeros((N, M), dtype=np.float32)
        for seg, batches in ((seg2, cb), (seg1, ub)):
            for k0, k1 in batches:
                total += seg[at[k0]:at[k1], :N].sum(axis=0, dtype=np.float32).astype(np.float16).astype(np.float32)
        d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device="cuda:0")
        d_W = torch.full((s1[N] + s2[N], N, M), float("nan"), dtype=torch.float16, device="cuda:0")
        print(f"[gpu case] exact hybrid M={M} K={K} N={N} split_k={s1[N]}/{s2[N]} sparsity={sparsity}", flush=True)
        spmm.HeteroSparse_SpMM_API(stream, d_packed, d_items2, d_offs2, d_B[:N], d_C, M, N, K, d_W, s1[N], s2[N])
        torch.cuda.synchronize()
        _assert_identical(d_C.cpu().numpy(), total.astype(np.float16), f"two kernels {M}x{K} N={N}")
        d_Bt = d_B[:N].t().contiguous()   # the same call on row-major operands: B[K][N], C[M][N], M x N slabs
        d_Ct = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda:0")
        d_W.fill_(float("nan"))
        spmm.HeteroSparse_SpMM_API_RowMajor(stream, d_packed, d_items2, d_offs2, d_Bt, d_Ct, M, N, K, d_W, s1[N], s2[N])
        torch.cuda.synchronize()
        _assert_identical(d_Ct.t().contiguous().cpu().numpy(), total.astype(np.float16), f"two kernels, row-major {M}x{K} N={N}")
        if longest > spmm.HETERO_FUSED_MAX_LIST:
            continue
        # one launch: per batch of units one fp16 slab of both parts' sum (no rounding with one batch)
        total = np.zeros((N, M), dtype=np.float32)
        for k0, k1 in ub:
            part = (seg1[at[k0]:at[k1], :N].sum(axis=0, dtype=np.float32) + seg2[at[k0]:at[k1], :N].sum(axis=0, dtype=np.float32))
            total += part.astype(np.float16).astype(np.float32) if len(ub) > 1 else part
        d_C.fill_(float("nan"))
        print(f"[gpu case] exact one launch M={M} K={K} N={N} split_k={s1[N]} longest={longest}", flush=True)
        spmm.HeteroSparse_Fused_SpMM_API(stream, d_packed, d_words, d_lists, longest, d_B[:N], d_C, M, N, K, d_W, s1[N])
        torch.cuda.synchronize()
        _assert_identical(d_C.cpu().numpy(), total.astype(np.float16), f"one launch {M}x{K} N={N}")
        d_Ct.fill_(float("nan"))
        spmm.HeteroSparse_Fused_SpMM_API_RowMajor(stream, d_packed, d_words, d_lists, longest, d_Bt, d_Ct, M, N, K, d_W, s1[N])
        torch.cuda.synchronize()
        _assert_identical(d_Ct.t().contiguous().cpu().numpy(), total.astype(np.float16), f"one launch, row-major {M}x{K} N={N}")
