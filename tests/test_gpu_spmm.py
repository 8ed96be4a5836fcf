"""GPU parity: SpMM_SplitK_API through the C ABI against the CPU oracle.

Tolerance (stated by the task for this fp16 path): |gpu - ref| <= 1e-2 + 1e-2 * |ref|
per element, ref = fp32-accumulate dense product on the decoded matrix.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ATOL, RTOL = 1e-2, 1e-2


def _torch():
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch


def run_gpu(spmm, items, offsets, B, M, N, K, split_k, poison=True):
    """One call through the C ABI; returns (C fp16 N x M, workspace fp16 or None)."""
    torch = _torch()
    dev = torch.device("cuda:0")
    d_items = torch.from_numpy(items.view(np.int32).copy()).to(dev) if len(items) else torch.zeros(4, dtype=torch.int32, device=dev)
    d_offs = torch.from_numpy(offsets.copy()).to(dev)
    d_B = torch.from_numpy(np.ascontiguousarray(B).view(np.int16).copy()).to(dev)
    d_C = torch.full((N, M), float("nan") if poison else 0.0, dtype=torch.float16, device=dev)
    d_W = torch.full((split_k, N, M), float("nan"), dtype=torch.float16, device=dev) if split_k > 1 else None
    print(f"[gpu case] M={M} N={N} K={K} split_k={split_k} words={len(items)}", flush=True)
    spmm.SpMM_SplitK_API(torch.cuda.current_stream(), None, d_items, d_offs, d_B, d_C, M, N, K, d_W, split_k)
    torch.cuda.synchronize()
    C = d_C.cpu().numpy()
    W = d_W.cpu().numpy() if d_W is not None else None
    return C, W


def assert_close(C, ref):
    C = C.astype(np.float32)
    ref = ref.astype(np.float32)
    assert np.isfinite(C).all(), "non-finite output (unwritten or corrupt)"
    err = np.abs(C - ref)
    bound = ATOL + RTOL * np.abs(ref)
    bad = err > bound
    assert not bad.any(), f"{bad.sum()} elements out of tolerance, max err {err.max()} at {np.unravel_index(err.argmax(), err.shape)}"


def make_case(spmm, M, K, N, sparsity, skew=False, seed=0):
    A = spmm.synth_weights(M, K, sparsity, skew, seed=seed)
    B = spmm.synth_activations(N, K, seed=seed + 1000)
    items, offsets = spmm.InitSparseMatrixA_API(A)
    return A, B, items, offsets


def test_layout_probe_one_hot(spmm, oracle):
    """Pins rows/columns/tokens: A holds distinct exactly-representable integers
    on a sparse pattern, B is one-hot per token, so C[n, m] must equal A[m, k_n] exactly."""
    M, K, N = 256, 128, 16
    rng = np.random.default_rng(5)
    A = np.zeros((M, K), dtype=np.float16)
    mask = rng.random((M, K)) < 0.3
    vals = (np.arange(M * K).reshape(M, K) % 1999 + 1).astype(np.float16)
    A[mask] = vals[mask]
    ks = rng.permutation(K)[:N]
    B = np.zeros((N, K), dtype=np.float16)
    B[np.arange(N), ks] = 1.0
    items, offsets = spmm.InitSparseMatrixA_API(A)
    C, _ = run_gpu(spmm, items, offsets, B, M, N, K, 1)
    expect = A[:, ks].T
    assert np.array_equal(C.view(np.uint16), expect.view(np.uint16))


@pytest.mark.parametrize("N", [8, 16, 32, 64])
@pytest.mark.parametrize("split_k", [1, 2, 3])
def test_small_vs_oracle(spmm, oracle, N, split_k):
    M, K = 256, 512
    A, B, items, offsets = make_case(spmm, M, K, N, 0.8, seed=N * 10 + split_k)
    C, W = run_gpu(spmm, items, offsets, B, M, N, K, split_k)
    ref = oracle.gemm_f32(oracle.decode(items, offsets, M, K), B)
    assert_close(C, ref)
    # the CPU restatement of the whole call (fp16 slabs, fp32 reduction) agrees as well
    C_or, W_or = oracle.spmm_splitk(items, offsets, B, M, N, K, split_k)
    assert_close(C, C_or)
    if split_k > 1:
        assert_close(W, W_or)


def test_config1_cpu_reference_case(spmm, oracle):
    """The CPU-runnable reference case: M=K=1024, N=8, 80 % Bernoulli, Split_K=1, seed 0."""
    M = K = 1024
    A, B, items, offsets = make_case(spmm, M, K, 8, 0.8, seed=0)
    C, _ = run_gpu(spmm, items, offsets, B, M, 8, K, 1)
    assert_close(C, oracle.gemm_f32(A, B))


@pytest.mark.parametrize("sparsity,skew", [(0.0, False), (0.3, False), (0.5, True), (0.7, True), (0.9, False), (0.999, False), (1.0, False)])
def test_density_sweep(spmm, oracle, sparsity, skew):
    """Dense tiles (several register windows per tile), nearly empty and empty tiles."""
    M, K, N = 256, 256, 16
    A, B, items, offsets = make_case(spmm, M, K, N, sparsity, skew, seed=int(sparsity * 1000))
    C, _ = run_gpu(spmm, items, offsets, B, M, N, K, 2)
    assert_close(C, oracle.gemm_f32(A, B))


def test_uneven_and_oversized_split(spmm, oracle):
    """K/64 = 9 tiles split 4 ways (3,3,3,0) and 7 ways; empty batches must write zeros."""
    M, K, N = 128, 576, 16
    A, B, items, offsets = make_case(spmm, M, K, N, 0.8, seed=77)
    ref = oracle.gemm_f32(A, B)
    for split_k in (4, 7, 9, 12):
        C, W = run_gpu(spmm, items, offsets, B, M, N, K, split_k)
        assert_close(C, ref)
        C_or, W_or = oracle.spmm_splitk(items, offsets, B, M, N, K, split_k)
        assert_close(W, W_or)


@pytest.mark.parametrize("M,K,N,split_k,sparsity", [
    (640, 1024, 16, 2, 0.8),     # 5 tile rows: workgroups of several waves, the last one with idle waves
    (896, 1792, 8, 4, 0.8),      # N = 8 with the activation slice staged in LDS
    (128, 8192, 16, 1, 0.8),     # one unit of 128 tiles: the offsets window slides; slice too large to stage
    (128, 12288, 8, 2, 0.9),     # 96-tile units with N = 8
    (1152, 512, 16, 8, 0.75),    # one tile per unit
    (384, 2048, 32, 3, 0.8),     # two column blocks, uneven batches (32 tiles over 3)
    (256, 2048, 64, 2, 0.6),     # four column blocks, tiles longer than one register window
    (2048, 256, 16, 2, 0.95),    # many tile rows, short K
])
def test_launch_shapes(spmm, oracle, M, K, N, split_k, sparsity):
    """Shapes chosen to reach every launch plan of the main kernel: several waves per
    workgroup with and without idle waves, staged and unstaged activations, long units."""
    A, B, items, offsets = make_case(spmm, M, K, N, sparsity, seed=M + K + N)
    C, W = run_gpu(spmm, items, offsets, B, M, N, K, split_k)
    assert_close(C, oracle.gemm_f32(A, B))
    C_or, W_or = oracle.spmm_splitk(items, offsets, B, M, N, K, split_k)
    assert_close(C, C_or)
    if split_k > 1:
        assert_close(W, W_or)


def test_partials_entry_point(spmm, oracle):
    """SpMM_SplitK_Partials writes the same slabs SpMM_SplitK_API leaves in the workspace."""
    import ctypes

    torch = _torch()
    M, K, N, split_k = 512, 1024, 16, 4
    A, B, items, offsets = make_case(spmm, M, K, N, 0.8, seed=99)
    dev = torch.device("cuda:0")
    d_items = torch.from_numpy(items.view(np.int32).copy()).to(dev)
    d_offs = torch.from_numpy(offsets.copy()).to(dev)
    d_B = torch.from_numpy(B.view(np.int16).copy()).to(dev)
    d_P = torch.full((split_k, N, M), float("nan"), dtype=torch.float16, device=dev)
    lib = spmm.load_library()
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    rc = lib.SpMM_SplitK_Partials(None, p(d_items), p(d_offs), p(d_B), p(d_P), M, N, K, split_k)
    assert rc == 0
    torch.cuda.synchronize()
    _, W_or = oracle.spmm_splitk(items, offsets, B, M, N, K, split_k)
    assert_close(d_P.cpu().numpy(), W_or)
    assert lib.SpMM_SplitK_Partials(None, p(d_items), p(d_offs), p(d_B), p(d_P), M, 24, K, split_k) != 0
    assert lib.SpMM_SplitK_Partials(None, p(d_items), p(d_offs), p(d_B), None, M, N, K, split_k) != 0


def test_repeated_calls_share_workspace(spmm, oracle):
    """Back-to-back calls on one stream with one workspace (the caller contract) and different weights."""
    torch = _torch()
    dev = torch.device("cuda:0")
    M, K, N, split_k = 384, 768, 16, 3
    cases = [make_case(spmm, M, K, N, 0.8, seed=500 + i) for i in range(3)]
    d_W = torch.empty((split_k, N, M), dtype=torch.float16, device=dev)
    outs = []
    keep = []
    for A, B, items, offsets in cases:
        d_items = torch.from_numpy(items.view(np.int32).copy()).to(dev)
        d_offs = torch.from_numpy(offsets.copy()).to(dev)
        d_B = torch.from_numpy(B.view(np.int16).copy()).to(dev)
        d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device=dev)
        keep.append((d_items, d_offs, d_B))
        spmm.SpMM_SplitK_API(torch.cuda.current_stream(), None, d_items, d_offs, d_B, d_C, M, N, K, d_W, split_k)
        outs.append(d_C)
    torch.cuda.synchronize()
    for (A, B, items, offsets), d_C in zip(cases, outs):
        assert_close(d_C.cpu().numpy(), oracle.gemm_f32(A, B))


def test_full_size_properties(spmm, oracle):
    """Headline shape (OPT-30B FFN1, 28672 x 7168, N=16, 80 %): checks that do not need the
    full CPU product: linearity in the activations, a one-hot activation reproducing a
    column of A exactly, and a row sample against the oracle."""
    torch = _torch()
    dev = torch.device("cuda:0")
    M, K, N = 28672, 7168, 16
    split_k = spmm.SpMM_SuggestSplitK(M, N, K)
    A = spmm.synth_weights(M, K, 0.8, False, seed=1234)
    items, offsets = spmm.InitSparseMatrixA_API(A)
    B1 = spmm.synth_activations(N, K, seed=1)
    B2 = spmm.synth_activations(N, K, seed=2)
    E = np.zeros((N, K), dtype=np.float16)
    ks = np.random.default_rng(3).integers(0, K, N)
    E[np.arange(N), ks] = 1.0
    d_items = torch.from_numpy(items.view(np.int32)).to(dev)
    d_offs = torch.from_numpy(offsets).to(dev)
    d_W = torch.empty((split_k, N, M), dtype=torch.float16, device=dev)

    def run(Bh):
        d_B = torch.from_numpy(np.ascontiguousarray(Bh).view(np.int16)).to(dev)
        d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device=dev)
        spmm.SpMM_SplitK_API(None, None, d_items, d_offs, d_B, d_C, M, N, K, d_W, split_k)
        torch.cuda.synchronize()
        return d_C.cpu().numpy()

    print(f"[gpu case] full size M={M} K={K} N={N} split_k={split_k}", flush=True)
    C1, C2 = run(B1), run(B2)
    # exact: one-hot activations pick columns of A (a single non-zero product per output)
    CE = run(E)
    assert np.array_equal(CE.view(np.uint16), (A[:, ks].T + np.float16(0)).view(np.uint16))
    # linearity within rounding: A*(B1 + B2) = A*B1 + A*B2
    Bs = (B1.astype(np.float32) + B2.astype(np.float32)).astype(np.float16)
    Cs = run(Bs)
    exact_sum = (Bs.astype(np.float32) == B1.astype(np.float32) + B2.astype(np.float32))
    cols = np.flatnonzero(exact_sum.all(axis=1))  # tokens whose fp16 sum is exact
    lin = C1.astype(np.float32) + C2.astype(np.float32)
    if len(cols):
        assert_close(Cs[cols], lin[cols])
    # row sample against the oracle
    rows = np.unique(np.concatenate([np.arange(128), np.arange(M - 128, M), np.random.default_rng(4).integers(0, M, 512)]))
    assert_close(C1[:, rows], oracle.gemm_f32(np.ascontiguousarray(A[rows]), B1))


def test_split1_leaves_workspace_alone(spmm):
    torch = _torch()
    M, K, N = 128, 128, 16
    A, B, items, offsets = make_case(spmm, M, K, N, 0.8, seed=3)
    dev = torch.device("cuda:0")
    d_items = torch.from_numpy(items.view(np.int32).copy()).to(dev)
    d_offs = torch.from_numpy(offsets.copy()).to(dev)
    d_B = torch.from_numpy(B.view(np.int16).copy()).to(dev)
    d_C = torch.zeros((N, M), dtype=torch.float16, device=dev)
    d_W = torch.full((N, M), 7.0, dtype=torch.float16, device=dev)
    spmm.SpMM_SplitK_API(None, None, d_items, d_offs, d_B, d_C, M, N, K, d_W, 1)
    torch.cuda.synchronize()
    assert (d_W == 7.0).all()


def test_errors_launch_nothing(spmm):
    torch = _torch()
    dev = torch.device("cuda:0")
    t = torch.zeros(1024, dtype=torch.int32, device=dev)
    C = torch.full((64, 128), 5.0, dtype=torch.float16, device=dev)
    with pytest.raises(spmm.SpMMError):
        spmm.SpMM_SplitK_API(None, None, t, t, t, C, 128, 24, 64, t, 1)   # unsupported N
    with pytest.raises(spmm.SpMMError):
        spmm.SpMM_SplitK_API(None, None, t, t, t, C, 100, 16, 64, t, 1)   # M % 128
    with pytest.raises(spmm.SpMMError):
        spmm.SpMM_SplitK_API(None, None, t, t, t, C, 128, 16, 96, t, 1)   # K % 64
    with pytest.raises(spmm.SpMMError):
        spmm.SpMM_SplitK_API(None, None, t, t, t, C, 128, 16, 64, t, 0)   # Split_K
    with pytest.raises(spmm.SpMMError):
        spmm.SpMM_SplitK_API(None, None, t, t, t, C, 128, 16, 64, None, 2)  # no workspace
    with pytest.raises(spmm.SpMMError):
        spmm.SpMM_SplitK_API(None, None, t, t, t, C, 128, 16, 64, t, 65536)  # beyond the launch grid
    torch.cuda.synchronize()
    assert (C == 5.0).all()


def test_midsize_rows_sampled(spmm, oracle):
    """7168 x 7168 (OPT-30B out-proj), N=16, Split_K=7: full output against the oracle GEMM."""
    M = K = 7168
    N = 16
    A, B, items, offsets = make_case(spmm, M, K, N, 0.8, seed=30)
    C, _ = run_gpu(spmm, items, offsets, B, M, N, K, 7)
    ref = oracle.gemm_f32(A, B)
    assert_close(C, ref)


PLANS = [
    # (M, K, N, split_k, mode, waves, stage_b)
    (1024, 1024, 16, 4, 0, 7, 1),    # shared slice, partial last workgroup (8 tile rows over 7 waves)
    (1024, 1024, 16, 4, 0, 8, 1),
    (1024, 1024, 8, 2, 0, 5, 1),
    (1024, 1024, 16, 3, 0, 3, 0),    # fragments from global memory
    (1024, 1024, 32, 4, 0, 4, 0),
    (1024, 1024, 64, 2, 0, 2, 0),
    (1024, 1024, 16, 1, 1, 8, 0),    # K split inside the workgroup, direct write of C
    (1024, 1024, 8, 1, 1, 7, 0),     # 16 tiles over 7 waves: runs of 3, last wave gets 1... and one gets none
    (1024, 1024, 16, 2, 1, 6, 0),
    (1024, 1024, 32, 1, 1, 8, 0),
    (1024, 1024, 32, 3, 1, 3, 0),
    (1024, 1024, 64, 1, 1, 4, 0),
    (1024, 1024, 64, 2, 1, 3, 0),
    (256, 64 * 3, 16, 1, 1, 8, 0),   # fewer tiles than waves: five waves have nothing to do
    (256, 64 * 70, 16, 1, 1, 1, 0),  # one wave, more than 63 tiles: the offsets window slides
    (384, 64 * 130, 8, 1, 1, 2, 0),
]


@pytest.mark.parametrize("M,K,N,split_k,mode,waves,stage_b", PLANS)
def test_explicit_launch_plans(spmm, oracle, M, K, N, split_k, mode, waves, stage_b):
    torch = _torch()
    dev = torch.device("cuda:0")
    A, B, items, offsets = make_case(spmm, M, K, N, 0.8, seed=M + K + N + 7 * mode + waves)
    ref = oracle.gemm_f32(A, B)
    d_items = torch.from_numpy(items.view(np.int32).copy()).to(dev)
    d_offs = torch.from_numpy(offsets.copy()).to(dev)
    d_B = torch.from_numpy(np.ascontiguousarray(B).view(np.int16).copy()).to(dev)
    d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device=dev)
    d_W = torch.full((split_k, N, M), float("nan"), dtype=torch.float16, device=dev) if split_k > 1 else None
    print(f"[gpu case] planned M={M} N={N} K={K} split_k={split_k} mode={mode} waves={waves} stage={stage_b}", flush=True)
    spmm.SpMM_SplitK_API_Planned(torch.cuda.current_stream(), d_items, d_offs, d_B, d_C, M, N, K, d_W, split_k, mode,
                                 waves, stage_b)
    torch.cuda.synchronize()
    assert_close(d_C.cpu().numpy(), ref)


def test_explicit_plan_rejects_what_does_not_fit(spmm):
    torch = _torch()
    dev = torch.device("cuda:0")
    z = torch.zeros(1024, dtype=torch.int32, device=dev)
    for (N, mode, waves, stage) in [(16, 0, 9, 0), (64, 1, 5, 0), (32, 0, 2, 1), (16, 1, 4, 1), (16, 2, 4, 0), (16, 0, 0, 0)]:
        with pytest.raises(spmm.SpMMError):
            spmm.SpMM_SplitK_API_Planned(None, z, z, z, z, 1024, N, 1024, z, 1, mode, waves, stage)
    with pytest.raises(spmm.SpMMError):  # row-major operands cannot use the staged slice
        spmm.SpMM_SplitK_API_Planned(None, z, z, z, z, 1024, 16, 1024, z, 1, 0, 4, 1, 1)
    # a staged slice that does not fit in LDS: 448 tiles x 16 tokens x 128 B
    with pytest.raises(spmm.SpMMError):
        spmm.SpMM_SplitK_API_Planned(None, z, z, z, z, 1024, 16, 28672, z, 1, 0, 4, 1)


def _row_major_case(spmm, oracle, M, K, N, split_k, plan=None, sparsity=0.8):
    torch = _torch()
    dev = torch.device("cuda:0")
    A, B, items, offsets = make_case(spmm, M, K, N, sparsity, seed=3 * M + K + N + split_k)
    ref = oracle.gemm_f32(A, B)  # N x M
    d_items = torch.from_numpy(items.view(np.int32).copy()).to(dev)
    d_offs = torch.from_numpy(offsets.copy()).to(dev)
    Bt = np.ascontiguousarray(B.T)  # K x N
    d_B = torch.from_numpy(Bt.view(np.int16).copy()).to(dev)
    d_C = torch.full((M, N), float("nan"), dtype=torch.float16, device=dev)
    d_W = torch.full((split_k, M, N), float("nan"), dtype=torch.float16, device=dev) if split_k > 1 else None
    print(f"[gpu case] row-major M={M} N={N} K={K} split_k={split_k} plan={plan}", flush=True)
    if plan is None:
        spmm.SpMM_SplitK_API_RowMajor(torch.cuda.current_stream(), None, d_items, d_offs, d_B, d_C, M, N, K, d_W, split_k)
    else:
        spmm.SpMM_SplitK_API_Planned(torch.cuda.current_stream(), d_items, d_offs, d_B, d_C, M, N, K, d_W, split_k,
                                     plan[0], plan[1], 0, 1)
    torch.cuda.synchronize()
    assert_close(d_C.cpu().numpy().T, ref)


@pytest.mark.parametrize("N", [8, 16, 32, 64])
@pytest.mark.parametrize("split_k", [1, 3])
def test_row_major_entry(spmm, oracle, N, split_k):
    _row_major_case(spmm, oracle, 512, 1024, N, split_k)


@pytest.mark.parametrize("M,K,N,split_k,mode,waves", [
    (1024, 1024, 16, 4, 0, 7), (1024, 1024, 8, 2, 0, 3), (1024, 1024, 32, 2, 0, 8), (1024, 1024, 64, 2, 0, 4),
    (1024, 1024, 16, 1, 1, 8), (1024, 1024, 8, 1, 1, 5), (1024, 1024, 32, 1, 1, 6), (1024, 1024, 64, 1, 1, 4),
    (256, 64 * 70, 16, 1, 0, 1), (128, 64, 16, 1, 1, 8),
])
def test_row_major_launch_shapes(spmm, oracle, M, K, N, split_k, mode, waves):
    _row_major_case(spmm, oracle, M, K, N, split_k, plan=(mode, waves))


def test_row_major_layout_probe(spmm, oracle):
    """One-hot activations: C[:, n] must be column k_n of A, exactly, in M x N order."""
    torch = _torch()
    dev = torch.device("cuda:0")
    M, K, N = 256, 256, 16
    A = spmm.synth_weights(M, K, 0.5, False, seed=77)
    items, offsets = spmm.InitSparseMatrixA_API(A)
    ks = [(17 * n + 3) % K for n in range(N)]
    Bt = np.zeros((K, N), dtype=np.float16)
    for n, k in enumerate(ks):
        Bt[k, n] = 1.0
    d_items = torch.from_numpy(items.view(np.int32).copy()).to(dev)
    d_offs = torch.from_numpy(offsets.copy()).to(dev)
    d_B = torch.from_numpy(Bt.view(np.int16).copy()).to(dev)
    d_C = torch.full((M, N), float("nan"), dtype=torch.float16, device=dev)
    spmm.SpMM_SplitK_API_RowMajor(None, None, d_items, d_offs, d_B, d_C, M, N, K, None, 1)
    torch.cuda.synchronize()
    C = d_C.cpu().numpy()
    for n, k in enumerate(ks):
        assert np.array_equal(C[:, n], A[:, k])


@pytest.mark.parametrize("N,split_k,relu", [(16, 1, 0), (16, 4, 1), (8, 1, 1), (32, 2, 0), (64, 1, 1), (16, 3, 0)])
def test_strided_operands_and_fused_relu(spmm, oracle, N, split_k, relu):
    """B and C live inside wider per-token buffers; everything outside C's window must stay untouched."""
    torch = _torch()
    dev = torch.device("cuda:0")
    M, K = 512, 1024
    ldb, ldc, boff, coff = 3 * K, M + 256, K, 128  # B = the middle third of a fused buffer
    A, B, items, offsets = make_case(spmm, M, K, N, 0.8, seed=11 * N + split_k)
    ref = oracle.gemm_f32(A, B)
    if relu:
        ref = np.maximum(ref, 0.0)
    wide_B = spmm.synth_activations(N, ldb, seed=5)  # junk around the real activations
    wide_B[:, boff:boff + K] = B
    d_items = torch.from_numpy(items.view(np.int32).copy()).to(dev)
    d_offs = torch.from_numpy(offsets.copy()).to(dev)
    d_B = torch.from_numpy(wide_B.view(np.int16).copy()).to(dev)
    d_C = torch.full((N, ldc), -7.0, dtype=torch.float16, device=dev)
    d_W = torch.full((split_k, N, M), float("nan"), dtype=torch.float16, device=dev) if split_k > 1 else None
    print(f"[gpu case] strided M={M} N={N} K={K} split_k={split_k} relu={relu}", flush=True)
    spmm.SpMM_SplitK_API_Strided(torch.cuda.current_stream(), d_items, d_offs, d_B.data_ptr() + 2 * boff, ldb,
                                 d_C.data_ptr() + 2 * coff, ldc, M, N, K, d_W, split_k,
                                 spmm.SPMM_FLAG_RELU if relu else 0)
    torch.cuda.synchronize()
    C = d_C.cpu().numpy()
    assert_close(C[:, coff:coff + M], ref)
    assert (C[:, :coff] == -7.0).all() and (C[:, coff + M:] == -7.0).all()
    if relu:
        assert (C[:, coff:coff + M] >= 0).all()


def test_strided_rejects_bad_strides(spmm):
    torch = _torch()
    z = torch.zeros(1024, dtype=torch.int32, device="cuda:0")
    for (ldb, ldc, flags) in [(1000, 1024, 0), (1024, 1000, 0), (1028, 1024, 0), (1024, 1028, 0), (1024, 1024, 4)]:
        with pytest.raises(spmm.SpMMError):
            spmm.SpMM_SplitK_API_Strided(None, z, z, z, ldb, z, ldc, 1024, 16, 1024, z, 1, flags)


def test_decoder_stack_matches_cpu_chain(spmm, oracle):
    """Three chained blocks (QKV -> out-proj on a slice -> FFN1+ReLU -> FFN2) against the same chain on the CPU."""
    torch = _torch()
    from graphneuralnetproj_amd import decoder_stack as DS

    dev = torch.device("cuda:0")
    h, N, nlayers = 512, 16, 3
    layers, dense = [], []
    for i in range(nlayers):
        L, d = DS.build_layer(spmm, torch, dev, h, N, 0.6, seed=40 + i, keep_dense=True, weight_scale=4.0)
        layers.append(L)
        dense.append(d)
    stack = DS.Stack(spmm, torch, layers, h, N)
    x0 = spmm.synth_activations(N, h, seed=99)
    stack.x[0].copy_(torch.from_numpy(x0.view(np.int16)).to(dev).view(torch.float16))
    print(f"[gpu case] decoder stack h={h} N={N} layers={nlayers}", flush=True)
    out = stack.step(torch.cuda.current_stream())
    torch.cuda.synchronize()
    got = out.cpu().numpy()

    x = x0
    f16 = lambda a: a.astype(np.float16)
    for d in dense:
        qkv = f16(oracle.gemm_f32(d["qkv"], x))
        o = f16(oracle.gemm_f32(d["out"], np.ascontiguousarray(qkv[:, :h])))
        f = f16(np.maximum(oracle.gemm_f32(d["ffn1"], o), 0.0))
        x = f16(oracle.gemm_f32(d["ffn2"], f))
    assert np.abs(x.astype(np.float32)).max() > 1e-3, "the reference chain must not have collapsed to zero"
    # Each product is within the per-call tolerance of its own inputs, but the inputs of later
    # products already differ by the earlier roundings (fp16 storage of every intermediate, and
    # split-K partial sums on the GPU only), and an output element near zero is a sum of large
    # terms that cancel: its error scales with the typical magnitude, not with its own.  So the
    # per-element tolerance is taken against max(|ref|, rms(ref)), times 3 for the twelve products.
    xr = x.astype(np.float32)
    err = np.abs(got.astype(np.float32) - xr)
    scale = np.maximum(np.abs(xr), np.sqrt(np.mean(xr * xr)))
    assert (err <= 3 * (ATOL + RTOL * scale)).all(), err.max()


def test_row_major_decoder_stack_matches_cpu_chain(spmm, oracle):
    """The same three blocks with every buffer as [features][tokens] (the fork's layout): the output
    projection reads the first h rows of the fused QKV result, the clamp rides on the row-major entry."""
    torch = _torch()
    from graphneuralnetproj_amd import decoder_stack as DS

    dev = torch.device("cuda:0")
    h, N, nlayers = 512, 16, 3
    layers, dense = [], []
    for i in range(nlayers):
        L, d = DS.build_layer(spmm, torch, dev, h, N, 0.6, seed=40 + i, keep_dense=True, weight_scale=4.0)
        layers.append(L)
        dense.append(d)
    stack = DS.Stack(spmm, torch, layers, h, N, row_major=True)
    x0 = spmm.synth_activations(N, h, seed=99)
    stack.x[0].copy_(torch.from_numpy(np.ascontiguousarray(x0.T).view(np.int16)).to(dev).view(torch.float16))
    print(f"[gpu case] row-major decoder stack h={h} N={N} layers={nlayers}", flush=True)
    out = stack.step(torch.cuda.current_stream())
    torch.cuda.synchronize()
    got = out.cpu().numpy().T
    x = x0
    f16 = lambda a: a.astype(np.float16)
    for d in dense:
        qkv = f16(oracle.gemm_f32(d["qkv"], x))
        o = f16(oracle.gemm_f32(d["out"], np.ascontiguousarray(qkv[:, :h])))
        f = f16(np.maximum(oracle.gemm_f32(d["ffn1"], o), 0.0))
        x = f16(oracle.gemm_f32(d["ffn2"], f))
    xr = x.astype(np.float32)
    assert np.abs(xr).max() > 1e-3
    err = np.abs(got.astype(np.float32) - xr)
    scale = np.maximum(np.abs(xr), np.sqrt(np.mean(xr * xr)))
    assert (err <= 3 * (ATOL + RTOL * scale)).all(), err.max()  # as for the column-major chain


@pytest.mark.parametrize("M,K,N,split_k", [
    (1024, 1024, 16, 4), (1024, 1024, 8, 2), (1024, 2048, 32, 8), (1024, 1024, 64, 3),
    (1152, 1024, 16, 5),      # nine tile rows: a partly filled workgroup in the row-sharing layout
    (7168, 7168, 16, 4),      # an OPT-30B attention projection, the planner's own choice of split
])
def test_fused_reduction_matches_separate_kernel_bit_for_bit(spmm, oracle, M, K, N, split_k):
    """Split_K > 1: the in-launch reduction and the second-kernel reduction sum the same slabs in the same order."""
    torch = _torch()
    dev = torch.device("cuda:0")
    A, B, items, offsets = make_case(spmm, M, K, N, 0.8, seed=M + 3 * K + N + split_k)
    d_items = torch.from_numpy(items.view(np.int32).copy()).to(dev)
    d_offs = torch.from_numpy(offsets.copy()).to(dev)
    d_B = torch.from_numpy(np.ascontiguousarray(B).view(np.int16).copy()).to(dev)
    outs = []
    for flags in (0, spmm.SPMM_FLAG_SEPARATE_REDUCTION, spmm.SPMM_FLAG_RELU,
                  spmm.SPMM_FLAG_RELU | spmm.SPMM_FLAG_SEPARATE_REDUCTION):
        d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device=dev)
        d_W = torch.full((split_k, N, M), float("nan"), dtype=torch.float16, device=dev)
        print(f"[gpu case] fused-vs-separate M={M} N={N} K={K} split_k={split_k} flags={flags}", flush=True)
        for _ in range(3):  # repeated calls: the arrival counters must come back to zero every time
            spmm.SpMM_SplitK_API_Strided(torch.cuda.current_stream(), d_items, d_offs, d_B, K, d_C, M, M, N, K, d_W,
                                         split_k, flags)
        torch.cuda.synchronize()
        outs.append(d_C.cpu().numpy())
    assert np.array_equal(outs[0].view(np.uint16), outs[1].view(np.uint16))
    assert np.array_equal(outs[2].view(np.uint16), outs[3].view(np.uint16))
    if M * K <= 4 * 1024 * 1024:
        ref = oracle.gemm_f32(A, B)
        assert_close(outs[0], ref)
        assert_close(outs[2], np.maximum(ref, 0.0))


@pytest.mark.parametrize("M,K,N,split_k,waves", [(1024, 1024, 16, 4, 4), (1024, 2048, 8, 3, 8), (1152, 1024, 32, 5, 5),
                                                 (1024, 1024, 64, 2, 4), (7168, 7168, 16, 4, 5)])
def test_row_major_fused_reduction_matches_separate_kernel_bit_for_bit(spmm, oracle, M, K, N, split_k, waves):
    """The fork's layout (B[K][N], C[M][N]) in the K-splitting layout: the reduction inside the launch
    and the second kernel give the same bits, with and without the clamp, on repeated calls."""
    torch = _torch()
    dev = torch.device("cuda:0")
    A, B, items, offsets = make_case(spmm, M, K, N, 0.8, seed=M + 5 * K + N + split_k)
    d_items = torch.from_numpy(items.view(np.int32).copy()).to(dev)
    d_offs = torch.from_numpy(offsets.copy()).to(dev)
    d_Bt = torch.from_numpy(np.ascontiguousarray(B.T).view(np.int16).copy()).to(dev)
    outs = []
    for flags in (0, spmm.SPMM_FLAG_SEPARATE_REDUCTION, spmm.SPMM_FLAG_RELU,
                  spmm.SPMM_FLAG_RELU | spmm.SPMM_FLAG_SEPARATE_REDUCTION):
        d_C = torch.full((M, N), float("nan"), dtype=torch.float16, device=dev)
        d_W = torch.full((split_k, M, N), float("nan"), dtype=torch.float16, device=dev)
        print(f"[gpu case] row-major fused-vs-separate M={M} N={N} K={K} split_k={split_k} waves={waves} flags={flags}", flush=True)
        for _ in range(3):  # repeated calls: the arrival counters must come back to zero every time
            spmm.SpMM_SplitK_API_Planned(torch.cuda.current_stream(), d_items, d_offs, d_Bt, d_C, M, N, K, d_W, split_k, 1, waves,
                                         0, 1, flags)
        torch.cuda.synchronize()
        outs.append(d_C.cpu().numpy())
    assert np.array_equal(outs[0].view(np.uint16), outs[1].view(np.uint16))
    assert np.array_equal(outs[2].view(np.uint16), outs[3].view(np.uint16))
    if M * K <= 4 * 1024 * 1024:
        ref = oracle.gemm_f32(A, B)
        assert_close(outs[0].T, ref)
        assert_close(outs[2].T, np.maximum(ref, 0.0))
    # the library's own entry (its own launch shape) agrees too
    d_C = torch.full((M, N), float("nan"), dtype=torch.float16, device=dev)
    d_W = torch.full((split_k, M, N), float("nan"), dtype=torch.float16, device=dev)
    spmm.SpMM_SplitK_API_RowMajor(torch.cuda.current_stream(), None, d_items, d_offs, d_Bt, d_C, M, N, K, d_W, split_k)
    torch.cuda.synchronize()
    got = d_C.cpu().numpy().astype(np.float32)
    want = outs[0].astype(np.float32)
    assert (np.abs(got - want) <= 2e-2 + 2e-2 * np.abs(want)).all()


@pytest.mark.parametrize("mode,waves,stage_b", [(0, 7, 1), (0, 3, 0), (1, 8, 0), (1, 5, 0)])
def test_fused_reduction_in_every_launch_shape(spmm, oracle, mode, waves, stage_b):
    torch = _torch()
    dev = torch.device("cuda:0")
    M, K, N, split_k = 1152, 1536, 16, 6
    A, B, items, offsets = make_case(spmm, M, K, N, 0.8, seed=5 + mode + waves)
    ref = oracle.gemm_f32(A, B)
    d_items = torch.from_numpy(items.view(np.int32).copy()).to(dev)
    d_offs = torch.from_numpy(offsets.copy()).to(dev)
    d_B = torch.from_numpy(np.ascontiguousarray(B).view(np.int16).copy()).to(dev)
    d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device=dev)
    d_W = torch.full((split_k, N, M), float("nan"), dtype=torch.float16, device=dev)
    print(f"[gpu case] fused planned mode={mode} waves={waves} stage={stage_b}", flush=True)
    for _ in range(2):
        spmm.SpMM_SplitK_API_Planned(torch.cuda.current_stream(), d_items, d_offs, d_B, d_C, M, N, K, d_W, split_k,
                                     mode, waves, stage_b, 0)
    torch.cuda.synchronize()
    assert_close(d_C.cpu().numpy(), ref)


def test_fused_reduction_on_two_streams(spmm, oracle):
    """Calls that overlap on different streams count their arrivals on different pages."""
    torch = _torch()
    dev = torch.device("cuda:0")
    M, K, N, split_k = 2048, 2048, 16, 4
    cases = []
    for i in range(2):
        A, B, items, offsets = make_case(spmm, M, K, N, 0.8, seed=900 + i)
        cases.append((oracle.gemm_f32(A, B),
                      torch.from_numpy(items.view(np.int32).copy()).to(dev), torch.from_numpy(offsets.copy()).to(dev),
                      torch.from_numpy(np.ascontiguousarray(B).view(np.int16).copy()).to(dev),
                      torch.full((N, M), float("nan"), dtype=torch.float16, device=dev),
                      torch.full((split_k, N, M), float("nan"), dtype=torch.float16, device=dev),
                      torch.cuda.Stream()))
    torch.cuda.synchronize()
    print("[gpu case] fused reduction on two streams", flush=True)
    for _ in range(20):
        for (_, it, of, b, c, w, st) in cases:
            spmm.SpMM_SplitK_API(st, None, it, of, b, c, M, N, K, w, split_k)
    torch.cuda.synchronize()
    for (ref, _, _, _, c, _, _) in cases:
        assert_close(c.cpu().numpy(), ref)


@pytest.mark.parametrize("N,split_k,mode,waves,stage_b", [
    (32, 8, 0, 1, 0),   # one-wave workgroups, eight resident per compute unit: hundreds finish together
    (16, 8, 0, 7, 1), (16, 4, 1, 6, 0), (64, 4, 0, 4, 0), (8, 6, 1, 8, 0),
])
def test_fused_reduction_under_load_bit_for_bit(spmm, N, split_k, mode, waves, stage_b):
    """Full-size weight: every compute unit busy and many workgroups arriving at once."""
    torch = _torch()
    dev = torch.device("cuda:0")
    M, K = 28672, 7168
    A, B, items, offsets = make_case(spmm, M, K, N, 0.8, seed=4242)
    d_items = torch.from_numpy(items.view(np.int32).copy()).to(dev)
    d_offs = torch.from_numpy(offsets.copy()).to(dev)
    d_B = torch.from_numpy(np.ascontiguousarray(B).view(np.int16).copy()).to(dev)
    outs = []
    for flags in (spmm.SPMM_FLAG_SEPARATE_REDUCTION, 0, 0, 0):
        d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device=dev)
        d_W = torch.full((split_k, N, M), float("nan"), dtype=torch.float16, device=dev)
        print(f"[gpu case] fused under load N={N} split_k={split_k} plan=({mode},{waves},{stage_b}) flags={flags}", flush=True)
        spmm.SpMM_SplitK_API_Planned(torch.cuda.current_stream(), d_items, d_offs, d_B, d_C, M, N, K, d_W, split_k,
                                     mode, waves, stage_b, 0, flags)
        torch.cuda.synchronize()
        outs.append(d_C.cpu().numpy().view(np.uint16))
    for o in outs[1:]:
        assert np.array_equal(outs[0], o)


@pytest.mark.parametrize("N,split_k", [(16, 1), (8, 3), (64, 2)])
def test_product_on_unreordered_encoding(spmm, oracle, N, split_k):
    """The kernels take a tile's words in any order: the reference's no-reorder encoding works unchanged."""
    M, K = 512, 1024
    A = spmm.synth_weights(M, K, 0.8, False, seed=31 + N)
    B = spmm.synth_activations(N, K, seed=32)
    items, offsets = spmm.InitSparseMatrixA_API_NoReorder(A)
    C, _ = run_gpu(spmm, items, offsets, B, M, N, K, split_k)
    assert_close(C, oracle.gemm_f32(A, B))


def test_hip_graph_replays_match_eager(spmm, oracle):
    """A captured chain (one product with the fused reduction, one without a split, one with the
    second-kernel reduction) replayed several times, with eager work in between, gives the eager bits."""
    torch = _torch()
    dev = torch.device("cuda:0")
    M, K, N = 1024, 1024, 16
    A, B, items, offsets = make_case(spmm, M, K, N, 0.8, seed=77)
    d_items = torch.from_numpy(items.view(np.int32).copy()).to(dev)
    d_offs = torch.from_numpy(offsets.copy()).to(dev)
    d_B = torch.from_numpy(np.ascontiguousarray(B).view(np.int16).copy()).to(dev).view(torch.float16)
    d_x = torch.zeros((N, K), dtype=torch.float16, device=dev)
    d_y = torch.zeros((N, M), dtype=torch.float16, device=dev)
    d_z = torch.zeros((N, M), dtype=torch.float16, device=dev)
    d_u = torch.zeros((N, M), dtype=torch.float16, device=dev)
    d_W = torch.zeros((4, N, M), dtype=torch.float16, device=dev)

    def chain(stream):
        # y = A x (Split_K 4, mode 1: fused), z = A y (no split), u = relu(A z) (mode 0: second kernel)
        spmm.SpMM_SplitK_API_Planned(stream, d_items, d_offs, d_x, d_y, M, N, K, d_W, 4, 1, 4, 0, 0, 0)
        spmm.SpMM_SplitK_API_Planned(stream, d_items, d_offs, d_y, d_z, M, N, K, None, 1, 1, 8, 0, 0, 0)
        spmm.SpMM_SplitK_API_Planned(stream, d_items, d_offs, d_z, d_u, M, N, K, d_W, 4, 0, 4, 1, 0,
                                     spmm.SPMM_FLAG_RELU)

    print("[gpu case] graph capture of three chained products", flush=True)
    d_x.copy_(d_B)
    chain(torch.cuda.current_stream())  # eager reference; also arms the kernels' attributes before capture
    torch.cuda.synchronize()
    want = d_u.clone()
    assert torch.isfinite(want).all() and float(want.abs().max()) > 0
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            chain(torch.cuda.current_stream())
    torch.cuda.synchronize()
    for rep in range(4):
        d_y.zero_(); d_z.zero_(); d_u.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(d_u, want), f"replay {rep} differs from the eager result"
        d_u.zero_()
        chain(torch.cuda.current_stream())  # eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(d_u, want)


@pytest.mark.parametrize("N", [16, 32])
def test_wave_count_follows_each_tile_rows_density(spmm, oracle, N):
    """A planner shape whose K-splitting plan uses fewer than eight waves: the library launches
    eight and each workgroup keeps all of them (sparse tile row) or the plan's number (dense one).
    Rows alternate between 50 % and 97 % sparsity in blocks of 128, so both choices occur in one
    launch; the planner's own Split_K (> 1) also puts the fused reduction behind both."""
    M = K = 7168
    split_k = spmm.SpMM_SuggestSplitK(M, N, K)
    plan = spmm.SpMM_PlanLaunch(M, N, K, split_k)
    assert plan["mode"] == 1 and plan["waves"] < 8 and split_k > 1, (plan, split_k)
    dense = spmm.synth_weights(M, K, 0.5, False, seed=61).view(np.uint16)
    sparse = spmm.synth_weights(M, K, 0.97, False, seed=62).view(np.uint16)
    pick = (np.arange(M) // 128) % 2 == 0
    A = np.where(pick[:, None], dense, sparse).view(np.float16)
    B = spmm.synth_activations(N, K, seed=63)
    items, offsets = spmm.InitSparseMatrixA_API(A)
    per_tile = np.diff(offsets[:-1]).reshape(M // 128, K // 64).mean(axis=1)
    assert per_tile.min() < 100 and per_tile.max() > 900  # both sides of the kernel's threshold
    C, _ = run_gpu(spmm, items, offsets, B, M, N, K, split_k)
    assert_close(C, oracle.gemm_f32(A, B))


@pytest.mark.parametrize("flags", [0, 4])
def test_every_partition_of_a_tile_row_among_the_waves(spmm, oracle, flags):
    """The K-splitting layout deals a batch's tiles to 1..8 waves in runs of unequal length.  One
    tile row, 1..113 tiles, every wave count, with exactly representable data (A in {0, 1},
    B in {-5..3}: the reference's own near-exact test values, kernel_benchmark/spmm_test_utils.h:111-141),
    so a tile left out or taken twice changes the result by whole numbers.  flags = 4 launches
    eight waves and lets the kernel choose, as a planned call does."""
    torch = _torch()
    dev = torch.device("cuda:0")
    M, N = 128, 16
    rng = np.random.default_rng(17)
    for tiles in (1, 2, 3, 4, 5, 7, 8, 9, 13, 23, 31, 61, 64, 65, 100, 113):
        K = 64 * tiles
        A = (rng.random((M, K)) < 0.2).astype(np.float16)
        B = rng.integers(-5, 4, size=(N, K)).astype(np.float16)
        ref = oracle.gemm_f32(A, B)
        items, offsets = spmm.InitSparseMatrixA_API(A)
        d_items = torch.from_numpy(items.view(np.int32).copy()).to(dev)
        d_offs = torch.from_numpy(offsets.copy()).to(dev)
        d_B = torch.from_numpy(B.view(np.int16).copy()).to(dev)
        for waves in range(1, 9):
            d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device=dev)
            print(f"[gpu case] partition tiles={tiles} waves={waves} flags={flags}", flush=True)
            spmm.SpMM_SplitK_API_Planned(torch.cuda.current_stream(), d_items, d_offs, d_B, d_C, M, N, K, None, 1, 1,
                                         waves, 0, 0, flags)
            torch.cuda.synchronize()
            assert np.array_equal(d_C.cpu().numpy(), ref.astype(np.float16)), (tiles, waves)  # integers: exact


@pytest.mark.parametrize("N,split_k,waves", [(16, 1, 5), (8, 2, 8), (16, 3, 3)])
def test_long_segments_follow_each_tile_rows_density(spmm, oracle, N, split_k, waves):
    """In the K-splitting layout a workgroup whose tiles mostly exceed 512 vectors streams them in
    segments of 640 instead of 512.  Tile rows alternate between 70 % sparsity (about 614 vectors
    per tile: the long segments), 80 % (410: the short ones) and 55 % (920: short ones, two per
    tile), so all three cases run in one launch; a few tiles of the first kind exceed 640 and
    take two long segments."""
    torch = _torch()
    dev = torch.device("cuda:0")
    M, K = 128 * 9, 64 * 40
    parts = [spmm.synth_weights(M, K, sp, False, seed=70 + i).view(np.uint16) for i, sp in enumerate((0.7, 0.8, 0.55))]
    which = (np.arange(M) // 128) % 3
    A = np.choose(which[:, None], parts).view(np.float16)
    A[0:128, 0:64] = spmm.synth_weights(128, 64, 0.6, False, seed=77)  # one tile of 820 vectors in a 614-average row
    B = spmm.synth_activations(N, K, seed=78)
    items, offsets = spmm.InitSparseMatrixA_API(A)
    per_tile = np.diff(offsets[:-1]).reshape(M // 128, K // 64)
    means = per_tile.mean(axis=1)
    assert 498 <= means[0] <= 640 and means[1] < 498 and means[2] > 640 and per_tile[0].max() > 640
    ref = oracle.gemm_f32(A, B)
    d_items = torch.from_numpy(items.view(np.int32).copy()).to(dev)
    d_offs = torch.from_numpy(offsets.copy()).to(dev)
    d_B = torch.from_numpy(B.view(np.int16).copy()).to(dev)
    for flags in (0, 4):
        d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device=dev)
        d_W = torch.full((split_k, N, M), float("nan"), dtype=torch.float16, device=dev) if split_k > 1 else None
        print(f"[gpu case] long segments N={N} split_k={split_k} waves={waves} flags={flags}", flush=True)
        spmm.SpMM_SplitK_API_Planned(torch.cuda.current_stream(), d_items, d_offs, d_B, d_C, M, N, K, d_W, split_k, 1,
                                     waves, 0, 0, flags)
        torch.cuda.synchronize()
        assert_close(d_C.cpu().numpy(), ref)


@pytest.mark.parametrize("M,K", [(21504, 7168), (7168, 28672), (27648, 9216), (9216, 9216), (36864, 9216), (9216, 36864)])
def test_benchmark_shapes_with_their_planned_launch(spmm, oracle, M, K):
    """The other OPT-30B / OPT-66B shapes of the benchmark at full size, each with the Split_K and launch
    shape the library plans for it, for 8, 16 and 32 tokens: 96 sampled output rows (whole tile rows are
    too slow for the CPU checker) against the oracle, and every row through linearity in B:
    C(B1 + B2) = C(B1) + C(B2) within fp16 rounding of the three results."""
    torch = _torch()
    dev = torch.device("cuda:0")
    A = spmm.synth_weights(M, K, 0.8, False, seed=M // 128 + K)
    items, offsets = spmm.InitSparseMatrixA_API(A)
    d_items = torch.from_numpy(items.view(np.int32)).to(dev)
    d_offs = torch.from_numpy(offsets).to(dev)
    rows = np.sort(np.random.default_rng(M + K).choice(M, size=96, replace=False))
    A_rows = np.ascontiguousarray(A[rows])
    for N in (8, 16, 32):
        split_k = spmm.SpMM_SuggestSplitK(M, N, K)
        B1 = spmm.synth_activations(N, K, seed=5 + N)
        B2 = spmm.synth_activations(N, K, seed=6 + N)
        B3 = (B1.astype(np.float32) + B2.astype(np.float32)).astype(np.float16)
        outs = []
        d_W = torch.zeros((max(split_k, 1), N, M), dtype=torch.float16, device=dev)
        for Bx in (B1, B2, B3):
            d_B = torch.from_numpy(Bx.view(np.int16).copy()).to(dev)
            d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device=dev)
            print(f"[gpu case] benchmark shape M={M} K={K} N={N} split_k={split_k}", flush=True)
            spmm.SpMM_SplitK_API(torch.cuda.current_stream(), None, d_items, d_offs, d_B, d_C, M, N, K, d_W, split_k)
            torch.cuda.synchronize()
            outs.append(d_C.cpu().numpy().astype(np.float32))
        assert_close(outs[0][:, rows], oracle.gemm_f32(A_rows, B1))
        # B3 is B1 + B2 rounded to fp16: compare against the sum within the tolerance of each term
        # plus the effect of that rounding (2^-11 relative on every input of a sum of K * 0.2 terms)
        lin = np.abs(outs[2] - (outs[0] + outs[1]))
        bound = 3 * (ATOL + RTOL * np.maximum(np.abs(outs[2]), np.abs(outs[0]) + np.abs(outs[1])))
        assert (lin <= bound).all(), float(lin.max())


@pytest.mark.parametrize("N,split_k,mode,waves,stage_b", [(16, 1, 1, 5, 0), (8, 2, 1, 8, 0), (32, 1, 1, 4, 0), (64, 2, 1, 4, 0),
                                                         (16, 4, 0, 6, 1), (32, 2, 0, 4, 0)])
def test_short_segments_on_sparse_tile_rows(spmm, oracle, N, split_k, mode, waves, stage_b):
    """Runs whose tiles average at most 232 (112) vectors are streamed in segments of 256 (128)
    vectors.  Tile rows alternate between 90 % sparsity (205 vectors per tile), 96 % (82) and 80 %
    (410, the regular segments); one 80 % tile sits in a 96 % row and takes four of its row's short
    segments, and one tile of that row is empty."""
    torch = _torch()
    dev = torch.device("cuda:0")
    M, K = 128 * 9, 64 * 40
    parts = [spmm.synth_weights(M, K, sp, False, seed=90 + i).view(np.uint16) for i, sp in enumerate((0.9, 0.96, 0.8))]
    which = (np.arange(M) // 128) % 3
    A = np.choose(which[:, None], parts).view(np.float16).copy()
    A[128:256, 64:128] = spmm.synth_weights(128, 64, 0.8, False, seed=97)
    A[128:256, 192:256] = 0
    B = spmm.synth_activations(N, K, seed=98)
    items, offsets = spmm.InitSparseMatrixA_API(A)
    per_tile = np.diff(offsets[:-1]).reshape(M // 128, K // 64)
    means = per_tile.mean(axis=1)
    assert 112 < means[0] <= 232 and means[1] <= 112 and means[2] > 232 and per_tile[1].max() > 384 and per_tile[1].min() == 0
    ref = oracle.gemm_f32(A, B)
    d_items = torch.from_numpy(items.view(np.int32).copy()).to(dev)
    d_offs = torch.from_numpy(offsets.copy()).to(dev)
    d_B = torch.from_numpy(B.view(np.int16).copy()).to(dev)
    for flags in ((0, 4) if mode == 1 and N <= 32 else (0,)):
        d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device=dev)
        d_W = torch.full((split_k, N, M), float("nan"), dtype=torch.float16, device=dev) if split_k > 1 else None
        print(f"[gpu case] short segments N={N} split_k={split_k} mode={mode} waves={waves} flags={flags}", flush=True)
        spmm.SpMM_SplitK_API_Planned(torch.cuda.current_stream(), d_items, d_offs, d_B, d_C, M, N, K, d_W, split_k, mode,
                                     waves, stage_b, 0, flags)
        torch.cuda.synchronize()
        assert_close(d_C.cpu().numpy(), ref)


def _hip_runtime():
    """The HIP runtime this process already holds (torch's), for making and destroying raw streams."""
    import ctypes

    _torch()
    with open("/proc/self/maps") as f:
        paths = {line.split()[-1] for line in f if "libamdhip64" in line}
    assert len(paths) == 1, paths
    hip = ctypes.CDLL(paths.pop())
    hip.hipStreamCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
    hip.hipStreamDestroy.argtypes = [ctypes.c_void_p]
    hip.hipStreamSynchronize.argtypes = [ctypes.c_void_p]
    return hip


def _fused_case(spmm, M=1024, K=2048, N=16, split_k=4, seed=321):
    """Device operands of a call that takes the in-launch reduction (K-splitting launch, Split_K > 1),
    and the bits of the same call with the reduction as a second kernel."""
    torch = _torch()
    dev = torch.device("cuda:0")
    A, B, items, offsets = make_case(spmm, M, K, N, 0.8, seed=seed)
    d_items = torch.from_numpy(items.view(np.int32).copy()).to(dev)
    d_offs = torch.from_numpy(offsets.copy()).to(dev)
    d_B = torch.from_numpy(np.ascontiguousarray(B).view(np.int16).copy()).to(dev)
    d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device=dev)
    d_W = torch.full((split_k, N, M), float("nan"), dtype=torch.float16, device=dev)
    spmm.SpMM_SplitK_API_Planned(None, d_items, d_offs, d_B, d_C, M, N, K, d_W, split_k, 1, 4, 0, 0,
                                 spmm.SPMM_FLAG_SEPARATE_REDUCTION)
    torch.cuda.synchronize()
    return (d_items, d_offs, d_B, M, N, K, split_k), d_C.cpu().numpy().view(np.uint16)


def test_fused_reduction_with_many_short_lived_streams(spmm):
    """More stream handles than there are counter pages, each used once and destroyed: every call
    must still give the bits of the separate reduction (pages of idle or destroyed streams change
    hands; a call that finds none runs the second kernel)."""
    import ctypes

    torch = _torch()
    hip = _hip_runtime()
    (d_items, d_offs, d_B, M, N, K, split_k), want = _fused_case(spmm)
    print("[gpu case] fused reduction on 200 short-lived streams", flush=True)
    for i in range(200):
        s = ctypes.c_void_p()
        assert hip.hipStreamCreate(ctypes.byref(s)) == 0
        d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device="cuda:0")
        d_W = torch.full((split_k, N, M), float("nan"), dtype=torch.float16, device="cuda:0")
        torch.cuda.synchronize()
        spmm.SpMM_SplitK_API_Planned(s.value, d_items, d_offs, d_B, d_C, M, N, K, d_W, split_k, 1, 4, 0, 0, 0)
        assert hip.hipStreamSynchronize(s) == 0
        assert np.array_equal(d_C.cpu().numpy().view(np.uint16), want), f"stream {i}"
        assert hip.hipStreamDestroy(s) == 0


def test_fused_reduction_with_more_live_streams_than_pages(spmm):
    """96 streams alive at once, calls dealt round robin without waiting: streams beyond the pages
    get one only when an owner has gone idle, else the second kernel; same bits either way."""
    import ctypes

    torch = _torch()
    hip = _hip_runtime()
    (d_items, d_offs, d_B, M, N, K, split_k), want = _fused_case(spmm, seed=322)
    streams, outs = [], []
    for i in range(96):
        s = ctypes.c_void_p()
        assert hip.hipStreamCreate(ctypes.byref(s)) == 0
        streams.append(s)
        outs.append((torch.full((N, M), float("nan"), dtype=torch.float16, device="cuda:0"),
                     torch.full((split_k, N, M), float("nan"), dtype=torch.float16, device="cuda:0")))
    torch.cuda.synchronize()
    print("[gpu case] fused reduction on 96 live streams", flush=True)
    for rep in range(3):
        for s, (d_C, d_W) in zip(streams, outs):
            spmm.SpMM_SplitK_API_Planned(s.value, d_items, d_offs, d_B, d_C, M, N, K, d_W, split_k, 1, 4, 0, 0, 0)
    for s in streams:
        assert hip.hipStreamSynchronize(s) == 0
    for i, (d_C, _) in enumerate(outs):
        assert np.array_equal(d_C.cpu().numpy().view(np.uint16), want), f"stream {i}"
    for s in streams:
        assert hip.hipStreamDestroy(s) == 0


def test_graph_replay_beside_eager_calls_on_the_capture_stream(spmm):
    """A graph captured on stream S keeps counting on its own page: replays on another stream run
    while eager calls with the in-launch reduction are queued on S, and both give the right bits."""
    torch = _torch()
    (d_items, d_offs, d_B, M, N, K, split_k), want = _fused_case(spmm, M=2048, K=4096, seed=323)
    dev = torch.device("cuda:0")
    mk = lambda: (torch.full((N, M), float("nan"), dtype=torch.float16, device=dev),
                  torch.full((split_k, N, M), float("nan"), dtype=torch.float16, device=dev))
    (gC, gW), (eC, eW) = mk(), mk()
    S, other = torch.cuda.Stream(), torch.cuda.Stream()

    def call(stream, C, W):
        spmm.SpMM_SplitK_API_Planned(stream, d_items, d_offs, d_B, C, M, N, K, W, split_k, 1, 4, 0, 0, 0)

    call(S, eC, eW)  # eager first: arms the kernel's attributes, gives S its eager page
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(S):
        with torch.cuda.graph(g, stream=S):
            for _ in range(4):
                call(torch.cuda.current_stream(), gC, gW)
    torch.cuda.synchronize()
    print("[gpu case] graph replays on one stream beside eager calls on the capture stream", flush=True)
    for rep in range(5):
        gC.fill_(float("nan"))
        eC.fill_(float("nan"))
        torch.cuda.synchronize()
        with torch.cuda.stream(other):
            g.replay()
        for _ in range(8):
            call(S, eC, eW)
        torch.cuda.synchronize()
        assert np.array_equal(gC.cpu().numpy().view(np.uint16), want), f"replay {rep}"
        assert np.array_equal(eC.cpu().numpy().view(np.uint16), want), f"eager beside replay {rep}"


@pytest.mark.parametrize("M,K,N,split_k,waves,sparsity", [
    (1024, 1024, 32, 4, 4, 0.8),
    (1024, 1024, 32, 2, 8, 0.8),
    (1024, 1024, 64, 2, 4, 0.8),
    (1152, 1536, 64, 3, 4, 0.8),     # nine tile rows: the last workgroup has three waves without rows
    (640, 2048, 32, 1, 8, 0.8),      # five tile rows over eight waves, no split: the kernel writes C itself
    (512, 1024, 64, 2, 4, 0.5),      # tiles of several segments (the image is cleared, not un-scattered)
    (512, 1024, 32, 2, 4, 0.3),
    (1024, 2048, 64, 4, 4, 0.95),    # short segments, some waves on sparser rows than others
    (512, 64 * 70, 32, 1, 4, 0.9),   # more than 63 tiles per wave: the offsets window slides
])
def test_shared_activation_tiles_through_lds(spmm, oracle, M, K, N, split_k, waves, sparsity):
    """Row-sharing launch whose waves walk their tile rows in step and share each activation tile
    through LDS (StageB = 2), 32 and 64 tokens: against the oracle, with the second-kernel and the
    in-launch reduction, and with empty tiles and rows of different density in one workgroup."""
    torch = _torch()
    dev = torch.device("cuda:0")
    A = spmm.synth_weights(M, K, sparsity, False, seed=M + K + N + waves)
    A[128:256, :] = spmm.synth_weights(128, K, min(0.99, sparsity + 0.15), False, seed=3)   # a sparser tile row
    A[0:128, 64:192] = 0                                                                   # two empty tiles
    if M >= 512:
        A[384:512, :] = 0                                                                  # a whole empty tile row
    B = spmm.synth_activations(N, K, seed=M + 1)
    items, offsets = spmm.InitSparseMatrixA_API(A)
    ref = oracle.gemm_f32(A, B)
    d_items = torch.from_numpy(items.view(np.int32).copy()).to(dev)
    d_offs = torch.from_numpy(offsets.copy()).to(dev)
    d_B = torch.from_numpy(B.view(np.int16).copy()).to(dev)
    for flags in (0, spmm.SPMM_FLAG_SEPARATE_REDUCTION):
        d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device=dev)
        d_W = torch.full((split_k, N, M), float("nan"), dtype=torch.float16, device=dev) if split_k > 1 else None
        print(f"[gpu case] shared activation tiles M={M} K={K} N={N} split_k={split_k} waves={waves} flags={flags}", flush=True)
        spmm.SpMM_SplitK_API_Planned(torch.cuda.current_stream(), d_items, d_offs, d_B, d_C, M, N, K, d_W, split_k, 0,
                                     waves, 2, 0, flags)
        torch.cuda.synchronize()
        assert_close(d_C.cpu().numpy(), ref)


def test_shared_activation_tiles_rejects_other_shapes(spmm):
    torch = _torch()
    z = torch.zeros(1024, dtype=torch.int32, device="cuda:0")
    for (N, mode, waves, row_major) in [(16, 0, 4, 0), (32, 0, 2, 0), (64, 0, 2, 0), (32, 1, 4, 0), (64, 0, 4, 1), (8, 0, 8, 0)]:
        with pytest.raises(spmm.SpMMError):
            spmm.SpMM_SplitK_API_Planned(None, z, z, z, z, 1024, N, 1024, z, 1, mode, waves, 2, row_major)
