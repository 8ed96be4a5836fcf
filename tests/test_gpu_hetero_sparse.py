"""GPU parity of the 2:4 + residual path through the C ABI against the CPU oracle.

ref = fp32-accumulate dense product (oracle) on the matrix the device data decodes to;
tolerance |gpu - ref| <= 1e-2 + 1e-2 * |ref| per element, as for the Tiled-CSL path.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ATOL, RTOL = 1e-2, 1e-2


def _torch():
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch


def _dev(a):
    torch = _torch()
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        a = a.view(np.int16)
    elif a.dtype == np.uint32:
        a = a.view(np.int32)
    if a.size == 0:
        return torch.zeros(4, dtype=torch.int32, device="cuda:0")
    return torch.from_numpy(a.copy()).to("cuda:0")


def assert_close(C, ref):
    C = C.astype(np.float32)
    assert np.isfinite(C).all(), "non-finite output (unwritten or corrupt)"
    err = np.abs(C - ref)
    bad = err > ATOL + RTOL * np.abs(ref)
    assert not bad.any(), f"{bad.sum()} elements out of tolerance, max err {err.max()} at {np.unravel_index(err.argmax(), err.shape)}"


def run_a1(spmm, packed, B, M, N, K, split_k, rb=0, waves=0, share_b=0):
    torch = _torch()
    d_p, d_B = _dev(packed), _dev(B)
    d_W = torch.full((split_k, N, M), float("nan"), dtype=torch.float16, device="cuda:0")
    print(f"[gpu case] A1 partials M={M} N={N} K={K} split_k={split_k} rb={rb} waves={waves} share_b={share_b}", flush=True)
    spmm.HeteroSparse_A1_Partials(torch.cuda.current_stream(), d_p, d_B, d_W, M, N, K, split_k, rb, waves, share_b)
    torch.cuda.synchronize()
    return d_W.cpu().numpy()


def run_hybrid(spmm, packed, items, offsets, B, M, N, K, s1, s2, flags=0):
    torch = _torch()
    d_p, d_B = _dev(packed), _dev(B)
    d_items = _dev(items) if items is not None else None
    d_offs = _dev(offsets) if offsets is not None else None
    d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device="cuda:0")
    d_W = torch.full((s1 + s2, N, M), float("nan"), dtype=torch.float16, device="cuda:0")
    print(f"[gpu case] hybrid M={M} N={N} K={K} split_k={s1}/{s2}", flush=True)
    spmm.HeteroSparse_SpMM_API(torch.cuda.current_stream(), d_p, d_items, d_offs, d_B, d_C, M, N, K, d_W, s1, s2, flags)
    torch.cuda.synchronize()
    return d_C.cpu().numpy()


def test_a1_layout_one_hot(spmm, oracle):
    """Pins rows, columns, tokens and the position fields: distinct exactly representable integers
    on a 2:4 pattern, one-hot activations, so C[n, m] must equal A1[m, k_n] exactly."""
    M, K, N = 128, 256, 16
    rng = np.random.default_rng(3)
    A = np.zeros((M, K), dtype=np.float16)
    mask = rng.random((M, K)) < 0.6
    vals = (np.arange(M * K).reshape(M, K) % 1999 + 1).astype(np.float16)
    A[mask] = vals[mask]
    A1, _ = spmm.HeteroSparse_Decompose(A)
    packed = spmm.HeteroSparse_PackA1(A1)
    for trial in range(4):
        ks = rng.permutation(K)[:N]
        B = np.zeros((N, K), dtype=np.float16)
        B[np.arange(N), ks] = 1.0
        W = run_a1(spmm, packed, B, M, N, K, 1)
        assert np.array_equal(W[0].view(np.uint16), A1[:, ks].T.view(np.uint16))


@pytest.mark.parametrize("N", [8, 16, 32, 64])
@pytest.mark.parametrize("rb,waves", [(1, 4), (2, 2), (2, 4), (2, 8), (4, 1), (4, 4), (8, 2)])
def test_a1_launch_shapes_vs_oracle(spmm, oracle, N, rb, waves):
    M, K = 256, 640  # five units: uneven among 2, 4 and 8 waves, some waves idle
    A = spmm.synth_weights(M, K, 0.5, False, seed=N + rb)
    B = spmm.synth_activations(N, K, seed=77)
    A1, _ = spmm.HeteroSparse_Decompose(A)
    packed = spmm.HeteroSparse_PackA1(A1)
    if N == 64 and rb == 8:
        with pytest.raises(spmm.SpMMError):  # not in the kernel table: too many accumulators
            run_a1(spmm, packed, B, M, N, K, 1, rb, waves)
        return
    for split_k in (1, 2):
        W = run_a1(spmm, packed, B, M, N, K, split_k, rb, waves)
        per = -(-(K // 128) // split_k)
        for b in range(split_k):
            ref = oracle.gemm_f32(oracle.a24_unpack(packed, M, K), B, b * per * 128, min(K, (b + 1) * per * 128))
            assert_close(W[b], ref)


@pytest.mark.parametrize("N", [8, 16, 32, 64])
@pytest.mark.parametrize("rb,waves", [(2, 4), (2, 8), (4, 2), (4, 4), (4, 8), (8, 2), (8, 4)])
def test_a1_shared_tile_shapes_vs_oracle(spmm, oracle, N, rb, waves):
    """The layout whose waves own rows and share the activation tile through LDS."""
    M, K = 512, 640  # five units: odd count, both buffers and both loop phases end a batch
    A = spmm.synth_weights(M, K, 0.5, False, seed=N + rb + waves)
    B = spmm.synth_activations(N, K, seed=78)
    A1, _ = spmm.HeteroSparse_Decompose(A)
    packed = spmm.HeteroSparse_PackA1(A1)
    dense = oracle.a24_unpack(packed, M, K)
    if rb > (2 if N == 64 else 4):
        with pytest.raises(spmm.SpMMError):  # not in the kernel table: too many registers
            run_a1(spmm, packed, B, M, N, K, 1, rb, waves, 1)
        return
    for split_k in (1, 2, 5):
        W = run_a1(spmm, packed, B, M, N, K, split_k, rb, waves, 1)
        per = -(-(K // 128) // split_k)
        for b in range(split_k):
            assert_close(W[b], oracle.gemm_f32(dense, B, b * per * 128, min(K, (b + 1) * per * 128)))


def test_a1_shared_tile_rejects_partial_workgroups(spmm):
    torch = _torch()
    d = torch.zeros(1 << 16, dtype=torch.int32, device="cuda:0")
    with pytest.raises(spmm.SpMMError):  # 128 rows are not a multiple of 16 * 4 * 4
        spmm.HeteroSparse_A1_Partials(None, d, d, d, 128, 16, 128, 1, 4, 4, 1)


@pytest.mark.parametrize("sparsity", [0.5, 0.7, 0.8, 0.95])
@pytest.mark.parametrize("N", [8, 16, 64])
def test_hybrid_vs_oracle(spmm, oracle, sparsity, N):
    M, K = 512, 1024
    A = spmm.synth_weights(M, K, sparsity, False, seed=int(sparsity * 100))
    B = spmm.synth_activations(N, K, seed=5)
    A1, A2 = spmm.HeteroSparse_Decompose(A)
    packed = spmm.HeteroSparse_PackA1(A1)
    items, offsets = spmm.InitSparseMatrixA_API(A2)
    ref = oracle.gemm_f32(A, B)
    for s1, s2, flags in ((1, 1, 0), (2, 3, 0), (2, 2, spmm.HETERO_FLAG_TWO_STREAMS)):
        C = run_hybrid(spmm, packed, items, offsets, B, M, N, K, s1, s2, flags)
        assert_close(C, ref)


def test_hybrid_without_residual_and_errors(spmm, oracle):
    torch = _torch()
    M, K, N = 256, 512, 16
    A = spmm.synth_weights(M, K, 0.9, False, seed=9)
    A1, A2 = spmm.HeteroSparse_Decompose(A)
    B = spmm.synth_activations(N, K, seed=6)
    packed = spmm.HeteroSparse_PackA1(A1)
    ref = oracle.gemm_f32(A1, B)
    for s1 in (1, 4):
        C = run_hybrid(spmm, packed, None, None, B, M, N, K, s1, 0)
        assert_close(C, ref)
    d = torch.zeros(16, dtype=torch.int32, device="cuda:0")
    for bad in (dict(M=200), dict(K=576), dict(N=24), dict(s1=5)):  # K=512 has 4 units: 5 batches leave one empty
        a = dict(M=M, K=K, N=N, s1=1)
        a.update(bad)
        with pytest.raises(spmm.SpMMError):
            spmm.HeteroSparse_SpMM_API(None, d, None, None, d, d, a["M"], a["N"], a["K"], d, a["s1"], 0, 0)


def test_hybrid_full_size_sampled_rows(spmm, oracle):
    """OPT-30B FFN1 at 70 % sparsity, N = 16: sampled rows against the oracle, and linearity
    (C(B1 + B2) == C(B1) + C(B2) within rounding) on every row."""
    M, K, N = 28672, 7168, 16
    A = spmm.synth_weights(M, K, 0.7, False, seed=21)
    A1, A2 = spmm.HeteroSparse_Decompose(A)
    packed = spmm.HeteroSparse_PackA1(A1)
    items, offsets = spmm.InitSparseMatrixA_API(A2)
    B1 = spmm.synth_activations(N, K, seed=1)
    B2 = spmm.synth_activations(N, K, seed=2)
    s1 = spmm.HeteroSparse_SuggestSplitK(M, N, K)
    s2 = spmm.SpMM_SuggestSplitK(M, N, K)
    C1 = run_hybrid(spmm, packed, items, offsets, B1, M, N, K, s1, s2)
    rows = np.random.default_rng(0).choice(M, 512, replace=False)
    rows.sort()
    ref = oracle.gemm_f32(np.ascontiguousarray(A[rows]), B1)
    assert_close(C1[:, rows], ref)
    Bs = (B1.astype(np.float32) * 0.5 + B2.astype(np.float32) * 0.5).astype(np.float16)
    exact = np.array_equal(Bs.astype(np.float32), B1.astype(np.float32) * 0.5 + B2.astype(np.float32) * 0.5)
    C2 = run_hybrid(spmm, packed, items, offsets, B2, M, N, K, s1, s2)
    Cs = run_hybrid(spmm, packed, items, offsets, Bs, M, N, K, s1, s2)
    lin = 0.5 * C1.astype(np.float32) + 0.5 * C2.astype(np.float32)
    tol = 2e-2 if exact else 4e-2
    assert np.isfinite(Cs).all()
    assert (np.abs(Cs.astype(np.float32) - lin) <= tol + tol * np.abs(lin)).all()


@pytest.mark.parametrize("flags_name", ["one_stream", "two_streams"])
def test_hybrid_hip_graph_replays_match_eager(spmm, oracle, flags_name):
    """The hybrid call captured into a HIP graph and replayed, with eager calls in between, gives
    the eager bits every time (the library records kernels and event edges only, no memset nodes)."""
    torch = _torch()
    flags = spmm.HETERO_FLAG_TWO_STREAMS if flags_name == "two_streams" else 0
    M, K, N = 1024, 1024, 16
    A = spmm.synth_weights(M, K, 0.6, False, seed=31)
    A1, A2 = spmm.HeteroSparse_Decompose(A)
    d_p = _dev(spmm.HeteroSparse_PackA1(A1))
    items, offsets = spmm.InitSparseMatrixA_API(A2)
    d_items, d_offs = _dev(items), _dev(offsets)
    d_B = _dev(spmm.synth_activations(N, K, seed=32))
    d_C = torch.zeros((N, M), dtype=torch.float16, device="cuda:0")
    d_W = torch.zeros((6, N, M), dtype=torch.float16, device="cuda:0")

    def call(stream):
        spmm.HeteroSparse_SpMM_API(stream, d_p, d_items, d_offs, d_B, d_C, M, N, K, d_W, 2, 4, flags)

    print(f"[gpu case] graph capture of the hybrid call, {flags_name}", flush=True)
    call(torch.cuda.current_stream())  # eager reference; creates the library's second stream before capture
    torch.cuda.synchronize()
    want = d_C.clone()
    assert_close(want.cpu().numpy(), oracle.gemm_f32(A, spmm.synth_activations(N, K, seed=32)))
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        call(torch.cuda.current_stream())  # the capturing stream gets its own second stream first
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            call(torch.cuda.current_stream())
    torch.cuda.synchronize()
    for rep in range(3):
        d_C.zero_()
        d_W.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(d_C, want), f"replay {rep} differs from the eager result"
        d_C.zero_()
        call(torch.cuda.current_stream())
        torch.cuda.synchronize()
        assert torch.equal(d_C, want)


def test_a1_full_size_ffn2_n64_sampled_rows(spmm, oracle):
    """OPT-30B FFN2 (7168 x 28672) as a 2:4 weight, N = 64, the library's own launch: sampled rows."""
    M, K, N = 7168, 28672, 64
    A = spmm.synth_weights(M, K, 0.6, False, seed=41)
    A1, _ = spmm.HeteroSparse_Decompose(A)
    packed = spmm.HeteroSparse_PackA1(A1)
    B = spmm.synth_activations(N, K, seed=42)
    s1 = spmm.HeteroSparse_SuggestSplitK(M, N, K)
    assert s1 > 1
    C = run_hybrid(spmm, packed, None, None, B, M, N, K, s1, 0)
    rows = np.sort(np.random.default_rng(1).choice(M, 256, replace=False))
    assert_close(C[:, rows], oracle.gemm_f32(np.ascontiguousarray(A1[rows]), B))


@pytest.mark.parametrize("M,K,sparsity", [(128, 128, 0.5), (256, 640, 0.2), (1024, 2048, 0.8), (128, 128, 1.0), (384, 256, 0.0)])
def test_device_split_pack_equals_host(spmm, oracle, M, K, sparsity):
    """The GPU's split + pack against the host's (itself pinned by the oracle), bit for bit,
    including -0, NaN, denormal and infinity patterns; then the device-made pair through the hybrid."""
    torch = _torch()
    A = spmm.synth_weights(M, K, sparsity, False, seed=M + K)
    A.view(np.uint16)[0, :8] = [0x8000, 0x7E00, 0x0001, 0x3C00, 0xFC00, 0x8001, 0, 0x7C00]
    A1, A2 = oracle.decompose(A)
    want = spmm.HeteroSparse_PackA1(A1)
    d_A = torch.from_numpy(A.view(np.int16).copy()).to("cuda:0").view(torch.float16)
    print(f"[gpu case] device split+pack M={M} K={K} sparsity={sparsity}", flush=True)
    packed, residual = spmm.split_pack_on_device(d_A)
    torch.cuda.synchronize()
    assert np.array_equal(packed.cpu().numpy(), want)
    assert np.array_equal(residual.cpu().numpy().view(np.uint16), A2.view(np.uint16))
    packed_only, none = spmm.split_pack_on_device(d_A, want_residual=False)
    torch.cuda.synchronize()
    assert none is None and torch.equal(packed_only, packed)


def test_device_pipeline_dense_to_hybrid(spmm, oracle):
    """Dense weight on the GPU -> records + residual -> Tiled-CSL of the residual -> product, no host step."""
    torch = _torch()
    M, K, N = 512, 1024, 16
    A = spmm.synth_weights(M, K, 0.6, False, seed=55)
    A.view(np.uint16)[A.view(np.uint16) == 0x8000] = 0
    B = spmm.synth_activations(N, K, seed=56)
    d_A = torch.from_numpy(A.view(np.int16).copy()).to("cuda:0").view(torch.float16)
    packed, residual = spmm.split_pack_on_device(d_A)
    items, offs = spmm.encode_on_device(residual)
    d_B = _dev(B)
    d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device="cuda:0")
    d_W = torch.empty((4, N, M), dtype=torch.float16, device="cuda:0")
    print("[gpu case] device pipeline dense -> hybrid", flush=True)
    spmm.HeteroSparse_SpMM_API(torch.cuda.current_stream(), packed, items, offs, d_B, d_C, M, N, K, d_W, 2, 2)
    torch.cuda.synchronize()
    assert_close(d_C.cpu().numpy(), oracle.gemm_f32(A, B))


def test_device_split_pack_rejects_bad_shapes(spmm):
    torch = _torch()
    d = torch.zeros((64, 128), dtype=torch.float16, device="cuda:0")
    with pytest.raises(spmm.SpMMError):
        spmm.split_pack_on_device(d)


@pytest.mark.parametrize("N", [16, 64])
def test_hybrid_with_row_sharing_residual_launch(spmm, oracle, N):
    """A shape whose residual launch is of the row-sharing kind, which has no in-launch reduction:
    the hybrid must fall back to the separate reduction kernel over all slabs."""
    M, K, s1, s2 = 16384, 512, 2, 3
    assert spmm.SpMM_PlanLaunch(M, N, K, s2)["mode"] == 0
    A = spmm.synth_weights(M, K, 0.6, False, seed=71 + N)
    A1, A2 = spmm.HeteroSparse_Decompose(A)
    packed = spmm.HeteroSparse_PackA1(A1)
    items, offsets = spmm.InitSparseMatrixA_API(A2)
    B = spmm.synth_activations(N, K, seed=72)
    C = run_hybrid(spmm, packed, items, offsets, B, M, N, K, s1, s2)
    assert_close(C, oracle.gemm_f32(A, B))


# ---------------------------------------------------------------------------------------------
# both parts in one launch


def run_fused(spmm, packed, words, offs, longest, B, M, N, K, split_k):
    torch = _torch()
    d_p, d_B, d_w, d_o = _dev(packed), _dev(B), _dev(words), _dev(offs)
    d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device="cuda:0")
    d_W = torch.full((max(split_k, 1), N, M), float("nan"), dtype=torch.float16, device="cuda:0")
    print(f"[gpu case] fused M={M} N={N} K={K} split_k={split_k} longest={longest}", flush=True)
    spmm.HeteroSparse_Fused_SpMM_API(torch.cuda.current_stream(), d_p, d_w, d_o, longest, d_B, d_C, M, N, K, d_W, split_k)
    torch.cuda.synchronize()
    return d_C.cpu().numpy()


def test_fused_layout_one_hot(spmm, oracle):
    """Pins rows, columns and tokens of both parts at once: distinct exactly representable integers,
    one-hot activations, so C[n, m] must equal A[m, k_n] exactly whichever part holds that element."""
    M, K, N = 256, 384, 16
    rng = np.random.default_rng(4)
    A = np.zeros((M, K), dtype=np.float16)
    mask = rng.random((M, K)) < 0.45
    vals = (np.arange(M * K).reshape(M, K) % 1999 + 1).astype(np.float16)
    A[mask] = vals[mask]
    A1, A2 = oracle.decompose(A)
    assert np.count_nonzero(A2) > 1000
    packed = spmm.HeteroSparse_PackA1(A1)
    words, offs, longest = spmm.HeteroSparse_PackA2(A2)
    for trial in range(4):
        ks = rng.permutation(K)[:N]
        B = np.zeros((N, K), dtype=np.float16)
        B[np.arange(N), ks] = 1.0
        C = run_fused(spmm, packed, words, offs, longest, B, M, N, K, 1)
        assert np.array_equal(C.view(np.uint16), A[:, ks].T.view(np.uint16))


@pytest.mark.parametrize("sparsity", [0.45, 0.5, 0.6, 0.7, 0.8, 0.95])
@pytest.mark.parametrize("N", [8, 16, 32, 64])
@pytest.mark.parametrize("M", [384, 512])
def test_fused_vs_oracle(spmm, oracle, sparsity, N, M):
    """One to five loads per list (45 % ... 95 % sparsity), four waves (384 rows) and eight (512 rows,
    once the split gives enough workgroups), nine units split one, two and three ways."""
    K = 1152
    A = spmm.synth_weights(M, K, sparsity, False, seed=int(sparsity * 100) + N)
    B = spmm.synth_activations(N, K, seed=5)
    A1, A2 = spmm.HeteroSparse_Decompose(A)
    packed = spmm.HeteroSparse_PackA1(A1)
    words, offs, longest = spmm.HeteroSparse_PackA2(A2)
    ref = oracle.gemm_f32(A, B)
    for split_k in (1, 2, 3):
        C = run_fused(spmm, packed, words, offs, longest, B, M, N, K, split_k)
        assert_close(C, ref)


@pytest.mark.parametrize("M,K,split_k", [(128, 128, 1), (128, 384, 3), (256, 256, 2), (640, 512, 1)])
def test_fused_shortest_batches(spmm, oracle, M, K, split_k):
    """Batches of a single unit (the pipeline's start and end only) and of two."""
    N = 32
    A = spmm.synth_weights(M, K, 0.55, False, seed=M + K)
    B = spmm.synth_activations(N, K, seed=9)
    A1, A2 = spmm.HeteroSparse_Decompose(A)
    words, offs, longest = spmm.HeteroSparse_PackA2(A2)
    C = run_fused(spmm, spmm.HeteroSparse_PackA1(A1), words, offs, longest, B, M, N, K, split_k)
    assert_close(C, oracle.gemm_f32(A, B))


@pytest.mark.parametrize("N", [16, 64])
def test_fused_eight_waves_and_empty_lists(spmm, oracle, N):
    """49152 rows in workgroups of eight waves (192 of them > 160); rows 0..255 have no residual at
    all (empty lists at the start), one record's list is the only one of its row block."""
    M, K = 49152, 256
    A = spmm.synth_weights(M, K, 0.6, False, seed=N)
    A[:256] = np.where(np.arange(K) % 4 < 2, A[:256], 0)   # two of four everywhere: nothing left over
    A[4096:4112, 128:] = np.where(np.arange(128) % 4 < 2, A[4096:4112, 128:], 0)
    B = spmm.synth_activations(N, K, seed=8)
    A1, A2 = spmm.HeteroSparse_Decompose(A)
    assert not A2[:256].any() and not A2[4096:4112, 128:].any()
    packed = spmm.HeteroSparse_PackA1(A1)
    words, offs, longest = spmm.HeteroSparse_PackA2(A2)
    C = run_fused(spmm, packed, words, offs, longest, B, M, N, K, 1)
    rows = np.r_[0:512, 4000:4200, np.sort(np.random.default_rng(2).choice(M, 1024, replace=False))]
    assert_close(C[:, rows], oracle.gemm_f32(np.ascontiguousarray(A[rows]), B))


def test_fused_without_any_residual(spmm, oracle):
    M, K, N = 256, 512, 16
    A, _ = spmm.HeteroSparse_Decompose(spmm.synth_weights(M, K, 0.5, False, seed=10))
    B = spmm.synth_activations(N, K, seed=6)
    A1, A2 = spmm.HeteroSparse_Decompose(A)
    assert not A2.any()
    words, offs, longest = spmm.HeteroSparse_PackA2(A2)
    assert longest == 0 and offs[-1] == 0
    C = run_fused(spmm, spmm.HeteroSparse_PackA1(A1), words, offs, longest, B, M, N, K, 2)
    assert_close(C, oracle.gemm_f32(A, B))


def test_fused_rejects(spmm):
    torch = _torch()
    d = torch.zeros(1 << 12, dtype=torch.int32, device="cuda:0")
    ok = dict(M=256, N=16, K=512, longest=10, s=1)
    for bad in (dict(M=200), dict(K=576), dict(N=24), dict(s=5), dict(longest=spmm.HETERO_FUSED_MAX_LIST + 1), dict(longest=-1)):
        a = dict(ok)
        a.update(bad)
        with pytest.raises(spmm.SpMMError):
            spmm.HeteroSparse_Fused_SpMM_API(None, d, d, d, a["longest"], d, d, a["M"], a["N"], a["K"], d, a["s"])
    with pytest.raises(spmm.SpMMError):
        spmm.HeteroSparse_Fused_SpMM_API(None, d, None, d, 10, d, d, 256, 16, 512, d, 1)
    with pytest.raises(spmm.SpMMError):  # a split needs the workspace
        spmm.HeteroSparse_Fused_SpMM_API(None, d, d, d, 10, d, d, 256, 16, 512, None, 2)


@pytest.mark.parametrize("N", [8, 16, 32, 64])
@pytest.mark.parametrize("sparsity,skew", [(0.5, True), (0.3, False), (0.1, False)])
def test_fused_lists_longer_than_the_pipelined_rounds(spmm, oracle, N, sparsity, skew):
    """Beta(2, 8) row densities (and a nearly dense weight) leave blocks with more than 320 residual
    values, up to the 1024 a block can hold: the first five rounds of such a list travel with the
    records, the rest is fetched inside the multiplication.  Both layouts, one and three batches,
    against the oracle; exact one-hot probe of where every word lands."""
    M, K = 1024, 1024
    A = spmm.synth_weights(M, K, sparsity, skew, seed=3)
    A1, A2 = spmm.HeteroSparse_Decompose(A)
    packed = spmm.HeteroSparse_PackA1(A1)
    words, offs, longest = spmm.HeteroSparse_PackA2(A2)
    lengths = np.diff(offs)
    assert longest > 64 * spmm.HETERO_FUSED_PIPELINED_ROUNDS and longest <= spmm.HETERO_FUSED_MAX_LIST
    assert (lengths <= 64 * spmm.HETERO_FUSED_PIPELINED_ROUNDS).any() or not skew  # short and long lists side by side
    B = spmm.synth_activations(N, K, seed=5)
    ref = oracle.gemm_f32(A, B)
    for split_k in (1, 3):
        col = run_fused(spmm, packed, words, offs, longest, B, M, N, K, split_k)
        assert_close(col, ref)
        row = run_fused_row_major(spmm, packed, words, offs, longest, B, M, N, K, split_k)
        assert np.array_equal(row.view(np.uint16), col.view(np.uint16))
    # every element of the weight, whichever part and whichever round of its list holds it
    ints = np.where(A != 0, (np.arange(M * K).reshape(M, K) % 1999 + 1).astype(np.float16), np.float16(0))
    I1, I2 = oracle.decompose(ints)
    p1 = spmm.HeteroSparse_PackA1(I1)
    w2, o2, l2 = spmm.HeteroSparse_PackA2(I2)
    rng = np.random.default_rng(N)
    ks = rng.permutation(K)[:N]
    onehot = np.zeros((N, K), dtype=np.float16)
    onehot[np.arange(N), ks] = 1.0
    C = run_fused(spmm, p1, w2, o2, l2, onehot, M, N, K, 1)
    assert np.array_equal(C.view(np.uint16), ints[:, ks].T.view(np.uint16))


def test_fused_full_size_sampled_rows(spmm, oracle):
    """OPT-30B FFN1 at 60 % sparsity, N = 16 and 64: sampled rows against the oracle, the whole
    result against the two-kernel path (same products, other summation order), and linearity."""
    M, K = 28672, 7168
    A = spmm.synth_weights(M, K, 0.6, False, seed=22)
    A1, A2 = spmm.HeteroSparse_Decompose(A)
    packed = spmm.HeteroSparse_PackA1(A1)
    words, offs, longest = spmm.HeteroSparse_PackA2(A2)
    items, offsets = spmm.InitSparseMatrixA_API(A2)
    rows = np.sort(np.random.default_rng(0).choice(M, 384, replace=False))
    Asub = np.ascontiguousarray(A[rows])
    for N in (16, 64):
        B1 = spmm.synth_activations(N, K, seed=1)
        B2 = spmm.synth_activations(N, K, seed=2)
        s = spmm.HeteroSparse_SuggestSplitK(M, N, K)
        C1 = run_fused(spmm, packed, words, offs, longest, B1, M, N, K, s)
        assert_close(C1[:, rows], oracle.gemm_f32(Asub, B1))
        two = run_hybrid(spmm, packed, items, offsets, B1, M, N, K, s, spmm.SpMM_SuggestSplitK(M, N, K))
        assert np.isfinite(C1).all()
        diff = np.abs(C1.astype(np.float32) - two.astype(np.float32))
        assert (diff <= 2e-2 + 2e-2 * np.abs(two.astype(np.float32))).all()
        Bs = (B1.astype(np.float32) * 0.5 + B2.astype(np.float32) * 0.5).astype(np.float16)
        exact = np.array_equal(Bs.astype(np.float32), B1.astype(np.float32) * 0.5 + B2.astype(np.float32) * 0.5)
        C2 = run_fused(spmm, packed, words, offs, longest, B2, M, N, K, s)
        Cs = run_fused(spmm, packed, words, offs, longest, Bs, M, N, K, s)
        lin = 0.5 * C1.astype(np.float32) + 0.5 * C2.astype(np.float32)
        tol = 2e-2 if exact else 4e-2
        assert (np.abs(Cs.astype(np.float32) - lin) <= tol + tol * np.abs(lin)).all()


def test_fused_hip_graph_replays_match_eager(spmm, oracle):
    torch = _torch()
    M, K, N = 1024, 1024, 16
    A = spmm.synth_weights(M, K, 0.6, False, seed=33)
    A1, A2 = spmm.HeteroSparse_Decompose(A)
    d_p = _dev(spmm.HeteroSparse_PackA1(A1))
    words, offs, longest = spmm.HeteroSparse_PackA2(A2)
    d_w, d_o = _dev(words), _dev(offs)
    Bh = spmm.synth_activations(N, K, seed=34)
    d_B = _dev(Bh)
    d_C = torch.zeros((N, M), dtype=torch.float16, device="cuda:0")
    d_W = torch.zeros((2, N, M), dtype=torch.float16, device="cuda:0")

    def call(stream):
        spmm.HeteroSparse_Fused_SpMM_API(stream, d_p, d_w, d_o, longest, d_B, d_C, M, N, K, d_W, 2)

    print("[gpu case] graph capture of the one-launch 2:4 + residual call", flush=True)
    call(torch.cuda.current_stream())
    torch.cuda.synchronize()
    want = d_C.clone()
    assert_close(want.cpu().numpy(), oracle.gemm_f32(A, Bh))
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            call(torch.cuda.current_stream())
    torch.cuda.synchronize()
    for rep in range(3):
        d_C.zero_()
        d_W.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(d_C, want), f"replay {rep} differs from the eager result"
        d_C.zero_()
        call(torch.cuda.current_stream())
        torch.cuda.synchronize()
        assert torch.equal(d_C, want)


@pytest.mark.parametrize("M,K,sparsity,skew", [(128, 128, 0.5, False), (256, 640, 0.45, False), (1024, 2048, 0.7, False),
                                               (128, 128, 1.0, False), (384, 256, 0.0, False), (512, 512, 0.5, True),
                                               (256, 128, 0.97, False)])
def test_device_residual_lists_equal_host(spmm, oracle, M, K, sparsity, skew):
    """The GPU's residual lists against the host's, bit for bit (words, offsets, longest list, the 64
    words of padding), with -0, NaN, denormal and infinity patterns, lists of one round (left as
    collected), of several (ordered by bank) and of the maximum length (a dense matrix: 1024)."""
    torch = _torch()
    A = spmm.synth_weights(M, K, sparsity, skew, seed=M + K + 7)
    A.view(np.uint16)[0, :8] = [0x8000, 0x7E00, 0x0001, 0x3C00, 0xFC00, 0x8001, 0, 0x7C00]
    A.view(np.uint16)[17, 4:8] = [0x7E00, 0x8000, 0xFE00, 0x0001]
    _, A2 = oracle.decompose(A)
    want_words, want_offs, want_longest = spmm.HeteroSparse_PackA2(A2)
    d_A2 = torch.from_numpy(A2.view(np.int16).copy()).to("cuda:0").view(torch.float16)
    print(f"[gpu case] device residual lists M={M} K={K} sparsity={sparsity} skew={skew}", flush=True)
    words, offs, longest = spmm.pack_residual_on_device(d_A2)
    torch.cuda.synchronize()
    assert longest == want_longest
    assert np.array_equal(offs.cpu().numpy(), want_offs)
    assert np.array_equal(words.cpu().numpy().view(np.uint32), want_words)
    # and from the GPU's own split, through the one-launch product
    d_A = torch.from_numpy(A.view(np.int16).copy()).to("cuda:0").view(torch.float16)
    packed, residual = spmm.split_pack_on_device(d_A)
    words2, offs2, longest2 = spmm.pack_residual_on_device(residual)
    assert torch.equal(words2, words) and torch.equal(offs2, offs) and longest2 == longest
    if longest <= spmm.HETERO_FUSED_MAX_LIST:
        N = 16
        Bh = spmm.synth_activations(N, K, seed=3)
        d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device="cuda:0")
        spmm.HeteroSparse_Fused_SpMM_API(torch.cuda.current_stream(), packed, words2, offs2, longest2, _dev(Bh), d_C, M, N, K,
                                         None, 1)
        torch.cuda.synchronize()
        rows = np.isfinite(A).all(axis=1)  # the product is NaN in the rows that hold NaN or infinity: compare the others
        assert_close(d_C.cpu().numpy()[:, rows], oracle.gemm_f32(np.ascontiguousarray(A[rows]), Bh))


@pytest.mark.parametrize("split_k", [1, 3])
def test_fused_strided_operands_and_clamp(spmm, oracle, split_k):
    """Token strides wider than the vectors, ReLU in the launch (one batch) or in the reduction
    (three), and the bytes of C outside the result untouched."""
    torch = _torch()
    M, K, N, ldb, ldc = 384, 768, 16, 768 + 64, 384 + 128
    A = spmm.synth_weights(M, K, 0.6, False, seed=61)
    A1, A2 = spmm.HeteroSparse_Decompose(A)
    words, offs, longest = spmm.HeteroSparse_PackA2(A2)
    Bh = spmm.synth_activations(N, K, seed=62)
    wide = np.full((N, ldb), np.float16(7.0))
    wide[:, :K] = Bh
    d_B = _dev(wide)
    d_C = torch.full((N, ldc), -3.0, dtype=torch.float16, device="cuda:0")
    d_W = torch.zeros((split_k, N, M), dtype=torch.float16, device="cuda:0")
    print(f"[gpu case] fused strided M={M} N={N} K={K} ldb={ldb} ldc={ldc} split_k={split_k} relu", flush=True)
    spmm.HeteroSparse_Fused_SpMM_API_Strided(torch.cuda.current_stream(), _dev(spmm.HeteroSparse_PackA1(A1)), _dev(words), _dev(offs),
                                             longest, d_B, ldb, d_C, ldc, M, N, K, d_W, split_k, spmm.SPMM_FLAG_RELU)
    torch.cuda.synchronize()
    C = d_C.cpu().numpy()
    ref = oracle.gemm_f32(A, Bh)
    assert (ref < -0.1).any()
    assert_close(C[:, :M], np.maximum(ref, 0.0))
    assert (C[:, :M] >= 0).all() and (C[:, M:] == np.float16(-3.0)).all()
    d = torch.zeros(1 << 12, dtype=torch.int32, device="cuda:0")
    for ldb_bad, ldc_bad in ((K - 8, ldc), (ldb, M - 8), (K + 4, ldc), (ldb, M + 4)):
        with pytest.raises(spmm.SpMMError):
            spmm.HeteroSparse_Fused_SpMM_API_Strided(None, d, d, d, 10, d, ldb_bad, d, ldc_bad, M, N, K, d, 1, 0)


@pytest.mark.parametrize("row_major", [False, True])
def test_split_decoder_stack_matches_cpu_chain(spmm, oracle, row_major):
    """Three chained blocks with every weight split into 2:4 records + residual lists on the GPU,
    each product one launch, against the same chain on the CPU; and replays of the captured chain.
    row_major: every buffer [features][tokens], products through HeteroSparse_Fused_SpMM_API_RowMajor."""
    torch = _torch()
    from graphneuralnetproj_amd import decoder_stack as DS

    dev = torch.device("cuda:0")
    h, N, nlayers = 512, 16, 3
    layers, dense = [], []
    for i in range(nlayers):
        L, samples = DS.build_split_layer_on_device(spmm, torch, dev, h, N, 0.6, seed=50 + i, weight_std=0.08, sample_rows=4 * h)
        layers.append(L)
        d = {}
        for name, (M, K) in DS.layer_shapes(h).items():
            rows, vals = samples[name]
            assert rows.size == M  # every row: the whole matrix comes back, in row order
            d[name] = vals
        dense.append(d)
    stack = DS.Stack(spmm, torch, layers, h, N, row_major=row_major)
    x0 = spmm.synth_activations(N, h, seed=98)
    x0_d = torch.from_numpy(x0.view(np.int16)).to(dev).view(torch.float16)
    if row_major:
        x0_d = x0_d.t().contiguous()
    stack.x[0].copy_(x0_d)
    print(f"[gpu case] split decoder stack h={h} N={N} layers={nlayers} row_major={row_major}", flush=True)
    out = stack.step(torch.cuda.current_stream())
    torch.cuda.synchronize()
    got = out.clone()
    x = x0
    f16 = lambda a: a.astype(np.float16)
    for d in dense:
        qkv = f16(oracle.gemm_f32(d["qkv"], x))
        o = f16(oracle.gemm_f32(d["out"], np.ascontiguousarray(qkv[:, :h])))
        f = f16(np.maximum(oracle.gemm_f32(d["ffn1"], o), 0.0))
        x = f16(oracle.gemm_f32(d["ffn2"], f))
    xr = x.astype(np.float32)
    assert np.abs(xr).max() > 1e-3, "the reference chain must not have collapsed to zero"
    got_h = (got.t() if row_major else got).cpu().numpy().astype(np.float32)
    err = np.abs(got_h - xr)
    scale = np.maximum(np.abs(xr), np.sqrt(np.mean(xr * xr)))
    assert (err <= 3 * (ATOL + RTOL * scale)).all(), err.max()  # twelve products, fp16 between them
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        stack.x[0].copy_(x0_d)
        with torch.cuda.graph(g, stream=side):
            out_g = stack.step(torch.cuda.current_stream())
    torch.cuda.synchronize()
    for rep in range(3):
        stack.x[0].copy_(x0_d)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, got), f"replay {rep} differs from the eager result"


def test_device_residual_lists_refuse_what_is_no_residual(spmm):
    """A dense matrix has 2048 kept values per 16 x 128 block, twice what a residual can hold: the
    offsets step reports it, the Python wrapper raises, and the words step writes nothing for such blocks."""
    torch = _torch()
    M, K = 128, 256
    A = torch.ones((M, K), dtype=torch.float16, device="cuda:0")
    with pytest.raises(spmm.SpMMError):
        spmm.pack_residual_on_device(A)
    lib = spmm.load_library()
    import ctypes

    lists = (M // 16) * (K // 128)
    offsets = torch.zeros(lists + 2, dtype=torch.int32, device="cuda:0")
    words = torch.full((lists * 2048 + 64,), 7, dtype=torch.int32, device="cuda:0")
    print("[gpu case] device residual lists on a dense matrix", flush=True)
    rc = lib.HeteroSparse_DevicePackA2_Offsets(None, ctypes.c_void_p(A.data_ptr()), M, K, ctypes.c_void_p(offsets.data_ptr()),
                                               ctypes.c_void_p(offsets.data_ptr() + 4 * (lists + 1)))
    assert rc == 0
    rc = lib.HeteroSparse_DevicePackA2_Words(None, ctypes.c_void_p(A.data_ptr()), M, K, ctypes.c_void_p(offsets.data_ptr()),
                                             ctypes.c_void_p(words.data_ptr()))
    assert rc == 0
    torch.cuda.synchronize()
    o = offsets.cpu().numpy()
    assert o[lists] == lists * 2048 and o[lists + 1] == 2048
    w = words.cpu().numpy()
    assert (w[:lists * 2048] == 7).all() and (w[lists * 2048:] == 0).all()  # only the padding was written


@pytest.mark.parametrize("M,K,N,split_k", [(512, 1152, 16, 3), (384, 1152, 8, 2), (1024, 2048, 32, 4), (512, 1024, 64, 2),
                                           (7168, 7168, 16, 4)])
def test_fused_call_sums_its_slabs_in_the_launch_bit_for_bit(spmm, oracle, M, K, N, split_k):
    """More than one batch: the 2:4 kernel's own sum of its slabs (the last workgroup of a group of rows)
    and the reduction kernel give the same bits, with and without the clamp, on repeated calls; and
    the call without a residual (HeteroSparse_SpMM_API on a 2:4 weight) goes the same way."""
    torch = _torch()
    A = spmm.synth_weights(M, K, 0.6, False, seed=M + K + N)
    A1, A2 = spmm.HeteroSparse_Decompose(A)
    words, offs, longest = spmm.HeteroSparse_PackA2(A2)
    d_p, d_w, d_o = _dev(spmm.HeteroSparse_PackA1(A1)), _dev(words), _dev(offs)
    Bh = spmm.synth_activations(N, K, seed=63)
    d_B = _dev(Bh)
    outs = []
    for flags in (0, spmm.SPMM_FLAG_SEPARATE_REDUCTION, spmm.SPMM_FLAG_RELU, spmm.SPMM_FLAG_RELU | spmm.SPMM_FLAG_SEPARATE_REDUCTION):
        d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device="cuda:0")
        d_W = torch.full((split_k, N, M), float("nan"), dtype=torch.float16, device="cuda:0")
        print(f"[gpu case] one launch, slabs summed in the launch or not: M={M} N={N} K={K} split_k={split_k} flags={flags}", flush=True)
        for _ in range(3):  # the arrival counters must come back to zero every time
            spmm.HeteroSparse_Fused_SpMM_API_Strided(torch.cuda.current_stream(), d_p, d_w, d_o, longest, d_B, K, d_C, M, M, N, K,
                                                     d_W, split_k, flags)
        torch.cuda.synchronize()
        outs.append(d_C.cpu().numpy())
    assert np.array_equal(outs[0].view(np.uint16), outs[1].view(np.uint16))
    assert np.array_equal(outs[2].view(np.uint16), outs[3].view(np.uint16))
    if M * K <= 4 * 1024 * 1024:
        ref = oracle.gemm_f32(A, Bh)
        assert_close(outs[0], ref)
        assert_close(outs[2], np.maximum(ref, 0.0))
        C1 = run_hybrid(spmm, spmm.HeteroSparse_PackA1(A1), None, None, Bh, M, N, K, split_k, 0)
        assert_close(C1, oracle.gemm_f32(A1, Bh))



# ---------------------------------------------------------------------------------------------
# row-major operands (B[K][N], C[M][N]): this fork's own layout, csrc/SpMM_Kernel.cuh:372-374,731-734


def run_fused_row_major(spmm, packed, words, offs, longest, B, M, N, K, split_k, flags=0):
    """B is the usual [N][K] host array; the call gets its transpose and the result comes back as [N][M]."""
    torch = _torch()
    d_p, d_w, d_o = _dev(packed), _dev(words), _dev(offs)
    d_Bt = _dev(B).view(torch.float16).t().contiguous()
    d_Ct = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda:0")
    d_W = torch.full((max(split_k, 1), M, N), float("nan"), dtype=torch.float16, device="cuda:0")
    print(f"[gpu case] fused row-major M={M} N={N} K={K} split_k={split_k} longest={longest} flags={flags}", flush=True)
    spmm.HeteroSparse_Fused_SpMM_API_RowMajor(torch.cuda.current_stream(), d_p, d_w, d_o, longest, d_Bt, d_Ct, M, N, K, d_W,
                                              split_k, flags)
    torch.cuda.synchronize()
    return d_Ct.t().contiguous().cpu().numpy()


def run_hybrid_row_major(spmm, packed, items, offsets, B, M, N, K, s1, s2, flags=0):
    torch = _torch()
    d_p = _dev(packed)
    d_items = _dev(items) if items is not None else None
    d_offs = _dev(offsets) if offsets is not None else None
    d_Bt = _dev(B).view(torch.float16).t().contiguous()
    d_Ct = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda:0")
    d_W = torch.full((s1 + s2, M, N), float("nan"), dtype=torch.float16, device="cuda:0")
    print(f"[gpu case] hybrid row-major M={M} N={N} K={K} split_k={s1}/{s2} flags={flags}", flush=True)
    spmm.HeteroSparse_SpMM_API_RowMajor(torch.cuda.current_stream(), d_p, d_items, d_offs, d_Bt, d_Ct, M, N, K, d_W, s1, s2, flags)
    torch.cuda.synchronize()
    return d_Ct.t().contiguous().cpu().numpy()


@pytest.mark.parametrize("N", [8, 16, 32, 64])
def test_row_major_layout_one_hot(spmm, oracle, N):
    """Rows, columns and tokens of the row-major entries, through both parts: distinct exactly
    representable integers and one-hot activations, so C[m][n] must equal A[m][k_n] exactly (the
    staging of the K x N block, the transposing reads and the M x N stores all have to be right)."""
    M, K = 256, 384
    rng = np.random.default_rng(40 + N)
    A = np.zeros((M, K), dtype=np.float16)
    mask = rng.random((M, K)) < 0.45
    vals = (np.arange(M * K).reshape(M, K) % 1999 + 1).astype(np.float16)
    A[mask] = vals[mask]
    A1, A2 = oracle.decompose(A)
    packed = spmm.HeteroSparse_PackA1(A1)
    words, offs, longest = spmm.HeteroSparse_PackA2(A2)
    items, offsets = spmm.InitSparseMatrixA_API(A2)
    for trial in range(3):
        ks = rng.permutation(K)[:N]
        B = np.zeros((N, K), dtype=np.float16)
        B[np.arange(N), ks] = 1.0
        want = A[:, ks].T.view(np.uint16)
        for split_k in (1, 3):
            C = run_fused_row_major(spmm, packed, words, offs, longest, B, M, N, K, split_k)
            assert np.array_equal(C.view(np.uint16), want), (trial, split_k)
        C = run_hybrid_row_major(spmm, packed, items, offsets, B, M, N, K, 1, 2)
        assert np.array_equal(C.view(np.uint16), want), trial
        C = run_hybrid_row_major(spmm, packed, None, None, B, M, N, K, 3, 0)   # the 2:4 part alone, three batches
        assert np.array_equal(C.view(np.uint16), A1[:, ks].T.view(np.uint16)), trial
        C = run_hybrid_row_major(spmm, packed, None, None, B, M, N, K, 1, 0)   # ... and one
        assert np.array_equal(C.view(np.uint16), A1[:, ks].T.view(np.uint16)), trial


@pytest.mark.parametrize("sparsity", [0.45, 0.6, 0.8, 0.95])
@pytest.mark.parametrize("N", [8, 16, 32, 64])
@pytest.mark.parametrize("M,K,split_k", [(384, 1152, 1), (512, 1024, 2), (2048, 640, 5)])
def test_row_major_fused_equals_column_major_bit_for_bit(spmm, oracle, sparsity, N, M, K, split_k):
    """The one-launch call in both layouts: every element takes the same products in the same order
    (units, steps and the order of the two parts do not depend on the layout), so the results are
    the same bits, with and without the clamp and the in-launch sum; and they match the oracle."""
    A = spmm.synth_weights(M, K, sparsity, False, seed=M + K + N)
    A1, A2 = spmm.HeteroSparse_Decompose(A)
    packed = spmm.HeteroSparse_PackA1(A1)
    words, offs, longest = spmm.HeteroSparse_PackA2(A2)
    B = spmm.synth_activations(N, K, seed=71)
    col = run_fused(spmm, packed, words, offs, longest, B, M, N, K, split_k)
    assert_close(col, oracle.gemm_f32(A, B))
    for flags in (0, spmm.SPMM_FLAG_SEPARATE_REDUCTION):
        row = run_fused_row_major(spmm, packed, words, offs, longest, B, M, N, K, split_k, flags)
        assert np.array_equal(row.view(np.uint16), col.view(np.uint16)), flags
    row = run_fused_row_major(spmm, packed, words, offs, longest, B, M, N, K, split_k, spmm.SPMM_FLAG_RELU)
    assert np.array_equal(row, np.maximum(col, np.float16(0)))


@pytest.mark.parametrize("sparsity", [0.5, 0.7])
@pytest.mark.parametrize("N", [8, 16, 64])
def test_row_major_hybrid_vs_oracle(spmm, oracle, sparsity, N):
    """The two-kernel call in the row-major layout (the residual on the Tiled-CSL kernel's row-major
    form, which adds all slabs up, the 2:4 part's included), one and two streams."""
    M, K = 1024, 2048
    A = spmm.synth_weights(M, K, sparsity, False, seed=81 + N)
    A1, A2 = spmm.HeteroSparse_Decompose(A)
    packed = spmm.HeteroSparse_PackA1(A1)
    items, offsets = spmm.InitSparseMatrixA_API(A2)
    B = spmm.synth_activations(N, K, seed=82)
    ref = oracle.gemm_f32(A, B)
    for s1, s2, flags in ((1, 1, 0), (2, 4, 0), (4, 3, 0), (2, 2, spmm.HETERO_FLAG_TWO_STREAMS)):
        assert_close(run_hybrid_row_major(spmm, packed, items, offsets, B, M, N, K, s1, s2, flags), ref)


def test_row_major_full_size_and_rejects(spmm, oracle):
    """OPT-30B FFN1 at 60 %, N = 16 and 64, the one-launch call in the row-major layout at full size:
    the same bits as the column-major call.  And what the entry refuses."""
    torch = _torch()
    M, K = 28672, 7168
    A = spmm.synth_weights(M, K, 0.6, False, seed=23)
    A1, A2 = spmm.HeteroSparse_Decompose(A)
    packed = spmm.HeteroSparse_PackA1(A1)
    words, offs, longest = spmm.HeteroSparse_PackA2(A2)
    for N in (16, 64):
        B = spmm.synth_activations(N, K, seed=3)
        s = spmm.HeteroSparse_SuggestSplitK(M, N, K)
        col = run_fused(spmm, packed, words, offs, longest, B, M, N, K, s)
        row = run_fused_row_major(spmm, packed, words, offs, longest, B, M, N, K, s)
        assert np.array_equal(row.view(np.uint16), col.view(np.uint16))
    d = torch.zeros(64, dtype=torch.int32, device="cuda:0")
    for bad in (dict(M=200), dict(K=576), dict(N=24), dict(flags=8)):
        a = dict(M=256, K=512, N=16, flags=0)
        a.update(bad)
        with pytest.raises(spmm.SpMMError):
            spmm.HeteroSparse_Fused_SpMM_API_RowMajor(torch.cuda.current_stream(), d, d, d, 10, d, d, a["M"], a["N"], a["K"], d, 1,
                                                      a["flags"])


def test_fused_row_skewed_weight_full_size(spmm, oracle):
    """OPT-30B FFN1 with Beta(2, 8) row densities at 60 % sparsity, N = 16, through the one-launch call:
    some blocks' lists exceed what travels with the records.  The rows of the blocks with the longest
    lists and random rows against the oracle, every row against the two-kernel call."""
    M, K, N = 28672, 7168, 16
    A = spmm.synth_weights(M, K, 0.6, True, seed=29)
    A1, A2 = spmm.HeteroSparse_Decompose(A)
    packed = spmm.HeteroSparse_PackA1(A1)
    words, offs, longest = spmm.HeteroSparse_PackA2(A2)
    assert 64 * spmm.HETERO_FUSED_PIPELINED_ROUNDS < longest <= spmm.HETERO_FUSED_MAX_LIST
    units = K // 128
    lengths = np.diff(offs).reshape(M // 128, units, 8)  # lists are numbered by group of eight row blocks, unit, block
    per_block = lengths.max(axis=1).reshape(-1)           # the longest list of every 16-row block
    blocks = np.argsort(per_block)[-6:]
    rows = np.unique(np.concatenate([np.arange(16 * b, 16 * b + 16) for b in blocks]
                                    + [np.random.default_rng(1).choice(M, 160, replace=False)]))
    B = spmm.synth_activations(N, K, seed=30)
    s = spmm.HeteroSparse_SuggestSplitK(M, N, K)
    C = run_fused(spmm, packed, words, offs, longest, B, M, N, K, s)
    assert_close(C[:, rows], oracle.gemm_f32(np.ascontiguousarray(A[rows]), B))
    items, offsets = spmm.InitSparseMatrixA_API(A2)
    two = run_hybrid(spmm, packed, items, offsets, B, M, N, K, s, spmm.SpMM_SuggestSplitK(M, N, K))
    diff = np.abs(C.astype(np.float32) - two.astype(np.float32))
    assert np.isfinite(C).all() and (diff <= 2e-2 + 2e-2 * np.abs(two.astype(np.float32))).all()
