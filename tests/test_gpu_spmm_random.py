"""Seeded random shapes, launch shapes and flags through the Tiled-CSL entry points, every element
bit for bit.

Data: the value pattern of the reference's harness (kernel_benchmark/spmm_test_utils.h:111-141: kept
weights exactly 1.0, activations in {-5, -3, -1, 1, 3}); cases whose sums leave +-2048 are redrawn,
so every partial sum and every fp16 slab entry is an exact integer and the expected result is numpy's
float32 product of integers, whatever the split (csrc/SpMM_Kernel.cuh:312-320), the layout of the
launch or the order of summation.  Per case the draw picks M, K, the token count, the sparsity (0 to
99 %, Bernoulli or Beta(2,8) row densities, so tiles from empty to full and of one, two or three
segments), Split_K, and a launch shape of SpMM_SplitK_API_Planned (K-splitting or row-sharing
workgroups of 1 to 8 waves, the activation slice staged, shared tile by tile or read as fragments,
either operand layout, ReLU, the separate reduction kernel, density-dependent wave counts); the
same product then goes through SpMM_SplitK_API, its row-major, strided and static-workspace forms
with the library's own plan.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

CASES = 96
LDS_PER_CU = 160 * 1024
TILE_LDS = 16 * 1024


def _dev(torch, a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        return torch.from_numpy(a.view(np.int16)).to("cuda:0").view(torch.float16)
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).to("cuda:0")
    return torch.from_numpy(a).to("cuda:0")


def _fits(N, K, split_k, mode, waves, stage_b, row_major):
    """The launch shapes SpMM_SplitK_API_Planned accepts (the library's own rule, restated)."""
    if waves > (4 if N == 64 else 8):
        return False
    tiles = (K // 64 - 1) // split_k + 1
    lds = waves * TILE_LDS
    if row_major:
        if stage_b:
            return False
        lds += waves * N * 128
    if mode == 0:
        if stage_b == 1:
            if N > 16:
                return False
            lds += tiles * (8 if N == 8 else 16) * 128
        elif stage_b == 2:
            if not ((N == 32 and waves in (4, 8)) or (N == 64 and waves == 4)):
                return False
            lds += 2 * N * 128
    else:
        if stage_b:
            return False
        lds = max(lds, 8 * waves * (1 if N <= 16 else N // 16) * 1024)
    return lds <= LDS_PER_CU


def test_random_shapes_launch_shapes_and_flags_exact(spmm):
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    G = spmm
    st = torch.cuda.current_stream()
    rng = np.random.default_rng(77031)
    seen = set()
    nan = float("nan")
    for case in range(CASES):
        while True:
            M = int(rng.integers(1, 13)) * 128
            K = int(rng.integers(1, 41)) * 64
            N = int(rng.choice([8, 16, 32, 64]))
            sp = float(rng.choice([0.0, 0.2, 0.5, 0.7, 0.8, 0.9, 0.95, 0.99]))
            skew = bool(rng.integers(0, 2)) and 0.2 <= sp
            A = G.synth_harness_weights(M, K, sp, skew, seed=5 * case + 1)
            B = G.synth_harness_activations(N, K, seed=5 * case + 2)
            ref = (A.astype(np.float32) @ B.astype(np.float32).T).T  # [N][M]
            if np.abs(ref).max() <= 2048:
                break
        ref16 = ref.astype(np.float16)
        nkb = K // 64
        split_k = int(rng.integers(1, min(nkb, 9) + 1))
        while (-(-nkb // split_k)) * (split_k - 1) >= nkb:  # no empty batch
            split_k -= 1
        while True:
            mode, waves = int(rng.integers(0, 2)), int(rng.integers(1, 9))
            stage_b, row_major = int(rng.integers(0, 3)), int(rng.integers(0, 2))
            if _fits(N, K, split_k, mode, waves, stage_b, row_major):
                break
        flags = int(rng.integers(0, 8))
        relu = flags & G.SPMM_FLAG_RELU
        want = np.maximum(ref16, 0) if relu else ref16
        seen.add((mode, stage_b, row_major))
        what = (f"case {case}: M={M} K={K} N={N} sparsity={sp} skew={skew} Split_K={split_k} mode={mode} waves={waves} "
                f"stage_b={stage_b} row_major={row_major} flags={flags}")
        print(what, flush=True)
        items, offsets = G.InitSparseMatrixA_API(A)
        d_items, d_offsets = _dev(torch, items), _dev(torch, offsets)
        dB, dBt = _dev(torch, B), _dev(torch, np.ascontiguousarray(B.T))

        def fresh(rm):
            shape = (M, N) if rm else (N, M)
            return (torch.full(shape, nan, dtype=torch.float16, device="cuda:0"),
                    torch.full((split_k,) + shape, nan, dtype=torch.float16, device="cuda:0"))

        C, W = fresh(row_major)
        G.SpMM_SplitK_API_Planned(st, d_items, d_offsets, dBt if row_major else dB, C, M, N, K, W, split_k, mode, waves,
                                  stage_b, row_major, flags)
        got = C.cpu().numpy()
        assert np.array_equal(got.T if row_major else got, want), "chosen launch shape, " + what
        C, W = fresh(0)
        G.SpMM_SplitK_API(st, None, d_items, d_offsets, dB, C, M, N, K, W, split_k)
        assert np.array_equal(C.cpu().numpy(), ref16), "SpMM_SplitK_API, " + what
        C, W = fresh(1)
        G.SpMM_SplitK_API_RowMajor_Flags(st, d_items, d_offsets, dBt, C, M, N, K, W, split_k, flags & 3)
        assert np.array_equal(C.cpu().numpy().T, want), "row-major entry, " + what
        ldb, ldc = K + 64 * int(rng.integers(0, 3)), M + 8 * int(rng.integers(0, 3))
        Bp = np.zeros((N, ldb), dtype=np.float16)
        Bp[:, :K] = B
        C = torch.full((N, ldc), nan, dtype=torch.float16, device="cuda:0")
        _, W = fresh(0)
        G.SpMM_SplitK_API_Strided(st, d_items, d_offsets, _dev(torch, Bp), ldb, C, ldc, M, N, K, W, split_k, flags & 3)
        out = C.cpu().numpy()
        assert np.array_equal(out[:, :M], want), "strided entry, " + what
        assert np.isnan(out[:, M:]).all(), "strided entry wrote between the token vectors, " + what
        C, _ = fresh(0)
        G.SpMM_SplitK_API_StaticWorkspace(st, None, d_items, d_offsets, dB, C, M, N, K, split_k)
        assert np.array_equal(C.cpu().numpy(), ref16), "static workspace, " + what
    # every layout of the launch was drawn at least once
    assert {(1, 0, 0), (1, 0, 1), (0, 0, 0), (0, 0, 1), (0, 1, 0), (0, 2, 0)} <= seen, seen
