"""SpMM_SplitK_API_StaticWorkspace (the entry point that allocates nothing) against SpMM_SplitK_API.

Same bits are required: both run the same kernels, the only difference is where the slabs of
partial sums and the arrival counters live.  Two calls in a row share the static array, the
second with a smaller input, so stale contents of the first must not show."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _torch():
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch


def _operands(spmm, torch, M, K, N, seed):
    dev = torch.device("cuda:0")
    A = spmm.synth_weights(M, K, 0.8, False, seed=seed)
    B = spmm.synth_activations(N, K, seed=seed + 1)
    items, offsets = spmm.InitSparseMatrixA_API(A)
    return (torch.from_numpy(items.view(np.int32).copy()).to(dev), torch.from_numpy(offsets.copy()).to(dev),
            torch.from_numpy(B.view(np.int16).copy()).to(dev))


def _free_bytes(torch):
    return torch.cuda.mem_get_info()[0]


# (M, K, N, Split_K): first a larger call, then a smaller one on the same static array.  7168^2 with
# Split_K 4 takes the K-splitting launch with the in-launch reduction (counters inside the array),
# 16384 x 512 the row-sharing launch with the reduction kernel, Split_K 1 touches no workspace.
SEQUENCES = [
    [(7168, 7168, 16, 4), (1024, 2048, 16, 3)],
    [(16384, 512, 64, 3), (2048, 512, 8, 2)],
    [(4096, 4096, 32, 6), (4096, 4096, 32, 1), (512, 1024, 32, 5)],
]


@pytest.mark.parametrize("sequence", SEQUENCES, ids=["fused", "row-sharing", "mixed"])
def test_static_workspace_matches_caller_workspace(spmm, sequence):
    torch = _torch()
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream()
    cases = []
    for i, (M, K, N, split_k) in enumerate(sequence):
        ops = _operands(spmm, torch, M, K, N, seed=7000 + i)
        want = torch.full((N, M), float("nan"), dtype=torch.float16, device=dev)
        ws = torch.full((split_k, N, M), float("nan"), dtype=torch.float16, device=dev)
        spmm.SpMM_SplitK_API(stream, None, *ops, want, M, N, K, ws, split_k)
        got = torch.full((N, M), float("nan"), dtype=torch.float16, device=dev)
        cases.append((M, K, N, split_k, ops, want, got))
    torch.cuda.synchronize()
    # the calls under test, back to back on one stream, nothing allocated in between
    free_before = _free_bytes(torch)
    for (M, K, N, split_k, ops, want, got) in cases:
        print(f"[gpu case] static workspace M={M} K={K} N={N} split_k={split_k}", flush=True)
        spmm.SpMM_SplitK_API_StaticWorkspace(stream, None, *ops, got, M, N, K, split_k)
    torch.cuda.synchronize()
    assert _free_bytes(torch) == free_before, "device memory changed hands during the calls"
    for (M, K, N, split_k, ops, want, got) in cases:
        assert torch.isfinite(got).all()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (M, K, N, split_k)


def test_static_workspace_refuses_what_does_not_fit(spmm):
    torch = _torch()
    dev = torch.device("cuda:0")
    z = torch.zeros(1024, dtype=torch.int32, device=dev)
    C = torch.full((64, 28672), 5.0, dtype=torch.float16, device=dev)
    with pytest.raises(spmm.SpMMError):   # 64 x 28672 x 64 x 2 bytes = 235 MB of partial sums
        spmm.SpMM_SplitK_API_StaticWorkspace(None, None, z, z, z, C, 28672, 64, 7168, 64)
    with pytest.raises(spmm.SpMMError):   # the usual refusals
        spmm.SpMM_SplitK_API_StaticWorkspace(None, None, z, z, z, C, 28672, 24, 7168, 2)
    with pytest.raises(spmm.SpMMError):
        spmm.SpMM_SplitK_API_StaticWorkspace(None, None, z, z, z, C, 100, 16, 64, 1)
    with pytest.raises(spmm.SpMMError):
        spmm.SpMM_SplitK_API_StaticWorkspace(None, None, z, None, z, C, 128, 16, 64, 2)
    torch.cuda.synchronize()
    assert (C == 5.0).all()
