"""The GPU Tiled-CSL encoder must produce the host encoder's bits (which equal the reference's)."""
import time

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _torch():
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch


def _compare(spmm, A):
    torch = _torch()
    items, offsets = spmm.InitSparseMatrixA_API(A)
    d_A = torch.from_numpy(np.ascontiguousarray(A).view(np.int16).copy()).cuda().view(torch.float16)
    print(f"[gpu case] device encode {A.shape}", flush=True)
    d_items, d_offsets = spmm.encode_on_device(d_A)
    torch.cuda.synchronize()
    assert np.array_equal(d_offsets.cpu().numpy(), offsets)
    assert np.array_equal(d_items.cpu().numpy().view(np.uint32), items)
    return d_items, d_offsets


@pytest.mark.parametrize("M,K,sparsity,skew", [
    (128, 64, 0.8, False), (256, 192, 0.5, False), (1024, 1024, 0.8, False), (1024, 1024, 0.9, True),
    (512, 512, 0.0, False), (512, 512, 0.999, False), (384, 64 * 5, 0.3, True),
])
def test_device_encoder_matches_host(spmm, M, K, sparsity, skew):
    _compare(spmm, spmm.synth_weights(M, K, sparsity, skew, seed=M + K))


def test_device_encoder_special_tiles(spmm):
    """All-zero tiles, a fully dense tile, single elements, and the values the reference treats specially."""
    rng = np.random.default_rng(7)
    A = np.zeros((512, 256), dtype=np.float16)
    A[0:128, 0:64] = rng.standard_normal((128, 64)).astype(np.float16) + np.float16(3)  # dense tile (no zeros)
    A[128 + 5, 64 + 9] = 1.5                               # a single element: three pads
    A[256:384, 128:192][::7, ::5] = -2.0                   # regular pattern
    bits = A.view(np.uint16)
    bits[384 + 1, 192 + 1] = 0x8000                        # -0: dropped
    bits[384 + 2, 192 + 2] = 0x7e00                        # NaN: dropped (fabs(NaN) > 0 is false)
    bits[384 + 3, 192 + 3] = 0x7c00                        # +inf: kept
    bits[384 + 4, 192 + 4] = 0x0001                        # smallest subnormal: kept
    bits[384 + 5, 192 + 5] = 0xfc00                        # -inf: kept
    _compare(spmm, A)


def test_device_encoded_weight_feeds_the_product(spmm, oracle):
    torch = _torch()
    M, K, N = 512, 1024, 16
    A = spmm.synth_weights(M, K, 0.8, False, seed=5)
    B = spmm.synth_activations(N, K, seed=6)
    d_items, d_offsets = _compare(spmm, A)
    d_B = torch.from_numpy(B.view(np.int16).copy()).cuda()
    d_C = torch.full((N, M), float("nan"), dtype=torch.float16, device="cuda")
    spmm.SpMM_SplitK_API(None, None, d_items, d_offsets, d_B, d_C, M, N, K, None, 1)
    torch.cuda.synchronize()
    ref = oracle.gemm_f32(A, B)
    err = np.abs(d_C.cpu().numpy().astype(np.float32) - ref)
    assert (err <= 1e-2 + 1e-2 * np.abs(ref)).all()


def test_device_encoder_full_size(spmm):
    """OPT-30B FFN1: bit equality on 25088 tiles, and the time of the two device passes."""
    torch = _torch()
    M, K = 28672, 7168
    A = spmm.synth_weights(M, K, 0.8, False, seed=1234)
    t0 = time.perf_counter()
    items, offsets = spmm.InitSparseMatrixA_API(A)
    t_host = time.perf_counter() - t0
    d_A = torch.from_numpy(A.view(np.int16)).cuda().view(torch.float16)
    spmm.encode_on_device(d_A)  # warm up
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    d_items, d_offsets = spmm.encode_on_device(d_A)
    torch.cuda.synchronize()
    t_dev = time.perf_counter() - t0
    print(f"[gpu case] full-size encode: host {t_host * 1e3:.1f} ms, device {t_dev * 1e3:.2f} ms", flush=True)
    assert np.array_equal(d_offsets.cpu().numpy(), offsets)
    assert np.array_equal(d_items.cpu().numpy().view(np.uint32), items)


def test_device_encoder_rejects_bad_shapes(spmm):
    torch = _torch()
    z = torch.zeros(1024, dtype=torch.int32, device="cuda")
    lib = spmm.load_library()
    assert lib.SpMM_DeviceEncodeOffsets(None, z.data_ptr(), 100, 64, z.data_ptr()) != 0
    assert lib.SpMM_DeviceEncodeOffsets(None, z.data_ptr(), 128, 60, z.data_ptr()) != 0
    assert lib.SpMM_DeviceEncodeOffsets(None, None, 128, 64, z.data_ptr()) != 0
    assert lib.SpMM_DeviceEncodeItems(None, z.data_ptr(), 128, 64, None, z.data_ptr()) != 0
