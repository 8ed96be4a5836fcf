"""The GPU Tiled-CSL encoder must produce the reference's bits: it is compared with the CPU
oracle, with the committed outputs of the reference's own encoder (tests/golden/), and with
the product's host encoder."""
import hashlib
import json
import os
import time

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _torch():
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch


def _encode(spmm, A):
    torch = _torch()
    d_A = torch.from_numpy(np.ascontiguousarray(A).view(np.int16).copy()).cuda().view(torch.float16)
    print(f"[gpu case] device encode {A.shape}", flush=True)
    d_items, d_offsets = spmm.encode_on_device(d_A)
    torch.cuda.synchronize()
    return d_items, d_offsets


def _compare(spmm, oracle, A):
    """Device encoder against the CPU oracle (the checker) and against the product's host encoder."""
    d_items, d_offsets = _encode(spmm, A)
    got_items, got_offsets = d_items.cpu().numpy().view(np.uint32), d_offsets.cpu().numpy()
    o_items, o_offsets = oracle.encode(A)
    assert np.array_equal(got_offsets, o_offsets)
    assert np.array_equal(got_items, o_items)
    items, offsets = spmm.InitSparseMatrixA_API(A)
    assert np.array_equal(got_offsets, offsets)
    assert np.array_equal(got_items, items)
    return d_items, d_offsets


def test_device_encoder_matches_reference_golden_small(spmm):
    """Full arrays written by the reference's own encoder (tests/golden/make_golden.py)."""
    z = np.load(os.path.join(GOLD, "encoder_small.npz"))
    names = sorted({k.rsplit(".", 1)[0] for k in z.files})
    assert len(names) >= 10
    for n in names:
        d_items, d_offsets = _encode(spmm, z[n + ".A"])
        assert np.array_equal(d_offsets.cpu().numpy(), z[n + ".offsets"]), n
        assert np.array_equal(d_items.cpu().numpy().view(np.uint32), z[n + ".items"]), n


def test_device_encoder_matches_reference_golden_large(spmm):
    """SHA-256 of the reference encoder's output on larger seeded matrices."""
    with open(os.path.join(GOLD, "encoder_large.json")) as f:
        cases = json.load(f)
    for c in cases:
        A = spmm.synth_weights(c["M"], c["K"], c["sparsity"], c["row_skewed"], seed=c["seed"])
        assert hashlib.sha256(A.tobytes()).hexdigest() == c["input_sha256"]
        d_items, d_offsets = _encode(spmm, A)
        assert hashlib.sha256(d_items.cpu().numpy().tobytes()).hexdigest() == c["items_sha256"]
        assert hashlib.sha256(d_offsets.cpu().numpy().tobytes()).hexdigest() == c["offsets_sha256"]


def test_device_split_pack_matches_reference_golden(spmm, oracle):
    """The GPU's 2:4 split against the committed outputs of the reference's decompose()
    (tests/golden/decompose_small.npz).  The device entry point takes M % 128 == 0 and K % 128 == 0,
    so each case sits in the top left corner of an otherwise zero matrix of that shape (groups of
    four never cross a row, so the expected parts are the golden ones in the same corner).  The
    records are read back with the oracle's reader of the record layout."""
    torch = _torch()
    z = np.load(os.path.join(GOLD, "decompose_small.npz"))
    names = sorted({k.rsplit(".", 1)[0] for k in z.files})
    assert len(names) >= 7
    for n in names:
        A, A1, A2 = z[n + ".A"], z[n + ".A1"], z[n + ".A2"]
        m, k = A.shape
        M, K = -(-m // 128) * 128, -(-k // 128) * 128
        big = np.zeros((M, K), dtype=np.uint16)
        big[:m, :k] = A.view(np.uint16)
        want1 = np.zeros((M, K), dtype=np.uint16)
        want1[:m, :k] = A1.view(np.uint16)
        want2 = np.zeros((M, K), dtype=np.uint16)
        want2[:m, :k] = A2.view(np.uint16)
        d_A = torch.from_numpy(big.view(np.int16).copy()).to("cuda:0").view(torch.float16)
        print(f"[gpu case] device split+pack of golden case {n}", flush=True)
        packed, residual = spmm.split_pack_on_device(d_A)
        torch.cuda.synchronize()
        assert np.array_equal(residual.cpu().numpy().view(np.uint16), want2), n
        assert np.array_equal(oracle.a24_unpack(packed.cpu().numpy(), M, K).view(np.uint16), want1), n


@pytest.mark.parametrize("M,K,sparsity,skew", [
    (128, 64, 0.8, False), (256, 192, 0.5, False), (1024, 1024, 0.8, False), (1024, 1024, 0.9, True),
    (512, 512, 0.0, False), (512, 512, 0.999, False), (384, 64 * 5, 0.3, True),
])
def test_device_encoder_matches_oracle(spmm, oracle, M, K, sparsity, skew):
    _compare(spmm, oracle, spmm.synth_weights(M, K, sparsity, skew, seed=M + K))


def test_device_encoder_special_tiles(spmm, oracle):
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
    _compare(spmm, oracle, A)


def test_device_encoded_weight_feeds_the_product(spmm, oracle):
    torch = _torch()
    M, K, N = 512, 1024, 16
    A = spmm.synth_weights(M, K, 0.8, False, seed=5)
    B = spmm.synth_activations(N, K, seed=6)
    d_items, d_offsets = _compare(spmm, oracle, A)
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
