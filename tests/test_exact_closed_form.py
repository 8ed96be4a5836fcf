"""The closed form that tests/test_gpu_exact.py compares the GPU with, pinned on the CPU: on the
reference harness's value pattern (weights 1.0, activations in {-5, -3, -1, 1, 3}) it must equal the
oracle's whole-call restatement (encode -> per-batch fp32 products -> fp16 slabs -> reduction) bit
for bit, for even, uneven and oversized splits."""
import numpy as np

import test_gpu_exact as X


def test_harness_pattern_values(spmm):
    A = spmm.synth_harness_weights(256, 512, 0.8, False, seed=3)
    G = spmm.synth_weights(256, 512, 0.8, False, seed=3)
    assert set(np.unique(A.view(np.uint16)).tolist()) == {0, 0x3C00}
    # the keep decisions are synth_weights' own (a drawn value may round to zero there, never here)
    assert ((G.view(np.uint16) & 0x7FFF) != 0).sum() <= (A.view(np.uint16) != 0).sum()
    assert not (((G.view(np.uint16) & 0x7FFF) != 0) & (A.view(np.uint16) == 0)).any()
    assert abs((A.view(np.uint16) != 0).mean() - 0.2) < 0.01
    B = spmm.synth_harness_activations(64, 512, seed=4)
    values, counts = np.unique(B.astype(np.float32), return_counts=True)
    assert values.tolist() == [-5.0, -3.0, -1.0, 1.0, 3.0] and counts.min() > 0.15 * B.size
    assert np.array_equal(B, spmm.synth_harness_activations(64, 512, seed=4))


def test_closed_form_equals_the_oracle_call(spmm, oracle):
    M, K = 384, 1152  # 18 column tiles: 7 batches of 3, 3, 3, 3, 3, 3, 0; 20 batches mostly of one tile
    A = spmm.synth_harness_weights(M, K, 0.75, True, seed=11)
    B = spmm.synth_harness_activations(X.TOKENS, K, seed=12)
    items, offsets = oracle.encode(A)
    splits = (1, 2, 4, 7, 20)
    batches = {s: X._csl_batches(oracle, K, s) for s in splits}
    assert batches[7][-1][0] == batches[7][-1][1] == K  # an empty last batch is part of the sweep
    cuts = X._cuts(K, batches.values())
    seg = X._segment_sums(A, B, cuts)
    assert np.array_equal(seg.sum(axis=0), B.astype(np.float64) @ A.astype(np.float64).T)
    for N in (8, 16, 64):
        for s in splits:
            C, _ = oracle.spmm_splitk(items, offsets, B[:N], M, N, K, s)
            want = X._expected(seg, cuts, batches[s], N)
            assert np.array_equal(C.astype(np.float32), want.astype(np.float32)), (N, s)


def test_unit_batches_partition_the_columns():
    for K, s in [(1024, 1), (1024, 3), (7168, 2), (9216, 5), (28672, 8)]:
        b = X._unit_batches(K, s)
        assert b[0][0] == 0 and b[-1][1] == K and all(x[1] == y[0] for x, y in zip(b, b[1:]))
        assert all((k1 - k0) % 128 == 0 for k0, k1 in b)
