"""The product's host side through the C ABI: encoder bit-exactness, file wrapper, errors, exports."""
import hashlib
import json
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = os.path.join(ROOT, "tests", "golden")


def test_library_exports_every_declared_symbol(spmm):
    """Every SPMM_EXPORT declaration of include/SpMM_API.h resolves in the shared library."""
    header = open(os.path.join(ROOT, "include", "SpMM_API.h")).read()
    declared = re.findall(r"SPMM_EXPORT\s+[\w\s\*]+?\b(\w+)\s*\(", header)
    assert len(declared) >= 9
    lib = spmm.load_library()
    for name in declared:
        assert hasattr(lib, name), f"{name} declared but not exported"
    from graphneuralnetproj_amd import spmm_api

    assert sorted(declared) == sorted(spmm_api.EXPORTED_SYMBOLS)


def test_mirror_constants_equal_the_headers(spmm):
    """The flag and limit values of the Python mirror are the header's."""
    header = open(os.path.join(ROOT, "include", "SpMM_API.h")).read()
    defines = {name: int(value) for name, value in re.findall(r"#define\s+((?:SPMM_FLAG|HETERO)_\w+)\s+(\d+)", header)}
    assert len(defines) >= 5
    for name, value in defines.items():
        assert getattr(spmm, name) == value, name


def test_product_encoder_matches_golden_small(spmm):
    z = np.load(os.path.join(GOLD, "encoder_small.npz"))
    names = sorted({k.rsplit(".", 1)[0] for k in z.files})
    assert len(names) >= 10
    for n in names:
        items, offs = spmm.InitSparseMatrixA_API(z[n + ".A"])
        assert np.array_equal(offs, z[n + ".offsets"]), n
        assert np.array_equal(items, z[n + ".items"]), n


def test_product_encoder_matches_golden_large(spmm):
    with open(os.path.join(GOLD, "encoder_large.json")) as f:
        cases = json.load(f)
    for c in cases:
        A = spmm.synth_weights(c["M"], c["K"], c["sparsity"], c["row_skewed"], seed=c["seed"])
        assert hashlib.sha256(A.tobytes()).hexdigest() == c["input_sha256"]
        items, offs = spmm.InitSparseMatrixA_API(A)
        assert hashlib.sha256(items.tobytes()).hexdigest() == c["items_sha256"]
        assert hashlib.sha256(offs.tobytes()).hexdigest() == c["offsets_sha256"]


@pytest.mark.parametrize("M,K,sparsity,skew", [(128, 64, 0.8, False), (640, 448, 0.8, False), (256, 1024, 0.6, True),
                                               (1152, 128, 0.93, True), (128, 128, 0.0, False), (256, 64, 1.0, False)])
def test_product_encoder_matches_oracle(spmm, oracle, M, K, sparsity, skew):
    A = spmm.synth_weights(M, K, sparsity, skew, seed=M ^ K)
    items, offs = spmm.InitSparseMatrixA_API(A)
    o_items, o_offs = oracle.encode(A)
    assert np.array_equal(offs, o_offs) and np.array_equal(items, o_items)


def test_encoder_thread_count_does_not_change_output(spmm, monkeypatch):
    A = spmm.synth_weights(1024, 512, 0.8, True, seed=21)
    monkeypatch.setenv("SPMM_ENCODE_THREADS", "1")
    one = spmm.InitSparseMatrixA_API(A)
    monkeypatch.setenv("SPMM_ENCODE_THREADS", "7")
    many = spmm.InitSparseMatrixA_API(A)
    assert np.array_equal(one[0], many[0]) and np.array_equal(one[1], many[1])


def test_encoder_error_codes(spmm):
    """Shapes the reference asserts on (csrc/SpMM_API.cu:310) come back as -1, nothing is allocated."""
    import ctypes

    lib = spmm.load_library()
    buf = np.zeros(128 * 128, dtype=np.uint16)
    for M, K in [(100, 64), (128, 96), (0, 64), (128, 0), (-128, 64)]:
        items = ctypes.POINTER(ctypes.c_uint32)()
        offs = ctypes.POINTER(ctypes.c_int)()
        rc = lib.InitSparseMatrixA_API(buf.ctypes.data_as(ctypes.POINTER(ctypes.c_uint16)), M, 0, K,
                                       ctypes.byref(items), ctypes.byref(offs))
        assert rc == -1 and not items and not offs
    rc = lib.InitSparseMatrixA_API(None, 128, 0, 64, ctypes.byref(items), ctypes.byref(offs))
    assert rc == -3
    with pytest.raises(spmm.SpMMError) as e:
        spmm.InitSparseMatrixA_API(np.zeros((100, 64), dtype=np.uint16))
    assert e.value.code == -1


def test_ignored_n_argument(spmm):
    A = spmm.synth_weights(128, 128, 0.8, False, seed=2)
    a = spmm.InitSparseMatrixA_API(A, N=0)
    b = spmm.InitSparseMatrixA_API(A, N=64)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


def test_gen_sparse_matrix_bin_file(spmm, oracle, tmp_path):
    """File triple of the reference's converter: X.bin -> X.NZWeights.bin (uint32 words),
    X.TileOffsets.bin (int32), X.OutputSizes.bin (int32 word count, int32 number of offsets)."""
    M, K = 256, 192
    A = spmm.synth_weights(M, K, 0.8, False, seed=31)
    base = str(tmp_path / "model.layers.0.mlp.dense_h_to_4h.weight.0")
    A.tofile(base + ".bin")
    spmm.GenSparseMatrixBinFile(base + ".bin", M, K, base + ".NZWeights.bin", base + ".TileOffsets.bin",
                                base + ".OutputSizes.bin")
    sizes = np.fromfile(base + ".OutputSizes.bin", dtype=np.int32)
    items = np.fromfile(base + ".NZWeights.bin", dtype=np.uint32)
    offs = np.fromfile(base + ".TileOffsets.bin", dtype=np.int32)
    o_items, o_offs = oracle.encode(A)
    assert sizes.tolist() == [len(o_items), len(o_offs)]
    assert sizes[0] == 4 * offs[-1]
    assert np.array_equal(items, o_items) and np.array_equal(offs, o_offs)


def test_gen_sparse_matrix_bin_file_errors(spmm, tmp_path):
    base = str(tmp_path / "w")
    with pytest.raises(spmm.SpMMError) as e:  # missing input
        spmm.GenSparseMatrixBinFile(base + ".bin", 128, 64, base + ".nz", base + ".off", base + ".sz")
    assert e.value.code == -4
    np.zeros(100, dtype=np.float16).tofile(base + ".bin")
    with pytest.raises(spmm.SpMMError) as e:  # short input
        spmm.GenSparseMatrixBinFile(base + ".bin", 128, 64, base + ".nz", base + ".off", base + ".sz")
    assert e.value.code == -4
    with pytest.raises(spmm.SpMMError) as e:  # bad shape
        spmm.GenSparseMatrixBinFile(base + ".bin", 10, 10, base + ".nz", base + ".off", base + ".sz")
    assert e.value.code == -1


def test_synthetic_inputs_are_deterministic_and_shaped(spmm):
    A1 = spmm.synth_weights(512, 512, 0.8, False, seed=5)
    A2 = spmm.synth_weights(512, 512, 0.8, False, seed=5)
    assert np.array_equal(A1.view(np.uint16), A2.view(np.uint16))
    dens = np.count_nonzero(A1) / A1.size
    assert abs(dens - 0.2) < 0.01
    nz = A1[A1 != 0].astype(np.float32)
    assert abs(nz.std() - 0.02) < 0.002 and abs(nz.mean()) < 0.001
    B = spmm.synth_activations(16, 4096, seed=6).astype(np.float32)
    assert abs(B.std() - 1.0) < 0.02 and abs(B.mean()) < 0.02
    S = spmm.synth_weights(2048, 256, 0.8, True, seed=5)
    row_dens = (S != 0).mean(axis=1)
    assert row_dens.std() > 0.08 and abs(row_dens.mean() - 0.2) < 0.03  # Beta(2,8): sd 0.12


SHAPES = [(28672, 7168), (7168, 28672), (21504, 7168), (7168, 7168), (36864, 9216), (9216, 36864), (1024, 1024),
          (128, 64), (4096, 4096), (14336, 4096), (53248, 13312), (384, 64 * 97)]


def test_suggest_split_k(spmm):
    for (M, K) in SHAPES:
        for N in (8, 16, 32, 64):
            s = spmm.SpMM_SuggestSplitK(M, N, K)
            assert 1 <= s <= min(32, K // 64)
            # no batch may be empty: the last one starts inside the matrix
            tiles = -(-(K // 64) // s)
            assert tiles * (s - 1) < K // 64
    assert spmm.SpMM_SuggestSplitK(1024, 24, 1024) == 1  # a token count the kernels do not take


def test_planner_gives_runnable_plans(spmm):
    for (M, K) in SHAPES:
        for N in (8, 16, 32, 64):
            for s in (1, 2, 3, 7, 8, 32):
                if s > K // 64:
                    continue
                p = spmm.SpMM_PlanLaunch(M, N, K, s)
                assert p["mode"] in (0, 1)
                assert 1 <= p["waves"] <= (8 if N <= 32 else 4)
                assert p["lds_bytes"] <= 160 * 1024
                assert p["lds_bytes"] >= p["waves"] * 16384
                if p["stage_b"] == 1:    # the batch's slice staged once
                    assert p["mode"] == 0 and N <= 16
                elif p["stage_b"] == 2:  # tile by tile through two buffers
                    assert p["mode"] == 0 and ((N == 32 and p["waves"] in (4, 8)) or (N == 64 and p["waves"] == 4))
                    assert p["lds_bytes"] == p["waves"] * 16384 + 2 * N * 128
                else:
                    assert p["stage_b"] == 0
                assert 0 < p["estimated_us"] < 1e6
    with pytest.raises(spmm.SpMMError):
        spmm.SpMM_PlanLaunch(1000, 16, 1024, 1)
    with pytest.raises(spmm.SpMMError):
        spmm.SpMM_PlanLaunch(1024, 12, 1024, 1)


def test_planner_uses_every_compute_unit_on_the_headline_shapes(spmm):
    # one round of workgroups, at least 200 of them, for the big OPT layers at N = 16
    for (M, K) in [(28672, 7168), (7168, 28672), (36864, 9216), (9216, 36864)]:
        s = spmm.SpMM_SuggestSplitK(M, 16, K)
        p = spmm.SpMM_PlanLaunch(M, 16, K, s)
        wgs = (M // 128) * s if p["mode"] == 1 else -(-(M // 128) // p["waves"]) * s
        assert 200 <= wgs <= 512, (M, K, s, p)


def test_noreorder_encoder_matches_golden_and_oracle(spmm, oracle):
    z = np.load(os.path.join(GOLD, "encoder_small.npz"))
    names = sorted({k.rsplit(".", 1)[0] for k in z.files})
    for n in names:
        items, offs = spmm.InitSparseMatrixA_API_NoReorder(z[n + ".A"])
        assert np.array_equal(offs, z[n + ".offsets"]), n
        assert np.array_equal(items, z[n + ".items_noreorder"]), n
    with open(os.path.join(GOLD, "encoder_large.json")) as f:
        cases = json.load(f)
    for c in cases:
        A = spmm.synth_weights(c["M"], c["K"], c["sparsity"], c["row_skewed"], seed=c["seed"])
        items, offs = spmm.InitSparseMatrixA_API_NoReorder(A)
        assert hashlib.sha256(items.tobytes()).hexdigest() == c["items_noreorder_sha256"]
        assert hashlib.sha256(offs.tobytes()).hexdigest() == c["offsets_sha256"]
    A = spmm.synth_weights(640, 448, 0.75, True, seed=9)
    items, offs = spmm.InitSparseMatrixA_API_NoReorder(A)
    o_items, o_offs = oracle.encode_noreorder(A)
    assert np.array_equal(items, o_items) and np.array_equal(offs, o_offs)
    with pytest.raises(spmm.SpMMError):
        spmm.InitSparseMatrixA_API_NoReorder(np.zeros((100, 64), dtype=np.float16))


def test_split_suggestion_follows_the_weights_density(spmm):
    """SpMM_SuggestSplitK_Bytes: no size given = SpMM_SuggestSplitK; a size picks the table measured at
    the nearest sparsity, and the launch shape that goes with the suggested Split_K is found again
    from (M, N, K, Split_K) alone, which is all a call knows."""
    import re

    def table(name):
        """(M, K, N) -> rows in file order: the shape's measured best first, then rows for other given Split_K."""
        rows = {}
        for ln in open(os.path.join(ROOT, "graphneuralnetproj_amd", "csrc", name)):
            m = re.match(r"\s*\{(\d+), (\d+), (\d+), (\d+), (\d+), (\d+), (\d+)(?:, [01])?\}", ln)  # (an eighth value: reduction kernel)
            if m:
                M, K, N, S, mode, waves, stage = map(int, m.groups())
                rows.setdefault((M, K, N), []).append((S, mode, waves, stage))
        return rows

    t80, t70, t90 = table("tuned_plans.inc"), table("tuned_plans_70.inc"), table("tuned_plans_90.inc")
    assert len(t70) >= 32 and len(t90) >= 32
    for (M, K, N), rows in t80.items():
        assert spmm.SpMM_SuggestSplitK_Bytes(M, N, K, 0) == spmm.SpMM_SuggestSplitK(M, N, K) == rows[0][0]
        assert len({r[0] for r in rows}) == len(rows)  # one row per Split_K
        for row in rows:  # a caller that fixes Split_K gets the launch shape measured for it
            p = spmm.SpMM_PlanLaunch(M, N, K, row[0])
            assert (row[0], p["mode"], p["waves"], p["stage_b"]) == row
    for tab, sparsity in ((t70, 0.7), (t90, 0.9), (t80, 0.8)):
        for (M, K, N), rows in tab.items():
            if (M, K, N) not in t80:
                continue
            S = rows[0][0]
            vectors = int(M * K * (1 - sparsity) / 4 * 1.004)  # 4 words per vector, a little padding
            assert spmm.SpMM_SuggestSplitK_Bytes(M, N, K, vectors) == S, (M, K, N, sparsity)
            p = spmm.SpMM_PlanLaunch(M, N, K, S)
            same_split = [r for t in (t80, t70, t90) for r in t.get((M, K, N), []) if r[0] == S]
            assert (S, p["mode"], p["waves"], p["stage_b"]) == same_split[0]  # the densest-first table that holds this Split_K
    assert spmm.SpMM_SuggestSplitK_Bytes(1024, 24, 1024, 100) == 1
    assert spmm.SpMM_SuggestSplitK_Bytes(1000, 16, 1024, 100) == 1


def test_where_the_slabs_are_added_up(spmm):
    """SpMM_PlanReductionInLaunch: nothing to add with one batch; a K-splitting call adds few batches up
    inside its launch and leaves many (or many tokens' worth) to the reduction kernel; the row-sharing
    layout always uses the kernel; shapes the kernels do not take are refused."""
    assert spmm.SpMM_PlanReductionInLaunch(7168, 16, 7168, 1) is False
    assert spmm.SpMM_PlanLaunch(7168, 16, 7168, 4)["mode"] == 1 and spmm.SpMM_PlanReductionInLaunch(7168, 16, 7168, 4) is True
    assert spmm.SpMM_PlanLaunch(4096, 64, 4096, 8)["mode"] == 1 and spmm.SpMM_PlanReductionInLaunch(4096, 64, 4096, 8) is False
    assert spmm.SpMM_PlanLaunch(2048, 16, 8192, 16)["mode"] == 1 and spmm.SpMM_PlanReductionInLaunch(2048, 16, 8192, 16) is False
    assert spmm.SpMM_PlanLaunch(36864, 16, 9216, 6)["mode"] == 0 and spmm.SpMM_PlanReductionInLaunch(36864, 16, 9216, 6) is False
    for M, N, K, S in ((1000, 16, 1024, 2), (1024, 12, 1024, 2), (1024, 16, 1000, 2), (1024, 16, 1024, 0)):
        with pytest.raises(spmm.SpMMError):
            spmm.SpMM_PlanReductionInLaunch(M, N, K, S)
