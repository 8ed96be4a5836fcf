"""Model-directory converter and loader against the file formats of the reference's tooling.

Formats pinned by source lines of the reference (no file of it is run):
  huggingface_opt_convert_Phase2.py:13-18 (names), :36-41 (suffixes), :132-134 (shapes per rank),
  :76-81 (dense matrices are skipped), :160-195 (three lists of num_layer * 4 int32);
  csrc/SpMM_API.cu:1598,1613-1619 (OutputSizes = {NNZ, NumOffsets}, NNZ = 4 * last offset);
  third_party/ft.patch:1864-1958,2350-2375 (what the loader reads).
"""
import os

import numpy as np
import pytest

from graphneuralnetproj_amd import model_files as mf

HIDDEN, LAYERS = 256, 2


def write_model(tmp_path, g, sparsity=0.8, dense_at=()):
    """A synthetic FasterTransformer-style directory: every weight file is [K inputs][M outputs] fp16."""
    rank_dir = tmp_path / f"{g}-gpu"
    rank_dir.mkdir()
    (rank_dir / "config.ini").write_text(
        "[gpt]\nweight_data_type = fp16\nnum_layer = %d\nhead_num = 4\nsize_per_head = %d\ninter_size = %d\n"
        % (LAYERS, HIDDEN // 4, 4 * HIDDEN))
    rng = np.random.default_rng(7)
    weights = {}
    for i in range(g):
        for j in range(LAYERS):
            for k, (M, K) in enumerate(mf.rank_shapes(HIDDEN, g)):
                s = 0.3 if (i, j, k) in dense_at else sparsity
                w = (rng.standard_normal((K, M)) * 0.05).astype(np.float16)
                w[rng.random((K, M)) < s] = 0
                w.tofile(rank_dir / (mf.WEIGHT_NAMES[k].format(j, i) + ".bin"))
                weights[(i, j, k)] = w
    return str(rank_dir), weights


def test_rank_shapes_follow_the_reference():
    assert mf.rank_shapes(7168, 1) == [(21504, 7168), (7168, 7168), (28672, 7168), (7168, 28672)]
    assert mf.rank_shapes(9216, 2) == [(13824, 9216), (9216, 4608), (18432, 9216), (9216, 18432)]
    with pytest.raises(ValueError):
        mf.rank_shapes(100, 3)


@pytest.mark.parametrize("g", [1, 2])
def test_converter_writes_the_reference_file_set(tmp_path, spmm, oracle, g):
    rank_dir, weights = write_model(tmp_path, g, dense_at={(0, 1, 2)})
    replaced, skipped = mf.convert_model_dir(str(tmp_path), g, processes=3, tokens=16)
    assert skipped == [0, 0, 1, 0] and replaced == [LAYERS * g, LAYERS * g, LAYERS * g - 1, LAYERS * g]
    shapes = mf.rank_shapes(HIDDEN, g)
    for i in range(g):
        lists = [np.fromfile(os.path.join(rank_dir, f"{n}.{i}.bin"), dtype=np.int32)
                 for n in ("NNZ_List", "NumOffsets_List", "SplitK_List")]
        assert all(a.size == LAYERS * 4 for a in lists)
        for j in range(LAYERS):
            for k, (M, K) in enumerate(shapes):
                stem = os.path.join(rank_dir, mf.WEIGHT_NAMES[k].format(j, i))
                nnz, noff, s = (int(a[j * 4 + k]) for a in lists)
                if (i, j, k) == (0, 1, 2):
                    assert (nnz, noff, s) == (0, 0, 0)
                    assert not os.path.exists(stem + ".NZWeights.bin") and os.path.exists(stem + ".bin")
                    continue
                # the encoded matrix is the transpose of the [K][M] file, bit for bit the oracle's encoding
                o_items, o_offs = oracle.encode(np.ascontiguousarray(weights[(i, j, k)].T))
                assert np.array_equal(np.fromfile(stem + ".NZWeights.bin", dtype=np.uint32), o_items)
                assert np.array_equal(np.fromfile(stem + ".TileOffsets.bin", dtype=np.int32), o_offs)
                sizes = np.fromfile(stem + ".OutputSizes.bin", dtype=np.int32)
                assert sizes.tolist() == [o_items.size, o_offs.size] == [nnz, noff]
                assert nnz == 4 * o_offs[-1] and noff == (M // 128) * (K // 64) + 2
                assert s == spmm.SpMM_SuggestSplitK_Bytes(M, 16, K, nnz // 4) and s >= 1
                # the dense file is untouched without artificial sparsity
                assert np.array_equal(np.fromfile(stem + ".bin", dtype=np.float16).view(np.uint16),
                                      weights[(i, j, k)].view(np.uint16).ravel())


def test_loader_round_trip_and_checks(tmp_path, spmm, oracle):
    rank_dir, weights = write_model(tmp_path, 1, dense_at={(0, 0, 1)})
    mf.convert_model_dir(str(tmp_path), 1)
    layers = mf.load_rank(rank_dir, 0, 1)
    assert len(layers) == LAYERS and all(len(m) == 4 for m in layers)
    for j, mats in enumerate(layers):
        for k, m in enumerate(mats):
            w = weights[(0, j, k)]
            if (0, j, k) == (0, 0, 1):
                assert m.split_k == 0 and m.items is None
                assert np.array_equal(np.array(m.dense).view(np.uint16), w.view(np.uint16))
            else:
                A = oracle.decode(np.array(m.items), np.array(m.offsets), m.M, m.K)
                assert np.array_equal(A, w.T)  # no -0 or NaN in these weights: exact
    # a truncated words file, a wrong list entry and a missing list are all refused
    stem = os.path.join(rank_dir, mf.WEIGHT_NAMES[0].format(1, 0))
    words = np.fromfile(stem + ".NZWeights.bin", dtype=np.uint32)
    words[:-4].tofile(stem + ".NZWeights.bin")
    with pytest.raises(ValueError, match="NZWeights"):
        mf.load_rank(rank_dir, 0, 1)
    words.tofile(stem + ".NZWeights.bin")
    nnz = np.fromfile(os.path.join(rank_dir, "NNZ_List.0.bin"), dtype=np.int32)
    bad = nnz.copy()
    bad[4] += 4
    bad.tofile(os.path.join(rank_dir, "NNZ_List.0.bin"))
    with pytest.raises(ValueError, match="disagrees"):
        mf.load_rank(rank_dir, 0, 1)
    nnz.tofile(os.path.join(rank_dir, "NNZ_List.0.bin"))
    mf.load_rank(rank_dir, 0, 1)
    os.remove(os.path.join(rank_dir, "SplitK_List.0.bin"))
    with pytest.raises(FileNotFoundError):
        mf.load_rank(rank_dir, 0, 1)


def test_reference_orientation_reproduces_the_reference_bytes(tmp_path, spmm, oracle):
    """orientation='as_reference': the dense file is encoded as it lies, read as M x K row-major
    (huggingface_opt_convert_Phase2.py:52-59 passes the untouched file name when no artificial
    sparsity is applied); with artificial sparsity the file is first rewritten as the (K, M)
    transposed view of its (M, K) reshape (:67-72)."""
    rank_dir, weights = write_model(tmp_path, 1)
    M, K = mf.rank_shapes(HIDDEN, 1)[2]
    stem = os.path.join(rank_dir, mf.WEIGHT_NAMES[2].format(0, 0))
    raw = np.fromfile(stem + ".bin", dtype=np.float16)
    r = mf.convert_matrix(stem, M, K, orientation="as_reference")
    o_items, o_offs = oracle.encode(raw.reshape(M, K))
    assert r["replaced"] and r["nnz"] == o_items.size
    assert np.array_equal(np.fromfile(stem + ".NZWeights.bin", dtype=np.uint32), o_items)
    assert np.array_equal(np.fromfile(stem + ".TileOffsets.bin", dtype=np.int32), o_offs)

    stem = os.path.join(rank_dir, mf.WEIGHT_NAMES[2].format(1, 0))
    raw = np.fromfile(stem + ".bin", dtype=np.float16)
    r = mf.convert_matrix(stem, M, K, orientation="as_reference", fake_sparsity=0.5, seed=3)
    rewritten = np.fromfile(stem + ".bin", dtype=np.float16)
    view = raw.reshape(M, K).T  # (K, M)
    kept = rewritten.reshape(K, M) != 0
    assert np.array_equal(rewritten.reshape(K, M)[kept], view[kept])
    assert 0.85 < r["sparsity"] < 0.95  # 80 % zeros already, half of the rest removed
    o_items, _ = oracle.encode(rewritten.reshape(M, K))
    assert np.array_equal(np.fromfile(stem + ".NZWeights.bin", dtype=np.uint32), o_items)
    # for a square matrix both orientations are the same matrix
    Ms, Ks = mf.rank_shapes(HIDDEN, 1)[1]
    a = os.path.join(rank_dir, mf.WEIGHT_NAMES[1].format(0, 0))
    mf.convert_matrix(a, Ms, Ks, orientation="ft")
    ft_words = np.fromfile(a + ".NZWeights.bin", dtype=np.uint32)
    w = np.fromfile(a + ".bin", dtype=np.float16)
    assert np.array_equal(ft_words, oracle.encode(np.ascontiguousarray(w.reshape(Ks, Ms).T))[0])


def test_artificial_sparsity_keeps_dense_and_sparse_files_consistent(tmp_path, spmm, oracle):
    rank_dir, weights = write_model(tmp_path, 1, sparsity=0.0)
    M, K = mf.rank_shapes(HIDDEN, 1)[0]
    stem = os.path.join(rank_dir, mf.WEIGHT_NAMES[0].format(0, 0))
    r = mf.convert_matrix(stem, M, K, fake_sparsity=0.8, seed=11)
    assert r["replaced"] and 0.78 < r["sparsity"] < 0.82
    w = np.fromfile(stem + ".bin", dtype=np.float16).reshape(K, M)
    A = oracle.decode(np.fromfile(stem + ".NZWeights.bin", dtype=np.uint32),
                      np.fromfile(stem + ".TileOffsets.bin", dtype=np.int32), M, K)
    assert np.array_equal(A, w.T)
    kept = w != 0
    assert np.array_equal(w[kept], weights[(0, 0, 0)][kept])
    # same seed, same mask
    weights[(0, 0, 0)].tofile(stem + ".bin")
    mf.convert_matrix(stem, M, K, fake_sparsity=0.8, seed=11)
    assert np.array_equal(np.fromfile(stem + ".bin", dtype=np.float16).reshape(K, M), w)


def test_config_checks(tmp_path):
    d = tmp_path / "1-gpu"
    d.mkdir()
    with pytest.raises(FileNotFoundError):
        mf.read_config(str(d))
    (d / "config.ini").write_text("[gpt]\nweight_data_type = fp32\nnum_layer = 1\nhead_num = 2\nsize_per_head = 64\n"
                                  "inter_size = 512\n")
    with pytest.raises(ValueError, match="fp16"):
        mf.read_config(str(d))
    (d / "config.ini").write_text("[gpt]\nweight_data_type = fp16\nnum_layer = 1\nhead_num = 2\nsize_per_head = 64\n"
                                  "inter_size = 500\n")
    with pytest.raises(ValueError, match="inter_size"):
        mf.read_config(str(d))
