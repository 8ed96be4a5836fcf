#!/usr/bin/env python3
"""The on-disk model format of the sparse decoder weights: converter and loader.

Converter = the reference's phase-2 script
(end2end_inference/ft_tools/huggingface_opt_convert_Phase2.py:13-200): for every tensor-parallel
rank i, decoder layer j and each of the four weight matrices

    model.layers.{j}.attention.query_key_value.weight.{i}    M = 3h/g   K = h
    model.layers.{j}.attention.dense.weight.{i}              M = h      K = h/g
    model.layers.{j}.mlp.dense_h_to_4h.weight.{i}            M = 4h/g   K = h
    model.layers.{j}.mlp.dense_4h_to_h.weight.{i}            M = h      K = 4h/g

it reads `<name>.bin` (fp16), and if the matrix is at least 50 % zeros writes
`<name>.NZWeights.bin` (uint32 Tiled-CSL words), `<name>.TileOffsets.bin` (int32) and
`<name>.OutputSizes.bin` (int32 {NNZ, NumOffsets}) next to it (:36-59); denser matrices stay
dense (:76-81).  Then it writes, per rank, `NNZ_List.{i}.bin`, `NumOffsets_List.{i}.bin` and
`SplitK_List.{i}.bin`: num_layer * 4 int32 each, in the order above, all three zero for a
matrix that stayed dense (:160-195).

Loader = what the patched FasterTransformer does with those files
(third_party/ft.patch:1864-1958 per layer, :2350-2375 the three lists): `SplitK != 0` selects
the sparse pair of files, whose lengths are the list entries; otherwise the dense file.

Differences from the reference's script, on purpose:
  * Split_K comes from the library's planner for the 256-CU part (SpMM_SuggestSplitK_Bytes) instead
    of the table keyed by M (:20).
  * `orientation="ft"` (default) treats `<name>.bin` as what phase 1 wrote, [K inputs][M
    outputs] (huggingface_opt_convert_Phase1.py:195-271 permutes every weight to that), and
    encodes its transpose, the M x K matrix the kernel multiplies by.  The reference reshapes
    the file to (M, K) and then transposes (:67), which is the same thing only for square
    matrices; `orientation="as_reference"` reproduces that byte for byte.
  * artificial sparsity (:69-72) is off unless asked for, and seeded.
"""
import argparse
import configparser
import os
import time
from concurrent.futures import ThreadPoolExecutor

import numpy as np

WEIGHT_NAMES = (
    "model.layers.{}.attention.query_key_value.weight.{}",
    "model.layers.{}.attention.dense.weight.{}",
    "model.layers.{}.mlp.dense_h_to_4h.weight.{}",
    "model.layers.{}.mlp.dense_4h_to_h.weight.{}",
)
THRESHOLD_SKIPPING_REPLACE = 0.5  # huggingface_opt_convert_Phase2.py:21


def rank_shapes(hidden_size, infer_gpu_num):
    """(M, K) of the four matrices on one of g ranks (huggingface_opt_convert_Phase2.py:132-134)."""
    h, g = hidden_size, infer_gpu_num
    if h % g:
        raise ValueError(f"hidden size {h} is not divisible by {g} ranks")
    return [(3 * h // g, h), (h, h // g), (4 * h // g, h), (h, 4 * h // g)]


def read_config(rank_dir):
    """num_layer, hidden_size from config.ini, with the checks of the reference (:113-130)."""
    cfg = configparser.ConfigParser()
    if not cfg.read(os.path.join(rank_dir, "config.ini")):
        raise FileNotFoundError(os.path.join(rank_dir, "config.ini"))
    if len(cfg.sections()) != 1:
        raise ValueError("config.ini must have exactly one section")
    sec = cfg[cfg.sections()[0]]
    if sec.get("weight_data_type") != "fp16":
        raise ValueError("weight_data_type must be fp16")
    num_layer = int(sec["num_layer"])
    hidden = int(sec["head_num"]) * int(sec["size_per_head"])
    if int(sec["inter_size"]) != 4 * hidden:
        raise ValueError("inter_size must be 4 * hidden size")
    return num_layer, hidden


def _sparse_names(stem):
    return stem + ".NZWeights.bin", stem + ".TileOffsets.bin", stem + ".OutputSizes.bin"


def convert_matrix(stem, M, K, orientation="ft", fake_sparsity=None, seed=0, remove_dense=False):
    """Convert `<stem>.bin`; returns dict(replaced, nnz, num_offsets, sparsity).

    fake_sparsity = p zeroes each element with probability p first and rewrites the dense file
    (the reference's FAKE_SPARSITY branch, :69-72, p = 0.8 there).
    """
    import graphneuralnetproj_amd as G

    if orientation not in ("ft", "as_reference"):
        raise ValueError("orientation must be 'ft' or 'as_reference'")
    dense_name = stem + ".bin"
    w = np.fromfile(dense_name, dtype=np.float16)
    if w.size != M * K:
        raise ValueError(f"{dense_name}: {w.size} elements, expected {M} x {K}")
    if orientation == "ft":
        A = w.reshape(K, M).T           # file is [K][M]; the kernel's matrix is its transpose
    else:
        A = w.reshape(M, K).T           # the reference's view (:67), shape (K, M)
    if fake_sparsity is not None:
        keep = np.random.default_rng(seed).random(A.shape) >= fake_sparsity
        A = A * keep.astype(np.float16)
        if orientation == "ft":
            np.ascontiguousarray(A.T).tofile(dense_name)
        else:
            A.tofile(dense_name)        # row-major (K, M), which the encoder then reads as M x K
    nnz = int(np.count_nonzero(A))
    sparsity = 1.0 - nnz / float(M * K)
    nz_name, off_name, sizes_name = _sparse_names(stem)
    if sparsity < THRESHOLD_SKIPPING_REPLACE:
        return {"replaced": False, "nnz": 0, "num_offsets": 0, "sparsity": sparsity}
    if orientation == "ft":
        items, offsets = G.InitSparseMatrixA_API(np.ascontiguousarray(A))
        items.tofile(nz_name)
        offsets.tofile(off_name)
        np.array([items.size, offsets.size], dtype=np.int32).tofile(sizes_name)
    else:
        G.GenSparseMatrixBinFile(dense_name, M, K, nz_name, off_name, sizes_name)
    sizes = np.fromfile(sizes_name, dtype=np.int32)
    if remove_dense:
        os.remove(dense_name)
    return {"replaced": True, "nnz": int(sizes[0]), "num_offsets": int(sizes[1]), "sparsity": sparsity}


def convert_model_dir(model_dir, infer_gpu_num, processes=1, tokens=16, orientation="ft", fake_sparsity=None,
                      seed=0, remove_dense=False, log=None):
    """Convert `<model_dir>/<g>-gpu/` in place and write the three per-rank lists.

    `processes` matrices are converted at a time (threads: the encoder releases the interpreter
    and is itself multi-threaded).  `tokens` is the batch the Split_K values are planned for.
    Returns (replaced, skipped) counts per matrix kind.
    """
    import graphneuralnetproj_amd as G

    g = infer_gpu_num
    rank_dir = os.path.join(model_dir, f"{g}-gpu")
    num_layer, hidden = read_config(rank_dir)
    shapes = rank_shapes(hidden, g)
    jobs = [(i, j, k) for i in range(g) for j in range(num_layer) for k in range(4)]

    def one(job):
        i, j, k = job
        stem = os.path.join(rank_dir, WEIGHT_NAMES[k].format(j, i))
        M, K = shapes[k]
        r = convert_matrix(stem, M, K, orientation, fake_sparsity, seed + (i * num_layer + j) * 4 + k, remove_dense)
        if log:
            log(f"{stem}: sparsity {r['sparsity']:.4f} " + ("replaced" if r["replaced"] else "kept dense"))
        return r

    with ThreadPoolExecutor(max_workers=max(1, processes)) as pool:
        results = dict(zip(jobs, pool.map(one, jobs)))

    replaced, skipped = [0] * 4, [0] * 4
    for i in range(g):
        nnz, noff, splitk = [], [], []
        for j in range(num_layer):
            for k in range(4):
                r = results[(i, j, k)]
                M, K = shapes[k]
                nnz.append(r["nnz"])
                noff.append(r["num_offsets"])
                # (the planner is told how much the weight holds: nnz words = nnz / 4 vectors)
                splitk.append(G.SpMM_SuggestSplitK_Bytes(M, tokens, K, r["nnz"] // 4) if r["replaced"] else 0)
                (replaced if r["replaced"] else skipped)[k] += 1
        for name, vals in (("NNZ_List", nnz), ("NumOffsets_List", noff), ("SplitK_List", splitk)):
            np.array(vals, dtype=np.int32).tofile(os.path.join(rank_dir, f"{name}.{i}.bin"))
    return replaced, skipped


class Matrix:
    """One weight of one layer as the loader found it.

    Sparse (`split_k != 0`): `items` uint32[NNZ] and `offsets` int32[NumOffsets].
    Dense (`split_k == 0`): `dense` fp16 [K][M], the layout of the file.
    Arrays are memory maps of the files.
    """

    def __init__(self, M, K, split_k, items=None, offsets=None, dense=None):
        self.M, self.K, self.split_k = M, K, split_k
        self.items, self.offsets, self.dense = items, offsets, dense


def _map(path, dtype, count):
    size = os.path.getsize(path)
    if size != count * np.dtype(dtype).itemsize:
        raise ValueError(f"{path}: {size} bytes, expected {count} x {np.dtype(dtype).itemsize}")
    if count == 0:
        return np.zeros(0, dtype=dtype)
    return np.memmap(path, dtype=dtype, mode="r", shape=(count,))


def load_rank(rank_dir, rank, infer_gpu_num, num_layer=None, hidden_size=None):
    """Weights of one rank: list over layers of four `Matrix` (order of WEIGHT_NAMES).

    Follows third_party/ft.patch:2350-2375 (lists of num_layer * 4 ints) and :1864-1958 (file
    choice per matrix); also checks what the reference leaves unchecked: file lengths against
    the lists, offsets shape, and NNZ = 4 * last offset (csrc/SpMM_API.cu:1598).
    """
    if num_layer is None or hidden_size is None:
        num_layer, hidden_size = read_config(rank_dir)
    shapes = rank_shapes(hidden_size, infer_gpu_num)
    lists = [_map(os.path.join(rank_dir, f"{n}.{rank}.bin"), np.int32, num_layer * 4)
             for n in ("NNZ_List", "NumOffsets_List", "SplitK_List")]
    nnz_list, noff_list, splitk_list = lists
    layers = []
    for j in range(num_layer):
        mats = []
        for k in range(4):
            stem = os.path.join(rank_dir, WEIGHT_NAMES[k].format(j, rank))
            M, K = shapes[k]
            nnz, noff, s = (int(a[j * 4 + k]) for a in (nnz_list, noff_list, splitk_list))
            if s != 0:
                if noff != (M // 128) * (K // 64) + 2:
                    raise ValueError(f"{stem}: {noff} tile offsets do not fit a {M} x {K} matrix")
                offsets = _map(stem + ".TileOffsets.bin", np.int32, noff)
                if nnz != 4 * int(offsets[-1]) or offsets[0] != 0 or offsets[-1] != offsets[-2]:
                    raise ValueError(f"{stem}: NNZ {nnz} disagrees with its tile offsets")
                mats.append(Matrix(M, K, s, items=_map(stem + ".NZWeights.bin", np.uint32, nnz), offsets=offsets))
            else:
                mats.append(Matrix(M, K, 0, dense=_map(stem + ".bin", np.float16, M * K).reshape(K, M)))
        layers.append(mats)
    return layers


def upload_layers(layers, device, tokens=None):
    """Device copies as `decoder_stack.Layer`s; tokens re-plans Split_K for that batch (None keeps the files')."""
    import torch

    import graphneuralnetproj_amd as G
    from .decoder_stack import Layer

    out = []
    for mats in layers:
        d = {}
        for name, m in zip(("qkv", "out", "ffn1", "ffn2"), mats):
            if m.split_k != 0:
                s = G.SpMM_SuggestSplitK_Bytes(m.M, tokens, m.K, len(m.items) // 4) if tokens else m.split_k
                items = torch.from_numpy(np.array(m.items).view(np.int32)).to(device)
                if items.numel() == 0:
                    items = torch.zeros(4, dtype=torch.int32, device=device)
                d[name] = (items, torch.from_numpy(np.array(m.offsets)).to(device), m.M, m.K, s)
            else:
                w = torch.from_numpy(np.array(m.dense).view(np.int16)).to(device).view(torch.float16)
                d[name] = (None, w, m.M, m.K, 0)
        out.append(Layer(d))
    return out


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("-model_dir", "-m", required=True, help="directory holding <g>-gpu/")
    ap.add_argument("-infer_gpu_num", "-i_g", type=int, required=True)
    ap.add_argument("-processes", "-p", type=int, default=1, help="matrices converted at a time")
    ap.add_argument("-tokens", type=int, default=16, help="batch the Split_K list is planned for")
    ap.add_argument("-orientation", choices=("ft", "as_reference"), default="ft")
    ap.add_argument("-fake_sparsity", type=float, default=None, help="zero this fraction of every matrix first")
    ap.add_argument("-seed", type=int, default=0)
    ap.add_argument("-remove_dense", action="store_true")
    args = ap.parse_args()
    t0 = time.time()
    replaced, skipped = convert_model_dir(args.model_dir, args.infer_gpu_num, args.processes, args.tokens,
                                          args.orientation, args.fake_sparsity, args.seed, args.remove_dense, log=print)
    for k in range(4):
        print(f"{WEIGHT_NAMES[k].format('*', '*')}: replaced {replaced[k]}, kept dense {skipped[k]}")
    print(f"converted in {time.time() - t0:.1f} s")


if __name__ == "__main__":
    main()
