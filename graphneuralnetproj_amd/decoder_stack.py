#!/usr/bin/env python3
"""A stack of decoder-block linear layers on Tiled-CSL weights, chained without copies.

Per layer, with hidden size h and N tokens (all buffers one contiguous vector per token):

    qkv = W_qkv x            (3h x h)      x:   [N][h]
    o   = W_out qkv[:, :h]   (h x h)       the projection reads the first third of the fused buffer
    f   = relu(W_ffn1 o)     (4h x h)      clamp fused into the product
    x'  = W_ffn2 f           (h x 4h)      input of the next layer

This is the sequence of sparse products FasterTransformer's patched OPT decoder issues per token
(third_party/ft.patch:513-632 feed-forward, :1248-1339 attention projections) with everything
between them (attention itself, biases, layer norms) left out: a linear-stack microbenchmark
of the weight stream, sized so that the weights of all layers stay resident in HBM.

    python -m graphneuralnetproj_amd.decoder_stack --hidden 9216 --layers 64 --tokens 16

prints one JSON line with the time per token step for the whole stack, eager and as a HIP graph.
"""
import argparse
import json
import time

import numpy as np


class Layer:
    """Device-resident weights of one block: name -> (items, offsets, M, K, split_k).

    A matrix that stayed dense on disk (split_k == 0, third_party/ft.patch:1864-1958) is
    (None, W, M, K, 0) with W the fp16 [K][M] tensor of its file; it goes through the
    library GEMM, as it goes to cuBLAS in the reference.
    """

    def __init__(self, mats):
        self.mats = mats

    @staticmethod
    def is_split(mat):
        return isinstance(mat[0], tuple)

    def clone(self):
        return Layer({k: (it.clone() if it is not None else None, of if it is not None else of.clone(), M, K, s)
                      for k, (it, of, M, K, s) in self.mats.items()})

    def bytes(self):
        total = 0
        for mat in self.mats.values():
            it, of = mat[0], mat[1]
            if Layer.is_split(mat):  # ((records, words), (list offsets, longest list), M, K, split_k)
                total += it[0].numel() + 4 * (it[1].numel() - 64)
            else:
                total += it.numel() * 4 if it is not None else of.numel() * 2
        return total


def layer_shapes(h):
    return {"qkv": (3 * h, h), "out": (h, h), "ffn1": (4 * h, h), "ffn2": (h, 4 * h)}


def build_layer(G, torch, dev, h, N, sparsity, seed, keep_dense=False, weight_scale=1.0):
    """Synthesise, encode and upload one block; weight_scale multiplies the N(0, 0.02) weights."""
    mats, dense = {}, {}
    for i, (name, (M, K)) in enumerate(layer_shapes(h).items()):
        A = G.synth_weights(M, K, sparsity, False, seed=seed * 16 + i)
        if weight_scale != 1.0:
            A = (A.astype(np.float32) * weight_scale).astype(np.float16)
        items, offsets = G.InitSparseMatrixA_API(A)
        mats[name] = (torch.from_numpy(items.view(np.int32)).to(dev), torch.from_numpy(offsets).to(dev), M, K,
                      G.SpMM_SuggestSplitK_Bytes(M, N, K, int(offsets[-1])))
        if keep_dense:
            dense[name] = A
    return Layer(mats), dense


def build_layer_on_device(G, torch, dev, h, N, sparsity, seed, weight_std=0.02, sample_rows=0):
    """One block with random-init weights made and encoded on the GPU (nothing crosses PCIe).

    Every matrix is N(0, weight_std) fp16 with Bernoulli(1 - sparsity) kept entries, drawn from a
    torch generator seeded with `seed`, and goes through the device encoder (same bits as the host
    encoder would give for the same matrix).  With sample_rows > 0 the second value maps each
    matrix name to (row indices, those rows of the dense matrix as a host fp16 array), for
    checking products against a CPU reference without keeping the dense matrices.
    """
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    mats, samples = {}, {}
    for name, (M, K) in layer_shapes(h).items():
        A = torch.randn((M, K), generator=gen, device=dev, dtype=torch.float32)
        A.mul_(weight_std)
        A.mul_(torch.rand((M, K), generator=gen, device=dev) >= sparsity)
        A = A.to(torch.float16)
        items, offsets = G.encode_on_device(A)
        mats[name] = (items, offsets, M, K, G.SpMM_SuggestSplitK_Bytes(M, N, K, items.numel() // 4))
        if sample_rows:
            rows = torch.randperm(M, generator=gen, device=dev)[:sample_rows].sort().values
            samples[name] = (rows.cpu().numpy(), A[rows].cpu().numpy())
        del A, items
    return Layer(mats), samples


def build_split_layer_on_device(G, torch, dev, h, N, sparsity, seed, weight_std=0.02, sample_rows=0):
    """build_layer_on_device with every weight split into a 2:4 part (records for the sparse matrix
    instruction) and a residual (lists), the fork's decomposition (kernel_benchmark/spmm_decompose.h:12-51),
    for the one-launch product.  Same random matrices as build_layer_on_device gives for the seed.
    A matrix is ((records, words), (list offsets, longest list), M, K, split_k)."""
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    mats, samples = {}, {}
    for name, (M, K) in layer_shapes(h).items():
        A = torch.randn((M, K), generator=gen, device=dev, dtype=torch.float32)
        A.mul_(weight_std)
        A.mul_(torch.rand((M, K), generator=gen, device=dev) >= sparsity)
        A = A.to(torch.float16)
        records, residual = G.split_pack_on_device(A)
        words, offsets, longest = G.pack_residual_on_device(residual)
        if longest > G.HETERO_FUSED_MAX_LIST:
            raise ValueError(f"{name}: a residual list of {longest} words: more than a residual can hold ({G.HETERO_FUSED_MAX_LIST})")
        mats[name] = ((records, words), (offsets, longest), M, K, G.HeteroSparse_SuggestSplitK(M, N, K))
        if sample_rows:
            rows = torch.randperm(M, generator=gen, device=dev)[:sample_rows].sort().values
            samples[name] = (rows.cpu().numpy(), A[rows].cpu().numpy())
        del A, residual
    return Layer(mats), samples


class Stack:
    """row_major: every buffer holds [features][N] (this fork's operand layout) instead of one vector per
    token; the output projection then reads the first h rows of the fused QKV result."""

    def __init__(self, G, torch, layers, h, N, row_major=False):
        self.G, self.torch, self.layers, self.h, self.N, self.row_major = G, torch, layers, h, N, row_major
        first = layers[0].mats["qkv"]
        dev = (first[1][0] if Layer.is_split(first) else first[1]).device
        f16 = torch.float16
        shape = (lambda rows: (rows, N)) if row_major else (lambda rows: (N, rows))
        self.x = [torch.zeros(shape(h), dtype=f16, device=dev) for _ in range(2)]  # ping-pong layer inputs
        self.qkv = torch.zeros(shape(3 * h), dtype=f16, device=dev)
        self.o = torch.zeros(shape(h), dtype=f16, device=dev)
        self.f = torch.zeros(shape(4 * h), dtype=f16, device=dev)
        max_split = max(1, max(s for L in layers for (_, _, _, _, s) in L.mats.values()))
        # one workspace for every product, as the reference's caller keeps (third_party/ft.patch:2762-2765)
        self.ws = torch.zeros((max_split, N, 4 * h), dtype=f16, device=dev)

    def _product(self, stream, mat, src, ldb, dst, ldc, flags=0):
        it, of, M, K, s = mat
        if self.row_major:
            if it is None:
                raise ValueError("the row-major chain takes encoded weights only")
            if Layer.is_split(mat):
                self.G.HeteroSparse_Fused_SpMM_API_RowMajor(stream, it[0], it[1], of[0], of[1], src, dst, M, self.N, K, self.ws, s, flags)
            else:
                self.G.SpMM_SplitK_API_RowMajor_Flags(stream, it, of, src, dst, M, self.N, K, self.ws, s, flags)
        elif Layer.is_split(mat):
            self.G.HeteroSparse_Fused_SpMM_API_Strided(stream, it[0], it[1], of[0], of[1], src, ldb, dst, ldc, M, self.N, K,
                                                       self.ws, s, flags)
        elif it is not None:
            self.G.SpMM_SplitK_API_Strided(stream, it, of, src, ldb, dst, ldc, M, self.N, K, self.ws, s, flags)
        else:  # dense on disk: [N][K] x [K][M] on the library GEMM (torch's current stream)
            self.torch.mm(src[:, :K], of, out=dst[:, :M])
            if flags & self.G.SPMM_FLAG_RELU:
                dst[:, :M].relu_()

    def step(self, stream):
        """Enqueue one token step through every layer; returns the buffer holding the result."""
        h = self.h
        cur = 0
        for L in self.layers:
            m = L.mats
            x, nxt = self.x[cur], self.x[cur ^ 1]
            self._product(stream, m["qkv"], x, h, self.qkv, 3 * h)
            self._product(stream, m["out"], self.qkv, 3 * h, self.o, h)
            self._product(stream, m["ffn1"], self.o, h, self.f, 4 * h, self.G.SPMM_FLAG_RELU)
            self._product(stream, m["ffn2"], self.f, 4 * h, nxt, h)
            cur ^= 1
        return self.x[cur]


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--hidden", type=int, default=9216, help="h; 9216 = OPT-66B, 7168 = OPT-30B")
    ap.add_argument("--layers", type=int, default=64)
    ap.add_argument("--tokens", type=int, default=16)
    ap.add_argument("--sparsity", type=float, default=0.8)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--weights", choices=("device", "host", "copied"), default="device",
                    help="device: every layer's weights are drawn and encoded on the GPU (default); host: drawn and "
                         "encoded on the host by the library's generator and encoder; copied: one host-made layer, "
                         "copied in HBM for the others")
    ap.add_argument("--row-major", action="store_true",
                    help="keep the activations as [features][tokens] (this fork's layout) and use the row-major entry")
    ap.add_argument("--split", action="store_true",
                    help="split every weight into a 2:4 part and a residual and multiply both in one launch "
                         "(worth it up to about 70 %% sparsity); weights are made on the GPU")
    ap.add_argument("--model-dir", help="run rank 0 of a converted one-rank model directory (<dir>/1-gpu/, written by "
                                        "graphneuralnetproj_amd.model_files) instead of synthetic weights")
    args = ap.parse_args()

    import torch

    import graphneuralnetproj_amd as G

    G.load_library()
    dev = torch.device("cuda:0")
    h, N = args.hidden, args.tokens
    t0 = time.perf_counter()
    if args.model_dir:
        import os

        from . import model_files

        rank_dir = os.path.join(args.model_dir, "1-gpu")
        args.layers, h = model_files.read_config(rank_dir)
        layers = model_files.upload_layers(model_files.load_rank(rank_dir, 0, 1), dev, tokens=N)
    else:
        if args.split:
            layers = [build_split_layer_on_device(G, torch, dev, h, N, args.sparsity, seed=1 + i)[0] for i in range(args.layers)]
        elif args.weights == "device":
            layers = [build_layer_on_device(G, torch, dev, h, N, args.sparsity, seed=1 + i)[0] for i in range(args.layers)]
        else:
            first, _ = build_layer(G, torch, dev, h, N, args.sparsity, seed=1)
            layers = [first]
            for i in range(1, args.layers):
                layers.append(build_layer(G, torch, dev, h, N, args.sparsity, seed=1 + i)[0] if args.weights == "host"
                              else first.clone())
    torch.cuda.synchronize()
    prep_s = time.perf_counter() - t0
    stack = Stack(G, torch, layers, h, N, row_major=args.row_major)
    x0 = torch.from_numpy(G.synth_activations(N, h, seed=99).view(np.int16)).to(dev).view(torch.float16)
    if args.row_major:
        x0 = x0.t().contiguous()
    stream = torch.cuda.current_stream()

    def run_eager():
        stack.x[0].copy_(x0)
        return stack.step(stream)

    for _ in range(args.warmup):
        run_eager()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        stack.step(stream)  # chained on the previous step's output: same work, no reset copy
    torch.cuda.synchronize()
    eager_ms = (time.perf_counter() - t0) * 1e3 / args.steps

    graph_ms = None
    graph_matches = None
    try:
        want = run_eager().clone()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        stack.x[0].copy_(x0)
        with torch.cuda.graph(g):
            out = stack.step(torch.cuda.current_stream())
        for _ in range(3):  # replays checked against the eager result, with eager work in between
            stack.x[0].copy_(x0)
            g.replay()
            torch.cuda.synchronize()
            graph_matches = bool(torch.equal(out, want))
            if not graph_matches:
                break
            run_eager()
            torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            g.replay()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    except Exception as e:  # graph capture is an optimisation; the eager figure stands on its own
        graph_matches = f"capture failed: {e}"

    weight_bytes = sum(L.bytes() for L in layers)
    best_ms = min(eager_ms, graph_ms) if graph_ms and graph_matches is True else eager_ms
    flops = 2.0 * N * sum(M * K for (M, K) in layer_shapes(h).values()) * args.layers
    print(json.dumps({
        "metric": "decoder linear stack: time per token step",
        "value": best_ms, "unit": "ms", "higher_is_better": False,
        "eager_ms": eager_ms, "graph_ms": graph_ms, "graph_matches_eager": graph_matches,
        "config": {"workload": f"{args.layers} layers x (QKV, out-proj, FFN1+ReLU, FFN2), h={h}, N={N}, "
                               f"{args.sparsity * 100:.0f}% sparse",
                   "form": "2:4 records + residual lists, one launch per product" if args.split else "Tiled-CSL",
                   "layout": "B[K][N], C[M][N]" if args.row_major else "B[N][K], C[N][M]",
                   "weights": "model directory" if args.model_dir else
                   {"device": "random-init per layer, drawn and encoded on the GPU",
                    "host": "random-init per layer, drawn and encoded on the host",
                    "copied": "one layer's weights copied per layer"}[args.weights]},
        "resident_weight_bytes": weight_bytes,
        "hbm_gbps": weight_bytes / (best_ms * 1e-3) / 1e9,
        "hbm_frac_of_peak": weight_bytes / (best_ms * 1e-3) / 1e9 / 8000.0,
        "effective_tflops": flops / (best_ms * 1e-3) / 1e12,
        "hbm_floor_ms": weight_bytes / 8e12 * 1e3,
        "prep_s": prep_s, "data": "files" if args.model_dir else "synthetic",
    }))


if __name__ == "__main__":
    main()
