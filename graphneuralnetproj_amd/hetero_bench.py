"""Times the 2:4 + residual path beside the Tiled-CSL path on one weight shape.

    python -m graphneuralnetproj_amd.hetero_bench [--m 28672 --k 7168] [--sparsity 50,60,70,80] [--n 8,16,32,64]

For each sparsity the weight is split as the reference's benchmark does
(kernel_benchmark/spmm_test.cu:285-330: decompose, then one device form per part) and three
figures are printed per token count, in microseconds per call (events around `--iters` calls,
weights rotated over several copies so that no cache level holds the stream):
  csl     SpMM_SplitK_API on the whole matrix with the planner's Split_K;
  a1      the 2:4 kernel alone (its bytes do not depend on the sparsity);
  hybrid  HeteroSparse_SpMM_API: 2:4 kernel, then the residual's Tiled-CSL kernel (--residual-split-k), which
          adds all slabs up itself where its launch allows, else one reduction kernel;
  2-str   the same with HETERO_FLAG_TWO_STREAMS (the two kernels side by side);
  fused   HeteroSparse_Fused_SpMM_API: both parts in the 2:4 kernel's launch (residual as lists).
"""
import argparse

import numpy as np


def main():
    import torch

    import graphneuralnetproj_amd as G

    ap = argparse.ArgumentParser()
    ap.add_argument("--m", type=int, default=28672)
    ap.add_argument("--k", type=int, default=7168)
    ap.add_argument("--sparsity", default="50,60,70,80")
    ap.add_argument("--n", default="8,16,32,64")
    ap.add_argument("--iters", type=int, default=200)
    ap.add_argument("--copies", type=int, default=3)
    ap.add_argument("--residual-split-k", type=int, default=0,
                    help="Split_K of the residual's Tiled-CSL kernel (0 = the planner's choice for the whole matrix)")
    args = ap.parse_args()
    G.load_library()
    M, K = args.m, args.k
    dev = torch.device("cuda:0")
    st = torch.cuda.current_stream()

    def up(a):
        a = np.ascontiguousarray(a)
        a = a.view(np.int16) if a.dtype == np.float16 else a.view(np.int32) if a.dtype == np.uint32 else a
        return torch.from_numpy(a).to(dev) if a.size else torch.zeros(4, dtype=torch.int32, device=dev)

    def time_us(fn):
        for i in range(args.iters // 4):
            fn(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(args.iters):
            fn(i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.iters * 1e3

    for sp in [int(x) for x in args.sparsity.split(",")]:
        A = G.synth_weights(M, K, sp / 100.0, False, seed=sp)
        A1, A2 = G.HeteroSparse_Decompose(A)
        packed = G.HeteroSparse_PackA1(A1)
        items, offs = G.InitSparseMatrixA_API(A)
        items2, offs2 = G.InitSparseMatrixA_API(A2)
        words, woffs, longest = G.HeteroSparse_PackA2(A2)
        share = float((A2 != 0).sum()) / max(1, int((A != 0).sum()))
        print(f"# {M}x{K} at {sp} %: Tiled-CSL {items.nbytes / 1e6:.1f} MB; 2:4 records {packed.nbytes / 1e6:.1f} MB + "
              f"residual {items2.nbytes / 1e6:.1f} MB ({100 * share:.1f} % of the kept values)", flush=True)
        c = args.copies
        d_items, d_offs = [up(items) for _ in range(c)], [up(offs) for _ in range(c)]
        d_p, d_i2, d_o2 = [up(packed) for _ in range(c)], [up(items2) for _ in range(c)], [up(offs2) for _ in range(c)]
        d_w, d_wo = [up(words) for _ in range(c)], [up(woffs) for _ in range(c)]
        first = True
        for N in [int(x) for x in args.n.split(",")]:
            B = up(G.synth_activations(N, K, seed=1))
            C = torch.empty((N, M), dtype=torch.float16, device=dev)
            s0 = G.SpMM_SuggestSplitK(M, N, K)
            s1 = G.HeteroSparse_SuggestSplitK(M, N, K)
            W = torch.empty((s0 + s1 + 64, N, M), dtype=torch.float16, device=dev)
            if first:  # the host work above let the clocks drop: bring them back before timing anything
                for i in range(1500):
                    G.SpMM_SplitK_API(st, None, d_items[i % c], d_offs[i % c], B, C, M, N, K, W, s0)
                torch.cuda.synchronize()
                first = False
            t_csl = time_us(lambda i: G.SpMM_SplitK_API(st, None, d_items[i % c], d_offs[i % c], B, C, M, N, K, W, s0))
            t_a1 = time_us(lambda i: G.HeteroSparse_A1_Partials(st, d_p[i % c], B, W, M, N, K, s1))
            S2 = args.residual_split_k or s0
            t_h = time_us(lambda i: G.HeteroSparse_SpMM_API(st, d_p[i % c], d_i2[i % c], d_o2[i % c], B, C, M, N, K, W, s1, S2))
            t_2 = time_us(lambda i: G.HeteroSparse_SpMM_API(st, d_p[i % c], d_i2[i % c], d_o2[i % c], B, C, M, N, K, W, s1, S2,
                                                           G.HETERO_FLAG_TWO_STREAMS))
            t_f = float("nan")
            if longest <= G.HETERO_FUSED_MAX_LIST:
                t_f = time_us(lambda i: G.HeteroSparse_Fused_SpMM_API(st, d_p[i % c], d_w[i % c], d_wo[i % c], longest, B, C, M, N, K,
                                                                      W, s1))
            print(f"sparsity {sp} N={N:2d}: csl {t_csl:6.1f} us (Split_K {s0}) | a1 {t_a1:6.1f} us (Split_K {s1}, "
                  f"{packed.nbytes / t_a1 / 1e6:.2f} TB/s) | hybrid {t_h:6.1f} us (residual Split_K {S2}) | 2-str {t_2:6.1f} us | "
                  f"fused {t_f:6.1f} us ({(packed.nbytes + words.nbytes) / t_f / 1e6:.2f} TB/s, longest list {longest})", flush=True)
        del d_items, d_offs, d_p, d_i2, d_o2, d_w, d_wo
        torch.cuda.empty_cache()


if __name__ == "__main__":
    main()
