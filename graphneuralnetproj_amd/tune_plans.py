#!/usr/bin/env python3
"""Measure launch plans on this machine's GPU and print table rows for the planner.

For every requested (M, K, N) the script times SpMM_SplitK_API_Planned over a grid of
(Split_K, mode, waves, stage_b), checks each result against the library's default plan, and
prints the fastest as a row of graphneuralnetproj_amd/csrc/tuned_plans.inc (rebuild the
library after replacing that file).  It is the counterpart of the reference's hand-edited
per-shape Split_K table (end2end_inference/ft_tools/huggingface_opt_convert_Phase2.py:20).

    python -m graphneuralnetproj_amd.tune_plans --shapes 28672x7168,7168x28672 --tokens 8,16 --out rows.inc
"""
import argparse
import ctypes
import json
import sys
import time

import numpy as np

OPT_SHAPES = ("28672x7168,7168x28672,21504x7168,7168x7168,27648x9216,9216x9216,36864x9216,9216x36864,"
              "36864x12288,12288x12288,49152x12288,12288x49152,"  # OPT-30B, 66B and 175B on one GPU
              "10752x7168,7168x3584,14336x7168,7168x14336,5376x7168,7168x1792,"  # one GPU's share of OPT-30B on 2 and 4
              "13824x9216,9216x4608,18432x9216,9216x18432,6912x9216,9216x2304")  # ... and of OPT-66B


SEPARATE = 3  # in a plan tuple's last place with mode 1: the slabs are added up by the reduction kernel


def planned_args(plan):
    """(Split_K, Mode, Waves, StageB, Flags) of SpMM_SplitK_API_Planned for a plan tuple, launched as a planned call would be."""
    from graphneuralnetproj_amd import SPMM_FLAG_ADAPTIVE_WAVES, SPMM_FLAG_SEPARATE_REDUCTION

    S, mode, w, st = plan
    if mode == 1 and st == SEPARATE:
        return S, mode, w, 0, SPMM_FLAG_ADAPTIVE_WAVES | SPMM_FLAG_SEPARATE_REDUCTION
    return S, mode, w, st, SPMM_FLAG_ADAPTIVE_WAVES


def table_row(M, K, N, plan):
    S, mode, w, st = plan
    if mode == 1 and st == SEPARATE:
        return f"{{{M}, {K}, {N}, {S}, {mode}, {w}, 0, 1}}"
    return f"{{{M}, {K}, {N}, {S}, {mode}, {w}, {st}}}"


def candidate_plans(N, tiles_k, only=None):
    """The grid of (Split_K, mode, waves, stage_b); only = the Split_K values to keep (then every launch
    shape of the grid is tried with each of them, also those the full grid skips for that Split_K).
    Mode 1 with more than one batch is tried with the sum inside the launch and, from four batches on and
    with four waves, with the reduction kernel (last place SEPARATE)."""
    max_w = 8 if N <= 32 else 4
    if only:
        plans = []
        for S in only:
            if S > tiles_k or (S > 1 and -(-tiles_k // S) * (S - 1) >= tiles_k):
                continue  # a batch would be empty
            plans += [(S, 1, w, 0) for w in range(3, max_w + 1)]
            if S >= 4:
                plans.append((S, 1, 4, SEPARATE))
            if N <= 16:
                plans += [(S, 0, w, st) for w in (5, 6, 7, 8) for st in (1, 0)]
            else:
                plans += [(S, 0, w, 0) for w in ((1, 2, 3, 4, 5, 6, 8) if N == 32 else (1, 2, 3, 4))]
                plans += [(S, 0, w, 2) for w in ((4, 8) if N == 32 else (4,))]
        return plans
    plans = []
    for S in (1, 2, 3, 4, 6, 8, 12, 16, 24, 32):
        if S <= tiles_k:
            plans += [(S, 1, w, 0) for w in range(3, max_w + 1)]
            if S >= 4:
                plans.append((S, 1, 4, SEPARATE))
    for S in (1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 14, 16, 20, 24, 28, 32):
        if S <= tiles_k and N <= 16:
            plans += [(S, 0, w, 1) for w in (5, 6, 7, 8)]
            plans += [(S, 0, w, 0) for w in (6, 7, 8)]  # the slice not staged (what fits when it would not): fragments from the L2
    for S in (1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 14, 16, 20, 24, 28, 32):  # few batches too: matrices of several hundred tile rows
        if S <= tiles_k and N >= 32:
            plans += [(S, 0, w, 0) for w in ((1, 2, 3, 4, 5, 6, 8) if N == 32 else (1, 2, 3, 4))]
    if N >= 32:  # the waves share each activation tile through LDS
        for S in (1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 14, 16, 20, 24, 28, 32):
            if S <= tiles_k:
                plans += [(S, 0, w, 2) for w in ((4, 8) if N == 32 else (4,))]
    return plans


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--shapes", default=OPT_SHAPES, help="comma-separated MxK list")
    ap.add_argument("--tokens", default="8,16,32,64")
    ap.add_argument("--sparsity", type=float, default=0.8)
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--split-k", default=None,
                    help="comma-separated Split_K values: one row per (shape, N, Split_K) with the best launch shape "
                         "for that Split_K (rows to append after the shape's own best, for callers that fix Split_K)")
    ap.add_argument("--out", default=None, help="write the table rows here (default: stdout only)")
    ap.add_argument("--log", default=None, help="write every measurement as JSON lines here")
    args = ap.parse_args()

    import torch

    import graphneuralnetproj_amd as G

    lib = G.load_library()
    dev = torch.device("cuda:0")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rows = []
    log = open(args.log, "w") if args.log else None
    warmed = False
    for shape in args.shapes.split(","):
        M, K = (int(x) for x in shape.split("x"))
        A = G.synth_weights(M, K, args.sparsity, False, seed=1234)
        items, offsets = G.InitSparseMatrixA_API(A)
        a_bytes = 16 * int(offsets[-1])
        copies = max(2, -(-640 * 1024 * 1024 // max(a_bytes, 1)))  # more than the 256 MB last-level cache
        d_items = [torch.from_numpy(items.view(np.int32)).to(dev)]
        d_items += [d_items[0].clone() for _ in range(copies - 1)]
        d_offs = torch.from_numpy(offsets).to(dev)
        for N in (int(x) for x in args.tokens.split(",")):
            B = G.synth_activations(N, K, seed=4321)
            d_B = torch.from_numpy(B.view(np.int16)).to(dev)
            d_C = torch.zeros((N, M), dtype=torch.float16, device=dev)
            d_W = torch.zeros((32, N, M), dtype=torch.float16, device=dev)

            def call(i, plan):
                S, mode, w, st, flags = planned_args(plan)
                return lib.SpMM_SplitK_API_Planned(stream, d_items[i % copies].data_ptr(), d_offs.data_ptr(),
                                                   d_B.data_ptr(), d_C.data_ptr(), M, N, K, d_W.data_ptr(), S, mode, w, st, 0,
                                                   flags)  # as a planned call launches it

            S0 = G.SpMM_SuggestSplitK(M, N, K)
            G.SpMM_SplitK_API(None, None, d_items[0], d_offs, d_B, d_C, M, N, K, d_W, S0)
            torch.cuda.synchronize()
            want = d_C.float().clone()
            tol = 2e-2 + 2e-2 * want.abs()
            results = []
            only = [int(x) for x in args.split_k.split(",")] if args.split_k else None
            for plan in candidate_plans(N, K // 64, only):
                if call(0, plan) != 0:
                    continue  # does not fit
                torch.cuda.synchronize()
                if not bool(((d_C.float() - want).abs() <= tol).all()):
                    raise SystemExit(f"plan {plan} disagrees with the default plan on {shape} N={N}")
                for i in range(150 if warmed else 1500):  # the first plan also lets the clocks settle
                    call(i, plan)
                warmed = True
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for i in range(args.steps):
                    call(i, plan)
                torch.cuda.synchronize()
                results.append(((time.perf_counter() - t0) / args.steps * 1e6, plan))
            results.sort()
            if only:
                for S in only:
                    per = [r for r in results if r[1][0] == S]
                    if per:
                        us, (_, mode, w, st) = per[0]
                        rows.append(f"    {table_row(M, K, N, (S, mode, w, st))},  // {us:.1f} us")
                        print(rows[-1], "   runners-up:", "  ".join(f"{p}: {u:.1f}" for u, p in per[1:4]), flush=True)
            else:
                us, (S, mode, w, st) = results[0]
                rows.append(f"    {table_row(M, K, N, (S, mode, w, st))},  // {us:.1f} us")
                print(rows[-1], "   runners-up:", "  ".join(f"{p}: {u:.1f}" for u, p in results[1:4]), flush=True)
            if log:
                log.write(json.dumps({"M": M, "K": K, "N": N, "a_bytes": a_bytes,
                                      "results": [[u, *p] for u, p in results]}) + "\n")
                log.flush()
        del d_items
        torch.cuda.empty_cache()
    text = ("// {M, K, N, Split_K, mode, waves, stage_b[, 1 = mode 1 with the reduction kernel]}"
            "  -- written by graphneuralnetproj_amd/tune_plans.py\n"
            + "\n".join(rows) + "\n")
    if args.out:
        with open(args.out, "w") as f:
            f.write(text)
    else:
        sys.stdout.write(text)


if __name__ == "__main__":
    main()
