#!/usr/bin/env python3
"""Headline benchmark: Tiled-CSL SpMM, OPT-30B FFN1 (M=28672, K=7168), N=16, 80 % sparse.

One "step" is one SpMM_SplitK_API call (main kernel + split-K reduction) on
inputs already resident in HBM.  The compressed weight is held in several
distinct HBM copies that the steps rotate through, so the stream cannot be
served from the 256 MB Infinity Cache.

Prints ONE JSON line:
  value           effective TFLOPS, 2*M*N*K / step time (whole call)
  hbm_gbps        compressed-weight bytes / step time
  roofline        the main kernel alone: algorithmic bytes (16 * TileOffsets[last])
                  / its average duration, from two HIP events recorded on the launch
                  stream around K back-to-back launches of it, against the 8 TB/s HBM peak
  cpu_baseline    the CPU path timed on this host: reference encoder (oracle/_ref,
                  single thread) + fp32-accumulate dense GEMM (oracle, single thread)

One GPU only: --gpus above 1 exits with a message.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# HBM bytes per launch of the main kernel from rocprofv3 counter runs (FETCH_SIZE and WRITE_SIZE,
# each scaled by what the same counter reads for a copy kernel of known size); summaries of
# those runs are kept under profiles/.  Keyed by (workload, N, split_k); None where not measured.
MEASURED_TRAFFIC_BYTES = {
    ("opt30b_ffn1", 16, 1): 168.70e6,  # mode 1: no partial sums
    ("opt30b_ffn1", 16, 8): 175.50e6,  # mode 0: plus 7.34 MB of partial sums
}
FP16_MFMA_PEAK_TFLOPS = 2500.0

WORKLOADS = {
    # name: (M, K, N, sparsity, row_skewed)
    "opt30b_ffn1": (28672, 7168, 16, 0.8, False),
    "opt30b_ffn2": (7168, 28672, 16, 0.8, False),
    "opt30b_qkv": (21504, 7168, 16, 0.8, False),
    "opt30b_outproj": (7168, 7168, 16, 0.8, False),
    "opt66b_qkv": (27648, 9216, 16, 0.8, False),
    "opt66b_outproj": (9216, 9216, 16, 0.8, False),
    "opt66b_ffn1": (36864, 9216, 16, 0.8, False),
    "opt66b_ffn2": (9216, 36864, 16, 0.8, False),
    "config1": (1024, 1024, 8, 0.8, False),
}


def cpu_baseline(A, B, M, N, K, max_seconds=30.0):
    """The CPU path on this host's cores, single thread: encode + fp32 GEMM.

    The encoder is the reference's own (oracle/_ref) when that build is present,
    else the C restatement.  The GEMM is the oracle's textbook loop, run on as
    many leading 128-row tile rows as fit the time budget (scaled to the full M).
    """
    from oracle import oracle_lib as O

    t0 = time.perf_counter()
    if O.have_ref():
        O.ref_encode(A)
        enc_kind = "reference"
    else:
        O.encode(A)
        enc_kind = "port"
    t_enc = time.perf_counter() - t0

    # calibrate the GEMM on 256 rows, then take what fits
    probe = 256
    t0 = time.perf_counter()
    O.gemm_f32(A[:probe], B)
    t_probe = time.perf_counter() - t0
    rows = int(min(M, max(probe, (max_seconds - t_enc) / max(t_probe / probe, 1e-9))))
    rows = max(probe, rows // 128 * 128)
    t0 = time.perf_counter()
    O.gemm_f32(A[:rows], B)
    t_gemm = (time.perf_counter() - t0) * (M / rows)
    flops = 2.0 * M * N * K

    # the same GEMM spread over the host's cores by 128-row blocks (ctypes releases the GIL)
    from concurrent.futures import ThreadPoolExecutor

    threads = max(1, min(16, os.cpu_count() or 1))
    blocks = [(r, min(r + 128, rows)) for r in range(0, rows, 128)]
    t0 = time.perf_counter()
    with ThreadPoolExecutor(threads) as pool:
        list(pool.map(lambda rb: O.gemm_f32(A[rb[0]:rb[1]], B), blocks))
    t_gemm_mt = (time.perf_counter() - t0) * (M / rows)
    return {
        "value": flops / t_gemm / 1e12,
        "unit": "TFLOPS",
        "cores": 1,
        "kind": "port",
        "sample": (f"fp32-accumulate dense GEMM (oracle C loop) on the first {rows} of {M} rows, scaled to M; "
                   f"Tiled-CSL encode of the full matrix by the {enc_kind} encoder took {t_enc:.2f} s"),
        "gemm_s": t_gemm,
        "encode_s": t_enc,
        "encode_kind": enc_kind,
        "value_with_encode": flops / (t_gemm + t_enc) / 1e12,
        "all_cores": {"value": flops / t_gemm_mt / 1e12, "unit": "TFLOPS", "cores": threads, "gemm_s": t_gemm_mt},
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=1000,
                    help="untimed steps; the default is long enough for the GPU clocks to settle")
    ap.add_argument("--workload", default="opt30b_ffn1", choices=sorted(WORKLOADS))
    ap.add_argument("--n", type=int, default=None, help="override the token count N")
    ap.add_argument("--sparsity", type=float, default=None)
    ap.add_argument("--skew", action="store_true")
    ap.add_argument("--split-k", type=int, default=0, help="0 = SpMM_SuggestSplitK")
    ap.add_argument("--copies", type=int, default=0, help="distinct HBM copies of the weight (0 = enough for > 640 MB)")
    ap.add_argument("--no-reorder", action="store_true",
                    help="encode with InitSparseMatrixA_API_NoReorder (the reference's ablation of its bank-aware reordering)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-check", action="store_true")
    ap.add_argument("--calibration-copies", type=int, default=0,
                    help="after the timed regions, run this many device-to-device copies of the compressed "
                         "weight (SpMM_CalibrationCopy): a kernel of known traffic for scaling byte counters")
    args = ap.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1).", file=sys.stderr)
        sys.exit(2)

    import torch

    import graphneuralnetproj_amd as G

    lib = G.load_library()
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    M, K, N, sparsity, skew = WORKLOADS[args.workload]
    if args.n:
        N = args.n
    if args.sparsity is not None:
        sparsity = args.sparsity
    skew = skew or args.skew
    split_k = args.split_k or G.SpMM_SuggestSplitK(M, N, K)

    # ---- synthetic inputs (host), encode (host), upload
    t0 = time.perf_counter()
    A = G.synth_weights(M, K, sparsity, skew, seed=1234)
    B = G.synth_activations(N, K, seed=4321)
    t_synth = time.perf_counter() - t0
    t0 = time.perf_counter()
    items, offsets = (G.InitSparseMatrixA_API_NoReorder if args.no_reorder else G.InitSparseMatrixA_API)(A)
    t_encode = time.perf_counter() - t0
    a_bytes = 16 * int(offsets[-1])
    copies = args.copies or max(2, -(-640 * 1024 * 1024 // max(a_bytes, 1)))
    copies = min(copies, 64)

    t0 = time.perf_counter()
    d_items = [torch.from_numpy(items.view(np.int32)).to(dev)]
    for _ in range(copies - 1):
        d_items.append(d_items[0].clone())
    # every weight copy has its own TileOffsets array, as every layer of a model would
    d_offs = [torch.from_numpy(offsets).to(dev) for _ in range(copies)]
    d_B = torch.from_numpy(B.view(np.int16)).to(dev)
    d_C = torch.zeros((N, M), dtype=torch.float16, device=dev)
    d_W = torch.zeros((max(split_k, 1), N, M), dtype=torch.float16, device=dev)
    torch.cuda.synchronize()
    t_upload = time.perf_counter() - t0

    stream = torch.cuda.current_stream()
    sptr = ctypes.c_void_p(stream.cuda_stream)
    p_items = [ctypes.c_void_p(t.data_ptr()) for t in d_items]
    p_offs = [ctypes.c_void_p(t.data_ptr()) for t in d_offs]
    p_B, p_C, p_W = (ctypes.c_void_p(t.data_ptr()) for t in (d_B, d_C, d_W))

    def step(i):
        rc = lib.SpMM_SplitK_API(sptr, None, p_items[i % copies], p_offs[i % copies], p_B, p_C, M, N, K, p_W, split_k)
        if rc:
            raise RuntimeError(f"SpMM_SplitK_API -> {rc}")

    # ---- parity of this exact configuration on a row sample (oracle = checker only)
    check = None
    if not args.no_check:
        from oracle import oracle_lib as O

        step(0)
        torch.cuda.synchronize()
        C = d_C.cpu().numpy().astype(np.float32)
        rows = np.unique(np.concatenate([np.arange(0, 256), np.arange(M - 128, M),
                                         np.random.default_rng(0).integers(0, M, 256)]))
        ref = O.gemm_f32(np.ascontiguousarray(A[rows]), B)  # N x len(rows)
        err = np.abs(C[:, rows] - ref)
        ok = bool((err <= 1e-2 + 1e-2 * np.abs(ref)).all())
        check = {"rows": int(len(rows)), "max_abs_err": float(err.max()), "within_tolerance": ok}
        if not ok:
            print(json.dumps({"error": "parity check failed", "check": check}))
            sys.exit(1)

    # ---- timed region: W warm-up steps, then exactly K steps between synchronisations
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps

    # ---- the main kernel alone, live: K back-to-back launches of it (no reduction in between)
    # bracketed by two HIP events recorded on the launch stream; the average includes the
    # dispatch gap between consecutive kernels but no per-launch event overhead.
    for i in range(min(args.warmup, 200)):
        lib.SpMM_SplitK_Partials(sptr, p_items[i % copies], p_offs[i % copies], p_B, p_W, M, N, K, split_k)
    ev0, ev1 = lib.SpMM_EventCreate(), lib.SpMM_EventCreate()
    lib.SpMM_EventRecord(ev0, sptr)
    for i in range(args.steps):
        rc = lib.SpMM_SplitK_Partials(sptr, p_items[i % copies], p_offs[i % copies], p_B, p_W, M, N, K, split_k)
        if rc:
            raise RuntimeError(f"SpMM_SplitK_Partials -> {rc}")
    lib.SpMM_EventRecord(ev1, sptr)
    kernel_ms_avg = float(lib.SpMM_EventElapsedMs(ev0, ev1)) / args.steps
    lib.SpMM_EventDestroy(ev0)
    lib.SpMM_EventDestroy(ev1)
    torch.cuda.synchronize()

    for i in range(args.calibration_copies):
        src, dst = d_items[i % copies], d_items[(i + 1) % copies]  # all copies hold the same bytes
        rc = lib.SpMM_CalibrationCopy(sptr, ctypes.c_void_p(dst.data_ptr()), ctypes.c_void_p(src.data_ptr()), a_bytes)
        if rc:
            raise RuntimeError(f"SpMM_CalibrationCopy -> {rc}")
    torch.cuda.synchronize()

    flops = 2.0 * M * N * K
    tflops = flops / (ms_per_step * 1e-3) / 1e12
    kernel_gbps = a_bytes / (kernel_ms_avg * 1e-3) / 1e9
    out = {
        "metric": "SpMM eff. TFLOPS + HBM GB/s (% roofline), OPT-30B FFN1 80% sparse, N=16",
        "value": tflops,
        "unit": "TFLOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": (f"{args.workload}: M={M} K={K} N={N}, {sparsity * 100:.0f}% "
                         f"{'Beta(2,8) row-skewed' if skew else 'Bernoulli'} sparsity, fp16, fp32 accumulate"),
            "split_k": split_k,
            "compressed_bytes": a_bytes,
            "total_algorithmic_bytes": (a_bytes + 4 * len(offsets) + 2 * K * N + 2 * M * N
                                        + (4 * split_k * M * N if split_k > 1 else 0)),
            "weight_copies_rotated": copies,
            "layout": "B[N][K], C[N][M]",
            "encoding": "scan order (no reordering)" if args.no_reorder else "bank-aware reordering",
        },
        "hbm_gbps": a_bytes / (ms_per_step * 1e-3) / 1e9,
        "hbm_frac_of_peak": a_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        "mfma_frac_of_peak": tflops / FP16_MFMA_PEAK_TFLOPS,
        "roofline": {
            "bound": "hbm",
            "achieved": kernel_gbps,
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": kernel_gbps / HBM_PEAK_GBPS,
            "traffic": (MEASURED_TRAFFIC_BYTES.get((args.workload, N, split_k))
                        if sparsity == 0.8 and not skew else None),
            "kernel": "tcsl_spmm_kernel",
            "kernel_ms_avg": kernel_ms_avg,
            "algorithmic_bytes_per_launch": a_bytes,
        },
        "check": check,
        "host_prep_s": {"synth": t_synth, "encode": t_encode, "upload": t_upload},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(A, B, M, N, K)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
