#!/usr/bin/env python3
"""Headline benchmark: Tiled-CSL SpMM, OPT-30B FFN1 (M=28672, K=7168), N=16, 80 % sparse.

One "step" is one SpMM_SplitK_API call (main kernel + split-K reduction) on
inputs already resident in HBM.  The compressed weight is held in several
distinct HBM copies that the steps rotate through, so the stream cannot be
served from the 256 MB Infinity Cache.

The clocks are settled by the benchmark itself: before the --warmup steps it launches the
same call, untimed, for at least PREWARM_SECONDS (1 s: behind a process that held tens of GB the
kernel runs 6-7 % slow for its first 0.65 s of launches) and then until a block of 1000 launches is no
faster than the three blocks before it (at most 10 s; reported as prewarm_launches,
prewarm_seconds_spent and settle_blocks_us), so a short --steps/--warmup run measures the same
machine state as a long one, also when another process has just worked the GPU.  The block of --steps
steps, bracketed by synchronisations, is then timed --repeats times and the median reported.

Prints ONE JSON line:
  value           effective TFLOPS, 2*M*N*K / step time (whole call)
  hbm_gbps        compressed-weight bytes / step time
  roofline        the main kernel alone: algorithmic bytes (16 * TileOffsets[last])
                  / its average duration, from two HIP events recorded on the launch stream
                  around --repeats x K back-to-back launches of it (one pair of events: an
                  event between two kernels costs the stream microseconds), against the
                  8 TB/s HBM peak
  cpu_baseline    the CPU path timed on this host: reference encoder (oracle/_ref,
                  single thread) + fp32-accumulate dense GEMM (oracle, single thread)
  sweep           the benchmark's other configurations, each timed for a fraction of a
                  second after the headline: ms per whole call (events around 100 calls) and
                  the fraction of 8 TB/s on that weight's compressed bytes; kernel_ms, the main
                  kernel alone writing C or its slabs of partial sums (events around 100
                  launches of SpMM_SplitK_Partials); traffic where a counter profile of the
                  case is kept under profiles/.  Covers N, sparsity and skew on FFN1, both
                  operand layouts, the attention projections with Split_K in {1, 2, 4, 7} and
                  N in {8, 16, 32}, the OPT-66B shapes at N in {8, 16, 32}, the OPT-175B shapes,
                  the 2:4 + residual split, and the 64-layer decoder stack's time per token step.
                  The sweep's weights are drawn and encoded on the GPU.

--hetero times the 2:4 + residual path beside the Tiled-CSL path on one weight shape and prints
one line per sparsity and token count instead of the JSON line.

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
    # (workload, N, split_k, sparsity): (bytes, profile that holds the counter run)
    ("opt30b_ffn1", 16, 1, 0.8): (168.70e6, "profiles/tcsl_spmm_kernel_opt30b_ffn1_n16_pmc.txt"),  # mode 1: no partial sums
    ("opt30b_ffn1", 16, 8, 0.8): (175.50e6, "profiles/tcsl_spmm_kernel_opt30b_ffn1_n16_pmc.txt"),  # mode 0: plus 7.34 MB of partial sums
    ("opt30b_ffn1", 64, 1, 0.8): (177.52e6, "profiles/tcsl_spmm_kernel_sweep_cases_hbm_traffic.txt"),
    ("opt30b_ffn1", 32, 1, 0.8): (171.70e6, "profiles/tcsl_spmm_kernel_sweep_cases_hbm_traffic.txt"),
    ("opt30b_ffn1", 8, 1, 0.8): (167.29e6, "profiles/tcsl_spmm_kernel_sweep_cases_hbm_traffic.txt"),
    ("opt30b_ffn1", 16, 1, 0.9): (86.15e6, "profiles/tcsl_spmm_kernel_sweep_cases_hbm_traffic.txt"),
    ("opt30b_ffn1", 16, 1, 0.7): (251.38e6, "profiles/tcsl_spmm_kernel_sweep_cases_hbm_traffic.txt"),
    ("opt30b_ffn2", 16, 4, 0.8): (174.77e6, "profiles/tcsl_spmm_kernel_sweep_cases_hbm_traffic.txt"),
    ("opt30b_outproj", 16, 4, 0.8): (44.78e6, "profiles/tcsl_spmm_kernel_sweep_cases_hbm_traffic.txt"),
    ("opt30b_qkv", 16, 8, 0.8): (132.20e6, "profiles/tcsl_spmm_kernel_sweep_cases_hbm_traffic.txt"),
    ("opt66b_ffn1", 16, 6, 0.8): (285.10e6, "profiles/tcsl_spmm_kernel_sweep_cases_hbm_traffic.txt"),
}
TRAFFIC_SOURCE = ("rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command, scaled by a copy kernel of known "
                  "size; summary in the named profile (not measured live)")


def measured_traffic(workload, N, split_k, sparsity, skew):
    """(bytes per launch, profile file) from a kept counter run of exactly this case, else (None, None)."""
    if skew:
        return None, None
    return MEASURED_TRAFFIC_BYTES.get((workload, N, split_k, sparsity), (None, None))
PREWARM_SECONDS = 1.0
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
    "opt175b_qkv": (36864, 12288, 16, 0.8, False),
    "opt175b_outproj": (12288, 12288, 16, 0.8, False),
    "opt175b_ffn1": (49152, 12288, 16, 0.8, False),
    "opt175b_ffn2": (12288, 49152, 16, 0.8, False),
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

    nproc = os.cpu_count() or 1
    threads = max(1, min(16, nproc))
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
        "kinds": {"gemm": "port (oracle/tiled_csl_oracle.c)", "encode": f"{enc_kind}" + (" (oracle/_ref)" if enc_kind == "reference" else "")},
        "nproc": nproc,
        "sample": (f"fp32-accumulate dense GEMM (oracle C loop) on the first {rows} of {M} rows, scaled to M; "
                   f"Tiled-CSL encode of the full matrix by the {enc_kind} encoder took {t_enc:.2f} s"),
        "gemm_s": t_gemm,
        "encode_s": t_enc,
        "encode_kind": enc_kind,
        "value_with_encode": flops / (t_gemm + t_enc) / 1e12,
        "all_cores": {"value": flops / t_gemm_mt / 1e12, "unit": "TFLOPS", "cores": threads, "gemm_s": t_gemm_mt},
    }


def prewarm(call, torch, seconds=PREWARM_SECONDS):
    """Launch call(i) back to back, untimed, until `seconds` of wall time have passed; returns the count."""
    n = 0
    t_end = time.perf_counter() + seconds
    while time.perf_counter() < t_end:
        for _ in range(100):
            call(n)
            n += 1
        torch.cuda.synchronize()
    return n


SETTLE_BLOCK = 1000        # launches per block whose time is watched
SETTLE_TOLERANCE = 0.003   # a block within 0.3 % of the best of the three before it: no longer getting faster
SETTLE_MAX_SECONDS = 10.0


def settle(lib, sptr, call, torch, min_seconds, adaptive=True):
    """Launch call(i) back to back, untimed for the benchmark's purposes, until the machine has reached
    its steady state: at least `min_seconds`, then until a block of SETTLE_BLOCK launches is no
    faster than the three before it (bounded by SETTLE_MAX_SECONDS).  On an idle GPU the clocks come up
    within some 15 ms of continuous launches.  Straight after another process that held tens of GB
    and worked the GPU hard (the 52 GB decoder stack, or a test run that ends with it), the same kernel
    runs on a plateau 6-7 % slow for the first 0.65 s of continuous launches (31.05 us per launch,
    flat, then one step down to 29.05 us; measured three times, 1000 launches per point), whatever
    the pause in between: PREWARM_SECONDS is set past that plateau, and the blocks behind it catch a
    slower ramp.  Returns (launches, seconds spent, [us per launch of every block])."""
    t0 = time.perf_counter()
    n = prewarm(call, torch, min_seconds)
    blocks = []
    while adaptive and time.perf_counter() - t0 < SETTLE_MAX_SECONDS:
        blocks.append(events_ms(lib, sptr, lambda i: call(n + i), SETTLE_BLOCK) / SETTLE_BLOCK * 1e3)
        n += SETTLE_BLOCK
        if len(blocks) >= 4 and blocks[-1] >= (1.0 - SETTLE_TOLERANCE) * min(blocks[-4:-1]):
            break
    return n, time.perf_counter() - t0, blocks


def events_ms(lib, sptr, call, n):
    """Milliseconds between two HIP events recorded on the launch stream around call(0) .. call(n-1)."""
    ev0, ev1 = lib.SpMM_EventCreate(), lib.SpMM_EventCreate()
    lib.SpMM_EventRecord(ev0, sptr)
    for i in range(n):
        call(i)
    lib.SpMM_EventRecord(ev1, sptr)
    ms = float(lib.SpMM_EventElapsedMs(ev0, ev1))
    lib.SpMM_EventDestroy(ev0)
    lib.SpMM_EventDestroy(ev1)
    return ms


def sweep_cases():
    """(label, workload, N, sparsity, row_skewed, split_k); split_k 0 = the planner's choice for the
    weight's density.  A label ending in _row_major goes through SpMM_SplitK_API_RowMajor (B[K][N],
    C[M][N]: this fork's own operand layout).  Cases that share a weight are adjacent."""
    cases = [
        ("ffn1_n16_row_major", "opt30b_ffn1", 16, 0.8, False, 0),
        ("ffn1_n64_row_major", "opt30b_ffn1", 64, 0.8, False, 0),
        ("ffn1_n8", "opt30b_ffn1", 8, 0.8, False, 0),
        ("ffn1_n32", "opt30b_ffn1", 32, 0.8, False, 0),
        ("ffn1_n64", "opt30b_ffn1", 64, 0.8, False, 0),
        ("ffn1_70pct", "opt30b_ffn1", 16, 0.7, False, 0),
        ("ffn1_90pct", "opt30b_ffn1", 16, 0.9, False, 0),
        ("ffn1_skewed", "opt30b_ffn1", 16, 0.8, True, 0),
        ("ffn2", "opt30b_ffn2", 16, 0.8, False, 0),
        ("ffn2_n64", "opt30b_ffn2", 64, 0.8, False, 0),
    ]
    # the attention projections: the planner's choice and the sweep's Split_K in {1, 2, 4, 7}, N in {8, 16, 32}
    for name in ("qkv", "outproj"):
        for N in (16, 8, 32):
            cases.append((name if N == 16 else f"{name}_n{N}", f"opt30b_{name}", N, 0.8, False, 0))
            for split_k in (1, 2, 4, 7):
                cases.append((f"{name}_n{N}_split{split_k}", f"opt30b_{name}", N, 0.8, False, split_k))
    for model in ("opt66b", "opt175b"):
        for name in ("qkv", "outproj", "ffn1", "ffn2"):
            # 64 tokens where the matrix has 288 and more tile rows (few batches of row-sharing workgroups)
            for N in (16, 8, 32) + ((64,) if (model, name) in (("opt66b", "ffn1"), ("opt175b", "qkv"), ("opt175b", "ffn1")) else ()):
                cases.append((f"{model}_{name}" if N == 16 else f"{model}_{name}_n{N}", f"{model}_{name}", N, 0.8, False, 0))
    return cases


def device_weight(G, torch, dev, M, K, sparsity, skew, seed):
    """A synthetic weight of the benchmark's distribution made and encoded on the GPU (nothing crosses
    PCIe): N(0, 0.02) fp16 values, kept with probability 1 - sparsity, or, row-skewed, with a per-row
    probability (1 - sparsity) * Beta(2, 8) / 0.2 (Beta as Gamma(2) / (Gamma(2) + Gamma(8)), a Gamma(k)
    being minus the log of a product of k uniforms).  Returns (items, offsets) as device tensors; the
    device encoder gives the bits the host encoder would."""
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    A = torch.randn((M, K), generator=gen, device=dev, dtype=torch.float32)
    A.mul_(0.02)
    keep = torch.full((M, 1), 1.0 - sparsity, device=dev)
    if skew:
        u = torch.rand((M, 10), generator=gen, device=dev).clamp_min_(1e-12).log_().neg_()
        x, y = u[:, :2].sum(1, keepdim=True), u[:, 2:].sum(1, keepdim=True)
        keep = ((1.0 - sparsity) * (x / (x + y)) / 0.2).clamp_max_(1.0)
    A.mul_(torch.rand((M, K), generator=gen, device=dev) < keep)
    A = A.to(torch.float16)
    items, offsets = G.encode_on_device(A)
    return items, offsets


def sweep(G, lib, torch, dev, sptr, with_stack):
    """The benchmark's other configurations.  Per case: whole calls (main kernel + reduction) between
    two events, 100 calls after a pre-warm, median of three; the main kernel alone the same way; weights
    rotated over > 640 MB of copies."""
    out = []
    cache = {}
    for label, workload, N, sparsity, skew, forced_split in sweep_cases():
        M, K = WORKLOADS[workload][:2]
        key = (workload, sparsity, skew)
        if key not in cache:
            cache.clear()  # one weight resident at a time
            torch.cuda.empty_cache()
            items, offsets = device_weight(G, torch, dev, M, K, sparsity, skew, seed=1234)
            a_bytes = 4 * items.numel()
            copies = min(64, max(2, -(-640 * 1024 * 1024 // max(a_bytes, 1))))
            d_items = [items] + [items.clone() for _ in range(copies - 1)]
            d_offs = [offsets] + [offsets.clone() for _ in range(copies - 1)]
            cache[key] = (a_bytes, copies, d_items, d_offs)
        a_bytes, copies, d_items, d_offs = cache[key]
        split_k = forced_split or G.SpMM_SuggestSplitK_Bytes(M, N, K, a_bytes // 16)
        d_B = torch.from_numpy(G.synth_activations(N, K, seed=4321).view(np.int16)).to(dev)
        d_C = torch.zeros((N, M), dtype=torch.float16, device=dev)
        d_W = torch.zeros((max(split_k, 1), N, M), dtype=torch.float16, device=dev)
        p_items = [ctypes.c_void_p(t.data_ptr()) for t in d_items]
        p_offs = [ctypes.c_void_p(t.data_ptr()) for t in d_offs]
        p_B, p_C, p_W = (ctypes.c_void_p(t.data_ptr()) for t in (d_B, d_C, d_W))

        row_major = label.endswith("_row_major")  # the same buffers hold either layout's elements
        entry = lib.SpMM_SplitK_API_RowMajor if row_major else lib.SpMM_SplitK_API

        def call(i):
            rc = entry(sptr, None, p_items[i % copies], p_offs[i % copies], p_B, p_C, M, N, K, p_W, split_k)
            if rc:
                raise RuntimeError(f"{'SpMM_SplitK_API_RowMajor' if row_major else 'SpMM_SplitK_API'} -> {rc}")

        def kernel(i):
            rc = lib.SpMM_SplitK_Partials(sptr, p_items[i % copies], p_offs[i % copies], p_B, p_W if split_k > 1 else p_C,
                                          M, N, K, split_k)
            if rc:
                raise RuntimeError(f"SpMM_SplitK_Partials -> {rc}")

        settle(lib, sptr, call, torch, 0.05)
        ms = float(np.median([events_ms(lib, sptr, call, 100) for _ in range(3)])) / 100
        kernel_ms = None
        if not row_major:  # (the kernel-alone entry point takes the column-major layout)
            for i in range(20):
                kernel(i)
            kernel_ms = float(np.median([events_ms(lib, sptr, kernel, 100) for _ in range(3)])) / 100
        torch.cuda.synchronize()
        plan = G.SpMM_PlanLaunch(M, N, K, split_k)
        traffic, traffic_profile = measured_traffic(workload, N, split_k, sparsity, skew)
        out.append({"case": label, "M": M, "K": K, "N": N, "sparsity": sparsity, "row_skewed": skew, "split_k": split_k,
                    "split_k_from": "sweep" if forced_split else "planner",
                    "layout": "B[K][N], C[M][N]" if row_major else "B[N][K], C[N][M]",
                    "plan": f"mode {plan['mode']}, {plan['waves']} waves", "compressed_bytes": a_bytes,
                    "reduction": ("none" if split_k == 1 else
                                  "in launch" if G.SpMM_PlanReductionInLaunch(M, N, K, split_k) else "kernel"),
                    "ms": ms, "frac": a_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                    "kernel_ms": kernel_ms,
                    "kernel_frac": a_bytes / (kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS if kernel_ms else None,
                    "traffic": traffic, "traffic_profile": traffic_profile,
                    "tflops": 2.0 * M * N * K / (ms * 1e-3) / 1e12})
    cache.clear()
    torch.cuda.empty_cache()
    for sparsity in (0.6, 0.7):
        out.append(split_case(G, lib, torch, dev, sptr, "opt30b_ffn1", 16, sparsity))
    # row-skewed: residual lists of up to several hundred words, beyond what travels with the records
    out.append(split_case(G, lib, torch, dev, sptr, "opt30b_ffn1", 16, 0.6, skew=True))
    if with_stack:
        out.append(stack_step(G, torch, dev))
        # the same stack at a sparsity where the fork's split pays, in both forms
        out.append(stack_step(G, torch, dev, sparsity=0.6))
        out.append(stack_step(G, torch, dev, sparsity=0.6, split=True))
    return out


def split_case(G, lib, torch, dev, sptr, workload, N, sparsity, skew=False):
    """The fork's split of a weight into a 2:4 part and a residual, at a sparsity where it can pay:
    plain Tiled-CSL, the two-kernel call and the one-launch call on the same weight, whole calls
    between two events, weights rotated over three copies."""
    M, K = WORKLOADS[workload][:2]
    A = G.synth_weights(M, K, sparsity, skew, seed=1234)
    A1, A2 = G.HeteroSparse_Decompose(A)
    items, offsets = G.InitSparseMatrixA_API(A)
    del A
    packed = G.HeteroSparse_PackA1(A1)
    del A1
    items2, offsets2 = G.InitSparseMatrixA_API(A2)
    words, list_offsets, longest = G.HeteroSparse_PackA2(A2)
    del A2
    copies = 3

    def up(a):
        a = a.view(np.int32) if a.dtype == np.uint32 else a
        return [torch.from_numpy(a).to(dev) for _ in range(copies)]

    d = {k: up(v) for k, v in dict(items=items, offs=offsets, packed=packed, items2=items2, offs2=offsets2, words=words,
                                    lists=list_offsets).items()}
    p = {k: [ctypes.c_void_p(t.data_ptr()) for t in v] for k, v in d.items()}
    s_csl = G.SpMM_SuggestSplitK_Bytes(M, N, K, int(offsets[-1]))
    s_res = G.SpMM_SuggestSplitK(M, N, K)
    s_a1 = G.HeteroSparse_SuggestSplitK(M, N, K)
    d_B = torch.from_numpy(G.synth_activations(N, K, seed=4321).view(np.int16)).to(dev)
    d_C = torch.zeros((N, M), dtype=torch.float16, device=dev)
    d_W = torch.zeros((s_csl + s_res + s_a1, N, M), dtype=torch.float16, device=dev)
    p_B, p_C, p_W = (ctypes.c_void_p(t.data_ptr()) for t in (d_B, d_C, d_W))

    def check(rc, what):
        if rc:
            raise RuntimeError(f"{what} -> {rc}")

    def csl(i):
        check(lib.SpMM_SplitK_API(sptr, None, p["items"][i % copies], p["offs"][i % copies], p_B, p_C, M, N, K, p_W, s_csl),
              "SpMM_SplitK_API")

    def two(i):
        check(lib.HeteroSparse_SpMM_API(sptr, p["packed"][i % copies], p["items2"][i % copies], p["offs2"][i % copies], p_B, p_C,
                                        M, N, K, p_W, s_a1, s_res, 0), "HeteroSparse_SpMM_API")

    def one(i):
        check(lib.HeteroSparse_Fused_SpMM_API(sptr, p["packed"][i % copies], p["words"][i % copies], p["lists"][i % copies], longest,
                                              p_B, p_C, M, N, K, p_W, s_a1), "HeteroSparse_Fused_SpMM_API")

    def one_row_major(i):  # the same buffers hold either layout's elements
        check(lib.HeteroSparse_Fused_SpMM_API_RowMajor(sptr, p["packed"][i % copies], p["words"][i % copies], p["lists"][i % copies],
                                                       longest, p_B, p_C, M, N, K, p_W, s_a1, 0), "HeteroSparse_Fused_SpMM_API_RowMajor")

    res = {}
    outputs = {}
    for name, fn in (("tiled_csl", csl), ("two_kernels", two), ("one_launch", one), ("one_launch_row_major", one_row_major)):
        if name.startswith("one_launch") and longest > G.HETERO_FUSED_MAX_LIST:
            res[name] = None
            continue
        settle(lib, sptr, fn, torch, 0.05)
        res[name] = float(np.median([events_ms(lib, sptr, fn, 100) for _ in range(3)])) / 100
        torch.cuda.synchronize()
        if name != "one_launch_row_major":  # (its operands are the other layout's bytes: timing only)
            outputs[name] = d_C.float().cpu().numpy()
    ref = outputs["tiled_csl"]
    agree = all(bool((np.abs(o - ref) <= 2e-2 + 2e-2 * np.abs(ref)).all()) for o in outputs.values())
    one_bytes = packed.nbytes + 4 * int(list_offsets[-1])
    best = res["one_launch"] or res["two_kernels"]
    return {"case": f"ffn1_{int(sparsity * 100)}pct{'_skewed' if skew else ''}_2to4_plus_residual", "M": M, "K": K, "N": N,
            "sparsity": sparsity, "row_skewed": skew, "longest_residual_list": longest,
            "one_launch_row_major_ms": res["one_launch_row_major"],
            "tiled_csl_bytes": 16 * int(offsets[-1]), "records_bytes": packed.nbytes, "residual_list_bytes": 4 * int(list_offsets[-1]),
            "tiled_csl_ms": res["tiled_csl"], "two_kernels_ms": res["two_kernels"], "one_launch_ms": res["one_launch"],
            "split_k": {"tiled_csl": s_csl, "records": s_a1, "residual": s_res}, "outputs_agree": agree,
            "ms": best, "frac": one_bytes / (best * 1e-3) / 1e9 / HBM_PEAK_GBPS}


def stack_step(G, torch, dev, layers=64, h=9216, N=16, sparsity=0.8, split=False):
    """64 OPT-66B-shaped blocks, random-init weights drawn and encoded on the GPU (about 52 GB
    resident at 80 % sparsity): time per token step, eager and as a HIP graph.  split: every weight
    as 2:4 records + residual lists, one launch per product, instead of Tiled-CSL."""
    from graphneuralnetproj_amd import decoder_stack as DS

    torch.cuda.empty_cache()
    t0 = time.perf_counter()
    build = DS.build_split_layer_on_device if split else DS.build_layer_on_device
    blocks = [build(G, torch, dev, h, N, sparsity, seed=1 + i)[0] for i in range(layers)]
    torch.cuda.synchronize()
    build_s = time.perf_counter() - t0
    stack = DS.Stack(G, torch, blocks, h, N)
    x0 = torch.from_numpy(G.synth_activations(N, h, seed=99).view(np.int16)).to(dev).view(torch.float16)
    stream = torch.cuda.current_stream()
    stack.x[0].copy_(x0)
    for _ in range(5):
        stack.step(stream)
    torch.cuda.synchronize()
    times = []
    for _ in range(5):
        t0 = time.perf_counter()
        for _ in range(5):
            stack.step(stream)
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) * 1e3 / 5)
    eager_ms = float(np.median(times))
    graph_ms = None
    g = None
    try:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            stack.step(torch.cuda.current_stream())
        g.replay()
        torch.cuda.synchronize()
        times = []
        for _ in range(5):
            t0 = time.perf_counter()
            for _ in range(5):
                g.replay()
            torch.cuda.synchronize()
            times.append((time.perf_counter() - t0) * 1e3 / 5)
        graph_ms = float(np.median(times))
    except Exception as e:  # the eager figure stands on its own
        graph_ms = None
        print(f"bench.py: graph capture of the stack failed: {e}", file=sys.stderr)
    weight_bytes = sum(L.bytes() for L in blocks)
    ms = min(eager_ms, graph_ms) if graph_ms else eager_ms
    row_major_ms = None
    # the same weights with the activations in this fork's layout, [features][tokens]
    del stack, g
    stack = DS.Stack(G, torch, blocks, h, N, row_major=True)
    stack.x[0].copy_(x0.t())
    for _ in range(5):
        stack.step(stream)
    torch.cuda.synchronize()
    times = []
    for _ in range(5):
        t0 = time.perf_counter()
        for _ in range(5):
            stack.step(stream)
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) * 1e3 / 5)
    row_major_ms = float(np.median(times))
    g = None
    del stack, blocks, g
    torch.cuda.empty_cache()
    case = "decoder_stack" if sparsity == 0.8 and not split else f"decoder_stack_{int(sparsity * 100)}pct" + ("_split" if split else "")
    return {"case": case, "layers": layers, "hidden": h, "N": N, "sparsity": sparsity,
            "form": "2:4 records + residual lists, one launch per product" if split else "Tiled-CSL",
            "weights": "random-init per layer, drawn and encoded on the GPU", "resident_weight_bytes": weight_bytes,
            "ms": ms, "eager_ms": eager_ms, "graph_ms": graph_ms, "frac": weight_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            "row_major_eager_ms": row_major_ms,
            "row_major_frac": weight_bytes / (row_major_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS if row_major_ms else None,
            "hbm_floor_ms": weight_bytes / (HBM_PEAK_GBPS * 1e9) * 1e3, "build_s": build_s}


def hetero_mode(args):
    """Times the 2:4 + residual path beside the Tiled-CSL path on one weight shape.  For each sparsity
    the weight is split as the reference's benchmark does (kernel_benchmark/spmm_test.cu:285-330:
    decompose, then one device form per part) and five figures are printed per token count, in
    microseconds per call (events around --hetero-iters calls, weights rotated over three copies so
    that no cache level holds the stream):
      csl     SpMM_SplitK_API on the whole matrix with the planner's Split_K;
      a1      the 2:4 kernel alone (its bytes do not depend on the sparsity);
      hybrid  HeteroSparse_SpMM_API: 2:4 kernel, then the residual's Tiled-CSL kernel, which adds all
              slabs up itself where its launch allows, else one reduction kernel;
      2-str   the same with HETERO_FLAG_TWO_STREAMS (the two kernels side by side);
      fused   HeteroSparse_Fused_SpMM_API: both parts in the 2:4 kernel's launch (residual as lists)."""
    import torch

    import graphneuralnetproj_amd as G

    G.load_library()
    M, K = (int(x) for x in args.hetero_shape.lower().split("x"))
    dev = torch.device("cuda:0")
    st = torch.cuda.current_stream()
    iters, c = args.hetero_iters, 3

    def up(a):
        a = np.ascontiguousarray(a)
        a = a.view(np.int16) if a.dtype == np.float16 else a.view(np.int32) if a.dtype == np.uint32 else a
        return torch.from_numpy(a).to(dev) if a.size else torch.zeros(4, dtype=torch.int32, device=dev)

    def time_us(fn):
        for i in range(iters // 4):
            fn(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(iters):
            fn(i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters * 1e3

    for sp in [int(x) for x in args.hetero_sparsity.split(",")]:
        A = G.synth_weights(M, K, sp / 100.0, False, seed=sp)
        A1, A2 = G.HeteroSparse_Decompose(A)
        packed = G.HeteroSparse_PackA1(A1)
        items, offs = G.InitSparseMatrixA_API(A)
        items2, offs2 = G.InitSparseMatrixA_API(A2)
        words, woffs, longest = G.HeteroSparse_PackA2(A2)
        share = float((A2 != 0).sum()) / max(1, int((A != 0).sum()))
        print(f"# {M}x{K} at {sp} %: Tiled-CSL {items.nbytes / 1e6:.1f} MB; 2:4 records {packed.nbytes / 1e6:.1f} MB + "
              f"residual {items2.nbytes / 1e6:.1f} MB ({100 * share:.1f} % of the kept values)", flush=True)
        d_items, d_offs = [up(items) for _ in range(c)], [up(offs) for _ in range(c)]
        d_p, d_i2, d_o2 = [up(packed) for _ in range(c)], [up(items2) for _ in range(c)], [up(offs2) for _ in range(c)]
        d_w, d_wo = [up(words) for _ in range(c)], [up(woffs) for _ in range(c)]
        first = True
        for N in [int(x) for x in args.hetero_n.split(",")]:
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
            S2 = args.hetero_residual_split_k or s0
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
    ap.add_argument("--split-k", type=int, default=0, help="0 = SpMM_SuggestSplitK_Bytes")
    ap.add_argument("--copies", type=int, default=0, help="distinct HBM copies of the weight (0 = enough for > 640 MB)")
    ap.add_argument("--no-reorder", action="store_true",
                    help="encode with InitSparseMatrixA_API_NoReorder (the reference's ablation of its bank-aware reordering)")
    ap.add_argument("--repeats", type=int, default=15, help="timed blocks of --steps steps; the median is reported")
    ap.add_argument("--prewarm-seconds", type=float, default=PREWARM_SECONDS,
                    help="least time of untimed launches before --warmup, to settle the clocks; blocks of 1000 launches follow "
                         "until they stop getting faster (shorten it under a counter-collecting profiler)")
    ap.add_argument("--no-settle", action="store_true",
                    help="pre-warm for --prewarm-seconds only, without the blocks that wait for the steady state "
                         "(for runs under a counter-collecting profiler, where every launch is slow)")
    ap.add_argument("--no-sweep", action="store_true", help="skip the other configurations after the headline")
    ap.add_argument("--no-stack", action="store_true", help="sweep without the 64-layer decoder stack (52 GB)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-check", action="store_true")
    ap.add_argument("--calibration-copies", type=int, default=0,
                    help="after the timed regions, run this many device-to-device copies of the compressed "
                         "weight (SpMM_CalibrationCopy): a kernel of known traffic for scaling byte counters")
    ap.add_argument("--hetero", action="store_true",
                    help="time the 2:4 + residual path beside Tiled-CSL on one shape and print one line per case (no JSON)")
    ap.add_argument("--hetero-shape", default="28672x7168", help="MxK of --hetero")
    ap.add_argument("--hetero-sparsity", default="50,60,70,80", help="sparsities of --hetero, in percent")
    ap.add_argument("--hetero-n", default="8,16,32,64", help="token counts of --hetero")
    ap.add_argument("--hetero-iters", type=int, default=200)
    ap.add_argument("--hetero-residual-split-k", type=int, default=0,
                    help="Split_K of the residual's Tiled-CSL kernel (0 = the planner's choice for the whole matrix)")
    args = ap.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1).", file=sys.stderr)
        sys.exit(2)
    if args.hetero:
        hetero_mode(args)
        return

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
    split_k = args.split_k  # 0: chosen below, once the weight's size is known

    # ---- synthetic inputs (host), encode (host), upload
    t0 = time.perf_counter()
    A = G.synth_weights(M, K, sparsity, skew, seed=1234)
    B = G.synth_activations(N, K, seed=4321)
    t_synth = time.perf_counter() - t0
    t0 = time.perf_counter()
    items, offsets = (G.InitSparseMatrixA_API_NoReorder if args.no_reorder else G.InitSparseMatrixA_API)(A)
    t_encode = time.perf_counter() - t0
    a_bytes = 16 * int(offsets[-1])
    split_k = split_k or G.SpMM_SuggestSplitK_Bytes(M, N, K, a_bytes // 16)
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

    # ---- settle the clocks: the same call, untimed, for a fixed wall time whatever --warmup says
    # (after an idle spell this GPU needs some 10 ms of continuous launches to reach its clocks)
    prewarm_launches, prewarm_spent, settle_blocks = settle(lib, sptr, step, torch, args.prewarm_seconds,
                                                            adaptive=not args.no_settle)

    # ---- the main kernel alone, live: back-to-back launches of it (no reduction in between)
    # bracketed by two HIP events recorded on the launch stream, straight after the pre-warm; the
    # average includes the dispatch gap between consecutive kernels but no per-launch event
    # overhead.  --repeats x K launches between ONE pair of events: recording an event between two
    # kernels costs the stream a few microseconds, which at K = 20 would add 1-2 % to every block
    # timed on its own.
    def partials(i):
        rc = lib.SpMM_SplitK_Partials(sptr, p_items[i % copies], p_offs[i % copies], p_B, p_W, M, N, K, split_k)
        if rc:
            raise RuntimeError(f"SpMM_SplitK_Partials -> {rc}")

    for i in range(200):
        partials(i)
    kernel_launches = args.steps * max(1, args.repeats)
    kernel_ms_avg = events_ms(lib, sptr, partials, kernel_launches) / kernel_launches

    # ---- timed region: W warm-up steps, then exactly K steps between synchronisations; that
    # block is timed --repeats times (each with its own synchronisations) and the median reported
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    blocks_ms = []
    for r in range(max(1, args.repeats)):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            step(i)
        torch.cuda.synchronize()
        blocks_ms.append((time.perf_counter() - t0) * 1e3)
    ms_per_step = float(np.median(blocks_ms)) / args.steps

    for i in range(args.calibration_copies):
        src, dst = d_items[i % copies], d_items[(i + 1) % copies]  # all copies hold the same bytes
        rc = lib.SpMM_CalibrationCopy(sptr, ctypes.c_void_p(dst.data_ptr()), ctypes.c_void_p(src.data_ptr()), a_bytes)
        if rc:
            raise RuntimeError(f"SpMM_CalibrationCopy -> {rc}")
    torch.cuda.synchronize()

    flops = 2.0 * M * N * K
    tflops = flops / (ms_per_step * 1e-3) / 1e12
    kernel_gbps = a_bytes / (kernel_ms_avg * 1e-3) / 1e9
    default_workload = (args.workload == "opt30b_ffn1" and N == 16 and sparsity == 0.8 and not skew)
    out = {
        "metric": ("SpMM eff. TFLOPS + HBM GB/s (% roofline), OPT-30B FFN1 80% sparse, N=16" if default_workload else
                   f"SpMM eff. TFLOPS + HBM GB/s (% roofline), {args.workload} {sparsity * 100:.0f}% sparse"
                   f"{' (row-skewed)' if skew else ''}, N={N}"),
        "value": tflops,
        "unit": "TFLOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "timing": {"repeats": len(blocks_ms), "statistic": "median of the timed blocks of --steps steps",
                   "block_ms_min": float(min(blocks_ms)), "block_ms_max": float(max(blocks_ms)),
                   "prewarm_launches": prewarm_launches, "prewarm_seconds": args.prewarm_seconds,
                   "prewarm_seconds_spent": prewarm_spent,
                   "settle_blocks_us": {"launches_per_block": SETTLE_BLOCK, "first": settle_blocks[0] if settle_blocks else None,
                                        "fastest": min(settle_blocks) if settle_blocks else None,
                                        "last": settle_blocks[-1] if settle_blocks else None, "count": len(settle_blocks)}},
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
            "traffic": measured_traffic(args.workload, N, split_k, sparsity, skew)[0],
            "traffic_source": TRAFFIC_SOURCE,
            "traffic_profile": measured_traffic(args.workload, N, split_k, sparsity, skew)[1],
            "kernel": "tcsl_spmm_kernel",
            "kernel_ms_avg": kernel_ms_avg,
            "kernel_launches_timed": kernel_launches,
            "algorithmic_bytes_per_launch": a_bytes,
        },
        "check": check,
        "host_prep_s": {"synth": t_synth, "encode": t_encode, "upload": t_upload},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(A, B, M, N, K)
    if not args.no_sweep:
        del d_items, d_offs, p_items, p_offs
        torch.cuda.empty_cache()
        out["sweep"] = sweep(G, lib, torch, dev, sptr, with_stack=not args.no_stack)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
