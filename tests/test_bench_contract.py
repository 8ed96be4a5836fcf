"""Host-side contract of bench.py that needs no GPU: one GPU only, the sweep covers what the
benchmark's configurations name, and every traffic figure points at a profile summary that exists."""
import importlib.util
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2 and "one GPU" in r.stderr and r.stdout == ""


def test_sweep_covers_the_named_configurations():
    B = _bench()
    cases = B.sweep_cases()
    labels = [c[0] for c in cases]
    assert len(labels) == len(set(labels))
    assert all(c[1] in B.WORKLOADS for c in cases)
    have = {(c[1], c[2], c[3], c[4], c[5]) for c in cases}
    # attention projections: Split_K in {1, 2, 4, 7} x N in {8, 16, 32}, and the planner's own choice
    for w in ("opt30b_qkv", "opt30b_outproj"):
        for n in (8, 16, 32):
            assert (w, n, 0.8, False, 0) in have
            for s in (1, 2, 4, 7):
                assert (w, n, 0.8, False, s) in have
    # feed-forward: N, sparsity and skew on FFN1, FFN2 at 16 and 64 tokens, both operand layouts
    for n in (8, 32, 64):
        assert ("opt30b_ffn1", n, 0.8, False, 0) in have
    for sp, skew in ((0.7, False), (0.9, False), (0.8, True)):
        assert ("opt30b_ffn1", 16, sp, skew, 0) in have
    assert ("opt30b_ffn2", 16, 0.8, False, 0) in have and ("opt30b_ffn2", 64, 0.8, False, 0) in have
    assert sum(1 for label in labels if label.endswith("_row_major")) >= 2
    # OPT-66B and the OPT-175B shapes of the reference's sweep (kernel_benchmark/benchmark.sh:13-14)
    for model in ("opt66b", "opt175b"):
        for name in ("qkv", "outproj", "ffn1", "ffn2"):
            for n in (8, 16, 32):
                assert (f"{model}_{name}", n, 0.8, False, 0) in have
    assert B.WORKLOADS["opt175b_ffn1"][:2] == (49152, 12288) and B.WORKLOADS["opt175b_ffn2"][:2] == (12288, 49152)
    # cases that share a weight are adjacent (one weight resident at a time)
    seen, last = set(), None
    for c in cases:
        key = (c[1], c[3], c[4])
        if key != last:
            assert key not in seen, key
            seen.add(key)
            last = key


def test_traffic_figures_name_existing_profiles():
    B = _bench()
    assert B.measured_traffic("opt30b_ffn1", 16, 1, 0.8, False)[0] == 168.70e6
    assert B.measured_traffic("opt30b_ffn1", 16, 1, 0.8, True) == (None, None)
    assert B.measured_traffic("opt30b_ffn1", 16, 3, 0.8, False) == (None, None)
    for (workload, n, split_k, sparsity), (nbytes, profile) in B.MEASURED_TRAFFIC_BYTES.items():
        assert workload in B.WORKLOADS and nbytes > 0
        assert os.path.exists(os.path.join(ROOT, profile)), profile
