"""The build-time verifier of the kernels' hand-managed loads, on synthetic gfx950 assembly.

Each snippet is a tiny kernel body; the checker must accept the ones that wait before
touching a loaded register and flag the ones that do not (straight-line, across a branch
join, and around a loop back edge).
"""
import importlib.util
import os
import subprocess
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CHECKER = os.path.join(HERE, "..", "graphneuralnetproj_amd", "csrc", "check_async_loads.py")

spec = importlib.util.spec_from_file_location("check_async_loads", CHECKER)
chk = importlib.util.module_from_spec(spec)
spec.loader.exec_module(chk)


def kernel(body, name="_Z16tcsl_spmm_kernelv", scratch=0):
    return f"""
	.amdhsa_kernel {name}
		.amdhsa_private_segment_fixed_size {scratch}
	.end_amdhsa_kernel
{name}:
{body}
	s_endpgm
.Lfunc_end0:
"""


def violations(body):
    text = kernel(body)
    found = list(chk.split_kernels(text.splitlines()))
    assert len(found) == 1
    return chk.check_kernel(*found[0])


def test_wait_before_use_is_clean():
    rep = violations("""
	buffer_load_dwordx4 v[4:7], v1, s[0:3], 0 offen
	buffer_load_dwordx4 v[8:11], v1, s[0:3], 0 offen offset:1024
	s_waitcnt vmcnt(1)
	v_add_u32 v20, v4, v5
	s_waitcnt vmcnt(0)
	v_add_u32 v21, v8, v9
""")
    assert rep == []


def test_use_without_wait_is_flagged():
    rep = violations("""
	buffer_load_dwordx4 v[4:7], v1, s[0:3], 0 offen
	v_add_u32 v20, v4, v5
""")
    assert len(rep) == 1 and rep[0][3] == [4, 5]


def test_partial_wait_covers_only_the_oldest_loads():
    rep = violations("""
	buffer_load_dwordx4 v[4:7], v1, s[0:3], 0 offen
	buffer_load_dwordx4 v[8:11], v1, s[0:3], 0 offen offset:1024
	s_waitcnt vmcnt(1)
	v_mov_b32 v8, 0
""")
    assert len(rep) == 1 and rep[0][3] == [8]  # a write into an in-flight destination counts too


def test_lgkm_wait_does_not_release_vector_loads():
    rep = violations("""
	global_load_dwordx4 v[4:7], v[2:3], off
	s_waitcnt lgkmcnt(0)
	ds_write_b16 v30, v4
""")
    assert len(rep) == 1


def test_join_takes_the_union_of_both_paths():
    # one arm waits, the other does not: after the join the load may still be in flight
    rep = violations("""
	buffer_load_dwordx4 v[4:7], v1, s[0:3], 0 offen
	s_cbranch_scc1 .LBB0_2
	s_waitcnt vmcnt(0)
.LBB0_2:
	v_add_u32 v20, v4, v4
""")
    assert len(rep) == 1
    rep = violations("""
	buffer_load_dwordx4 v[4:7], v1, s[0:3], 0 offen
	s_cbranch_scc1 .LBB0_2
	s_waitcnt vmcnt(0)
	s_branch .LBB0_3
.LBB0_2:
	s_waitcnt vmcnt(0)
.LBB0_3:
	v_add_u32 v20, v4, v4
""")
    assert rep == []


def test_loop_back_edge_carries_loads_into_the_next_iteration():
    # the load at the bottom of the loop is still in flight when the top runs again
    rep = violations("""
	buffer_load_dwordx4 v[4:7], v1, s[0:3], 0 offen
	s_waitcnt vmcnt(0)
.LBB0_1:
	v_add_u32 v20, v4, v4
	buffer_load_dwordx4 v[4:7], v1, s[0:3], 0 offen
	s_cbranch_scc1 .LBB0_1
	s_waitcnt vmcnt(0)
""")
    assert len(rep) == 1
    rep = violations("""
	buffer_load_dwordx4 v[4:7], v1, s[0:3], 0 offen
.LBB0_1:
	s_waitcnt vmcnt(0)
	v_add_u32 v20, v4, v4
	buffer_load_dwordx4 v[4:7], v1, s[0:3], 0 offen
	s_cbranch_scc1 .LBB0_1
	s_waitcnt vmcnt(0)
""")
    assert rep == []


def test_stores_occupy_queue_slots():
    # vmcnt counts stores as well: with a store issued after the load, vmcnt(1) releases the load
    rep = violations("""
	buffer_load_dwordx4 v[4:7], v1, s[0:3], 0 offen
	global_store_dwordx4 v[2:3], v[12:15], off
	s_waitcnt vmcnt(1)
	v_add_u32 v20, v4, v4
""")
    assert rep == []


def test_command_line_flags_scratch_and_violations(tmp_path):
    good = tmp_path / "good.s"
    good.write_text(kernel("\tbuffer_load_dwordx4 v[4:7], v1, s[0:3], 0 offen\n\ts_waitcnt vmcnt(0)\n\tv_mov_b32 v9, v4\n"))
    spill = tmp_path / "spill.s"
    spill.write_text(kernel("\tv_mov_b32 v9, v4\n", scratch=92))
    bad = tmp_path / "bad.s"
    bad.write_text(kernel("\tbuffer_load_dwordx4 v[4:7], v1, s[0:3], 0 offen\n\tv_mov_b32 v9, v4\n"))
    run = lambda p: subprocess.run([sys.executable, CHECKER, str(p), "tcsl_spmm_kernel"], capture_output=True, text=True)
    assert run(good).returncode == 0
    r = run(spill)
    assert r.returncode == 1 and "scratch" in r.stdout
    r = run(bad)
    assert r.returncode == 1 and "in flight" in r.stdout
    other = tmp_path / "other.s"
    other.write_text(kernel("\tv_mov_b32 v9, v4\n", name="_Z5otherv"))
    assert run(other).returncode == 2  # nothing matched: a renamed kernel must not pass silently


def test_built_kernels_pass():
    asm = os.path.join(HERE, "..", "graphneuralnetproj_amd", "csrc", "obj", "spmm_kernels.gfx950.s")
    if not os.path.exists(asm):
        pytest.skip("library not built in this tree")
    r = subprocess.run([sys.executable, CHECKER, asm, "tcsl_spmm_kernel"], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout
    assert r.stdout.count("ok ") >= 10


def test_built_sparse_mfma_kernels_pass():
    """The 2:4 kernel that issues its loads from inline assembly: every instantiation in the launch table."""
    asm = os.path.join(HERE, "..", "graphneuralnetproj_amd", "csrc", "obj", "a24_kernels.gfx950.s")
    if not os.path.exists(asm):
        pytest.skip("library not built in this tree")
    r = subprocess.run([sys.executable, CHECKER, asm, "a24_spmm_shared_b_kernel"], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout
    # column-major: 2 + 5 + 5 launch shapes for 64, 32 and up to 16 tokens, and 9 + 10 + 10 that take the residual along;
    # row-major (two row blocks per wave only): 2 + 2 + 2 and 8 + 10 + 10
    assert r.stdout.count("ok ") == 41 + 34
