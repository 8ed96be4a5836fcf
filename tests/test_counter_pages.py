"""Host logic that hands out the arrival-counter pages of the in-launch split-K reduction
(graphneuralnetproj_amd/csrc/counter_pages.cpp), driven on the CPU with made-up stream handles.

The rule under test: two launches that may overlap in time never count on the same page."""
import ctypes
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def cp(tmp_path_factory):
    out = tmp_path_factory.mktemp("cp") / "libcounter_pages_test.so"
    subprocess.run(["g++", "-std=c++17", "-O1", "-fPIC", "-shared", "-pthread", "-o", str(out),
                    os.path.join(ROOT, "tests", "support", "counter_pages_shim.cpp"),
                    os.path.join(ROOT, "graphneuralnetproj_amd", "csrc", "counter_pages.cpp")], check=True)
    lib = ctypes.CDLL(str(out))
    lib.cp_new.restype = ctypes.c_void_p
    lib.cp_delete.argtypes = [ctypes.c_void_p]
    lib.cp_set_busy.argtypes = [ctypes.c_ulong, ctypes.c_int]
    lib.cp_acquire.argtypes = [ctypes.c_void_p, ctypes.c_ulong, ctypes.c_int, ctypes.c_ulonglong]
    lib.cp_eager_in_use.argtypes = [ctypes.c_void_p]
    lib.cp_capture_in_use.argtypes = [ctypes.c_void_p]
    lib.cp_recycled.argtypes = [ctypes.c_int]
    return lib


@pytest.fixture
def pages(cp):
    p = cp.cp_new()
    yield p
    cp.cp_delete(p)


def stream(i):
    return 0x1000 + 0x40 * i


def test_one_page_per_stream_and_stable(cp, pages):
    E = cp.cp_eager_pages()
    got = [cp.cp_acquire(pages, stream(i), 0, 0) for i in range(E)]
    assert sorted(got) == list(range(E))                      # all different
    assert [cp.cp_acquire(pages, stream(i), 0, 0) for i in range(E)] == got   # and kept
    assert cp.cp_eager_in_use(pages) == E


def test_exhaustion_with_busy_streams_gives_no_page(cp, pages):
    E = cp.cp_eager_pages()
    for i in range(E):
        cp.cp_set_busy(stream(i), 1)
        cp.cp_acquire(pages, stream(i), 0, 0)
    try:
        assert cp.cp_acquire(pages, stream(E), 0, 0) == -1    # every owner is still running: fall back
        assert cp.cp_acquire(pages, stream(3), 0, 0) >= 0     # owners are unaffected
    finally:
        for i in range(E):
            cp.cp_set_busy(stream(i), 0)


def test_first_streams_keep_their_pages_for_good(cp, pages):
    """The pages of the first streams never change hands (no event is recorded behind their
    launches, so nobody could tell when they are idle); only the later, recycled pages do."""
    E, P = cp.cp_eager_pages(), cp.cp_permanent_pages()
    first = [cp.cp_acquire(pages, stream(i), 0, 0) for i in range(E)]
    assert [cp.cp_recycled(p) for p in first] == [0] * P + [1] * (E - P)
    for i in range(20 * E):                                   # a crowd of newcomers, everybody idle
        assert cp.cp_recycled(cp.cp_acquire(pages, stream(1000 + i), 0, 0)) == 1
    assert [cp.cp_acquire(pages, stream(i), 0, 0) for i in range(P)] == first[:P]


def test_idle_least_recently_used_page_changes_hands(cp, pages):
    E, P = cp.cp_eager_pages(), cp.cp_permanent_pages()
    first = [cp.cp_acquire(pages, stream(i), 0, 0) for i in range(E)]
    cp.cp_acquire(pages, stream(P), 0, 0)                     # the first recycled page's owner is now the most recent user
    cp.cp_set_busy(stream(P + 1), 1)                          # the oldest remaining one is busy ...
    try:
        p = cp.cp_acquire(pages, stream(E), 0, 0)
        assert p == first[P + 2]                              # ... so the next oldest idle one gives way
        # the evicted stream comes back: it must not get the page its successor now counts on
        cp.cp_set_busy(stream(E), 1)
        q = cp.cp_acquire(pages, stream(P + 2), 0, 0)
        assert q != p and q >= 0
    finally:
        cp.cp_set_busy(stream(P + 1), 0)
        cp.cp_set_busy(stream(E), 0)


def test_many_short_lived_streams_always_get_a_page(cp, pages):
    """A process that keeps making and destroying streams (every launch finished when the next
    stream appears) never falls off the fused path."""
    E = cp.cp_eager_pages()
    for i in range(10 * E):
        assert 0 <= cp.cp_acquire(pages, stream(i), 0, 0) < E


def test_eviction_looks_at_a_bounded_number_of_pages(cp, pages):
    E, P, T = cp.cp_eager_pages(), cp.cp_permanent_pages(), cp.cp_eviction_tries()
    for i in range(E):
        cp.cp_acquire(pages, stream(i), 0, 0)
    for i in range(P, P + T):                                 # the T oldest recycled pages are busy, the rest idle
        cp.cp_set_busy(stream(i), 1)
    try:
        assert cp.cp_acquire(pages, stream(E), 0, 0) == -1
        cp.cp_set_busy(stream(P + T - 1), 0)
        assert cp.cp_acquire(pages, stream(E), 0, 0) >= 0
    finally:
        for i in range(P, P + T):
            cp.cp_set_busy(stream(i), 0)


def test_captures_have_their_own_pages_for_good(cp, pages):
    E, C = cp.cp_eager_pages(), cp.cp_capture_pages()
    s = stream(7)
    eager = cp.cp_acquire(pages, s, 0, 0)
    a = cp.cp_acquire(pages, s, 1, 11)                        # the same stream, recording
    b = cp.cp_acquire(pages, s, 1, 12)                        # a later capture on it
    c = cp.cp_acquire(pages, stream(8), 1, 11)                # a forked stream of capture 11
    assert len({eager, a, b, c}) == 4 and min(a, b, c) >= E
    assert cp.cp_acquire(pages, s, 1, 11) == a                # calls of one capture on one stream are ordered
    # eager traffic, however heavy, never takes a capture's page
    for i in range(5 * E):
        assert cp.cp_acquire(pages, stream(100 + i), 0, 0) < E
    assert cp.cp_acquire(pages, s, 1, 11) == a
    # capture pages run out, they are never recycled
    for i in range(C - 3):
        assert cp.cp_acquire(pages, s, 1, 1000 + i) >= E
    assert cp.cp_capture_in_use(pages) == C
    assert cp.cp_acquire(pages, s, 1, 5000) == -1
    assert cp.cp_acquire(pages, s, 1, 12) == b


def test_per_thread_default_stream_is_one_stream_per_host_thread(cp, pages):
    """hipStreamPerThread is a single handle value that names a different stream in every host
    thread: launches from two threads may overlap, so they must not count on one page, while an
    ordinary handle is the same stream whoever launches on it."""
    import threading

    cp.cp_per_thread_handle.restype = ctypes.c_ulong
    h = cp.cp_per_thread_handle()
    got = {}
    gate = threading.Barrier(3)  # all three threads alive at once: their thread-local storage is distinct

    def worker(name):
        first = cp.cp_acquire(pages, h, 0, 0)
        gate.wait()
        got[name] = (first, cp.cp_acquire(pages, h, 0, 0), cp.cp_acquire(pages, stream(5), 0, 0),
                     cp.cp_acquire(pages, h, 1, 77))
        gate.wait()

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(3)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    firsts = [got[i][0] for i in range(3)]
    assert len(set(firsts)) == 3 and min(firsts) >= 0          # one page per calling thread
    assert all(got[i][1] == got[i][0] for i in range(3))       # and the thread keeps it
    assert len({got[i][2] for i in range(3)}) == 1             # an ordinary handle: one stream, one page
    captures = [got[i][3] for i in range(3)]                   # captures on it are per thread as well
    assert len(set(captures)) == 3 and min(captures) >= cp.cp_eager_pages()
    # the main thread's per-thread stream is yet another one
    assert cp.cp_acquire(pages, h, 0, 0) not in firsts
