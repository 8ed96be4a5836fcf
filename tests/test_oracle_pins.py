"""Pins the CPU oracle itself (it is the checker for everything else).

Each oracle function is checked against something that does not restate its
formula: the committed golden vectors produced by the reference's own encoder,
hand-derived encodings, format invariants, numpy's float16/float64 arithmetic,
and brute force.
"""
import json
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def small_golden():
    z = np.load(os.path.join(GOLD, "encoder_small.npz"))
    names = sorted({k.rsplit(".", 1)[0] for k in z.files})
    return [(n, z[n + ".A"], z[n + ".items"], z[n + ".offsets"]) for n in names]


def kept_mask(bits):
    mag = bits & 0x7FFF
    return (mag != 0) & (mag <= 0x7C00)


# ----------------------------------------------------------------- fp16 ---

def test_half_to_float_exhaustive(oracle):
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([oracle.lib().oracle_half_to_float(int(x)) for x in h], dtype=np.float32)
    same = (want.view(np.uint32) == got.view(np.uint32)) | (np.isnan(want) & np.isnan(got))
    assert same.all()


def test_float_to_half_rn_against_numpy(oracle):
    rng = np.random.default_rng(1)
    h = np.arange(65536, dtype=np.uint16)
    finite = h.view(np.float16)[np.isfinite(h.view(np.float16))].astype(np.float32)
    xs = [rng.standard_normal(20000).astype(np.float32) * s for s in (1e-8, 6e-8, 1e-6, 1e-4, 0.02, 1, 100, 6e4)]
    xs += [finite, np.nextafter(finite, np.float32(np.inf)), np.nextafter(finite, np.float32(-np.inf))]
    # exact midpoints between neighbouring halves: ties must go to even
    lo = h[(h & 0x7FFF) < 0x7BFF]
    mid = ((lo.view(np.float16).astype(np.float64) + (lo + 1).astype(np.uint16).view(np.float16).astype(np.float64)) / 2)
    xs.append(mid.astype(np.float32))
    x = np.concatenate(xs)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = np.array([oracle.lib().oracle_float_to_half_rn(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(want, got)


# -------------------------------------------------------------- encoder ---

@pytest.mark.parametrize("name,A,items,offsets", small_golden(), ids=[c[0] for c in small_golden()])
def test_encode_matches_reference_golden(oracle, name, A, items, offsets):
    got_items, got_offsets = oracle.encode(A)
    assert np.array_equal(got_offsets, offsets)
    assert np.array_equal(got_items, items)


def test_encode_matches_reference_golden_large(oracle, spmm):
    import hashlib

    with open(os.path.join(GOLD, "encoder_large.json")) as f:
        cases = json.load(f)
    for c in cases:
        A = spmm.synth_weights(c["M"], c["K"], c["sparsity"], c["row_skewed"], seed=c["seed"])
        assert hashlib.sha256(A.tobytes()).hexdigest() == c["input_sha256"], "input generator drifted"
        items, offs = oracle.encode(A)
        assert len(items) == c["words"] and len(offs) == c["num_offsets"]
        assert hashlib.sha256(items.tobytes()).hexdigest() == c["items_sha256"]
        assert hashlib.sha256(offs.tobytes()).hexdigest() == c["offsets_sha256"]


def test_encode_against_live_reference_build(oracle, spmm):
    """Where oracle/_ref was built, compare directly on fresh random inputs."""
    if not oracle.have_ref():
        pytest.skip("oracle/_ref not built here (needs the reference checkout)")
    for seed, (M, K, s, skew) in enumerate([(256, 320, 0.8, False), (384, 128, 0.6, True), (128, 640, 0.95, False)]):
        A = spmm.synth_weights(M, K, s, skew, seed=100 + seed)
        it, of = oracle.encode(A)
        rit, rof = oracle.ref_encode(A)
        assert np.array_equal(it, rit) and np.array_equal(of, rof)


def test_single_nonzero_hand_derived(oracle):
    """One element at (37, 21): swizzled column 21 ^ (5 << 3) = 61, bank 30,
    position 37*64 + 61 = 2429.  Three pads go to the smallest banks 0, 1, 2 at
    their first zero positions 0, 2, 4; one lane draws them largest-bank-first
    (banks 0, 1, 2, 30) and emits in reverse."""
    A = np.zeros((128, 64), dtype=np.uint16)
    A[37, 21] = 0x3C00
    items, offs = oracle.encode(A)
    assert offs.tolist() == [0, 1, 1]
    assert items.tolist() == [0x3C00 | (2429 << 16), 4 << 16, 2 << 16, 0]


def test_dense_tile_closed_form(oracle):
    """A full tile has 256 words per bank and no padding; lane b of round r ends
    up with bank b's words 4r..4r+3 in scan order, i.e. word v of vector (r, b)
    sits at swizzled position (2r + v//2)*64 + 2b + v%2."""
    rng = np.random.default_rng(2)
    A = rng.integers(1, 0x7C00, size=(128, 64), dtype=np.uint16)
    items, offs = oracle.encode(A)
    assert offs.tolist() == [0, 2048, 2048]
    r, b, v = np.meshgrid(np.arange(64), np.arange(32), np.arange(4), indexing="ij")
    m = 2 * r + v // 2
    swz = 2 * b + v % 2
    n = swz ^ ((m % 8) << 3)
    want = A[m, n].astype(np.uint32) | ((m * 64 + swz).astype(np.uint32) << 16)
    assert np.array_equal(items, want.reshape(-1))


@pytest.mark.parametrize("extra", [4, 8])
def test_full_round_plus_tail_hand_derived(oracle, spmm, extra):
    """A tile with one full round of 32 vectors AND a tail (R = 1, Rem = 1 or 2), worked out by hand
    from csrc/SpMM_API.cu:379-424.  Rows 0 and 8 are full (row % 8 == 0: no swizzle, column n sits in
    bank n / 2), so every bank stacks [r0 c2b, r0 c2b+1, r8 c2b, r8 c2b+1]; row 16 adds columns
    0 .. extra-1, two more words on top of banks 0 .. extra/2-1.  No padding (132 or 136 words).
      Tail first (:384-391), v outer, b inner, always the fullest stack, lowest bank on ties:
        extra = 4: b0 b1 b0 b1 give (16,1) (16,3) (16,0) (16,2), all to Tail[0];
        extra = 8: b0 b1 b2 b3 b0 b1 b2 b3 give (16,1) (16,3) (16,5) (16,7) (16,0) (16,2) (16,4) (16,6),
                   dealt alternately to Tail[0] and Tail[1].
      Then the round (:394-403): all stacks hold 4, so each of its four passes pops banks 0 .. 31 in
      order and Main[b] = bank b's words from the top down.
      Emitted last in, first out (:406-424): vector b of the round = bank b's words in scan order,
      tail vector b = Tail[b] reversed.
    Drawing the round before the tail, popping first in first out, or breaking ties upwards each
    gives another order."""
    A = np.zeros((128, 64), dtype=np.uint16)
    value = lambda m, n: 0x3C00 + m * 64 + n + 1  # distinct, non-zero, finite
    for m, cols in ((0, 64), (8, 64), (16, extra)):
        for n in range(cols):
            A[m, n] = value(m, n)
    word = lambda m, n: value(m, n) | ((m * 64 + n) << 16)  # rows 0, 8, 16: position = m * 64 + n
    want = []
    for b in range(32):
        want += [word(0, 2 * b), word(0, 2 * b + 1), word(8, 2 * b), word(8, 2 * b + 1)]
    if extra == 4:
        want += [word(16, 2), word(16, 0), word(16, 3), word(16, 1)]
    else:
        want += [word(16, 4), word(16, 0), word(16, 5), word(16, 1), word(16, 6), word(16, 2), word(16, 7), word(16, 3)]
    for encode in (oracle.encode, spmm.InitSparseMatrixA_API):
        items, offs = encode(A.view(np.float16) if encode is spmm.InitSparseMatrixA_API else A)
        assert offs.tolist() == [0, len(want) // 4, len(want) // 4]
        assert items.tolist() == want


def test_encode_rejects_bad_shapes(oracle):
    for M, K in [(100, 64), (128, 96), (64, 64), (128, 32)]:
        with pytest.raises(ValueError):
            oracle.encode(np.zeros((M, K), dtype=np.uint16))


@pytest.mark.parametrize("M,K,sparsity,skew", [(256, 256, 0.8, False), (128, 512, 0.5, True), (384, 64, 0.97, False),
                                               (128, 64, 0.0, False)])
def test_format_invariants(oracle, spmm, M, K, sparsity, skew):
    A = spmm.synth_weights(M, K, sparsity, skew, seed=7).view(np.uint16)
    items, offs = oracle.encode(A)
    tr, tc = M // 128, K // 64
    assert len(offs) == tr * tc + 2 and offs[0] == 0 and offs[-1] == offs[-2]
    assert (np.diff(offs) >= 0).all() and len(items) == 4 * offs[-1]
    for t in range(tr * tc):
        i, j = divmod(t, tc)
        tile = A[i * 128:(i + 1) * 128, j * 64:(j + 1) * 64]
        w = items[4 * offs[t]:4 * offs[t + 1]]
        nnz = int(kept_mask(tile).sum())
        assert len(w) == (nnz + 3) // 4 * 4            # padded to a multiple of 4, fewer than 4 pads
        val, pos = (w & 0xFFFF).astype(np.uint16), (w >> 16).astype(np.int64)
        assert (pos < 8192).all()
        row, col = pos >> 6, (pos & 63) ^ (((pos >> 6) & 7) << 3)
        real = val != 0
        assert real.sum() == nnz
        assert len(np.unique(pos[real])) == nnz        # distinct positions
        assert np.array_equal(tile[row[real], col[real]], val[real])
        assert (~kept_mask(tile[row[~real], col[~real]])).all()  # pads only where A is zero


def test_decode_is_inverse(oracle, spmm):
    A = spmm.synth_weights(256, 192, 0.75, True, seed=9).view(np.uint16).copy()
    A[3, 5] = 0x8000  # -0 is dropped and comes back as +0
    A[4, 6] = 0x7E00  # NaN is dropped too (the reference's > 0 test)
    items, offs = oracle.encode(A)
    back = oracle.decode(items, offs, 256, 192).view(np.uint16)
    want = np.where(kept_mask(A), A, 0)
    assert np.array_equal(back, want)


def test_decode_hand_position(oracle):
    """Independent of the encoder: a word with index r*64 + (c ^ ((r%8)<<3)) lands at (r, c)."""
    r, c = 77, 13
    word = np.array([0x4200 | ((r * 64 + (c ^ ((r % 8) << 3))) << 16), 0, 0, 0], dtype=np.uint32)
    offs = np.array([0, 0, 1, 1], dtype=np.int32)  # second tile of a 128 x 128 matrix
    D = oracle.decode(word, offs, 128, 128).view(np.uint16)
    assert D[r, 64 + c] == 0x4200 and np.count_nonzero(D) == 1


# ----------------------------------------------------------------- GEMM ---

def test_gemm_exact_small_integers(oracle):
    """Products and sums of small integers are exact in fp32, so the fp32 loop must
    equal numpy's float64 result bit for bit; a transposed operand, a dropped
    term or a wrong stride fails."""
    rng = np.random.default_rng(3)
    M, K, N = 96, 160, 5
    A = rng.integers(-4, 5, size=(M, K)).astype(np.float16)
    B = rng.integers(-5, 6, size=(N, K)).astype(np.float16)
    C = oracle.gemm_f32(A, B)
    want = (B.astype(np.float64) @ A.astype(np.float64).T)
    assert C.shape == (N, M) and np.array_equal(C.astype(np.float64), want)
    # one-hot activations pick columns of A
    ks = [7, 0, 159]
    E = np.zeros((3, K), dtype=np.float16)
    E[np.arange(3), ks] = 1
    assert np.array_equal(oracle.gemm_f32(A, E), A[:, ks].T.astype(np.float32))


def test_gemm_close_to_float64_on_random(oracle, spmm):
    A = spmm.synth_weights(128, 1024, 0.8, False, seed=4)
    B = spmm.synth_activations(8, 1024, seed=5)
    C = oracle.gemm_f32(A, B)
    want = B.astype(np.float64) @ A.astype(np.float64).T
    assert np.abs(C - want).max() < 1e-5


def test_gemm_k_range(oracle):
    rng = np.random.default_rng(6)
    A = rng.integers(-3, 4, size=(32, 256)).astype(np.float16)
    B = rng.integers(-3, 4, size=(4, 256)).astype(np.float16)
    part = oracle.gemm_f32(A, B, 64, 192)
    want = B[:, 64:192].astype(np.float64) @ A[:, 64:192].astype(np.float64).T
    assert np.array_equal(part.astype(np.float64), want)


# -------------------------------------------------------------- split-K ---

@pytest.mark.parametrize("K", [64, 576, 1024, 7168, 9216, 28672, 36864])
def test_splitk_ranges_partition_the_tiles(oracle, K):
    nkb = K // 64
    for split_k in range(1, 13):
        avg = -(-nkb // split_k)
        covered = []
        for b in range(split_k):
            s, e = oracle.splitk_range(K, split_k, b)
            assert 0 <= s <= e <= nkb and e - s <= avg
            covered += list(range(s, e))
        assert covered == list(range(nkb))
        # where the reference's own arithmetic is well defined it agrees:
        # batch b starts at b*avg and all but the last hold avg tiles
        if avg * (split_k - 1) < nkb:
            for b in range(split_k - 1):
                assert oracle.splitk_range(K, split_k, b) == (b * avg, (b + 1) * avg)
            assert oracle.splitk_range(K, split_k, split_k - 1) == (avg * (split_k - 1), nkb)


def test_reduce_closed_form(oracle):
    rng = np.random.default_rng(8)
    W = (rng.standard_normal((5, 1024)) * 3).astype(np.float16)
    C = oracle.reduce(W, 1024, 5)
    want = W.astype(np.float64).sum(axis=0)  # fp32 sums of five halves are exact in float64 too
    assert np.array_equal(C, want.astype(np.float32).astype(np.float16))
    # order matters only through fp32 rounding; with exact inputs the result is exact
    Wi = rng.integers(-100, 100, size=(7, 256)).astype(np.float16)
    assert np.array_equal(oracle.reduce(Wi, 256, 7).astype(np.float64), Wi.astype(np.float64).sum(axis=0))


def test_spmm_splitk_slabs_sum_to_full_product(oracle):
    """Integer data: every slab and the reduction are exact, so slabs must add up
    to the full product and C must equal it, for even and uneven splits."""
    rng = np.random.default_rng(10)
    M, K, N = 128, 576, 8
    A = (rng.integers(-3, 4, size=(M, K)) * (rng.random((M, K)) < 0.3)).astype(np.float16)
    B = rng.integers(-3, 4, size=(N, K)).astype(np.float16)
    items, offs = oracle.encode(A)
    full = (B.astype(np.float64) @ A.astype(np.float64).T)
    for split_k in (1, 2, 4, 9, 11):
        C, W = oracle.spmm_splitk(items, offs, B, M, N, K, split_k)
        assert np.array_equal(C.astype(np.float64), full)
        if split_k > 1:
            assert np.array_equal(W.astype(np.float64).sum(axis=0), full)
            s, e = oracle.splitk_range(K, split_k, 1)
            part = B[:, s * 64:e * 64].astype(np.float64) @ A[:, s * 64:e * 64].astype(np.float64).T
            assert np.array_equal(W[1].astype(np.float64), part)


# ------------------------------------------------- encoder, no reordering ---

def test_noreorder_encode_matches_reference_golden(oracle, spmm):
    import hashlib

    z = np.load(os.path.join(GOLD, "encoder_small.npz"))
    names = sorted({k.rsplit(".", 1)[0] for k in z.files})
    for n in names:
        items, offs = oracle.encode_noreorder(z[n + ".A"])
        assert np.array_equal(offs, z[n + ".offsets"]), n
        assert np.array_equal(items, z[n + ".items_noreorder"]), n
    with open(os.path.join(GOLD, "encoder_large.json")) as f:
        cases = json.load(f)
    for c in cases:
        A = spmm.synth_weights(c["M"], c["K"], c["sparsity"], c["row_skewed"], seed=c["seed"])
        items, offs = oracle.encode_noreorder(A)
        assert hashlib.sha256(items.tobytes()).hexdigest() == c["items_noreorder_sha256"]
        assert hashlib.sha256(offs.tobytes()).hexdigest() == c["offsets_sha256"]


def test_noreorder_hand_derived(oracle):
    """Scan order, and pads = the first elements of the scan that are not kept, with their own bits."""
    A = np.zeros((128, 64), dtype=np.uint16)
    A[0, 0] = 0x8000   # -0: not kept, becomes the first pad, value bits 0x8000
    A[0, 1] = 0x7E00   # NaN: not kept, second pad, value bits 0x7e00
    A[0, 2] = 0x3C00   # 1.0 at (0, 2)
    A[3, 3] = 0x4000   # 2.0 at (3, 3): swizzled column 3 ^ (3 << 3) = 27
    items, offs = oracle.encode_noreorder(A)
    assert list(offs) == [0, 1, 1]
    assert [int(w) for w in items] == [0x8000 | 0 << 16, 0x7E00 | 1 << 16, 0x3C00 | 2 << 16, 0x4000 | (3 * 64 + 27) << 16]


def test_noreorder_same_multiset_as_reordered(oracle, spmm):
    """Both encoders keep the same elements; only the order inside a tile (and the pad positions) differ."""
    A = spmm.synth_weights(256, 256, 0.8, True, seed=3)
    a_items, a_offs = oracle.encode(A)
    b_items, b_offs = oracle.encode_noreorder(A)
    assert np.array_equal(a_offs, b_offs)
    for t in range(len(a_offs) - 2):
        lo, hi = 4 * a_offs[t], 4 * a_offs[t + 1]
        x, y = a_items[lo:hi], b_items[lo:hi]
        assert np.array_equal(np.sort(x[(x & 0xFFFF) != 0]), np.sort(y[(y & 0xFFFF) != 0]))
    d = oracle.decode(b_items, b_offs, 256, 256)
    assert np.array_equal(d.astype(np.float32), A.astype(np.float32))
