"""CPU tests of the 2:4 + residual split and of the 2:4 record packer.

decompose() is pinned four ways: committed golden vectors written by the reference's own
function (tests/golden/decompose_small.npz), the oracle against that function compiled
from kernel_benchmark/spmm_decompose.h:12-51 (oracle/_ref, where that build ran), hand-made
groups whose answer is read off the reference's loop, and the properties the split must have.
The product's HeteroSparse_Decompose is then compared with the oracle bit for bit.
The record layout is this build's own (the reference's is made for NVIDIA's mma.sp); the
oracle's reader is pinned by records built by hand here, byte by byte, and the packer by
unpack(pack(A1)) == A1.
"""
import os

import numpy as np
import pytest

H = np.float16
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "decompose_small.npz")


def golden_cases():
    z = np.load(GOLD)
    names = sorted({k.rsplit(".", 1)[0] for k in z.files})
    return [(n, z[n + ".A"], z[n + ".A1"], z[n + ".A2"]) for n in names]


@pytest.mark.parametrize("name,A,A1,A2", golden_cases(), ids=[c[0] for c in golden_cases()])
def test_decompose_matches_reference_golden(oracle, spmm, name, A, A1, A2):
    """Committed outputs of the reference's own decompose() (tests/golden/make_golden.py): the oracle
    and the product must both reproduce them bit for bit, with or without the reference build at hand."""
    o1, o2 = oracle.decompose(A)
    assert np.array_equal(o1.view(np.uint16), A1) and np.array_equal(o2.view(np.uint16), A2)
    p1, p2 = spmm.HeteroSparse_Decompose(A)
    assert np.array_equal(p1.view(np.uint16), A1) and np.array_equal(p2.view(np.uint16), A2)


def _rand_sparse(rng, M, K, keep):
    A = (rng.standard_normal((M, K)) * 0.02).astype(H)
    A[rng.random((M, K)) >= keep] = 0
    return A


def test_oracle_decompose_hand_cases(oracle):
    nan = np.array([0x7E00], dtype=np.uint16).view(H)[0]
    negzero = np.array([0x8000], dtype=np.uint16).view(H)[0]
    A = np.array([
        [1, 2, 3, 4],          # first two stay, last two go to the residual
        [0, 5, 0, 6],          # already 2:4
        [7, 0, 8, 9],          # third kept value (9) is the residual
        [0, 0, 0, 0],
        [negzero, 1, 2, 3],    # -0 compares equal to zero: 1, 2 stay, 3 goes
        [nan, 1, 2, 0],        # NaN compares unequal: NaN, 1 stay, 2 goes
    ], dtype=H)
    A1, A2 = oracle.decompose(A)
    e1 = np.array([[1, 2, 0, 0], [0, 5, 0, 6], [7, 0, 8, 0], [0, 0, 0, 0], [0, 1, 2, 0], [nan, 1, 0, 0]], dtype=H)
    e2 = np.array([[0, 0, 3, 4], [0, 0, 0, 0], [0, 0, 0, 9], [0, 0, 0, 0], [0, 0, 0, 3], [0, 0, 2, 0]], dtype=H)
    assert np.array_equal(A1.view(np.uint16), e1.view(np.uint16))
    assert np.array_equal(A2.view(np.uint16), e2.view(np.uint16))


@pytest.mark.parametrize("keep", [0.1, 0.3, 0.5, 0.9])
def test_oracle_decompose_properties(oracle, keep):
    rng = np.random.default_rng(int(keep * 100))
    A = _rand_sparse(rng, 64, 256, keep)
    A1, A2 = oracle.decompose(A)
    nz, nz1, nz2 = A != 0, A1 != 0, A2 != 0
    assert not (nz1 & nz2).any()
    assert np.array_equal(np.where(nz1, A1, A2).view(np.uint16), np.where(nz, A, H(0)).view(np.uint16))
    g = nz.reshape(-1, 4)
    assert np.array_equal(nz1.reshape(-1, 4).sum(1), np.minimum(g.sum(1), 2))
    # the residual takes the LAST kept values of a group: rank of a kept value within its group >= 2
    rank = np.cumsum(g, axis=1) - 1
    assert np.array_equal(nz2.reshape(-1, 4), g & (rank >= 2))


def test_oracle_decompose_matches_reference_build(oracle):
    if not oracle.have_ref():
        pytest.skip("oracle/_ref not built (no reference checkout on this machine)")
    rng = np.random.default_rng(11)
    for keep in (0.2, 0.5, 0.8):
        A = _rand_sparse(rng, 128, 512, keep)
        A.view(np.uint16)[0, :8] = [0x8000, 0x7E00, 0x0001, 0x3C00, 0xFC00, 0x8001, 0, 0x7C00]
        o1, o2 = oracle.decompose(A)
        r1, r2 = oracle.ref_decompose(A)
        assert np.array_equal(o1.view(np.uint16), r1.view(np.uint16))
        assert np.array_equal(o2.view(np.uint16), r2.view(np.uint16))


@pytest.mark.parametrize("keep", [0.0, 0.2, 0.5, 1.0])
def test_product_decompose_equals_oracle(spmm, oracle, keep):
    rng = np.random.default_rng(7)
    A = _rand_sparse(rng, 128, 384, keep)
    A.view(np.uint16)[1, :4] = [0x8000, 0x7E00, 0x0001, 0x3C00]
    p1, p2 = spmm.HeteroSparse_Decompose(A)
    o1, o2 = oracle.decompose(A)
    assert np.array_equal(p1.view(np.uint16), o1.view(np.uint16))
    assert np.array_equal(p2.view(np.uint16), o2.view(np.uint16))


def test_decompose_rejects_bad_length(spmm):
    with pytest.raises(spmm.SpMMError):
        spmm.HeteroSparse_Decompose(np.zeros(6, dtype=H))


def test_oracle_unpack_reads_a_hand_built_record(oracle):
    """One 16 x 128 record written byte by byte from the layout's definition, as record 3 of the
    eight that a 128 x 128 matrix has (row block 3); the others hold zeros at valid positions."""
    M, K = 128, 128
    BLOCK = 3
    rec = np.zeros(2304, dtype=np.uint8)
    words = np.zeros(64, dtype=np.uint32)
    for L in range(64):  # every group of four: positions (0, 1), zero values
        for s in range(4):
            for j in range(4):
                words[L] |= np.uint32((j % 2)) << np.uint32(8 * s + 2 * j)
    expect = np.zeros((M, K), dtype=H)

    def put(L, s, j, q_pair, value):
        # slot j of lane L in step s holds `value` at position q_pair[j % 2]; the pair is ascending
        for t in range(2):
            jj = (j // 2) * 2 + t
            shift = 8 * s + 2 * jj
            words[L] = (int(words[L]) & ~(3 << shift)) | (q_pair[t] << shift)
        off = (s // 2) * 1024 + L * 16 + ((s % 2) * 4 + j) * 2
        rec[off:off + 2] = np.array([value], dtype=H).view(np.uint8)
        expect[BLOCK * 16 + L % 16, s * 32 + (L // 16) * 8 + (j // 2) * 4 + q_pair[j % 2]] = value

    put(0, 0, 0, (0, 1), 1.5)      # row 0, column 0
    put(0, 0, 3, (1, 3), -2.0)     # row 0, second group of the lane: column 4 + 3
    put(17, 2, 1, (2, 3), 3.0)     # row 1, column 2*32 + 1*8 + 3
    put(63, 3, 2, (1, 2), 0.25)    # row 15, column 3*32 + 3*8 + 4 + 1
    rec[2048:] = words.view(np.uint8)
    empty = np.zeros(2304, dtype=np.uint8)
    empty[2048:] = np.full(64, 0x44444444, dtype=np.uint32).view(np.uint8)  # positions (0, 1) everywhere
    packed = np.concatenate([rec if b == BLOCK else empty for b in range(8)])
    got = oracle.a24_unpack(packed, M, K)
    assert np.array_equal(got.view(np.uint16), expect.view(np.uint16))
    assert got[48, 0] == H(1.5) and got[48, 7] == H(-2.0) and got[49, 75] == H(3.0) and got[63, 125] == H(0.25)
    words[5] = 0  # positions (0, 0) in every pair: not a valid record
    rec[2048:] = words.view(np.uint8)
    with pytest.raises(ValueError):
        oracle.a24_unpack(np.concatenate([rec if b == BLOCK else empty for b in range(8)]), M, K)


@pytest.mark.parametrize("M,K,keep", [(128, 128, 0.5), (128, 256, 0.2), (384, 1024, 0.8), (128, 128, 0.0)])
def test_pack_round_trip(spmm, oracle, M, K, keep):
    rng = np.random.default_rng(M + K)
    A1, _ = oracle.decompose(_rand_sparse(rng, M, K, keep))
    packed = spmm.HeteroSparse_PackA1(A1)
    assert packed.size == (M // 16) * (K // 128) * 2304
    back = oracle.a24_unpack(packed, M, K)  # also checks ascending positions in every group
    assert np.array_equal(back.view(np.uint16), A1.view(np.uint16))


def test_pack_rejects_three_of_four_and_bad_shapes(spmm):
    A = np.zeros((128, 128), dtype=H)
    A[3, 8:11] = 1
    with pytest.raises(spmm.SpMMError) as e:
        spmm.HeteroSparse_PackA1(A)
    assert e.value.code == -6
    with pytest.raises(spmm.SpMMError):
        spmm.HeteroSparse_PackA1(np.zeros((128, 64), dtype=H))
    with pytest.raises(spmm.SpMMError):
        spmm.HeteroSparse_PackA1(np.zeros((64, 128), dtype=H))


def test_suggested_split_leaves_no_batch_empty(spmm):
    for M, K in [(28672, 7168), (7168, 28672), (7168, 7168), (9216, 36864), (128, 128), (256, 384)]:
        for N in (8, 16, 32, 64):
            s = spmm.HeteroSparse_SuggestSplitK(M, N, K)
            units = K // 128
            per = -(-units // s)
            assert s >= 1 and per * (s - 1) < units


def test_record_order_groups_eight_row_blocks(spmm, oracle):
    """Record of row block rb and unit u sits at ((rb // 8) * units + u) * 8 + rb % 8: a matrix with one
    value per (row block, unit) cell, whose value names the cell, must show each value in that record."""
    M, K = 384, 512
    units = K // 128
    A = np.zeros((M, K), dtype=H)
    for rb in range(M // 16):
        for u in range(units):
            A[rb * 16, u * 128] = H(rb * units + u + 1)  # lane 0, step 0, slot 0 of the record
    packed = spmm.HeteroSparse_PackA1(A).reshape(-1, 2304)
    assert packed.shape[0] == (M // 16) * units
    first = packed[:, :2].copy().view(H).reshape(-1)   # lane 0's first value of every record
    for rb in range(M // 16):
        for u in range(units):
            assert first[((rb // 8) * units + u) * 8 + rb % 8] == H(rb * units + u + 1)
    assert np.array_equal(oracle.a24_unpack(packed.reshape(-1), M, K).view(np.uint16), A.view(np.uint16))


def test_oracle_residual_unpack_reads_hand_built_lists(oracle):
    """Two words written by hand from the format's definition: row 5, column 77 of block 9 / unit 1
    and row 0, column 0 of block 0 / unit 0 of a 256 x 256 matrix."""
    M, K, units = 256, 256, 2
    offs = np.zeros((M // 16) * units + 1, dtype=np.int32)
    first = ((0 // 8) * units + 0) * 8 + 0
    second = ((9 // 8) * units + 1) * 8 + 9 % 8
    offs[first + 1:] += 1
    offs[second + 1:] += 1
    r, c = 5, 77
    addr = r * 256 + (((c // 8) ^ r) << 4) + (c % 8) * 2
    assert addr == 5 * 256 + ((9 ^ 5) << 4) + 10
    words = np.array([0x3C00 | 0 << 16, 0x4000 | addr << 16], dtype=np.uint32)  # 1.0 and 2.0
    A = oracle.residual_unpack(words, offs, M, K)
    want = np.zeros((M, K), dtype=H)
    want[0, 0] = 1
    want[9 * 16 + 5, 128 + 77] = 2
    assert np.array_equal(A.view(np.uint16), want.view(np.uint16))
    with pytest.raises(ValueError):  # the same place twice
        oracle.residual_unpack(np.array([0x3C00, 0x3C00], dtype=np.uint32), np.minimum(np.arange(offs.size), 2).astype(np.int32) * 0
                               + np.r_[0, np.full(offs.size - 1, 2)].astype(np.int32), M, K)


@pytest.mark.parametrize("M,K,keep", [(128, 128, 0.5), (256, 640, 0.4), (384, 1024, 0.2), (128, 256, 0.0), (128, 128, 1.0)])
def test_residual_lists_round_trip(spmm, oracle, M, K, keep):
    rng = np.random.default_rng(M + K + 1)
    A = _rand_sparse(rng, M, K, keep)
    A.view(np.uint16)[0, :8] = [0x8000, 0x7E00, 0x0001, 0x3C00, 0xFC00, 0x8001, 0, 0x7C00]  # -0, NaN, denormals, infinities
    _, A2 = oracle.decompose(A)
    words, offs, longest = spmm.HeteroSparse_PackA2(A2)
    units = K // 128
    assert offs.size == (M // 16) * units + 1 and offs[0] == 0
    assert words.size == offs[-1] + 64 and not words[offs[-1]:].any()  # the padding the kernel may read
    lengths = np.diff(offs)
    assert longest == (lengths.max() if lengths.size else 0)
    assert offs[-1] == np.count_nonzero(A2.view(np.uint16) & 0x7FFF)   # one word per kept value, -0 is not one
    back = oracle.residual_unpack(words[:offs[-1]], offs, M, K)
    want = A2.view(np.uint16).copy()
    want[(want & 0x7FFF) == 0] = 0
    assert np.array_equal(back.view(np.uint16), want)
    # Every round of 64 words spreads over the banks: with three or more rounds no round holds more of
    # a bank than an even split over the full rounds, and in all the serialised passes (the fullest
    # bank of every round, summed) are fewer than in row-major order.
    def passes(lst):
        bank = ((lst >> 16) >> 2) & 63
        return sum(np.bincount(bank[r:r + 64], minlength=64).max() for r in range(0, lst.size, 64))

    ordered = plain = 0
    for i in range(offs.size - 1):
        lst = words[offs[i]:offs[i + 1]]
        rounds = -(-lst.size // 64)
        if rounds <= 1:
            continue
        bank = ((lst >> 16) >> 2) & 63
        total = np.bincount(bank, minlength=64)
        if rounds >= 3:
            for r in range(rounds):
                assert (np.bincount(bank[r * 64:(r + 1) * 64], minlength=64) <= -(-total // (rounds - 1))).all()
        ordered += passes(lst)
        plain += passes(np.sort(lst >> 16) << 16)
    assert ordered <= plain
    if keep in (0.4, 0.5):  # lists of two to four rounds, banks unevenly filled
        assert ordered < 0.9 * plain


def test_residual_lists_reject_bad_shapes(spmm):
    for shape in ((128, 64), (64, 128), (200, 128)):
        with pytest.raises(spmm.SpMMError) as e:
            spmm.HeteroSparse_PackA2(np.zeros(shape, dtype=H))
        assert e.value.code == -1

