"""TEST INFRASTRUCTURE ONLY: ctypes doors onto the CPU checkers.

``liboracle.so`` is the C restatement (``tiled_csl_oracle.c``);
``_ref/libref_encoder.so`` is the reference's own host encoder compiled by
``oracle/Makefile`` (present only where that build ran).  Only tests,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this module; the product never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_ORACLE_SO = os.path.join(_HERE, "liboracle.so")
_REF_SO = os.path.join(_HERE, "_ref", "libref_encoder.so")

_u16p = ctypes.POINTER(ctypes.c_uint16)
_u32p = ctypes.POINTER(ctypes.c_uint32)
_i32p = ctypes.POINTER(ctypes.c_int)
_f32p = ctypes.POINTER(ctypes.c_float)


def build(with_ref=True):
    """(Re)build the checkers with oracle/Makefile."""
    targets = ["oracle"] + (["ref"] if with_ref else [])
    subprocess.run(["make", "-s", "-C", _HERE] + targets, check=True)


def _load():
    if not os.path.exists(_ORACLE_SO):
        build(with_ref=False)
    lib = ctypes.CDLL(_ORACLE_SO)
    lib.oracle_half_to_float.restype = ctypes.c_float
    lib.oracle_half_to_float.argtypes = [ctypes.c_uint16]
    lib.oracle_float_to_half_rn.restype = ctypes.c_uint16
    lib.oracle_float_to_half_rn.argtypes = [ctypes.c_float]
    lib.oracle_encode.restype = ctypes.c_int
    lib.oracle_encode.argtypes = [_u16p, ctypes.c_int, ctypes.c_int, ctypes.POINTER(_u32p), ctypes.POINTER(_i32p)]
    lib.oracle_encode_noreorder.restype = ctypes.c_int
    lib.oracle_encode_noreorder.argtypes = lib.oracle_encode.argtypes
    lib.oracle_free.argtypes = [ctypes.c_void_p]
    lib.oracle_decode.argtypes = [_u32p, _i32p, ctypes.c_int, ctypes.c_int, _u16p]
    lib.oracle_gemm_f32.argtypes = [_u16p, _u16p, _f32p] + [ctypes.c_int] * 5
    lib.oracle_splitk_range.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, _i32p, _i32p]
    lib.oracle_reduce.argtypes = [_u16p, _u16p, ctypes.c_long, ctypes.c_int]
    lib.oracle_spmm_splitk.restype = ctypes.c_int
    lib.oracle_spmm_splitk.argtypes = [_u32p, _i32p, _u16p, _u16p, ctypes.c_int, ctypes.c_int, ctypes.c_int, _u16p,
                                       ctypes.c_int]
    lib.oracle_decompose.argtypes = [_u16p, _u16p, _u16p, ctypes.c_long]
    lib.oracle_a24_unpack.restype = ctypes.c_int
    lib.oracle_a24_unpack.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, _u16p]
    return lib


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


def _bits(a):
    """fp16 array (or uint16 bit array) -> contiguous uint16 view."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        return a.view(np.uint16)
    assert a.dtype == np.uint16, a.dtype
    return a


def _take(ptr, n, dtype, free):
    out = np.ctypeslib.as_array(ptr, shape=(max(n, 1),))[:n].astype(dtype, copy=True)
    free(ptr)
    return out


def encode(A):
    """Oracle Tiled-CSL encode of a row-major fp16 M x K matrix -> (items u32, offsets i32)."""
    M, K = A.shape
    a = _bits(A)
    items, offs = _u32p(), _i32p()
    n = lib().oracle_encode(a.ctypes.data_as(_u16p), M, K, ctypes.byref(items), ctypes.byref(offs))
    if n < 0:
        raise ValueError(f"oracle_encode failed with {n} for M={M} K={K}")
    o = np.ctypeslib.as_array(offs, shape=(n,)).astype(np.int32, copy=True)
    it = _take(items, int(o[-1]) * 4, np.uint32, lib().oracle_free)
    lib().oracle_free(offs)
    return it, o


def encode_noreorder(A):
    """Oracle encode without the bank-aware reordering (csrc/SpMM_API.cu:441-567)."""
    M, K = A.shape
    a = _bits(A)
    items, offs = _u32p(), _i32p()
    n = lib().oracle_encode_noreorder(a.ctypes.data_as(_u16p), M, K, ctypes.byref(items), ctypes.byref(offs))
    if n < 0:
        raise ValueError(f"oracle_encode_noreorder failed with {n} for M={M} K={K}")
    o = np.ctypeslib.as_array(offs, shape=(n,)).astype(np.int32, copy=True)
    it = _take(items, int(o[-1]) * 4, np.uint32, lib().oracle_free)
    lib().oracle_free(offs)
    return it, o


def decode(items, offsets, M, K):
    items = np.ascontiguousarray(items, dtype=np.uint32)
    offsets = np.ascontiguousarray(offsets, dtype=np.int32)
    out = np.empty((M, K), dtype=np.uint16)
    lib().oracle_decode(items.ctypes.data_as(_u32p), offsets.ctypes.data_as(_i32p), M, K, out.ctypes.data_as(_u16p))
    return out.view(np.float16)


def gemm_f32(A, B, k_begin=0, k_end=None):
    """A: M x K fp16 row-major; B: N x K fp16 (one K-vector per token) -> C: N x M fp32."""
    M, K = A.shape
    N = B.shape[0]
    assert B.shape[1] == K
    a, b = _bits(A), _bits(B)
    C = np.empty((N, M), dtype=np.float32)
    lib().oracle_gemm_f32(a.ctypes.data_as(_u16p), b.ctypes.data_as(_u16p), C.ctypes.data_as(_f32p), M, N, K, k_begin,
                          K if k_end is None else k_end)
    return C


def splitk_range(K, split_k, b):
    s, e = ctypes.c_int(), ctypes.c_int()
    lib().oracle_splitk_range(K, split_k, b, ctypes.byref(s), ctypes.byref(e))
    return s.value, e.value


def reduce(W, MN, split_k):
    w = _bits(W).reshape(-1)
    C = np.empty(MN, dtype=np.uint16)
    lib().oracle_reduce(C.ctypes.data_as(_u16p), w.ctypes.data_as(_u16p), MN, split_k)
    return C.view(np.float16)


def spmm_splitk(items, offsets, B, M, N, K, split_k):
    """Whole call on the CPU -> (C fp16 N x M, workspace fp16 split_k x N x M)."""
    items = np.ascontiguousarray(items, dtype=np.uint32)
    offsets = np.ascontiguousarray(offsets, dtype=np.int32)
    b = _bits(B)
    C = np.zeros((N, M), dtype=np.uint16)
    W = np.zeros((split_k, N, M), dtype=np.uint16)
    rc = lib().oracle_spmm_splitk(items.ctypes.data_as(_u32p), offsets.ctypes.data_as(_i32p), b.ctypes.data_as(_u16p),
                                  C.ctypes.data_as(_u16p), M, N, K, W.ctypes.data_as(_u16p), split_k)
    if rc:
        raise ValueError(f"oracle_spmm_splitk rejected M={M} N={N} K={K} split_k={split_k}")
    return C.view(np.float16), W.view(np.float16)


def decompose(A):
    """2:4 part and residual of a row-major fp16 matrix (kernel_benchmark/spmm_decompose.h:12-51)."""
    a = _bits(A)
    A1 = np.empty(a.shape, dtype=np.uint16)
    A2 = np.empty(a.shape, dtype=np.uint16)
    lib().oracle_decompose(a.ctypes.data_as(_u16p), A1.ctypes.data_as(_u16p), A2.ctypes.data_as(_u16p), a.size)
    return A1.view(np.float16), A2.view(np.float16)


def a24_unpack(packed, M, K):
    """Dense fp16 M x K matrix held by 2:4 records (16 rows x 128 columns, 2304 bytes each)."""
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    assert packed.size == (M // 16) * (K // 128) * 2304, packed.size
    out = np.empty((M, K), dtype=np.uint16)
    rc = lib().oracle_a24_unpack(packed.ctypes.data_as(ctypes.c_void_p), M, K, out.ctypes.data_as(_u16p))
    if rc:
        raise ValueError("2:4 records with equal or descending positions inside a group")
    return out.view(np.float16)


def residual_unpack(words, offsets, M, K):
    """Dense fp16 M x K matrix held by residual lists (the build's own format for the launch that
    multiplies the 2:4 part and the residual together; the reference keeps its residual in a
    CSR-like form for kernel_benchmark/FSP_Batch8.h:129-206).  List i belongs to the record of the
    same number, ((rb // 8) * units + u) * 8 + rb % 8 for row block rb and unit u; a word is
    value | address << 16 with address = r * 256 + (((c // 8) ^ r) << 4) + (c % 8) * 2 for row r and
    column c of the 16 x 128 block.  Raises on an address twice in one list or out of range."""
    words = np.ascontiguousarray(words, dtype=np.uint32)
    offsets = np.ascontiguousarray(offsets, dtype=np.int64)
    units = K // 128
    assert offsets.size == (M // 16) * units + 1 and offsets[0] == 0 and (np.diff(offsets) >= 0).all()
    out = np.zeros((M, K), dtype=np.uint16)
    for rb in range(M // 16):
        for u in range(units):
            i = ((rb // 8) * units + u) * 8 + rb % 8
            lst = words[offsets[i]:offsets[i + 1]]
            addr = (lst >> 16).astype(np.int64)
            if addr.size and (addr.max() >= 4096 or (addr & 1).any() or np.unique(addr).size != addr.size):
                raise ValueError(f"bad addresses in list {i}")
            r = addr >> 8
            c = ((((addr >> 4) & 15) ^ r) << 3) + ((addr & 15) >> 1)
            out[rb * 16 + r, u * 128 + c] = (lst & 0xFFFF).astype(np.uint16)
    return out.view(np.float16)


# ----------------------------------------------------------------------------
# the reference's own encoder, where oracle/_ref was built


def have_ref():
    return os.path.exists(_REF_SO)


_ref = None


def ref_encode(A, reorder=True):
    """Encode with the reference's InitSparseMatrixA_API (csrc/SpMM_API.cu:241-438) or, with
    reorder=False, its InitSparseMatrixA_API_NoReorder (:441-567)."""
    global _ref
    if _ref is None:
        _ref = ctypes.CDLL(_REF_SO)
        _ref.ref_InitSparseMatrixA_API.restype = ctypes.c_int
        _ref.ref_InitSparseMatrixA_API.argtypes = [_u16p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                   ctypes.POINTER(_u32p), ctypes.POINTER(_i32p)]
        _ref.ref_InitSparseMatrixA_API_NoReorder.restype = ctypes.c_int
        _ref.ref_InitSparseMatrixA_API_NoReorder.argtypes = _ref.ref_InitSparseMatrixA_API.argtypes
        _ref.ref_free.argtypes = [ctypes.c_void_p]
    M, K = A.shape
    a = _bits(A).copy()
    items, offs = _u32p(), _i32p()
    fn = _ref.ref_InitSparseMatrixA_API if reorder else _ref.ref_InitSparseMatrixA_API_NoReorder
    n = fn(a.ctypes.data_as(_u16p), M, 0, K, ctypes.byref(items), ctypes.byref(offs))
    o = np.ctypeslib.as_array(offs, shape=(n,)).astype(np.int32, copy=True)
    it = _take(items, int(o[-1]) * 4, np.uint32, _ref.ref_free)
    _ref.ref_free(offs)
    return it, o


def ref_decompose(A):
    """The reference's own decompose() (kernel_benchmark/spmm_decompose.h:12-51); prints its statistics."""
    global _ref
    if _ref is None:
        ref_encode(np.zeros((128, 64), dtype=np.float16))  # loads the library
    _ref.ref_decompose.argtypes = [_u16p, _u16p, _u16p, ctypes.c_int]
    a = _bits(A).copy()
    A1 = np.empty(a.shape, dtype=np.uint16)
    A2 = np.empty(a.shape, dtype=np.uint16)
    _ref.ref_decompose(a.ctypes.data_as(_u16p), A1.ctypes.data_as(_u16p), A2.ctypes.data_as(_u16p), a.size)
    return A1.view(np.float16), A2.view(np.float16)
