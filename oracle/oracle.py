"""ctypes front end of the C checkers in this directory.  TEST INFRASTRUCTURE ONLY.

`liboracle.so` is our plain-C restatement (spmm_oracle.c).  `_ref/libref_encoder.so`
is the reference's own host encoder compiled from the reference tree by the
Makefile beside this file; it is optional (present only where it was built).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_u16p = C.POINTER(C.c_uint16)
_i32p = C.POINTER(C.c_int)
_u64p = C.POINTER(C.c_uint64)


def build(force=False):
    """Compile the checkers (the reference encoder only where its tree exists)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE, "all"], stdout=subprocess.DEVNULL)


def _load(path):
    if not os.path.exists(path):
        return None
    return C.CDLL(path)


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        _lib = C.CDLL(path)
        L = _lib
        L.oracle_encode_bitmap.restype = C.c_int
        L.oracle_encode_bitmap.argtypes = [C.c_void_p, C.c_int, C.c_int, C.POINTER(_u16p), C.POINTER(_i32p),
                                           C.POINTER(_i32p), C.POINTER(_i32p), C.POINTER(_u64p), _i32p]
        L.oracle_round_max_nnz.restype = C.c_int
        L.oracle_round_max_nnz.argtypes = [C.c_int]
        L.oracle_free.argtypes = [C.c_void_p]
        L.oracle_decode_bitmap.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]
        L.oracle_splitk_range.restype = C.c_int
        L.oracle_splitk_range.argtypes = [C.c_int, C.c_int, C.c_int, _i32p]
        L.oracle_spmm.argtypes = [C.c_void_p] * 5 + [C.c_int] * 5
        L.oracle_spmm_bias_act.argtypes = [C.c_void_p] * 5 + [C.c_int] * 5 + [C.c_void_p, C.c_int]
        L.oracle_num_threads.restype = C.c_int
        L.oracle_gemm_f64.argtypes = [C.c_void_p] * 3 + [C.c_int] * 3
        L.oracle_init_host_matrices.argtypes = [C.c_void_p, C.c_void_p] + [C.c_int] * 5
        L.oracle_total_error.restype = C.c_double
        L.oracle_total_error.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int]
        L.oracle_splitk_reduce_fp16.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int]
        L.oracle_half_to_float.restype = C.c_float
        L.oracle_half_to_float.argtypes = [C.c_uint16]
        L.oracle_float_to_half.restype = C.c_uint16
        L.oracle_float_to_half.argtypes = [C.c_float]
    return _lib


def ref_lib():
    """The reference's own encoder, or None where it has not been built."""
    global _ref
    if _ref is None:
        _ref = _load(os.path.join(_HERE, "_ref", "libref_encoder.so"))
        if _ref is not None:
            _ref.ref_InitSparseMatrixA_bitmap.restype = C.c_int
            _ref.ref_InitSparseMatrixA_bitmap.argtypes = [C.c_void_p, C.c_int, C.c_int, C.POINTER(_u16p),
                                                          C.POINTER(_i32p), C.POINTER(_i32p), C.POINTER(_i32p),
                                                          C.POINTER(_u64p), _i32p]
            _ref.ref_free.argtypes = [C.c_void_p]
    return _ref


def _as_u16(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    assert a.dtype == np.uint16
    return a


def _collect(fn, free, W, M, K):
    W = _as_u16(W)
    assert W.size == M * K
    vals, cnt, med, glo, bmp = _u16p(), _i32p(), _i32p(), _i32p(), _u64p()
    mx = C.c_int(0)
    G = fn(W.ctypes.data, M, K, C.byref(vals), C.byref(cnt), C.byref(med), C.byref(glo), C.byref(bmp), C.byref(mx))
    if G < 0:
        raise MemoryError("encoder returned -1")
    T = (M // 8) * (K // 8)
    out = {"num_gtiles": G, "max_nnz": mx.value}
    out["global"] = np.ctypeslib.as_array(glo, shape=(G + 1,)).copy()
    nnz = int(out["global"][G])
    # realloc(p, 0) may hand back NULL for an all-zero matrix
    out["values"] = (np.ctypeslib.as_array(vals, shape=(nnz,)).copy() if nnz else np.zeros(0, np.uint16))
    out["tile_cnt"] = np.ctypeslib.as_array(cnt, shape=(max(T, 1),))[:T].copy()
    out["median"] = np.ctypeslib.as_array(med, shape=(max(4 * G, 1),))[:4 * G].copy()
    out["bitmap"] = np.ctypeslib.as_array(bmp, shape=(max(T, 1),))[:T].copy()
    for p in (vals, cnt, med, glo, bmp):
        free(C.cast(p, C.c_void_p))
    return out


def encode(W, M, K):
    """oracle_encode_bitmap -> dict(values u16, tile_cnt, median, global, bitmap u64, max_nnz, num_gtiles)."""
    L = lib()
    return _collect(L.oracle_encode_bitmap, L.oracle_free, W, M, K)


def ref_encode(W, M, K):
    """Same, through the reference's own encoder (raises if it was not built)."""
    R = ref_lib()
    if R is None:
        raise RuntimeError("oracle/_ref/libref_encoder.so is not built")
    return _collect(R.ref_InitSparseMatrixA_bitmap, R.ref_free, W, M, K)


def round_max_nnz(v):
    return lib().oracle_round_max_nnz(int(v))


def decode(values, bitmap, global_off, M, K):
    values = _as_u16(values)
    if values.size == 0:
        values = np.zeros(1, np.uint16)
    bitmap = np.ascontiguousarray(bitmap, dtype=np.uint64)
    global_off = np.ascontiguousarray(global_off, dtype=np.int32)
    W = np.empty((M, K), np.uint16)
    lib().oracle_decode_bitmap(values.ctypes.data, bitmap.ctypes.data, global_off.ctypes.data, M, K, W.ctypes.data)
    return W.view(np.float16)


def splitk_range(K, split_k, batch):
    cnt = C.c_int(0)
    first = lib().oracle_splitk_range(K, split_k, batch, C.byref(cnt))
    return first, cnt.value


def spmm(values, bitmap, global_off, X, M, N, K, split_k=1, partial_fp16=False):
    """Host SpMM on the compressed arrays.  X: [N][K] fp16.  Returns C as [N][M] fp16."""
    values = _as_u16(values)
    if values.size == 0:
        values = np.zeros(1, np.uint16)
    bitmap = np.ascontiguousarray(bitmap, dtype=np.uint64)
    global_off = np.ascontiguousarray(global_off, dtype=np.int32)
    X = _as_u16(X)
    assert X.size == N * K
    Cout = np.empty((N, M), np.uint16)
    lib().oracle_spmm(values.ctypes.data, bitmap.ctypes.data, global_off.ctypes.data, X.ctypes.data,
                      Cout.ctypes.data, M, N, K, int(split_k), int(bool(partial_fp16)))
    return Cout.view(np.float16)


def spmm_bias_act(values, bitmap, global_off, X, M, N, K, split_k=1, bias=None, act=0):
    """Host SpMM with C = fp16(act(sum + bias[m])); bias: M fp16 values or None; act 0 none, 1 ReLU, 2 GELU."""
    values = _as_u16(values)
    if values.size == 0:
        values = np.zeros(1, np.uint16)
    bitmap = np.ascontiguousarray(bitmap, dtype=np.uint64)
    global_off = np.ascontiguousarray(global_off, dtype=np.int32)
    X = _as_u16(X)
    assert X.size == N * K
    b = None if bias is None else _as_u16(bias)
    assert b is None or b.size == M
    Cout = np.empty((N, M), np.uint16)
    lib().oracle_spmm_bias_act(values.ctypes.data, bitmap.ctypes.data, global_off.ctypes.data, X.ctypes.data,
                               Cout.ctypes.data, M, N, K, int(split_k), 0,
                               None if b is None else b.ctypes.data, int(act))
    return Cout.view(np.float16)


def num_threads():
    return lib().oracle_num_threads()


def gemm_f64(W, X, M, N, K):
    W, X = _as_u16(W), _as_u16(X)
    out = np.empty((N, M), np.float64)
    lib().oracle_gemm_f64(W.ctypes.data, X.ctypes.data, out.ctypes.data, M, N, K)
    return out


def init_host_matrices(M, K, N, pruning_percentage, reseed=True):
    """The reference harness generator (glibc rand()).  Returns (W [M][K], X [N][K]) fp16."""
    a = np.empty((M, K), np.uint16)
    b = np.empty((N, K), np.uint16)
    lib().oracle_init_host_matrices(a.ctypes.data, b.ctypes.data, M, K, N, pruning_percentage, int(reseed))
    return a.view(np.float16), b.view(np.float16)


def total_error(ref, other):
    ref, other = _as_u16(ref), _as_u16(other)
    return lib().oracle_total_error(ref.ctypes.data, other.ctypes.data, ref.size, 1)


def splitk_reduce_fp16(ws, M, N, split_k):
    ws = _as_u16(ws)
    out = np.empty((N, M), np.uint16)
    lib().oracle_splitk_reduce_fp16(ws.ctypes.data, out.ctypes.data, M, N, split_k)
    return out.view(np.float16)


def half_to_float(h):
    return lib().oracle_half_to_float(int(h))


def float_to_half(f):
    return lib().oracle_float_to_half(float(f))
