"""ctypes access to oracle/liboracle.so — test infrastructure only.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import
this module; nothing under flash-llm_amd/ does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liboracle.so")
_u16p = ctypes.POINTER(ctypes.c_uint16)
_u32p = ctypes.POINTER(ctypes.c_uint32)
_i32p = ctypes.POINTER(ctypes.c_int)
_f32p = ctypes.POINTER(ctypes.c_float)
_lib = None


def build():
    subprocess.run(["make", "-C", _HERE, "-B", "liboracle.so"], check=True, capture_output=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = ctypes.CDLL(LIB_PATH)
        for name in ("oracle_compress_reorder", "oracle_compress_noreorder"):
            f = getattr(L, name)
            f.restype = ctypes.c_int
            f.argtypes = [_u16p, ctypes.c_int, ctypes.c_int, ctypes.POINTER(_u32p), ctypes.POINTER(_i32p)]
        L.oracle_free.restype = None
        L.oracle_free.argtypes = [ctypes.c_void_p]
        L.oracle_scatter.restype = ctypes.c_int
        L.oracle_scatter.argtypes = [_u32p, _i32p, ctypes.c_int, ctypes.c_int, _u16p]
        L.oracle_spmm_model.restype = ctypes.c_int
        L.oracle_spmm_model.argtypes = [_u16p, _u16p, _u16p, _f32p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.oracle_splitk_reduce.restype = None
        L.oracle_splitk_reduce.argtypes = [_u16p, _u16p, ctypes.c_long, ctypes.c_int]
        L.oracle_gemm_f32.restype = ctypes.c_int
        L.oracle_gemm_f32.argtypes = [_u16p, _u16p, _f32p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.oracle_splitk_ranges.restype = None
        L.oracle_splitk_ranges.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, _i32p, _i32p]
        L.oracle_half_to_float.restype = ctypes.c_float
        L.oracle_half_to_float.argtypes = [ctypes.c_uint16]
        L.oracle_float_to_half.restype = ctypes.c_uint16
        L.oracle_float_to_half.argtypes = [ctypes.c_float]
        L.oracle_nonzero.restype = ctypes.c_int
        L.oracle_nonzero.argtypes = [ctypes.c_uint16]
        _lib = L
    return _lib


def _bits(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    assert a.dtype == np.uint16
    return a


def _compress(name, a):
    a = _bits(a)
    m, k = a.shape
    comp, offs = _u32p(), _i32p()
    n = getattr(lib(), name)(a.ctypes.data_as(_u16p), m, k, ctypes.byref(comp), ctypes.byref(offs))
    if n < 0:
        return n, None, None
    offsets = np.ctypeslib.as_array(offs, shape=(n,)).copy()
    nnz = int(offsets[-1]) * 4
    items = np.ctypeslib.as_array(comp, shape=(max(nnz, 1),))[:nnz].copy()
    lib().oracle_free(comp)
    lib().oracle_free(offs)
    return n, items, offsets


def compress_reorder(a):
    return _compress("oracle_compress_reorder", a)


def compress_noreorder(a):
    return _compress("oracle_compress_noreorder", a)


def scatter(items, offsets, m, k):
    items = np.ascontiguousarray(items, dtype=np.uint32)
    if items.size == 0:
        items = np.zeros(1, dtype=np.uint32)
    offsets = np.ascontiguousarray(offsets, dtype=np.int32)
    out = np.empty((m, k), dtype=np.uint16)
    rc = lib().oracle_scatter(items.ctypes.data_as(_u32p), offsets.ctypes.data_as(_i32p), m, k, out.ctypes.data_as(_u16p))
    if rc:
        raise ValueError(f"oracle_scatter: {rc}")
    return out


def spmm_model(a_dense, b_colmajor, n, split_k, want_f32=True):
    """a_dense: (M,K) fp16; b_colmajor: (N,K) fp16 (column-major K x N).
    Returns (C as (N,M) fp16 = column-major M x N, fp32-accumulated (N,M) float32)."""
    a = _bits(a_dense)
    b = _bits(b_colmajor)
    m, k = a.shape
    assert b.shape == (n, k)
    c = np.empty((n, m), dtype=np.uint16)
    cf = np.empty((n, m), dtype=np.float32)
    rc = lib().oracle_spmm_model(a.ctypes.data_as(_u16p), b.ctypes.data_as(_u16p), c.ctypes.data_as(_u16p),
                                 cf.ctypes.data_as(_f32p) if want_f32 else None, m, n, k, split_k)
    if rc:
        raise ValueError(f"oracle_spmm_model: {rc}")
    return c.view(np.float16), cf


def splitk_reduce(ws, mn, split_k):
    ws = _bits(ws).reshape(-1)
    c = np.empty(mn, dtype=np.uint16)
    lib().oracle_splitk_reduce(ws.ctypes.data_as(_u16p), c.ctypes.data_as(_u16p), mn, split_k)
    return c.view(np.float16)


def gemm_f32(a_dense, b_colmajor, n, row_begin=0, row_end=None):
    a = _bits(a_dense)
    b = _bits(b_colmajor)
    m, k = a.shape
    row_end = m if row_end is None else row_end
    c = np.zeros((n, m), dtype=np.float32)
    threads = lib().oracle_gemm_f32(a.ctypes.data_as(_u16p), b.ctypes.data_as(_u16p), c.ctypes.data_as(_f32p), m, n, k, row_begin, row_end)
    return c, threads


def splitk_ranges(k, split_k):
    out = []
    for s in range(split_k):
        b, e = ctypes.c_int(), ctypes.c_int()
        lib().oracle_splitk_ranges(k, split_k, s, ctypes.byref(b), ctypes.byref(e))
        out.append((b.value, e.value))
    return out
