"""ctypes binding of the CPU oracle (oracle/liboracle.so) -- TEST INFRASTRUCTURE ONLY.

Importable only from tests/, the smoke test and the CPU-baseline leg of bench.py.  The
library it loads is the checker, never the product path.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libref_host.so")

_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_i32p = ctypes.POINTER(ctypes.c_int32)
_u64p = ctypes.POINTER(ctypes.c_uint64)
_sz = ctypes.c_size_t


def build(force=False):
    """Compile the oracle (and oracle/_ref when the reference tree is mounted)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s", "all"], check=True)


def _ptr(a, typ):
    return a.ctypes.data_as(typ) if a is not None else None


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        L.oracle_engine_init.restype = ctypes.c_uint32
        L.oracle_engine_init.argtypes = [ctypes.c_uint64]
        L.oracle_engine_skip.restype = ctypes.c_uint32
        L.oracle_engine_skip.argtypes = [ctypes.c_uint32, ctypes.c_uint64]
        L.oracle_uniform_fill.restype = ctypes.c_uint32
        L.oracle_uniform_fill.argtypes = [ctypes.c_uint32, ctypes.c_float, ctypes.c_float, _f32p, _sz]
        L.oracle_normal_fill.restype = ctypes.c_uint32
        L.oracle_normal_fill.argtypes = [ctypes.c_uint32, ctypes.c_float, ctypes.c_float, _f32p, _sz]
        L.oracle_preprocess_ordering.restype = None
        L.oracle_preprocess_ordering.argtypes = [_f32p, _sz, _f32p, _sz, ctypes.c_int]
        L.oracle_parse_number.restype = ctypes.c_uint64
        L.oracle_parse_number.argtypes = [ctypes.c_char_p]
        L.oracle_parse_dim3.restype = None
        L.oracle_parse_dim3.argtypes = [ctypes.c_char_p, _u64p]
        for name in ("oracle_dist_l2", "oracle_dist_partial_l2"):
            fn = getattr(L, name)
            fn.restype = None
            fn.argtypes = [_f32p, _f32p, _sz, _sz, _sz, _f32p, _sz]
        L.oracle_dist_f64.restype = None
        L.oracle_dist_f64.argtypes = [_f32p, _f32p, _sz, _sz, _sz, ctypes.c_int, _f64p, _sz]
        L.oracle_topk.restype = None
        L.oracle_topk.argtypes = [_f32p, _sz, _i32p, _sz, _i32p, _sz, _sz, _sz, _f32p, _i32p, _sz]
        L.oracle_topk_serial.restype = None
        L.oracle_topk_serial.argtypes = [_f32p, _sz, _sz, _sz, _sz, _f32p, _i32p]
        L.oracle_topk_parallel.restype = ctypes.c_int
        L.oracle_topk_parallel.argtypes = [_f32p, _sz, _sz, _sz, _sz, _f32p, _i32p, ctypes.c_int]
        L.oracle_checksum.restype = ctypes.c_uint32
        L.oracle_checksum.argtypes = [_i32p, _sz]
        L.oracle_verify.restype = ctypes.c_int
        L.oracle_verify.argtypes = [_f32p, _i32p, _f32p, _i32p, _sz, _sz, ctypes.POINTER(_sz)]
        _lib = L
    return _lib


def ref():
    """The reference's own host headers behind a C shim, or None when not built."""
    global _ref
    if _ref is None and os.path.exists(_REF_PATH):
        R = ctypes.CDLL(_REF_PATH)
        for name in ("ref_uniform_generate", "ref_normal_generate"):
            fn = getattr(R, name)
            fn.restype = None
            fn.argtypes = [ctypes.c_uint64, ctypes.c_float, ctypes.c_float, _sz, _sz, _sz, _f32p, _f32p]
        R.ref_preprocess_ordering.restype = None
        R.ref_preprocess_ordering.argtypes = [_f32p, _sz, _f32p, _sz, _sz, ctypes.c_int]
        R.ref_parse_number.restype = ctypes.c_uint64
        R.ref_parse_number.argtypes = [ctypes.c_char_p]
        R.ref_parse_dim3.restype = None
        R.ref_parse_dim3.argtypes = [ctypes.c_char_p, _u64p]
        _ref = R
    return _ref


# ---------------------------------------------------------------------------------------------
# numpy-level helpers
# ---------------------------------------------------------------------------------------------

def generate(seed, n, q, d, generator="uniform", params=(0.0, 1.0), preprocessor="identity"):
    """Points (n x d) then queries (q x d) from one engine, like the reference driver
    (src/main.cpp:291-313), optionally followed by an ordering preprocessor."""
    L = lib()
    points = np.empty((n, d), dtype=np.float32)
    queries = np.empty((q, d), dtype=np.float32)
    state = L.oracle_engine_init(seed)
    fill = L.oracle_uniform_fill if generator == "uniform" else L.oracle_normal_fill
    state = fill(state, params[0], params[1], _ptr(points, _f32p), points.size)
    fill(state, params[0], params[1], _ptr(queries, _f32p), queries.size)
    if preprocessor != "identity":
        L.oracle_preprocess_ordering(_ptr(points, _f32p), points.size, _ptr(queries, _f32p),
                                     queries.size, 1 if preprocessor == "descending" else 0)
    return points, queries


def uniform_matrix(seed, rows, cols, lo=0.0, hi=1.0):
    """rows x cols matrix of i.i.d. uniform floats drawn from the reference engine."""
    L = lib()
    out = np.empty((rows, cols), dtype=np.float32)
    L.oracle_uniform_fill(L.oracle_engine_init(seed), lo, hi, _ptr(out, _f32p), out.size)
    return out


def dist(queries, points, kind="l2"):
    L = lib()
    queries = np.ascontiguousarray(queries, dtype=np.float32)
    points = np.ascontiguousarray(points, dtype=np.float32)
    q, d = queries.shape
    n = points.shape[0]
    if kind == "f64" or kind == "f64-partial":
        out = np.empty((q, n), dtype=np.float64)
        L.oracle_dist_f64(_ptr(queries, _f32p), _ptr(points, _f32p), q, n, d,
                          1 if kind == "f64-partial" else 0, _ptr(out, _f64p), n)
        return out
    out = np.empty((q, n), dtype=np.float32)
    fn = L.oracle_dist_l2 if kind == "l2" else L.oracle_dist_partial_l2
    fn(_ptr(queries, _f32p), _ptr(points, _f32p), q, n, d, _ptr(out, _f32p), n)
    return out


def topk(matrix, k, labels=None, label_offsets=None):
    L = lib()
    assert matrix.dtype == np.float32 and matrix.ndim == 2 and matrix.strides[1] == 4
    rows, cols = matrix.shape
    out_d = np.empty((rows, k), dtype=np.float32)
    out_l = np.empty((rows, k), dtype=np.int32)
    if labels is not None:
        labels = np.ascontiguousarray(labels, dtype=np.int32)
    if label_offsets is not None:
        label_offsets = np.ascontiguousarray(label_offsets, dtype=np.int32)
    L.oracle_topk(_ptr(matrix, _f32p), matrix.strides[0] // 4, _ptr(labels, _i32p),
                  cols if labels is not None else 0, _ptr(label_offsets, _i32p), rows, cols, k,
                  _ptr(out_d, _f32p), _ptr(out_l, _i32p), k)
    return out_d, out_l


def topk_serial(matrix, k):
    L = lib()
    matrix = np.ascontiguousarray(matrix, dtype=np.float32)
    rows, cols = matrix.shape
    out_d = np.empty((rows, k), dtype=np.float32)
    out_l = np.empty((rows, k), dtype=np.int32)
    L.oracle_topk_serial(_ptr(matrix, _f32p), cols, rows, cols, k, _ptr(out_d, _f32p),
                         _ptr(out_l, _i32p))
    return out_d, out_l


def topk_parallel(matrix, k, threads=0):
    L = lib()
    matrix = np.ascontiguousarray(matrix, dtype=np.float32)
    rows, cols = matrix.shape
    out_d = np.empty((rows, k), dtype=np.float32)
    out_l = np.empty((rows, k), dtype=np.int32)
    used = L.oracle_topk_parallel(_ptr(matrix, _f32p), cols, rows, cols, k, _ptr(out_d, _f32p),
                                  _ptr(out_l, _i32p), threads)
    return out_d, out_l, used


def checksum(labels_row):
    a = np.ascontiguousarray(labels_row, dtype=np.int32)
    return int(lib().oracle_checksum(_ptr(a, _i32p), a.size))


def verify(exp_d, exp_l, act_d, act_l, k):
    e_d = np.ascontiguousarray(exp_d, dtype=np.float32).ravel()
    e_l = np.ascontiguousarray(exp_l, dtype=np.int32).ravel()
    a_d = np.ascontiguousarray(act_d, dtype=np.float32).ravel()
    a_l = np.ascontiguousarray(act_l, dtype=np.int32).ravel()
    bad = _sz(0)
    ok = lib().oracle_verify(_ptr(e_d, _f32p), _ptr(e_l, _i32p), _ptr(a_d, _f32p), _ptr(a_l, _i32p),
                             e_d.size, k, ctypes.byref(bad))
    return bool(ok), int(bad.value)


def parse_number(text):
    return int(lib().oracle_parse_number(text.encode()))


def parse_dim3(text):
    out = (ctypes.c_uint64 * 3)()
    lib().oracle_parse_dim3(text.encode(), out)
    return tuple(int(v) for v in out)
