"""ctypes front-end of the CPU oracle (TEST INFRASTRUCTURE ONLY).

Only the test-suite, the smoke check and the benchmark's CPU-baseline leg may
import this module; the product package never does.  It loads
``oracle/libmx_oracle.so`` (built by ``oracle/Makefile`` from ``mx_oracle.c``)
and converts between numpy arrays and the C structures.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmx_oracle.so")


def build(force=False):
    """Compile the oracle with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libmx_oracle.so"])
    return _LIB_PATH


class _Partition(C.Structure):
    _fields_ = [
        ("elem", C.c_int), ("rows", C.c_int), ("cols", C.c_int), ("nnz", C.c_int),
        ("fragM", C.c_int), ("fragK", C.c_int),
        ("dCols", C.c_int), ("sCols", C.c_int), ("nnzColD", C.c_int), ("nnzColS", C.c_int),
        ("dRows", C.c_int), ("sRows", C.c_int), ("nnzRowD", C.c_int), ("nnzRowS", C.c_int),
        ("cols_ratio", C.c_float), ("tc_nnz_ratio", C.c_double),
        ("descColId", C.c_void_p), ("newArray", C.c_void_p), ("rId", C.c_void_p),
        ("newArray_", C.c_void_p),
        ("ddRowPtr", C.c_void_p), ("ddColInd", C.c_void_p), ("ddVal", C.c_void_p),
        ("chunkNum", C.c_int), ("totalTcFrags", C.c_int), ("tcValCount", C.c_int),
        ("chunkPtr", C.c_void_p), ("sparse_AToX_index", C.c_void_p), ("fragPtr", C.c_void_p),
        ("fragBit", C.c_void_p), ("tcVal", C.c_void_p),
        ("nnzCD", C.c_int),
        ("cdRowPtr", C.c_void_p), ("cdColInd", C.c_void_p), ("cdVal", C.c_void_p),
    ]


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        L.ora_h2f.restype = C.c_float
        L.ora_h2f.argtypes = [C.c_uint16]
        L.ora_f2h.restype = C.c_uint16
        L.ora_f2h.argtypes = [C.c_float]
        L.ora_threshold.restype = C.c_int
        L.ora_threshold.argtypes = [C.c_int, C.c_float]
        L.ora_partition_create.restype = C.POINTER(_Partition)
        L.ora_partition_create.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p,
                                           C.c_void_p, C.c_void_p, C.c_float, C.c_float]
        L.ora_partition_free.argtypes = [C.POINTER(_Partition)]
        L.ora_transpose.restype = C.c_int
        L.ora_transpose.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                                    C.c_void_p, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p),
                                    C.POINTER(C.c_void_p)]
        L.ora_free.argtypes = [C.c_void_p]
        L.ora_hash.restype = C.c_uint64
        L.ora_hash.argtypes = [C.c_void_p, C.c_size_t, C.c_uint64]
        L.ora_eqcheck_f64.restype = C.c_int
        L.ora_eqcheck_f64.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_double]
        L.ora_eqcheck_f16.restype = C.c_int
        L.ora_eqcheck_f16.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_float]
        for name in ("ora_spmv_f64", "ora_spmv_f16_f32acc", "ora_spmv_f16_halfacc",
                     "ora_tcspmv_f64", "ora_tcspmv_f16", "ora_hybrid_f64", "ora_hybrid_f16"):
            getattr(L, name).restype = None
        L.ora_spmv_f64.argtypes = [C.c_void_p] * 5 + [C.c_int]
        L.ora_spmv_f16_f32acc.argtypes = [C.c_void_p] * 6 + [C.c_int]
        L.ora_spmv_f16_halfacc.argtypes = [C.c_void_p] * 5 + [C.c_int]
        L.ora_tcspmv_f64.argtypes = [C.c_void_p] * 7 + [C.c_int]
        L.ora_tcspmv_f16.argtypes = [C.c_void_p] * 7 + [C.c_int]
        L.ora_hybrid_f64.argtypes = [C.POINTER(_Partition), C.c_void_p, C.c_void_p]
        L.ora_hybrid_f16.argtypes = [C.POINTER(_Partition), C.c_void_p, C.c_void_p]
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _val_dtype(elem):
    return np.float64 if elem == 8 else np.float16


def as_bits16(a):
    """float16 array -> its uint16 bit pattern (no copy when already uint16)."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        return a.view(np.uint16)
    assert a.dtype == np.uint16
    return a


def spmv_f64(val, rowPtr, colInd, x, y0=None):
    rowPtr, colInd = _i32(rowPtr), _i32(colInd)
    val = np.ascontiguousarray(val, dtype=np.float64)
    x = np.ascontiguousarray(x, dtype=np.float64)
    rows = len(rowPtr) - 1
    y = np.zeros(rows, np.float64) if y0 is None else np.array(y0, dtype=np.float64)
    lib().ora_spmv_f64(_p(val), _p(rowPtr), _p(colInd), _p(x), _p(y), rows)
    return y


def spmv_f16_f32acc(val, rowPtr, colInd, x):
    """Returns (y as float32, y rounded once to float16)."""
    rowPtr, colInd = _i32(rowPtr), _i32(colInd)
    val, x = as_bits16(val), as_bits16(x)
    rows = len(rowPtr) - 1
    y32 = np.zeros(rows, np.float32)
    y16 = np.zeros(rows, np.uint16)
    lib().ora_spmv_f16_f32acc(_p(val), _p(rowPtr), _p(colInd), _p(x), _p(y32), _p(y16), rows)
    return y32, y16.view(np.float16)


def spmv_f16_halfacc(val, rowPtr, colInd, x):
    rowPtr, colInd = _i32(rowPtr), _i32(colInd)
    val, x = as_bits16(val), as_bits16(x)
    rows = len(rowPtr) - 1
    y = np.zeros(rows, np.uint16)
    lib().ora_spmv_f16_halfacc(_p(val), _p(rowPtr), _p(colInd), _p(x), _p(y), rows)
    return y.view(np.float16)


def eqcheck(a, b, tol):
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    if a.dtype == np.float64:
        return lib().ora_eqcheck_f64(_p(a), _p(b), len(a), tol)
    return lib().ora_eqcheck_f16(_p(as_bits16(a)), _p(as_bits16(b)), len(a), tol)


def transpose(ptr, ind, val, inner):
    """Counting-sort transpose of a compressed matrix with `inner` minor indices."""
    ptr, ind = _i32(ptr), _i32(ind)
    val = np.ascontiguousarray(val)
    elem = val.dtype.itemsize
    outer, nnz = len(ptr) - 1, len(ind)
    tp, ti, tv = C.c_void_p(), C.c_void_p(), C.c_void_p()
    rc = lib().ora_transpose(elem, outer, inner, nnz, _p(ptr), _p(ind), _p(val),
                             C.byref(tp), C.byref(ti), C.byref(tv))
    assert rc == 0
    out = (_copy(tp.value, inner + 1, np.int32), _copy(ti.value, nnz, np.int32),
           _copy(tv.value, nnz, val.dtype))
    for q in (tp, ti, tv):
        lib().ora_free(q)
    return out


def _copy(addr, n, dtype):
    dtype = np.dtype(dtype)
    if n <= 0 or not addr:
        return np.zeros(0, dtype)
    buf = (C.c_char * (n * dtype.itemsize)).from_address(addr)
    return np.frombuffer(buf, dtype=dtype, count=n).copy()


class Partition:
    """Numpy copy of an ``ora_partition`` (keeps the C object for ora_hybrid_*)."""

    FIELDS = ("dCols", "sCols", "nnzColD", "nnzColS", "dRows", "sRows", "nnzRowD", "nnzRowS",
              "chunkNum", "totalTcFrags", "tcValCount", "nnzCD", "rows", "cols", "nnz",
              "fragM", "fragK", "elem", "cols_ratio", "tc_nnz_ratio")

    def __init__(self, ptr):
        self._ptr = ptr
        s = ptr.contents
        for f in self.FIELDS:
            setattr(self, f, getattr(s, f))
        vt = _val_dtype(s.elem)
        bt = np.uint32 if s.elem == 8 else np.uint64
        self.descColId = _copy(s.descColId, s.cols if s.dCols or s.dRows else 0, np.int32)
        self.newArray = _copy(s.newArray, s.sCols, np.int32)
        self.rId = _copy(s.rId, s.dRows, np.int32)
        self.newArray_ = _copy(s.newArray_, s.sRows, np.int32)
        self.ddRowPtr = _copy(s.ddRowPtr, s.dRows + 1, np.int32)
        self.ddColInd = _copy(s.ddColInd, s.nnzRowD, np.int32)
        self.ddVal = _copy(s.ddVal, s.nnzRowD, vt)
        self.chunkPtr = _copy(s.chunkPtr, s.chunkNum + 1, np.int32)
        self.sparse_AToX_index = _copy(s.sparse_AToX_index, s.totalTcFrags * s.fragK, np.int32)
        self.fragPtr = _copy(s.fragPtr, s.totalTcFrags + 1, np.int32)
        self.fragBit = _copy(s.fragBit, s.totalTcFrags, bt)
        self.tcVal = _copy(s.tcVal, s.tcValCount, vt)
        self.cdRowPtr = _copy(s.cdRowPtr, s.rows + 1, np.int32)
        self.cdColInd = _copy(s.cdColInd, s.nnzCD, np.int32)
        self.cdVal = _copy(s.cdVal, s.nnzCD, vt)

    def hybrid(self, x):
        """y of the whole hybrid product, computed on the CPU from this partition."""
        if self.elem == 8:
            x = np.ascontiguousarray(x, dtype=np.float64)
            y = np.zeros(self.rows, np.float64)
            lib().ora_hybrid_f64(self._ptr, _p(x), _p(y))
        else:
            x = as_bits16(x)
            y = np.zeros(self.rows, np.float32)
            lib().ora_hybrid_f16(self._ptr, _p(x), _p(y))
        return y

    def __del__(self):
        try:
            if self._ptr:
                lib().ora_partition_free(self._ptr)
                self._ptr = None
        except Exception:
            pass


def partition(rowPtr, colInd, val, cols, tau_c, tau_r):
    rowPtr, colInd = _i32(rowPtr), _i32(colInd)
    val = np.ascontiguousarray(val)
    if val.dtype == np.float16:
        val = val.view(np.uint16)
    assert val.dtype in (np.float64, np.uint16)
    rows, nnz = len(rowPtr) - 1, len(colInd)
    ptr = lib().ora_partition_create(val.dtype.itemsize, rows, cols, nnz, _p(rowPtr), _p(colInd),
                                     _p(val), np.float32(tau_c), np.float32(tau_r))
    return Partition(ptr)


def tcspmv(part, x_d):
    """Tile-only product A_dd * x_d from a Partition's canonical tile arrays."""
    if part.elem == 8:
        x_d = np.ascontiguousarray(x_d, dtype=np.float64)
        y = np.zeros(part.dRows, np.float64)
        lib().ora_tcspmv_f64(_p(x_d), _p(y), _p(part.chunkPtr), _p(part.fragPtr), _p(part.fragBit),
                             _p(part.tcVal), _p(part.sparse_AToX_index), part.dRows)
    else:
        x_d = as_bits16(x_d)
        y = np.zeros(part.dRows, np.float32)
        lib().ora_tcspmv_f16(_p(x_d), _p(y), _p(part.chunkPtr), _p(part.fragPtr), _p(part.fragBit),
                             _p(part.tcVal), _p(part.sparse_AToX_index), part.dRows)
    return y


def threshold(nnz, frac):
    return lib().ora_threshold(int(nnz), np.float32(frac))


def hash_arrays(*arrays):
    h = 0
    for a in arrays:
        a = np.ascontiguousarray(a)
        h = lib().ora_hash(_p(a), a.nbytes, h) if a.nbytes else lib().ora_hash(None, 0, h)
    return h
