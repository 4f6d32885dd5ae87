"""ctypes binding of the CPU oracle (oracle/oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py.  The mcsparse_amd package never imports this module.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")

_c_i64 = ctypes.c_int64
_c_int = ctypes.c_int
_c_dbl = ctypes.c_double
_vp = ctypes.c_void_p


def build(force=False):
    """Compile liboracle.so next to oracle.c."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)


_lib = None


def use_native_build():
    """Switches this binding to a copy of oracle.c compiled for the host it runs on
    (-O3 -march=native), for the timed CPU baseline.  The committed build recipe targets a generic
    x86-64-v3 machine because its output travels between hosts.  Returns False, and keeps the
    portable library, when no compiler is at hand."""
    global _lib, _native
    if _native is not None:
        return _native
    import tempfile
    out = os.path.join(tempfile.mkdtemp(prefix="oracle_native_"), "liboracle_native.so")
    cmd = ["gcc", "-O3", "-march=native", "-fopenmp", "-fPIC", "-std=c11", "-shared", "-o", out,
           os.path.join(_HERE, "oracle.c"), "-lm"]
    try:
        subprocess.check_call(cmd, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
        _lib = ctypes.CDLL(out)
        _native = True
    except (OSError, subprocess.CalledProcessError):
        _native = False
    return _native


_native = None


def first_touch_copy(a):
    """A copy of `a` whose pages are first written by the OpenMP threads (static schedule)."""
    a = np.ascontiguousarray(a)
    out = np.empty_like(a)
    if a.nbytes:
        lib().orc_first_touch_copy.restype = None
        lib().orc_first_touch_copy(_p(out), _p(a), _c_i64(a.nbytes))
    return out


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(_vp)


def _idx(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.int32:
        a = a.view(np.uint32)
    assert a.dtype == np.uint32, a.dtype
    return a


def spmv(op_t, m, n, base, ptr, col, val, alpha, beta, x, y=None):
    """Returns (y_ref, bound) as np.longdouble arrays; see orc_spmv_* in oracle.c."""
    ptr, col = _idx(ptr), _idx(col)
    val = np.ascontiguousarray(val)
    x = np.ascontiguousarray(x, dtype=val.dtype)
    if y is not None:
        y = np.ascontiguousarray(y, dtype=val.dtype)
    fn = {np.dtype(np.float32): lib().orc_spmv_f32, np.dtype(np.float64): lib().orc_spmv_f64}[val.dtype]
    out_len = n if op_t else m
    y_ref = np.zeros(out_len, dtype=np.longdouble)
    bound = np.zeros(out_len, dtype=np.longdouble)
    fn.restype = None
    fn(_c_int(int(bool(op_t))), _c_i64(m), _c_i64(n), _c_int(base), _p(ptr), _p(col), _p(val), _c_dbl(alpha),
       _c_dbl(beta), _p(x), _p(y), _p(y_ref), _p(bound))
    return y_ref, bound


def spmm(m, n, base, ptr, col, val, alpha, beta, B, ldb, b_row_major, C, ldc, c_row_major):
    """Returns (c_ref, bound) as dense m x n np.longdouble arrays."""
    ptr, col = _idx(ptr), _idx(col)
    val = np.ascontiguousarray(val)
    B = np.ascontiguousarray(B, dtype=val.dtype)
    if C is not None:
        C = np.ascontiguousarray(C, dtype=val.dtype)
    fn = {np.dtype(np.float32): lib().orc_spmm_f32, np.dtype(np.float64): lib().orc_spmm_f64}[val.dtype]
    c_ref = np.zeros((m, n), dtype=np.longdouble)
    bound = np.zeros((m, n), dtype=np.longdouble)
    fn.restype = None
    fn(_c_i64(m), _c_i64(n), _c_int(base), _p(ptr), _p(col), _p(val), _c_dbl(alpha), _c_dbl(beta), _p(B),
       _c_i64(ldb), _c_int(int(bool(b_row_major))), _p(C), _c_i64(ldc), _c_int(int(bool(c_row_major))), _p(c_ref),
       _p(bound))
    return c_ref, bound


def csr2coo(m, base, ptr, nnz):
    ptr = _idx(ptr)
    out = np.zeros(nnz, dtype=np.uint32)
    lib().orc_csr2coo.restype = None
    lib().orc_csr2coo(_c_i64(m), _c_int(base), _p(ptr), _p(out))
    return out


def coo2csr(nnz, m, base, coo_rows):
    coo_rows = _idx(coo_rows)
    out = np.zeros(m + 1, dtype=np.uint32)
    lib().orc_coo2csr.restype = None
    lib().orc_coo2csr(_c_i64(nnz), _c_i64(m), _c_int(base), _p(coo_rows), _p(out))
    return out


def csr2csc(m, n, base, ptr, col, val=None, method="radix2"):
    """Returns (col_ptr, row_ind, csc_val); csc_val is None when val is None.

    method "radix2" follows the reference step by step, "counting" is the fast equivalent, "omp" the
    multi-threaded one that bench.py times as the CPU baseline."""
    ptr, col = _idx(ptr), _idx(col)
    nnz = int(col.shape[0])
    col_ptr = np.zeros(n + 1, dtype=np.uint32)
    row_ind = np.zeros(nnz, dtype=np.uint32)
    if val is not None:
        val = np.ascontiguousarray(val)
        csc_val = np.zeros_like(val)
        vb = val.dtype.itemsize
    else:
        csc_val, vb = None, 0
    fn = {"radix2": lib().orc_csr2csc_radix2, "counting": lib().orc_csr2csc_counting,
          "omp": lib().orc_csr2csc_omp}[method]
    fn.restype = _c_int
    rc = fn(_c_i64(m), _c_i64(n), _c_i64(nnz), _c_int(base), _p(ptr), _p(col), _p(val), _c_i64(vb), _p(col_ptr),
            _p(row_ind), _p(csc_val))
    if rc != 0:
        raise MemoryError("oracle csr2csc")
    return col_ptr, row_ind, csc_val


def coosort(major_extent, minor_extent, major, minor, perm=None):
    """Stable sort by (major, minor); returns new (major, minor, perm) arrays, perm None if not given."""
    major, minor = _idx(major).copy(), _idx(minor).copy()
    perm = None if perm is None else _idx(perm).copy()
    fn = lib().orc_coosort
    fn.restype = _c_int
    if fn(_c_i64(major_extent), _c_i64(minor_extent), _c_i64(major.shape[0]), _p(major), _p(minor), _p(perm)) != 0:
        raise MemoryError("oracle coosort")
    return major, minor, perm


def csrsort(m, n, base, ptr, col, perm=None):
    """Sorts the columns inside every row; returns new (col, perm) arrays."""
    ptr, col = _idx(ptr), _idx(col).copy()
    perm = None if perm is None else _idx(perm).copy()
    fn = lib().orc_csrsort
    fn.restype = _c_int
    if fn(_c_i64(m), _c_i64(n), _c_i64(col.shape[0]), _c_int(base), _p(ptr), _p(col), _p(perm)) != 0:
        raise MemoryError("oracle csrsort")
    return col, perm


def row_bins(m, ptr):
    """Returns (row_bins uint8[m], hist uint32[34])."""
    ptr = _idx(ptr)
    bins = np.zeros(m, dtype=np.uint8)
    hist = np.zeros(34, dtype=np.uint32)
    lib().orc_row_bins.restype = None
    lib().orc_row_bins(_c_i64(m), _p(ptr), _p(bins), _p(hist))
    return bins, hist


# ---- CPU baseline (timed by bench.py; working precision, OpenMP over rows) ------------------

def max_threads():
    lib().orc_max_threads.restype = _c_int
    return int(lib().orc_max_threads())


def spmv_omp(m, base, ptr, col, val, alpha, beta, x, y, dynamic=False):
    """In place on y."""
    ptr, col = _idx(ptr), _idx(col)
    if val.dtype == np.float32:
        fn, ct = lib().orc_spmv_omp_f32, ctypes.c_float
    else:
        fn, ct = lib().orc_spmv_omp_f64, ctypes.c_double
    fn.restype = None
    fn(_c_i64(m), _c_int(base), _p(ptr), _p(col), _p(val), ct(alpha), ct(beta), _p(x), _p(y), _c_int(int(dynamic)))


def spmm_omp_f32(m, n, base, ptr, col, val, alpha, beta, B, C):
    """Row-major B and C with ld = n; in place on C."""
    ptr, col = _idx(ptr), _idx(col)
    lib().orc_spmm_omp_f32.restype = None
    lib().orc_spmm_omp_f32(_c_i64(m), _c_i64(n), _c_int(base), _p(ptr), _p(col), _p(val), ctypes.c_float(alpha),
                           ctypes.c_float(beta), _p(B), _p(C))


def csr2coo_omp(m, base, ptr, nnz):
    ptr = _idx(ptr)
    out = np.zeros(nnz, dtype=np.uint32)
    lib().orc_csr2coo_omp.restype = None
    lib().orc_csr2coo_omp(_c_i64(m), _c_int(base), _p(ptr), _p(out))
    return out
