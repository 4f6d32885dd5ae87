"""Thin Python view of the C ABI in include/mcsparse.h.

Names and argument order are those of the C functions; every call goes through
libmcsparse.so.  Device memory is passed as raw pointers (torch tensors' data_ptr()); torch is
only the allocator here.
"""
import ctypes

import numpy as np

from . import _lib

# ---- enum values (include/mcsparse.h) ----
STATUS_SUCCESS = 0
STATUS_NOT_INITIALIZED = 1
STATUS_ALLOC_FAILED = 2
STATUS_INVALID_VALUE = 3
STATUS_INTERNAL_ERROR = 7
STATUS_NOT_SUPPORTED = 10
STATUS_INSUFFICIENT_RESOURCES = 11

OP_N, OP_T, OP_C = 0, 1, 2
BASE_ZERO, BASE_ONE = 0, 1
PTR_HOST, PTR_DEVICE = 0, 1
ACTION_SYMBOLIC, ACTION_NUMERIC = 0, 1
FORMAT_CSR, FORMAT_CSC, FORMAT_COO, FORMAT_COO_AOS, FORMAT_BLOCKED_ELL = 1, 2, 3, 4, 5
ORDER_COL, ORDER_ROW = 1, 2
INDEX_16U, INDEX_32I, INDEX_64I = 1, 2, 3
R_32F, R_64F, R_16F, C_32F, C_64F, R_32I = 0, 1, 2, 4, 5, 10
SPMV_ALG_DEFAULT = 0
SPMV_CSR_ALG1 = 2  # need not give the same bits on every run
SPMV_CSR_ALG2 = 3  # the same bits on every run
SPMM_ALG_DEFAULT = 0
CSR2CSC_ALG1 = 1
ROW_BIN_COUNT = 33
FAMILY_AUTO, FAMILY_VECTOR, FAMILY_MERGE = 0, 1, 2

_DTYPE_OF = {np.dtype(np.float32): R_32F, np.dtype(np.float64): R_64F}


class McsparseError(RuntimeError):
    def __init__(self, status, where):
        self.status = status
        name = _lib.load().mcsparseGetErrorName(status).decode()
        super().__init__("%s returned %s" % (where, name))


def check(status, where="mcsparse call"):
    if status != STATUS_SUCCESS:
        raise McsparseError(status, where)


def maca_type(dtype):
    """macaDataType of a numpy/torch real dtype."""
    try:
        return _DTYPE_OF[np.dtype(dtype)]
    except TypeError:
        import torch  # torch dtypes
        return {torch.float32: R_32F, torch.float64: R_64F}[dtype]


def _ptr(t):
    """Raw address of a torch tensor / numpy array / int / None."""
    if t is None:
        return None
    if isinstance(t, int):
        return t
    if hasattr(t, "data_ptr"):
        return t.data_ptr()
    return t.ctypes.data


def _scalar(value, dtype_code):
    """Host scalar of the compute type, as a ctypes object whose address can be passed."""
    return (ctypes.c_float if dtype_code == R_32F else ctypes.c_double)(value)


class Handle:
    """mcsparseHandle_t with its stream bound to torch's current stream by default."""

    def __init__(self, stream=None):
        self.lib = _lib.load()
        self._h = ctypes.c_void_p()
        check(self.lib.mcsparseCreate(ctypes.byref(self._h)), "mcsparseCreate")
        if stream is not None:
            self.set_stream(stream)

    @property
    def ptr(self):
        return self._h

    def set_stream(self, raw_stream):
        check(self.lib.mcsparseSetStream(self._h, ctypes.c_void_p(raw_stream)), "mcsparseSetStream")

    def set_pointer_mode(self, mode):
        check(self.lib.mcsparseSetPointerMode(self._h, mode), "mcsparseSetPointerMode")

    def set_spmv_deterministic(self, on):
        check(self.lib.mcsparseSetSpMVDeterministic(self._h, 1 if on else 0), "mcsparseSetSpMVDeterministic")

    def spmv_deterministic(self):
        out = ctypes.c_int(-1)
        check(self.lib.mcsparseGetSpMVDeterministic(self._h, ctypes.byref(out)), "mcsparseGetSpMVDeterministic")
        return bool(out.value)

    def set_spmv_preprocess_trial(self, on):
        """mcsparseSetSpMVPreprocessTrial: whether mcsparseSpMV_preprocess times its copy against the row kernels and
        keeps it only where it is faster (the default) or keeps every copy."""
        check(self.lib.mcsparseSetSpMVPreprocessTrial(self._h, 1 if on else 0), "mcsparseSetSpMVPreprocessTrial")

    def spmv_preprocess_trial(self):
        out = ctypes.c_int(-1)
        check(self.lib.mcsparseGetSpMVPreprocessTrial(self._h, ctypes.byref(out)), "mcsparseGetSpMVPreprocessTrial")
        return bool(out.value)

    def destroy(self):
        if self._h:
            self.lib.mcsparseDestroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class SpMat:
    """mcsparseSpMatDescr_t for CSR or CSC device arrays (borrowed, kept alive by this object)."""

    def __init__(self, rows, cols, nnz, offsets, indices, values, base=BASE_ZERO, fmt=FORMAT_CSR,
                 index_type=INDEX_32I, value_type=None):
        self.lib = _lib.load()
        self._keep = (offsets, indices, values)
        self._d = ctypes.c_void_p()
        vt = value_type if value_type is not None else maca_type(values.dtype)
        if fmt == FORMAT_COO:  # offsets = row indices, indices = column indices
            check(self.lib.mcsparseCreateCoo(ctypes.byref(self._d), rows, cols, nnz, _ptr(offsets), _ptr(indices),
                                             _ptr(values), index_type, base, vt), "mcsparseCreateCoo")
            return
        create = self.lib.mcsparseCreateCsr if fmt == FORMAT_CSR else self.lib.mcsparseCreateCsc
        check(create(ctypes.byref(self._d), rows, cols, nnz, _ptr(offsets), _ptr(indices), _ptr(values), index_type,
                     index_type, base, vt), "mcsparseCreateCsr/Csc")

    @property
    def ptr(self):
        return self._d

    def set_plan(self, family, lanes=0):
        check(self.lib.mcsparseSpMatSetSpMVPlan(self._d, family, lanes), "mcsparseSpMatSetSpMVPlan")

    def plan(self):
        fam, lanes = ctypes.c_int(), ctypes.c_int()
        check(self.lib.mcsparseSpMatGetSpMVPlan(self._d, ctypes.byref(fam), ctypes.byref(lanes)))
        return fam.value, lanes.value

    def set_band_bytes(self, band_bytes):
        check(self.lib.mcsparseSpMatSetSpMVBandBytes(self._d, band_bytes), "mcsparseSpMatSetSpMVBandBytes")

    def spmv_preprocess_state(self):
        """(state, bands, rows_per_tile) left by mcsparseSpMV_preprocess; state 2 = banded copy, 3 = copy in column
        order (both in use), 0 = none."""
        state, bands, rows = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        check(self.lib.mcsparseSpMatGetSpMVPreprocess(self._d, ctypes.byref(state), ctypes.byref(bands),
                                                      ctypes.byref(rows)))
        return state.value, bands.value, rows.value

    def spmm_schedule(self):
        """(state, entries) left by mcsparseSpMM_preprocess; state 2 = merged column lists, 3 = diagonal blocks over
        groups of eight rows, 4 = diagonal blocks over groups of strips (all three in use), 1 = built and declined."""
        state, entries = ctypes.c_int(), ctypes.c_int64()
        check(self.lib.mcsparseSpMatGetSpMMSchedule(self._d, ctypes.byref(state), ctypes.byref(entries)))
        return state.value, entries.value

    def destroy(self):
        if self._d:
            self.lib.mcsparseDestroySpMat(self._d)
            self._d = ctypes.c_void_p()

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class DnVec:
    def __init__(self, values, size=None, value_type=None):
        self.lib = _lib.load()
        self._keep = values
        self._d = ctypes.c_void_p()
        n = size if size is not None else values.numel()
        vt = value_type if value_type is not None else maca_type(values.dtype)
        check(self.lib.mcsparseCreateDnVec(ctypes.byref(self._d), n, _ptr(values), vt), "mcsparseCreateDnVec")

    @property
    def ptr(self):
        return self._d

    def destroy(self):
        if self._d:
            self.lib.mcsparseDestroyDnVec(self._d)
            self._d = ctypes.c_void_p()

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class DnMat:
    def __init__(self, rows, cols, ld, values, order=ORDER_ROW, value_type=None):
        self.lib = _lib.load()
        self._keep = values
        self._d = ctypes.c_void_p()
        vt = value_type if value_type is not None else maca_type(values.dtype)
        check(self.lib.mcsparseCreateDnMat(ctypes.byref(self._d), rows, cols, ld, _ptr(values), vt, order),
              "mcsparseCreateDnMat")

    @property
    def ptr(self):
        return self._d

    def destroy(self):
        if self._d:
            self.lib.mcsparseDestroyDnMat(self._d)
            self._d = ctypes.c_void_p()

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


# ---- compute calls: return the status code (tests of error paths need it) -------------------

def spmv_buffer_size(handle, op, alpha, mat, x, beta, y, compute_type):
    size = ctypes.c_size_t(0)
    a, b = _scalar(alpha, compute_type), _scalar(beta, compute_type)
    st = handle.lib.mcsparseSpMV_bufferSize(handle.ptr, op, ctypes.addressof(a), mat.ptr, x.ptr, ctypes.addressof(b),
                                            y.ptr, compute_type, SPMV_ALG_DEFAULT, ctypes.byref(size))
    return st, size.value


def spmv(handle, op, alpha, mat, x, beta, y, compute_type, buffer, alg=0):
    """alpha/beta are Python floats (host pointer mode) or device tensors (device pointer mode)."""
    if hasattr(alpha, "data_ptr"):
        pa, pb = alpha.data_ptr(), beta.data_ptr()
        keep = None
    else:
        a, b = _scalar(alpha, compute_type), _scalar(beta, compute_type)
        pa, pb = ctypes.addressof(a), ctypes.addressof(b)
        keep = (a, b)
    st = handle.lib.mcsparseSpMV(handle.ptr, op, pa, mat.ptr, x.ptr, pb, y.ptr, compute_type, alg, _ptr(buffer))
    del keep
    return st


def spmv_preprocess_buffer_size(handle, op, alpha, mat, x, beta, y, compute_type, alg=0):
    size = ctypes.c_size_t(0)
    a, b = _scalar(alpha, compute_type), _scalar(beta, compute_type)
    st = handle.lib.mcsparseSpMV_preprocess_bufferSize(handle.ptr, op, ctypes.addressof(a), mat.ptr, x.ptr,
                                                       ctypes.addressof(b), y.ptr, compute_type, alg,
                                                       ctypes.byref(size))
    return st, size.value


def spmv_preprocess(handle, op, alpha, mat, x, beta, y, compute_type, buffer, alg=0):
    a, b = _scalar(alpha, compute_type), _scalar(beta, compute_type)
    return handle.lib.mcsparseSpMV_preprocess(handle.ptr, op, ctypes.addressof(a), mat.ptr, x.ptr, ctypes.addressof(b),
                                              y.ptr, compute_type, alg, _ptr(buffer))


def spmv_static_buffer(handle, op, alpha, mat, x, beta, y, compute_type):
    """mcsparseSpMV_staticBuffer: host scalars only, scratch inside the library."""
    a, b = _scalar(alpha, compute_type), _scalar(beta, compute_type)
    return handle.lib.mcsparseSpMV_staticBuffer(handle.ptr, op, ctypes.addressof(a), mat.ptr, x.ptr,
                                                ctypes.addressof(b), y.ptr, compute_type, SPMV_ALG_DEFAULT)


def stream_probe(handle, mode, src, dst, nbytes, sink):
    """mcsparseXstreamProbe: mode 0 reads src, 1 writes dst, 2 copies (torch tensors; sink: int32/uint32 tensor)."""
    return handle.lib.mcsparseXstreamProbe(handle.ptr, mode, ctypes.c_void_p(src.data_ptr() if src is not None else 0),
                                           ctypes.c_void_p(dst.data_ptr() if dst is not None else 0), nbytes,
                                           ctypes.c_void_p(sink.data_ptr() if sink is not None else 0),
                                           sink.numel() if sink is not None else 0)


def spmm_buffer_size(handle, op_a, op_b, alpha, mat, B, beta, C, compute_type):
    size = ctypes.c_size_t(0)
    a, b = _scalar(alpha, compute_type), _scalar(beta, compute_type)
    st = handle.lib.mcsparseSpMM_bufferSize(handle.ptr, op_a, op_b, ctypes.addressof(a), mat.ptr, B.ptr,
                                            ctypes.addressof(b), C.ptr, compute_type, SPMM_ALG_DEFAULT,
                                            ctypes.byref(size))
    return st, size.value


def spmm_preprocess(handle, op_a, op_b, alpha, mat, B, beta, C, compute_type, buffer):
    a, b = _scalar(alpha, compute_type), _scalar(beta, compute_type)
    return handle.lib.mcsparseSpMM_preprocess(handle.ptr, op_a, op_b, ctypes.addressof(a), mat.ptr, B.ptr,
                                              ctypes.addressof(b), C.ptr, compute_type, SPMM_ALG_DEFAULT, _ptr(buffer))


def spmm(handle, op_a, op_b, alpha, mat, B, beta, C, compute_type, buffer):
    a, b = _scalar(alpha, compute_type), _scalar(beta, compute_type)
    return handle.lib.mcsparseSpMM(handle.ptr, op_a, op_b, ctypes.addressof(a), mat.ptr, B.ptr, ctypes.addressof(b),
                                   C.ptr, compute_type, SPMM_ALG_DEFAULT, _ptr(buffer))


def xcsr2coo(handle, csr_rows, nnz, m, coo_rows, base):
    return handle.lib.mcsparseXcsr2coo(handle.ptr, _ptr(csr_rows), nnz, m, _ptr(coo_rows), base)


def xcoo2csr(handle, coo_rows, nnz, m, csr_rows, base):
    return handle.lib.mcsparseXcoo2csr(handle.ptr, _ptr(coo_rows), nnz, m, _ptr(csr_rows), base)


def csr2csc_buffer_size(handle, m, n, nnz, csr_val, csr_rows, csr_cols, csc_val, csc_cols, csc_rows, val_type,
                        action, base):
    size = ctypes.c_size_t(0)
    st = handle.lib.mcsparseCsr2cscEx2_bufferSize(handle.ptr, m, n, nnz, _ptr(csr_val), _ptr(csr_rows),
                                                  _ptr(csr_cols), _ptr(csc_val), _ptr(csc_cols), _ptr(csc_rows),
                                                  val_type, action, base, CSR2CSC_ALG1, ctypes.byref(size))
    return st, size.value


def csr2csc(handle, m, n, nnz, csr_val, csr_rows, csr_cols, csc_val, csc_cols, csc_rows, val_type, action, base,
            buffer):
    """csc_cols = n+1 column offsets, csc_rows = nnz row indices (the reference's naming)."""
    return handle.lib.mcsparseCsr2cscEx2(handle.ptr, m, n, nnz, _ptr(csr_val), _ptr(csr_rows), _ptr(csr_cols),
                                         _ptr(csc_val), _ptr(csc_cols), _ptr(csc_rows), val_type, action, base,
                                         CSR2CSC_ALG1, _ptr(buffer))


def csr_row_bins(handle, m, csr_rows, base, row_bins, bin_hist):
    return handle.lib.mcsparseXcsrRowBins(handle.ptr, m, _ptr(csr_rows), base, _ptr(row_bins), _ptr(bin_hist))


def sort_buffer_size(handle, kind, m, n, nnz, a, b):
    """kind is "csr", "csc" or "coo"; a, b are the two index arrays of that structure."""
    fn = {"csr": handle.lib.mcsparseXcsrsort_bufferSizeExt, "csc": handle.lib.mcsparseXcscsort_bufferSizeExt,
          "coo": handle.lib.mcsparseXcoosort_bufferSizeExt}[kind]
    size = ctypes.c_size_t(0)
    st = fn(handle.ptr, m, n, nnz, _ptr(a), _ptr(b), ctypes.byref(size))
    return st, size.value


def xcsrsort(handle, m, n, nnz, descr, csr_rows, csr_cols, perm, buffer):
    return handle.lib.mcsparseXcsrsort(handle.ptr, m, n, nnz, descr, _ptr(csr_rows), _ptr(csr_cols), _ptr(perm),
                                       _ptr(buffer))


def xcscsort(handle, m, n, nnz, descr, csc_cols, csc_rows, perm, buffer):
    return handle.lib.mcsparseXcscsort(handle.ptr, m, n, nnz, descr, _ptr(csc_cols), _ptr(csc_rows), _ptr(perm),
                                       _ptr(buffer))


def xcoosort_by_row(handle, m, n, nnz, coo_rows, coo_cols, perm, buffer):
    return handle.lib.mcsparseXcoosortByRow(handle.ptr, m, n, nnz, _ptr(coo_rows), _ptr(coo_cols), _ptr(perm),
                                            _ptr(buffer))


def xcoosort_by_column(handle, m, n, nnz, coo_rows, coo_cols, perm, buffer):
    return handle.lib.mcsparseXcoosortByColumn(handle.ptr, m, n, nnz, _ptr(coo_rows), _ptr(coo_cols), _ptr(perm),
                                               _ptr(buffer))


def create_identity_permutation(handle, n, p):
    return handle.lib.mcsparseCreateIdentityPermutation(handle.ptr, n, _ptr(p))


def gthr(handle, nnz, y, x_val, x_ind, base):
    fn = handle.lib.mcsparseSgthr if maca_type(x_val.dtype) == R_32F else handle.lib.mcsparseDgthr
    return fn(handle.ptr, nnz, _ptr(y), _ptr(x_val), _ptr(x_ind), base)
