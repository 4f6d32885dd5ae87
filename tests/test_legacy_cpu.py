"""Legacy typed entry points and the matrix descriptor: host-side behaviour (no GPU needed).
Expected codes follow mcspSpmvCsrVectorTemplate (src/kernels/level2/spmv/mcsp_spmv_gpu.cpp:203-237),
mcspCsrSpmmTemplate (src/kernels/level3/spmm/mcsp_spmm_gpu.cpp:19-48) and src/common/mcsp_helper.cpp:90-292."""
import ctypes

from mcsparse_amd import api

FAKE = 0x1000


def make(lib):
    h, d = ctypes.c_void_p(), ctypes.c_void_p()
    assert lib.mcsparseCreate(ctypes.byref(h)) == 0
    assert lib.mcsparseCreateMatDescr(ctypes.byref(d)) == 0
    return h, d


def test_mat_descr(lib):
    assert lib.mcsparseCreateMatDescr(None) == api.STATUS_INVALID_VALUE
    h, d = make(lib)
    assert (lib.mcsparseGetMatType(d), lib.mcsparseGetMatFillMode(d), lib.mcsparseGetMatDiagType(d),
            lib.mcsparseGetMatIndexBase(d)) == (0, 2, 0, 0)  # GENERAL, FULL, NON_UNIT, base 0
    sm = ctypes.c_int(-1)
    assert lib.mcsparseGetStorageMode(d, ctypes.byref(sm)) == 0 and sm.value == 0
    assert lib.mcsparseSetMatIndexBase(d, 1) == 0 and lib.mcsparseGetMatIndexBase(d) == 1
    assert lib.mcsparseSetMatIndexBase(d, 2) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseSetMatType(d, 3) == 0 and lib.mcsparseGetMatType(d) == 3
    assert lib.mcsparseSetMatType(d, 9) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseSetMatFillMode(d, 0) == 0 and lib.mcsparseGetMatFillMode(d) == 0
    assert lib.mcsparseSetMatFillMode(d, 5) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseSetMatDiagType(d, 1) == 0 and lib.mcsparseGetMatDiagType(d) == 1
    assert lib.mcsparseSetMatDiagType(d, 4) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseSetStorageMode(d, 1) == 0
    assert lib.mcsparseGetStorageMode(d, ctypes.byref(sm)) == 0 and sm.value == 1
    assert lib.mcsparseSetStorageMode(d, 7) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseGetStorageMode(d, None) == api.STATUS_INVALID_VALUE
    for setter in (lib.mcsparseSetMatIndexBase, lib.mcsparseSetMatType, lib.mcsparseSetMatFillMode,
                   lib.mcsparseSetMatDiagType, lib.mcsparseSetStorageMode):
        assert setter(None, 0) == api.STATUS_INVALID_VALUE
    for getter in (lib.mcsparseGetMatIndexBase, lib.mcsparseGetMatType, lib.mcsparseGetMatFillMode,
                   lib.mcsparseGetMatDiagType):
        assert getter(None) == -1
    assert lib.mcsparseCopyMatDescr(d, d) == api.STATUS_NOT_SUPPORTED  # unimplemented in the reference too
    assert lib.mcsparseDestroyMatDescr(d) == 0 and lib.mcsparseDestroyMatDescr(None) == 0


def test_csrmv_argument_checks(lib):
    h, d = make(lib)
    one = ctypes.c_float(1.0)
    pa = ctypes.addressof(one)
    call = lambda hh=h, a=pa, dd=d, v=FAKE, r=FAKE, c=FAKE, x=FAKE, b=pa, y=FAKE, nnz=5, op=0: lib.mcsparseScsrmv(
        hh, op, 4, 4, nnz, a, dd, v, r, c, x, b, y)
    assert call(hh=None) == api.STATUS_NOT_INITIALIZED
    for kw in ({"a": None}, {"dd": None}, {"v": None}, {"r": None}, {"c": None}, {"x": None}, {"b": None},
               {"y": None}):
        assert call(**kw) == api.STATUS_INVALID_VALUE, kw
    assert call(nnz=0) == 0  # early return before any launch (pointers are fake)
    zero = ctypes.c_float(0.0)
    assert call(a=ctypes.addressof(zero), b=ctypes.addressof(zero)) == 0
    lib.mcsparseSetMatType(d, 1)  # symmetric is not implemented
    assert call() == api.STATUS_NOT_SUPPORTED
    lib.mcsparseSetMatType(d, 0)
    lib.mcsparseSetMatFillMode(d, 0)
    assert call() == api.STATUS_NOT_SUPPORTED
    lib.mcsparseSetMatFillMode(d, 2)
    # CsrmvEx: all types must agree (mcsp_spmv_gpu.cpp:911-914)
    size = ctypes.c_size_t()
    ex = lambda vt=api.R_32F, xt=api.R_32F, et=api.R_32F, nnz=0: lib.mcsparseCsrmvEx(
        h, 0, 0, 4, 4, nnz, pa, api.R_32F, d, FAKE, vt, FAKE, FAKE, FAKE, xt, pa, api.R_32F, FAKE, api.R_32F, et, FAKE)
    assert ex() == 0
    assert ex(xt=api.R_64F) == api.STATUS_NOT_SUPPORTED
    assert ex(et=api.R_64F) == api.STATUS_NOT_SUPPORTED
    assert lib.mcsparseCsrmvEx(h, 0, 0, 4, 4, 0, pa, api.C_32F, d, FAKE, api.C_32F, FAKE, FAKE, FAKE, api.C_32F, pa,
                               api.C_32F, FAKE, api.C_32F, api.C_32F, FAKE) == api.STATUS_NOT_SUPPORTED
    bs = lambda hh=h, out=ctypes.byref(size), nnz=1000: lib.mcsparseCsrmvEx_bufferSize(
        hh, 0, 0, 400, 400, nnz, pa, api.R_32F, d, FAKE, api.R_32F, FAKE, FAKE, FAKE, api.R_32F, pa, api.R_32F, FAKE,
        api.R_32F, api.R_32F, out)
    assert bs() == 0 and size.value == 128  # the reference's constant, mcsp_spmv_gpu.cpp:1149-1158
    assert bs(hh=None) == api.STATUS_NOT_INITIALIZED and bs(out=None) == api.STATUS_INVALID_VALUE


def test_csrmm_argument_checks(lib):
    h, d = make(lib)
    one = ctypes.c_double(1.0)
    pa = ctypes.addressof(one)
    call = lambda hh=h, ta=0, tb=0, a=pa, dd=d, v=FAKE, r=FAKE, c=FAKE, B=FAKE, ldb=6, b=pa, C=FAKE, ldc=8, nnz=0: \
        lib.mcsparseDcsrmm2(hh, ta, tb, 8, 3, 6, nnz, a, dd, v, r, c, B, ldb, b, C, ldc)
    assert call() == 0  # nnz == 0 and beta == 1: early return (mcsp_spmm_gpu.cpp:46-48)
    assert call(hh=None) == api.STATUS_NOT_INITIALIZED
    for kw in ({"a": None}, {"dd": None}, {"v": None}, {"r": None}, {"c": None}, {"B": None}, {"b": None},
               {"C": None}):
        assert call(**kw) == api.STATUS_INVALID_VALUE, kw
    assert call(ta=1) == api.STATUS_NOT_SUPPORTED  # transA must be N (:39-42)
    assert call(ldb=5) == api.STATUS_INVALID_VALUE and call(ldc=7) == api.STATUS_INVALID_VALUE
    assert call(tb=1, ldb=3) == 0 and call(tb=1, ldb=2) == api.STATUS_INVALID_VALUE  # B is n x k when transposed
    assert lib.mcsparseDcsrmm(h, 0, 8, 3, 6, 0, pa, d, FAKE, FAKE, FAKE, FAKE, 6, pa, FAKE, 8) == 0
    assert lib.mcsparseDcsrmm(h, 1, 8, 3, 6, 0, pa, d, FAKE, FAKE, FAKE, FAKE, 6, pa, FAKE, 8) == api.STATUS_NOT_SUPPORTED
