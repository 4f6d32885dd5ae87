"""Host-side behaviour of the C ABI that needs no GPU: exported symbols, handle and descriptor
objects, and the argument checks, which all return before any device work.  Expected codes
follow the reference's host drivers (cited per test, paths relative to mcsparse/src)."""
import ctypes
import re
import os

import numpy as np
import pytest

from mcsparse_amd import api, _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FAKE = 0x1000  # a non-NULL "device pointer"; never dereferenced on these paths


def test_library_exports_every_declared_symbol(lib):
    header = open(os.path.join(ROOT, "include", "mcsparse.h")).read()
    declared = set(re.findall(r"\b(mcsparse[A-Za-z0-9_]+)\s*\(", header))
    assert declared, "no prototypes found in include/mcsparse.h"
    assert declared == set(_lib.PROTOTYPES), declared ^ set(_lib.PROTOTYPES)
    for name in declared:
        assert hasattr(lib, name), name


def test_library_exports_nothing_else(lib):
    """nm -D: every defined dynamic symbol is a C function of the header (no C++ internals leak)."""
    import subprocess
    from mcsparse_amd.build import LIB_PATH
    out = subprocess.run(["nm", "-D", "--defined-only", LIB_PATH], stdout=subprocess.PIPE, text=True, check=True).stdout
    names = [line.split()[-1] for line in out.splitlines() if line.strip()]
    assert names, "no dynamic symbols"
    assert set(names) == set(_lib.PROTOTYPES), set(names) ^ set(_lib.PROTOTYPES)
    soname = subprocess.run(["readelf", "-d", LIB_PATH], stdout=subprocess.PIPE, text=True, check=True).stdout
    assert "libmcsparse.so" in [l.split("[")[-1].rstrip("]") for l in soname.splitlines() if "SONAME" in l]


def test_c99_caller_links_and_walks_the_argument_checks(lib, tmp_path):
    """A C program written against the header: compiles as C99, links with the library, and gets the
    reference's statuses on the paths that return before any launch."""
    import subprocess
    from mcsparse_amd.build import LIB_DIR
    src = os.path.join(ROOT, "tests", "c_abi", "spmv_caller.c")
    exe = str(tmp_path / "spmv_caller")
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"),
                    src, "-o", exe, "-L", LIB_DIR, "-lmcsparse", "-Wl,-rpath," + LIB_DIR,
                    "-Wl,-rpath-link,/opt/rocm/lib"], check=True)
    run = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert run.returncode == 0 and run.stdout.strip().endswith("ok"), run.stdout


def test_status_strings(lib):
    # wrapper/mcsp_interface_wrapper.cpp:48-108
    assert lib.mcsparseGetErrorName(0) == b"MCSPARSE_STATUS_SUCCESS"
    assert lib.mcsparseGetErrorName(10) == b"MCSPARSE_STATUS_NOT_SUPPORTED"
    assert lib.mcsparseGetErrorString(3) == b"invalid value"
    assert lib.mcsparseGetErrorString(6) == b"kernel launch failure"
    assert lib.mcsparseGetErrorName(99) == b"unrecognized error code"
    assert lib.mcsparseGetErrorString(-1) == b"unrecognized error code"


def test_handle_lifecycle(lib):
    # common/mcsp_helper.cpp:69-88, :154-198, :294-322
    assert lib.mcsparseCreate(None) == api.STATUS_INVALID_VALUE
    h = ctypes.c_void_p()
    assert lib.mcsparseCreate(ctypes.byref(h)) == 0 and h.value
    v = ctypes.c_int(-1)
    assert lib.mcsparseGetVersion(h, ctypes.byref(v)) == 0 and v.value == 1000000
    assert lib.mcsparseGetVersion(None, ctypes.byref(v)) == api.STATUS_NOT_INITIALIZED
    assert lib.mcsparseGetVersion(h, None) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseGetVersion(None, None) == api.STATUS_INVALID_VALUE  # pointer is tested first
    for prop, want in ((0, 1), (1, 0), (2, 0)):
        assert lib.mcsparseGetProperty(prop, ctypes.byref(v)) == 0 and v.value == want
    assert lib.mcsparseGetProperty(7, ctypes.byref(v)) == api.STATUS_INVALID_VALUE
    s = ctypes.c_void_p(123)
    assert lib.mcsparseGetStream(h, ctypes.byref(s)) == 0 and not s.value  # default: NULL stream
    assert lib.mcsparseSetStream(h, ctypes.c_void_p(0xABC0)) == 0
    assert lib.mcsparseGetStream(h, ctypes.byref(s)) == 0 and s.value == 0xABC0
    assert lib.mcsparseSetStream(None, None) == api.STATUS_NOT_INITIALIZED
    assert lib.mcsparseGetStream(h, None) == api.STATUS_INVALID_VALUE
    pm = ctypes.c_int(-1)
    assert lib.mcsparseGetPointerMode(h, ctypes.byref(pm)) == 0 and pm.value == api.PTR_HOST
    assert lib.mcsparseSetPointerMode(h, api.PTR_DEVICE) == 0
    assert lib.mcsparseGetPointerMode(h, ctypes.byref(pm)) == 0 and pm.value == api.PTR_DEVICE
    assert lib.mcsparseSetPointerMode(None, 0) == api.STATUS_NOT_INITIALIZED
    assert lib.mcsparseDestroy(h) == 0
    assert lib.mcsparseDestroy(None) == 0  # NULL accepted


def test_dense_descriptors(lib):
    # common/mcsp_helper.cpp:325-387, :715-800
    d = ctypes.c_void_p()
    assert lib.mcsparseCreateDnVec(ctypes.byref(d), -1, FAKE, api.R_32F) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseCreateDnVec(ctypes.byref(d), 4, None, api.R_32F) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseCreateDnVec(None, 4, FAKE, api.R_32F) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseCreateDnVec(ctypes.byref(d), 4, FAKE, 24) == api.STATUS_NOT_SUPPORTED  # R_64I
    assert lib.mcsparseCreateDnVec(ctypes.byref(d), 4, FAKE, api.R_64F) == 0
    size, vals, vt = ctypes.c_int64(), ctypes.c_void_p(), ctypes.c_int()
    assert lib.mcsparseDnVecGet(d, ctypes.byref(size), ctypes.byref(vals), ctypes.byref(vt)) == 0
    assert (size.value, vals.value, vt.value) == (4, FAKE, api.R_64F)
    assert lib.mcsparseDnVecGet(d, None, ctypes.byref(vals), ctypes.byref(vt)) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseDnVecSetValues(d, 0x2000) == 0
    assert lib.mcsparseDnVecGetValues(d, ctypes.byref(vals)) == 0 and vals.value == 0x2000
    assert lib.mcsparseDnVecSetValues(None, 0x2000) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseDestroyDnVec(d) == 0 and lib.mcsparseDestroyDnVec(None) == 0

    m = ctypes.c_void_p()
    assert lib.mcsparseCreateDnMat(ctypes.byref(m), 3, -2, 3, FAKE, api.R_32F, api.ORDER_ROW) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseCreateDnMat(ctypes.byref(m), 3, 2, 3, FAKE, 24, api.ORDER_ROW) == api.STATUS_NOT_SUPPORTED
    assert lib.mcsparseCreateDnMat(ctypes.byref(m), 3, 2, 3, None, api.R_32F, api.ORDER_ROW) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseCreateDnMat(ctypes.byref(m), 3, 2, 5, FAKE, api.R_32F, api.ORDER_COL) == 0
    r, c, ld, order = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int()
    assert lib.mcsparseDnMatGet(m, ctypes.byref(r), ctypes.byref(c), ctypes.byref(ld), ctypes.byref(vals),
                                ctypes.byref(vt), ctypes.byref(order)) == 0
    assert (r.value, c.value, ld.value, vals.value, vt.value, order.value) == (3, 2, 5, FAKE, api.R_32F, api.ORDER_COL)
    assert lib.mcsparseDnMatSetValues(m, 0x3000) == 0
    assert lib.mcsparseDnMatGetValues(m, ctypes.byref(vals)) == 0 and vals.value == 0x3000
    assert lib.mcsparseDestroyDnMat(m) == 0 and lib.mcsparseDestroyDnMat(None) == 0


def test_sparse_descriptors(lib):
    # common/mcsp_helper.cpp:389-452, :503-524, :587-683
    d = ctypes.c_void_p()
    mk = lib.mcsparseCreateCsr
    assert mk(ctypes.byref(d), -1, 4, 5, 0x10, 0x20, 0x30, 2, 2, 0, api.R_32F) == api.STATUS_INVALID_VALUE
    assert mk(ctypes.byref(d), 3, 4, 5, 0x10, 0x20, 0x30, 2, 2, 0, api.R_32I) == api.STATUS_NOT_SUPPORTED
    assert mk(None, 3, 4, 5, 0x10, 0x20, 0x30, 2, 2, 0, api.R_32F) == api.STATUS_INVALID_VALUE
    assert mk(ctypes.byref(d), 3, 4, 5, 0x10, 0x20, 0x30, 2, 2, 7, api.R_32F) == api.STATUS_INVALID_VALUE  # bad base
    assert mk(ctypes.byref(d), 3, 4, 5, None, None, None, 2, 2, 1, api.R_64F) == 0  # pointers are not checked
    i64 = [ctypes.c_int64() for _ in range(3)]
    ptrs = [ctypes.c_void_p() for _ in range(3)]
    ints = [ctypes.c_int() for _ in range(4)]
    assert lib.mcsparseCsrSetPointers(d, 0x10, 0x20, 0x30) == 0
    assert lib.mcsparseCsrGet(d, *[ctypes.byref(x) for x in i64 + ptrs + ints]) == 0
    assert [x.value for x in i64] == [3, 4, 5]
    assert [x.value for x in ptrs] == [0x10, 0x20, 0x30]
    assert [x.value for x in ints] == [2, 2, 1, api.R_64F]
    assert lib.mcsparseCsrGet(d, None, *[ctypes.byref(x) for x in i64[1:] + ptrs + ints]) == api.STATUS_INVALID_VALUE
    fmt, base = ctypes.c_int(), ctypes.c_int()
    assert lib.mcsparseSpMatGetFormat(d, ctypes.byref(fmt)) == 0 and fmt.value == api.FORMAT_CSR
    assert lib.mcsparseSpMatGetIndexBase(d, ctypes.byref(base)) == 0 and base.value == 1
    assert lib.mcsparseSpMatGetSize(d, *[ctypes.byref(x) for x in i64]) == 0
    assert lib.mcsparseSpMatSetValues(d, 0x44) == 0
    v = ctypes.c_void_p()
    assert lib.mcsparseSpMatGetValues(d, ctypes.byref(v)) == 0 and v.value == 0x44
    assert lib.mcsparseSpMatGetValues(None, ctypes.byref(v)) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseDestroySpMat(d) == 0 and lib.mcsparseDestroySpMat(None) == 0
    # CSC: offsets are the columns' (mcsp_helper.cpp:447-452)
    assert lib.mcsparseCreateCsc(ctypes.byref(d), 3, 4, 5, 0x50, 0x60, 0x70, 2, 2, 0, api.R_32F) == 0
    assert lib.mcsparseSpMatGetFormat(d, ctypes.byref(fmt)) == 0 and fmt.value == api.FORMAT_CSC
    assert lib.mcsparseCscSetPointers(d, 0x51, 0x61, 0x71) == 0
    assert lib.mcsparseCscSetPointers(None, 0x51, 0x61, 0x71) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseDestroySpMat(d) == 0
    # COO: one index type for both arrays (mcsp_helper.cpp:433-445, :526-549, :597-607)
    mkc = lib.mcsparseCreateCoo
    assert mkc(ctypes.byref(d), 3, -4, 5, 0x10, 0x20, 0x30, 2, 0, api.R_32F) == api.STATUS_INVALID_VALUE
    assert mkc(None, 3, 4, 5, 0x10, 0x20, 0x30, 2, 0, api.R_32F) == api.STATUS_INVALID_VALUE
    assert mkc(ctypes.byref(d), 3, 4, 5, 0x10, 0x20, 0x30, 2, 1, api.R_32F) == 0
    assert lib.mcsparseSpMatGetFormat(d, ctypes.byref(fmt)) == 0 and fmt.value == api.FORMAT_COO
    assert lib.mcsparseCooSetPointers(d, 0x11, 0x21, 0x31) == 0
    ints3 = [ctypes.c_int() for _ in range(3)]
    assert lib.mcsparseCooGet(d, *[ctypes.byref(x) for x in i64 + ptrs + ints3]) == 0
    assert [x.value for x in i64] == [3, 4, 5]
    assert [x.value for x in ptrs] == [0x11, 0x21, 0x31]
    assert [x.value for x in ints3] == [2, 1, api.R_32F]
    assert lib.mcsparseCooGet(d, *[ctypes.byref(x) for x in i64 + ptrs + ints3[:2]], None) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseCooSetPointers(None, 0x11, 0x21, 0x31) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseDestroySpMat(d) == 0


class Objs:
    """A handle and descriptors over fake pointers for the argument-check tests."""

    def __init__(self, lib, m=8, n=6, nnz=20, vt=api.R_32F, fmt=api.FORMAT_CSR, idx=(2, 2)):
        self.lib = lib
        self.h = ctypes.c_void_p()
        lib.mcsparseCreate(ctypes.byref(self.h))
        self.A = ctypes.c_void_p()
        if fmt == api.FORMAT_COO:
            assert lib.mcsparseCreateCoo(ctypes.byref(self.A), m, n, nnz, FAKE, FAKE, FAKE, idx[0], 0, vt) == 0
        else:
            mk = lib.mcsparseCreateCsr if fmt == api.FORMAT_CSR else lib.mcsparseCreateCsc
            assert mk(ctypes.byref(self.A), m, n, nnz, FAKE, FAKE, FAKE, idx[0], idx[1], 0, vt) == 0
        self.x, self.y, self.xm = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p()
        lib.mcsparseCreateDnVec(ctypes.byref(self.x), n, FAKE, vt)
        lib.mcsparseCreateDnVec(ctypes.byref(self.y), m, FAKE, vt)
        self.one = ctypes.c_float(1.0)
        self.pa = ctypes.addressof(self.one)

    def spmv(self, h="h", op=api.OP_N, alpha="a", A="A", x="x", beta="a", y="y", ct=api.R_32F, buf=FAKE):
        g = lambda k: {"h": self.h, "a": self.pa, "A": self.A, "x": self.x, "y": self.y, None: None}[k]
        return self.lib.mcsparseSpMV(g(h), op, g(alpha), g(A), g(x), g(beta), g(y), ct, 0, buf)

    def spmv_size(self, h="h", op=api.OP_N, alpha="a", A="A", x="x", beta="a", y="y", out=True):
        g = lambda k: {"h": self.h, "a": self.pa, "A": self.A, "x": self.x, "y": self.y, None: None}[k]
        size = ctypes.c_size_t(0)
        st = self.lib.mcsparseSpMV_bufferSize(g(h), op, g(alpha), g(A), g(x), g(beta), g(y), api.R_32F, 0,
                                              ctypes.byref(size) if out else None)
        return st, size.value


def test_spmv_argument_checks(lib):
    # level2/spmv/mcsp_spmv_gpu.cpp:686-720 in order
    o = Objs(lib)
    assert o.spmv(h=None) == api.STATUS_NOT_INITIALIZED
    for k in ("alpha", "A", "x", "beta", "y"):
        assert o.spmv(**{k: None}) == api.STATUS_INVALID_VALUE, k
    assert o.spmv(buf=None) == api.STATUS_INVALID_VALUE  # required even for op N (:703-705)
    assert o.spmv(op=api.OP_T) == api.STATUS_INVALID_VALUE  # x, y sizes do not fit the transpose (:711)
    assert o.spmv(x="y", y="x") == api.STATUS_INVALID_VALUE
    assert o.spmv(op=api.OP_T, x="y", y="x", ct=api.R_64F) == api.STATUS_NOT_SUPPORTED  # mixed types
    assert o.spmv(ct=api.R_64F) == api.STATUS_NOT_SUPPORTED
    sq = Objs(lib, m=6, n=6)
    assert sq.spmv(op=api.OP_C) == api.STATUS_INVALID_VALUE  # conjugate on a real type (:716-720)
    big = Objs(lib, m=1 << 32, n=6)
    assert big.spmv() == api.STATUS_NOT_SUPPORTED  # sizes must fit 32 bits (:698-701)
    mixed = Objs(lib, idx=(2, 3))
    assert mixed.spmv() == api.STATUS_NOT_SUPPORTED  # row/col index types differ (:1126-1132)
    assert mixed.spmv(h=None) == api.STATUS_NOT_SUPPORTED  # the index-type dispatch comes first
    i64 = Objs(lib, idx=(3, 3))
    assert i64.spmv(h=None) == api.STATUS_NOT_INITIALIZED  # 64-bit indices pass the dispatch (:1128-1129)
    assert i64.spmv(buf=None) == api.STATUS_INVALID_VALUE
    assert i64.spmv_size()[0] == 0 and i64.spmv_size()[1] > o.spmv_size()[1]  # room for the narrowed copies
    u16 = Objs(lib, idx=(1, 1))
    assert u16.spmv() == api.STATUS_NOT_SUPPORTED  # 16-bit indices: not dispatched (:1130-1132)
    cplx = Objs(lib, vt=api.C_32F)
    assert cplx.spmv(ct=api.C_32F) == api.STATUS_NOT_SUPPORTED


def test_spmv_early_outs_touch_nothing(lib):
    # mcsp_spmv_gpu.cpp:235-237: nnz == 0, or alpha == beta == 0, returns before any launch.
    # The pointers here are fake, so reaching a kernel would fault rather than pass.
    empty = Objs(lib, nnz=0)
    assert empty.spmv() == api.STATUS_SUCCESS
    o = Objs(lib)
    zero = ctypes.c_float(0.0)
    pz = ctypes.addressof(zero)
    assert lib.mcsparseSpMV(o.h, api.OP_N, pz, o.A, o.x, pz, o.y, api.R_32F, 0, FAKE) == api.STATUS_SUCCESS


def test_spmv_buffer_size(lib):
    # level2/spmv/mcsp_spmv_gpu.cpp:309-352
    o = Objs(lib, m=1000, n=800, nnz=16000)
    st, n_size = o.spmv_size()
    assert st == 0 and n_size >= 128 and n_size % 128 == 0
    assert o.spmv_size(h=None)[0] == api.STATUS_NOT_INITIALIZED
    assert o.spmv_size(out=False)[0] == api.STATUS_INVALID_VALUE
    assert o.spmv_size(A=None)[0] == api.STATUS_INVALID_VALUE
    assert o.spmv_size(op=api.OP_T)[0] == api.STATUS_INVALID_VALUE
    st, t_size = o.spmv_size(op=api.OP_T, x="y", y="x")
    assert st == 0 and t_size % 128 == 0
    # the transpose needs room for A^T (n+1+nnz indices, nnz values) on top of the sort scratch
    assert t_size >= (800 + 1 + 16000) * 4 + 16000 * 4
    bigger = Objs(lib, m=1000, n=800, nnz=32000)
    assert bigger.spmv_size(op=api.OP_T, x="y", y="x")[1] > t_size  # monotone in nnz
    csc = Objs(lib, m=1000, n=800, nnz=16000, fmt=api.FORMAT_CSC)
    assert csc.spmv_size()[1] > csc.spmv_size(op=api.OP_T, x="y", y="x")[1]  # CSC op N is the transposing case
    coo = Objs(lib, m=1000, n=800, nnz=16000, fmt=api.FORMAT_COO)
    assert coo.spmv_size()[1] >= n_size + 1001 * 4  # row offsets are rebuilt in the buffer
    assert coo.spmv_size(op=api.OP_T, x="y", y="x")[1] >= t_size + 1001 * 4


def test_spmm_argument_checks(lib):
    # level3/spmm/mcsp_spmm_gpu.cpp:785-807, :105-108, :309-342
    o = Objs(lib, m=8, n=6, nnz=20)
    B, C, Bt, Cbad = (ctypes.c_void_p() for _ in range(4))
    lib.mcsparseCreateDnMat(ctypes.byref(B), 6, 4, 4, FAKE, api.R_32F, api.ORDER_ROW)
    lib.mcsparseCreateDnMat(ctypes.byref(C), 8, 4, 4, FAKE, api.R_32F, api.ORDER_ROW)
    lib.mcsparseCreateDnMat(ctypes.byref(Bt), 4, 6, 6, FAKE, api.R_32F, api.ORDER_ROW)
    lib.mcsparseCreateDnMat(ctypes.byref(Cbad), 7, 4, 4, FAKE, api.R_32F, api.ORDER_ROW)
    call = lambda h=o.h, opA=0, opB=0, a=o.pa, A=o.A, b=B, be=o.pa, c=C, ct=api.R_32F, buf=FAKE: lib.mcsparseSpMM(
        h, opA, opB, a, A, b, be, c, ct, 0, buf)
    assert call(h=None) == api.STATUS_NOT_INITIALIZED
    for kw in ({"a": None}, {"A": None}, {"b": None}, {"be": None}, {"c": None}, {"buf": None}):
        assert call(**kw) == api.STATUS_INVALID_VALUE, kw
    assert call(opA=api.OP_T) == api.STATUS_NOT_SUPPORTED  # CSR op(A) != N (:105-108)
    assert call(ct=api.R_64F) == api.STATUS_NOT_SUPPORTED
    assert call(c=Cbad) == api.STATUS_INVALID_VALUE  # C rows != A rows
    assert call(b=Bt) == api.STATUS_INVALID_VALUE  # B is 4 x 6 but op(B) must be 6 x 4
    size = ctypes.c_size_t()
    assert lib.mcsparseSpMM_bufferSize(o.h, 0, 0, o.pa, o.A, B, o.pa, C, api.R_32F, 0, ctypes.byref(size)) == 0
    # room for the row-group schedule of mcsparseSpMM_preprocess: group offsets, 20 entries, scan scratch
    assert size.value % 128 == 0 and size.value >= 128 + 128 and size.value < 4096
    assert lib.mcsparseSpMM_bufferSize(None, 0, 0, o.pa, o.A, B, o.pa, C, api.R_32F, 0, ctypes.byref(size)) == 1
    assert lib.mcsparseSpMM_bufferSize(o.h, 0, 0, o.pa, o.A, None, o.pa, C, api.R_32F, 0, ctypes.byref(size)) == 3
    # preprocess (:965-970 is a no-op; here it checks its arguments like SpMM and builds a schedule for CSR)
    assert lib.mcsparseSpMM_preprocess(None, 0, 0, o.pa, o.A, B, o.pa, C, api.R_32F, 0, FAKE) == 1
    assert lib.mcsparseSpMM_preprocess(o.h, 0, 0, o.pa, o.A, B, o.pa, C, api.R_32F, 0, None) == 3
    assert lib.mcsparseSpMM_preprocess(o.h, 0, 0, o.pa, None, B, o.pa, C, api.R_32F, 0, FAKE) == 3
    assert lib.mcsparseSpMM_preprocess(o.h, api.OP_T, 0, o.pa, o.A, B, o.pa, C, api.R_32F, 0, FAKE) == 0  # nothing to do
    state, entries = ctypes.c_int(-1), ctypes.c_int64(-1)
    assert lib.mcsparseSpMatGetSpMMSchedule(o.A, ctypes.byref(state), ctypes.byref(entries)) == 0
    assert state.value == 0 and entries.value == 0
    assert lib.mcsparseSpMatGetSpMMSchedule(o.A, None, ctypes.byref(entries)) == 3
    for f, need in ((api.FORMAT_COO, 9 * 4), (api.FORMAT_CSC, (9 + 20) * 4 + 20 * 4)):
        o2 = Objs(lib, m=8, n=6, nnz=20, fmt=f)
        assert lib.mcsparseSpMM_bufferSize(o2.h, 0, 0, o2.pa, o2.A, B, o2.pa, C, api.R_32F, 0, ctypes.byref(size)) == 0
        assert size.value >= need and size.value % 128 == 0
        assert lib.mcsparseSpMM(o2.h, api.OP_T, 0, o2.pa, o2.A, B, o2.pa, C, api.R_32F, 0, FAKE) == 10
        assert lib.mcsparseSpMM(o2.h, 0, 0, o2.pa, o2.A, B, o2.pa, C, api.R_32F, 0, None) == 3
    # nnz == 0 with beta == 1 returns before any launch (:110-114)
    e = Objs(lib, m=8, n=6, nnz=0)
    assert lib.mcsparseSpMM(e.h, 0, 0, e.pa, e.A, B, e.pa, C, api.R_32F, 0, FAKE) == 0
    assert lib.mcsparseSpMM_preprocess(e.h, 0, 0, e.pa, e.A, B, e.pa, C, api.R_32F, 0, FAKE) == 0  # empty: no schedule
    assert lib.mcsparseSpMM_bufferSize(e.h, 0, 0, e.pa, e.A, B, e.pa, C, api.R_32F, 0, ctypes.byref(size)) == 0
    assert size.value == 128


def test_spmm_buffer_size_has_room_for_the_pieces_of_long_rows(lib):
    """Rows of more than 1024 nonzeros are cut into pieces of 4096; a row of several pieces needs a row of partial
    sums per piece, at most 2 * nnz / 4096 of them whatever the row lengths are (the size cannot depend on them: it
    is asked for before the matrix is looked at)."""
    m, k, nnz = 1 << 16, 1 << 16, 1 << 22
    o = Objs(lib, m=m, n=k, nnz=nnz)
    sizes = {}
    for n in (16, 64, 250):
        B, C = ctypes.c_void_p(), ctypes.c_void_p()
        lib.mcsparseCreateDnMat(ctypes.byref(B), k, n, n, FAKE, api.R_32F, api.ORDER_ROW)
        lib.mcsparseCreateDnMat(ctypes.byref(C), m, n, n, FAKE, api.R_32F, api.ORDER_ROW)
        size = ctypes.c_size_t()
        assert lib.mcsparseSpMM_bufferSize(o.h, 0, 0, o.pa, o.A, B, o.pa, C, api.R_32F, 0, ctypes.byref(size)) == 0
        sizes[n] = size.value
    padded = {16: 16, 64: 64, 250: 252}
    rows_of_sums = 2 * (nnz // 4096)
    for n in sizes:
        assert sizes[n] >= 4 * nnz + rows_of_sums * padded[n] * 4, (n, sizes[n])     # the schedule and the partial sums
        assert sizes[n] <= 4 * nnz + 4 * m + (rows_of_sums + 2) * padded[n] * 4 + (1 << 18), (n, sizes[n])
    assert sizes[16] < sizes[64] < sizes[250]


def test_conversion_argument_checks(lib):
    # conversion/mcsp_coo2csr.cpp:7-59, mcsp_csr2csc.cpp:9-63, :293-310
    h = ctypes.c_void_p()
    lib.mcsparseCreate(ctypes.byref(h))
    assert lib.mcsparseXcsr2coo(None, FAKE, 5, 3, FAKE, 0) == api.STATUS_NOT_INITIALIZED
    assert lib.mcsparseXcsr2coo(h, FAKE, 0, 3, FAKE, 0) == 0  # nnz == 0: nothing to do
    assert lib.mcsparseXcsr2coo(h, None, 0, 3, None, 0) == 0  # ... tested before the pointers
    assert lib.mcsparseXcsr2coo(h, None, 5, 3, FAKE, 0) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseXcsr2coo(h, FAKE, 5, 3, None, 0) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseXcoo2csr(None, FAKE, 5, 3, FAKE, 0) == api.STATUS_NOT_INITIALIZED
    assert lib.mcsparseXcoo2csr(h, FAKE, 0, 3, FAKE, 0) == 0
    assert lib.mcsparseXcoo2csr(h, None, 5, 3, FAKE, 0) == api.STATUS_INVALID_VALUE
    size = ctypes.c_size_t()
    bs = lambda hh=h, m=4, n=5, nnz=9, out=ctypes.byref(size): lib.mcsparseCsr2cscEx2_bufferSize(
        hh, m, n, nnz, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, api.R_32F, 1, 0, 1, out)
    assert bs(hh=None) == api.STATUS_NOT_INITIALIZED
    assert bs(out=None) == api.STATUS_INVALID_VALUE
    assert bs(nnz=0) == 0 and size.value == 128
    assert bs() == 0 and size.value >= 128
    small = size.value
    assert bs(nnz=9000) == 0 and size.value > small
    cv = lambda hh=h, m=4, n=5, nnz=9, vt=api.R_32F, val=FAKE, buf=FAKE, act=1: lib.mcsparseCsr2cscEx2(
        hh, m, n, nnz, val, FAKE, FAKE, FAKE, FAKE, FAKE, vt, act, 0, 1, buf)
    assert cv(vt=api.R_16F) == api.STATUS_INVALID_VALUE  # type switch comes first (:297-309)
    assert cv(hh=None) == api.STATUS_NOT_INITIALIZED
    assert cv(nnz=0) == 0 and cv(m=0) == 0 and cv(n=0) == 0  # early success, outputs untouched (:56-58)
    assert cv(val=None) == api.STATUS_INVALID_VALUE
    assert cv(val=None, act=0) == api.STATUS_INVALID_VALUE  # values required even for SYMBOLIC (:60-63)
    assert cv(buf=None) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseXcsrRowBins(None, 3, FAKE, 0, None, FAKE) == api.STATUS_NOT_INITIALIZED
    assert lib.mcsparseXcsrRowBins(h, 3, None, 0, None, FAKE) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseXcsrRowBins(h, 3, FAKE, 0, None, None) == api.STATUS_INVALID_VALUE


def test_plan_override_api(lib):
    o = Objs(lib)
    fam, lanes = ctypes.c_int(-1), ctypes.c_int(-1)
    assert lib.mcsparseSpMatGetSpMVPlan(o.A, ctypes.byref(fam), ctypes.byref(lanes)) == 0
    assert (fam.value, lanes.value) == (0, 0)  # nothing analysed yet
    assert lib.mcsparseSpMatSetSpMVPlan(o.A, 3, 0) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseSpMatSetSpMVPlan(o.A, 1, 3) == api.STATUS_INVALID_VALUE  # lanes must be a power of two
    assert lib.mcsparseSpMatSetSpMVPlan(o.A, 1, 16) == 0
    assert lib.mcsparseSpMatSetSpMVPlan(None, 1, 16) == api.STATUS_INVALID_VALUE


def test_sort_argument_checks(lib):
    # conversion/mcsp_csrsort.cpp:13-64, mcsp_coosort.cpp:12-61, mcsp_create_identity.cpp:6-20, level1/mcsp_gthr.cpp:7-23
    o = Objs(lib)
    d = ctypes.c_void_p()
    assert lib.mcsparseCreateMatDescr(ctypes.byref(d)) == 0
    size = ctypes.c_size_t()
    for fn in (lib.mcsparseXcsrsort_bufferSizeExt, lib.mcsparseXcscsort_bufferSizeExt, lib.mcsparseXcoosort_bufferSizeExt):
        assert fn(None, 4, 4, 8, FAKE, FAKE, ctypes.byref(size)) == api.STATUS_NOT_INITIALIZED
        assert fn(o.h, -1, 4, 8, FAKE, FAKE, ctypes.byref(size)) == api.STATUS_INVALID_VALUE
        assert fn(o.h, 4, 4, 8, None, FAKE, ctypes.byref(size)) == api.STATUS_INVALID_VALUE
        assert fn(o.h, 4, 4, 8, FAKE, FAKE, None) == api.STATUS_INVALID_VALUE
        assert fn(o.h, 4, 4, 0, FAKE, FAKE, ctypes.byref(size)) == 0 and size.value == 128
        assert fn(o.h, 4, 4, 5000, FAKE, FAKE, ctypes.byref(size)) == 0
        assert size.value % 128 == 0 and size.value >= 10 * 5000 * 4
    for fn in (lib.mcsparseXcsrsort, lib.mcsparseXcscsort):
        assert fn(None, 4, 4, 8, d, FAKE, FAKE, FAKE, FAKE) == api.STATUS_NOT_INITIALIZED
        assert fn(o.h, 4, -4, 8, d, FAKE, FAKE, FAKE, FAKE) == api.STATUS_INVALID_VALUE
        assert fn(o.h, 4, 4, 0, d, None, None, None, None) == 0  # empty: nothing is checked or touched
        assert fn(o.h, 4, 4, 8, d, None, FAKE, FAKE, FAKE) == api.STATUS_INVALID_VALUE
        assert fn(o.h, 4, 4, 8, d, FAKE, None, FAKE, FAKE) == api.STATUS_INVALID_VALUE
        assert fn(o.h, 4, 4, 8, d, FAKE, FAKE, FAKE, None) == api.STATUS_INVALID_VALUE
        assert fn(o.h, 4, 4, 8, None, FAKE, FAKE, FAKE, FAKE) == api.STATUS_INVALID_VALUE
    for fn in (lib.mcsparseXcoosortByRow, lib.mcsparseXcoosortByColumn):
        assert fn(None, 4, 4, 8, FAKE, FAKE, FAKE, FAKE) == api.STATUS_NOT_INITIALIZED
        assert fn(o.h, 4, 4, -8, FAKE, FAKE, FAKE, FAKE) == api.STATUS_INVALID_VALUE
        assert fn(o.h, 0, 4, 8, None, None, None, None) == 0
        assert fn(o.h, 4, 4, 8, None, FAKE, FAKE, FAKE) == api.STATUS_INVALID_VALUE
        assert fn(o.h, 4, 4, 8, FAKE, FAKE, FAKE, None) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseCreateIdentityPermutation(None, 4, FAKE) == api.STATUS_NOT_INITIALIZED
    assert lib.mcsparseCreateIdentityPermutation(o.h, -4, FAKE) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseCreateIdentityPermutation(o.h, 4, None) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseCreateIdentityPermutation(o.h, 0, FAKE) == 0
    for fn in (lib.mcsparseSgthr, lib.mcsparseDgthr):
        assert fn(None, 4, FAKE, FAKE, FAKE, 0) == api.STATUS_NOT_INITIALIZED
        assert fn(o.h, -4, FAKE, FAKE, FAKE, 0) == api.STATUS_INVALID_VALUE
        assert fn(o.h, 0, None, None, None, 0) == 0
        assert fn(o.h, 4, FAKE, None, FAKE, 0) == api.STATUS_INVALID_VALUE
    lib.mcsparseDestroyMatDescr(d)


def test_strided_batch_setters(lib):
    # src/kernels/generic/mcsp_generic.cpp:686-743: null descriptor, count <= 0, negative stride
    o = Objs(lib)
    assert lib.mcsparseCsrSetStridedBatch(None, 1, 0, 0) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseCsrSetStridedBatch(o.A, 0, 0, 0) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseCsrSetStridedBatch(o.A, 2, -1, 0) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseCsrSetStridedBatch(o.A, 2, 0, -1) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseCsrSetStridedBatch(o.A, 2, 8, 40) == 0
    assert lib.mcsparseCooSetStridedBatch(None, 1, 0) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseCooSetStridedBatch(o.A, -3, 0) == api.STATUS_INVALID_VALUE
    B = ctypes.c_void_p()
    assert lib.mcsparseCreateDnMat(ctypes.byref(B), 6, 4, 4, FAKE, api.R_32F, api.ORDER_ROW) == 0
    count, stride = ctypes.c_int(-1), ctypes.c_int64(-1)
    assert lib.mcsparseDnMatGetStridedBatch(B, ctypes.byref(count), ctypes.byref(stride)) == 0
    assert (count.value, stride.value) == (1, 0)  # defaults (src/include/mcsp_internal_types.h:143-144)
    assert lib.mcsparseDnMatSetStridedBatch(B, 0, 24) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseDnMatSetStridedBatch(B, 3, -24) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseDnMatSetStridedBatch(None, 3, 24) == api.STATUS_INVALID_VALUE
    assert lib.mcsparseDnMatSetStridedBatch(B, 3, 24) == 0
    assert lib.mcsparseDnMatGetStridedBatch(B, ctypes.byref(count), ctypes.byref(stride)) == 0
    assert (count.value, stride.value) == (3, 24)
    assert lib.mcsparseDnMatGetStridedBatch(B, None, ctypes.byref(stride)) == api.STATUS_INVALID_VALUE
    lib.mcsparseDestroyDnMat(B)


def _plan(lib, lengths, x_bytes=64 << 20):
    """Kernel choice for rows of these lengths, through the same bins the GPU analysis fills."""
    lengths = np.asarray(lengths, dtype=np.int64)
    hist = np.zeros(34, dtype=np.uint32)
    bins = np.where(lengths == 0, 0, np.floor(np.log2(np.maximum(lengths, 1))).astype(np.int64) + 1)
    np.add.at(hist, bins, 1)
    hist[33] = lengths.max()
    fam, lanes = ctypes.c_int(), ctypes.c_int()
    st = lib.mcsparseXcsrRowBinsPlan(hist.ctypes.data, int(lengths.size), int(lengths.sum()), x_bytes,
                                     ctypes.byref(fam), ctypes.byref(lanes))
    assert st == 0
    return fam.value, lanes.value


def test_spmv_family_choice_from_row_bins(lib):
    """The pure decision function behind mcsparseSpMV's dispatch, on a table of row-length spreads."""
    rng = np.random.default_rng(0)
    m = 1 << 16
    # rows of one length fill their lanes: the vector family with the matching width
    assert _plan(lib, np.full(m, 16)) == (api.FAMILY_VECTOR, 16)
    assert _plan(lib, np.full(m, 5)) == (api.FAMILY_VECTOR, 8)
    assert _plan(lib, np.full(m, 1)) == (api.FAMILY_VECTOR, 1)
    assert _plan(lib, np.full(m, 27)) == (api.FAMILY_VECTOR, 32)
    # the transposed power-law matrix: 28 +- 5 per row, every wavefront waits for a row of 33+
    assert _plan(lib, rng.poisson(28, m))[0] == api.FAMILY_MERGE
    # mild spreads stay with the vector family
    assert _plan(lib, rng.poisson(20, m)) == (api.FAMILY_VECTOR, 32)
    assert _plan(lib, rng.integers(12, 17, m)) == (api.FAMILY_VECTOR, 16)
    # 5-point Laplacian: 3..5 per row
    assert _plan(lib, rng.choice([3, 4, 5], m, p=[0.01, 0.04, 0.95])) == (api.FAMILY_VECTOR, 8)
    # rows far longer than the rest serialise a wavefront: merge path; in column order when such rows exceed a
    # tile, hold most of the nonzeros, and x does not fit an L2; in storage order otherwise
    skew = np.full(m, 4)
    skew[7:17] = 100000
    assert _plan(lib, skew) == (api.FAMILY_MERGE, 1)
    assert _plan(lib, skew, x_bytes=1 << 20) == (api.FAMILY_MERGE, 0)
    skew[7:17] = 700
    assert _plan(lib, skew) == (api.FAMILY_MERGE, 0)
    # a handful of long rows among many short ones (1 M rows of 16, 64 rows of 100000: a quarter of the nonzeros):
    # one merge-path launch over all rows in storage order (measured 140 us; the vector kernel on the short rows
    # plus the merge kernel on the long ones, as two launches, 107 + 37 us; tiles in column order 155 us)
    mixed = np.full(1 << 20, 16)
    mixed[::16384] = 100000
    assert _plan(lib, mixed) == (api.FAMILY_MERGE, 0)
    # power law: most rows hold one nonzero, the mean is carried by a few long ones
    zipf = np.minimum(rng.zipf(1.8, m), 200000)
    assert _plan(lib, zipf)[0] == api.FAMILY_MERGE
    # half the rows empty, the rest of one length: the lanes of the non-empty rows are full half the time
    half = np.where(rng.random(m) < 0.5, 0, 32)
    assert _plan(lib, half)[0] in (api.FAMILY_VECTOR, api.FAMILY_MERGE)
    # argument checks
    fam, lanes = ctypes.c_int(), ctypes.c_int()
    assert lib.mcsparseXcsrRowBinsPlan(None, 1, 1, 1, ctypes.byref(fam), ctypes.byref(lanes)) == api.STATUS_INVALID_VALUE


def test_topology_from_compute_unit_count():
    """32 compute units per XCD: a whole MI355X is eight, its partitions four, two and one; anything that is not a
    whole number of XCDs counts as one (the XCD-aware orders then turn into the plain order)."""
    import ctypes
    lib = _lib.load()
    for cus, want in ((256, 8), (128, 4), (64, 2), (32, 1), (304, 1), (120, 1), (1, 1), (512, 1)):
        xcds = ctypes.c_int(-1)
        assert lib.mcsparseXtopologyOfCuCount(cus, ctypes.byref(xcds)) == 0
        assert xcds.value == want, (cus, xcds.value)
    assert lib.mcsparseXtopologyOfCuCount(0, ctypes.byref(xcds)) != 0
    assert lib.mcsparseXtopologyOfCuCount(64, None) != 0


def test_spmv_deterministic_switch_is_off_by_default_and_checked():
    h = api.Handle()
    assert h.spmv_deterministic() is False
    h.set_spmv_deterministic(True)
    assert h.spmv_deterministic() is True
    h.set_spmv_deterministic(False)
    assert h.spmv_deterministic() is False
    lib = _lib.load()
    assert lib.mcsparseSetSpMVDeterministic(None, 1) == api.STATUS_NOT_INITIALIZED
    assert lib.mcsparseGetSpMVDeterministic(h.ptr, None) == api.STATUS_INVALID_VALUE
    h.destroy()


def test_spmv_preprocess_trial_switch_is_on_by_default_and_checked():
    h = api.Handle()
    assert h.spmv_preprocess_trial() is True
    h.set_spmv_preprocess_trial(False)
    assert h.spmv_preprocess_trial() is False
    h.set_spmv_preprocess_trial(True)
    assert h.spmv_preprocess_trial() is True
    lib = _lib.load()
    assert lib.mcsparseSetSpMVPreprocessTrial(None, 1) == api.STATUS_NOT_INITIALIZED
    assert lib.mcsparseGetSpMVPreprocessTrial(h.ptr, None) == api.STATUS_INVALID_VALUE
    h.destroy()
