"""Index sorts, the identity permutation and the gather, through the C ABI, bit-exact against the
CPU oracle (which the CPU suite pins against numpy's stable lexsort)."""
import ctypes

import numpy as np
import pytest

from mcsparse_amd import api
from mcsparse_amd import workloads as wl

from gpu_util import dev

pytestmark = pytest.mark.gpu


def _buffer(torch, handle, kind, m, n, nnz, a, b):
    st, size = api.sort_buffer_size(handle, kind, m, n, nnz, a, b)
    assert st == 0 and size % 128 == 0
    return torch.empty(size, dtype=torch.uint8, device="cuda")


@pytest.mark.parametrize("by", ["row", "column"])
@pytest.mark.parametrize("with_perm", [True, False])
@pytest.mark.parametrize("m,n,nnz,base", [(37, 53, 4000, 0), (5000, 3, 70000, 1), (300000, 70000, 1 << 20, 1),
                                          (1, 1, 5, 0), (9, 9, 1, 1)])
def test_coosort(torch_gpu, handle, oracle, by, with_perm, m, n, nnz, base):
    rng = np.random.default_rng(nnz + base)
    rows = (rng.integers(0, m, nnz) + base).astype(np.int32)
    cols = (rng.integers(0, max(1, n // 2), nnz) + base).astype(np.int32)  # repeated pairs: stability shows in perm
    perm0 = rng.permutation(nnz).astype(np.int32)
    d_r, d_c = dev(torch_gpu, rows), dev(torch_gpu, cols)
    d_p = dev(torch_gpu, perm0) if with_perm else None
    buf = _buffer(torch_gpu, handle, "coo", m, n, nnz, d_r, d_c)
    fn = api.xcoosort_by_row if by == "row" else api.xcoosort_by_column
    assert fn(handle, m, n, nnz, d_r, d_c, d_p, buf) == 0
    torch_gpu.cuda.synchronize()
    if by == "row":
        r, c, p = oracle.coosort(m + base, n + base, rows, cols, perm0 if with_perm else None)
    else:
        c, r, p = oracle.coosort(n + base, m + base, cols, rows, perm0 if with_perm else None)
    assert np.array_equal(d_r.cpu().numpy(), r.view(np.int32))
    assert np.array_equal(d_c.cpu().numpy(), c.view(np.int32))
    if with_perm:
        assert np.array_equal(d_p.cpu().numpy(), p.view(np.int32))


def _shuffle_rows(a, rng):
    col, val = a.col.copy(), a.val.copy()
    for r in np.flatnonzero(a.row_lengths() > 1):
        s, e = a.ptr[r] - a.base, a.ptr[r + 1] - a.base
        o = rng.permutation(e - s)
        col[s:e], val[s:e] = col[s:e][o], val[s:e][o]
    return col, val


@pytest.mark.parametrize("base", [0, 1])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_csrsort_then_gather_restores_a_sorted_matrix(torch_gpu, handle, oracle, base, dtype):
    """The use the reference makes of these calls (conversion/mcsp_csru2csr.cpp:63-77): identity
    permutation, sort the structure, gather the values through the permutation."""
    a = wl.power_law(m=3000, n=2500, max_len=1500, dtype=dtype).with_base(base)
    rng = np.random.default_rng(2)
    col, val = _shuffle_rows(a, rng)
    d_ptr, d_col, d_val = dev(torch_gpu, a.ptr), dev(torch_gpu, col), dev(torch_gpu, val)
    d_perm = torch_gpu.empty(a.nnz, dtype=torch_gpu.int32, device="cuda")
    d_sorted_val = torch_gpu.empty_like(d_val)
    descr = ctypes.c_void_p()
    lib = handle.lib
    assert lib.mcsparseCreateMatDescr(ctypes.byref(descr)) == 0
    assert lib.mcsparseSetMatIndexBase(descr, base) == 0
    assert api.create_identity_permutation(handle, a.nnz, d_perm) == 0
    buf = _buffer(torch_gpu, handle, "csr", a.m, a.n, a.nnz, d_ptr, d_col)
    assert api.xcsrsort(handle, a.m, a.n, a.nnz, descr, d_ptr, d_col, d_perm, buf) == 0
    assert api.gthr(handle, a.nnz, d_val, d_sorted_val, d_perm, api.BASE_ZERO) == 0
    torch_gpu.cuda.synchronize()
    ref_col, ref_perm = oracle.csrsort(a.m, a.n, base, a.ptr, col, np.arange(a.nnz, dtype=np.int32))
    assert np.array_equal(d_col.cpu().numpy(), ref_col.view(np.int32))
    assert np.array_equal(d_perm.cpu().numpy(), ref_perm.view(np.int32))
    assert np.array_equal(d_col.cpu().numpy(), a.col)           # back to the generator's sorted matrix
    assert np.array_equal(d_sorted_val.cpu().numpy(), a.val)    # bit-exact: values are only moved
    lib.mcsparseDestroyMatDescr(descr)


def test_cscsort_without_perm(torch_gpu, handle, oracle):
    a = wl.random_ragged(900, 1300, 6, dtype=np.float32, seed=9)  # read as the CSC of a 1300 x 900 matrix
    col, _ = _shuffle_rows(a, np.random.default_rng(4))
    d_ptr, d_ind = dev(torch_gpu, a.ptr), dev(torch_gpu, col)
    descr = ctypes.c_void_p()
    assert handle.lib.mcsparseCreateMatDescr(ctypes.byref(descr)) == 0
    buf = _buffer(torch_gpu, handle, "csc", 1300, 900, a.nnz, d_ptr, d_ind)
    assert api.xcscsort(handle, 1300, 900, a.nnz, descr, d_ptr, d_ind, None, buf) == 0
    torch_gpu.cuda.synchronize()
    assert np.array_equal(d_ind.cpu().numpy(), a.col)
    handle.lib.mcsparseDestroyMatDescr(descr)


def test_identity_and_gather_with_base(torch_gpu, handle):
    n = 100003
    d_p = torch_gpu.full((n,), -1, dtype=torch_gpu.int32, device="cuda")
    assert api.create_identity_permutation(handle, n, d_p) == 0
    torch_gpu.cuda.synchronize()
    assert np.array_equal(d_p.cpu().numpy(), np.arange(n, dtype=np.int32))
    rng = np.random.default_rng(0)
    y = rng.standard_normal(5000)
    ind = rng.integers(0, 5000, 777).astype(np.int32)
    d_x = torch_gpu.zeros(777, dtype=torch_gpu.float64, device="cuda")
    assert api.gthr(handle, 777, dev(torch_gpu, y), d_x, dev(torch_gpu, ind + 1), api.BASE_ONE) == 0
    torch_gpu.cuda.synchronize()
    assert np.array_equal(d_x.cpu().numpy(), y[ind])
