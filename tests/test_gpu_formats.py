"""COO (row-sorted) input to SpMV / SpMM and CSC input to SpMM, through the C ABI, against the
CPU oracle applied to the same matrix in CSR form."""
import numpy as np
import pytest

from mcsparse_amd import api
from mcsparse_amd import workloads as wl

from gpu_util import assert_within, dev

pytestmark = pytest.mark.gpu


def coo_rows_of(a):
    return (np.repeat(np.arange(a.m, dtype=np.int64), a.row_lengths()) + a.base).astype(np.int32)


@pytest.mark.parametrize("op", [api.OP_N, api.OP_T])
@pytest.mark.parametrize("base", [0, 1])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_coo_spmv(torch_gpu, handle, oracle, op, base, dtype):
    a = wl.power_law(m=7000, n=5000, max_len=3000, dtype=dtype).with_base(base)  # skewed, has 1-nnz rows
    rng = np.random.default_rng(3)
    t = op != api.OP_N
    xs, ys = (a.m, a.n) if t else (a.n, a.m)
    x = rng.uniform(-1, 1, xs).astype(dtype)
    y0 = rng.uniform(-1, 1, ys).astype(dtype)
    d_row, d_col, d_val = dev(torch_gpu, coo_rows_of(a)), dev(torch_gpu, a.col), dev(torch_gpu, a.val)
    d_x, d_y = dev(torch_gpu, x), dev(torch_gpu, y0)
    mat = api.SpMat(a.m, a.n, a.nnz, d_row, d_col, d_val, base=base, fmt=api.FORMAT_COO)
    vx, vy = api.DnVec(d_x), api.DnVec(d_y)
    ct = api.maca_type(dtype)
    st, size = api.spmv_buffer_size(handle, op, 1.5, mat, vx, 0.5, vy, ct)
    assert st == 0 and size % 128 == 0
    buf = torch_gpu.empty(size, dtype=torch_gpu.uint8, device="cuda")
    for _ in range(2):  # second call reuses the cached plan
        d_y.copy_(dev(torch_gpu, y0))
        assert api.spmv(handle, op, 1.5, mat, vx, 0.5, vy, ct, buf) == 0
        torch_gpu.cuda.synchronize()
        y_ref, bound = oracle.spmv(t, a.m, a.n, base, a.ptr, a.col, a.val, 1.5, 0.5, x, y0)
        assert_within(d_y.cpu().numpy(), y_ref, bound, dtype, what="COO SpMV op=%d" % op)


def test_coo_with_empty_leading_and_trailing_rows(torch_gpu, handle, oracle):
    a = wl.random_ragged(400, 300, 5, dtype=np.float32, seed=8, empty_fraction=0.5)
    a.ptr[:4] = a.ptr[0]   # first three rows empty
    # (lengths are re-derived from ptr, so the matrix stays consistent)
    a2 = wl.Csr(a.m, a.n, np.concatenate([np.zeros(3, np.int32), a.ptr[3:] - a.ptr[3]]),
                a.col[a.ptr[3]:], a.val[a.ptr[3]:])
    x = np.random.default_rng(0).uniform(-1, 1, a2.n).astype(np.float32)
    y0 = np.ones(a2.m, np.float32)
    d_y = dev(torch_gpu, y0)
    mat = api.SpMat(a2.m, a2.n, a2.nnz, dev(torch_gpu, coo_rows_of(a2)), dev(torch_gpu, a2.col),
                    dev(torch_gpu, a2.val), fmt=api.FORMAT_COO)
    vx, vy = api.DnVec(dev(torch_gpu, x)), api.DnVec(d_y)
    st, size = api.spmv_buffer_size(handle, api.OP_N, 1.0, mat, vx, 2.0, vy, api.R_32F)
    buf = torch_gpu.empty(size, dtype=torch_gpu.uint8, device="cuda")
    assert api.spmv(handle, api.OP_N, 1.0, mat, vx, 2.0, vy, api.R_32F, buf) == 0
    torch_gpu.cuda.synchronize()
    y_ref, bound = oracle.spmv(False, a2.m, a2.n, 0, a2.ptr, a2.col, a2.val, 1.0, 2.0, x, y0)
    assert_within(d_y.cpu().numpy(), y_ref, bound, np.float32)


@pytest.mark.parametrize("fmt", [api.FORMAT_COO, api.FORMAT_CSC])
@pytest.mark.parametrize("n", [4, 64])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_coo_and_csc_spmm(torch_gpu, handle, oracle, fmt, n, dtype):
    base = 1
    a = wl.random_ragged(1100, 800, 9, dtype=dtype, seed=n).with_base(base)
    rng = np.random.default_rng(4)
    B = rng.uniform(-1, 1, (a.n, n)).astype(dtype)
    C0 = rng.uniform(-1, 1, (a.m, n)).astype(dtype)
    if fmt == api.FORMAT_COO:
        arrays = (coo_rows_of(a), a.col, a.val)
    else:
        cp, ri, cv = oracle.csr2csc(a.m, a.n, base, a.ptr, a.col, a.val, method="counting")
        arrays = (cp.view(np.int32), ri.view(np.int32), cv)
    d0, d1, d2 = (dev(torch_gpu, v) for v in arrays)
    mat = api.SpMat(a.m, a.n, a.nnz, d0, d1, d2, base=base, fmt=fmt)
    d_B, d_C = dev(torch_gpu, B), dev(torch_gpu, C0)
    mB, mC = api.DnMat(a.n, n, n, d_B), api.DnMat(a.m, n, n, d_C)
    ct = api.maca_type(dtype)
    st, size = api.spmm_buffer_size(handle, api.OP_N, api.OP_N, 2.0, mat, mB, -1.0, mC, ct)
    assert st == 0 and size % 128 == 0 and size >= (a.m + 1) * 4
    buf = torch_gpu.empty(size, dtype=torch_gpu.uint8, device="cuda")
    assert api.spmm(handle, api.OP_T, api.OP_N, 2.0, mat, mB, -1.0, mC, ct, buf) == api.STATUS_NOT_SUPPORTED
    assert api.spmm(handle, api.OP_N, api.OP_N, 2.0, mat, mB, -1.0, mC, ct, buf) == 0
    torch_gpu.cuda.synchronize()
    c_ref, bound = oracle.spmm(a.m, n, base, a.ptr, a.col, a.val, 2.0, -1.0, B.ravel(), n, True, C0.ravel(), n, True)
    assert_within(d_C.cpu().numpy(), c_ref, bound, dtype, what="SpMM fmt=%d" % fmt)


@pytest.mark.parametrize("fmt", [api.FORMAT_COO, api.FORMAT_CSC])
def test_empty_matrix_scales_c(torch_gpu, handle, fmt):
    m, k, n = 50, 40, 8
    ptr_len = m if fmt == api.FORMAT_COO else k + 1
    d0 = torch_gpu.zeros(max(ptr_len, 1), dtype=torch_gpu.int32, device="cuda")
    d1 = torch_gpu.zeros(1, dtype=torch_gpu.int32, device="cuda")
    d2 = torch_gpu.zeros(1, dtype=torch_gpu.float32, device="cuda")
    mat = api.SpMat(m, k, 0, d0, d1, d2, fmt=fmt)
    C0 = np.random.default_rng(1).uniform(-1, 1, (m, n)).astype(np.float32)
    d_B = torch_gpu.ones((k, n), dtype=torch_gpu.float32, device="cuda")
    d_C = dev(torch_gpu, C0)
    mB, mC = api.DnMat(k, n, n, d_B), api.DnMat(m, n, n, d_C)
    st, size = api.spmm_buffer_size(handle, 0, 0, 1.0, mat, mB, 0.5, mC, api.R_32F)
    buf = torch_gpu.empty(size, dtype=torch_gpu.uint8, device="cuda")
    assert api.spmm(handle, 0, 0, 1.0, mat, mB, 0.5, mC, api.R_32F, buf) == 0
    torch_gpu.cuda.synchronize()
    assert np.array_equal(d_C.cpu().numpy(), 0.5 * C0)
