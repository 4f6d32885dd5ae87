"""GPU parity of mcsparseSpMM (through the C ABI) against the CPU oracle; tolerance as for SpMV:
|C - C_ref| <= 8*u*(|alpha| * (|A||B|)_ij + |beta*C_ij|)."""
import numpy as np
import pytest

from mcsparse_amd import api
from mcsparse_amd import workloads as wl

from gpu_util import assert_within, dev

pytestmark = pytest.mark.gpu


def run_spmm(torch, handle, a, B, C0, alpha, beta, op_b=api.OP_N, b_order=api.ORDER_ROW, c_order=api.ORDER_ROW,
             pad_b=0, pad_c=0):
    """B is the k x n operand op(B); it is stored as the call's (op_b, b_order) pair requires."""
    k, n = B.shape
    dt = a.val.dtype
    # memory image of op(B): row-major k x n  <=>  (N, ROW) or (T, COL)
    b_row_image = (op_b == api.OP_N) == (b_order == api.ORDER_ROW)
    if b_row_image:
        ldb = n + pad_b
        img = np.zeros((k, ldb), dt)
        img[:, :n] = B
    else:
        ldb = k + pad_b
        img = np.zeros((n, ldb), dt)
        img[:, :k] = B.T
    if c_order == api.ORDER_ROW:
        ldc = n + pad_c
        cimg = np.full((a.m, ldc), 99.0, dt)
        cimg[:, :n] = C0
    else:
        ldc = a.m + pad_c
        cimg = np.full((n, ldc), 99.0, dt)
        cimg[:, :a.m] = C0.T
    d_ptr, d_col, d_val = dev(torch, a.ptr), dev(torch, a.col), dev(torch, a.val)
    d_B, d_C = dev(torch, img), dev(torch, cimg)
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val, base=a.base)
    b_rows, b_cols = (k, n) if op_b == api.OP_N else (n, k)
    mB = api.DnMat(b_rows, b_cols, ldb, d_B, order=b_order)
    mC = api.DnMat(a.m, n, ldc, d_C, order=c_order)
    ct = api.maca_type(dt)
    st, size = api.spmm_buffer_size(handle, api.OP_N, op_b, alpha, mat, mB, beta, mC, ct)
    assert st == 0 and size >= 128
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    st = api.spmm(handle, api.OP_N, op_b, alpha, mat, mB, beta, mC, ct, buf)
    torch.cuda.synchronize()
    out = d_C.cpu().numpy()
    if c_order == api.ORDER_ROW:
        got, padding = out[:, :n], out[:, n:]
    else:
        got, padding = out[:, :a.m].T, out[:, a.m:]
    assert (padding == 99.0).all(), "wrote outside the leading dimension"
    return st, got, (img, ldb, b_row_image)


def check(torch, handle, oracle, a, n, alpha, beta, seed=0, **kw):
    rng = np.random.default_rng(seed)
    dt = a.val.dtype
    B = rng.uniform(-1, 1, (a.n, n)).astype(dt)
    C0 = rng.uniform(-1, 1, (a.m, n)).astype(dt)
    st, got, (img, ldb, b_row_image) = run_spmm(torch, handle, a, B, C0, alpha, beta, **kw)
    assert st == 0
    c_ref, bound = oracle.spmm(a.m, n, a.base, a.ptr, a.col, a.val, alpha, beta, img.ravel(), ldb, b_row_image,
                               np.ascontiguousarray(C0).ravel(), n, True)
    return assert_within(np.ascontiguousarray(got), c_ref, bound, dt, what="spmm n=%d %r" % (n, kw))


@pytest.mark.parametrize("n", [1, 5, 8, 64, 100, 256, 260])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_row_major_widths(torch_gpu, handle, oracle, n, dtype):
    a = wl.random_ragged(1201, 907, 14, dtype=dtype, seed=n)
    check(torch_gpu, handle, oracle, a, n, 1.0, 0.0)
    check(torch_gpu, handle, oracle, a, n, -1.5, 0.75)


@pytest.mark.parametrize("op_b", [api.OP_N, api.OP_T])
@pytest.mark.parametrize("b_order", [api.ORDER_ROW, api.ORDER_COL])
@pytest.mark.parametrize("c_order", [api.ORDER_ROW, api.ORDER_COL])
def test_layouts(torch_gpu, handle, oracle, op_b, b_order, c_order):
    a = wl.random_ragged(700, 500, 9, dtype=np.float32, seed=3).with_base(1)
    for n, pb, pc in ((12, 0, 0), (12, 4, 8), (7, 3, 1)):
        check(torch_gpu, handle, oracle, a, n, 2.0, -0.5, op_b=op_b, b_order=b_order, c_order=c_order, pad_b=pb,
              pad_c=pc)
        check(torch_gpu, handle, oracle, a, n, 2.0, 0.0, op_b=op_b, b_order=b_order, c_order=c_order, pad_b=pb,
              pad_c=pc)


@pytest.mark.parametrize("n", [8, 64, 256])
def test_config4_stencil_reduced(torch_gpu, handle, oracle, n):
    a = wl.stencil_27pt(24, dtype=np.float32)
    assert a.nnz == (3 * 24 - 2) ** 3
    check(torch_gpu, handle, oracle, a, n, 1.0, 0.0)


def test_exact_cases(torch_gpu, handle):
    # identity times B is B; beta = 0 ignores NaN in C; nnz == 0 scales C
    n = 64
    m = 300
    eye = wl.Csr(m, m, np.arange(m + 1), np.arange(m), np.ones(m, np.float32))
    B = np.random.default_rng(1).uniform(-1, 1, (m, n)).astype(np.float32)
    st, got, _ = run_spmm(torch_gpu, handle, eye, B, np.full((m, n), np.nan, np.float32), 1.0, 0.0)
    assert st == 0 and np.array_equal(got, B)
    empty = wl.Csr(m, m, np.zeros(m + 1, np.int32), np.zeros(0, np.int32), np.zeros(0, np.float32))
    C0 = np.random.default_rng(2).uniform(-1, 1, (m, n)).astype(np.float32)
    st, got, _ = run_spmm(torch_gpu, handle, empty, B, C0, 1.0, 0.5)
    assert st == 0 and np.array_equal(got, 0.5 * C0)
    st, got, _ = run_spmm(torch_gpu, handle, empty, B, C0, 1.0, 1.0)  # early return (mcsp_spmm_gpu.cpp:110-114)
    assert st == 0 and np.array_equal(got, C0)
