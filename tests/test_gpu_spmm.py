"""GPU parity of mcsparseSpMM (through the C ABI) against the CPU oracle; tolerance as for SpMV:
|C - C_ref| <= 8*u*(|alpha| * (|A||B|)_ij + |beta*C_ij|)."""
import numpy as np
import pytest

from mcsparse_amd import api
from mcsparse_amd import workloads as wl

from gpu_util import assert_within, dev

pytestmark = pytest.mark.gpu


def run_spmm(torch, handle, a, B, C0, alpha, beta, op_b=api.OP_N, b_order=api.ORDER_ROW, c_order=api.ORDER_ROW,
             pad_b=0, pad_c=0, preprocess=False, expect_schedule=None):
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
    if preprocess:
        assert api.spmm_preprocess(handle, api.OP_N, op_b, alpha, mat, mB, beta, mC, ct, buf) == 0
        if expect_schedule is not None:
            assert mat.spmm_schedule()[0] == expect_schedule, mat.spmm_schedule()
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


# ---- row-group schedule (mcsparseSpMM_preprocess) ------------------------------------------------

@pytest.mark.parametrize("n", [4, 8, 24, 64, 100, 256, 260])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_preprocessed_stencil(torch_gpu, handle, oracle, n, dtype):
    a = wl.stencil_27pt(13, dtype=dtype).with_base(1)  # row count not a multiple of the group size: the last group is short
    for c_order in (api.ORDER_ROW, api.ORDER_COL):
        check(torch_gpu, handle, oracle, a, n, 1.0, 0.0, preprocess=True, expect_schedule=2, c_order=c_order)
        check(torch_gpu, handle, oracle, a, n, -1.5, 0.75, preprocess=True, expect_schedule=2, c_order=c_order, pad_b=4,
              pad_c=8)


def test_preprocessed_stencil_in_xcd_stretches(torch_gpu, handle, oracle):
    """A stencil large enough for the row-group kernel to hand every XCD stretches of several
    workgroups (the column span of a 48^3 stencil is 4,706 rows), with a last round that is only
    partly filled."""
    a = wl.stencil_27pt(48, dtype=np.float32)
    for n in (64, 40):
        check(torch_gpu, handle, oracle, a, n, 1.0, 0.0, preprocess=True, expect_schedule=2)
    check(torch_gpu, handle, oracle, a, 64, 0.5, -1.0, preprocess=True, expect_schedule=2, c_order=api.ORDER_COL)


def test_preprocessed_ragged_rows_with_overlap(torch_gpu, handle, oracle):
    """Rows of different lengths, empty rows, unsorted columns inside rows, a group too long to merge."""
    rng = np.random.default_rng(12)
    m, k = 501, 3000
    rows = []
    for r in range(m):
        if r % 7 == 3:
            cols = np.zeros(0, np.int64)
        elif r in (100, 101):
            cols = rng.choice(k, 1100, replace=False)           # 2200 nonzeros in their group: not merged
        else:
            prev = rows[-1] if rows and len(rows[-1]) else rng.choice(k, 12, replace=False)
            keep = prev[rng.random(len(prev)) < 0.8]
            cols = np.unique(np.concatenate([keep, rng.choice(k, rng.integers(0, 6), replace=False)]))
        if r % 5 == 0:
            cols = rng.permutation(cols)                           # unsorted storage order
        rows.append(cols)
    ptr = np.concatenate([[0], np.cumsum([len(c) for c in rows])]).astype(np.int32)
    col = np.concatenate(rows).astype(np.int32)
    a = wl.Csr(m, k, ptr, col, rng.uniform(-1, 1, len(col)).astype(np.float32))
    for n in (8, 64, 72):
        check(torch_gpu, handle, oracle, a, n, 1.0, 0.0, preprocess=True, expect_schedule=2)
        check(torch_gpu, handle, oracle, a, n, 0.5, 2.0, preprocess=True, expect_schedule=2)


def test_preprocess_declines_rows_without_shared_columns(torch_gpu, handle, oracle):
    a = wl.random_ragged(2000, 100000, 10, dtype=np.float32, seed=1)
    check(torch_gpu, handle, oracle, a, 64, 1.0, 0.0, preprocess=True, expect_schedule=1)


def test_preprocessed_row_ignores_columns_only_its_partner_has(torch_gpu, handle):
    """Row 0 = {0}, row 1 = {1}: an infinity in B row 1 must not reach C row 0 (0 * inf = NaN)."""
    a = wl.Csr(2, 2, np.array([0, 1, 2], np.int32), np.array([0, 1], np.int32), np.array([2.0, 3.0], np.float32))
    a2 = wl.Csr(4, 2, np.array([0, 2, 3, 5, 6], np.int32), np.array([0, 1, 0, 0, 1, 0], np.int32),
                np.array([1, 1, 2, 1, 1, 5], np.float32))       # shares columns, so the schedule is used
    B = np.ones((2, 8), np.float32)
    B[1, :] = np.inf
    st, got, _ = run_spmm(torch_gpu, handle, a2, B, np.zeros((4, 8), np.float32), 1.0, 0.0, preprocess=True,
                          expect_schedule=2)
    assert st == 0
    assert np.all(np.isinf(got[0])) and np.all(got[1] == 2.0) and np.all(np.isinf(got[2])) and np.all(got[3] == 5.0)
    del a


def test_schedule_is_dropped_with_other_buffer_or_pointers(torch_gpu, handle, oracle):
    a = wl.stencil_27pt(10, dtype=np.float32)
    n = 16
    rng = np.random.default_rng(0)
    B = rng.uniform(-1, 1, (a.n, n)).astype(np.float32)
    d_ptr, d_col, d_val = dev(torch_gpu, a.ptr), dev(torch_gpu, a.col), dev(torch_gpu, a.val)
    d_B = dev(torch_gpu, B)
    d_C = torch_gpu.zeros((a.m, n), dtype=torch_gpu.float32, device="cuda")
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val)
    mB, mC = api.DnMat(a.n, n, n, d_B), api.DnMat(a.m, n, n, d_C)
    st, size = api.spmm_buffer_size(handle, 0, 0, 1.0, mat, mB, 0.0, mC, api.R_32F)
    buf = torch_gpu.empty(size, dtype=torch_gpu.uint8, device="cuda")
    other = torch_gpu.zeros(size, dtype=torch_gpu.uint8, device="cuda")  # zeros: unusable as a schedule
    assert api.spmm_preprocess(handle, 0, 0, 1.0, mat, mB, 0.0, mC, api.R_32F, buf) == 0
    assert mat.spmm_schedule()[0] == 2 and mat.spmm_schedule()[1] < a.nnz
    c_ref, bound = oracle.spmm(a.m, n, 0, a.ptr, a.col, a.val, 1.0, 0.0, B.ravel(), n, True, np.zeros(a.m * n, np.float32),
                               n, True)
    for b in (buf, other):   # with the other buffer the schedule-free kernel must run
        d_C.zero_()
        assert api.spmm(handle, 0, 0, 1.0, mat, mB, 0.0, mC, api.R_32F, b) == 0
        torch_gpu.cuda.synchronize()
        assert_within(d_C.cpu().numpy(), c_ref, bound, np.float32)
    d_col2 = d_col.clone()
    assert handle.lib.mcsparseCsrSetPointers(mat.ptr, d_ptr.data_ptr(), d_col2.data_ptr(), d_val.data_ptr()) == 0
    assert mat.spmm_schedule()[0] == 0


def test_overwritten_schedule_stays_in_bounds(torch_gpu, handle):
    """The reference's preprocess is a no-op, so a caller written against it may reuse the scratch
    buffer between preprocess and SpMM.  The schedule is then garbage: the product may be wrong, but
    every access stays inside the arrays (the call returns and the device stays healthy)."""
    torch = torch_gpu
    a = wl.stencil_27pt(10, dtype=np.float32)
    n = 64
    d_ptr, d_col, d_val = dev(torch, a.ptr), dev(torch, a.col), dev(torch, a.val)
    d_B = torch.ones((a.n, n), dtype=torch.float32, device="cuda")
    d_C = torch.zeros((a.m, n), dtype=torch.float32, device="cuda")
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val)
    mB, mC = api.DnMat(a.n, n, n, d_B), api.DnMat(a.m, n, n, d_C)
    st, size = api.spmm_buffer_size(handle, api.OP_N, api.OP_N, 1.0, mat, mB, 0.0, mC, api.R_32F)
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    assert api.spmm_preprocess(handle, api.OP_N, api.OP_N, 1.0, mat, mB, 0.0, mC, api.R_32F, buf) == 0
    assert mat.spmm_schedule()[0] == 2
    gen = torch.Generator(device="cuda")
    gen.manual_seed(3)
    for fill in (0xFF, None, 0x00):
        if fill is None:
            buf.copy_(torch.randint(0, 256, (size,), dtype=torch.uint8, device="cuda", generator=gen))
        else:
            buf.fill_(fill)
        assert api.spmm(handle, api.OP_N, api.OP_N, 1.0, mat, mB, 0.0, mC, api.R_32F, buf) == 0
        torch.cuda.synchronize()
    # a fresh preprocess makes the same buffer good again
    assert api.spmm_preprocess(handle, api.OP_N, api.OP_N, 1.0, mat, mB, 0.0, mC, api.R_32F, buf) == 0
    assert api.spmm(handle, api.OP_N, api.OP_N, 1.0, mat, mB, 0.0, mC, api.R_32F, buf) == 0
    torch.cuda.synchronize()
    want = np.asarray(a.to_scipy().sum(axis=1)).ravel()  # B = ones: row sums of A
    got = d_C.cpu().numpy()
    assert np.allclose(got, want[:, None].repeat(n, 1), rtol=1e-5, atol=1e-5)
