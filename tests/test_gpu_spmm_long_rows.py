"""mcsparseSpMM on matrices with rows far longer than the rest: rows above 1024 nonzeros are cut into pieces of
4096 that a workgroup each takes (one piece: the row of C written directly; several: partial sums added in the order
of the pieces).  Parity against the CPU oracle within 8*u*(|alpha| * (|A||B|)_ij + |beta*C_ij|), bits that repeat
from run to run, and the time of a call."""
import numpy as np
import pytest

from mcsparse_amd import api
from mcsparse_amd import workloads as wl

from gpu_util import assert_within, dev
from test_gpu_spmm import check, run_spmm

pytestmark = pytest.mark.gpu


def rows_of_lengths(lengths, n_cols, dtype, seed, base=0):
    """CSR matrix whose row i holds lengths[i] nonzeros in distinct, sorted, random columns."""
    rng = np.random.default_rng(seed)
    ptr = np.zeros(len(lengths) + 1, np.int64)
    ptr[1:] = np.cumsum(lengths)
    col = np.empty(ptr[-1], np.int32)
    for i, length in enumerate(lengths):
        col[ptr[i]:ptr[i + 1]] = np.sort(rng.choice(n_cols, size=length, replace=False))
    val = rng.uniform(-1, 1, ptr[-1]).astype(dtype)
    return wl.Csr(len(lengths), n_cols, ptr.astype(np.int32) + base, col + base, val, base=base)


# lengths around the two limits (1024: taken apart from the row kernels; 4096: one piece), empty rows between long ones
LENGTHS = [3, 1024, 1025, 0, 4095, 4096, 4097, 7, 0, 8192, 8193, 12289, 1, 2000, 0, 20000, 5, 1500, 16, 0]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n", [1, 3, 8, 16, 33, 64, 100, 260])
def test_rows_around_the_limits(torch_gpu, handle, oracle, n, dtype):
    a = rows_of_lengths(LENGTHS * 3, 30011, dtype, seed=n)
    check(torch_gpu, handle, oracle, a, n, 1.0, 0.0)
    check(torch_gpu, handle, oracle, a, n, -1.5, 0.75, seed=1)


@pytest.mark.parametrize("op_b", [api.OP_N, api.OP_T])
@pytest.mark.parametrize("b_order", [api.ORDER_ROW, api.ORDER_COL])
@pytest.mark.parametrize("c_order", [api.ORDER_ROW, api.ORDER_COL])
def test_layouts_and_padding(torch_gpu, handle, oracle, op_b, b_order, c_order):
    a = rows_of_lengths(LENGTHS, 25013, np.float32, seed=4, base=1)
    check(torch_gpu, handle, oracle, a, 24, 0.5, -2.0, op_b=op_b, b_order=b_order, c_order=c_order, pad_b=3, pad_c=5)
    check(torch_gpu, handle, oracle, a, 7, 0.5, 0.0, op_b=op_b, b_order=b_order, c_order=c_order, pad_b=1, pad_c=2)


def test_long_rows_among_many_short_ones(torch_gpu, handle, oracle):
    """The matrix of the mixed SpMV workload, smaller: 20,000 rows of 16 and 8 rows of 30,000."""
    a = wl.mixed_rows(m=20000, per_row=16, long_rows=8, long_len=30000, dtype=np.float32)
    for n in (8, 16, 64, 128):
        check(torch_gpu, handle, oracle, a, n, 1.25, 0.5, seed=n)


def test_preprocess_leaves_such_a_matrix_to_the_row_kernels(torch_gpu, handle, oracle):
    a = wl.mixed_rows(m=20000, per_row=16, long_rows=8, long_len=30000, dtype=np.float32)
    check(torch_gpu, handle, oracle, a, 64, 1.0, 0.0, preprocess=True, expect_schedule=1)
    check(torch_gpu, handle, oracle, a, 16, 1.0, 0.5, preprocess=True, expect_schedule=1)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_bits_repeat_from_run_to_run(torch_gpu, handle, dtype):
    a = rows_of_lengths(LENGTHS * 2, 30011, dtype, seed=9)
    rng = np.random.default_rng(3)
    B = rng.uniform(-1, 1, (a.n, 40)).astype(dtype)
    C0 = rng.uniform(-1, 1, (a.m, 40)).astype(dtype)
    first = None
    for _ in range(3):
        st, got, _ = run_spmm(torch_gpu, handle, a, B, C0, 1.5, 0.25)
        assert st == 0
        if first is None:
            first = got.copy()
        assert np.array_equal(first, got)


@pytest.mark.parametrize("fmt", ["coo", "csc"])
def test_coo_and_csc_inputs(torch_gpu, handle, oracle, fmt):
    torch = torch_gpu
    a = rows_of_lengths(LENGTHS, 20011, np.float64, seed=11)
    n = 12
    rng = np.random.default_rng(12)
    B = rng.uniform(-1, 1, (a.n, n))
    C0 = rng.uniform(-1, 1, (a.m, n))
    d_B, d_C = dev(torch, B), dev(torch, C0)
    if fmt == "coo":
        rows = np.repeat(np.arange(a.m, dtype=np.int32), np.diff(a.ptr))
        keep = [dev(torch, rows), dev(torch, a.col), dev(torch, a.val)]
        mat = api.SpMat(a.m, a.n, a.nnz, keep[0], keep[1], keep[2], fmt=api.FORMAT_COO)
    else:
        t_ptr, t_row, t_val = oracle.csr2csc(a.m, a.n, 0, a.ptr, a.col, a.val, method="counting")
        keep = [dev(torch, t_ptr.astype(np.int32)), dev(torch, t_row.astype(np.int32)), dev(torch, t_val)]
        mat = api.SpMat(a.m, a.n, a.nnz, keep[0], keep[1], keep[2], fmt=api.FORMAT_CSC)  # offsets, then indices
    mB, mC = api.DnMat(a.n, n, n, d_B), api.DnMat(a.m, n, n, d_C)
    st, size = api.spmm_buffer_size(handle, api.OP_N, api.OP_N, 2.0, mat, mB, -1.0, mC, api.R_64F)
    assert st == 0
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    assert api.spmm(handle, api.OP_N, api.OP_N, 2.0, mat, mB, -1.0, mC, api.R_64F, buf) == 0
    torch.cuda.synchronize()
    c_ref, bound = oracle.spmm(a.m, n, 0, a.ptr, a.col, a.val, 2.0, -1.0, B.ravel(), n, True, C0.ravel(), n, True)
    assert_within(d_C.cpu().numpy(), c_ref, bound, np.float64, what="spmm long rows, %s input" % fmt)


def test_a_row_of_fifty_thousand_does_not_hold_the_call_up(torch_gpu, handle):
    """1 M power-law rows, the longest of 50,000 nonzeros, N = 16: 7.3 ms when that row was one lane group's work;
    the operands are 0.35 GB, so anything near a millisecond says the row is being walked alone again."""
    torch = torch_gpu
    a = wl.power_law(m=1 << 20, max_len=50000, dtype=np.float32)
    n = 16
    d = [dev(torch, v) for v in (a.ptr, a.col, a.val)]
    B = torch.rand((a.n, n), dtype=torch.float32, device="cuda")
    C = torch.zeros((a.m, n), dtype=torch.float32, device="cuda")
    mat = api.SpMat(a.m, a.n, a.nnz, d[0], d[1], d[2], base=a.base)
    mB, mC = api.DnMat(a.n, n, n, B), api.DnMat(a.m, n, n, C)
    st, size = api.spmm_buffer_size(handle, api.OP_N, api.OP_N, 1.0, mat, mB, 0.0, mC, api.R_32F)
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    for _ in range(3):
        assert api.spmm(handle, api.OP_N, api.OP_N, 1.0, mat, mB, 0.0, mC, api.R_32F, buf) == 0
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(10):
        api.spmm(handle, api.OP_N, api.OP_N, 1.0, mat, mB, 0.0, mC, api.R_32F, buf)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / 10
    assert ms < 2.0, ms
