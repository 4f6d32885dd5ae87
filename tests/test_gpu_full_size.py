"""Parity at the full sizes of the benchmark configurations (config 2 is in test_gpu_spmv.py).

The CPU oracle is plain C and finishes these sizes in seconds, so SpMV and the conversions are
compared with it directly; SpMM is compared on a sample of rows (the oracle's long-double triple
loop over 2 M rows x 64 columns would take minutes) plus a linearity property over all rows."""
import numpy as np
import pytest

from mcsparse_amd import api
from mcsparse_amd import workloads as wl

from gpu_util import assert_within, dev, run_spmv
from test_gpu_convert import gpu_csr2coo, gpu_csr2csc
from test_gpu_spmm import run_spmm
from test_gpu_spmv_banded import run_banded
from test_gpu_spmv_column_order import run as run_column_order

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def power_law_full():
    a = wl.power_law(m=1 << 22, max_len=200000, dtype=np.float32)
    assert a.m == 4194304 and a.nnz > 100_000_000 and a.row_lengths().max() > 100_000
    return a


def test_config3_power_law_full_size(torch_gpu, handle, oracle, power_law_full):
    a = power_law_full
    rng = np.random.default_rng(3)
    x = rng.uniform(-1, 1, a.n).astype(np.float32)
    st, y, plan = run_spmv(torch_gpu, handle, a, x, np.zeros(a.m, np.float32), 1.0, 0.0)
    assert st == 0 and plan == (api.FAMILY_MERGE, 1)  # long rows, x of 16.8 MB: tiles in column order
    y_ref, bound = oracle.spmv(False, a.m, a.n, 0, a.ptr, a.col, a.val, 1.0, 0.0, x, None)
    worst = assert_within(y, y_ref, bound, np.float32, what="C3 op N")
    # Tiles take their places inside a column bucket in whatever order the atomics hand out, so a second
    # call runs them in another order: that cannot change a single bit of the result.
    st, y_again, _ = run_spmv(torch_gpu, handle, a, x, np.zeros(a.m, np.float32), 1.0, 0.0)
    assert st == 0 and np.array_equal(y_again.view(np.uint32), y.view(np.uint32))
    # the copy in column order (MCSPARSE_SPMV_CSR_ALG1): 8 planes of partial sums, two 1 MiB bands each
    state, bands, rows = run_banded(torch_gpu, handle, oracle, a, 1.0, 0.0, what="C3 op N, column order",
                                    reference=(x, y_ref, bound), alg=api.SPMV_CSR_ALG1, expect_state=3, calls=2)
    assert (bands, rows) == (8, 16384)
    # tiles in storage order are twice as long, which moves the seams between partial sums
    st, y_plain, _ = run_spmv(torch_gpu, handle, a, x, np.zeros(a.m, np.float32), 1.0, 0.0, family=api.FAMILY_MERGE)
    assert st == 0
    assert_within(y_plain, y_ref, bound, np.float32, what="C3 op N, tiles in storage order")
    # op T through the library's own transposition
    xt = rng.uniform(-1, 1, a.m).astype(np.float32)
    st, yt, _ = run_spmv(torch_gpu, handle, a, xt, np.zeros(a.n, np.float32), 1.0, 0.0, op=api.OP_T)
    assert st == 0
    yt_ref, bound_t = oracle.spmv(True, a.m, a.n, 0, a.ptr, a.col, a.val, 1.0, 0.0, xt, None)
    assert_within(yt, yt_ref, bound_t, np.float32, what="C3 op T")
    # op T from the copy in column order: x is gathered by row, and the long rows take most of the gathers (the row
    # lengths tell the preprocess call), so one band group spans all of x
    state, bands, rows, _, _ = run_column_order(torch_gpu, handle, oracle, a, 1.0, 0.0, op=api.OP_T,
                                                what="C3 op T, column order")
    assert (state, bands, rows) == (3, 1, 16384)


def test_config5_conversions_full_size(torch_gpu, handle, oracle, power_law_full):
    a = power_law_full
    st, coo = gpu_csr2coo(torch_gpu, handle, a)
    assert st == 0 and np.array_equal(coo.view(np.uint32), oracle.csr2coo(a.m, 0, a.ptr, a.nnz))
    del coo
    st, cp, ri, cv = gpu_csr2csc(torch_gpu, handle, a)
    assert st == 0
    w_cp, w_ri, w_cv = oracle.csr2csc(a.m, a.n, 0, a.ptr, a.col, a.val, method="counting")
    assert np.array_equal(cp.view(np.uint32), w_cp)
    assert np.array_equal(ri.view(np.uint32), w_ri)
    assert np.array_equal(cv.view(np.uint32), w_cv.view(np.uint32))
    # transposed SpMV from the produced CSC (descriptor of A in CSC format, op T -> direct kernel)
    rng = np.random.default_rng(5)
    xt = rng.uniform(-1, 1, a.m).astype(np.float32)
    csc_as_csr = wl.Csr(a.n, a.m, cp, ri, cv)  # arrays of A^T in CSR form
    st, yt, plan = run_spmv(torch_gpu, handle, csc_as_csr, xt, np.zeros(a.n, np.float32), 1.0, 0.0, op=api.OP_T,
                            fmt=api.FORMAT_CSC)
    # 28 +- 5 nonzeros per row of A^T: rows of 33 and more keep every wavefront of the vector family waiting
    assert st == 0 and plan[0] == api.FAMILY_MERGE
    yt_ref, bound_t = oracle.spmv(True, a.m, a.n, 0, a.ptr, a.col, a.val, 1.0, 0.0, xt, None)
    assert_within(yt, yt_ref, bound_t, np.float32, what="C5 A^T x from CSC")
    # the same product from the column-banded copy of mcsparseSpMV_preprocess (x = 16.8 MB: 8 bands)
    state, bands, rows = run_banded(torch_gpu, handle, oracle, csc_as_csr, 1.0, 0.0, as_csc=True,
                                    what="C5 A^T x from CSC, banded", reference=(xt, yt_ref, bound_t))
    assert (state, bands) == (2, 8)
    # and from the copy in column order: the long rows of A make a few lines of x take most of the gathers (78 % in
    # the 16384 hottest lines), which a sample of the indices shows the preprocess call: one band group over all of x
    state, bands, rows = run_banded(torch_gpu, handle, oracle, csc_as_csr, 1.0, 0.0, as_csc=True, calls=2,
                                    what="C5 A^T x from CSC, column order", reference=(xt, yt_ref, bound_t),
                                    alg=api.SPMV_CSR_ALG1, expect_state=3)
    assert (bands, rows) == (1, 16384)


def test_config2_full_size_banded(torch_gpu, handle, oracle):
    a = wl.uniform_rows(m=1 << 20, per_row=16, dtype=np.float64)
    assert a.nnz == 16777216
    state, bands, rows = run_banded(torch_gpu, handle, oracle, a, 1.5, 0.5, calls=2, what="C2 banded")
    assert (state, bands) == (2, 4)


def test_config2_margin_against_the_literal_bound(torch_gpu, handle, oracle):
    """Config 2 runs with alpha = 1.5, beta = 0.5, for which the tests accept 8u * (|alpha| (|A||x|)_i + |beta y_i|), the
    bound the stated one turns into when the sum is scaled and added to beta * y.  Here the same results are held
    against the literal (|A||x|)_i of the statement: the worst error, in units of u * (|A||x|)_i, of the direct kernel
    and of both preprocessed copies is printed and stays below 8 by a wide margin."""
    torch = torch_gpu
    a = wl.uniform_rows(m=1 << 20, per_row=16, dtype=np.float64)
    rng = np.random.default_rng(2)
    x = rng.uniform(-1, 1, a.n)
    y = rng.uniform(-1, 1, a.m)
    y_ref, _ = oracle.spmv(False, a.m, a.n, 0, a.ptr, a.col, a.val, 1.5, 0.5, x, y)
    _, literal = oracle.spmv(False, a.m, a.n, 0, a.ptr, a.col, a.val, 1.0, 0.0, x, None)  # (|A||x|)_i
    u = 2.0 ** -53
    d_ptr, d_col, d_val, d_x = dev(torch, a.ptr), dev(torch, a.col), dev(torch, a.val), dev(torch, x)
    worst = {}
    for name, alg, pre in (("direct", api.SPMV_ALG_DEFAULT, False), ("column order", api.SPMV_ALG_DEFAULT, True),
                           ("banded", api.SPMV_CSR_ALG2, True)):
        d_y = dev(torch, y)
        mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val)
        vx, vy = api.DnVec(d_x), api.DnVec(d_y)
        size_of = api.spmv_preprocess_buffer_size if pre else api.spmv_buffer_size
        st, size = size_of(handle, api.OP_N, 1.5, mat, vx, 0.5, vy, api.R_64F, **({"alg": alg} if pre else {}))
        assert st == api.STATUS_SUCCESS
        buf = torch.empty(size, dtype=torch.uint8, device="cuda")
        if pre:
            assert api.spmv_preprocess(handle, api.OP_N, 1.5, mat, vx, 0.5, vy, api.R_64F, buf, alg=alg) == api.STATUS_SUCCESS
        assert api.spmv(handle, api.OP_N, 1.5, mat, vx, 0.5, vy, api.R_64F, buf, alg=alg) == api.STATUS_SUCCESS
        torch.cuda.synchronize()
        err = np.abs(d_y.cpu().numpy().astype(np.longdouble) - y_ref)
        worst[name] = float((err / (u * literal)).max())
    print("config 2, worst |y - y_ref| / (u (|A||x|)_i):", {k: round(v, 3) for k, v in worst.items()})
    assert max(worst.values()) <= 8.0, worst


def test_config2_full_size_column_order(torch_gpu, handle, oracle):
    a = wl.uniform_rows(m=1 << 20, per_row=16, dtype=np.float64)
    state, bands, rows = run_banded(torch_gpu, handle, oracle, a, 1.5, 0.5, calls=2, what="C2 column order",
                                    alg=api.SPMV_CSR_ALG1, expect_state=3)
    assert (bands, rows) == (4, 16384)


@pytest.fixture(scope="module")
def stencil_full():
    a = wl.stencil_27pt(128, dtype=np.float32)
    assert (a.m, a.nnz) == (2097152, 55742968)
    return a


# preprocess = True runs the kernels that work from a schedule: blocks over groups of strips (state 4) for N = 64 and 256; for
# N = 8 merged column lists are built (state 2) but too narrow to use
@pytest.mark.parametrize("preprocess", [False, True])
@pytest.mark.parametrize("n", [8, 64, 256])
def test_config4_stencil_full_size(torch_gpu, handle, oracle, stencil_full, n, preprocess):
    a = stencil_full
    rng = np.random.default_rng(n)
    B = rng.uniform(-1, 1, (a.n, n)).astype(np.float32)
    st, got, _ = run_spmm(torch_gpu, handle, a, B, np.zeros((a.m, n), np.float32), 1.0, 0.0, preprocess=preprocess,
                          expect_schedule=(2 if n == 8 else 4) if preprocess else None)
    assert st == 0
    # oracle on a sample of rows: first/last planes, and random interior rows
    rows = np.unique(np.concatenate([np.arange(0, 300), np.arange(a.m - 300, a.m),
                                     rng.integers(0, a.m, 1500)]))
    lens = a.row_lengths()[rows]
    sub_ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    take = np.concatenate([np.arange(a.ptr[r], a.ptr[r + 1]) for r in rows])
    c_ref, bound = oracle.spmm(len(rows), n, 0, sub_ptr, a.col[take], a.val[take], 1.0, 0.0, B.ravel(), n, True, None,
                               n, True)
    assert_within(np.ascontiguousarray(got[rows]), c_ref, bound, np.float32, what="C4 N=%d sample" % n)
    # all rows: column j of C equals the SpMV of A with column j of B (checked for two columns)
    for j in (0, n - 1):
        y_ref, bnd = oracle.spmv(False, a.m, a.n, 0, a.ptr, a.col, a.val, 1.0, 0.0, np.ascontiguousarray(B[:, j]), None)
        assert_within(np.ascontiguousarray(got[:, j]), y_ref, bnd, np.float32, what="C4 N=%d column %d" % (n, j))
