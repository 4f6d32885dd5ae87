"""GPU parity of mcsparseSpMV (through the C ABI) against the CPU oracle.

Tolerance: |y - y_ref| <= 8*u*bound_i with u = 2^-24 (fp32) or 2^-53 (fp64) and
bound_i = |alpha| * sum_j |a_ij||x_j| + |beta*y_i|.  For alpha = 1, beta = 0 this is exactly the
8*u*(|A||x|)_i of the acceptance criterion; the alpha/beta terms are what the same rounding
analysis gives when the result is scaled and added to beta*y."""
import glob
import os

import numpy as np
import pytest

from mcsparse_amd import api
from mcsparse_amd import workloads as wl

from gpu_util import assert_within, run_spmv

pytestmark = pytest.mark.gpu

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "csr_*.npz")))


def check(torch, handle, oracle, csr, alpha, beta, op=api.OP_N, fmt=api.FORMAT_CSR, family=api.FAMILY_AUTO, lanes=0,
          seed=1, device_scalars=False, what=""):
    """Runs one SpMV and checks it; for FORMAT_CSC `csr` holds the CSC arrays of an n x m matrix."""
    rng = np.random.default_rng(seed)
    dt = csr.val.dtype
    # shape of the matrix the call sees, and whether the arrays must be applied transposed
    if fmt == api.FORMAT_CSR:
        t = op != api.OP_N
    else:
        t = op == api.OP_N
    xs, ys = (csr.m, csr.n) if t else (csr.n, csr.m)
    x = rng.uniform(-1, 1, xs).astype(dt)
    y = rng.uniform(-1, 1, ys).astype(dt)
    st, got, plan = run_spmv(torch, handle, csr, x, y, alpha, beta, op=op, fmt=fmt, family=family, lanes=lanes,
                             device_scalars=device_scalars)
    assert st == api.STATUS_SUCCESS, st
    y_ref, bound = oracle.spmv(t, csr.m, csr.n, csr.base, csr.ptr, csr.col, csr.val, alpha, beta, x, y)
    worst = assert_within(got, y_ref, bound, dt, what=what or "spmv")
    return worst, plan


def test_config1_laplacian(torch_gpu, handle, oracle):
    a = wl.laplacian_5pt(256, dtype=np.float32)
    assert (a.m, a.nnz) == (65536, 326656)
    worst, plan = check(torch_gpu, handle, oracle, a, 1.0, 0.0, what="C1")
    assert plan[0] == api.FAMILY_VECTOR
    # closed form: A * ones is 0 inside the grid, 1 on edges, 2 in corners -- exactly
    st, y, _ = run_spmv(torch_gpu, handle, a, np.ones(a.n, np.float32), np.zeros(a.m, np.float32), 1.0, 0.0)
    yy = y.reshape(256, 256)
    assert (yy[1:-1, 1:-1] == 0).all() and (yy[0, 1:-1] == 1).all() and yy[0, 0] == 2 and yy[-1, -1] == 2


@pytest.mark.parametrize("m", [1 << 14, 1 << 20])
def test_config2_uniform_fp64(torch_gpu, handle, oracle, m):
    a = wl.uniform_rows(m=m, per_row=16, dtype=np.float64)
    worst, plan = check(torch_gpu, handle, oracle, a, 1.5, 0.5, what="C2 m=%d" % m)
    assert plan == (api.FAMILY_VECTOR, 16)


@pytest.mark.parametrize("op", [api.OP_N, api.OP_T])
def test_config3_power_law_reduced(torch_gpu, handle, oracle, op):
    a = wl.power_law(m=1 << 16, max_len=30000, dtype=np.float32)
    assert a.row_lengths().max() > 5000
    worst, plan = check(torch_gpu, handle, oracle, a, 1.0, 0.0, op=op, what="C3 reduced op=%d" % op)
    if op == api.OP_N:
        assert plan[0] == api.FAMILY_MERGE


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("lanes", [1, 2, 4, 8, 16, 32, 64])
def test_vector_family_every_width(torch_gpu, handle, oracle, dtype, lanes):
    # ragged rows, 20 % empty, some longer than the lane group: exercises the strided loop
    a = wl.random_ragged(5003, 4099, 23, dtype=dtype, seed=lanes)
    check(torch_gpu, handle, oracle, a, -0.75, 1.25, family=api.FAMILY_VECTOR, lanes=lanes, what="vector L=%d" % lanes)
    check(torch_gpu, handle, oracle, a, 2.0, 0.0, family=api.FAMILY_VECTOR, lanes=lanes, what="vector beta0")


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("shape", [(1, 1, 1), (7, 5, 2), (5003, 4099, 23), (300, 100000, 3), (100000, 300, 0.4),
                                   (2048, 2048, 1), (40, 9000, 4000)])
def test_merge_family_shapes(torch_gpu, handle, oracle, dtype, shape):
    m, n, mean = shape
    a = wl.random_ragged(m, n, mean, dtype=dtype, seed=m % 97, empty_fraction=0.3 if m > 1 else 0.0)
    if a.nnz == 0:
        pytest.skip("empty draw")
    check(torch_gpu, handle, oracle, a, 1.0, 0.0, family=api.FAMILY_MERGE, what="merge %r" % (shape,))
    check(torch_gpu, handle, oracle, a, 0.5, -2.0, family=api.FAMILY_MERGE, what="merge beta %r" % (shape,))
    # lanes = 1: the tiles run in the order of their first column; same results
    check(torch_gpu, handle, oracle, a, 1.0, 0.0, family=api.FAMILY_MERGE, lanes=1, what="ordered merge %r" % (shape,))
    check(torch_gpu, handle, oracle, a, 0.5, -2.0, family=api.FAMILY_MERGE, lanes=1, what="ordered merge beta")


def test_merge_family_one_huge_row_and_many_empty(torch_gpu, handle, oracle):
    # 3 rows hold everything, thousands of empty rows around them: carries cross many tiles
    m, n = 20000, 300000
    lens = np.zeros(m, dtype=np.int64)
    lens[17], lens[9000], lens[m - 1] = 250000, 1, 70000
    ptr = np.concatenate([[0], np.cumsum(lens)])
    rng = np.random.default_rng(5)
    col = np.concatenate([np.sort(rng.choice(n, size=l, replace=False)) for l in lens if l])
    val = rng.uniform(-1, 1, int(ptr[-1])).astype(np.float32)
    a = wl.Csr(m, n, ptr, col, val)
    for fam, lanes in ((api.FAMILY_MERGE, 0), (api.FAMILY_MERGE, 1), (api.FAMILY_AUTO, 0)):
        worst, plan = check(torch_gpu, handle, oracle, a, 1.0, 0.0, family=fam, lanes=lanes, what="huge rows")
        check(torch_gpu, handle, oracle, a, 3.0, 0.25, family=fam, lanes=lanes, what="huge rows beta")
    assert plan == (api.FAMILY_MERGE, 0)  # x (1.2 MB) fits an L2: storage order


@pytest.mark.parametrize("base", [0, 1])
@pytest.mark.parametrize("op", [api.OP_N, api.OP_T])
@pytest.mark.parametrize("fmt", [api.FORMAT_CSR, api.FORMAT_CSC])
def test_base_op_format_matrix(torch_gpu, handle, oracle, base, op, fmt):
    a = wl.random_ragged(3001, 1777, 9, dtype=np.float64, seed=11).with_base(base)
    check(torch_gpu, handle, oracle, a, 1.5, 0.5, op=op, fmt=fmt, what="base=%d op=%d fmt=%d" % (base, op, fmt))


def test_device_pointer_mode(torch_gpu, handle, oracle):
    a = wl.random_ragged(2000, 2000, 12, dtype=np.float32, seed=2)
    check(torch_gpu, handle, oracle, a, 1.25, -0.5, device_scalars=True, what="device scalars")


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p) for p in GOLDEN])
def test_golden_fixtures_exact(torch_gpu, handle, path):
    # integer-valued data: every summation order gives the same bits
    with np.load(path) as z:
        g = {k: z[k] for k in z.files}
    for dt in (np.float32, np.float64):
        a = wl.Csr(int(g["m"]), int(g["n"]), g["ptr"], g["col"], g["val"].astype(dt))
        for fam in (api.FAMILY_VECTOR, api.FAMILY_MERGE):
            st, y, _ = run_spmv(torch_gpu, handle, a, g["x"].astype(dt), g["y0"].astype(dt), float(g["alpha"]),
                                float(g["beta"]), family=fam)
            assert st == 0 and np.array_equal(y.astype(np.float64), g["y_n"])
        st, y, _ = run_spmv(torch_gpu, handle, a, g["xt"].astype(dt), np.zeros(a.n, dt), float(g["alpha"]), 0.0,
                            op=api.OP_T)
        assert st == 0 and np.array_equal(y.astype(np.float64), g["y_t"])


def test_scalar_special_cases(torch_gpu, handle, oracle):
    a = wl.random_ragged(1500, 1500, 10, dtype=np.float32, seed=4)
    rng = np.random.default_rng(0)
    x = rng.uniform(-1, 1, a.n).astype(np.float32)
    y0 = rng.uniform(-1, 1, a.m).astype(np.float32)
    # alpha = 0: y = beta*y exactly
    st, y, _ = run_spmv(torch_gpu, handle, a, x, y0, 0.0, 2.0)
    assert st == 0 and np.array_equal(y, 2.0 * y0)
    # alpha = beta = 0: the reference returns without touching y (mcsp_spmv_gpu.cpp:235-237)
    st, y, _ = run_spmv(torch_gpu, handle, a, x, y0, 0.0, 0.0)
    assert st == 0 and np.array_equal(y, y0)
    # beta = 0 does not read y: NaNs there do not reach the result.  (The reference evaluates
    # beta*y regardless, csr_vector_device.hpp:75; not reading y is this library's choice.)
    for fam in (api.FAMILY_VECTOR, api.FAMILY_MERGE):
        st, y, _ = run_spmv(torch_gpu, handle, a, x, np.full(a.m, np.nan, np.float32), 1.0, 0.0, family=fam)
        y_ref, bound = oracle.spmv(False, a.m, a.n, 0, a.ptr, a.col, a.val, 1.0, 0.0, x, None)
        assert st == 0 and np.isfinite(y).all()
        assert_within(y, y_ref, bound, np.float32)


def test_unreferenced_infinite_x_stays_out(torch_gpu, handle, oracle):
    """x[0] = inf and x[last] = nan, columns no row but one names: only that row may see them.
    (Lanes past the end of a short row once multiplied 0 by x[0].)"""
    rng = np.random.default_rng(21)
    m, n = 3000, 4000
    rows = [np.sort(rng.choice(np.arange(1, n - 1), rng.integers(0, 40), replace=False)) for _ in range(m)]
    rows[7] = np.array([0, 5, n - 1])
    ptr = np.concatenate([[0], np.cumsum([len(c) for c in rows])]).astype(np.int32)
    col = np.concatenate(rows).astype(np.int32)
    for dt in (np.float32, np.float64):
        a = wl.Csr(m, n, ptr, col, rng.uniform(-1, 1, len(col)).astype(dt))
        x = rng.uniform(-1, 1, n).astype(dt)
        x[0], x[n - 1] = np.inf, np.nan
        for fam, lanes in ((api.FAMILY_VECTOR, 0), (api.FAMILY_VECTOR, 64), (api.FAMILY_VECTOR, 4), (api.FAMILY_MERGE, 0)):
            st, y, _ = run_spmv(torch_gpu, handle, a, x, np.zeros(m, dt), 1.0, 0.0, family=fam, lanes=lanes)
            assert st == 0
            assert np.isnan(y[7]) and np.isfinite(np.delete(y, 7)).all(), (dt, fam, lanes)
            xf = x.copy()
            xf[0] = xf[n - 1] = 0
            y_ref, bound = oracle.spmv(False, m, n, 0, ptr, col, a.val, 1.0, 0.0, xf, None)
            assert_within(np.delete(y, 7), np.delete(y_ref, 7), np.delete(bound, 7), dt)


def test_same_result_on_repeat_and_y_transpose_identity(torch_gpu, handle, oracle):
    # deterministic: two runs agree bit for bit, for both families; and y^T(Ax) = (A^T y)^T x
    a = wl.power_law(m=20000, max_len=9000, dtype=np.float64)
    rng = np.random.default_rng(3)
    x = rng.uniform(-1, 1, a.n)
    w = rng.uniform(-1, 1, a.m)
    zeros_m, zeros_n = np.zeros(a.m), np.zeros(a.n)
    for fam in (api.FAMILY_VECTOR, api.FAMILY_MERGE):
        _, y1, _ = run_spmv(torch_gpu, handle, a, x, zeros_m, 1.0, 0.0, family=fam)
        _, y2, _ = run_spmv(torch_gpu, handle, a, x, zeros_m, 1.0, 0.0, family=fam)
        assert np.array_equal(y1, y2)
    _, ax, _ = run_spmv(torch_gpu, handle, a, x, zeros_m, 1.0, 0.0)
    _, atw, _ = run_spmv(torch_gpu, handle, a, w, zeros_n, 1.0, 0.0, op=api.OP_T)
    lhs, rhs = np.dot(w.astype(np.longdouble), ax), np.dot(atw.astype(np.longdouble), x)
    scale = np.dot(np.abs(w), np.abs(a.to_scipy()) @ np.abs(x))
    assert abs(lhs - rhs) <= 64 * 2.0 ** -53 * scale


def test_a_few_long_rows_among_many_short_ones(torch_gpu, handle, oracle):
    """What a row-length-binned dispatch is for: rows of 16 with a handful of rows of 20000 among them.  The analysis
    sends the whole matrix to the merge-path family in storage order (the long rows hold a minority of the nonzeros);
    the result is held against the oracle, as is the vector family forced onto the same matrix."""
    a = wl.mixed_rows(m=1 << 16, per_row=16, long_rows=8, long_len=20000, dtype=np.float32)
    rng = np.random.default_rng(3)
    x = rng.uniform(-1, 1, a.n).astype(np.float32)
    y = rng.uniform(-1, 1, a.m).astype(np.float32)
    y_ref, bound = oracle.spmv(False, a.m, a.n, a.base, a.ptr, a.col, a.val, 1.0, 0.0, x, y)
    st, got, plan = run_spmv(torch_gpu, handle, a, x, y, 1.0, 0.0)
    assert st == api.STATUS_SUCCESS and plan == (api.FAMILY_MERGE, 0), plan
    assert_within(got, y_ref, bound, np.float32, what="mixed rows, analysed")
    st, got, _ = run_spmv(torch_gpu, handle, a, x, y, 1.0, 0.0, family=api.FAMILY_VECTOR)
    assert st == api.STATUS_SUCCESS
    assert_within(got, y_ref, bound, np.float32, what="mixed rows, vector family")
