"""GPU parity of the transposing mcsparseSpMV without a preprocess call (CSR op T, CSC op N, COO op T).

With more than 2^14 and at most 2^22 columns and any algorithm but MCSPARSE_SPMV_CSR_ALG2 the call orders the
products value * x[row] by the top eight bits of their column only and forms the sums of each bucket of columns in
LDS, in the order the products arrive; with at most 2^14 columns and many nonzeros in each it orders nothing and
sums into copies of y in LDS; otherwise, and under ALG2, it sorts the products completely and adds them in row
order.  Integer-valued operands make every order of summation exact, so those cases are compared bit for
bit; the rest within 8*u*(|alpha| (|A|^T |x|)_i + |beta y_i|)."""
import numpy as np
import pytest

from mcsparse_amd import api
from mcsparse_amd import workloads as wl

from gpu_util import assert_within, dev

pytestmark = pytest.mark.gpu


def run(torch, handle, a, x, y, alpha, beta, fmt=api.FORMAT_CSR, index_type=api.INDEX_32I, alg=api.SPMV_ALG_DEFAULT,
        repeats=1):
    """alpha * A^T x + beta * y for the m x n matrix `a`, asked for in the way the format transposes: CSR and COO
    arrays with op T, the same arrays read as the CSC of the n x m transpose with op N."""
    itype = np.int64 if index_type == api.INDEX_64I else np.int32
    first = a.ptr if fmt != api.FORMAT_COO else np.repeat(np.arange(a.m) + a.base, a.row_lengths())
    d_first, d_col, d_val = dev(torch, first.astype(itype)), dev(torch, a.col.astype(itype)), dev(torch, a.val)
    shape = (a.n, a.m) if fmt == api.FORMAT_CSC else (a.m, a.n)
    op = api.OP_N if fmt == api.FORMAT_CSC else api.OP_T
    mat = api.SpMat(shape[0], shape[1], a.nnz, d_first, d_col, d_val, base=a.base, fmt=fmt, index_type=index_type)
    d_x, d_y = dev(torch, x), dev(torch, y)
    vx, vy = api.DnVec(d_x), api.DnVec(d_y)
    ct = api.maca_type(a.val.dtype)
    st, size = api.spmv_buffer_size(handle, op, alpha, mat, vx, beta, vy, ct)
    assert st == api.STATUS_SUCCESS
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    out = []
    for _ in range(repeats):
        d_y.copy_(torch.from_numpy(y))
        assert api.spmv(handle, op, alpha, mat, vx, beta, vy, ct, buf, alg=alg) == api.STATUS_SUCCESS
        torch.cuda.synchronize()
        out.append(d_y.cpu().numpy())
    return out if repeats > 1 else out[0]


def integer_valued(a, seed):
    rng = np.random.default_rng(seed)
    a.val[:] = rng.integers(-3, 4, a.nnz)
    x = rng.integers(-4, 5, a.m).astype(a.val.dtype)
    y = rng.integers(-8, 9, a.n).astype(a.val.dtype)
    return x, y


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("base", [0, 1])
@pytest.mark.parametrize("n", [16384, 16385, 100003, 1 << 20, 1 << 22, (1 << 22) + 1])
def test_exact_on_integers_across_the_key_range(torch_gpu, handle, dtype, base, n):
    # 16384 columns with few nonzeros each take the full sort, 16385 are the first bucketed shape, 2^22 the last one;
    # the index base does not count
    a = wl.random_ragged(3001, n, 40, dtype=dtype, seed=n % 97 + base, base=base)
    x, y = integer_valued(a, n)
    want = 2 * (a.to_scipy().T.astype(np.float64) @ x.astype(np.float64)) - 3 * y
    got = run(torch_gpu, handle, a, x, y, 2.0, -3.0)
    assert np.array_equal(got.astype(np.float64), want), "n=%d base=%d" % (n, base)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_within_the_bound_and_columns_without_entries(torch_gpu, handle, oracle, dtype):
    # 200 rows of 30 entries over 70001 columns: most columns have no entry and must still get beta * y
    a = wl.random_ragged(200, 70001, 30, dtype=dtype, seed=5, empty_fraction=0.5)
    rng = np.random.default_rng(6)
    x = rng.uniform(-1, 1, a.m).astype(dtype)
    y = rng.uniform(-1, 1, a.n).astype(dtype)
    for alpha, beta in ((1.0, 0.0), (-0.75, 1.25), (0.0, 2.0)):
        got = run(torch_gpu, handle, a, x, y, alpha, beta)
        y_ref, bound = oracle.spmv(True, a.m, a.n, a.base, a.ptr, a.col, a.val, alpha, beta, x, y)
        assert_within(got, y_ref, bound, dtype, what="alpha %g beta %g" % (alpha, beta))
    # beta = 0 never reads y: what was there does not matter, in any column
    got = run(torch_gpu, handle, a, x, np.full(a.n, np.nan, dtype), 1.0, 0.0)
    y_ref, bound = oracle.spmv(True, a.m, a.n, a.base, a.ptr, a.col, a.val, 1.0, 0.0, x, np.zeros(a.n, dtype))
    assert_within(got, y_ref, bound, dtype, what="y of NaN under beta 0")


def test_one_column_with_most_of_the_entries(torch_gpu, handle):
    # every row has an entry in column 40000: one LDS sum takes 50000 products, one bucket most of the matrix
    m, n = 50000, 300000
    rng = np.random.default_rng(11)
    others = np.sort(rng.integers(0, n - 1, (m, 3)), axis=1)
    others[others >= 40000] += 1  # keep column 40000 for the common entry
    col = np.sort(np.concatenate([others, np.full((m, 1), 40000)], axis=1), axis=1)
    keep = np.ones(col.shape, bool)
    keep[:, 1:] = col[:, 1:] != col[:, :-1]  # no duplicates inside a row
    lens = keep.sum(axis=1)
    a = wl.Csr(m, n, np.concatenate([[0], np.cumsum(lens)]), col[keep], np.zeros(int(lens.sum()), np.float64))
    x, y = integer_valued(a, 12)
    want = a.to_scipy().T @ x + y
    got = run(torch_gpu, handle, a, x, y, 1.0, 1.0)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("fmt", [api.FORMAT_CSR, api.FORMAT_CSC, api.FORMAT_COO])
@pytest.mark.parametrize("index_type", [api.INDEX_32I, api.INDEX_64I])
def test_every_format_that_transposes(torch_gpu, handle, fmt, index_type):
    a = wl.random_ragged(20011, 50021, 9, dtype=np.float32, seed=20 + fmt, base=1)
    x, y = integer_valued(a, 21)
    want = (a.to_scipy().T.astype(np.float64) @ x.astype(np.float64)) + 2 * y
    got = run(torch_gpu, handle, a, x, y, 1.0, 2.0, fmt=fmt, index_type=index_type)
    assert np.array_equal(got.astype(np.float64), want)


def test_alg2_repeats_its_bits_and_both_agree(torch_gpu, handle, oracle):
    a = wl.power_law(m=60000, n=90001, max_len=20000, dtype=np.float32)
    rng = np.random.default_rng(31)
    x = rng.uniform(-1, 1, a.m).astype(np.float32)
    y = rng.uniform(-1, 1, a.n).astype(np.float32)
    y_ref, bound = oracle.spmv(True, a.m, a.n, a.base, a.ptr, a.col, a.val, 1.5, 0.5, x, y)
    first, second = run(torch_gpu, handle, a, x, y, 1.5, 0.5, alg=api.SPMV_CSR_ALG2, repeats=2)
    assert np.array_equal(first, second)
    assert_within(first, y_ref, bound, np.float32, what="sorted products")
    for got in run(torch_gpu, handle, a, x, y, 1.5, 0.5, repeats=2):
        assert_within(got, y_ref, bound, np.float32, what="bucketed products")


# ---- few columns, many nonzeros in each: no sort at all, copies of y in LDS ----

@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n,base", [(256, 0), (1000, 1), (16383, 1), (16384, 0), (16384, 1), (255, 0)])
def test_few_columns_exact_on_integers(torch_gpu, handle, dtype, n, base):
    # 16384 columns are the most a copy of y in LDS holds, whatever the index base; 255 columns are too few and
    # take the full sort
    m = 340000
    a = wl.random_ragged(m, n, 8, dtype=dtype, seed=n % 89 + base, base=base)  # a fifth of the rows empty
    assert a.nnz >= 128 * n
    x, y = integer_valued(a, n + 1)
    want = 3 * (a.to_scipy().T.astype(np.float64) @ x.astype(np.float64)) - y
    got = run(torch_gpu, handle, a, x, y, 3.0, -1.0)
    assert np.array_equal(got.astype(np.float64), want), "n=%d base=%d" % (n, base)


@pytest.mark.parametrize("fmt", [api.FORMAT_CSR, api.FORMAT_CSC, api.FORMAT_COO])
@pytest.mark.parametrize("index_type", [api.INDEX_32I, api.INDEX_64I])
def test_few_columns_every_format_within_the_bound(torch_gpu, handle, oracle, fmt, index_type):
    a = wl.random_ragged(150001, 3001, 5, dtype=np.float32, seed=60 + fmt, base=1, empty_fraction=0.3)
    assert a.nnz >= 128 * a.n
    rng = np.random.default_rng(61)
    x = rng.uniform(-1, 1, a.m).astype(np.float32)
    y = rng.uniform(-1, 1, a.n).astype(np.float32)
    y_ref, bound = oracle.spmv(True, a.m, a.n, a.base, a.ptr, a.col, a.val, -1.5, 0.75, x, y)
    got = run(torch_gpu, handle, a, x, y, -1.5, 0.75, fmt=fmt, index_type=index_type)
    assert_within(got, y_ref, bound, np.float32, what="fmt %d index %d" % (fmt, index_type))
    # beta = 0 never reads y
    got = run(torch_gpu, handle, a, x, np.full(a.n, np.nan, np.float32), 2.0, 0.0, fmt=fmt, index_type=index_type)
    y_ref, bound = oracle.spmv(True, a.m, a.n, a.base, a.ptr, a.col, a.val, 2.0, 0.0, x, np.zeros(a.n, np.float32))
    assert_within(got, y_ref, bound, np.float32, what="NaN in y, fmt %d index %d" % (fmt, index_type))


def test_few_columns_alg2_repeats_its_bits(torch_gpu, handle, oracle):
    a = wl.random_ragged(200000, 2048, 6, dtype=np.float64, seed=70)
    rng = np.random.default_rng(71)
    x, y = rng.uniform(-1, 1, a.m), rng.uniform(-1, 1, a.n)
    y_ref, bound = oracle.spmv(True, a.m, a.n, a.base, a.ptr, a.col, a.val, 1.0, 1.0, x, y)
    first, second = run(torch_gpu, handle, a, x, y, 1.0, 1.0, alg=api.SPMV_CSR_ALG2, repeats=2)
    assert np.array_equal(first, second)
    assert_within(first, y_ref, bound, np.float64, what="sorted products")
    assert_within(run(torch_gpu, handle, a, x, y, 1.0, 1.0), y_ref, bound, np.float64, what="copies of y in LDS")


# ---- columns that crowd into a few buckets: a crowded bucket is dealt to several workgroups ----

@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("rows,per_row", [(300, 3), (40000, 5), (400000, 12)])
@pytest.mark.parametrize("shape", ["one_bucket", "third_in_one", "two_buckets", "last_bucket"])
def test_crowded_buckets_exact_on_integers(torch_gpu, handle, dtype, rows, per_row, shape):
    """2^22 columns are 256 buckets of 16384.  With 900 nonzeros nothing is split (no room for planes of partial
    sums), with 200 000 the parts are as many as the spare scratch holds planes, with 4.8 M the crowded bucket is
    dealt out in shares of a 256th of the nonzeros."""
    n = 1 << 22
    rng = np.random.default_rng(rows + len(shape))
    nnz = rows * per_row
    if shape == "one_bucket":
        col = rng.integers(5 * 16384, 6 * 16384, nnz)
    elif shape == "third_in_one":
        col = np.where(rng.random(nnz) < 0.33, rng.integers(0, 16384, nnz), rng.integers(0, n, nnz))
    elif shape == "two_buckets":
        col = np.where(rng.random(nnz) < 0.5, rng.integers(16384, 2 * 16384, nnz), rng.integers(200 * 16384, 201 * 16384, nnz))
    else:
        col = rng.integers(n - 16384, n, nnz)
    a = wl.Csr(rows, n, np.arange(rows + 1) * per_row, col, np.zeros(nnz, dtype))  # duplicates in a row are fine
    x, y = integer_valued(a, 5)
    want = np.zeros(n, np.float64)
    np.add.at(want, col, (a.val.astype(np.float64) * np.repeat(x.astype(np.float64), per_row)))
    want = 2 * want + y
    for base in (0, 1):
        got = run(torch_gpu, handle, a.with_base(base), x, y, 2.0, 1.0)
        assert np.array_equal(got.astype(np.float64), want), (shape, rows, base)


@pytest.mark.parametrize("preprocess", [False, True])
@pytest.mark.parametrize("op", [api.OP_N, api.OP_T])
def test_deterministic_handle_repeats_its_bits_with_the_default_algorithm(torch_gpu, oracle, op, preprocess):
    """mcsparseSetSpMVDeterministic: a caller that passes MCSPARSE_SPMV_ALG_DEFAULT, as a program written against the
    reference does, gets the same bits from every run (the paths of MCSPARSE_SPMV_CSR_ALG2), with and without a
    preprocess call, in both directions.  Long rows and many rows per column make differing orders show."""
    torch = torch_gpu
    handle = api.Handle(stream=torch.cuda.current_stream().cuda_stream)
    handle.set_spmv_deterministic(True)
    a = wl.power_law(m=1 << 16, n=1 << 18, max_len=30000, dtype=np.float32)
    rng = np.random.default_rng(17)
    xs, ys = (a.n, a.m) if op == api.OP_N else (a.m, a.n)
    x = rng.uniform(-1, 1, xs).astype(np.float32)
    y0 = rng.uniform(-1, 1, ys).astype(np.float32)
    d_ptr, d_col, d_val, d_x = dev(torch, a.ptr), dev(torch, a.col), dev(torch, a.val), dev(torch, x)
    d_y = dev(torch, y0)
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val)
    mat.set_band_bytes(1 << 16)
    vx, vy = api.DnVec(d_x), api.DnVec(d_y)
    if preprocess:
        st, size = api.spmv_preprocess_buffer_size(handle, op, 1.25, mat, vx, 0.5, vy, api.R_32F)
    else:
        st, size = api.spmv_buffer_size(handle, op, 1.25, mat, vx, 0.5, vy, api.R_32F)
    assert st == api.STATUS_SUCCESS
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    if preprocess:
        assert api.spmv_preprocess(handle, op, 1.25, mat, vx, 0.5, vy, api.R_32F, buf) == api.STATUS_SUCCESS
        assert mat.spmv_preprocess_state()[0] in (0, 2)  # never the copy in column order
    runs = []
    for _ in range(3):
        d_y.copy_(torch.from_numpy(y0))
        assert api.spmv(handle, op, 1.25, mat, vx, 0.5, vy, api.R_32F, buf) == api.STATUS_SUCCESS
        torch.cuda.synchronize()
        runs.append(d_y.cpu().numpy())
    assert np.array_equal(runs[0].view(np.uint32), runs[1].view(np.uint32))
    assert np.array_equal(runs[0].view(np.uint32), runs[2].view(np.uint32))
    ref, bound = oracle.spmv(op == api.OP_T, a.m, a.n, 0, a.ptr, a.col, a.val, 1.25, 0.5, x, y0)
    assert_within(runs[0], ref, bound, np.float32, what="deterministic handle")
    handle.destroy()
