"""GPU parity of the SpMV copy whose tiles are in column order (mcsparseSpMV_preprocess with any algorithm
but MCSPARSE_SPMV_CSR_ALG2): products meet in LDS in the order the wavefronts reach them, so results are
within the tolerance of every other family but not bitwise reproducible."""
import numpy as np
import pytest

from mcsparse_amd import api
from mcsparse_amd import workloads as wl

from gpu_util import assert_within, dev

pytestmark = pytest.mark.gpu


@pytest.fixture()
def handle(handle):
    """These tests are of the copies themselves: preprocess keeps every copy it builds, also where the row kernels
    would be faster (small matrices)."""
    handle.set_spmv_preprocess_trial(False)
    return handle


def run(torch, handle, oracle, a, alpha, beta, op=api.OP_N, fmt=api.FORMAT_CSR, band_bytes=0, seed=1, expect_state=3,
        calls=2, call_alg=api.SPMV_CSR_ALG1, what="column order"):
    """a: the matrix whose arrays are handed over (m x n CSR).  fmt CSC reads the same arrays as the CSC of
    the n x m transpose.  The product computed is A x for (CSR, N) and (CSC, T), A^T x otherwise."""
    rng = np.random.default_rng(seed)
    dt = a.val.dtype
    ct = api.maca_type(dt)
    transposed = (fmt == api.FORMAT_CSR) == (op == api.OP_T)
    x = rng.uniform(-1, 1, a.m if transposed else a.n).astype(dt)
    y = rng.uniform(-1, 1, a.n if transposed else a.m).astype(dt)
    d_ptr, d_col, d_val, d_x, d_y = (dev(torch, v) for v in (a.ptr, a.col, a.val, x, y))
    if fmt == api.FORMAT_CSR:
        mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val, base=a.base)
    else:
        mat = api.SpMat(a.n, a.m, a.nnz, d_ptr, d_col, d_val, base=a.base, fmt=api.FORMAT_CSC)
    if band_bytes:
        mat.set_band_bytes(band_bytes)
    vx, vy = api.DnVec(d_x), api.DnVec(d_y)
    st, size = api.spmv_preprocess_buffer_size(handle, op, alpha, mat, vx, beta, vy, ct, alg=api.SPMV_CSR_ALG1)
    assert st == api.STATUS_SUCCESS
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    assert api.spmv_preprocess(handle, op, alpha, mat, vx, beta, vy, ct, buf, alg=api.SPMV_CSR_ALG1) == api.STATUS_SUCCESS
    state, bands, rows = mat.spmv_preprocess_state()
    assert state == expect_state, (state, bands, rows)
    y_ref, bound = oracle.spmv(transposed, a.m, a.n, a.base, a.ptr, a.col, a.val, alpha, beta, x, y)
    for _ in range(calls):
        d_y.copy_(torch.from_numpy(y))
        assert api.spmv(handle, op, alpha, mat, vx, beta, vy, ct, buf, alg=call_alg) == api.STATUS_SUCCESS
        torch.cuda.synchronize()
        assert_within(d_y.cpu().numpy(), y_ref, bound, dt, what=what)
    return state, bands, rows, mat, buf


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_integer_valued_product_is_exact(torch_gpu, handle, oracle, dtype):
    """Small integers: every summation order is exact, so the result must equal the oracle's bit for bit."""
    torch = torch_gpu
    a = wl.random_ragged(70001, 30011, 9, dtype=dtype, seed=4)
    rng = np.random.default_rng(4)
    a = wl.Csr(a.m, a.n, a.ptr, a.col, rng.integers(-8, 9, a.nnz).astype(dtype), a.base)
    x = rng.integers(-8, 9, a.n).astype(dtype)
    y = rng.integers(-8, 9, a.m).astype(dtype)
    d_ptr, d_col, d_val, d_x, d_y = (dev(torch, v) for v in (a.ptr, a.col, a.val, x, y))
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val)
    mat.set_band_bytes(1 << 12)
    vx, vy = api.DnVec(d_x), api.DnVec(d_y)
    ct = api.maca_type(dtype)
    st, size = api.spmv_preprocess_buffer_size(handle, api.OP_N, 2.0, mat, vx, -1.0, vy, ct)
    assert st == api.STATUS_SUCCESS
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    assert api.spmv_preprocess(handle, api.OP_N, 2.0, mat, vx, -1.0, vy, ct, buf) == api.STATUS_SUCCESS
    assert mat.spmv_preprocess_state()[0] == 3
    assert api.spmv(handle, api.OP_N, 2.0, mat, vx, -1.0, vy, ct, buf) == api.STATUS_SUCCESS
    torch.cuda.synchronize()
    y_ref, _ = oracle.spmv(False, a.m, a.n, a.base, a.ptr, a.col, a.val, 2.0, -1.0, x, y)
    assert np.array_equal(d_y.cpu().numpy().astype(np.float64), np.asarray(y_ref, dtype=np.float64))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("base", [0, 1])
def test_ragged_rows_several_chunks_and_bands(torch_gpu, handle, oracle, dtype, base):
    # nine row chunks of 16384, empty rows, 30 or 59 planes of partial sums, tiles without entries
    a = wl.random_ragged(140003, 30011, 9, dtype=dtype, seed=5, base=base)
    state, bands, rows, _, _ = run(torch_gpu, handle, oracle, a, -0.75, 1.25, band_bytes=1 << 12)
    assert rows == 16384 and bands >= 30


def test_tiles_are_halved_until_every_compute_unit_has_one(torch_gpu, handle, oracle):
    # two planes of the default width: 16384-row tiles would give 74 units for 256 compute units
    a = wl.uniform_rows(m=600000, n=300000, per_row=5, dtype=np.float64, config_id=94)
    state, bands, rows, _, _ = run(torch_gpu, handle, oracle, a, 2.0, 0.0)
    assert (bands, rows) == (2, 4096)


@pytest.mark.parametrize("fmt,op", [(api.FORMAT_CSR, api.OP_T), (api.FORMAT_CSC, api.OP_N), (api.FORMAT_CSC, api.OP_T)])
def test_other_directions(torch_gpu, handle, oracle, fmt, op):
    a = wl.random_ragged(60001, 90011, 11, dtype=np.float64, seed=6, base=1)
    run(torch_gpu, handle, oracle, a, 1.5, 0.5, op=op, fmt=fmt, band_bytes=1 << 14)


def test_small_matrix_is_left_to_the_row_kernels(torch_gpu, handle, oracle):
    # fewer units of work than compute units: no copy in column order, and x fits one band: no banded copy
    a = wl.random_ragged(300, 200, 7, dtype=np.float32, seed=7)
    run(torch_gpu, handle, oracle, a, 1.0, 0.0, expect_state=0)
    b = wl.laplacian_5pt(256, dtype=np.float32)
    run(torch_gpu, handle, oracle, b, 1.0, 0.0, expect_state=0)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_long_rows(torch_gpu, handle, oracle, dtype):
    # thousands of products of one row meet in one accumulator
    a = wl.power_law(m=1 << 15, n=1 << 20, max_len=20000, dtype=dtype)
    run(torch_gpu, handle, oracle, a, 1.0, 0.0, band_bytes=1 << 17)
    run(torch_gpu, handle, oracle, a, -1.5, 0.5, op=api.OP_T, band_bytes=1 << 17)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("dense", [1, 3])
def test_rows_with_an_entry_in_every_column(torch_gpu, handle, oracle, dtype, dense):
    """A row that holds more than half of what a row chunk holds on average selects the kernel variant that sums
    the products of such a row in registers before they go to LDS; integer values make every order exact."""
    torch = torch_gpu
    m, n, per_row = 40000, 60000, 6
    rng = np.random.default_rng(50 + dense)
    base = wl.uniform_rows(m=m, n=n, per_row=per_row, dtype=dtype, config_id=95)
    lens = base.row_lengths().copy()
    full = rng.choice(m, dense, replace=False)
    lens[full] = n
    ptr = np.concatenate([[0], np.cumsum(lens)])
    col = np.empty(int(ptr[-1]), np.int64)
    for r in range(m):
        col[ptr[r]:ptr[r + 1]] = np.arange(n) if lens[r] == n else base.col[base.ptr[r]:base.ptr[r + 1]]
    a = wl.Csr(m, n, ptr, col, rng.integers(-3, 4, col.size).astype(dtype))
    x = rng.integers(-4, 5, n).astype(dtype)
    y = rng.integers(-8, 9, m).astype(dtype)
    d_ptr, d_col, d_val, d_x, d_y = (dev(torch, v) for v in (a.ptr, a.col, a.val, x, y))
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val)
    mat.set_band_bytes(1 << 14)
    vx, vy = api.DnVec(d_x), api.DnVec(d_y)
    ct = api.maca_type(dtype)
    st, size = api.spmv_preprocess_buffer_size(handle, api.OP_N, 2.0, mat, vx, -1.0, vy, ct)
    assert st == api.STATUS_SUCCESS
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    assert api.spmv_preprocess(handle, api.OP_N, 2.0, mat, vx, -1.0, vy, ct, buf) == api.STATUS_SUCCESS
    assert mat.spmv_preprocess_state()[0] == 3
    want = 2 * (a.to_scipy().astype(np.float64) @ x.astype(np.float64)) - y
    for _ in range(2):
        d_y.copy_(torch.from_numpy(y))
        assert api.spmv(handle, api.OP_N, 2.0, mat, vx, -1.0, vy, ct, buf) == api.STATUS_SUCCESS
        torch.cuda.synchronize()
        assert np.array_equal(d_y.cpu().numpy().astype(np.float64), want)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_tiles_around_whole_sets_of_entries(torch_gpu, handle, oracle, dtype):
    """The kernel takes a tile in sets of 1024 x 12 (fp32) or 1024 x 13 (fp64) entries, the loads of a set issued
    under the arithmetic of the one before; with fp32 values the entries lie in blocks of 256 that are stored lane by
    lane, a tile's last block with fewer lanes.  Tiles of 0 to 9 entries, around one block, and one less than,
    exactly and one more than one, two and three sets, each several times and with their first entry at varying
    alignments, with integer values so that any order of the sums is exact."""
    torch = torch_gpu
    rows_per_tile, groups, chunks = 16384, 32, 8
    keys = (1 << 12) // np.dtype(dtype).itemsize  # columns per group with 4 KiB bands
    per_set = 1024 * (12 if dtype == np.float32 else 13)
    sizes = [0, 1, per_set - 1, per_set, per_set + 1, 2 * per_set - 1, 2 * per_set, 2 * per_set + 1, 3 * per_set,
             3 * per_set + 1, 777, per_set // 2, 2, 3, 4, 5, 7, 9, 255, 256, 257, 259, 511, 513, per_set + 255,
             per_set + 258]
    rng = np.random.default_rng(77)
    rows, cols = [], []
    for t in range(groups * chunks):
        g, c = divmod(t, chunks)
        count = sizes[(t * 5 + g) % len(sizes)]
        rows.append(rng.integers(0, rows_per_tile, count) + c * rows_per_tile)
        cols.append(rng.integers(0, keys, count) + g * keys)
    rows, cols = np.concatenate(rows), np.concatenate(cols)
    order = np.lexsort((cols, rows))
    rows, cols = rows[order], cols[order]
    m, n = rows_per_tile * chunks, keys * groups
    ptr = np.concatenate([[0], np.cumsum(np.bincount(rows, minlength=m))])
    a = wl.Csr(m, n, ptr, cols, rng.integers(-3, 4, cols.size).astype(dtype))
    x = rng.integers(-4, 5, n).astype(dtype)
    y = rng.integers(-8, 9, m).astype(dtype)
    d_ptr, d_col, d_val, d_x, d_y = (dev(torch, v) for v in (a.ptr, a.col, a.val, x, y))
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val)
    mat.set_band_bytes(1 << 12)
    vx, vy = api.DnVec(d_x), api.DnVec(d_y)
    ct = api.maca_type(dtype)
    st, size = api.spmv_preprocess_buffer_size(handle, api.OP_N, 1.0, mat, vx, 1.0, vy, ct)
    assert st == api.STATUS_SUCCESS
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    assert api.spmv_preprocess(handle, api.OP_N, 1.0, mat, vx, 1.0, vy, ct, buf) == api.STATUS_SUCCESS
    assert mat.spmv_preprocess_state() == (3, groups, rows_per_tile)
    want = a.to_scipy().astype(np.float64) @ x.astype(np.float64) + y
    for _ in range(2):
        d_y.copy_(torch.from_numpy(y))
        assert api.spmv(handle, api.OP_N, 1.0, mat, vx, 1.0, vy, ct, buf) == api.STATUS_SUCCESS
        torch.cuda.synchronize()
        assert np.array_equal(d_y.cpu().numpy().astype(np.float64), want)


@pytest.mark.parametrize("alg", [api.SPMV_CSR_ALG1, api.SPMV_CSR_ALG2])
@pytest.mark.parametrize("m,offset", [(70000, 0), (70000, 1), (70001, 0), (70001, 1)])
def test_fp64_reduce_with_any_alignment_of_y(torch_gpu, handle, oracle, alg, m, offset):
    """The reduce over the planes takes two rows per thread with 16-byte accesses when the number of rows is even and
    y is 16-byte aligned, and one row per thread otherwise: both kernels, both copies, same result."""
    torch = torch_gpu
    a = wl.random_ragged(m, 50000, 6, dtype=np.float64, seed=12)
    rng = np.random.default_rng(12)
    x = rng.uniform(-1, 1, a.n)
    y = rng.uniform(-1, 1, a.m)
    d_ptr, d_col, d_val, d_x = (dev(torch, v) for v in (a.ptr, a.col, a.val, x))
    backing = torch.zeros(m + 2, dtype=torch.float64, device="cuda")
    d_y = backing[offset:offset + m]  # offset 1: 8 bytes past a 16-byte boundary
    assert (d_y.data_ptr() % 16 == 0) == (offset == 0)
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val)
    mat.set_band_bytes(1 << 14)
    vx, vy = api.DnVec(d_x), api.DnVec(d_y)
    ct = api.maca_type(np.float64)
    st, size = api.spmv_preprocess_buffer_size(handle, api.OP_N, -0.5, mat, vx, 2.0, vy, ct, alg=alg)
    assert st == api.STATUS_SUCCESS
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    assert api.spmv_preprocess(handle, api.OP_N, -0.5, mat, vx, 2.0, vy, ct, buf, alg=alg) == api.STATUS_SUCCESS
    assert mat.spmv_preprocess_state()[0] == (2 if alg == api.SPMV_CSR_ALG2 else 3)
    y_ref, bound = oracle.spmv(False, a.m, a.n, a.base, a.ptr, a.col, a.val, -0.5, 2.0, x, y)
    d_y.copy_(torch.from_numpy(y))
    assert api.spmv(handle, api.OP_N, -0.5, mat, vx, 2.0, vy, ct, buf, alg=alg) == api.STATUS_SUCCESS
    torch.cuda.synchronize()
    assert_within(d_y.cpu().numpy(), y_ref, bound, np.float64, what="reduce, m %d, y offset %d" % (m, offset))
    assert backing[offset + m:].abs().sum().item() == 0 and (offset == 0 or backing[0].item() == 0)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (-1.5, 0.75), (0.0, 2.0)])
def test_one_band_group_writes_y_itself(torch_gpu, handle, oracle, dtype, alpha, beta):
    """x inside one band group: no planes of partial sums and no reduce kernel; the SpMV kernel applies alpha and
    beta, must not read y under beta = 0 (NaN in it), and puts its work counters back itself: three calls."""
    torch = torch_gpu
    a = wl.random_ragged(600000, 100000, 5, dtype=dtype, seed=21)
    rng = np.random.default_rng(21)
    x = rng.uniform(-1, 1, a.n).astype(dtype)
    y = rng.uniform(-1, 1, a.m).astype(dtype)
    if beta == 0.0:
        y[::7] = np.nan
    d_ptr, d_col, d_val, d_x, d_y = (dev(torch, v) for v in (a.ptr, a.col, a.val, x, y))
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val)
    vx, vy = api.DnVec(d_x), api.DnVec(d_y)
    ct = api.maca_type(dtype)
    st, size = api.spmv_preprocess_buffer_size(handle, api.OP_N, alpha, mat, vx, beta, vy, ct)
    assert st == api.STATUS_SUCCESS
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    assert api.spmv_preprocess(handle, api.OP_N, alpha, mat, vx, beta, vy, ct, buf) == api.STATUS_SUCCESS
    state, bands, rows = mat.spmv_preprocess_state()
    assert (state, bands) == (3, 1), (state, bands, rows)
    y_ref, bound = oracle.spmv(False, a.m, a.n, a.base, a.ptr, a.col, a.val, alpha, beta, x,
                               np.where(np.isnan(y), 0, y).astype(dtype))
    for _ in range(3):
        d_y.copy_(torch.from_numpy(y))
        assert api.spmv(handle, api.OP_N, alpha, mat, vx, beta, vy, ct, buf) == api.STATUS_SUCCESS
        torch.cuda.synchronize()
        assert_within(d_y.cpu().numpy(), y_ref, bound, dtype, what="one band group")


def test_alg2_does_not_use_the_copy(torch_gpu, handle, oracle):
    """MCSPARSE_SPMV_CSR_ALG2 promises the same bits on every run: the call runs the row kernels."""
    a = wl.uniform_rows(m=20000, n=300000, per_row=8, dtype=np.float64, config_id=91)
    run(torch_gpu, handle, oracle, a, 1.0, 0.0, call_alg=api.SPMV_CSR_ALG2, band_bytes=1 << 16)


def test_default_algorithm_gets_the_copy_in_column_order(torch_gpu, handle, oracle):
    torch = torch_gpu
    a = wl.uniform_rows(m=30000, n=400000, per_row=8, dtype=np.float64, config_id=93)
    rng = np.random.default_rng(9)
    x = rng.uniform(-1, 1, a.n)
    d_ptr, d_col, d_val, d_x = (dev(torch, v) for v in (a.ptr, a.col, a.val, x))
    d_y = torch.zeros(a.m, dtype=torch.float64, device="cuda")
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val)
    mat.set_band_bytes(1 << 16)
    vx, vy = api.DnVec(d_x), api.DnVec(d_y)
    sizes = {}
    for alg in (api.SPMV_ALG_DEFAULT, api.SPMV_CSR_ALG1, api.SPMV_CSR_ALG2):
        st, sizes[alg] = api.spmv_preprocess_buffer_size(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, api.R_64F, alg=alg)
        assert st == api.STATUS_SUCCESS
    assert sizes[api.SPMV_ALG_DEFAULT] == sizes[api.SPMV_CSR_ALG1] > sizes[api.SPMV_CSR_ALG2]
    buf = torch.empty(sizes[api.SPMV_ALG_DEFAULT], dtype=torch.uint8, device="cuda")
    y_ref, bound = oracle.spmv(False, a.m, a.n, 0, a.ptr, a.col, a.val, 1.0, 0.0, x, None)
    for alg, state in ((api.SPMV_ALG_DEFAULT, 3), (api.SPMV_CSR_ALG2, 2), (api.SPMV_CSR_ALG1, 3)):
        assert api.spmv_preprocess(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, api.R_64F, buf, alg=alg) == api.STATUS_SUCCESS
        assert mat.spmv_preprocess_state()[0] == state
        d_y.zero_()
        assert api.spmv(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, api.R_64F, buf) == api.STATUS_SUCCESS
        torch.cuda.synchronize()
        assert_within(d_y.cpu().numpy(), y_ref, bound, np.float64, what="alg %d" % alg)


def test_wide_matrix_falls_back_to_the_banded_copy(torch_gpu, handle, oracle):
    # more than 64 bands of this width: the reproducible banded copy is built instead
    a = wl.random_ragged(5003, 30011, 23, dtype=np.float64, seed=3)
    run(torch_gpu, handle, oracle, a, 1.0, 0.5, band_bytes=1024, expect_state=2)


def test_overwritten_copy_stays_in_bounds(torch_gpu, handle, oracle):
    torch = torch_gpu
    a = wl.uniform_rows(m=40000, n=100000, per_row=8, dtype=np.float32, config_id=92)
    run(torch, handle, oracle, a, 1.0, 0.0, band_bytes=1 << 14)
    x = torch.rand(a.n, dtype=torch.float32, device="cuda")
    y = torch.zeros(a.m, dtype=torch.float32, device="cuda")
    d_ptr, d_col, d_val = (dev(torch, v) for v in (a.ptr, a.col, a.val))
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val)
    mat.set_band_bytes(1 << 14)
    vx, vy = api.DnVec(x), api.DnVec(y)
    st, size = api.spmv_preprocess_buffer_size(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, api.R_32F, alg=api.SPMV_CSR_ALG1)
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    assert api.spmv_preprocess(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, api.R_32F, buf, alg=api.SPMV_CSR_ALG1) == 0
    assert mat.spmv_preprocess_state()[0] == 3
    for fill in (0xFF, 0x00, None):
        if fill is None:
            buf.copy_(torch.randint(0, 256, (size,), dtype=torch.uint8, device="cuda"))
        else:
            buf.fill_(fill)
        assert api.spmv(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, api.R_32F, buf, alg=api.SPMV_CSR_ALG1) == 0
        torch.cuda.synchronize()


@pytest.mark.parametrize("seed", [31, 32, 33, 34])
def test_random_shapes(torch_gpu, handle, oracle, seed):
    """Shapes drawn around the cuts the layout makes: tile heights 2048..16384, one to 64 planes, band groups of
    one and two bands, all four (format, op) pairs; whatever copy the library decides on, the product is right."""
    r = np.random.default_rng(seed)
    seen = set()
    for case in range(6):
        dtype = [np.float32, np.float64][int(r.integers(0, 2))]
        m = int(r.choice([9000, 20000, 33000, 70000, 150000]))
        n = int(r.choice([5000, 40000, 262144, 300001]))
        mean = int(r.choice([3, 9, 20]))
        band_bytes = int(r.choice([1 << 12, 1 << 14, 1 << 16, 1 << 20, 0]))
        a = wl.random_ragged(m, n, mean, dtype=dtype, seed=seed * 100 + case, base=int(r.integers(0, 2)))
        fmt, op = [(api.FORMAT_CSR, api.OP_N), (api.FORMAT_CSR, api.OP_T), (api.FORMAT_CSC, api.OP_N),
                   (api.FORMAT_CSC, api.OP_T)][int(r.integers(0, 4))]
        alpha, beta = [(1.0, 0.0), (-1.5, 0.75), (2.0, 1.0)][int(r.integers(0, 3))]
        what = "seed %d case %d: %d x %d, mean %d, %s, band %d, fmt %d op %d" % (
            seed, case, m, n, mean, np.dtype(dtype).name, band_bytes, fmt, op)
        rng = np.random.default_rng(seed)
        transposed = (fmt == api.FORMAT_CSR) == (op == api.OP_T)
        x = rng.uniform(-1, 1, a.m if transposed else a.n).astype(dtype)
        y = rng.uniform(-1, 1, a.n if transposed else a.m).astype(dtype)
        d_ptr, d_col, d_val, d_x, d_y = (dev(torch_gpu, v) for v in (a.ptr, a.col, a.val, x, y))
        if fmt == api.FORMAT_CSR:
            mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val, base=a.base)
        else:
            mat = api.SpMat(a.n, a.m, a.nnz, d_ptr, d_col, d_val, base=a.base, fmt=api.FORMAT_CSC)
        if band_bytes:
            mat.set_band_bytes(band_bytes)
        vx, vy = api.DnVec(d_x), api.DnVec(d_y)
        ct = api.maca_type(dtype)
        st, size = api.spmv_preprocess_buffer_size(handle, op, alpha, mat, vx, beta, vy, ct)
        assert st == api.STATUS_SUCCESS, what
        buf = torch_gpu.empty(size, dtype=torch_gpu.uint8, device="cuda")
        assert api.spmv_preprocess(handle, op, alpha, mat, vx, beta, vy, ct, buf) == api.STATUS_SUCCESS, what
        seen.add(mat.spmv_preprocess_state()[0])
        assert api.spmv(handle, op, alpha, mat, vx, beta, vy, ct, buf) == api.STATUS_SUCCESS, what
        torch_gpu.cuda.synchronize()
        y_ref, bound = oracle.spmv(transposed, a.m, a.n, a.base, a.ptr, a.col, a.val, alpha, beta, x, y)
        assert_within(d_y.cpu().numpy(), y_ref, bound, dtype, what=what)
    assert 3 in seen, seen


@pytest.mark.parametrize("alg,state", [(api.SPMV_ALG_DEFAULT, 3), (api.SPMV_CSR_ALG2, 2)])
@pytest.mark.parametrize("fmt", [api.FORMAT_CSR, api.FORMAT_CSC, api.FORMAT_COO])
@pytest.mark.parametrize("index_type", [api.INDEX_32I, api.INDEX_64I])
def test_copies_of_coo_and_64_bit_inputs(torch_gpu, handle, oracle, alg, state, fmt, index_type):
    """mcsparseSpMV_preprocess narrows 64-bit indices and turns COO rows into offsets once; the calls then read
    nothing but the copy.  Both directions of every format."""
    torch = torch_gpu
    a = wl.random_ragged(60001, 50021, 8, dtype=np.float64, seed=40 + fmt, base=1)
    if fmt == api.FORMAT_CSR and index_type == api.INDEX_32I:
        pytest.skip("covered by the tests above")
    itype = np.int64 if index_type == api.INDEX_64I else np.int32
    first = a.ptr if fmt != api.FORMAT_COO else np.repeat(np.arange(a.m) + a.base, np.diff(a.ptr.astype(np.int64)))
    d_first, d_col, d_val = dev(torch, first.astype(itype)), dev(torch, a.col.astype(itype)), dev(torch, a.val)
    shape = (a.n, a.m) if fmt == api.FORMAT_CSC else (a.m, a.n)
    rng = np.random.default_rng(8)
    for op in (api.OP_N, api.OP_T):
        # the arrays are A's CSR (or COO); read as CSC they are the n x m transpose
        transposed = (fmt != api.FORMAT_CSC) == (op == api.OP_T)
        x = rng.uniform(-1, 1, a.m if transposed else a.n)
        y = rng.uniform(-1, 1, a.n if transposed else a.m)
        d_x, d_y = dev(torch, x), dev(torch, y)
        mat = api.SpMat(shape[0], shape[1], a.nnz, d_first, d_col, d_val, base=1, fmt=fmt, index_type=index_type)
        mat.set_band_bytes(1 << 14)
        vx, vy = api.DnVec(d_x), api.DnVec(d_y)
        st, size = api.spmv_preprocess_buffer_size(handle, op, 1.5, mat, vx, -0.5, vy, api.R_64F, alg=alg)
        assert st == api.STATUS_SUCCESS
        buf = torch.empty(size, dtype=torch.uint8, device="cuda")
        assert api.spmv_preprocess(handle, op, 1.5, mat, vx, -0.5, vy, api.R_64F, buf, alg=alg) == api.STATUS_SUCCESS
        assert mat.spmv_preprocess_state()[0] == state
        y_ref, bound = oracle.spmv(transposed, a.m, a.n, 1, a.ptr, a.col, a.val, 1.5, -0.5, x, y)
        for _ in range(2):
            d_y.copy_(torch.from_numpy(y))
            assert api.spmv(handle, op, 1.5, mat, vx, -0.5, vy, api.R_64F, buf, alg=alg) == api.STATUS_SUCCESS
            torch.cuda.synchronize()
            assert_within(d_y.cpu().numpy(), y_ref, bound, np.float64, what="fmt %d index %d op %d" % (fmt, index_type, op))


@pytest.mark.parametrize("alg", [api.SPMV_ALG_DEFAULT, api.SPMV_CSR_ALG2])
def test_a_call_in_the_other_direction_on_the_same_buffer_ends_the_copy(torch_gpu, handle, oracle, alg):
    """The copy of op N sits behind the scratch of op N only.  A^T x on the same buffer (sized for both) writes its
    far larger scratch over the copy: the descriptor must drop the copy, so that the next A x reads the caller's
    arrays again instead of the overwritten region."""
    torch = torch_gpu
    a = wl.random_ragged(90001, 70003, 8, dtype=np.float64, seed=31)
    rng = np.random.default_rng(31)
    x_n, y_n = rng.uniform(-1, 1, a.n), rng.uniform(-1, 1, a.m)
    x_t, y_t = rng.uniform(-1, 1, a.m), rng.uniform(-1, 1, a.n)
    d_ptr, d_col, d_val = (dev(torch, v) for v in (a.ptr, a.col, a.val))
    d_xn, d_yn, d_xt, d_yt = (dev(torch, v) for v in (x_n, y_n, x_t, y_t))
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val)
    mat.set_band_bytes(1 << 14)
    vxn, vyn, vxt, vyt = api.DnVec(d_xn), api.DnVec(d_yn), api.DnVec(d_xt), api.DnVec(d_yt)
    ct = api.R_64F
    st, size_pre = api.spmv_preprocess_buffer_size(handle, api.OP_N, 1.5, mat, vxn, 0.5, vyn, ct, alg=alg)
    assert st == api.STATUS_SUCCESS
    st, size_t = api.spmv_buffer_size(handle, api.OP_T, 1.5, mat, vxt, 0.5, vyt, ct)
    assert st == api.STATUS_SUCCESS
    buf = torch.empty(max(size_pre, size_t), dtype=torch.uint8, device="cuda")
    assert api.spmv_preprocess(handle, api.OP_N, 1.5, mat, vxn, 0.5, vyn, ct, buf, alg=alg) == api.STATUS_SUCCESS
    assert mat.spmv_preprocess_state()[0] in (2, 3)
    ref_n, bound_n = oracle.spmv(False, a.m, a.n, 0, a.ptr, a.col, a.val, 1.5, 0.5, x_n, y_n)
    ref_t, bound_t = oracle.spmv(True, a.m, a.n, 0, a.ptr, a.col, a.val, 1.5, 0.5, x_t, y_t)
    assert api.spmv(handle, api.OP_N, 1.5, mat, vxn, 0.5, vyn, ct, buf, alg=alg) == api.STATUS_SUCCESS
    torch.cuda.synchronize()
    assert_within(d_yn.cpu().numpy(), ref_n, bound_n, np.float64, what="A x from the copy")
    assert api.spmv(handle, api.OP_T, 1.5, mat, vxt, 0.5, vyt, ct, buf, alg=alg) == api.STATUS_SUCCESS
    torch.cuda.synchronize()
    assert_within(d_yt.cpu().numpy(), ref_t, bound_t, np.float64, what="A^T x on the copy's buffer")
    assert mat.spmv_preprocess_state()[0] == 0  # the copy is gone
    d_yn.copy_(torch.from_numpy(y_n))
    assert api.spmv(handle, api.OP_N, 1.5, mat, vxn, 0.5, vyn, ct, buf, alg=alg) == api.STATUS_SUCCESS
    torch.cuda.synchronize()
    assert_within(d_yn.cpu().numpy(), ref_n, bound_n, np.float64, what="A x after the copy was written over")
