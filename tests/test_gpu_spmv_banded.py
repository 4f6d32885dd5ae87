"""GPU parity of the column-banded SpMV (mcsparseSpMV_preprocess, then mcsparseSpMV on the same buffer)
against the CPU oracle, within 8*u*(|alpha| * |A||x| + |beta*y|) as for every other SpMV family."""
import glob
import os

import numpy as np
import pytest

from mcsparse_amd import api
from mcsparse_amd import workloads as wl

from gpu_util import assert_within, dev

pytestmark = pytest.mark.gpu

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "csr_*.npz")))


@pytest.fixture()
def handle(handle):
    """These tests are of the copies themselves: preprocess keeps every copy it builds, also where the row kernels
    would be faster (small matrices)."""
    handle.set_spmv_preprocess_trial(False)
    return handle


def run_banded(torch, handle, oracle, a, alpha, beta, band_bytes=0, seed=1, expect_state=2, what="", calls=1,
               as_csc=False, reference=None, alg=api.SPMV_CSR_ALG2):
    """as_csc: the arrays are handed over as the CSC of the n x m transpose and applied with op T.
    reference: (x, y_ref, bound) of a product the caller has already worked out with the oracle, for
    beta == 0 (saves a second pass of the oracle over a large matrix).
    alg: MCSPARSE_SPMV_CSR_ALG2 asks for the reproducible banded copy (state 2); the default algorithm and
    MCSPARSE_SPMV_CSR_ALG1 get the copy in column order (state 3), whose sums need not repeat bit for bit."""
    rng = np.random.default_rng(seed)
    dt = a.val.dtype
    ct = api.maca_type(dt)
    x = rng.uniform(-1, 1, a.n).astype(dt) if reference is None else reference[0]
    y = rng.uniform(-1, 1, a.m).astype(dt)
    d_ptr, d_col, d_val, d_x, d_y = (dev(torch, v) for v in (a.ptr, a.col, a.val, x, y))
    if as_csc:
        mat = api.SpMat(a.n, a.m, a.nnz, d_ptr, d_col, d_val, base=a.base, fmt=api.FORMAT_CSC)
        op = api.OP_T
    else:
        mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val, base=a.base)
        op = api.OP_N
    if band_bytes:
        mat.set_band_bytes(band_bytes)
    vx, vy = api.DnVec(d_x), api.DnVec(d_y)
    st, size = api.spmv_preprocess_buffer_size(handle, op, alpha, mat, vx, beta, vy, ct, alg=alg)
    assert st == api.STATUS_SUCCESS
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    assert api.spmv_preprocess(handle, op, alpha, mat, vx, beta, vy, ct, buf, alg=alg) == api.STATUS_SUCCESS
    state, bands, rows = mat.spmv_preprocess_state()
    assert state == expect_state, (state, bands, rows)
    if reference is None:
        y_ref, bound = oracle.spmv(False, a.m, a.n, a.base, a.ptr, a.col, a.val, alpha, beta, x, y)
    else:
        assert beta == 0.0
        y_ref, bound = alpha * reference[1], abs(alpha) * reference[2]
    first = None
    for _ in range(calls):
        d_y.copy_(torch.from_numpy(y))
        assert api.spmv(handle, op, alpha, mat, vx, beta, vy, ct, buf, alg=alg) == api.STATUS_SUCCESS
        torch.cuda.synchronize()
        got = d_y.cpu().numpy()
        assert_within(got, y_ref, bound, dt, what=what or "banded spmv")
        if first is None:
            first = got
        elif state == 2:  # fixed summation order: the same bits every time
            assert np.array_equal(first.view(np.uint8), got.view(np.uint8))
    return state, bands, rows


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
@pytest.mark.parametrize("base", [0, 1])
def test_golden_fixtures_banded(torch_gpu, handle, path, base):
    """Integer-valued fixtures: every summation order is exact, so the result must equal the fixture's."""
    torch = torch_gpu
    with np.load(path) as z:
        g = {k: z[k] for k in z.files}
    for dt in (np.float32, np.float64):
        a = wl.Csr(int(g["m"]), int(g["n"]), g["ptr"], g["col"], g["val"].astype(dt)).with_base(base)
        ct = api.maca_type(dt)
        alpha, beta = float(g["alpha"]), float(g["beta"])
        d_ptr, d_col, d_val, d_x, d_y = (dev(torch, v) for v in (a.ptr, a.col, a.val, g["x"].astype(dt),
                                                                   g["y0"].astype(dt)))
        mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val, base=base)
        mat.set_band_bytes(64)  # 16 or 8 columns per band: even these small fixtures are cut into several
        vx, vy = api.DnVec(d_x), api.DnVec(d_y)
        st, size = api.spmv_preprocess_buffer_size(handle, api.OP_N, alpha, mat, vx, beta, vy, ct, alg=api.SPMV_CSR_ALG2)
        assert st == api.STATUS_SUCCESS
        buf = torch.empty(size, dtype=torch.uint8, device="cuda")
        assert api.spmv_preprocess(handle, api.OP_N, alpha, mat, vx, beta, vy, ct, buf, alg=api.SPMV_CSR_ALG2) == api.STATUS_SUCCESS
        assert api.spmv(handle, api.OP_N, alpha, mat, vx, beta, vy, ct, buf) == api.STATUS_SUCCESS
        torch.cuda.synchronize()
        assert np.array_equal(d_y.cpu().numpy().astype(np.float64), g["y_n"])


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("base", [0, 1])
@pytest.mark.parametrize("band_bytes", [1024, 8192, 1 << 16])
def test_ragged_rows_small_bands(torch_gpu, handle, oracle, dtype, base, band_bytes):
    # empty rows, rows that straddle bands, several bands per XCD and bands without entries in a chunk
    a = wl.random_ragged(5003, 30011, 23, dtype=dtype, seed=band_bytes % 97, base=base)
    state, bands, rows = run_banded(torch_gpu, handle, oracle, a, -0.75, 1.25, band_bytes=band_bytes, calls=2)
    assert bands >= 2
    run_banded(torch_gpu, handle, oracle, a, 2.0, 0.0, band_bytes=band_bytes)


@pytest.mark.parametrize("per_row", [1, 3, 16, 61])
def test_tiles_of_every_fill(torch_gpu, handle, oracle, per_row):
    # per_row steers the rows per tile (32 .. 1024) and whether tiles need more than one slab
    a = wl.uniform_rows(m=6000, n=50000, per_row=per_row, dtype=np.float64, config_id=20 + per_row)
    run_banded(torch_gpu, handle, oracle, a, 1.5, 0.5, band_bytes=1 << 15)
    b = wl.uniform_rows(m=3000, n=4000, per_row=min(per_row * 4, 200), dtype=np.float32, config_id=40 + per_row)
    run_banded(torch_gpu, handle, oracle, b, 1.0, 0.0, band_bytes=4096)


def test_csc_applied_transposed(torch_gpu, handle, oracle):
    # CSC with op T runs the row kernels on the arrays as they lie, so it can be banded like CSR op N
    a = wl.random_ragged(4001, 20011, 17, dtype=np.float32, seed=21, base=1)
    run_banded(torch_gpu, handle, oracle, a, 1.25, -0.5, band_bytes=4096, as_csc=True, calls=2)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("fmt", [api.FORMAT_CSR, api.FORMAT_CSC])
def test_transposing_directions_get_a_copy_of_the_transpose(torch_gpu, handle, oracle, dtype, fmt):
    """CSR with op T and CSC with op N: the preprocess call transposes once, the calls run the banded kernel."""
    torch = torch_gpu
    a = wl.random_ragged(6001, 20011, 13, dtype=dtype, seed=22, base=1)
    ct = api.maca_type(dtype)
    rng = np.random.default_rng(2)
    x = rng.uniform(-1, 1, a.m).astype(dtype)
    y0 = rng.uniform(-1, 1, a.n).astype(dtype)
    d_ptr, d_col, d_val, d_x = (dev(torch, v) for v in (a.ptr, a.col, a.val, x))
    d_y = dev(torch, y0)
    if fmt == api.FORMAT_CSR:  # the arrays are A (m x n): op T gives A^T x
        mat, op = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val, base=1), api.OP_T
    else:  # the same arrays read as the CSC of the n x m matrix A^T: op N gives A^T x
        mat, op = api.SpMat(a.n, a.m, a.nnz, d_ptr, d_col, d_val, base=1, fmt=api.FORMAT_CSC), api.OP_N
    mat.set_band_bytes(4096)
    vx, vy = api.DnVec(d_x), api.DnVec(d_y)
    st, size = api.spmv_preprocess_buffer_size(handle, op, 1.5, mat, vx, 0.5, vy, ct, alg=api.SPMV_CSR_ALG2)
    assert st == api.STATUS_SUCCESS
    st2, plain = api.spmv_buffer_size(handle, op, 1.5, mat, vx, 0.5, vy, ct)
    assert size > plain
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    assert api.spmv_preprocess(handle, op, 1.5, mat, vx, 0.5, vy, ct, buf, alg=api.SPMV_CSR_ALG2) == api.STATUS_SUCCESS
    assert mat.spmv_preprocess_state()[0] == 2
    y_ref, bound = oracle.spmv(True, a.m, a.n, 1, a.ptr, a.col, a.val, 1.5, 0.5, x, y0)
    for _ in range(2):
        d_y.copy_(torch.from_numpy(y0))
        assert api.spmv(handle, op, 1.5, mat, vx, 0.5, vy, ct, buf) == api.STATUS_SUCCESS
        torch.cuda.synchronize()
        assert_within(d_y.cpu().numpy(), y_ref, bound, dtype, what="transposing direction, banded")
    # the copy serves its own direction only: the other one runs the row kernels on the arrays as they lie
    other = api.OP_N if op == api.OP_T else api.OP_T
    x2 = rng.uniform(-1, 1, a.n).astype(dtype)
    d_x2 = dev(torch, x2)
    d_y2 = torch.zeros(a.m, dtype=d_x2.dtype, device="cuda")
    vx2, vy2 = api.DnVec(d_x2), api.DnVec(d_y2)
    assert api.spmv(handle, other, 1.0, mat, vx2, 0.0, vy2, ct, buf) == api.STATUS_SUCCESS
    torch.cuda.synchronize()
    y_ref2, bound2 = oracle.spmv(False, a.m, a.n, 1, a.ptr, a.col, a.val, 1.0, 0.0, x2, None)
    assert_within(d_y2.cpu().numpy(), y_ref2, bound2, dtype, what="the other direction")


def test_default_band_width_config2_reduced(torch_gpu, handle, oracle):
    a = wl.uniform_rows(m=1 << 16, n=1 << 20, per_row=16, dtype=np.float64)
    state, bands, rows = run_banded(torch_gpu, handle, oracle, a, 1.5, 0.5, calls=2)
    assert bands == 4


def test_declined_structures_fall_back(torch_gpu, handle, oracle):
    # x fits one band: nothing to do.  SpMV still answers.
    small = wl.random_ragged(2000, 3000, 9, dtype=np.float32, seed=3)
    run_banded(torch_gpu, handle, oracle, small, 1.0, 0.0, expect_state=0)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_long_rows_in_a_band(torch_gpu, handle, oracle, dtype):
    # power-law rows: runs of thousands of entries inside one band, over several slabs of a tile, next
    # to rows of one entry; default bands (2 bands of fp32, 4 of fp64) and narrow ones
    a = wl.power_law(m=1 << 14, n=1 << 20, max_len=20000, dtype=dtype)
    assert a.row_lengths().max() > 5000
    run_banded(torch_gpu, handle, oracle, a, 1.0, 0.0, calls=2)
    run_banded(torch_gpu, handle, oracle, a, -1.5, 0.5, band_bytes=1 << 16)
    b = wl.power_law(m=3000, n=3000, max_len=2500, dtype=dtype, config_id=8)
    run_banded(torch_gpu, handle, oracle, b, 1.0, 0.0, band_bytes=2048)
    # runs just around the length at which a wavefront takes over from a thread
    for per_row in (47, 48, 49, 50, 97):
        c = wl.uniform_rows(m=700, n=per_row + 3, per_row=per_row, dtype=dtype, config_id=60 + per_row)
        c = wl.Csr(c.m, 4 * c.n, c.ptr, c.col, c.val)  # columns in the first of several bands
        run_banded(torch_gpu, handle, oracle, c, 1.0, 0.0, band_bytes=128 * c.val.dtype.itemsize)


def test_copy_is_dropped_with_the_arrays(torch_gpu, handle, oracle):
    torch = torch_gpu
    a = wl.uniform_rows(m=4000, n=30000, per_row=8, dtype=np.float32, config_id=77)
    rng = np.random.default_rng(5)
    x = rng.uniform(-1, 1, a.n).astype(np.float32)
    d_ptr, d_col, d_val, d_x = (dev(torch, v) for v in (a.ptr, a.col, a.val, x))
    d_y = torch.zeros(a.m, dtype=torch.float32, device="cuda")
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val)
    mat.set_band_bytes(8192)
    vx, vy = api.DnVec(d_x), api.DnVec(d_y)
    st, size = api.spmv_preprocess_buffer_size(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, api.R_32F, alg=api.SPMV_CSR_ALG2)
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    assert api.spmv_preprocess(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, api.R_32F, buf, alg=api.SPMV_CSR_ALG2) == api.STATUS_SUCCESS
    assert mat.spmv_preprocess_state()[0] == 2
    # new values through the descriptor: the copy (which holds the old ones) must not be used
    new_val = rng.uniform(-1, 1, a.nnz).astype(np.float32)
    d_new = dev(torch, new_val)
    assert mat.lib.mcsparseSpMatSetValues(mat.ptr, d_new.data_ptr()) == 0
    assert mat.spmv_preprocess_state()[0] == 0
    assert api.spmv(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, api.R_32F, buf) == api.STATUS_SUCCESS
    torch.cuda.synchronize()
    y_ref, bound = oracle.spmv(False, a.m, a.n, 0, a.ptr, a.col, new_val, 1.0, 0.0, x, np.zeros(a.m, np.float32))
    assert_within(d_y.cpu().numpy(), y_ref, bound, np.float32, what="after SetValues")


def test_overwritten_buffer_stays_in_bounds(torch_gpu, handle, oracle):
    """A caller that scribbles over the buffer after preprocess gets wrong numbers, not a fault."""
    torch = torch_gpu
    a = wl.uniform_rows(m=4000, n=30000, per_row=8, dtype=np.float64, config_id=78)
    d_ptr, d_col, d_val = (dev(torch, v) for v in (a.ptr, a.col, a.val))
    d_x = torch.ones(a.n, dtype=torch.float64, device="cuda")
    d_y = torch.zeros(a.m, dtype=torch.float64, device="cuda")
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val)
    mat.set_band_bytes(1 << 14)
    vx, vy = api.DnVec(d_x), api.DnVec(d_y)
    st, size = api.spmv_preprocess_buffer_size(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, api.R_64F, alg=api.SPMV_CSR_ALG2)
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    assert api.spmv_preprocess(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, api.R_64F, buf, alg=api.SPMV_CSR_ALG2) == api.STATUS_SUCCESS
    buf.fill_(0xFF)
    assert api.spmv(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, api.R_64F, buf) == api.STATUS_SUCCESS
    torch.cuda.synchronize()
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1)
    buf.copy_(torch.randint(0, 256, (size,), dtype=torch.uint8, device="cuda", generator=gen))
    assert api.spmv(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, api.R_64F, buf) == api.STATUS_SUCCESS
    torch.cuda.synchronize()
