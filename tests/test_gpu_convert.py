"""GPU parity of the index conversions (through the C ABI): bit-exact against the CPU oracle."""
import glob
import os

import numpy as np
import pytest

from mcsparse_amd import api
from mcsparse_amd import workloads as wl

from gpu_util import dev

pytestmark = pytest.mark.gpu

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "csr_*.npz")))


def gpu_csr2coo(torch, handle, a):
    d_ptr = dev(torch, a.ptr)
    d_out = torch.full((max(a.nnz, 1),), -7, dtype=torch.int32, device="cuda")
    st = api.xcsr2coo(handle, d_ptr, a.nnz, a.m, d_out, a.base)
    torch.cuda.synchronize()
    return st, d_out.cpu().numpy()[:a.nnz]


def gpu_coo2csr(torch, handle, coo, nnz, m, base):
    d_coo = dev(torch, coo)
    d_out = torch.full((m + 1,), -7, dtype=torch.int32, device="cuda")
    st = api.xcoo2csr(handle, d_coo, nnz, m, d_out, base)
    torch.cuda.synchronize()
    return st, d_out.cpu().numpy()


def gpu_csr2csc(torch, handle, a, action=api.ACTION_NUMERIC):
    d_ptr, d_col, d_val = dev(torch, a.ptr), dev(torch, a.col), dev(torch, a.val)
    vt = api.maca_type(a.val.dtype)
    o_val = torch.zeros_like(d_val)
    o_ptr = torch.full((a.n + 1,), -7, dtype=torch.int32, device="cuda")
    o_row = torch.full((max(a.nnz, 1),), -7, dtype=torch.int32, device="cuda")
    st, size = api.csr2csc_buffer_size(handle, a.m, a.n, a.nnz, d_val, d_ptr, d_col, o_val, o_ptr, o_row, vt, action,
                                       a.base)
    assert st == 0 and size >= 128
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    st = api.csr2csc(handle, a.m, a.n, a.nnz, d_val, d_ptr, d_col, o_val, o_ptr, o_row, vt, action, a.base, buf)
    torch.cuda.synchronize()
    return st, o_ptr.cpu().numpy(), o_row.cpu().numpy()[:a.nnz], o_val.cpu().numpy()


def check_csr2csc(torch, handle, oracle, a, what):
    st, cp, ri, cv = gpu_csr2csc(torch, handle, a)
    assert st == 0
    w_cp, w_ri, w_cv = oracle.csr2csc(a.m, a.n, a.base, a.ptr, a.col, a.val, method="counting")
    assert np.array_equal(cp.view(np.uint32), w_cp), what + ": col_ptr"
    assert np.array_equal(ri.view(np.uint32), w_ri), what + ": row_ind"
    assert np.array_equal(cv.view(np.uint8), w_cv.view(np.uint8)), what + ": values"
    return cp, ri, cv


def one_per_row(m, seed):
    """A permutation matrix: every 4096-nonzero tile of the sort spans exactly 4096 rows."""
    rng = np.random.default_rng(seed)
    return wl.Csr(m, m, np.arange(m + 1), rng.permutation(m), rng.uniform(-1, 1, m).astype(np.float32))


def empty_stretches(seed):
    """Long runs of empty rows before, between and after a few long rows."""
    rng = np.random.default_rng(seed)
    lens = np.zeros(30000, np.int64)
    lens[[7000, 7001, 19000, 24999]] = [5000, 1, 9000, 300]
    ptr = np.concatenate([[0], np.cumsum(lens)])
    col = np.concatenate([np.sort(rng.choice(12000, n, replace=False)) for n in lens if n])
    return wl.Csr(30000, 12000, ptr, col, rng.uniform(-1, 1, int(ptr[-1])))


def absent_columns(seed):
    """Columns used only in the middle of a wide range: long stretches of equal offsets on both sides."""
    rng = np.random.default_rng(seed)
    m, n = 2000, 3_000_000
    lens = rng.integers(0, 21, m)
    ptr = np.concatenate([[0], np.cumsum(lens)])
    col = np.concatenate([np.sort(rng.choice(np.arange(500_000, 2_500_000, 7), k, replace=False)) for k in lens])
    return wl.Csr(m, n, ptr, col, rng.uniform(-1, 1, int(ptr[-1])).astype(np.float32))


CASES = {
    "ragged_f32": lambda: wl.random_ragged(5003, 4099, 23, dtype=np.float32, seed=1),
    "ragged_f64_base1": lambda: wl.random_ragged(5003, 4099, 23, dtype=np.float64, seed=2).with_base(1),
    "wide": lambda: wl.random_ragged(300, 100000, 3, dtype=np.float32, seed=3),
    "tall_sparse": lambda: wl.random_ragged(100000, 300, 0.4, dtype=np.float32, seed=4),
    "one_by_one": lambda: wl.random_ragged(1, 1, 1, dtype=np.float64, seed=5, empty_fraction=0.0),
    "power_law": lambda: wl.power_law(m=1 << 16, max_len=30000, dtype=np.float32),
    "power_law_base1_f64": lambda: wl.power_law(m=1 << 14, max_len=9000, dtype=np.float64).with_base(1),
    "n_pow2": lambda: wl.random_ragged(4096, 65536, 20, dtype=np.float32, seed=6),
    "n_pow2_minus1_base1": lambda: wl.random_ragged(4096, 65535, 20, dtype=np.float32, seed=7).with_base(1),
    "n_small": lambda: wl.random_ragged(70000, 3, 2, dtype=np.float32, seed=8),
    "stencil": lambda: wl.stencil_27pt(20, dtype=np.float32),
    "one_per_row": lambda: one_per_row(10000, 10),
    "empty_stretches": lambda: empty_stretches(11),
    "empty_stretches_base1": lambda: empty_stretches(12).with_base(1),
    "absent_columns": lambda: absent_columns(13),
    "absent_columns_base1": lambda: absent_columns(14).with_base(1),
}


@pytest.mark.parametrize("name", list(CASES))
def test_conversions_bit_exact(torch_gpu, handle, oracle, name):
    a = CASES[name]()
    if a.nnz == 0:
        pytest.skip("empty draw")
    st, coo = gpu_csr2coo(torch_gpu, handle, a)
    assert st == 0
    want = oracle.csr2coo(a.m, a.base, a.ptr, a.nnz)
    assert np.array_equal(coo.view(np.uint32), want), name + ": csr2coo"
    st, back = gpu_coo2csr(torch_gpu, handle, coo, a.nnz, a.m, a.base)
    assert st == 0 and np.array_equal(back, a.ptr), name + ": coo2csr"
    assert np.array_equal(back.view(np.uint32), oracle.coo2csr(a.nnz, a.m, a.base, want))
    cp, ri, cv = check_csr2csc(torch_gpu, handle, oracle, a, name)
    assert int(cp[0]) == a.base and int(cp[-1]) - a.base == a.nnz
    # transposing the result gives the matrix back (sorted, duplicate-free input)
    t = wl.Csr(a.n, a.m, cp, ri, cv, a.base)
    st, cp2, ri2, cv2 = gpu_csr2csc(torch_gpu, handle, t)
    assert st == 0 and np.array_equal(cp2, a.ptr) and np.array_equal(ri2, a.col)
    assert np.array_equal(cv2.view(np.uint8), a.val.view(np.uint8))


def test_csr2csc_symbolic_and_literal_oracle(torch_gpu, handle, oracle):
    a = wl.random_ragged(3000, 5000, 11, dtype=np.float32, seed=5)
    st, cp, ri, cv = gpu_csr2csc(torch_gpu, handle, a, action=api.ACTION_SYMBOLIC)
    w_cp, w_ri, _ = oracle.csr2csc(a.m, a.n, 0, a.ptr, a.col, a.val, method="radix2")
    assert st == 0 and np.array_equal(cp.view(np.uint32), w_cp) and np.array_equal(ri.view(np.uint32), w_ri)
    assert not cv.any()  # values are not written for SYMBOLIC


def test_csr2csc_keeps_input_order_of_duplicates(torch_gpu, handle, oracle):
    # unsorted columns with repeated (row, col) pairs: a stable sort keeps them in input order
    rng = np.random.default_rng(9)
    m, n, nnz = 500, 37, 20000
    lens = rng.multinomial(nnz, np.ones(m) / m)
    ptr = np.concatenate([[0], np.cumsum(lens)])
    col = rng.integers(0, n, nnz)
    val = np.arange(nnz, dtype=np.float64)
    a = wl.Csr(m, n, ptr, col, val)
    cp, ri, cv = check_csr2csc(torch_gpu, handle, oracle, a, "duplicates")
    assert np.array_equal(cv, val[np.argsort(col, kind="stable")])


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p) for p in GOLDEN])
def test_golden_conversions(torch_gpu, handle, path):
    with np.load(path) as z:
        g = {k: z[k] for k in z.files}
    for base in (0, 1):
        a = wl.Csr(int(g["m"]), int(g["n"]), g["ptr"] + base, g["col"] + base, g["val"], base)
        st, cp, ri, cv = gpu_csr2csc(torch_gpu, handle, a)
        assert st == 0 and np.array_equal(cp, g["csc_ptr"] + base) and np.array_equal(ri, g["csc_row"] + base)
        assert np.array_equal(cv, g["csc_val"])
        st, coo = gpu_csr2coo(torch_gpu, handle, a)
        assert st == 0 and np.array_equal(coo, g["coo_row"] + base)


def test_empty_inputs_leave_outputs_untouched(torch_gpu, handle):
    # nnz == 0 returns before any work in the reference (mcsp_coo2csr.cpp:14-16, mcsp_csr2csc.cpp:56-58)
    a = wl.Csr(5, 4, np.zeros(6, np.int32), np.zeros(0, np.int32), np.zeros(0, np.float32))
    st, cp, ri, cv = gpu_csr2csc(torch_gpu, handle, a)
    assert st == 0 and (cp == -7).all()
    st, back = gpu_coo2csr(torch_gpu, handle, np.zeros(1, np.int32), 0, 5, 0)
    assert st == 0 and (back == -7).all()


@pytest.mark.parametrize("name", ["ragged_f32", "power_law", "tall_sparse", "one_by_one"])
def test_row_bins_bit_exact(torch_gpu, handle, oracle, name):
    a = CASES[name]()
    d_ptr = dev(torch_gpu, a.ptr)
    d_bins = torch_gpu.full((a.m,), 255, dtype=torch_gpu.uint8, device="cuda")
    d_hist = torch_gpu.full((34,), 12345, dtype=torch_gpu.int32, device="cuda")
    assert api.csr_row_bins(handle, a.m, d_ptr, a.base, d_bins, d_hist) == 0
    torch_gpu.cuda.synchronize()
    bins, hist = oracle.row_bins(a.m, a.ptr)
    assert np.array_equal(d_bins.cpu().numpy(), bins)
    assert np.array_equal(d_hist.cpu().numpy().view(np.uint32), hist)


@pytest.mark.parametrize("shift", [1, 3])
def test_unaligned_input_arrays(torch_gpu, handle, oracle, shift):
    """Index and value arrays that start 4 bytes past a 16-byte boundary (a sub-array of a larger
    allocation): the kernels may not assume 128-bit alignment of the caller's arrays."""
    torch = torch_gpu
    a = wl.random_ragged(9001, 7001, 11, dtype=np.float32, seed=31)
    big_col = torch.zeros(a.nnz + 8, dtype=torch.int32, device="cuda")
    big_val = torch.zeros(a.nnz + 8, dtype=torch.float32, device="cuda")
    big_ptr = torch.zeros(a.m + 9, dtype=torch.int32, device="cuda")
    d_col, d_val, d_ptr = big_col[shift:shift + a.nnz], big_val[shift:shift + a.nnz], big_ptr[shift:shift + a.m + 1]
    d_col.copy_(torch.from_numpy(a.col))
    d_val.copy_(torch.from_numpy(a.val))
    d_ptr.copy_(torch.from_numpy(a.ptr))
    assert d_col.data_ptr() % 16 != 0
    o_val = torch.zeros(a.nnz + 8, dtype=torch.float32, device="cuda")[shift:shift + a.nnz]
    o_ptr = torch.zeros(a.n + 9, dtype=torch.int32, device="cuda")[shift:shift + a.n + 1]
    o_row = torch.zeros(a.nnz + 8, dtype=torch.int32, device="cuda")[shift:shift + a.nnz]
    st, size = api.csr2csc_buffer_size(handle, a.m, a.n, a.nnz, d_val, d_ptr, d_col, o_val, o_ptr, o_row, api.R_32F,
                                       api.ACTION_NUMERIC, 0)
    assert st == 0
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    assert api.csr2csc(handle, a.m, a.n, a.nnz, d_val, d_ptr, d_col, o_val, o_ptr, o_row, api.R_32F,
                       api.ACTION_NUMERIC, 0, buf) == 0
    torch.cuda.synchronize()
    w_cp, w_ri, w_cv = oracle.csr2csc(a.m, a.n, 0, a.ptr, a.col, a.val, method="counting")
    assert np.array_equal(o_ptr.cpu().numpy().view(np.uint32), w_cp)
    assert np.array_equal(o_row.cpu().numpy().view(np.uint32), w_ri)
    assert np.array_equal(o_val.cpu().numpy(), w_cv)
    # the transposing SpMV sorts the same way, reading the caller's arrays in its first pass
    rng = np.random.default_rng(2)
    x = rng.uniform(-1, 1, a.m).astype(np.float32)
    d_x = torch.from_numpy(x).cuda()
    d_y = torch.zeros(a.n, dtype=torch.float32, device="cuda")
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val)
    vx, vy = api.DnVec(d_x), api.DnVec(d_y)
    st, size = api.spmv_buffer_size(handle, api.OP_T, 1.0, mat, vx, 0.0, vy, api.R_32F)
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    assert api.spmv(handle, api.OP_T, 1.0, mat, vx, 0.0, vy, api.R_32F, buf) == 0
    torch.cuda.synchronize()
    y_ref, bound = oracle.spmv(True, a.m, a.n, 0, a.ptr, a.col, a.val, 1.0, 0.0, x, None)
    err = np.abs(d_y.cpu().numpy().astype(np.longdouble) - y_ref)
    assert (err <= 8 * 2.0 ** -24 * bound).all()
    # coo2csr on an unaligned, mostly empty structure: long stretches of empty rows
    rows = np.sort(rng.integers(0, 50, 300)).astype(np.int32)
    d_rows = torch.zeros(308, dtype=torch.int32, device="cuda")[shift:shift + 300]
    d_rows.copy_(torch.from_numpy(rows))
    m_big = 1 << 20
    d_out = torch.full((m_big + 1,), -7, dtype=torch.int32, device="cuda")
    assert api.xcoo2csr(handle, d_rows, 300, m_big, d_out, 0) == 0
    torch.cuda.synchronize()
    assert np.array_equal(d_out.cpu().numpy().view(np.uint32), oracle.coo2csr(300, m_big, 0, rows))


@pytest.mark.parametrize("nnz", [4095, 4096, 4097, 8 * 4096 - 1, 8 * 4096, 8 * 4096 + 1, 3 * 8 * 4096 + 5])
@pytest.mark.parametrize("shape", ["ones", "even", "empty_head", "empty_tail", "one_long_row", "every_other_empty"])
def test_csr2coo_around_the_tile_and_group_sizes(torch_gpu, handle, oracle, nnz, shape):
    """csr2coo cuts the nonzeros into tiles of 4096 and walks 8 tiles per workgroup; the rows of a tile come from a
    map of the 4096 places a row can begin at (rows of one nonzero fill it), from the staged offsets when a row is
    empty, and from row_ptr itself when more than 4096 rows begin in a tile."""
    rng = np.random.default_rng(nnz)
    if shape == "ones":
        lens = np.ones(nnz, np.int64)
    elif shape == "even":
        m = nnz // 3
        lens = np.full(m, nnz // m, np.int64)
        lens[: nnz - lens.sum()] += 1
    elif shape == "empty_head":   # every row begins at the first nonzero, the nonzeros come last
        lens = np.zeros(nnz // 2, np.int64)
        lens[-3:] = [nnz - 2, 1, 1]
    elif shape == "empty_tail":
        lens = np.zeros(nnz // 2, np.int64)
        lens[:2] = [1, nnz - 1]
    elif shape == "one_long_row":
        lens = np.zeros(nnz // 2, np.int64)
        lens[int(rng.integers(0, lens.size))] = nnz
    else:                         # two rows begin at every nonzero: 8192 in a tile
        lens = np.zeros(2 * nnz, np.int64)
        lens[1::2] = 1
    m = lens.size
    assert lens.sum() == nnz
    ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    for base in (0, 1):
        a = wl.Csr(m, nnz + 1, ptr + base, np.zeros(nnz, np.int32) + base, np.zeros(nnz, np.float32), base)
        st, coo = gpu_csr2coo(torch_gpu, handle, a)
        assert st == 0
        assert np.array_equal(coo.view(np.uint32), oracle.csr2coo(m, base, a.ptr, nnz)), (nnz, shape, base)
    # an output array that is not 16-byte aligned is written one element at a time
    d_ptr = dev(torch_gpu, ptr)
    d_out = torch_gpu.full((nnz + 3,), -7, dtype=torch_gpu.int32, device="cuda")
    assert api.xcsr2coo(handle, d_ptr, nnz, m, d_out[1:nnz + 1], 0) == 0
    torch_gpu.cuda.synchronize()
    got = d_out.cpu().numpy()
    assert got[0] == -7 and (got[nnz + 1:] == -7).all()
    assert np.array_equal(got[1:nnz + 1].view(np.uint32), oracle.csr2coo(m, 0, ptr, nnz)), (nnz, shape, "unaligned")


@pytest.mark.parametrize("base", [0, 1])
@pytest.mark.parametrize("n", [256, 257, 65536, 65537, 1 << 24])
def test_csr2csc_where_the_column_count_fills_whole_digits(torch_gpu, handle, oracle, n, base):
    """The passes of the sort are counted from the columns without their index base: a one-based matrix whose last
    column is 2^8, 2^16 or 2^24 sorts in as many passes as the zero-based one, and in the same order."""
    a = wl.random_ragged(3000, n, 12, dtype=np.float32, seed=n % 101 + base, base=base)
    # the first and the last column are there, so the smallest and the largest key are
    a.col[0] = base
    a.col[-1] = n - 1 + base
    check_csr2csc(torch_gpu, handle, oracle, a, "n %d base %d" % (n, base))


@pytest.mark.parametrize("m", [8191, 8192, 8193, 12289, 1 << 20, 3000001])
@pytest.mark.parametrize("shape", ["few", "clump", "both_ends", "one_row", "gaps_8192", "gaps_8193", "none_after_half"])
def test_coo2csr_long_stretches_of_empty_rows(torch_gpu, handle, oracle, m, shape):
    """Stretches of more than 8192 equal offsets (rows without entries) are left to a second kernel, a workgroup per
    4096 offsets; shorter ones are filled where they are found."""
    rng = np.random.default_rng(m % 1000 + len(shape))
    if shape == "few":
        rows = rng.integers(0, m, 7)
    elif shape == "clump":
        rows = rng.integers(m // 2, min(m, m // 2 + 40), 5000)
    elif shape == "both_ends":
        rows = np.concatenate([rng.integers(0, 10, 100), rng.integers(m - 10, m, 100)])
    elif shape == "one_row":
        rows = np.full(3000, m // 3)
    elif shape == "gaps_8192":
        rows = np.arange(0, m, 8192)   # stretches of exactly 8192 offsets: filled in place
    elif shape == "gaps_8193":
        rows = np.arange(0, m, 8193)   # one more: left to the second kernel
    else:
        rows = rng.integers(0, m // 2, 20000)
    rows = np.sort(rows).astype(np.int32)
    for base in (0, 1):
        st, ptr = gpu_coo2csr(torch_gpu, handle, rows + base, rows.size, m, base)
        assert st == 0
        assert np.array_equal(ptr.view(np.uint32), oracle.coo2csr(rows.size, m, base, rows + base)), (m, shape, base)
