"""GPU parity of mcsparseSpMM (through the C ABI) against the CPU oracle; tolerance as for SpMV:
|C - C_ref| <= 8*u*(|alpha| * (|A||B|)_ij + |beta*C_ij|)."""
import numpy as np
import pytest

from mcsparse_amd import api
from mcsparse_amd import workloads as wl

from gpu_util import assert_within, dev

pytestmark = pytest.mark.gpu


def run_spmm(torch, handle, a, B, C0, alpha, beta, op_b=api.OP_N, b_order=api.ORDER_ROW, c_order=api.ORDER_ROW,
             pad_b=0, pad_c=0, preprocess=False, expect_schedule=None, prepare_for_row_major_c=False, seen=None):
    """B is the k x n operand op(B); it is stored as the call's (op_b, b_order) pair requires.
    prepare_for_row_major_c: mcsparseSpMM_preprocess is given a row-major C of the same shape, whatever the call's is
    (a schedule belongs to the structure of A; which kind is built depends on the operands of the preprocess call)."""
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
        mC_pre = mC
        if prepare_for_row_major_c:
            d_C_pre = torch.zeros((a.m, n), dtype=d_C.dtype, device="cuda")
            mC_pre = api.DnMat(a.m, n, n, d_C_pre, order=api.ORDER_ROW)
        assert api.spmm_preprocess(handle, api.OP_N, op_b, alpha, mat, mB, beta, mC_pre, ct, buf) == 0
        if expect_schedule is not None:
            wanted = expect_schedule if isinstance(expect_schedule, tuple) else (expect_schedule,)
            assert mat.spmm_schedule()[0] in wanted, mat.spmm_schedule()
        if seen is not None:
            seen.add(mat.spmm_schedule()[0])
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
    # state 2: merged column lists; state 3: diagonal blocks, for operands of more than 64 bytes per row
    for c_order in (api.ORDER_ROW, api.ORDER_COL):
        check(torch_gpu, handle, oracle, a, n, 1.0, 0.0, preprocess=True, expect_schedule=(2, 3), c_order=c_order)
        check(torch_gpu, handle, oracle, a, n, -1.5, 0.75, preprocess=True, expect_schedule=(2, 3), c_order=c_order,
              pad_b=4, pad_c=8)


def test_preprocessed_stencil_in_xcd_stretches(torch_gpu, handle, oracle):
    """A stencil large enough for the row-group kernel to hand every XCD stretches of several
    workgroups (the column span of a 48^3 stencil is 4,706 rows), with a last round that is only
    partly filled."""
    a = wl.stencil_27pt(48, dtype=np.float32)
    # lines of 48 points, a whole number of strips of four rows: state 4, blocks over groups of strips a line apart
    for n in (64, 40):
        check(torch_gpu, handle, oracle, a, n, 1.0, 0.0, preprocess=True, expect_schedule=4)
    # for a column-major C the groups of eight rows are built, unless the call prepared for a row-major one
    check(torch_gpu, handle, oracle, a, 64, 0.5, -1.0, preprocess=True, expect_schedule=3, c_order=api.ORDER_COL)
    check(torch_gpu, handle, oracle, a, 64, 0.5, -1.0, preprocess=True, expect_schedule=4, c_order=api.ORDER_COL,
          prepare_for_row_major_c=True)
    # lines of 46 points: no stride the strips could use, blocks over groups of eight consecutive rows (state 3)
    a = wl.stencil_27pt(46, dtype=np.float32)
    check(torch_gpu, handle, oracle, a, 64, 1.0, 0.0, preprocess=True, expect_schedule=3)
    check(torch_gpu, handle, oracle, a, 64, 0.5, -1.0, preprocess=True, expect_schedule=3, c_order=api.ORDER_COL)
    check(torch_gpu, handle, oracle, a, 16, 1.0, 0.0, preprocess=True, expect_schedule=2)  # too narrow for blocks


def test_preprocessed_ragged_rows_with_overlap(torch_gpu, handle, oracle):
    """Rows of different lengths, empty rows, unsorted columns inside rows, a group too long to merge."""
    rng = np.random.default_rng(12)
    m, k = 501, 3000
    rows = []
    for r in range(m):
        if r % 7 == 3:
            cols = np.zeros(0, np.int64)
        elif r in (100, 101, 102):
            # 2700 nonzeros in their group: not merged (each row short of the 1024 above which rows are cut into
            # pieces and preprocess builds no schedule at all)
            cols = rng.choice(k, 900, replace=False)
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


@pytest.mark.parametrize("grid,n", [(10, 64), (40, 64), (40, 128), (41, 64), (41, 128), (10, 16)])
def test_overwritten_schedule_stays_in_bounds(torch_gpu, handle, grid, n):
    """The reference's preprocess is a no-op, so a caller written against it may reuse the scratch
    buffer between preprocess and SpMM.  The schedule is then garbage: the product may be wrong, but
    every access stays inside the arrays (the call returns and the device stays healthy)."""
    torch = torch_gpu
    a = wl.stencil_27pt(grid, dtype=np.float32)
    d_ptr, d_col, d_val = dev(torch, a.ptr), dev(torch, a.col), dev(torch, a.val)
    d_B = torch.ones((a.n, n), dtype=torch.float32, device="cuda")
    d_C = torch.zeros((a.m, n), dtype=torch.float32, device="cuda")
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val)
    mB, mC = api.DnMat(a.n, n, n, d_B), api.DnMat(a.m, n, n, d_C)
    st, size = api.spmm_buffer_size(handle, api.OP_N, api.OP_N, 1.0, mat, mB, 0.0, mC, api.R_32F)
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    assert api.spmm_preprocess(handle, api.OP_N, api.OP_N, 1.0, mat, mB, 0.0, mC, api.R_32F, buf) == 0
    assert mat.spmm_schedule()[0] == (4 if grid == 40 else 3 if grid == 41 else 2), mat.spmm_schedule()
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


# ---- diagonal blocks (mcsparseSpMM_preprocess on matrices whose neighbouring rows hold the same diagonals) ----

def read_blocks(torch, buf, m):
    """The block schedule as it lies in the buffer: offsets per group of 8 rows, then (c, shape) pairs."""
    def align(x):
        return (x + 127) // 128 * 128
    raw = buf.cpu().numpy()
    groups = (m + 7) // 8
    ptr = raw[:4 * (groups + 1)].view(np.uint32)
    at = align(4 * ((m + 3) // 4 + 1)) + 128  # behind the offsets of the 4-row groups and the counters
    words = raw[at:at + 8 * int(ptr[groups])].view(np.uint32).reshape(-1, 2)
    return ptr, words


def columns_from_blocks(ptr, words, m):
    """Expands the blocks into every row's column sequence (zero-based): shape bits 0-2 = number of diagonals n, and
    for p < n bits 8+8p.. = first row, 12+8p.. = end row of diagonal p; row r holds it in column c + r + p."""
    rows = [[] for _ in range(m)]
    for g in range(len(ptr) - 1):
        for c, shape in words[ptr[g]:ptr[g + 1]]:
            c, shape = int(np.int32(c)), int(shape)
            n = shape & 7
            assert 1 <= n <= 3
            for p in range(n):
                lo, hi = (shape >> (8 + 8 * p)) & 15, (shape >> (12 + 8 * p)) & 15
                assert 0 <= lo < hi <= 8
            for r in range(8):
                for p in range(n):
                    lo, hi = (shape >> (8 + 8 * p)) & 15, (shape >> (12 + 8 * p)) & 15
                    if lo <= r < hi:
                        rows[8 * g + r].append(c + r + p)
    return rows


def read_strip_blocks(torch, buf, m):
    """The strip schedule as it lies in the buffer: the stride among the counters, offsets per group, 16-byte blocks."""
    def align(x):
        return (x + 127) // 128 * 128
    raw = buf.cpu().numpy()
    counters_at = align(4 * ((m + 3) // 4 + 1))
    stride = int(raw[counters_at + 24:counters_at + 28].view(np.uint32)[0])
    groups = (m + 4 * stride - 1) // (4 * stride) * (stride // 4)
    ptr = raw[:4 * (groups + 1)].view(np.uint32)
    at = counters_at + 128
    words = raw[at:at + 16 * int(ptr[groups])].view(np.uint32).reshape(-1, 4)
    return stride, ptr, words


def columns_from_strip_blocks(stride, ptr, words, m):
    """Expands the blocks of the groups of strips into every row's column sequence (zero-based).  Group g of the
    stretch t of 4 * stride rows holds the rows t * 4 * stride + q * stride + 4 * g + i (strip q, row i); bit
    3 * (4 * q + i) + p of a block's 48 bits says that this row holds column c + i + p."""
    rows = [[] for _ in range(m)]
    per_stretch = stride // 4
    for g in range(len(ptr) - 1):
        g0 = g // per_stretch * 4 * stride + g % per_stretch * 4
        for c, shape, lo, hi in words[ptr[g]:ptr[g + 1]]:
            c, shape, held = int(np.int32(c)), int(shape), int(lo) | (int(hi) << 32)
            n, j_first, j_last = shape & 15, (shape >> 4) & 15, (shape >> 8) & 15
            assert 1 <= n <= 3 and held != 0 and held >> 48 == 0
            needed = set()
            for r in range(16):
                for p in range(3):
                    if (held >> (3 * r + p)) & 1:
                        assert p < n
                        row = g0 + (r // 4) * stride + r % 4
                        assert row < m
                        rows[row].append(c + r % 4 + p)
                        needed.add(r % 4 + p)
            assert j_first == min(needed) and j_last == max(needed)
    return rows


@pytest.mark.parametrize("shape", ["stencil", "stencil41", "banded", "unsorted", "banded69", "unsorted69"])
def test_blocks_cover_every_nonzero_once_and_in_storage_order(torch_gpu, handle, shape):
    """Structural outputs are bit-exact: the blocks of a group, expanded, are the rows' column indices as stored."""
    torch = torch_gpu
    rng = np.random.default_rng(3)
    if shape == "stencil":
        a = wl.stencil_27pt(40, dtype=np.float32).with_base(1)   # lines of 40 points: groups of strips a line apart
    elif shape == "stencil41":
        a = wl.stencil_27pt(41, dtype=np.float32).with_base(1)   # no usable stride: groups of eight consecutive rows
    else:
        m = 4099
        offsets = np.array([-70, -69, -68, -2, -1, 0, 1, 2, 3, 64, 65, 66, 67, 68, 69])  # runs of 3, 6 (cut at 4) and 6
        if shape.endswith("69"):
            offsets[:3] -= 1   # the runs begin 69 and 66 apart: no distance the strips could use, groups of eight rows
        rows = []
        for r in range(m):
            c = r + offsets
            c = c[(c >= 0) & (c < m)]
            if r % 97 == 5:
                c = c[::2]                      # a row with holes breaks the blocks around it
            if r % 211 == 7:
                c = np.zeros(0, np.int64)       # an empty row
            if shape.startswith("unsorted") and r % 120 == 0:
                c = rng.permutation(c)          # consumed in storage order: single nonzeros around intact blocks
            rows.append(c)
        ptr = np.concatenate([[0], np.cumsum([len(c) for c in rows])]).astype(np.int32)
        a = wl.Csr(m, m, ptr, np.concatenate(rows).astype(np.int32), rng.uniform(-1, 1, int(ptr[-1])).astype(np.float32))
    n = 64
    d_ptr, d_col, d_val = dev(torch, a.ptr), dev(torch, a.col), dev(torch, a.val)
    d_B = torch.ones((a.n, n), dtype=torch.float32, device="cuda")
    d_C = torch.zeros((a.m, n), dtype=torch.float32, device="cuda")
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val, base=a.base)
    mB, mC = api.DnMat(a.n, n, n, d_B), api.DnMat(a.m, n, n, d_C)
    st, size = api.spmm_buffer_size(handle, api.OP_N, api.OP_N, 1.0, mat, mB, 0.0, mC, api.R_32F)
    buf = torch.zeros(size, dtype=torch.uint8, device="cuda")
    assert api.spmm_preprocess(handle, api.OP_N, api.OP_N, 1.0, mat, mB, 0.0, mC, api.R_32F, buf) == 0
    state, blocks = mat.spmm_schedule()
    # the stencils' kind follows from the length of their lines; the banded matrices get whichever loads fewer rows
    assert state == {"stencil": 4, "stencil41": 3, "banded69": 3, "unsorted69": 3}.get(shape, state) and state in (3, 4), (state, blocks)
    torch.cuda.synchronize()
    if state == 4:
        stride, ptr, words = read_strip_blocks(torch, buf, a.m)
        assert stride == (40 if shape == "stencil" else 68)
        got = columns_from_strip_blocks(stride, ptr, words, a.m)
    else:
        ptr, words = read_blocks(torch, buf, a.m)
        got = columns_from_blocks(ptr, words, a.m)
    assert int(ptr[-1]) == blocks and (np.diff(ptr.astype(np.int64)) >= 0).all()
    for r in range(a.m):
        want = (a.col[a.ptr[r] - a.base:a.ptr[r + 1] - a.base].astype(np.int64) - a.base).tolist()
        assert got[r] == want, (r, got[r], want)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n", [20, 36, 64, 72, 128, 256, 264])
def test_blocks_banded_matrix_with_broken_rows(torch_gpu, handle, oracle, dtype, n):
    """Diagonal runs of one to six, rows with holes, empty rows, unsorted rows, a group too long to cover, a row
    count that leaves the last group short; every width of lane group; both layouts of C."""
    rng = np.random.default_rng(5)
    m, k = 3003, 3100
    offsets = np.array([-71, -70, -69, -2, -1, 0, 1, 2, 3, 64, 65, 66, 67, 68, 69, 201])  # runs 69, 66 and 137 apart
    rows = []
    for r in range(m):
        c = r + offsets
        c = c[(c >= 0) & (c < k)]
        if r % 97 == 5:
            c = c[::2]
        if r % 211 == 7:
            c = np.zeros(0, np.int64)
        if r in (1000, 1001, 1002):
            c = rng.choice(k, 900, replace=False)   # 2700 nonzeros in their group: not covered, row by row
        if r % 120 == 0:
            c = rng.permutation(c)
        rows.append(c)
    ptr = np.concatenate([[0], np.cumsum([len(c) for c in rows])]).astype(np.int32)
    a = wl.Csr(m, k, ptr, np.concatenate(rows).astype(np.int32), rng.uniform(-1, 1, int(ptr[-1])).astype(dtype))
    # blocks for operands of 65 (fp64: 129) to 1024 bytes per row, merged column lists beyond
    least = 128 if dtype == np.float64 else 64
    want = 3 if least < n * np.dtype(dtype).itemsize <= 1024 else (1, 2)
    for c_order in (api.ORDER_ROW, api.ORDER_COL):
        check(torch_gpu, handle, oracle, a, n, 1.0, 0.0, preprocess=True, expect_schedule=want, c_order=c_order)
    check(torch_gpu, handle, oracle, a.with_base(1), n, -0.5, 1.5, preprocess=True, expect_schedule=want, pad_b=4, pad_c=8)


def test_blocks_row_ignores_rows_of_b_only_its_neighbours_use(torch_gpu, handle):
    """A block loads rows of op(B) for all its rows of A; a row must only see the ones it names (0 * inf = NaN)."""
    m = 64
    rows = [np.array([r, r + 1, r + 2]) for r in range(m)]
    ptr = np.concatenate([[0], np.cumsum([len(c) for c in rows])]).astype(np.int32)
    a = wl.Csr(m, m + 2, ptr, np.concatenate(rows).astype(np.int32), np.ones(3 * m, np.float32))
    n = 64
    B = np.ones((m + 2, n), np.float32)
    B[10, :] = np.inf   # named by rows 8, 9, 10 only
    st, got, _ = run_spmm(torch_gpu, handle, a, B, np.zeros((m, n), np.float32), 1.0, 0.0, preprocess=True,
                          expect_schedule=3)
    assert st == 0
    for r in range(m):
        if r in (8, 9, 10):
            assert np.all(np.isinf(got[r]))
        else:
            assert np.all(got[r] == 3.0), r


def grid_9pt(line, lines, dtype, rng, broken=False):
    """9-point stencil on `lines` grid lines of `line` points, numbered line by line; broken: rows with holes, empty
    rows, unsorted rows, three rows with 800 nonzeros each (their group is too long to cover) and a duplicate column."""
    m = line * lines
    rows = []
    for r in range(m):
        y, x = divmod(r, line)
        c = [yy * line + xx for yy in (y - 1, y, y + 1) for xx in (x - 1, x, x + 1) if 0 <= yy < lines and 0 <= xx < line]
        c = np.array(c, np.int64)
        if broken:
            if r % 97 == 5:
                c = c[::2]
            if r % 211 == 7:
                c = np.zeros(0, np.int64)
            if r % 120 == 0:
                c = rng.permutation(c)
            if r % 333 == 9 and len(c) > 2:
                c = np.concatenate([c[:2], c[1:]])     # a column twice in a row
            if r in (1000, 1001, 1002):
                c = rng.choice(m, 800, replace=False)
        rows.append(c)
    ptr = np.concatenate([[0], np.cumsum([len(c) for c in rows])]).astype(np.int32)
    return wl.Csr(m, m, ptr, np.concatenate(rows).astype(np.int32), rng.uniform(-1, 1, int(ptr[-1])).astype(dtype))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n", [20, 36, 64, 72, 128, 260])
def test_strips_grid_with_broken_rows(torch_gpu, handle, oracle, dtype, n):
    """Groups of strips a grid line apart (lines of 20 points, 151 of them: the last stretch of four lines is short),
    rows with holes, empty, unsorted and overlong rows, duplicates; panels of 16 lanes; both layouts of C."""
    a = grid_9pt(20, 151, dtype, np.random.default_rng(6), broken=True)
    row_bytes = n * np.dtype(dtype).itemsize
    # strips for operands of 129 to 1024 bytes per row, groups of eight rows from 65 bytes, merged column lists otherwise
    want = 4 if 128 < row_bytes <= 1024 else 3 if 64 < row_bytes <= 128 and dtype == np.float32 else (1, 2)
    for c_order in (api.ORDER_ROW, api.ORDER_COL):
        check(torch_gpu, handle, oracle, a, n, 1.0, 0.0, preprocess=True, expect_schedule=want, c_order=c_order,
              prepare_for_row_major_c=True)
    check(torch_gpu, handle, oracle, a.with_base(1), n, -0.5, 1.5, preprocess=True, expect_schedule=want, pad_b=4, pad_c=8)
    check(torch_gpu, handle, oracle, a, n, 0.5, -1.0, preprocess=True, expect_schedule=want, c_order=api.ORDER_COL, pad_c=4,
          prepare_for_row_major_c=True)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_strips_and_the_size_of_their_copy_in_lds(torch_gpu, handle, oracle, dtype):
    """A strip's values are copied into LDS when they are at most 128: a 27-point stencil in fp64 (4 rows x 27 values)
    gets groups of strips; a 7 x 7 stencil on a plane grid (4 x 49 values) is left to the groups of eight rows."""
    if dtype == np.float64:
        a = wl.stencil_27pt(16, dtype=dtype)
    else:
        line, lines = 24, 40
        rng = np.random.default_rng(2)
        rows = []
        for r in range(line * lines):
            y, x = divmod(r, line)
            rows.append(np.array([yy * line + xx for yy in range(y - 3, y + 4) for xx in range(x - 3, x + 4)
                                  if 0 <= yy < lines and 0 <= xx < line], np.int64))
        ptr = np.concatenate([[0], np.cumsum([len(c) for c in rows])]).astype(np.int32)
        a = wl.Csr(line * lines, line * lines, ptr, np.concatenate(rows).astype(np.int32),
                   rng.uniform(-1, 1, int(ptr[-1])).astype(dtype))
    want = 4 if dtype == np.float64 else 3
    for n in (48, 64):
        check(torch_gpu, handle, oracle, a, n, 1.0, 0.0, preprocess=True, expect_schedule=want)
        check(torch_gpu, handle, oracle, a.with_base(1), n, -1.5, 0.5, preprocess=True, expect_schedule=want, pad_b=4, pad_c=4)


@pytest.mark.parametrize("grid,state", [(40, 4), (41, 3)])
def test_blocks_with_a_value_array_that_is_not_16_byte_aligned(torch_gpu, handle, oracle, grid, state):
    """The copies of the values in LDS are made of 16-byte pieces: an array that does not begin on such a boundary
    is read where it lies (both kinds of diagonal blocks)."""
    torch = torch_gpu
    a = wl.stencil_27pt(grid, dtype=np.float32)
    n = 64
    rng = np.random.default_rng(4)
    B = rng.uniform(-1, 1, (a.n, n)).astype(np.float32)
    d_ptr, d_col = dev(torch, a.ptr), dev(torch, a.col)
    d_val_room = torch.zeros(a.nnz + 1, dtype=torch.float32, device="cuda")
    d_val = d_val_room[1:]
    d_val.copy_(torch.from_numpy(a.val))
    assert d_val.data_ptr() % 16 == 4
    d_B = dev(torch, B)
    d_C = torch.zeros((a.m, n), dtype=torch.float32, device="cuda")
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val)
    mB, mC = api.DnMat(a.n, n, n, d_B), api.DnMat(a.m, n, n, d_C)
    st, size = api.spmm_buffer_size(handle, api.OP_N, api.OP_N, 1.0, mat, mB, 0.0, mC, api.R_32F)
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    assert api.spmm_preprocess(handle, api.OP_N, api.OP_N, 1.0, mat, mB, 0.0, mC, api.R_32F, buf) == 0
    assert mat.spmm_schedule()[0] == state
    assert api.spmm(handle, api.OP_N, api.OP_N, 1.0, mat, mB, 0.0, mC, api.R_32F, buf) == 0
    torch.cuda.synchronize()
    c_ref, bound = oracle.spmm(a.m, n, 0, a.ptr, a.col, a.val, 1.0, 0.0, B.ravel(), n, True, np.zeros(a.m * n, np.float32),
                               n, True)
    assert_within(d_C.cpu().numpy(), c_ref, bound, np.float32)


def test_strips_row_ignores_rows_of_b_only_other_strips_use(torch_gpu, handle):
    """A block of a group of strips loads rows of op(B) for up to sixteen rows of A; a row must only see the ones it
    names (0 * inf = NaN)."""
    line, lines, n = 16, 64, 64
    a = grid_9pt(line, lines, np.float32, np.random.default_rng(1))
    a = wl.Csr(a.m, a.n, a.ptr, a.col, np.ones(a.nnz, np.float32))
    B = np.ones((a.n, n), np.float32)
    hot = 20 * line + 7
    B[hot, :] = np.inf
    st, got, _ = run_spmm(torch_gpu, handle, a, B, np.zeros((a.m, n), np.float32), 1.0, 0.0, preprocess=True,
                          expect_schedule=4)
    assert st == 0
    names = {r for r in range(a.m) if hot in a.col[a.ptr[r]:a.ptr[r + 1]]}
    assert len(names) == 9
    for r in range(a.m):
        if r in names:
            assert np.all(np.isinf(got[r])), r
        else:
            assert np.all(got[r] == float(a.ptr[r + 1] - a.ptr[r])), r


@pytest.mark.parametrize("grid,state", [(40, 4), (41, 3)])
def test_blocks_schedule_used_with_a_wider_operand_than_it_was_built_for(torch_gpu, handle, oracle, grid, state):
    """The schedule belongs to the structure of A: built with a 64-column operand it also serves 256 columns (cut into
    panels) and 8 columns (too narrow for its kernel: the schedule-free kernel runs)."""
    torch = torch_gpu
    a = wl.stencil_27pt(grid, dtype=np.float32)
    rng = np.random.default_rng(9)
    d_ptr, d_col, d_val = dev(torch, a.ptr), dev(torch, a.col), dev(torch, a.val)
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val)
    sizes = {}
    ops = {}
    for n in (64, 256, 8):
        B = rng.uniform(-1, 1, (a.n, n)).astype(np.float32)
        d_B = dev(torch, B)
        d_C = torch.zeros((a.m, n), dtype=torch.float32, device="cuda")
        ops[n] = (B, d_B, d_C, api.DnMat(a.n, n, n, d_B), api.DnMat(a.m, n, n, d_C))
        st, sizes[n] = api.spmm_buffer_size(handle, api.OP_N, api.OP_N, 1.0, mat, ops[n][3], 0.0, ops[n][4], api.R_32F)
        assert st == 0
    buf = torch.empty(max(sizes.values()), dtype=torch.uint8, device="cuda")
    assert api.spmm_preprocess(handle, api.OP_N, api.OP_N, 1.0, mat, ops[64][3], 0.0, ops[64][4], api.R_32F, buf) == 0
    assert mat.spmm_schedule()[0] == state
    for n in (64, 256, 8):
        B, d_B, d_C, mB, mC = ops[n]
        assert api.spmm(handle, api.OP_N, api.OP_N, 1.0, mat, mB, 0.0, mC, api.R_32F, buf) == 0
        torch.cuda.synchronize()
        c_ref, bound = oracle.spmm(a.m, n, 0, a.ptr, a.col, a.val, 1.0, 0.0, B.ravel(), n, True,
                                   np.zeros(a.m * n, np.float32), n, True)
        assert_within(d_C.cpu().numpy(), c_ref, bound, np.float32, what="n=%d" % n)
