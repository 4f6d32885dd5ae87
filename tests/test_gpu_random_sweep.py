"""Seeded random sweep on the GPU: SpMV, SpMM and csr2csc through the C ABI against the CPU oracle
on shapes drawn around the sizes the kernels cut their work at (workgroups of 256 threads, merge
tiles of 1024 and 2048 path items, sort tiles of 4096 triples, radix digits of 8 bits), with
sorted and unsorted rows, both index bases, both value types and every kernel family.  The cases
are a fixed function of the seeds below; a failure names its case."""
import numpy as np
import pytest

from mcsparse_amd import api
from mcsparse_amd import workloads as wl

import test_gpu_convert as conv
import test_gpu_spmm as spmm
import test_gpu_spmv as spmv

pytestmark = pytest.mark.gpu

CASES_PER_SEED = 60


def draw_matrix(rng, dtype, base):
    kind = int(rng.integers(0, 5))
    if kind == 0:    # a few rows with lengths on either side of the merge tiles
        m = int(rng.integers(1, 40))
        n = int(rng.integers(3000, 9000))
        lens = rng.choice([0, 1, 255, 256, 257, 1023, 1024, 1025, 2047, 2048, 2049, 2999], size=m)
    elif kind == 1:  # many short rows, row counts on either side of workgroup multiples
        m = int(rng.choice([1, 63, 64, 65, 255, 256, 257, 1023, 1025, 4095, 4097, 10007]))
        n = int(rng.integers(1, 5000))
        lens = rng.poisson(rng.choice([0.3, 1, 3, 9, 17, 33, 70]), size=m)
    elif kind == 2:  # power-law row lengths
        m = int(rng.integers(100, 20000))
        n = int(rng.integers(100, 60000))
        lens = wl.zipf_row_lengths(m, 1.8, max(1, n // 2), rng)
    elif kind == 3:  # one to three huge rows among empty ones
        m = int(rng.integers(2, 5000))
        n = int(rng.integers(5000, 200000))
        lens = np.zeros(m, np.int64)
        for _ in range(int(rng.integers(1, 4))):
            lens[int(rng.integers(0, m))] = int(rng.integers(1, n))
    else:            # column ranges on either side of one, two and three radix digits
        m = int(rng.integers(10, 3000))
        n = int(rng.choice([255, 256, 257, 65535, 65536, 65537, 1 << 20, (1 << 24) + 1]))
        lens = rng.poisson(8, size=m)
    lens = np.minimum(np.asarray(lens, np.int64), n)
    ptr = np.concatenate([[0], np.cumsum(lens)])
    nnz = int(ptr[-1])
    col = np.empty(nnz, np.int64)
    for r in range(m):
        k = int(lens[r])
        if k == 0:
            continue
        if k * 4 > n:
            c = rng.permutation(n)[:k]
        else:
            c = np.unique(rng.integers(0, n, size=2 * k))[:k]
            while c.size < k:
                c = np.unique(np.concatenate([c, rng.integers(0, n, size=k)]))[:k]
        col[ptr[r]:ptr[r + 1]] = np.sort(c) if rng.random() < 0.8 else rng.permutation(c)
    val = rng.uniform(-1, 1, nnz).astype(dtype)
    return wl.Csr(m, n, ptr + base, col + base, val, base), kind


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_sweep(torch_gpu, handle, oracle, seed):
    top = np.random.default_rng(seed)
    for case in range(CASES_PER_SEED):
        case_seed = int(top.integers(0, 1 << 30))
        r = np.random.default_rng(case_seed)
        dtype = [np.float32, np.float64][int(r.integers(0, 2))]
        base = int(r.integers(0, 2))
        a, kind = draw_matrix(r, dtype, base)
        what = int(r.integers(0, 3))
        name = "seed %d case %d (%d): kind %d op %d, %d x %d, %d nonzeros, %s, base %d" % (
            seed, case, case_seed, kind, what, a.m, a.n, a.nnz, np.dtype(dtype).name, base)
        if a.nnz == 0:
            continue
        if what == 0:
            alpha, beta = [(1.0, 0.0), (-1.5, 0.75), (0.0, 2.0), (2.0, 1.0)][int(r.integers(0, 4))]
            op = [api.OP_N, api.OP_T][int(r.integers(0, 2))]
            family = [api.FAMILY_AUTO, api.FAMILY_VECTOR, api.FAMILY_MERGE][int(r.integers(0, 3))]
            lanes = 0
            if family == api.FAMILY_VECTOR:
                lanes = int(r.choice([1, 2, 4, 8, 16, 32, 64]))
            elif family == api.FAMILY_MERGE:
                lanes = int(r.integers(0, 2))  # 1: tiles in the order of their first column
            spmv.check(torch_gpu, handle, oracle, a, alpha, beta, op=op, family=family, lanes=lanes, seed=case_seed,
                       what=name)
        elif what == 1:
            if a.m * 300 > 4_000_000 or a.n * 300 > 6_000_000:
                n = int(r.choice([1, 4, 8, 16]))
            else:
                n = int(r.choice([1, 3, 4, 8, 12, 13, 16, 32, 60, 64, 68, 128, 200, 256, 300]))
            alpha, beta = [(1.0, 0.0), (-1.5, 0.75), (2.0, 1.0)][int(r.integers(0, 3))]
            try:
                spmm.check(torch_gpu, handle, oracle, a, n, alpha, beta, seed=case_seed,
                           op_b=[api.OP_N, api.OP_T][int(r.integers(0, 2))],
                           b_order=[api.ORDER_ROW, api.ORDER_COL][int(r.integers(0, 2))],
                           c_order=[api.ORDER_ROW, api.ORDER_COL][int(r.integers(0, 2))],
                           pad_b=int(r.choice([0, 0, 4, 5])), pad_c=int(r.choice([0, 0, 4, 3])),
                           preprocess=bool(r.integers(0, 2)))
            except AssertionError as e:
                raise AssertionError(name + ": " + str(e)) from e
        else:
            conv.check_csr2csc(torch_gpu, handle, oracle, a, name)


def draw_grid_matrix(rng, dtype, base):
    """A matrix with diagonals: a stencil on `lines` grid lines of `line` points (sometimes in planes), with random
    rows thinned out, emptied, shuffled or given a duplicate, so that mcsparseSpMM_preprocess builds diagonal blocks
    over groups of eight rows or over groups of strips a line apart, whichever the matrix suits."""
    line = int(rng.choice([8, 9, 12, 16, 20, 24, 30, 36, 64]))
    lines = int(rng.integers(9, 80))
    planes = int(rng.choice([1, 1, 2, 3]))
    reach_x = int(rng.choice([1, 1, 2]))
    reach_y = int(rng.choice([1, 1, 2]))
    m = line * lines * planes
    k = m + int(rng.choice([0, 0, 7]))  # sometimes more columns than rows
    offs = [(dz, dy, dx) for dz in range(-(planes > 1), (planes > 1) + 1) for dy in range(-reach_y, reach_y + 1)
            for dx in range(-reach_x, reach_x + 1)]
    rows = []
    for r in range(m):
        z, rest = divmod(r, line * lines)
        y, x = divmod(rest, line)
        c = np.array([(z + dz) * line * lines + (y + dy) * line + (x + dx) for dz, dy, dx in offs
                      if 0 <= z + dz < planes and 0 <= y + dy < lines and 0 <= x + dx < line], np.int64)
        u = rng.random()
        if u < 0.02:
            c = c[rng.random(len(c)) < 0.6]
        elif u < 0.03:
            c = np.zeros(0, np.int64)
        elif u < 0.05:
            c = rng.permutation(c)
        elif u < 0.06 and len(c) > 1:
            c = np.concatenate([c[:1], c])
        rows.append(c)
    if rng.random() < 0.3:
        rows[int(rng.integers(0, m))] = rng.choice(k, min(k, 2300), replace=False)  # a group too long to cover
    ptr = np.concatenate([[0], np.cumsum([len(c) for c in rows])])
    col = np.concatenate(rows) if int(ptr[-1]) else np.zeros(0, np.int64)
    val = rng.uniform(-1, 1, int(ptr[-1])).astype(dtype)
    return wl.Csr(m, k, ptr + base, col + base, val, base), (line, lines, planes)


@pytest.mark.parametrize("seed", [21, 22])
def test_random_grid_sweep(torch_gpu, handle, oracle, seed):
    top = np.random.default_rng(seed)
    kinds = set()
    for case in range(40):
        case_seed = int(top.integers(0, 1 << 30))
        r = np.random.default_rng(case_seed)
        dtype = [np.float32, np.float64][int(r.integers(0, 2))]
        base = int(r.integers(0, 2))
        a, shape = draw_grid_matrix(r, dtype, base)
        n = int(r.choice([20, 32, 36, 48, 64, 68, 100, 128, 256, 260]))
        alpha, beta = [(1.0, 0.0), (-1.5, 0.75), (2.0, 1.0)][int(r.integers(0, 3))]
        c_order = [api.ORDER_ROW, api.ORDER_ROW, api.ORDER_COL][int(r.integers(0, 3))]
        name = "seed %d case %d (%d): grid %r, %d x %d, %d nonzeros, %s, base %d, n %d" % (
            seed, case, case_seed, shape, a.m, a.n, a.nnz, np.dtype(dtype).name, base, n)
        try:
            spmm.check(torch_gpu, handle, oracle, a, n, alpha, beta, seed=case_seed, c_order=c_order,
                       pad_b=int(r.choice([0, 0, 4])), pad_c=int(r.choice([0, 0, 4])), preprocess=True,
                       prepare_for_row_major_c=bool(r.integers(0, 2)), expect_schedule=(1, 2, 3, 4), seen=kinds)
        except AssertionError as e:
            raise AssertionError(name + ": " + str(e)) from e
    assert 4 in kinds and len(kinds) >= 2, kinds  # groups of strips, and at least one other kind of schedule
