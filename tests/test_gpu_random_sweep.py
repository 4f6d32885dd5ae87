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
