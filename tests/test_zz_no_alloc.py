"""mcsparseSpMV_staticBuffer (the entry point that allocates nothing) against mcsparseSpMV.

Both run the same kernels on the same inputs, so the outputs must agree bit for bit; the result is
also held against the CPU oracle.  Two calls in a row share the library's scratch array, the second
on a smaller matrix, so stale contents of the first call would show."""
import numpy as np
import pytest

from mcsparse_amd import api
from mcsparse_amd import workloads as wl

from gpu_util import assert_within, dev

pytestmark = pytest.mark.gpu


def _both(torch, handle, oracle, a, alpha, beta, family, seed):
    rng = np.random.default_rng(seed)
    dt = a.val.dtype
    ct = api.maca_type(dt)
    x = rng.uniform(-1, 1, a.n).astype(dt)
    y = rng.uniform(-1, 1, a.m).astype(dt)
    d_ptr, d_col, d_val, d_x = dev(torch, a.ptr), dev(torch, a.col), dev(torch, a.val), dev(torch, x)
    outs = []
    for static in (False, True):
        d_y = dev(torch, y)
        mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val, base=a.base)
        mat.set_plan(family)
        vx, vy = api.DnVec(d_x), api.DnVec(d_y)
        if static:
            st = api.spmv_static_buffer(handle, api.OP_N, alpha, mat, vx, beta, vy, ct)
        else:
            st, size = api.spmv_buffer_size(handle, api.OP_N, alpha, mat, vx, beta, vy, ct)
            assert st == api.STATUS_SUCCESS
            buf = torch.empty(size, dtype=torch.uint8, device="cuda")
            st = api.spmv(handle, api.OP_N, alpha, mat, vx, beta, vy, ct, buf)
        assert st == api.STATUS_SUCCESS, st
        torch.cuda.synchronize()
        outs.append(d_y.cpu().numpy())
    if family != api.FAMILY_AUTO:  # the same kernels ran: the same bits
        assert np.array_equal(outs[0].view(np.uint8), outs[1].view(np.uint8)), \
            "static-buffer call differs from mcsparseSpMV"
    y_ref, bound = oracle.spmv(False, a.m, a.n, a.base, a.ptr, a.col, a.val, alpha, beta, x, y)
    assert_within(outs[1], y_ref, bound, dt, what="mcsparseSpMV_staticBuffer")


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_static_buffer_matches_spmv_twice(torch_gpu, handle, oracle, dtype):
    # merge family: the kernels that use the scratch (tile table, carries); long rows cross tiles
    big = wl.power_law(m=1 << 15, max_len=20000, dtype=dtype)
    small = wl.random_ragged(3001, 2999, 9, dtype=dtype, seed=5, base=1)
    _both(torch_gpu, handle, oracle, big, 1.5, 0.5, api.FAMILY_MERGE, 1)
    _both(torch_gpu, handle, oracle, small, -2.0, 0.0, api.FAMILY_MERGE, 2)
    # no forced family and no plan: the call must not analyse (mcsparseSpMV does, and may pick the other
    # family, so only the tolerance holds between the two), and still be right
    _both(torch_gpu, handle, oracle, small, 1.0, 1.0, api.FAMILY_AUTO, 3)


def test_static_buffer_refuses_what_does_not_fit(torch_gpu, handle):
    torch = torch_gpu
    a = wl.random_ragged(64, 64, 4, dtype=np.float32, seed=1)
    d_ptr, d_col, d_val = dev(torch, a.ptr), dev(torch, a.col), dev(torch, a.val)
    d_x, d_y = torch.zeros(64, device="cuda"), torch.zeros(64, device="cuda")
    # a descriptor that claims more nonzeros than the scratch has room for: refused before any launch
    huge = api.SpMat(1 << 22, 64, 1 << 31, d_ptr, d_col, d_val)
    vx, vy = api.DnVec(d_x), api.DnVec(d_y, size=1 << 22)
    assert api.spmv_static_buffer(handle, api.OP_N, 1.0, huge, vx, 0.0, vy, api.R_32F) == \
        api.STATUS_INSUFFICIENT_RESOURCES
    handle.set_pointer_mode(api.PTR_DEVICE)
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val)
    st = api.spmv_static_buffer(handle, api.OP_N, 1.0, mat, api.DnVec(d_x), 0.0, api.DnVec(d_y), api.R_32F)
    handle.set_pointer_mode(api.PTR_HOST)
    assert st == api.STATUS_NOT_SUPPORTED
