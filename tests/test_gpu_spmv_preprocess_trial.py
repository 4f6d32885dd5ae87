"""mcsparseSpMV_preprocess ends, for a direction that does not transpose, with a trial of its copy against the row
kernels and keeps the copy only where it is the faster one.  Checked here: a preprocessed call is never much slower
than a call that was not prepared; the trial leaves the caller's y and the handle alone; results stay within
8*u*(|alpha| * |A||x| + |beta*y|) whichever way the trial went."""
import numpy as np
import pytest

from mcsparse_amd import api
from mcsparse_amd import workloads as wl

from gpu_util import assert_within, dev

pytestmark = pytest.mark.gpu


def timed_us(torch, handle, mat, vx, vy, ct, buf, alg, steps=20):
    for _ in range(3):
        assert api.spmv(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, ct, buf, alg=alg) == api.STATUS_SUCCESS
    torch.cuda.synchronize()
    best = None
    for _ in range(3):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            api.spmv(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, ct, buf, alg=alg)
        e1.record()
        torch.cuda.synchronize()
        t = e0.elapsed_time(e1) / steps * 1000
        best = t if best is None else min(best, t)
    return best


def prepared(torch, handle, a, d, x, alg, trial):
    """(matrix, buffer, y, state) after mcsparseSpMV_preprocess; y is filled with a pattern the call must leave."""
    ct = api.maca_type(a.val.dtype)
    mat = api.SpMat(a.m, a.n, a.nnz, d[0], d[1], d[2], base=a.base)
    y = torch.full((a.m,), 7.25, dtype=x.dtype, device="cuda")
    vx, vy = api.DnVec(x), api.DnVec(y)
    handle.set_spmv_preprocess_trial(trial)
    st, size = api.spmv_preprocess_buffer_size(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, ct, alg=alg)
    assert st == api.STATUS_SUCCESS
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    assert api.spmv_preprocess(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, ct, buf, alg=alg) == api.STATUS_SUCCESS
    torch.cuda.synchronize()
    assert bool((y == 7.25).all()), "preprocess wrote the caller's y"
    return mat, buf, y, vx, vy, mat.spmv_preprocess_state()[0]


MATRICES = {
    # rows that read x line by line as they lie: the row kernels are the faster
    "laplacian 2048^2 fp32": (lambda: wl.laplacian_5pt(2048, dtype=np.float32), {1}),
    "stencil 96^3 fp64": (lambda: wl.stencil_27pt(96, dtype=np.float64), {1}),
    # short rows scattered over an x of 16 MB: the copy is more than twice as fast
    "uniform 4M x 8 fp32": (lambda: wl.uniform_rows(m=1 << 22, per_row=8, dtype=np.float32), {2, 3}),
}


@pytest.mark.parametrize("alg", [api.SPMV_ALG_DEFAULT, api.SPMV_CSR_ALG2], ids=["default", "alg2"])
@pytest.mark.parametrize("name", sorted(MATRICES))
def test_a_prepared_call_is_not_slower_than_one_that_was_not(torch_gpu, handle, oracle, name, alg):
    torch = torch_gpu
    make, states = MATRICES[name]
    a = make()
    dt = a.val.dtype
    ct = api.maca_type(dt)
    rng = np.random.default_rng(5)
    x_host = rng.uniform(-1, 1, a.n).astype(dt)
    d = [dev(torch, v) for v in (a.ptr, a.col, a.val)]
    x = dev(torch, x_host)

    plain = api.SpMat(a.m, a.n, a.nnz, d[0], d[1], d[2], base=a.base)
    y_plain = torch.zeros(a.m, dtype=x.dtype, device="cuda")
    vx, vy_plain = api.DnVec(x), api.DnVec(y_plain)
    st, size = api.spmv_buffer_size(handle, api.OP_N, 1.0, plain, vx, 0.0, vy_plain, ct)
    assert st == api.STATUS_SUCCESS
    plain_buf = torch.empty(max(size, 128), dtype=torch.uint8, device="cuda")
    t_plain = timed_us(torch, handle, plain, vx, vy_plain, ct, plain_buf, alg)

    mat, buf, y, vx2, vy, state = prepared(torch, handle, a, d, x, alg, trial=True)
    assert state in states, (name, state)
    t_prepared = timed_us(torch, handle, mat, vx2, vy, ct, buf, alg)
    # the trial keeps a copy that is faster by a twentieth; the slack here is for the noise of two timings (the copies
    # that were turned down took 1.5 to 3.6 times as long as the row kernels)
    assert t_prepared <= 1.25 * t_plain, (name, state, t_plain, t_prepared)

    y_ref, bound = oracle.spmv(False, a.m, a.n, a.base, a.ptr, a.col, a.val, 1.0, 0.0, x_host, np.zeros(a.m, dt))
    assert api.spmv(handle, api.OP_N, 1.0, mat, vx2, 0.0, vy, ct, buf, alg=alg) == api.STATUS_SUCCESS
    torch.cuda.synchronize()
    assert_within(y.cpu().numpy(), y_ref, bound, dt, what="%s after the trial (state %d)" % (name, state))


def test_without_the_trial_every_copy_is_kept(torch_gpu, handle, oracle):
    torch = torch_gpu
    a = wl.laplacian_5pt(2048, dtype=np.float32)
    rng = np.random.default_rng(6)
    x_host = rng.uniform(-1, 1, a.n).astype(np.float32)
    d = [dev(torch, v) for v in (a.ptr, a.col, a.val)]
    x = dev(torch, x_host)
    mat, buf, y, vx, vy, state = prepared(torch, handle, a, d, x, api.SPMV_ALG_DEFAULT, trial=False)
    assert state == 3
    assert api.spmv(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, api.R_32F, buf) == api.STATUS_SUCCESS
    torch.cuda.synchronize()
    y_ref, bound = oracle.spmv(False, a.m, a.n, a.base, a.ptr, a.col, a.val, 1.0, 0.0, x_host, np.zeros(a.m, np.float32))
    assert_within(y.cpu().numpy(), y_ref, bound, np.float32, what="copy kept without a trial")


def test_the_trial_leaves_the_pointer_mode_and_takes_any_x(torch_gpu, handle, oracle):
    """Scalars on the device (the trial multiplies with host scalars of its own), an x full of NaN at preprocess
    time (only its memory is used), the real x afterwards."""
    torch = torch_gpu
    a = wl.uniform_rows(m=1 << 20, per_row=8, dtype=np.float64)
    rng = np.random.default_rng(7)
    x_host = rng.uniform(-1, 1, a.n)
    y_host = rng.uniform(-1, 1, a.m)
    d = [dev(torch, v) for v in (a.ptr, a.col, a.val)]
    x = torch.full((a.n,), float("nan"), dtype=torch.float64, device="cuda")
    y = dev(torch, y_host)
    scalars = dev(torch, np.array([1.5, -0.5]))
    mat = api.SpMat(a.m, a.n, a.nnz, d[0], d[1], d[2], base=a.base)
    vx, vy = api.DnVec(x), api.DnVec(y)
    st, size = api.spmv_preprocess_buffer_size(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, api.R_64F)
    assert st == api.STATUS_SUCCESS
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    handle.set_pointer_mode(api.PTR_DEVICE)
    lib = handle.lib
    import ctypes
    alpha_p, beta_p = ctypes.c_void_p(scalars.data_ptr()), ctypes.c_void_p(scalars.data_ptr() + 8)
    assert lib.mcsparseSpMV_preprocess(handle.ptr, api.OP_N, alpha_p, mat.ptr, vx.ptr, beta_p, vy.ptr, api.R_64F,
                                       api.SPMV_ALG_DEFAULT, ctypes.c_void_p(buf.data_ptr())) == api.STATUS_SUCCESS
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy(), y_host)
    state = mat.spmv_preprocess_state()[0]
    assert state in (1, 3)
    x.copy_(torch.from_numpy(x_host))
    assert lib.mcsparseSpMV(handle.ptr, api.OP_N, alpha_p, mat.ptr, vx.ptr, beta_p, vy.ptr, api.R_64F,
                            api.SPMV_ALG_DEFAULT, ctypes.c_void_p(buf.data_ptr())) == api.STATUS_SUCCESS
    torch.cuda.synchronize()
    handle.set_pointer_mode(api.PTR_HOST)
    y_ref, bound = oracle.spmv(False, a.m, a.n, a.base, a.ptr, a.col, a.val, 1.5, -0.5, x_host, y_host)
    assert_within(y.cpu().numpy(), y_ref, bound, np.float64, what="device scalars after the trial (state %d)" % state)


def test_a_band_width_set_by_the_caller_is_not_tried(torch_gpu, handle, oracle):
    """mcsparseSpMatSetSpMVBandBytes says that the caller is measuring the copy by itself: it is kept, also on the
    Laplacian, where the trial turns it down."""
    torch = torch_gpu
    a = wl.laplacian_5pt(2048, dtype=np.float32)
    rng = np.random.default_rng(8)
    x_host = rng.uniform(-1, 1, a.n).astype(np.float32)
    d = [dev(torch, v) for v in (a.ptr, a.col, a.val)]
    x = dev(torch, x_host)
    y = torch.zeros(a.m, dtype=torch.float32, device="cuda")
    mat = api.SpMat(a.m, a.n, a.nnz, d[0], d[1], d[2], base=a.base)
    mat.set_band_bytes(1 << 21)
    vx, vy = api.DnVec(x), api.DnVec(y)
    assert handle.spmv_preprocess_trial() is True
    st, size = api.spmv_preprocess_buffer_size(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, api.R_32F)
    assert st == api.STATUS_SUCCESS
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    assert api.spmv_preprocess(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, api.R_32F, buf) == api.STATUS_SUCCESS
    assert mat.spmv_preprocess_state()[0] == 3
    assert api.spmv(handle, api.OP_N, 1.0, mat, vx, 0.0, vy, api.R_32F, buf) == api.STATUS_SUCCESS
    torch.cuda.synchronize()
    y_ref, bound = oracle.spmv(False, a.m, a.n, a.base, a.ptr, a.col, a.val, 1.0, 0.0, x_host, np.zeros(a.m, np.float32))
    assert_within(y.cpu().numpy(), y_ref, bound, np.float32, what="copy of a caller who set the band width")
