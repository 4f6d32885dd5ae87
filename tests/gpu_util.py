"""Helpers shared by the GPU parity tests: upload a host CSR, run calls through the C ABI."""
import numpy as np

from mcsparse_amd import api

U = {np.dtype(np.float32): 2.0 ** -24, np.dtype(np.float64): 2.0 ** -53}


def dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def run_spmv(torch, handle, csr, x, y, alpha, beta, op=api.OP_N, fmt=api.FORMAT_CSR, family=api.FAMILY_AUTO, lanes=0,
             device_scalars=False):
    """y <- alpha*op(A)*x + beta*y on the GPU through mcsparseSpMV; returns (status, y as numpy, plan)."""
    d_ptr, d_col, d_val = dev(torch, csr.ptr), dev(torch, csr.col), dev(torch, csr.val)
    d_x, d_y = dev(torch, x), dev(torch, y)
    ct = api.maca_type(csr.val.dtype)
    if fmt == api.FORMAT_CSR:
        mat = api.SpMat(csr.m, csr.n, csr.nnz, d_ptr, d_col, d_val, base=csr.base, fmt=fmt)
    else:  # the arrays are the CSC of an n x m matrix
        mat = api.SpMat(csr.n, csr.m, csr.nnz, d_ptr, d_col, d_val, base=csr.base, fmt=fmt)
    if family != api.FAMILY_AUTO or lanes:
        mat.set_plan(family, lanes)
    vx, vy = api.DnVec(d_x), api.DnVec(d_y)
    st, size = api.spmv_buffer_size(handle, op, alpha, mat, vx, beta, vy, ct)
    assert st == api.STATUS_SUCCESS, st
    assert size >= 128 and size % 128 == 0
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    if device_scalars:
        handle.set_pointer_mode(api.PTR_DEVICE)
        td = torch.float32 if ct == api.R_32F else torch.float64
        a_dev = torch.tensor([alpha], dtype=td, device="cuda")
        b_dev = torch.tensor([beta], dtype=td, device="cuda")
        st = api.spmv(handle, op, a_dev, mat, vx, b_dev, vy, ct, buf)
        handle.set_pointer_mode(api.PTR_HOST)
    else:
        st = api.spmv(handle, op, alpha, mat, vx, beta, vy, ct, buf)
    torch.cuda.synchronize()
    return st, d_y.cpu().numpy(), mat.plan()


def assert_within(y, y_ref, bound, dtype, factor=8.0, what=""):
    """|y - y_ref| <= factor * u * bound elementwise (bound already carries |alpha|, |beta*y|)."""
    u = U[np.dtype(dtype)]
    err = np.abs(y.astype(np.longdouble) - y_ref)
    tol = factor * u * bound
    bad = err > tol
    if bad.any():
        i = int(np.argmax(err - tol))
        raise AssertionError("%s: %d of %d entries outside %gu*bound; worst at %d: got %r want %r err %g tol %g" % (
            what, int(bad.sum()), y.size, factor, i, y.flat[i], y_ref.flat[i], float(err.flat[i]),
            float(tol.flat[i])))
    finite = bound > 0
    return float((err[finite] / (u * bound[finite])).max()) if finite.any() else 0.0
