"""Writes tests/golden/*.npz: small CSR inputs with the outputs scipy.sparse gives for them.

The reference ships no tests, fixtures or golden vectors and cannot run outside MetaX hardware,
so these vectors come from an independent implementation of the same mathematics:
  * SpMV / SpMM: scipy's csr @ dense on integer-valued float64 data, where every product and
    partial sum is exact, so any correct summation order gives the same bits;
  * csr2csc: scipy's csr.tocsc(), a stable counting sort by column -- the order the
    reference's stable LSD radix sort produces (entries of a column keep their CSR order);
  * csr2coo / coo2csr: scipy's tocoo().row and the offsets of the CSR itself.
Run from the repository root:  python tests/golden/make_golden.py
"""
import os

import numpy as np
import scipy.sparse as sp

HERE = os.path.dirname(os.path.abspath(__file__))


def integer_csr(rng, m, n, density, with_empty=True):
    a = sp.random(m, n, density=density, random_state=np.random.RandomState(rng.integers(1 << 30)), format="csr",
                  dtype=np.float64)
    a.data = rng.integers(-4, 5, size=a.data.shape).astype(np.float64)
    a.data[a.data == 0] = 3.0  # keep explicit entries non-zero so scipy never drops them
    if with_empty and m > 3:
        lil = a.tolil()
        lil[1, :] = 0
        lil[m - 1, :] = 0
        a = lil.tocsr()
    a.sort_indices()
    return a


def main():
    rng = np.random.Generator(np.random.PCG64(20240611))
    cases = {}
    for name, (m, n, dens) in {"tall": (37, 11, 0.3), "wide": (9, 50, 0.25), "square": (64, 64, 0.1),
                               "tiny": (1, 1, 1.0), "hollow": (20, 20, 0.02)}.items():
        a = integer_csr(rng, m, n, dens, with_empty=(name != "tiny"))
        x = rng.integers(-3, 4, size=n).astype(np.float64)
        xt = rng.integers(-3, 4, size=m).astype(np.float64)
        y0 = rng.integers(-3, 4, size=m).astype(np.float64)
        B = rng.integers(-3, 4, size=(n, 5)).astype(np.float64)
        C0 = rng.integers(-3, 4, size=(m, 5)).astype(np.float64)
        alpha, beta = 2.0, -3.0
        csc = a.tocsc()
        coo = a.tocoo()
        cases[name] = dict(
            m=m, n=n, ptr=a.indptr.astype(np.int32), col=a.indices.astype(np.int32), val=a.data,
            x=x, xt=xt, y0=y0, alpha=alpha, beta=beta,
            y_n=alpha * (a @ x) + beta * y0,
            y_t=alpha * (a.T @ xt),
            B=B, C0=C0, C=alpha * (a @ B) + beta * C0,
            csc_ptr=csc.indptr.astype(np.int32), csc_row=csc.indices.astype(np.int32), csc_val=csc.data,
            coo_row=coo.row.astype(np.int32),
        )
    for name, c in cases.items():
        np.savez(os.path.join(HERE, "csr_%s.npz" % name), **c)
        print(name, c["m"], c["n"], c["col"].shape[0])


if __name__ == "__main__":
    main()
