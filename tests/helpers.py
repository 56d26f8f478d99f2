"""Shared comparison helpers for the parity tests."""
import numpy as np
import scipy.sparse as sp

RTOL, ATOL = 1e-4, 1e-5          # fp32 parity bar: rel 1e-4, abs 1e-5
EPS32 = float(np.finfo(np.float32).eps)
MASS_FACTOR = 8 * EPS32          # share of a sum's absolute mass allowed as rounding error


def assert_sum_close(got, ref64, mass, what=""):
    """|got - ref| <= ATOL + RTOL*|ref| + MASS_FACTOR * mass, elementwise.

    `mass` is the sum of the absolute values of the terms that were added up.  For short sums
    the last term is far below ATOL and this is the plain rel 1e-4 / abs 1e-5 bar; for hub rows
    (thousands of N(0,1)-sized terms cancelling) no fp32 summation order, the reference's
    sequential one included, can meet an absolute 1e-5, and the rounding allowance scales with
    what was summed.  A dropped, doubled or misplaced term is orders of magnitude above it.
    """
    got = np.asarray(got, dtype=np.float64)
    err = np.abs(got - ref64)
    tol = ATOL + RTOL * np.abs(ref64) + MASS_FACTOR * mass
    bad = err > tol
    if bad.any():
        i = np.unravel_index(np.argmax(err - tol), err.shape)
        raise AssertionError("%s: %d element(s) out of tolerance; worst at %s: got %r, expected %r, tol %g"
                             % (what, int(bad.sum()), i, got[i], ref64[i], tol[i]))


def spmm_mass(adj, x):
    a = sp.csr_matrix(adj).astype(np.float64)
    a.data = np.abs(a.data)
    return np.asarray(a.dot(np.abs(np.asarray(x, dtype=np.float64))))


def sddmm_mass(row, col, src, dst, chunk=1 << 18):
    """Per edge (and head if 3-D) sum of |src * dst|."""
    three = src.ndim == 3
    out = np.empty((len(row), src.shape[1]) if three else (len(row),), dtype=np.float64)
    for s in range(0, len(row), chunk):
        e = slice(s, s + chunk)
        p = np.abs(src[col[e]].astype(np.float64) * dst[row[e]].astype(np.float64))
        out[e] = p.sum(-1)
    return out
