"""Size-independent output checks for SpMM / SDDMM at sizes where a CPU product would take minutes.

Everything is formed on the device in float64 from the operator's own inputs, so a 114M-edge operator is
checked in well under a second: a checksum of the whole product (SpMM column sums against the weighted
out-degree contraction of X), closed forms (all-ones operands), and samples (rows / edges) against their
float64 sums.  The bar is the parity bar of the test-suite: |got - ref| <= 1e-5 + 1e-4 |ref| + 8 eps32 * (sum
of the absolute values of the terms added up).  Each function returns a list of failure messages (empty:
the output passed); `bench.py` and the full-size GPU tests both call them.
"""
import numpy as np
import torch

RTOL, ATOL = 1e-4, 1e-5
MASS_FACTOR = 8 * float(np.finfo(np.float32).eps)


def _within(got, ref64, mass):
    return ((got.double() - ref64).abs() <= ATOL + RTOL * ref64.abs() + MASS_FACTOR * mass).all().item()


def spmm_failures(out, indptr, indices_d, vals_d, x_d, what="spmm"):
    """`out` = A X for the CSR adjacency (indptr: host int array, indices_d: device int64, vals_d: device fp32).
    Column sums of `out` against sum_u (sum of the weights of u's out-edges) * X[u, :]  -- every stored element
    enters it once -- and five rows (largest, smallest, first, middle, last) against their float64 sums."""
    failures = []
    n_dst = indptr.shape[0] - 1
    if not torch.isfinite(out).all().item():
        failures.append("%s: non-finite output" % what)
    col_w = torch.zeros(x_d.shape[0], device=x_d.device, dtype=torch.float64)
    col_w.index_add_(0, indices_d, vals_d.double())
    x64 = x_d.double()
    expect = (col_w[:, None] * x64).sum(0)
    scale = (col_w[:, None] * x64.abs()).sum(0)
    if not ((out.double().sum(0) - expect).abs() <= 1e-5 * scale).all().item():
        failures.append("%s: column sums differ from the out-degree contraction of X" % what)
    del x64
    deg = np.diff(indptr)
    for v in sorted({int(np.argmax(deg)), int(np.argmin(deg)), 0, n_dst // 2, n_dst - 1}):
        e = slice(int(indptr[v]), int(indptr[v + 1]))
        terms = vals_d[e].double()[:, None] * x_d[indices_d[e]].double()
        if not _within(out[v], terms.sum(0), terms.abs().sum(0)):
            failures.append("%s: row %d differs from its float64 sum" % (what, v))
    return failures


def spmm_ones_failures(out_ones, indptr, vals_d, what="spmm"):
    """`out_ones` = A 1: every column holds the row's weight sum."""
    failures = []
    row_of = torch.repeat_interleave(torch.arange(indptr.shape[0] - 1, device=vals_d.device),
                                     torch.from_numpy(np.diff(indptr).astype(np.int64)).to(vals_d.device))
    row_sum = torch.zeros(indptr.shape[0] - 1, device=vals_d.device, dtype=torch.float64)
    row_sum.index_add_(0, row_of, vals_d.double())
    if not _within(out_ones[:, 0], row_sum, row_sum):            # weights are non-negative in every benchmark input
        failures.append("%s: all-ones features do not give the rows' weight sums" % what)
    if not (out_ones == out_ones[:, :1]).all().item():
        failures.append("%s: all-ones features give different columns" % what)
    return failures


def sddmm_failures(out, row_d, col_d, src_d, dst_d, samples=200000, seed=7, what="sddmm"):
    """`out[e]` (or `out[e, h]` for [n, H, D] operands) = <src[col e], dst[row e]>, in the order of row_d / col_d
    (device int64): all results finite, and `samples` random edges plus the first and the last one against float64."""
    failures = []
    nnz = row_d.shape[0]
    if not torch.isfinite(out).all().item():
        failures.append("%s: non-finite scores" % what)
    g = torch.Generator(device=out.device)
    g.manual_seed(seed)
    pick = torch.randint(0, nnz, (samples,), generator=g, device=out.device)
    pick[0], pick[1] = 0, nnz - 1
    prod = src_d[col_d[pick]].double() * dst_d[row_d[pick]].double()
    if not _within(out[pick], prod.sum(-1), prod.abs().sum(-1)):
        failures.append("%s: sampled edges differ from their float64 dot products" % what)
    return failures


def sddmm_ones_failures(out, col_d, src_d, what="sddmm"):
    """`out` for dst = ones: every edge holds the sum of its source row (per head for [n, H, D] operands)."""
    s64 = src_d.double()
    ref, mass = s64.sum(-1)[col_d], s64.abs().sum(-1)[col_d]
    if not _within(out, ref, mass):
        return ["%s: all-ones destination features do not give the source rows' sums" % what]
    return []
