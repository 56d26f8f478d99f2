"""Non-finite source rows stay in the destination rows that reference them.

The reference sums only a row's own elements (python/featgraph/op/vanilla_spmm.py:114-123), so an
Inf or NaN in X[u] reaches out[v] exactly when (v, u) is a stored element.  The kernels issue
loads for slots without an element (a re-read of the row's last element, or the next row's
element in the walk that gives every lane group rows of its own); what those loads return must be
discarded, not multiplied by zero.  The graphs below hold many rows of 1-3 elements (items of far
more than 2 * 64/L rows, which is what selects that walk), medium rows, empty rows and one row
longer than the split threshold.
"""
import numpy as np
import pytest
import scipy.sparse as sp

pytestmark = pytest.mark.gpu

BAD = {11: np.inf, 222: np.nan, 1500: -np.inf}      # source row -> value of every feature of that row


def _short_row_graph(rng, n_rows=1200, n_cols=3000):
    lens = rng.integers(1, 4, size=n_rows)
    lens[rng.choice(n_rows, 40, replace=False)] = 0              # empty rows
    lens[rng.choice(n_rows, 60, replace=False)] = rng.integers(5, 60, size=60)
    lens[700] = 1500                                             # longer than the split threshold
    rows, cols = [], []
    for r, l in enumerate(lens):
        c = np.sort(rng.choice(n_cols, size=int(l), replace=False))
        rows.append(np.full(len(c), r)); cols.append(c)
    rows, cols = np.concatenate(rows), np.concatenate(cols)
    # make sure the bad sources are referenced by short rows that sit between clean short rows
    vals = (rng.random(len(rows)) * 0.9 + 0.1).astype("float32")
    a = sp.csr_matrix((vals, (rows, cols)), shape=(n_rows, n_cols)).tolil()
    for i, c in enumerate(BAD):
        for r in (100 + 7 * i, 400 + 7 * i, 900 + 7 * i):
            if lens[r] == 0:
                continue
            a[r, c] = 0.5
    a = a.tocsr().astype("float32"); a.sort_indices()
    return a


def _touching(adj, cols):
    """Boolean per row: does the row hold an element in one of `cols`?"""
    mask = np.zeros(adj.shape[1], bool); mask[list(cols)] = True
    hit = np.zeros(adj.shape[0], bool)
    rows = np.repeat(np.arange(adj.shape[0]), np.diff(adj.indptr))
    hit[rows[mask[adj.indices]]] = True
    return hit


def _same_nonfinite(got, ref):
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    assert np.array_equal(np.isposinf(got), np.isposinf(ref))
    assert np.array_equal(np.isneginf(got), np.isneginf(ref))


@pytest.mark.parametrize("feat_len", [96, 128, 32, 6])
@pytest.mark.parametrize("P", [1, 3])
def test_spmm_nonfinite_rows_do_not_leak(oracle, feat_len, P):
    import torch
    from featgraph_amd.module import VanillaSpMMhip, placeholder
    rng = np.random.default_rng(feat_len * 10 + P)
    adj = _short_row_graph(rng)
    x = rng.standard_normal((adj.shape[1], feat_len)).astype("float32")
    xb = x.copy()
    for c, v in BAD.items():
        xb[c, :] = v
    m = VanillaSpMMhip(adj, P)
    m.build([placeholder(x.shape)], {}, {'num_src_partitions': None})
    clean = m.run([torch.from_numpy(x).cuda()]).cpu().numpy().copy()
    got = m.run([torch.from_numpy(xb).cuda()]).cpu().numpy().copy()
    text = m.lower_to_ir([placeholder(x.shape)], {}, {'num_src_partitions': None})
    assert "hold several rows" in text
    with np.errstate(invalid="ignore", over="ignore"):
        ref = oracle.spmm_csr_rowwise(adj.indptr, adj.indices, adj.data, xb)
    hit = _touching(adj, BAD)
    assert hit.sum() >= 6 and not np.isfinite(ref[hit]).all(axis=1).any()
    # rows that reference a bad source: same kind of non-finite value as the sequential sum
    _same_nonfinite(got[hit], ref[hit])
    # every other row: finite and bit-identical to the run on clean features
    assert np.isfinite(got[~hit]).all()
    assert np.array_equal(got[~hit], clean[~hit])


def test_spmm_inf_stays_inf_in_a_single_row():
    """A row that sums +Inf gives +Inf (not NaN) whether it is one item, shares an item or is split."""
    import torch
    from featgraph_amd.module import VanillaSpMMhip, placeholder
    n_cols = 4000
    x = np.ones((n_cols, 64), np.float32)
    x[5, :] = np.inf
    for length in (1, 3, 7, 17, 70, 300, 2500):
        cols = np.arange(5, 5 + length, dtype=np.int32)
        adj = sp.csr_matrix((np.ones(length, np.float32), cols, np.array([0, length], np.int32)), shape=(1, n_cols))
        m = VanillaSpMMhip(adj)
        m.build([placeholder(x.shape)], {}, {'num_src_partitions': None})
        out = m.run([torch.from_numpy(x).cuda()]).cpu().numpy()
        assert np.isposinf(out).all(), length


@pytest.mark.parametrize("H,D", [(4, 16), (2, 64)])
def test_per_head_weights_nonfinite_rows_do_not_leak(H, D):
    """The kernel tiles that hold several heads (own staged weight rows) take the same walk."""
    import torch
    from featgraph_amd.module import GSpMMhip, placeholder
    rng = np.random.default_rng(H + D)
    adj = _short_row_graph(rng)
    nnz = adj.nnz
    x = rng.standard_normal((adj.shape[1], H, D)).astype("float32")
    w = (rng.random((nnz, H)) + 0.1).astype("float32")
    xb = x.copy()
    for c, v in BAD.items():
        xb[c] = v
    m = GSpMMhip(adj)
    m.build([placeholder(x.shape), placeholder((nnz, H))], {'reduce': 'sum'}, {})
    wd = torch.from_numpy(w).cuda()
    clean = m.run([torch.from_numpy(x).cuda(), wd]).cpu().numpy().copy()
    got = m.run([torch.from_numpy(xb).cuda(), wd]).cpu().numpy().copy()
    hit = _touching(adj, BAD)
    assert not np.isfinite(got[hit]).all(axis=(1, 2)).any()
    assert np.isfinite(got[~hit]).all()
    assert np.array_equal(got[~hit], clean[~hit])


@pytest.mark.parametrize("D", [64, 16])
@pytest.mark.parametrize("P", [None, 3])
def test_attention_nonfinite_values_do_not_leak(oracle, D, P):
    import torch
    from featgraph_amd.module import GraphAttentionhip, placeholder
    rng = np.random.default_rng(D + (P or 0))
    adj = _short_row_graph(rng)
    H = 2
    q = rng.standard_normal((adj.shape[0], H, D)).astype("float32")
    k = rng.standard_normal((adj.shape[1], H, D)).astype("float32")
    v = rng.standard_normal((adj.shape[1], H, D)).astype("float32")
    vb = v.copy()
    for c, val in BAD.items():
        vb[c] = val
    m = GraphAttentionhip(adj)
    m.build([placeholder(q.shape), placeholder(k.shape), placeholder(v.shape)], {}, {'num_src_partitions': P})
    qd, kd = torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda()
    clean = m.run([qd, kd, torch.from_numpy(v).cuda()]).cpu().numpy().copy()
    got = m.run([qd, kd, torch.from_numpy(vb).cuda()]).cpu().numpy().copy()
    hit = _touching(adj, BAD)
    assert not np.isfinite(got[hit]).all(axis=(1, 2)).any()
    assert np.isfinite(got[~hit]).all()
    assert np.array_equal(got[~hit], clean[~hit])
    # a non-finite K row: the scores of the rows that reference it are non-finite, nothing else changes
    kb = k.copy()
    kb[222] = np.nan
    got = m.run([qd, torch.from_numpy(kb).cuda(), torch.from_numpy(v).cuda()]).cpu().numpy().copy()
    hit = _touching(adj, [222])
    assert np.isfinite(got[~hit]).all()
    assert np.array_equal(got[~hit], clean[~hit])


@pytest.mark.parametrize("reduce", ["max", "min"])
@pytest.mark.parametrize("P", [None, 3])
@pytest.mark.parametrize("return_arg", [False, True])
def test_extremes_propagate_nan(oracle, reduce, P, return_arg):
    """max / min of messages: a NaN message becomes the row's result (as it would through a sum, and as numpy's
    reductions do), the selected element is the row's first NaN message, a row of nothing but NaN messages gives NaN --
    in rows that lane groups walk on their own, in rows the wavefront shares, in the pieces of a split row, with one
    partition and with three, with and without the selected positions.  Rows that reference no NaN are bit-identical
    to a run on clean features."""
    import torch
    from featgraph_amd.module import GSpMMhip, placeholder
    rng = np.random.default_rng(5 + (P or 0))
    adj = _short_row_graph(rng)
    F = 32
    nnz = adj.nnz
    x = rng.standard_normal((adj.shape[1], F)).astype("float32")
    e = (rng.random((nnz, 1)) + 0.5).astype("float32")
    xb = x.copy()
    xb[222] = np.nan                                   # referenced by three short rows (see _short_row_graph)
    xb[1500, :7] = np.nan                              # some features only
    # every source of one short row and of one medium row: rows whose messages are all NaN
    lens = np.diff(adj.indptr)
    r_short = int(np.flatnonzero((lens >= 1) & (lens <= 3))[5])
    r_mid = int(np.flatnonzero((lens >= 20) & (lens < 100))[0])
    for r in (r_short, r_mid):
        xb[adj.indices[adj.indptr[r]:adj.indptr[r + 1]], 9] = np.nan
    # the split row: a NaN among its last elements (another piece than the one holding its first elements)
    xb[adj.indices[adj.indptr[701] - 3], 11] = np.nan
    m = GSpMMhip(adj)
    m.build([placeholder(x.shape), placeholder(e.shape)], {'msg': 'u_mul_e', 'reduce': reduce, 'return_arg': return_arg},
            {'num_src_partitions': P})
    assert m._active['P'] == (P or 1)
    ed = torch.from_numpy(e).cuda()
    clean = m.run([torch.from_numpy(x).cuda(), ed]).cpu().numpy().copy()
    got = m.run([torch.from_numpy(xb).cuda(), ed]).cpu().numpy().copy()
    want, want_arg = oracle.gspmm_bcast(adj.indptr, adj.indices, "mul", reduce, xb, e, "u", "e")
    assert np.array_equal(got, want, equal_nan=True)
    assert np.isnan(got[r_short, 9]) and np.isnan(got[r_mid, 9]) and np.isnan(got[700, 11])
    touched = np.isnan(want).any(axis=1)
    assert touched.sum() >= 5 and np.array_equal(got[~touched], clean[~touched])
    if return_arg:
        assert np.array_equal(m.arg_tvm.cpu().numpy(), want_arg)


@pytest.mark.parametrize("reduce", ["max", "min"])
def test_weighted_extremes_propagate_nan(oracle, reduce):
    """The same through the C ABI's weighted max / min (fg_gspmm_f32 / fg_gspmm_arg_f32: one weight per edge)."""
    import ctypes
    import torch
    from featgraph_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(8)
    adj = _short_row_graph(rng)
    F = 32
    x = rng.standard_normal((adj.shape[1], F)).astype("float32")
    x[222] = np.nan
    x[1500, :7] = np.nan
    x[adj.indices[adj.indptr[701] - 3], 11] = np.nan
    lens = np.diff(adj.indptr)
    r_mid = int(np.flatnonzero((lens >= 20) & (lens < 100))[0])
    x[adj.indices[adj.indptr[r_mid]:adj.indptr[r_mid + 1]], 9] = np.nan
    want, want_arg = oracle.gspmm_arg(adj.indptr, adj.indices, adj.data, x, reduce)
    indptr = np.ascontiguousarray(adj.indptr, dtype=np.int32)
    plan = ctypes.c_void_p()
    _lib.check(L.fg_spmm_plan_create(_lib.host_ptr(indptr), adj.shape[0], adj.shape[1], 1, None, ctypes.byref(plan)))
    try:
        ip, ix, vl, xd = (torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (indptr, adj.indices, adj.data, x))
        out = torch.full((adj.shape[0], F), 7.0, device="cuda")
        arg = torch.full((adj.shape[0], F), -5, dtype=torch.int32, device="cuda")
        p = _lib.dev_ptr
        red = {"max": 1, "min": 2}[reduce]
        _lib.check(L.fg_gspmm_arg_f32(plan, p(ip), p(ix), p(vl), p(xd), p(out), p(arg), F, 1, 0, red, 0, None))
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), want, equal_nan=True)
        assert np.array_equal(arg.cpu().numpy(), want_arg)
        out.fill_(7.0)
        _lib.check(L.fg_gspmm_f32(plan, p(ip), p(ix), p(vl), p(xd), p(out), F, 1, 0, red, 0, None))
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), want, equal_nan=True)
        assert np.isnan(want[r_mid, 9]) and np.isnan(want[700, 11])
    finally:
        L.fg_spmm_plan_destroy(plan)
