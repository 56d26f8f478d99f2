"""Pins the CPU oracle before anything is compared with it (CPU only).

Each oracle function is checked against something it does not share code with:
the reference's stored vectors, scipy/numpy library routines (the reference's
own checks), exact special cases and brute force on tiny inputs.
"""
import itertools
import json
import os

import numpy as np
import pytest
import scipy.sparse as sp

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "util_5x5.json")


def _golden():
    with open(GOLDEN) as f:
        g = json.load(f)
    coo = sp.coo_matrix((np.array(g["data"], dtype="int32"), (g["row"], g["col"])),
                        shape=tuple(g["shape"]), dtype="int32")
    return g, coo


def _rand_csr(rng, n_rows, n_cols, density, dtype="float32"):
    a = sp.random(n_rows, n_cols, density=density, format="csr", random_state=rng,
                  data_rvs=lambda k: rng.random(k)).astype(dtype)
    a.sort_indices()
    return a


# ---- partitioners: stored vectors ---------------------------------------------------

def test_dds_golden(oracle):
    g, coo = _golden()
    s1_pos, s1_idx, vals = oracle.csr_to_dds(coo.tocsr(), g["dds_num_col_partitions"])
    assert vals.tolist() == g["dds_vals"]
    assert s1_idx.tolist() == g["dds_s1_idx"]
    assert s1_pos.tolist() == g["dds_s1_pos"]
    assert s1_pos.dtype == np.int32 and s1_idx.dtype == np.int32


def test_partition_2d_golden(oracle):
    g, coo = _golden()
    data_before = coo.data.copy()
    eid, row, col = oracle.partition_coo_2d(coo, g["part2d_num_row_partitions"],
                                            g["part2d_num_col_partitions"])
    assert eid.tolist() == g["part2d_edge_id_list"]
    # global ids of the permuted edges are the original edges' ids
    assert row.tolist() == [g["row"][i - 1] for i in eid]
    assert col.tolist() == [g["col"][i - 1] for i in eid]
    assert (coo.data == data_before).all()


# ---- partitioners: scipy sub-matrix slicing on random matrices ------------------------

def _dds_by_slicing(a, P):
    """Column slices through scipy's own sub-matrix routine."""
    n_rows, n_cols = a.shape
    c = -(-n_cols // P)
    pos, idx, vals, counter = [], [], [], 0
    for p in range(P):
        sub = a[:, p * c:] if p == P - 1 else a[:, p * c:(p + 1) * c]
        pos.append(sub.indptr + counter); idx.append(sub.indices); vals.append(sub.data)
        counter += sub.nnz
    return np.concatenate(pos), np.concatenate(idx), np.concatenate(vals)


@pytest.mark.parametrize("shape,P", [((127, 255), 4), ((127, 255), 1), ((64, 7), 3),
                                     ((5, 40), 7), ((33, 33), 33), ((9, 4), 6)])
def test_dds_vs_scipy_slicing(oracle, shape, P):
    rng = np.random.default_rng(11)
    a = _rand_csr(rng, shape[0], shape[1], 0.15)
    s1_pos, s1_idx, vals = oracle.csr_to_dds(a, P)
    epos, eidx, evals = _dds_by_slicing(a, P)
    np.testing.assert_array_equal(s1_pos, epos)
    np.testing.assert_array_equal(s1_idx, eidx)
    np.testing.assert_array_equal(vals, evals)


def _part2d_by_slicing(coo, R, C):
    n_rows, n_cols = coo.shape
    ids = sp.coo_matrix((np.arange(1, coo.nnz + 1, dtype="int32"), (coo.row, coo.col)),
                        shape=coo.shape).tocsr()
    rp, cp = -(-n_rows // R), -(-n_cols // C)
    eid, rows, cols = [], [], []
    for r in range(R):
        for c in range(C):
            rs = slice(r * rp, None if r == R - 1 else (r + 1) * rp)
            cs = slice(c * cp, None if c == C - 1 else (c + 1) * cp)
            blk = ids[rs, cs].tocoo()
            eid.append(blk.data); rows.append(blk.row + r * rp); cols.append(blk.col + c * cp)
    return np.concatenate(eid), np.concatenate(rows), np.concatenate(cols)


@pytest.mark.parametrize("shape,R,C", [((127, 255), 4, 4), ((127, 255), 1, 1), ((127, 255), 3, 5),
                                       ((20, 9), 7, 2), ((6, 6), 6, 6), ((5, 5), 4, 4)])
def test_partition_2d_vs_scipy_slicing(oracle, shape, R, C):
    rng = np.random.default_rng(5)
    coo = _rand_csr(rng, shape[0], shape[1], 0.2).tocoo()
    perm = rng.permutation(coo.nnz)            # arbitrary stored COO order
    coo = sp.coo_matrix((coo.data[perm], (coo.row[perm], coo.col[perm])), shape=coo.shape)
    eid, row, col = oracle.partition_coo_2d(coo, R, C)
    e2, r2, c2 = _part2d_by_slicing(coo, R, C)
    np.testing.assert_array_equal(eid, e2)
    np.testing.assert_array_equal(row, r2)
    np.testing.assert_array_equal(col, c2)
    # argsort of the ids is the inverse permutation (module/sddmm.py:49)
    mapping = np.argsort(eid)
    np.testing.assert_array_equal(row[mapping], coo.row)
    np.testing.assert_array_equal(col[mapping], coo.col)


def test_partitioners_bruteforce_tiny(oracle):
    """Every pattern on a 3x3 grid (512 matrices), every partition count up to 4."""
    cells = [(r, c) for r in range(3) for c in range(3)]
    for mask in range(1, 512):
        rc = [cells[i] for i in range(9) if mask >> i & 1]
        row = np.array([r for r, _ in rc], dtype="int32"); col = np.array([c for _, c in rc], dtype="int32")
        data = np.arange(1, len(rc) + 1, dtype="int32")
        coo = sp.coo_matrix((data, (row, col)), shape=(3, 3))
        csr = coo.tocsr()
        for P in (1, 2, 3, 4):
            s1_pos, s1_idx, vals = oracle.csr_to_dds(csr, P)
            c = -(-3 // P)
            d2 = 4
            assert s1_pos[-1] == len(rc)
            got = set()
            for p in range(P):
                pos = s1_pos[p * d2:(p + 1) * d2]
                assert (np.diff(pos) >= 0).all()
                for r in range(3):
                    for e in range(pos[r], pos[r + 1]):
                        got.add((r, int(s1_idx[e]) + p * c, int(vals[e])))
            assert got == {(r, c_, int(csr[r, c_])) for r, c_ in rc}
        for R, C in itertools.product((1, 2, 3), (1, 2, 3)):
            eid, orow, ocol = oracle.partition_coo_2d(coo, R, C)
            assert sorted(eid.tolist()) == list(range(1, len(rc) + 1))
            rp, cp = -(-3 // R), -(-3 // C)
            keys = [(orow[i] // rp, ocol[i] // cp, orow[i], ocol[i]) for i in range(len(rc))]
            assert keys == sorted(keys)
            assert [rc[i - 1] for i in eid] == list(zip(orow.tolist(), ocol.tolist()))


def test_partition_2d_rejects_duplicates(oracle):
    coo = sp.coo_matrix((np.ones(3, dtype="int32"), ([0, 0, 1], [1, 1, 0])), shape=(2, 2))
    with pytest.raises(RuntimeError):
        oracle.partition_coo_2d(coo, 2, 2)


# ---- SpMM restatements --------------------------------------------------------------

@pytest.mark.parametrize("T,P", [(1, 1), (4, 1), (1, 4), (4, 4), (128, 7)])
def test_spmm_reference_shape(oracle, T, P):
    """The reference's case: 127x255, density 0.1, F=128, csr.dot, rtol=atol=1e-4
    (tests/test_module_spmm.py:16-34, :63)."""
    rng = np.random.default_rng(0)
    a = _rand_csr(rng, 127, 255, 0.1)
    x = rng.random((255, 128)).astype("float32")
    expect = a.dot(x)
    if P == 1:
        out = oracle.spmm_csr_x86(a.indptr, a.indices, a.data, x, T, nthreads=2)
    else:
        s1_pos, s1_idx, vals = oracle.csr_to_dds(a, P)
        out = oracle.spmm_dds_x86(s1_pos, s1_idx, vals, x, 127, P, T, nthreads=2)
    np.testing.assert_allclose(out, expect, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(out, oracle.spmm_f64(a, x), rtol=1e-4, atol=1e-5)


def test_spmm_bit_invariance_and_special_cases(oracle):
    rng = np.random.default_rng(1)
    a = _rand_csr(rng, 200, 150, 0.05).tolil()
    a[[0, 17, 199], :] = 0                      # rows without any edge
    a = a.tocsr().astype("float32")
    a.eliminate_zeros()
    x = rng.standard_normal((150, 64)).astype("float32")
    base = oracle.spmm_csr_x86(a.indptr, a.indices, a.data, x, 1)
    for T in (2, 4, 16, 64):
        # feature tiling leaves each output element's summation order unchanged
        assert np.array_equal(base, oracle.spmm_csr_x86(a.indptr, a.indices, a.data, x, T, nthreads=3))
    assert np.array_equal(base, oracle.spmm_csr_rowwise(a.indptr, a.indices, a.data, x, nthreads=2))
    # one column partition == CSR
    s1_pos, s1_idx, vals = oracle.csr_to_dds(a, 1)
    assert np.array_equal(base, oracle.spmm_dds_x86(s1_pos, s1_idx, vals, x, 200, 1, 4))
    # empty rows are exact zeros
    empty = np.diff(a.indptr) == 0
    assert empty.any() and (base[empty] == 0).all()
    # identity adjacency copies X bit-exactly; a transposed operand would fail the shape
    eye = sp.identity(150, dtype="float32", format="csr")
    assert np.array_equal(oracle.spmm_csr_x86(eye.indptr, eye.indices, eye.data, x, 4), x)
    # a permutation matrix gathers rows: pins indices[] -> X row (not column) indexing
    perm = rng.permutation(150)
    pm = sp.csr_matrix((np.ones(150, "float32"), perm, np.arange(151)), shape=(150, 150))
    assert np.array_equal(oracle.spmm_csr_rowwise(pm.indptr, pm.indices, pm.data, x), x[perm])
    # linear in the edge weights
    twice = oracle.spmm_csr_x86(a.indptr, a.indices, 2 * a.data, x, 1)
    assert np.array_equal(twice, 2 * base)


def test_spmm_rejects_bad_feature_partition(oracle):
    a = sp.identity(4, dtype="float32", format="csr")
    with pytest.raises(RuntimeError):
        oracle.spmm_csr_x86(a.indptr, a.indices, a.data, np.ones((4, 6), "float32"), 4)


# ---- SDDMM restatements -------------------------------------------------------------

@pytest.mark.parametrize("T,par", [(1, False), (4, False), (4, True), (128, False)])
def test_sddmm_reference_shape(oracle, T, par):
    """127x255, density 0.1, F=128; Src is (num_cols, F) gathered by col, Dst is
    (num_rows, F) gathered by row (tests/test_module_sddmm.py:18-19, :34-37)."""
    rng = np.random.default_rng(2)
    coo = _rand_csr(rng, 127, 255, 0.1).tocoo()
    src = rng.random((255, 128)).astype("float32")
    dst = rng.random((127, 128)).astype("float32")
    expect = (src[coo.col] * dst[coo.row]).sum(axis=-1)
    out = oracle.sddmm_x86(coo.row, coo.col, src, dst, T, parallel_edges=par, nthreads=3)
    np.testing.assert_allclose(out, expect, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(out, oracle.sddmm_f64(coo.row, coo.col, src, dst), rtol=1e-4, atol=1e-5)


def test_sddmm_invariants(oracle):
    rng = np.random.default_rng(3)
    coo = _rand_csr(rng, 90, 90, 0.1).tocoo()
    src = rng.standard_normal((90, 32)).astype("float32")
    dst = rng.standard_normal((90, 32)).astype("float32")
    base = oracle.sddmm_x86(coo.row, coo.col, src, dst)
    for T in (2, 8, 32):
        assert np.array_equal(base, oracle.sddmm_x86(coo.row, coo.col, src, dst, T))
    assert np.array_equal(base, oracle.sddmm_x86(coo.row, coo.col, src, dst, 1, True, 4))
    # swapping (Src, col) with (Dst, row) is the same product
    assert np.array_equal(base, oracle.sddmm_x86(coo.col, coo.row, dst, src))
    # one-hot operands pick single entries: pins which index gathers which operand
    n = 6
    row = np.array([0, 1, 5], "int32"); col = np.array([2, 2, 4], "int32")
    s = np.zeros((n, n), "float32"); d = np.zeros((n, n), "float32")
    s[np.arange(n), np.arange(n)] = np.arange(1, n + 1)      # src[c] = (c+1) e_c
    d[:] = 1.0
    assert oracle.sddmm_x86(row, col, s, d).tolist() == [3.0, 3.0, 5.0]


def test_multihead_closed_form(oracle):
    rng = np.random.default_rng(4)
    coo = _rand_csr(rng, 80, 120, 0.1).tocoo()
    for H, D in ((1, 32), (4, 32), (8, 64), (3, 5)):
        src = rng.standard_normal((120, H, D)).astype("float32")
        dst = rng.standard_normal((80, H, D)).astype("float32")
        out = oracle.sddmm_multihead(coo.row, coo.col, src, dst, nthreads=2)
        expect = np.einsum("ehd,ehd->eh", src[coo.col].astype("f8"), dst[coo.row].astype("f8"))
        np.testing.assert_allclose(out, expect, rtol=1e-4, atol=1e-5)
        np.testing.assert_allclose(oracle.sddmm_multihead_f64(coo.row, coo.col, src, dst), expect)
        flat = oracle.sddmm_x86(coo.row, coo.col, src.reshape(120, -1), dst.reshape(80, -1))
        np.testing.assert_allclose(out.sum(1), flat, rtol=1e-4, atol=1e-4)
        if H == 1:
            assert np.array_equal(out[:, 0], flat)


def test_gspmm_closed_forms(oracle):
    """Max / min / per-head aggregation (no counterpart in the reference): numpy reduceat over
    the gathered messages, sum with one head == the plain SpMM restatement, empty rows give 0."""
    rng = np.random.default_rng(9)
    a = _rand_csr(rng, 60, 80, 0.15).tolil()
    a[[3, 59], :] = 0
    a = a.tocsr().astype("float32"); a.eliminate_zeros(); a.sort_indices()
    nonempty = np.diff(a.indptr) > 0
    starts = a.indptr[:-1][nonempty]
    for H, D in ((1, 24), (4, 16), (3, 5)):
        x = rng.standard_normal((80, H, D)).astype("float32")
        w = rng.standard_normal((a.nnz, H)).astype("float32")
        msg = w[:, :, None] * x[a.indices]
        for red, fn in (("max", np.maximum), ("min", np.minimum), ("sum", np.add)):
            expect = np.zeros((60, H, D), "float32")
            expect[nonempty] = fn.reduceat(msg, starts, axis=0)
            got = oracle.gspmm(a.indptr, a.indices, w, x, red, nthreads=2)
            if red == "sum":
                np.testing.assert_allclose(got, expect, rtol=1e-4, atol=1e-5)
            else:
                assert np.array_equal(got, expect)
            assert (got[~nonempty] == 0).all()
        plain = oracle.gspmm(a.indptr, a.indices, None, x, "max")
        e2 = np.zeros((60, H, D), "float32"); e2[nonempty] = np.maximum.reduceat(x[a.indices], starts, axis=0)
        assert np.array_equal(plain, e2)
    x = rng.standard_normal((80, 24)).astype("float32")
    assert np.array_equal(oracle.gspmm(a.indptr, a.indices, a.data, x, "sum"),
                          oracle.spmm_csr_rowwise(a.indptr, a.indices, a.data, x))


# ---- edge softmax (not in the reference: pinned by library routines and invariants) ---------

def _ragged_indptr(rng, n_rows, max_len):
    lens = rng.integers(0, max_len, size=n_rows)
    lens[::7] = 0                       # empty rows
    lens[3] = 1                         # a one-element row
    lens[5] = 4 * max_len               # a long row
    return np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)


@pytest.mark.parametrize("H", [1, 3, 4])
def test_edge_softmax_closed_forms(oracle, H):
    import scipy.special
    rng = np.random.default_rng(11 + H)
    indptr = _ragged_indptr(rng, 60, 40)
    nnz = int(indptr[-1])
    x = (rng.standard_normal((nnz, H)) * 3).astype(np.float32)
    got = oracle.edge_softmax(indptr, x)
    np.testing.assert_allclose(got, oracle.edge_softmax_f64(indptr, x), rtol=2e-6, atol=1e-7)
    # dense masked softmax through scipy on the whole matrix at once (a second, differently shaped route)
    for h in range(H):
        dense = np.full((60, int(np.diff(indptr).max())), -np.inf)
        for r in range(60):
            dense[r, :indptr[r + 1] - indptr[r]] = x[indptr[r]:indptr[r + 1], h]
        with np.errstate(invalid="ignore"):
            sm = scipy.special.softmax(dense, axis=1)
        for r in range(60):
            np.testing.assert_allclose(got[indptr[r]:indptr[r + 1], h], sm[r, :indptr[r + 1] - indptr[r]],
                                       rtol=2e-6, atol=1e-7)
    # every non-empty row sums to one per head; a one-element row is exactly one
    sums = np.add.reduceat(got.astype(np.float64), indptr[:-1][np.diff(indptr) > 0], axis=0)
    np.testing.assert_allclose(sums, 1.0, rtol=0, atol=1e-5)
    assert np.all(got[indptr[3]:indptr[4]] == 1.0)
    # adding a per-row, per-head constant changes nothing beyond rounding; large inputs do not overflow
    shift = np.repeat(rng.standard_normal((60, H)).astype(np.float32) * 50, np.diff(indptr), axis=0)
    np.testing.assert_allclose(oracle.edge_softmax(indptr, x + shift), got, rtol=2e-4, atol=1e-6)
    assert np.isfinite(oracle.edge_softmax(indptr, x * 1e4)).all()
    # 1-D input is the one-head case
    if H == 1:
        assert np.array_equal(oracle.edge_softmax(indptr, x[:, 0]), got[:, 0])


def test_edge_softmax_backward_closed_forms(oracle):
    import torch
    rng = np.random.default_rng(5)
    H = 2
    indptr = _ragged_indptr(rng, 30, 12)
    nnz = int(indptr[-1])
    x = rng.standard_normal((nnz, H)).astype(np.float32)
    g = rng.standard_normal((nnz, H)).astype(np.float32)
    a = oracle.edge_softmax(indptr, x)
    got = oracle.edge_softmax_backward(indptr, a, g)
    # float64 autograd of torch.softmax applied row by row
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    pieces = [torch.softmax(xt[indptr[r]:indptr[r + 1]], dim=0) for r in range(30) if indptr[r + 1] > indptr[r]]
    (torch.cat(pieces) * torch.tensor(g, dtype=torch.float64)).sum().backward()
    np.testing.assert_allclose(got, xt.grad.numpy(), rtol=1e-4, atol=1e-6)
    # central finite differences of the float64 closed form, a few coordinates
    def loss(xx):
        return float((oracle.edge_softmax_f64(indptr, xx) * g).sum())
    for (e, h) in [(0, 0), (int(indptr[5]) + 3, 1), (nnz - 1, 0)]:
        xp = x.astype(np.float64).copy(); xm = xp.copy()
        xp[e, h] += 1e-5; xm[e, h] -= 1e-5
        np.testing.assert_allclose(got[e, h], (loss(xp) - loss(xm)) / 2e-5, rtol=1e-3, atol=1e-6)
    # the gradient of each row sums to zero per head (softmax is shift-invariant)
    rows = indptr[:-1][np.diff(indptr) > 0]
    np.testing.assert_allclose(np.add.reduceat(got.astype(np.float64), rows, axis=0), 0.0, atol=1e-6)


def test_gspmm_arg_closed_form(oracle):
    """Selected elements of max / min aggregation against numpy argmax / argmin over the gathered
    messages (both return the first occurrence), with repeated values so that ties occur."""
    rng = np.random.default_rng(21)
    adj = _rand_csr(rng, 40, 60, 0.2).tolil()
    adj[[0, 17], :] = 0
    adj = adj.tocsr().astype("float32"); adj.eliminate_zeros(); adj.sort_indices()
    adj.data = rng.integers(-2, 3, size=adj.nnz).astype("float32")          # few distinct weights
    x = rng.integers(-3, 4, size=(60, 6)).astype("float32")                  # few distinct values: many ties
    for reduce, pick in (("max", np.argmax), ("min", np.argmin)):
        out, arg = oracle.gspmm_arg(adj.indptr, adj.indices, adj.data, x, reduce)
        assert np.array_equal(out, oracle.gspmm(adj.indptr, adj.indices, adj.data, x, reduce))
        for r in range(40):
            b, e = adj.indptr[r], adj.indptr[r + 1]
            if e == b:
                assert (arg[r] == -1).all() and (out[r] == 0).all()
                continue
            msgs = adj.data[b:e, None] * x[adj.indices[b:e]]
            assert np.array_equal(arg[r], b + pick(msgs, axis=0))
            assert np.array_equal(out[r], msgs[arg[r] - b, np.arange(6)])


# ---- attention in one operator: the dense masked form ---------------------------------

def _dense_attention(adj, scores, v):
    """softmax over each row's stored columns of a dense [H, n_dst, n_src] score array, times V, with torch in
    float64; rows without stored columns give 0."""
    import torch
    mask = torch.from_numpy(adj.toarray() != 0)
    s = torch.from_numpy(scores).masked_fill(~mask[None], float("-inf"))
    a = torch.nan_to_num(torch.softmax(s, dim=2), nan=0.0)          # rows of -inf only: nan -> 0
    return torch.einsum("hvu,uhd->vhd", a, torch.from_numpy(np.asarray(v, dtype=np.float64))).numpy()


def test_graph_attention_dense_form(oracle):
    rng = np.random.default_rng(21)
    adj = _rand_csr(rng, 23, 31, 0.2)
    adj = adj.tolil(); adj[4, :] = 0; adj[9, :] = 1; adj = adj.tocsr(); adj.eliminate_zeros(); adj.sort_indices()
    H, D = 3, 8
    q = rng.standard_normal((23, H, D)); k = rng.standard_normal((31, H, D)); v = rng.standard_normal((31, H, D))
    scale = 0.37
    got = oracle.graph_attention_f64(adj.indptr, adj.indices, q.astype("float32"), k.astype("float32"),
                                     v.astype("float32"), scale)
    f32 = lambda a: a.astype("float32").astype(np.float64)
    ref = _dense_attention(adj, scale * np.einsum("vhd,uhd->hvu", f32(q), f32(k)), f32(v))
    np.testing.assert_allclose(got, ref, rtol=1e-12, atol=1e-13)
    assert (got[4] == 0).all()
    # one stored column: the output is that column's V, whatever the scores
    one = sp.csr_matrix((np.ones(1), ([0], [5])), shape=(1, 31))
    np.testing.assert_allclose(oracle.graph_attention_f64(one.indptr, one.indices, q[:1], k, v, 5.0)[0], v[5], rtol=1e-14)
    # swapping the roles of two heads permutes the output's heads (catches a head mixed into another)
    perm = [2, 0, 1]
    swapped = oracle.graph_attention_f64(adj.indptr, adj.indices, q[:, perm], k[:, perm], v[:, perm], scale)
    np.testing.assert_allclose(swapped, oracle.graph_attention_f64(adj.indptr, adj.indices, q, k, v, scale)[:, perm], rtol=1e-13)


def test_graph_attention_additive_dense_form(oracle):
    rng = np.random.default_rng(22)
    adj = _rand_csr(rng, 19, 27, 0.25)
    adj = adj.tolil(); adj[2, :] = 0; adj = adj.tocsr(); adj.eliminate_zeros(); adj.sort_indices()
    H, D = 4, 6
    er = rng.standard_normal((19, H)); el = rng.standard_normal((27, H)); v = rng.standard_normal((27, H, D))
    slope = 0.2
    got = oracle.graph_attention_additive_f64(adj.indptr, adj.indices, er, el, v, slope)
    z = el.T[:, None, :] + er.T[:, :, None]                          # [H, n_dst, n_src]
    ref = _dense_attention(adj, np.maximum(z, 0) + slope * np.minimum(z, 0), v)
    np.testing.assert_allclose(got, ref, rtol=1e-12, atol=1e-13)
    assert (got[2] == 0).all()
    # a shift of er moves every score of a row on the positive side by the same amount: nothing changes there
    pos = oracle.graph_attention_additive_f64(adj.indptr, adj.indices, er + 50.0, np.abs(el), v, slope)
    pos2 = oracle.graph_attention_additive_f64(adj.indptr, adj.indices, er + 70.0, np.abs(el), v, slope)
    np.testing.assert_allclose(pos, pos2, rtol=1e-9)
    # slope 1 makes the score el + er, and er cancels in the softmax
    lin = oracle.graph_attention_additive_f64(adj.indptr, adj.indices, er, el, v, 1.0)
    lin0 = oracle.graph_attention_additive_f64(adj.indptr, adj.indices, np.zeros_like(er), el, v, 1.0)
    np.testing.assert_allclose(lin, lin0, rtol=1e-9, atol=1e-12)


def test_timing_copies_stay_within_tolerance_of_the_pinned_loops(oracle):
    """orcf_* (fused multiply-add, AVX-512 clones) are what bench.py times beside the pinned loops; they
    pin nothing themselves and only have to agree with the pinned functions within the fp32 bar."""
    rng = np.random.default_rng(77)
    a = sp.random(300, 500, density=0.08, format="csr", random_state=rng).astype("float32")
    a.sort_indices()
    for F, T in ((64, 1), (64, 4), (96, 3), (7, 1)):
        x = rng.standard_normal((500, F)).astype("float32")
        y = rng.standard_normal((300, F)).astype("float32")
        ref = oracle.spmm_csr_x86(a.indptr, a.indices, a.data, x, T, 2)
        np.testing.assert_allclose(oracle.spmm_csr_x86(a.indptr, a.indices, a.data, x, T, 2, fast=True), ref,
                                   rtol=1e-4, atol=1e-5)
        for P in (1, 3):
            s1_pos, s1_idx, vals = oracle.csr_to_dds(a, P)
            ref = oracle.spmm_dds_x86(s1_pos, s1_idx, vals, x, 300, P, T, 2)
            np.testing.assert_allclose(oracle.spmm_dds_x86(s1_pos, s1_idx, vals, x, 300, P, T, 2, fast=True), ref,
                                       rtol=1e-4, atol=1e-5)
        coo = a.tocoo()
        ref = oracle.sddmm_x86(coo.row, coo.col, x, y, T)
        for par in (False, True):
            np.testing.assert_allclose(oracle.sddmm_x86(coo.row, coo.col, x, y, T, par, 3, fast=True), ref,
                                       rtol=1e-4, atol=1e-5)
    empty = sp.csr_matrix((5, 9), dtype="float32")
    x = rng.standard_normal((9, 8)).astype("float32")
    assert (oracle.spmm_csr_x86(empty.indptr, empty.indices, empty.data, x, 2, 2, fast=True) == 0).all()


def test_gspmm_extremes_propagate_nan(oracle):
    """max / min aggregation treats a NaN message as numpy's maximum / minimum reductions and argmax / argmin do: it
    becomes the row's result, and the selected element is the row's first NaN message -- in the C restatement and in
    the numpy restatement of the broadcasting operator alike.  Rows of all-NaN messages give NaN, not an identity."""
    rng = np.random.default_rng(22)
    adj = _rand_csr(rng, 50, 40, 0.25).tolil()
    adj[[3, 30], :] = 0
    adj = adj.tocsr().astype("float32"); adj.eliminate_zeros(); adj.sort_indices()
    adj.data = (rng.random(adj.nnz) + 0.5).astype("float32")
    x = rng.standard_normal((40, 5)).astype("float32")
    x[7] = np.nan                    # a whole source row
    x[21, 2] = np.nan                # one feature of another
    x[33] = np.inf
    indptr, indices = adj.indptr, adj.indices
    # a row whose messages are all NaN: every source it references is made NaN in column 4
    r_all = int(np.argmax(np.diff(indptr) > 0))
    x[indices[indptr[r_all]:indptr[r_all + 1]], 4] = np.nan
    rows = np.flatnonzero(np.diff(indptr) > 0)
    msgs = adj.data[:, None] * x[indices]
    for reduce, ufunc, pick in (("max", np.maximum, np.argmax), ("min", np.minimum, np.argmin)):
        want = np.zeros((50, 5), np.float32)
        want[rows] = ufunc.reduceat(msgs, indptr[rows], axis=0)
        out, arg = oracle.gspmm_arg(indptr, indices, adj.data, x, reduce)
        assert np.array_equal(out, want, equal_nan=True)
        assert np.array_equal(oracle.gspmm(indptr, indices, adj.data, x, reduce), want, equal_nan=True)
        out_b, arg_b = oracle.gspmm_bcast(indptr, indices, "mul", reduce, x, adj.data.reshape(-1, 1), "u", "e")
        assert np.array_equal(out_b, want, equal_nan=True)
        for r in rows:
            b, e = indptr[r], indptr[r + 1]
            assert np.array_equal(arg[r], b + pick(msgs[b:e], axis=0))           # numpy: the first NaN wins
            assert np.array_equal(arg_b[r], arg[r])
        assert np.isnan(out[r_all, 4]) and arg[r_all, 4] == indptr[r_all]
        assert np.isnan(want).any() and np.isfinite(want).any()
