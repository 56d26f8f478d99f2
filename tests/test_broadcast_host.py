"""CPU checks of the host side of the broadcasting operators and of their numpy restatement.

The reference has no generalised SpMM / SDDMM (README.md:9-11 names them): parity is unpinned by it.  What pins
oracle.gspmm_bcast / gsddmm_bcast here: special cases that reduce to scipy sparse products in float64, to the
pinned restatements (oracle.gspmm, oracle.sddmm_f64) and to brute-force loops on small inputs.
"""
import numpy as np
import pytest
import scipy.sparse as sp

from featgraph_amd.module import general


def _adj(rng, n_rows=40, n_cols=55):
    a = sp.random(n_rows, n_cols, density=0.15, format="csr", random_state=rng,
                  data_rvs=lambda k: rng.standard_normal(k)).astype("float32").tolil()
    a[[0, 7], :] = 0
    a = a.tocsr().astype("float32"); a.sort_indices()
    return a


SHAPES = [((4,), (4,)), ((4,), (1,)), ((1,), (5,)), ((2, 3), (2, 1)), ((2, 1, 4), (3, 4)), ((3, 1), (1, 6)),
          ((), (3,)), ((2, 3, 4), (4,))]


@pytest.mark.parametrize("l_shape,r_shape", SHAPES)
def test_offset_arrays_are_numpy_broadcasting(l_shape, r_shape):
    out_shape, lo, ro, R = general.broadcast_plan(l_shape, r_shape)
    assert R == 1
    l = np.arange(int(np.prod(l_shape)) or 1, dtype=np.float64).reshape(l_shape or (1,)) + 100
    r = np.arange(int(np.prod(r_shape)) or 1, dtype=np.float64).reshape(r_shape or (1,)) + 500
    want = l - r                                     # not symmetric: a swapped pair of arrays fails
    assert tuple(want.shape) == out_shape
    n = want.size
    li = lo if lo is not None else np.arange(n)
    ri = ro if ro is not None else np.arange(n)
    assert np.array_equal(l.reshape(-1)[li] - r.reshape(-1)[ri], want.reshape(-1))


def test_offset_arrays_for_dot():
    out_shape, lo, ro, R = general.broadcast_plan((3, 1, 8), (5, 8), dot=True)
    assert out_shape == (3, 5) and R == 8
    l = np.random.default_rng(0).standard_normal((3, 1, 8)); r = np.random.default_rng(1).standard_normal((5, 8))
    want = (l * r).sum(-1)
    got = np.array([np.dot(l.reshape(-1, 8)[lo[f]], r.reshape(-1, 8)[ro[f]]) for f in range(15)])
    assert np.allclose(got, want.reshape(-1))
    assert general.broadcast_plan((8,), (8,), dot=True) == ((), None, None, 8)
    with pytest.raises(ValueError):
        general.broadcast_plan((2, 8), (2, 7), dot=True)
    with pytest.raises(ValueError):
        general.broadcast_plan((2, 8), (3, 8))


def test_vector_flags():
    """Which offset arrays let a lane read its 4 output features by one 128-bit load, or as one value 4 times."""
    def flags(l_shape, r_shape):
        out_shape, lo, ro, _ = general.broadcast_plan(l_shape, r_shape)
        n = int(np.prod(out_shape))
        return general.vector_flags(lo, n, 1, 2), general.vector_flags(ro, n, 4, 8)
    assert flags((4, 16), (4, 1)) == (0, 8)          # identity lhs needs no flag; one weight per head: splat
    assert flags((4, 16), (1, 16)) == (0, 4)         # the same 16 features for every head: consecutive
    assert flags((4, 2), (4, 1)) == (0, 0)           # 2-float heads: groups of 4 mix two weights
    assert flags((2, 1, 8), (3, 8)) == (1, 4)
    assert flags((3,), (1,)) == (0, 0)               # 3 outputs: no groups of 4
    assert flags((8, 1), (8, 12)) == (2, 0)


def test_message_names():
    assert general.parse_message("u_mul_e") == ("mul", "u", "e")
    assert general.parse_message("e_div_u") == ("div", "e", "u")
    assert general.parse_message("copy_e") == ("copy_lhs", "e", None)
    for bad in ("u_pow_e", "mul", "x_add_e", "copy_x"):
        with pytest.raises(ValueError):
            general.parse_message(bad)


def test_oracle_weighted_sum_is_the_scipy_product(oracle):
    rng = np.random.default_rng(3)
    adj = _adj(rng)
    x = rng.standard_normal((adj.shape[1], 6)).astype("float32")
    w = adj.data.reshape(-1, 1)
    out, arg = oracle.gspmm_bcast(adj.indptr, adj.indices, "mul", "sum", x, w, "u", "e")
    assert arg is None
    # every message is rounded to float32 before the float64 sum: equal within that rounding
    assert np.allclose(out, adj.astype(np.float64).dot(x.astype(np.float64)), rtol=1e-6, atol=1e-5)
    # operands swapped, same product
    out2, _ = oracle.gspmm_bcast(adj.indptr, adj.indices, "mul", "sum", w, x, "e", "u")
    assert np.allclose(out, out2, rtol=1e-12, atol=1e-12)
    # mean = sum / degree
    mean, _ = oracle.gspmm_bcast(adj.indptr, adj.indices, "mul", "mean", x, w, "u", "e")
    deg = np.maximum(np.diff(adj.indptr), 1)[:, None]
    assert np.allclose(mean, out / deg, rtol=1e-12, atol=1e-12)


def test_oracle_sum_of_edge_features_and_of_sums(oracle):
    """copy_e with ones counts the row's elements; u_add_e = (structure @ X) + row sums of the edge features;
    e_sub_u = -(u_sub_e)."""
    rng = np.random.default_rng(4)
    adj = _adj(rng)
    nnz = adj.nnz
    deg = np.diff(adj.indptr)
    out, _ = oracle.gspmm_bcast(adj.indptr, adj.indices, "copy_lhs", "sum", np.ones((nnz, 3), "float32"), None, "e", None)
    assert np.array_equal(out, np.repeat(deg[:, None], 3, 1))
    x = rng.standard_normal((adj.shape[1], 5)).astype("float32")
    ef = rng.standard_normal((nnz, 5)).astype("float32")
    structure = sp.csr_matrix((np.ones(nnz), adj.indices, adj.indptr), shape=adj.shape)
    rows = np.repeat(np.arange(adj.shape[0]), deg)
    edge_sums = sp.csr_matrix((np.ones(nnz), (rows, np.arange(nnz))), shape=(adj.shape[0], nnz)).dot(ef.astype(np.float64))
    # the oracle rounds each message to float32 before summing: compare within that rounding
    out, _ = oracle.gspmm_bcast(adj.indptr, adj.indices, "add", "sum", x, ef, "u", "e")
    assert np.allclose(out, structure.dot(x.astype(np.float64)) + edge_sums, rtol=1e-5, atol=1e-5)
    a, _ = oracle.gspmm_bcast(adj.indptr, adj.indices, "sub", "sum", x, ef, "u", "e")
    b, _ = oracle.gspmm_bcast(adj.indptr, adj.indices, "sub", "sum", ef, x, "e", "u")
    assert np.array_equal(a, -b)
    assert np.allclose(a, structure.dot(x.astype(np.float64)) - edge_sums, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("reduce", ["max", "min"])
def test_oracle_extremes_match_the_pinned_restatement_and_brute_force(oracle, reduce):
    rng = np.random.default_rng(5)
    adj = _adj(rng)
    x = rng.standard_normal((adj.shape[1], 2, 4)).astype("float32")
    w = adj.data.reshape(-1, 1, 1)
    out, arg = oracle.gspmm_bcast(adj.indptr, adj.indices, "mul", reduce, x, w, "u", "e")
    # oracle.gspmm / gspmm_arg: the C restatement pinned against numpy reduceat in tests/test_oracle.py
    ref, ref_arg = oracle.gspmm_arg(adj.indptr, adj.indices, adj.data, x.reshape(-1, 8), reduce)
    assert np.array_equal(out.reshape(-1, 8), ref)
    assert np.array_equal(arg.reshape(-1, 8), ref_arg)
    # brute force with division and broadcasting over a middle axis
    ef = (np.abs(rng.standard_normal((adj.nnz, 3, 1))) + 0.5).astype("float32")
    out, arg = oracle.gspmm_bcast(adj.indptr, adj.indices, "div", reduce, x[:, :1, :], ef, "u", "e")
    pick = max if reduce == "max" else min
    for v in (1, 5, 20, 39):
        es = range(adj.indptr[v], adj.indptr[v + 1])
        for i in range(3):
            for j in range(4):
                vals = [np.float32(x[adj.indices[e], 0, j]) / np.float32(ef[e, i, 0]) for e in es]
                if not vals:
                    assert out[v, i, j] == 0 and arg[v, i, j] == -1
                    continue
                best = pick(vals)
                assert out[v, i, j] == best
                assert arg[v, i, j] == adj.indptr[v] + vals.index(best)


def test_oracle_edge_operators(oracle):
    rng = np.random.default_rng(6)
    adj = _adj(rng).tocoo()
    row, col = adj.row, adj.col
    src = rng.standard_normal((adj.shape[1], 4, 8)).astype("float32")
    dst = rng.standard_normal((adj.shape[0], 4, 8)).astype("float32")
    # dot over the last axis = the pinned multi-head closed form; flat = the pinned vanilla closed form
    assert np.allclose(oracle.gsddmm_bcast(row, col, "dot", src, dst), oracle.sddmm_multihead_f64(row, col, src, dst),
                       rtol=1e-12, atol=1e-12)
    assert np.allclose(oracle.gsddmm_bcast(row, col, "dot", src.reshape(-1, 32), dst.reshape(-1, 32)),
                       oracle.sddmm_f64(row, col, src.reshape(-1, 32), dst.reshape(-1, 32)), rtol=1e-12, atol=1e-12)
    # operand pairing: lhs on 'u' is read at the edge's column, rhs on 'v' at its row (one-hot operands)
    lhs = np.zeros((adj.shape[1], 1), "float32"); lhs[col[3]] = 2
    rhs = np.zeros((adj.shape[0], 1), "float32"); rhs[row[3]] = 5
    out = oracle.gsddmm_bcast(row, col, "sub", lhs, rhs, "u", "v")
    assert out[3, 0] == -3 and out.shape == (adj.nnz, 1)
    assert np.array_equal(out[:, 0], lhs[col, 0] - rhs[row, 0])
    # element operands and broadcasting against a node operand
    ef = rng.standard_normal((adj.nnz, 4, 1)).astype("float32")
    out = oracle.gsddmm_bcast(row, col, "mul", ef, dst, "e", "v")
    assert out.shape == (adj.nnz, 4, 8)
    e = 11
    assert np.array_equal(out[e], ef[e] * dst[row[e]])
    assert np.array_equal(oracle.gsddmm_bcast(row, col, "copy_rhs", None, dst, "u", "v"), dst[row])
    # dot between operands of different rank: feature axes align to the right (brute force)
    a = rng.standard_normal((adj.shape[0], 2, 1, 4)).astype("float32")
    b = rng.standard_normal((adj.nnz, 5, 4)).astype("float32")
    out = oracle.gsddmm_bcast(row, col, "dot", a, b, "v", "e")
    assert out.shape == (adj.nnz, 2, 5)
    for e in (0, 17, adj.nnz - 1):
        for i in range(2):
            for j in range(5):
                want = sum(float(a[row[e], i, 0, k]) * float(b[e, j, k]) for k in range(4))
                assert abs(out[e, i, j] - want) < 1e-12
