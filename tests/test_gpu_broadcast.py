"""GPU tests of the generalised SpMM / SDDMM with broadcasting (vector edge features, operands on u / v / e).

The reference has no such operators (README.md:9-11 names them), so parity is unpinned by it.  The GPU
results are compared with the numpy restatement (oracle.gspmm_bcast / gsddmm_bcast), which
tests/test_broadcast_host.py pins through special cases that reduce to scipy products and to the pinned
operators.  Element-wise operators, max / min and the selected positions are exact (one correctly rounded
float32 operation per message); sums meet the fp32 bar (rel 1e-4 / abs 1e-5 plus 8 eps32 of the summed mass).
"""
import numpy as np
import pytest
import scipy.sparse as sp

from helpers import RTOL, ATOL, assert_sum_close

pytestmark = pytest.mark.gpu


def _graph(rng, n_rows=260, n_cols=700, long_len=2700 // 4):
    """Short rows, empty rows, and one row beyond the split threshold when long_len is large enough."""
    a = sp.random(n_rows, n_cols, density=0.03, format="csr", random_state=rng,
                  data_rvs=lambda k: rng.standard_normal(k)).astype("float32").tolil()
    a[[0, n_rows // 2, n_rows - 1], :] = 0
    cols = rng.choice(n_cols, size=long_len, replace=False)
    a[5, cols] = 1.0
    a = a.tocsr().astype("float32"); a.sort_indices()
    return a


def _hub_graph(rng):
    return _graph(rng, n_rows=150, n_cols=3000, long_len=2700)


def _operand(rng, rows, shape, positive=False):
    x = rng.standard_normal((rows,) + tuple(shape)).astype("float32")
    return (np.abs(x) + 0.5).astype("float32") if positive else x


def _run_spmm(adj, msg, reduce, arrays, return_arg=False, partitions=None):
    """partitions: None = the CSR arrays as they are (these graphs are too small for the default to partition them);
    an int = that many source-column partitions."""
    import torch
    from featgraph_amd.module import GSpMMhip, placeholder
    m = GSpMMhip(adj)
    args = {'reduce': reduce, 'msg': msg}
    if return_arg:
        args['return_arg'] = True
    m.build([placeholder(a.shape) for a in arrays], args, {'num_src_partitions': partitions})
    assert m._active['P'] == (partitions or 1)
    m.out_tvm.fill_(float("nan"))
    out = m.run([torch.from_numpy(a).cuda() for a in arrays]).cpu().numpy()
    return (out, m.arg_tvm.cpu().numpy()) if return_arg else out


CASES = [
    # msg, lhs feature shape, rhs feature shape
    ("u_mul_e", (96,), (96,)),
    ("u_mul_e", (4, 16), (4, 1)),
    ("u_mul_e", (4, 16), (1, 16)),
    ("u_mul_e", (4, 2), (4, 1)),       # groups of 4 outputs that are neither consecutive nor equal in the edge operand
    ("e_add_u", (8, 1), (8, 12)),
    ("u_add_e", (64,), (64,)),
    ("u_add_e", (3,), (1,)),
    ("u_sub_e", (1,), (7,)),
    ("e_sub_u", (130,), (130,)),
    ("u_div_e", (32,), (32,)),
    ("e_div_u", (2, 1, 8), (3, 8)),
    ("e_mul_u", (256,), (256,)),       # 128 features and more, in multiples of 64: feature tiles over the workgroups
    ("u_mul_e", (2, 64), (2, 64)),
    ("u_add_e", (192,), (1,)),
    ("u_mul_e", (8, 64), (8, 1)),
    ("copy_e", (40,), None),
    ("copy_e", (1,), None),
    ("copy_e", (2, 50), None),
]


def _arrays(rng, adj, msg, l_shape, r_shape):
    from featgraph_amd.module.general import parse_message
    op, lt, rt = parse_message(msg)
    rows = {'u': adj.shape[1], 'e': adj.nnz}
    lhs = _operand(rng, rows[lt], l_shape, positive=(op == 'div'))
    rhs = _operand(rng, rows[rt], r_shape, positive=(op == 'div')) if rt is not None else None
    return op, lt, rt, lhs, rhs


@pytest.mark.parametrize("reduce", ["sum", "mean"])
@pytest.mark.parametrize("msg,l_shape,r_shape", CASES)
@pytest.mark.parametrize("hub", [False, True])
def test_gspmm_broadcast_sum(oracle, msg, l_shape, r_shape, reduce, hub):
    rng = np.random.default_rng(len(msg) + sum(l_shape) + (7 if hub else 0))
    adj = _hub_graph(rng) if hub else _graph(rng)
    op, lt, rt, lhs, rhs = _arrays(rng, adj, msg, l_shape, r_shape)
    arrays = [lhs] + ([rhs] if rhs is not None else [])
    out = _run_spmm(adj, msg, reduce, arrays)
    ref, _ = oracle.gspmm_bcast(adj.indptr, adj.indices, op, reduce, lhs, rhs, lt, rt or 'e')
    mass, _ = oracle.gspmm_bcast(adj.indptr, adj.indices, op, reduce,
                                 np.abs(lhs), None if rhs is None else np.abs(rhs), lt, rt or 'e')
    if op == 'sub':      # |l - r| <= |l| + |r|
        mass, _ = oracle.gspmm_bcast(adj.indptr, adj.indices, 'add', reduce, np.abs(lhs), np.abs(rhs), lt, rt)
    assert out.shape == ref.shape
    assert_sum_close(out, ref, mass, "%s %s" % (msg, reduce))
    assert (out[np.diff(adj.indptr) == 0] == 0).all()


@pytest.mark.parametrize("reduce", ["max", "min"])
@pytest.mark.parametrize("msg,l_shape,r_shape", CASES)
def test_gspmm_broadcast_extreme_is_exact(oracle, msg, l_shape, r_shape, reduce):
    rng = np.random.default_rng(len(msg) * 3 + sum(l_shape))
    adj = _hub_graph(rng)
    op, lt, rt, lhs, rhs = _arrays(rng, adj, msg, l_shape, r_shape)
    arrays = [lhs] + ([rhs] if rhs is not None else [])
    out = _run_spmm(adj, msg, reduce, arrays)
    ref, ref_arg = oracle.gspmm_bcast(adj.indptr, adj.indices, op, reduce, lhs, rhs, lt, rt or 'e')
    assert np.array_equal(out, ref), (msg, reduce)
    out2, arg = _run_spmm(adj, msg, reduce, arrays, return_arg=True)
    assert np.array_equal(out2, ref)
    assert np.array_equal(arg, ref_arg)


@pytest.mark.parametrize("reduce", ["sum", "mean"])
@pytest.mark.parametrize("msg,l_shape,r_shape", CASES)
@pytest.mark.parametrize("partitions", [2, 5])
def test_gspmm_broadcast_sum_over_source_partitions(oracle, msg, l_shape, r_shape, reduce, partitions):
    """The same messages with the source columns cut into partitions (2: the hub row's segments are still split into
    pieces; 5: most segments are empty): operands on the edges stay in CSR order."""
    rng = np.random.default_rng(len(msg) + sum(l_shape) + partitions)
    adj = _hub_graph(rng)
    op, lt, rt, lhs, rhs = _arrays(rng, adj, msg, l_shape, r_shape)
    arrays = [lhs] + ([rhs] if rhs is not None else [])
    out = _run_spmm(adj, msg, reduce, arrays, partitions=partitions)
    ref, _ = oracle.gspmm_bcast(adj.indptr, adj.indices, op, reduce, lhs, rhs, lt, rt or 'e')
    mass, _ = oracle.gspmm_bcast(adj.indptr, adj.indices, 'add' if op == 'sub' else op, reduce,
                                 np.abs(lhs), None if rhs is None else np.abs(rhs), lt, rt or 'e')
    assert out.shape == ref.shape
    assert_sum_close(out, ref, mass, "%s %s P=%d" % (msg, reduce, partitions))
    assert (out[np.diff(adj.indptr) == 0] == 0).all()


@pytest.mark.parametrize("reduce", ["max", "min"])
@pytest.mark.parametrize("msg,l_shape,r_shape", CASES)
@pytest.mark.parametrize("partitions", [2, 5])
def test_gspmm_broadcast_extreme_over_source_partitions_is_exact(oracle, msg, l_shape, r_shape, reduce, partitions):
    rng = np.random.default_rng(len(msg) * 3 + sum(l_shape) + partitions)
    adj = _hub_graph(rng)
    op, lt, rt, lhs, rhs = _arrays(rng, adj, msg, l_shape, r_shape)
    arrays = [lhs] + ([rhs] if rhs is not None else [])
    ref, ref_arg = oracle.gspmm_bcast(adj.indptr, adj.indices, op, reduce, lhs, rhs, lt, rt or 'e')
    out = _run_spmm(adj, msg, reduce, arrays, partitions=partitions)
    assert np.array_equal(out, ref), (msg, reduce)
    out2, arg = _run_spmm(adj, msg, reduce, arrays, return_arg=True, partitions=partitions)
    assert np.array_equal(out2, ref)
    assert np.array_equal(arg, ref_arg)          # positions in the caller's CSR order
    assert (out[np.diff(adj.indptr) == 0] == 0).all() and (arg[np.diff(adj.indptr) == 0] == -1).all()


def test_source_partitions_with_unsorted_columns_and_ties(oracle):
    """Rows whose columns are not stored in ascending order: a partition's elements are then not consecutive in the
    CSR arrays, and the first stored one among equal candidates may lie in a later partition."""
    rng = np.random.default_rng(21)
    adj = _hub_graph(rng)
    indices = adj.indices.copy()
    perm = np.arange(adj.nnz)
    for r in range(adj.shape[0]):
        lo, hi = adj.indptr[r], adj.indptr[r + 1]
        perm[lo:hi] = lo + rng.permutation(hi - lo)
    shuffled = sp.csr_matrix((adj.data[perm], indices[perm], adj.indptr), shape=adj.shape)
    assert not shuffled.has_sorted_indices
    lhs = rng.integers(0, 3, size=(adj.shape[1], 8)).astype("float32")
    rhs = rng.integers(0, 3, size=(adj.nnz, 1)).astype("float32")
    for reduce in ("max", "min"):
        out, arg = _run_spmm(shuffled, "u_add_e", reduce, [lhs, rhs], return_arg=True, partitions=4)
        ref, ref_arg = oracle.gspmm_bcast(shuffled.indptr, shuffled.indices, "add", reduce, lhs, rhs, 'u', 'e')
        assert np.array_equal(out, ref)
        assert np.array_equal(arg, ref_arg)
    out = _run_spmm(shuffled, "u_mul_e", "sum", [lhs, rhs], partitions=4)
    ref, _ = oracle.gspmm_bcast(shuffled.indptr, shuffled.indices, "mul", "sum", lhs, rhs, 'u', 'e')
    assert np.array_equal(out, ref)              # small integers: every sum is exact in any order


@pytest.mark.parametrize("partitions", [None, 3])
def test_edge_operands_in_another_order(oracle, partitions):
    """set_weight_order: the edge operands given to run() lie in another edge order (as those of the transposed graph's
    calls do); the kernel follows the positions, and the positions it reports refer to the given order."""
    import torch
    from featgraph_amd.module import GSpMMhip, placeholder
    rng = np.random.default_rng(31)
    adj = _hub_graph(rng)
    nnz = adj.nnz
    where = rng.permutation(nnz)                           # edge i of the adjacency lies at where[i] in the given arrays
    x = _operand(rng, adj.shape[1], (8, 4))
    ef_csr = _operand(rng, nnz, (8, 1))
    given = np.empty_like(ef_csr); given[where] = ef_csr
    for reduce in ("sum", "max"):
        m = GSpMMhip(adj)
        args = {'msg': 'u_mul_e', 'reduce': reduce}
        if reduce == "max":
            args['return_arg'] = True
        m.build([placeholder(x.shape), placeholder(given.shape)], args, {'num_src_partitions': partitions})
        m.set_weight_order(where)
        out = m.run([torch.from_numpy(x).cuda(), torch.from_numpy(given).cuda()]).cpu().numpy()
        ref, ref_arg = oracle.gspmm_bcast(adj.indptr, adj.indices, 'mul', reduce, x, ef_csr, 'u', 'e')
        if reduce == "sum":
            mass, _ = oracle.gspmm_bcast(adj.indptr, adj.indices, 'mul', reduce, np.abs(x), np.abs(ef_csr), 'u', 'e')
            assert_sum_close(out, ref, mass, "given order, sum")
        else:
            assert np.array_equal(out, ref)
            arg = m.arg_tvm.cpu().numpy()
            # the same values are selected; among equal candidates the one that comes first in the given order
            picked = np.where(arg >= 0, np.argsort(where)[np.maximum(arg, 0)], -1)
            rows = np.repeat(np.arange(adj.shape[0]), np.diff(adj.indptr))
            assert ((arg >= 0) == (ref_arg >= 0)).all()
            ok = arg >= 0
            assert (rows[picked[ok]] == np.nonzero(ok)[0]).all()          # an edge of the output's own row
            msgs = x[adj.indices[picked[ok]]] * ef_csr[picked[ok]]
            f = np.nonzero(ok)[1:]
            assert np.array_equal(msgs.reshape(msgs.shape[0], -1)[np.arange(msgs.shape[0]), np.ravel_multi_index(f, (8, 4))], out[ok])


def test_selected_position_with_ties(oracle):
    """Integer-valued messages: many equal candidates per row, the first stored one is reported (also across
    the lane groups that share a row and across the pieces of the split row)."""
    rng = np.random.default_rng(0)
    adj = _hub_graph(rng)
    lhs = rng.integers(0, 3, size=(adj.shape[1], 5)).astype("float32")
    rhs = rng.integers(0, 3, size=(adj.nnz, 1)).astype("float32")
    for reduce in ("max", "min"):
        out, arg = _run_spmm(adj, "u_add_e", reduce, [lhs, rhs], return_arg=True)
        ref, ref_arg = oracle.gspmm_bcast(adj.indptr, adj.indices, "add", reduce, lhs, rhs, 'u', 'e')
        assert np.array_equal(out, ref)
        assert np.array_equal(arg, ref_arg)
        assert (arg[np.diff(adj.indptr) == 0] == -1).all()


def test_edge_features_that_repeat_a_weight_match_the_weighted_sum(oracle):
    """u_mul_e with [nnz, F] edge features that hold one weight per edge F times = the plain SpMM."""
    import torch
    from featgraph_amd.module import VanillaSpMMhip, placeholder
    rng = np.random.default_rng(5)
    adj = _hub_graph(rng)
    x = _operand(rng, adj.shape[1], (260,))
    ef = np.repeat(adj.data[:, None], 260, axis=1).astype("float32")
    out = _run_spmm(adj, "u_mul_e", "sum", [x, ef])
    m = VanillaSpMMhip(adj)
    m.build([placeholder(x.shape)], {}, {'num_src_partitions': None})
    plain = m.run([torch.from_numpy(x).cuda()]).cpu().numpy()
    ref64 = oracle.spmm_f64(adj, x)
    mass = np.asarray(abs(adj).astype(np.float64).dot(np.abs(x).astype(np.float64)))
    assert_sum_close(out, ref64, mass, "edge features")
    assert_sum_close(plain, ref64, mass, "plain")
    # 260 features (65 vectors of 4, not cut into 64-float tiles): one lane group per row, so rows that are not split
    # are summed in stored order, with separately rounded products: the sequential float32 sum, bit for bit
    seq = oracle.spmm_csr_rowwise(adj.indptr, adj.indices, adj.data, x)
    short = np.diff(adj.indptr) <= 1024
    assert np.array_equal(out[short], seq[short])


def test_nonfinite_messages_stay_in_their_rows(oracle):
    rng = np.random.default_rng(9)
    adj = _graph(rng)
    x = _operand(rng, adj.shape[1], (8,))
    ef = _operand(rng, adj.nnz, (8,))
    clean = _run_spmm(adj, "u_mul_e", "sum", [x, ef])
    xb = x.copy(); xb[17] = np.inf; xb[400] = np.nan
    got = _run_spmm(adj, "u_mul_e", "sum", [xb, ef])
    hit = np.zeros(adj.shape[0], bool)
    rows = np.repeat(np.arange(adj.shape[0]), np.diff(adj.indptr))
    hit[rows[np.isin(adj.indices, [17, 400])]] = True
    assert hit.any() and not np.isfinite(got[hit]).all(axis=1).any()
    assert np.isfinite(got[~hit]).all() and np.array_equal(got[~hit], clean[~hit])


def test_gspmm_broadcast_errors():
    from featgraph_amd.module import GSpMMhip, placeholder
    rng = np.random.default_rng(1)
    adj = _graph(rng)
    n, nnz = adj.shape[1], adj.nnz
    m = GSpMMhip(adj)
    with pytest.raises(ValueError):     # destination-node operands have no place in an aggregation over the row
        m.build([placeholder((adj.shape[0], 4)), placeholder((nnz, 4))], {'msg': 'v_mul_e'}, {})
    with pytest.raises(ValueError):     # shapes that do not broadcast
        m.build([placeholder((n, 4)), placeholder((nnz, 3))], {'msg': 'u_add_e'}, {})
    with pytest.raises(ValueError):     # wrong number of rows for the target
        m.build([placeholder((n, 4)), placeholder((n, 4))], {'msg': 'u_add_e'}, {})
    with pytest.raises(ValueError):
        m.build([placeholder((n, 4)), placeholder((nnz, 4))], {'msg': 'u_pow_e'}, {})
    with pytest.raises(ValueError):     # one operand only
        m.build([placeholder((nnz, 4)), placeholder((nnz, 4))], {'msg': 'copy_e'}, {})
    with pytest.raises(ValueError):
        m.build([placeholder((n, 4)), placeholder((nnz, 4))], {'msg': 'u_add_e', 'reduce': 'sum', 'return_arg': True}, {})
    with pytest.raises(ValueError):
        m.build([placeholder((n, 4)), placeholder((nnz, 4))], {'msg': 'u_add_e'}, {'num_src_partitions': 0})
    m2 = GSpMMhip(adj, 2)               # the constructor's partitions are honoured
    m2.build([placeholder((n, 4)), placeholder((nnz, 4))], {'msg': 'u_add_e'}, {})
    assert m2._active['P'] == 2
    m.build([placeholder((n, 4)), placeholder((nnz, 4))], {'msg': 'u_add_e'}, {})
    assert "gspmm_bcast_kernel" in m.lower_to_ir([placeholder((n, 4)), placeholder((nnz, 4))], {'msg': 'u_add_e'}, {})


# ---- SDDMM ---------------------------------------------------------------------------------------------

EDGE_CASES = [
    # op, lhs target, lhs feature shape, rhs target, rhs feature shape
    ("add", 'u', (64,), 'v', (64,)),              # equal shapes, default targets: the element-wise kernel
    ("div", 'u', (64,), 'v', (64,)),
    ("add", 'u', (5,), 'v', (1,)),
    ("mul", 'v', (4, 8), 'u', (4, 1)),
    ("sub", 'u', (4, 2), 'v', (4, 1)),
    ("mul", 'e', (64,), 'v', (64,)),
    ("sub", 'e', (33,), 'u', (33,)),
    ("mul", 'e', (1,), 'e', (130,)),
    ("div", 'u', (2, 1), 'e', (1, 3)),
    ("dot", 'u', (4, 16), 'v', (4, 16)),
    ("dot", 'u', (40,), 'v', (40,)),
    ("dot", 'e', (3, 8), 'u', (1, 8)),
    ("dot", 'v', (2, 1, 4), 'e', (5, 4)),
    ("dot", 'u', (8, 64), 'v', (1, 64)),          # contracted axes of 16 floats and more: lane groups with 128-bit loads
    ("dot", 'u', (100,), 'u', (100,)),            # 25 of a group's 32 lanes hold a word
    ("dot", 'e', (2, 256), 'v', (256,)),
    ("dot", 'v', (520,), 'u', (3, 520)),          # more than 64 words: a lane walks the axis
    ("dot", 'u', (3, 6), 'e', (6,)),              # not a multiple of 4: lane by lane
    ("copy_lhs", 'u', (7,), None, None),
    ("copy_lhs", 'v', (70,), None, None),
    ("copy_rhs", None, None, 'e', (3,)),
]


@pytest.mark.parametrize("op,lt,l_shape,rt,r_shape", EDGE_CASES)
@pytest.mark.parametrize("partitions", [(1, 1), (2, 3)])
def test_gsddmm_broadcast(oracle, op, lt, l_shape, rt, r_shape, partitions):
    import torch
    from featgraph_amd.module import GSDDMMhip, placeholder
    rng = np.random.default_rng(len(op) + sum(l_shape or ()) + sum(r_shape or ()))
    adj = _graph(rng).tocoo()
    m = GSDDMMhip(adj, *partitions)
    row, col = m._adj_row_indices, m._adj_col_indices          # the stored order (2-D partitioned or COO)
    rows = {'u': adj.shape[1], 'v': adj.shape[0], 'e': adj.nnz, None: 0}
    lhs = _operand(rng, rows[lt], l_shape, positive=(op == 'div')) if lt else None
    rhs = _operand(rng, rows[rt], r_shape, positive=(op == 'div')) if rt else None
    arrays = [a for a in (lhs, rhs) if a is not None]
    args = {'op': op}
    if lt:
        args['lhs_target'] = lt
    if rt:
        args['rhs_target'] = rt
    m.build([placeholder(a.shape) for a in arrays], args, {})
    m.out_tvm.fill_(float("nan"))
    out = m.run([torch.from_numpy(a).cuda() for a in arrays]).cpu().numpy()
    ref = oracle.gsddmm_bcast(row, col, op, lhs, rhs, lt or 'u', rt or 'v')
    assert out.shape == ref.shape, (out.shape, ref.shape)
    if op == 'dot':
        mass = oracle.gsddmm_bcast(row, col, op, np.abs(lhs), np.abs(rhs), lt, rt)
        assert_sum_close(out, ref, mass, "dot")
    else:
        assert np.array_equal(out, ref)
    if partitions != (1, 1):
        # back in the caller's COO order through edge_mapping
        ref_coo = oracle.gsddmm_bcast(adj.row, adj.col, op,
                                      lhs if lt != 'e' else lhs[m.edge_mapping],
                                      rhs if rt != 'e' else rhs[m.edge_mapping], lt or 'u', rt or 'v')
        assert np.allclose(out[m.edge_mapping], ref_coo, rtol=RTOL, atol=ATOL)


def test_gsddmm_dot_heads_match_the_multihead_kernel(oracle):
    import torch
    from featgraph_amd.module import GSDDMMhip, MultiHeadSDDMMhip, placeholder
    rng = np.random.default_rng(2)
    adj = _graph(rng).tocoo()
    src = _operand(rng, adj.shape[1], (4, 32)); dst = _operand(rng, adj.shape[0], (4, 32))
    g = GSDDMMhip(adj); g.build([placeholder(src.shape), placeholder(dst.shape)], {'op': 'dot'}, {})
    mh = MultiHeadSDDMMhip(adj); mh.build([placeholder(src.shape), placeholder(dst.shape)], {}, {})
    s, d = torch.from_numpy(src).cuda(), torch.from_numpy(dst).cuda()
    a, b = g.run([s, d]).cpu().numpy(), mh.run([s, d]).cpu().numpy()
    ref = oracle.sddmm_multihead_f64(adj.row, adj.col, src, dst)
    mass = oracle.gsddmm_bcast(adj.row, adj.col, 'dot', np.abs(src), np.abs(dst), 'u', 'v')
    assert_sum_close(a, ref, mass, "broadcast dot")
    assert_sum_close(b, ref, mass, "multi-head kernel")


def test_gsddmm_broadcast_errors():
    from featgraph_amd.module import GSDDMMhip, placeholder
    rng = np.random.default_rng(1)
    adj = _graph(rng).tocoo()
    m = GSDDMMhip(adj)
    nr, nc, nnz = adj.shape[0], adj.shape[1], adj.nnz
    with pytest.raises(ValueError):
        m.build([placeholder((nc, 4)), placeholder((nr, 3))], {'op': 'add'}, {})
    with pytest.raises(ValueError):
        m.build([placeholder((nc, 4)), placeholder((nr, 4))], {'op': 'add', 'lhs_target': 'e'}, {})
    with pytest.raises(ValueError):
        m.build([placeholder((nc, 2, 4)), placeholder((nr, 2, 3))], {'op': 'dot'}, {})
    with pytest.raises(ValueError):
        m.build([placeholder((nc, 4)), placeholder((nr, 4))], {'op': 'pow'}, {})
    with pytest.raises(ValueError):
        m.build([placeholder((nc, 4)), placeholder((nr, 4))], {'op': 'copy_lhs'}, {})


def test_graphs_without_edges_or_rows(oracle):
    """No edges: every output row is 0 (also for max / min) and the per-edge result is empty."""
    import torch
    from featgraph_amd.module import GSpMMhip, GSDDMMhip, placeholder
    adj = sp.csr_matrix((7, 9), dtype="float32")
    x = np.ones((9, 5), "float32")
    ef = np.zeros((0, 5), "float32")
    for reduce in ("sum", "max", "mean"):
        m = GSpMMhip(adj)
        m.build([placeholder(x.shape), placeholder(ef.shape)], {'msg': 'u_add_e', 'reduce': reduce}, {})
        m.out_tvm.fill_(float("nan"))
        out = m.run([torch.from_numpy(x).cuda(), torch.from_numpy(ef).cuda()]).cpu().numpy()
        assert out.shape == (7, 5) and (out == 0).all()
    g = GSDDMMhip(adj.tocoo())
    g.build([placeholder((9, 5)), placeholder((7, 1))], {'op': 'mul'}, {})
    out = g.run([torch.from_numpy(x).cuda(), torch.ones((7, 1), device="cuda")])
    assert tuple(out.shape) == (0, 5)
    # one row, one element
    one = sp.csr_matrix((np.ones(1, "float32"), np.array([3], np.int32), np.array([0, 1], np.int32)), shape=(1, 9))
    m = GSpMMhip(one)
    m.build([placeholder((9, 5)), placeholder((1, 5))], {'msg': 'u_sub_e', 'reduce': 'min', 'return_arg': True}, {})
    xs = np.arange(45, dtype="float32").reshape(9, 5)
    out = m.run([torch.from_numpy(xs).cuda(), torch.ones((1, 5), device="cuda")]).cpu().numpy()
    assert np.array_equal(out, xs[3:4] - 1) and (m.arg_tvm.cpu().numpy() == 0).all()


def test_operands_that_are_not_16_byte_aligned(oracle):
    """Contiguous views that start 4 bytes into an allocation: the 128-bit paths must not be taken for them."""
    import torch
    from featgraph_amd.module import GSpMMhip, GSDDMMhip, placeholder
    rng = np.random.default_rng(21)
    adj = _hub_graph(rng)
    n, nnz, F = adj.shape[1], adj.nnz, 32
    x = _operand(rng, n, (F,)); ef = _operand(rng, nnz, (F,)); y = _operand(rng, adj.shape[0], (F,))

    def shifted(a):
        flat = torch.empty(a.size + 1, dtype=torch.float32, device="cuda")
        view = flat[1:].view(a.shape)
        view.copy_(torch.from_numpy(a))
        assert view.data_ptr() % 16 == 4 and view.is_contiguous()
        return view

    m = GSpMMhip(adj)
    m.build([placeholder(x.shape), placeholder(ef.shape)], {'msg': 'u_mul_e', 'reduce': 'max'}, {})
    ref, _ = oracle.gspmm_bcast(adj.indptr, adj.indices, 'mul', 'max', x, ef, 'u', 'e')
    for xs, es in ((shifted(x), torch.from_numpy(ef).cuda()), (torch.from_numpy(x).cuda(), shifted(ef)), (shifted(x), shifted(ef))):
        assert np.array_equal(m.run([xs, es]).cpu().numpy(), ref)
    coo = adj.tocoo()
    g = GSDDMMhip(coo)
    g.build([placeholder(ef.shape), placeholder(y.shape)], {'op': 'sub', 'lhs_target': 'e'}, {})
    ref = oracle.gsddmm_bcast(coo.row, coo.col, 'sub', ef, y, 'e', 'v')
    assert np.array_equal(g.run([shifted(ef), shifted(y)]).cpu().numpy(), ref)
    g.build([placeholder(ef.shape), placeholder(y.shape)], {'op': 'dot', 'lhs_target': 'e'}, {})
    ref = oracle.gsddmm_bcast(coo.row, coo.col, 'dot', ef, y, 'e', 'v')
    mass = oracle.gsddmm_bcast(coo.row, coo.col, 'dot', np.abs(ef), np.abs(y), 'e', 'v')
    for es, ys in ((shifted(ef), torch.from_numpy(y).cuda()), (torch.from_numpy(ef).cuda(), shifted(y))):
        assert_sum_close(g.run([es, ys]).cpu().numpy(), ref, mass, "dot of a shifted operand")


def test_square_head_shapes_follow_numpy_broadcasting_on_request(oracle):
    """SrcFeat (num_cols, H, D) with D == H and a second input (nnz, H): the module reads it as one weight per edge and
    head unless compute_args say 'broadcast', in which case (as for DGL's gspmm, and in featgraph_amd.ops) the second
    input lines up with the last axis; (num_cols, H, D) with one weight per edge (nnz,) is a broadcast either way."""
    import torch
    from featgraph_amd.module import GSpMMhip, placeholder
    from featgraph_amd import ops
    from featgraph_amd.autograd import Graph
    rng = np.random.default_rng(4)
    adj = _graph(rng)
    x = _operand(rng, adj.shape[1], (4, 4))
    w = _operand(rng, adj.nnz, (4,))
    xd, wd = torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()
    per_head, _ = oracle.gspmm_bcast(adj.indptr, adj.indices, 'mul', 'sum', x, w[:, :, None], 'u', 'e')
    last_axis, _ = oracle.gspmm_bcast(adj.indptr, adj.indices, 'mul', 'sum', x, w, 'u', 'e')
    assert not np.allclose(per_head, last_axis)
    m = GSpMMhip(adj)
    m.build([placeholder(x.shape), placeholder(w.shape)], {'msg': 'u_mul_e'}, {})
    assert np.allclose(m.run([xd, wd]).cpu().numpy(), per_head, rtol=1e-4, atol=1e-4)
    m.build([placeholder(x.shape), placeholder(w.shape)], {'msg': 'u_mul_e', 'broadcast': True}, {})
    assert np.allclose(m.run([xd, wd]).cpu().numpy(), last_axis, rtol=1e-4, atol=1e-4)
    assert np.allclose(ops.gspmm(Graph(adj), "mul", "sum", xd, wd).cpu().numpy(), last_axis, rtol=1e-4, atol=1e-4)
    one = _operand(rng, adj.nnz, ())
    m.build([placeholder(x.shape), placeholder(one.shape)], {'msg': 'u_mul_e'}, {})
    ref, _ = oracle.gspmm_bcast(adj.indptr, adj.indices, 'mul', 'sum', x, one, 'u', 'e')
    assert np.allclose(m.run([xd, torch.from_numpy(one).cuda()]).cpu().numpy(), ref, rtol=1e-4, atol=1e-4)
