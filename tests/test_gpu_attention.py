"""Graph attention in one operator (multi-head SDDMM + edge softmax + per-head weighted SpMM without stored
scores) against the float64 composition of the three, and against the three GPU operators chained."""
import numpy as np
import pytest
import scipy.sparse as sp

pytestmark = pytest.mark.gpu


def _graph(rng, n_rows=300, n_cols=700, long_len=650, density=0.03):
    a = sp.random(n_rows, n_cols, density=density, format="csr", random_state=rng,
                  data_rvs=lambda k: np.ones(k)).astype("float32").tolil()
    a[[0, n_rows // 2], :] = 0                                   # rows without edges
    a[7, rng.choice(n_cols, size=long_len, replace=False)] = 1   # a long row (several staging rounds)
    a = a.tocsr().astype("float32"); a.eliminate_zeros(); a.sort_indices()
    return a


def _run(adj, q, k, v, P, scale=None):
    import torch
    from featgraph_amd.module import GraphAttentionhip, placeholder
    m = GraphAttentionhip(adj)
    m.build([placeholder(q.shape), placeholder(k.shape), placeholder(v.shape)],
            {} if scale is None else {'scale': scale}, {'num_src_partitions': P})
    m.out_tvm.fill_(float("nan"))
    return m.run([torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda()]).cpu().numpy().copy()


@pytest.mark.parametrize("H,D", [(1, 64), (4, 64), (8, 64), (16, 64), (4, 32), (8, 16), (3, 64), (10, 32)])
@pytest.mark.parametrize("P", [None, 2, 5])
def test_against_float64_composition(oracle, H, D, P):
    rng = np.random.default_rng(H * 100 + D + (P or 0))
    adj = _graph(rng)
    q = rng.standard_normal((adj.shape[0], H, D)).astype("float32")
    k = rng.standard_normal((adj.shape[1], H, D)).astype("float32")
    v = rng.standard_normal((adj.shape[1], H, D)).astype("float32")
    out = _run(adj, q, k, v, P)
    ref = oracle.graph_attention_f64(adj.indptr, adj.indices, q, k, v, 1.0 / np.sqrt(D))
    assert np.isfinite(out).all()
    assert (out[np.diff(adj.indptr) == 0] == 0).all()
    np.testing.assert_allclose(out, ref, rtol=1e-4, atol=2e-5)


def test_large_scores_do_not_overflow(oracle):
    """Scores in the thousands: the running maximum keeps every exponential at or below 1."""
    rng = np.random.default_rng(11)
    adj = _graph(rng)
    H, D = 4, 64
    q = (30 * rng.standard_normal((adj.shape[0], H, D))).astype("float32")
    k = (30 * rng.standard_normal((adj.shape[1], H, D))).astype("float32")
    v = rng.standard_normal((adj.shape[1], H, D)).astype("float32")
    out = _run(adj, q, k, v, 3, scale=1.0)
    ref = oracle.graph_attention_f64(adj.indptr, adj.indices, q, k, v, 1.0)
    assert np.isfinite(out).all()
    np.testing.assert_allclose(out, ref, rtol=1e-3, atol=1e-4)


def test_uniform_scores_give_the_mean(oracle):
    """K = 0: every edge weighs the same and the result is the mean of the neighbours' V."""
    rng = np.random.default_rng(12)
    adj = _graph(rng)
    H, D = 2, 32
    q = rng.standard_normal((adj.shape[0], H, D)).astype("float32")
    k = np.zeros((adj.shape[1], H, D), np.float32)
    v = rng.standard_normal((adj.shape[1], H, D)).astype("float32")
    out = _run(adj, q, k, v, 2)
    deg = np.diff(adj.indptr)
    mean = np.asarray(adj.astype(np.float64).dot(v.reshape(v.shape[0], -1).astype(np.float64)))
    mean[deg > 0] /= deg[deg > 0, None]
    np.testing.assert_allclose(out.reshape(mean.shape), mean, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("tile_major", [1, 2])
def test_equals_the_three_operators_chained(monkeypatch, tile_major):
    import torch
    from featgraph_amd import _lib
    from featgraph_amd.autograd import Graph
    monkeypatch.setattr(_lib, "plan_opts", _lib.FgPlanOpts(tile_major=tile_major))
    rng = np.random.default_rng(13)
    adj = _graph(rng, 500, 900, 800, 0.05)
    H, D = 8, 64
    q = rng.standard_normal((adj.shape[0], H, D)).astype("float32")
    k = rng.standard_normal((adj.shape[1], H, D)).astype("float32")
    v = rng.standard_normal((adj.shape[1], H, D)).astype("float32")
    out = _run(adj, q, k, v, 4)
    g = Graph(adj)
    s = g.sddmm(torch.from_numpy(k).cuda(), torch.from_numpy(q).cuda()) * (1.0 / np.sqrt(D))
    chained = g.spmm(torch.from_numpy(v).cuda(), g.edge_softmax(s)).cpu().numpy()
    np.testing.assert_allclose(out, chained, rtol=2e-4, atol=5e-5)


def test_repeatable_and_shapes_are_checked():
    import torch
    from featgraph_amd.module import GraphAttentionhip, placeholder
    rng = np.random.default_rng(14)
    adj = _graph(rng)
    H, D = 4, 64
    q = rng.standard_normal((adj.shape[0], H, D)).astype("float32")
    k = rng.standard_normal((adj.shape[1], H, D)).astype("float32")
    v = rng.standard_normal((adj.shape[1], H, D)).astype("float32")
    a = _run(adj, q, k, v, 3)
    b = _run(adj, q, k, v, 3)
    assert np.array_equal(a, b)
    m = GraphAttentionhip(adj)
    with pytest.raises(ValueError):
        m.build([placeholder((adj.shape[0], H, 48)), placeholder((adj.shape[1], H, 48)), placeholder((adj.shape[1], H, 48))])
    with pytest.raises(ValueError):
        m.build([placeholder(q.shape), placeholder(k.shape), placeholder((adj.shape[1], H, 32))])
    with pytest.raises(RuntimeError):
        GraphAttentionhip(adj).run([torch.from_numpy(q).cuda()] * 3)


def test_empty_graph_and_empty_partition():
    adj = sp.csr_matrix((50, 40), dtype=np.float32)
    rng = np.random.default_rng(15)
    q = rng.standard_normal((50, 2, 64)).astype("float32")
    k = rng.standard_normal((40, 2, 64)).astype("float32")
    out = _run(adj, q, k, k, 2)
    assert (out == 0).all()
    # all edges in the last partition's columns
    adj = sp.csr_matrix((np.ones(3, np.float32), (np.array([1, 1, 4]), np.array([38, 39, 39]))), shape=(50, 40))
    out = _run(adj, q, k, k, 4)
    assert np.isfinite(out).all() and (out[0] == 0).all() and np.allclose(out[4], k[39], atol=1e-6)


def test_full_size_graph(oracle):
    """232,965 nodes / 114.77M edges, H=4, D=64 (the tile-by-tile copies of K and V are in use at this size):
    sampled rows against float64, and K = 0 against the mean aggregation of the SpMM path."""
    import torch
    from featgraph_amd import synthetic
    from featgraph_amd.module import GraphAttentionhip, GSpMMhip, placeholder
    indptr, indices = synthetic.make_workload("powerlaw-233k")
    n, nnz = indptr.shape[0] - 1, int(indptr[-1])
    adj = sp.csr_matrix((np.ones(nnz, np.float32), indices, indptr), shape=(n, n))
    H, D = 4, 64
    gen = torch.Generator(device="cuda"); gen.manual_seed(3)
    q, k, v = (torch.randn((n, H, D), generator=gen, device="cuda") for _ in range(3))
    m = GraphAttentionhip(adj)
    m.build([placeholder((n, H, D))] * 3, {}, {})
    out = m.run([q, k, v]).cpu().numpy().copy()
    assert np.isfinite(out).all()
    deg = np.diff(indptr)
    rows = np.unique(np.concatenate([[0, n - 1, int(deg.argmax()), int(deg.argmin())],
                                     np.random.default_rng(0).integers(0, n, 60)]))
    qh, kh, vh = q.cpu().numpy(), k.cpu().numpy(), v.cpu().numpy()
    sub_ptr = np.concatenate([[0], np.cumsum(deg[rows])]).astype(np.int64)
    sub_idx = np.concatenate([indices[indptr[r]:indptr[r + 1]] for r in rows])
    ref = oracle.graph_attention_f64(sub_ptr, sub_idx, qh[rows], kh, vh, 1.0 / np.sqrt(D))
    np.testing.assert_allclose(out[rows], ref, rtol=1e-4, atol=2e-5)
    # uniform scores: the neighbours' mean
    got = m.run([q, torch.zeros_like(k), v]).reshape(n, H * D).clone()
    agg = GSpMMhip(adj)
    agg.build([placeholder((n, H * D))], {'reduce': 'mean', 'msg': 'copy_u'}, {})
    want = agg.run([v.reshape(n, H * D)])
    err = (got - want).abs().max().item()
    assert err < 2e-5, err


def _dense_reference(adj, q, k, v, scale, dout):
    """out and (dq, dk, dv) for sum(out * dout) by float64 torch autograd on the dense masked form."""
    import torch
    coo = adj.tocoo()
    mask = torch.zeros(adj.shape, dtype=torch.bool)
    mask[coo.row, coo.col] = True
    q64, k64, v64 = (torch.from_numpy(t).double().requires_grad_() for t in (q, k, v))
    s = torch.einsum("rhd,chd->hrc", q64, k64) * scale
    a = torch.nan_to_num(torch.softmax(s.masked_fill(~mask, float("-inf")), dim=-1), nan=0.0)
    out = torch.einsum("hrc,chd->rhd", a, v64)
    (out * torch.from_numpy(dout).double()).sum().backward()
    return out.detach().numpy(), q64.grad.numpy(), k64.grad.numpy(), v64.grad.numpy()


@pytest.mark.parametrize("H,D,P,Pt", [(1, 64, None, None), (4, 64, 2, 3), (8, 64, 3, 2), (4, 32, 2, 2), (8, 16, 5, 4),
                                      (3, 64, 1, 4), (16, 32, 4, 1)])
@pytest.mark.parametrize("tile_major", [0, 1])
def test_gradients_against_float64(monkeypatch, H, D, P, Pt, tile_major):
    import torch
    from featgraph_amd import _lib
    from featgraph_amd.module import GraphAttentionhip, placeholder
    if tile_major:
        monkeypatch.setattr(_lib, "plan_opts", _lib.FgPlanOpts(tile_major=1))
    rng = np.random.default_rng(H * 1000 + D * 10 + (P or 0))
    adj = _graph(rng, 200, 260, 250, 0.05)
    q = rng.standard_normal((adj.shape[0], H, D)).astype("float32")
    k = rng.standard_normal((adj.shape[1], H, D)).astype("float32")
    v = rng.standard_normal((adj.shape[1], H, D)).astype("float32")
    dout = rng.standard_normal(q.shape).astype("float32")
    m = GraphAttentionhip(adj)
    m.build([placeholder(q.shape), placeholder(k.shape), placeholder(v.shape)], {},
            {'num_src_partitions': P, 'num_dst_partitions': Pt})
    qd, kd, vd, dd = (torch.from_numpy(t).cuda() for t in (q, k, v, dout))
    out = m.run([qd, kd, vd])
    dq, dk, dv = m.backward(qd, kd, vd, out, m.state_tvm, dd)
    ref_out, ref_dq, ref_dk, ref_dv = _dense_reference(adj, q, k, v, 1.0 / np.sqrt(D), dout)
    np.testing.assert_allclose(out.cpu().numpy(), ref_out, rtol=1e-4, atol=2e-5)
    for got, want, name in ((dq, ref_dq, "dq"), (dk, ref_dk, "dk"), (dv, ref_dv, "dv")):
        got = got.cpu().numpy()
        assert np.isfinite(got).all(), name
        np.testing.assert_allclose(got, want, rtol=1e-3, atol=1e-4, err_msg=name)
    # rows / columns without edges get zero gradients
    assert (dq.cpu().numpy()[np.diff(adj.indptr) == 0] == 0).all()
    no_in = np.diff(adj.T.tocsr().indptr) == 0
    assert (dk.cpu().numpy()[no_in] == 0).all() and (dv.cpu().numpy()[no_in] == 0).all()


@pytest.mark.parametrize("H,D,P", [(1, 64, None), (4, 64, 3), (8, 32, 2), (8, 16, 5), (3, 64, 1)])
def test_additive_scores_against_float64(oracle, H, D, P):
    """The attention of GAT layers: leaky_relu(El[col] + Er[row]) as scores."""
    import torch
    from featgraph_amd.module import GraphAttentionhip, placeholder
    rng = np.random.default_rng(H * 7 + D + (P or 0))
    adj = _graph(rng)
    er = rng.standard_normal((adj.shape[0], H)).astype("float32")
    el = (3 * rng.standard_normal((adj.shape[1], H))).astype("float32")
    v = rng.standard_normal((adj.shape[1], H, D)).astype("float32")
    m = GraphAttentionhip(adj)
    m.build([placeholder(er.shape), placeholder(el.shape), placeholder(v.shape)],
            {'scores': 'additive', 'negative_slope': 0.2}, {'num_src_partitions': P})
    m.out_tvm.fill_(float("nan"))
    out = m.run([torch.from_numpy(er).cuda(), torch.from_numpy(el).cuda(), torch.from_numpy(v).cuda()]).cpu().numpy()
    ref = oracle.graph_attention_additive_f64(adj.indptr, adj.indices, er, el, v, 0.2)
    assert np.isfinite(out).all() and (out[np.diff(adj.indptr) == 0] == 0).all()
    np.testing.assert_allclose(out, ref, rtol=1e-4, atol=2e-5)


@pytest.mark.parametrize("H,D,P,Pt", [(1, 64, None, None), (4, 64, 2, 3), (8, 32, 3, 2), (8, 16, 5, 4), (3, 64, 1, 4)])
@pytest.mark.parametrize("tile_major", [0, 1])
def test_additive_gradients_against_float64(monkeypatch, H, D, P, Pt, tile_major):
    import torch
    from featgraph_amd import _lib
    from featgraph_amd.module import GraphAttentionhip, placeholder
    if tile_major:
        monkeypatch.setattr(_lib, "plan_opts", _lib.FgPlanOpts(tile_major=1))
    rng = np.random.default_rng(H * 1000 + D * 10 + (P or 0) + 5)
    adj = _graph(rng, 200, 260, 250, 0.05)
    er = rng.standard_normal((adj.shape[0], H)).astype("float32")
    el = (2 * rng.standard_normal((adj.shape[1], H))).astype("float32")
    v = rng.standard_normal((adj.shape[1], H, D)).astype("float32")
    dout = rng.standard_normal((adj.shape[0], H, D)).astype("float32")
    m = GraphAttentionhip(adj)
    m.build([placeholder(er.shape), placeholder(el.shape), placeholder(v.shape)], {'scores': 'additive', 'negative_slope': 0.2},
            {'num_src_partitions': P, 'num_dst_partitions': Pt})
    erd, eld, vd, dd = (torch.from_numpy(t).cuda() for t in (er, el, v, dout))
    out = m.run([erd, eld, vd])
    der, del_, dv = m.backward(erd, eld, vd, out, m.state_tvm, dd)
    # float64 torch autograd on the dense masked form
    coo = adj.tocoo()
    mask = torch.zeros(adj.shape, dtype=torch.bool); mask[coo.row, coo.col] = True
    er64, el64, v64 = (torch.from_numpy(t).double().requires_grad_() for t in (er, el, v))
    z = er64.t()[:, :, None] + el64.t()[:, None, :]                      # [H, rows, cols]
    s = torch.nn.functional.leaky_relu(z, 0.2).masked_fill(~mask, float("-inf"))
    a = torch.nan_to_num(torch.softmax(s, dim=-1), nan=0.0)
    ref = torch.einsum("hrc,chd->rhd", a, v64)
    (ref * torch.from_numpy(dout).double()).sum().backward()
    np.testing.assert_allclose(out.cpu().numpy(), ref.detach().numpy(), rtol=1e-4, atol=2e-5)
    for got, want, name in ((der, er64.grad, "d_er"), (del_, el64.grad, "d_el"), (dv, v64.grad, "dv")):
        got = got.cpu().numpy()
        assert np.isfinite(got).all(), name
        np.testing.assert_allclose(got, want.numpy(), rtol=1e-3, atol=1e-4, err_msg=name)
