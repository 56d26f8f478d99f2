"""Seeded random sweep over graph shapes, densities, feature lengths, partition and tile counts:
every case is compared with the CPU oracle / float64 closed forms.  The point is breadth -- kernel
variants and boundary conditions that the hand-picked cases may not reach.  Half of the SpMM and SDDMM
seeds run with the tile-by-tile copy of the gathered operand forced on.  FG_TEST_SEED_BASE=<int> in the
environment shifts every seed, for sweeps beyond the committed cases."""
import os

import numpy as np
import pytest
import scipy.sparse as sp

from helpers import RTOL, ATOL, assert_sum_close, spmm_mass, sddmm_mass

pytestmark = pytest.mark.gpu

SEED_BASE = int(os.environ.get("FG_TEST_SEED_BASE", "0"))

FEATS = [1, 2, 3, 4, 5, 8, 12, 16, 20, 31, 32, 48, 64, 65, 96, 100, 128, 160, 192, 256, 257, 320, 384, 512, 768, 1024]


def _random_graph(rng):
    n_rows = int(rng.integers(1, 400))
    n_cols = int(rng.integers(1, 400))
    density = float(rng.choice([0.0, 0.002, 0.02, 0.1, 0.5, 1.0]))
    a = sp.random(n_rows, n_cols, density=density, format="csr", random_state=rng,
                  data_rvs=lambda k: rng.standard_normal(k)).astype("float32")
    if rng.random() < 0.5 and n_cols > 4:                      # a long row, split into pieces at threshold 1024
        a = a.tolil()
        r = int(rng.integers(0, n_rows))
        a[r, :] = rng.standard_normal(n_cols).astype("float32")
        a = a.tocsr().astype("float32")
    a.eliminate_zeros(); a.sort_indices()
    return a


@pytest.mark.parametrize("seed", range(8))
def test_random_spmm(oracle, monkeypatch, seed):
    import torch
    from featgraph_amd import _lib
    from featgraph_amd.module import VanillaSpMMhip, placeholder
    if seed % 2:        # odd seeds: gather from the tile-by-tile copy wherever the kernel allows it
        monkeypatch.setattr(_lib, "plan_opts", _lib.FgPlanOpts(tile_major=1))
    rng = np.random.default_rng(SEED_BASE + 1000 + seed)
    for case in range(20):
        adj = _random_graph(rng)
        F = int(rng.choice(FEATS))
        P = int(rng.choice([1, 1, 2, 3, 5, 8]))
        divisors = [t for t in (1, 2, 4, 8, 16) if F % t == 0]
        T = int(rng.choice([0] + divisors))
        x = rng.standard_normal((adj.shape[1], F)).astype("float32")
        m = VanillaSpMMhip(adj, P)
        m.build([placeholder(x.shape)], {'num_feat_partitions': T}, {'num_src_partitions': None})
        m.out_tvm.fill_(float("nan"))
        out = m.run([torch.from_numpy(x).cuda()]).cpu().numpy()
        what = "seed %d case %d: %s nnz %d F=%d P=%d T=%d" % (seed, case, adj.shape, adj.nnz, F, P, T)
        assert np.isfinite(out).all(), what
        assert_sum_close(out, oracle.spmm_f64(adj, x), spmm_mass(adj, x), what)


@pytest.mark.parametrize("seed", range(8))
def test_random_sddmm(oracle, monkeypatch, seed):
    import torch
    from featgraph_amd import _lib
    from featgraph_amd.module import VanillaSDDMMhip, MultiHeadSDDMMhip, placeholder
    if seed % 2:
        monkeypatch.setattr(_lib, "plan_opts", _lib.FgPlanOpts(tile_major=1))
    rng = np.random.default_rng(SEED_BASE + 2000 + seed)
    for case in range(20):
        adj = _random_graph(rng)
        coo = adj.tocoo()
        if rng.random() < 0.5:
            H, D = 1, int(rng.choice(FEATS))
        else:
            H, D = int(rng.choice([2, 3, 4, 8, 16])), int(rng.choice([4, 8, 12, 16, 32, 64, 128]))
        shp = (H, D) if H > 1 else (D,)
        src = rng.standard_normal((adj.shape[1],) + shp).astype("float32")
        dst = rng.standard_normal((adj.shape[0],) + shp).astype("float32")
        order = str(rng.choice(["auto", "csr", "coo", "tiled"]))
        sched = {'order': order}
        F = H * D
        if order == "tiled":
            tiles = [t for t in (1, 2, 4, 8) if F % t == 0 and (F // t) in (16, 32, 64, 128, 256)
                     and (H == 1 or (F // t) % D == 0 or D == (F // t))]
            if not tiles or (H > 1 and (D % 4 != 0 or D < 8 or (D & (D - 1)) != 0)):
                sched = {'order': 'auto'}
            else:
                sched.update({'num_src_partitions': int(rng.choice([1, 2, 3, 8])), 'num_feat_tiles': int(rng.choice(tiles))})
        m = (MultiHeadSDDMMhip if H > 1 else VanillaSDDMMhip)(coo if rng.random() < 0.5 else adj)
        m.build([placeholder(src.shape), placeholder(dst.shape)], {}, sched)
        m.out_tvm.fill_(float("nan"))
        out = m.run([torch.from_numpy(src).cuda(), torch.from_numpy(dst).cuda()]).cpu().numpy()
        what = "seed %d case %d: %s nnz %d H=%d D=%d %s" % (seed, case, adj.shape, adj.nnz, H, D, sched)
        assert np.isfinite(out).all(), what
        ref = oracle.sddmm_multihead_f64(coo.row, coo.col, src, dst) if H > 1 else oracle.sddmm_f64(coo.row, coo.col, src, dst)
        assert_sum_close(out, ref, sddmm_mass(coo.row, coo.col, src, dst), what)


@pytest.mark.parametrize("seed", range(4))
def test_random_softmax_and_aggregation(oracle, seed):
    import torch
    from featgraph_amd.module import EdgeSoftmaxhip, GSpMMhip, placeholder
    rng = np.random.default_rng(SEED_BASE + 3000 + seed)
    for case in range(20):
        adj = _random_graph(rng)
        H = int(rng.choice([1, 2, 3, 4, 5, 8, 16, 64]))
        shape = (adj.nnz,) if H == 1 else (adj.nnz, H)
        s = (rng.standard_normal(shape) * 3).astype("float32")
        sm = EdgeSoftmaxhip(adj)
        sm.build([placeholder(shape)])
        a = sm.run([torch.from_numpy(s).cuda()]).cpu().numpy()
        what = "seed %d case %d: %s nnz %d H=%d" % (seed, case, adj.shape, adj.nnz, H)
        np.testing.assert_allclose(a, oracle.edge_softmax_f64(adj.indptr, s), rtol=RTOL, atol=ATOL, err_msg=what)
        g = rng.standard_normal(shape).astype("float32")
        dx = sm.backward(torch.from_numpy(a).cuda(), torch.from_numpy(g).cuda()).cpu().numpy()
        np.testing.assert_allclose(dx, oracle.edge_softmax_backward(adj.indptr, a, g), rtol=1e-3, atol=2e-5, err_msg=what)
        F = int(rng.choice([1, 4, 7, 32, 100, 256]))
        x = rng.integers(-3, 4, size=(adj.shape[1], F)).astype("float32")
        red = str(rng.choice(["max", "min"]))
        gm = GSpMMhip(adj)
        gm.build([placeholder(x.shape)], {'reduce': red, 'return_arg': True}, {})
        out = gm.run([torch.from_numpy(x).cuda()]).cpu().numpy()
        ref_out, ref_arg = oracle.gspmm_arg(adj.indptr, adj.indices, adj.data, x, red)
        assert np.array_equal(out, ref_out), what
        assert np.array_equal(gm.arg_tvm.cpu().numpy(), ref_arg), what


@pytest.mark.parametrize("seed", range(4))
def test_random_attention(oracle, monkeypatch, seed):
    import torch
    from featgraph_amd import _lib
    from featgraph_amd.module import GraphAttentionhip, placeholder
    if seed % 2:
        monkeypatch.setattr(_lib, "plan_opts", _lib.FgPlanOpts(tile_major=1))
    rng = np.random.default_rng(SEED_BASE + 4000 + seed)
    for case in range(10):
        adj = _random_graph(rng)
        H = int(rng.choice([1, 2, 3, 4, 8, 9, 16]))
        D = int(rng.choice([16, 32, 64]))
        P = rng.choice([None, 1, 2, 3, 7])
        P = None if P is None else int(P)
        q = rng.standard_normal((adj.shape[0], H, D)).astype("float32")
        k = rng.standard_normal((adj.shape[1], H, D)).astype("float32")
        v = rng.standard_normal((adj.shape[1], H, D)).astype("float32")
        m = GraphAttentionhip(adj)
        m.build([placeholder(q.shape), placeholder(k.shape), placeholder(v.shape)], {}, {'num_src_partitions': P})
        m.out_tvm.fill_(float("nan"))
        out = m.run([torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda()]).cpu().numpy()
        what = "seed %d case %d: %s nnz %d H=%d D=%d P=%s" % (seed, case, adj.shape, adj.nnz, H, D, P)
        ref = oracle.graph_attention_f64(adj.indptr, adj.indices, q, k, v, 1.0 / np.sqrt(D))
        assert np.isfinite(out).all(), what
        np.testing.assert_allclose(out, ref, rtol=1e-4, atol=2e-5, err_msg=what)


def _random_feature_shapes(rng):
    """Two feature shapes that broadcast against each other (possibly of different rank)."""
    nd = int(rng.integers(1, 4))
    dims = [int(rng.choice([1, 2, 3, 4, 5, 8, 16, 33])) for _ in range(nd)]
    l, r = [], []
    for d in dims:
        which = rng.integers(0, 4)
        l.append(1 if which == 1 else d)
        r.append(1 if which == 2 else d)
    cut = int(rng.integers(0, nd))          # drop leading axes of one operand
    if rng.random() < 0.5:
        l = l[cut:]
    else:
        r = r[cut:]
    return tuple(l), tuple(r)


@pytest.mark.parametrize("seed", range(6))
def test_random_broadcast_operators(oracle, monkeypatch, seed):
    """Generalised SpMM / SDDMM with broadcasting: random graphs, operators, targets and feature shapes (odd
    seeds: rows split into pieces of 64 elements, so that split rows occur on these small graphs; the SpMM over the
    CSR arrays or over 2, 3 or 7 source-column partitions)."""
    import torch
    from featgraph_amd import _lib
    from featgraph_amd.module import GSpMMhip, GSDDMMhip, placeholder
    if seed % 2:
        monkeypatch.setattr(_lib, "plan_opts", _lib.FgPlanOpts(split_threshold=64))
    rng = np.random.default_rng(SEED_BASE + 5000 + seed)
    for case in range(16):
        adj = _random_graph(rng)
        nnz = adj.nnz
        l_shape, r_shape = _random_feature_shapes(rng)
        op = str(rng.choice(["add", "sub", "mul", "div"]))
        what = "seed %d case %d: %s nnz %d %s %s %s" % (seed, case, adj.shape, nnz, op, l_shape, r_shape)

        def operand(rows, shape):
            x = rng.standard_normal((rows,) + shape).astype("float32")
            return (np.abs(x) + 0.5).astype("float32") if op == "div" else x

        # SpMM: operands on (u, e) or (e, u)
        lt, rt = ("u", "e") if rng.random() < 0.5 else ("e", "u")
        rows = {"u": adj.shape[1], "e": nnz}
        lhs, rhs = operand(rows[lt], l_shape), operand(rows[rt], r_shape)
        reduce = str(rng.choice(["sum", "mean", "max", "min"]))
        m = GSpMMhip(adj)
        args = {'msg': "%s_%s_%s" % (lt, op, rt), 'reduce': reduce, 'broadcast': True}     # numpy broadcasting throughout
        if reduce in ("max", "min"):
            args['return_arg'] = True
        parts = [None, 2, 3, 7][int(rng.integers(0, 4))]         # source-column partitions (None: the CSR arrays as they are)
        what += " parts %s" % parts
        m.build([placeholder(lhs.shape), placeholder(rhs.shape)], args, {'num_src_partitions': parts})
        m.out_tvm.fill_(float("nan"))
        out = m.run([torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda()]).cpu().numpy()
        ref, ref_arg = oracle.gspmm_bcast(adj.indptr, adj.indices, op, reduce, lhs, rhs, lt, rt)
        assert out.shape == ref.shape, what
        if reduce in ("max", "min"):
            assert np.array_equal(out, ref), what + " " + reduce
            assert np.array_equal(m.arg_tvm.cpu().numpy(), ref_arg), what + " arg " + reduce
        else:
            mass_op = "add" if op == "sub" else op
            mass, _ = oracle.gspmm_bcast(adj.indptr, adj.indices, mass_op, reduce, np.abs(lhs), np.abs(rhs), lt, rt)
            assert_sum_close(out, ref, mass, what + " " + reduce)

        # SDDMM: any two different targets
        targets = ["u", "v", "e"]
        lt = str(rng.choice(targets))
        rt = str(rng.choice([t for t in targets if t != lt]))
        coo = adj.tocoo()
        rows = {"u": adj.shape[1], "v": adj.shape[0], "e": nnz}
        lhs, rhs = operand(rows[lt], l_shape), operand(rows[rt], r_shape)
        g = GSDDMMhip(coo)
        g.build([placeholder(lhs.shape), placeholder(rhs.shape)], {'op': op, 'lhs_target': lt, 'rhs_target': rt}, {})
        g.out_tvm.fill_(float("nan"))
        out = g.run([torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda()]).cpu().numpy()
        ref = oracle.gsddmm_bcast(coo.row, coo.col, op, lhs, rhs, lt, rt)
        assert out.shape == ref.shape and np.array_equal(out, ref), what + " sddmm %s %s" % (lt, rt)


def test_tuned_choice_is_one_of_the_candidates_and_right():
    """schedule_args {'tune': k}: the module times the cost model's candidates on its own graph, keeps the
    fastest, and the result is the same product."""
    import torch
    from featgraph_amd import tuning
    from featgraph_amd.module import VanillaSpMMhip, VanillaSDDMMhip, placeholder
    rng = np.random.default_rng(5)
    adj = sp.random(3000, 4000, density=0.01, format="csr", random_state=rng).astype("float32")
    adj.sort_indices()
    F = 128
    x = rng.standard_normal((4000, F)).astype("float32")
    y = rng.standard_normal((3000, F)).astype("float32")
    m = VanillaSpMMhip(adj)
    m.build([placeholder((4000, F))], {}, {'tune': 3})
    assert len(m._tuned) == 3 and m._tuned[0][0] <= m._tuned[-1][0]
    ranked = tuning.rank_spmm(m._graph_stats(), F)[:3]
    assert (m._tuned[0][1], m._tuned[0][2]) in ranked
    out = m.run([torch.from_numpy(x).cuda()]).cpu().numpy()
    np.testing.assert_allclose(out, adj.astype(np.float64).dot(x.astype(np.float64)), rtol=1e-4, atol=1e-4)
    s = VanillaSDDMMhip(adj)
    s.build([placeholder((4000, F)), placeholder((3000, F))], {}, {'tune': True})
    assert len(s._tuned) >= 2
    coo = adj.tocoo()
    got = s.run([torch.from_numpy(x).cuda(), torch.from_numpy(y).cuda()]).cpu().numpy()
    ref = (x[coo.col].astype(np.float64) * y[coo.row].astype(np.float64)).sum(1)
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=1e-4)
    # explicit knobs win over 'tune'
    m.build([placeholder((4000, F))], {'num_feat_partitions': 2}, {'tune': True, 'num_src_partitions': 2})
    assert m._active['P'] == 2 and m._num_feat_partitions == 2
