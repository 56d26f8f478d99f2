"""With several feature tiles the SpMM and the tiled SDDMM gather from a copy of the source features that
stores every tile's slices back to back.  The copy changes addresses only: forced on (plan option
`tile_major=1`) and forced off (`2`) the results must agree bit for bit, on shapes small enough that the
default would not use it, and once on the full-size graph where the default does."""
import numpy as np
import pytest
import scipy.sparse as sp

from helpers import assert_sum_close, spmm_mass, sddmm_mass

pytestmark = pytest.mark.gpu


def _graph(rng, n_rows=300, n_cols=2000, long_len=1500):
    a = sp.random(n_rows, n_cols, density=0.03, format="csr", random_state=rng,
                  data_rvs=lambda k: rng.standard_normal(k)).astype("float32").tolil()
    a[[0, n_rows // 2], :] = 0
    a[7, rng.choice(n_cols, size=long_len, replace=False)] = 1.5
    a = a.tocsr().astype("float32"); a.eliminate_zeros(); a.sort_indices()
    return a


def _spmm(adj, x, P, T):
    import torch
    from featgraph_amd.module import VanillaSpMMhip, placeholder
    m = VanillaSpMMhip(adj, P)
    m.build([placeholder(x.shape)], {'num_feat_partitions': T}, {'num_src_partitions': None})
    text = m.lower_to_ir(m._placeholders, {'num_feat_partitions': T}, {'num_src_partitions': None})
    return m.run([torch.from_numpy(x).cuda()]).cpu().numpy().copy(), text


@pytest.mark.parametrize("feat_len,P,T", [(128, 1, 2), (128, 3, 2), (256, 2, 4), (512, 4, 8), (1024, 1, 16), (96, 2, 3), (64, 2, 4)])
def test_spmm_copy_equals_row_major(oracle, monkeypatch, feat_len, P, T):
    from featgraph_amd import _lib
    rng = np.random.default_rng(feat_len + P)
    adj = _graph(rng)
    x = rng.standard_normal((adj.shape[1], feat_len)).astype("float32")
    monkeypatch.setattr(_lib, "plan_opts", _lib.FgPlanOpts(tile_major=2))
    plain, text = _spmm(adj, x, P, T)
    assert "row-major" in text
    monkeypatch.setattr(_lib, "plan_opts", _lib.FgPlanOpts(tile_major=1))
    tiled, text = _spmm(adj, x, P, T)
    assert "tile-by-tile copy" in text
    assert np.array_equal(plain, tiled)
    assert_sum_close(tiled, oracle.spmm_f64(adj, x), spmm_mass(adj, x), "F=%d P=%d T=%d" % (feat_len, P, T))


def test_spmm_copy_is_reused_across_shapes(oracle, monkeypatch):
    """One module, rebuilt for a longer and then a shorter feature length: the copy's buffer grows and is reused."""
    import torch
    from featgraph_amd import _lib
    from featgraph_amd.module import VanillaSpMMhip, placeholder
    monkeypatch.setattr(_lib, "plan_opts", _lib.FgPlanOpts(tile_major=1))
    rng = np.random.default_rng(5)
    adj = _graph(rng)
    m = VanillaSpMMhip(adj, 2)
    for feat_len, T in ((128, 2), (512, 8), (256, 4), (512, 8)):
        x = rng.standard_normal((adj.shape[1], feat_len)).astype("float32")
        m.build([placeholder(x.shape)], {'num_feat_partitions': T}, {'num_src_partitions': None})
        got = m.run([torch.from_numpy(x).cuda()]).cpu().numpy()
        assert_sum_close(got, oracle.spmm_f64(adj, x), spmm_mass(adj, x), "F=%d" % feat_len)


@pytest.mark.parametrize("H,D", [(4, 64), (8, 32), (4, 16), (2, 128)])
def test_per_head_weights_copy_equals_row_major(oracle, monkeypatch, H, D):
    import torch
    from featgraph_amd import _lib
    from featgraph_amd.module import GSpMMhip, placeholder
    rng = np.random.default_rng(H * 100 + D)
    adj = _graph(rng)
    x = rng.standard_normal((adj.shape[1], H, D)).astype("float32")
    w = rng.standard_normal((adj.nnz, H)).astype("float32")

    def run():
        m = GSpMMhip(adj, 2)
        m.build([placeholder(x.shape), placeholder(w.shape)], {}, {})
        return m.run([torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()]).cpu().numpy().copy()

    monkeypatch.setattr(_lib, "plan_opts", _lib.FgPlanOpts(tile_major=2))
    plain = run()
    monkeypatch.setattr(_lib, "plan_opts", _lib.FgPlanOpts(tile_major=1))
    tiled = run()
    assert np.array_equal(plain, tiled)
    want = oracle.gspmm(adj.indptr, adj.indices, w, x, "sum")
    np.testing.assert_allclose(tiled.reshape(want.shape), want, rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("H,D,P,T", [(1, 128, 2, 2), (1, 512, 3, 8), (1, 512, 4, 4), (1, 256, 2, 2), (4, 32, 2, 2), (8, 64, 2, 8),
                                     (8, 64, 3, 4), (1, 2048, 2, 16)])
def test_sddmm_copy_equals_row_major(oracle, monkeypatch, H, D, P, T):
    import torch
    from featgraph_amd import _lib
    from featgraph_amd.module import MultiHeadSDDMMhip, VanillaSDDMMhip, placeholder
    rng = np.random.default_rng(H * 10 + D + P)
    adj = _graph(rng)
    shp = (H, D) if H > 1 else (D,)
    src = rng.standard_normal((adj.shape[1],) + shp).astype("float32")
    dst = rng.standard_normal((adj.shape[0],) + shp).astype("float32")

    def run():
        m = (MultiHeadSDDMMhip if H > 1 else VanillaSDDMMhip)(adj)
        m.build([placeholder(src.shape), placeholder(dst.shape)], {},
                {'order': 'tiled', 'num_src_partitions': P, 'num_feat_tiles': T})
        return m.run([torch.from_numpy(src).cuda(), torch.from_numpy(dst).cuda()]).cpu().numpy().copy()

    monkeypatch.setattr(_lib, "plan_opts", _lib.FgPlanOpts(tile_major=2))
    plain = run()
    monkeypatch.setattr(_lib, "plan_opts", _lib.FgPlanOpts(tile_major=1))
    tiled = run()
    assert np.array_equal(plain, tiled)
    coo = adj.tocoo()
    want = oracle.sddmm_multihead_f64(coo.row, coo.col, src, dst) if H > 1 else oracle.sddmm_f64(coo.row, coo.col, src, dst)
    assert_sum_close(tiled, want, sddmm_mass(coo.row, coo.col, src, dst), "H=%d D=%d" % (H, D))


@pytest.mark.parametrize("reduce", ["max", "min"])
@pytest.mark.parametrize("feat_len", [128, 256, 512])
def test_extreme_aggregation_copy_equals_row_major(oracle, monkeypatch, reduce, feat_len):
    """max / min gather from the copy too; the positions of the selected elements are found by a second
    sweep over the caller's matrix and must still match."""
    import torch
    from featgraph_amd import _lib
    from featgraph_amd.module import GSpMMhip, placeholder
    rng = np.random.default_rng(feat_len)
    adj = _graph(rng)
    x = rng.standard_normal((adj.shape[1], feat_len)).astype("float32")

    def run():
        m = GSpMMhip(adj)
        m.build([placeholder(x.shape)], {'reduce': reduce, 'msg': 'u_mul_e', 'return_arg': True}, {})
        out = m.run([torch.from_numpy(x).cuda()]).cpu().numpy().copy()
        return out, m.arg_tvm.cpu().numpy().copy()

    monkeypatch.setattr(_lib, "plan_opts", _lib.FgPlanOpts(tile_major=2))
    plain, plain_arg = run()
    monkeypatch.setattr(_lib, "plan_opts", _lib.FgPlanOpts(tile_major=1))
    tiled, tiled_arg = run()
    assert np.array_equal(plain, tiled) and np.array_equal(plain_arg, tiled_arg)
    ref_out, ref_arg = oracle.gspmm_arg(adj.indptr, adj.indices, adj.data, x, reduce, 2)
    assert np.array_equal(tiled, ref_out) and np.array_equal(tiled_arg, ref_arg)
