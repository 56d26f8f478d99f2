"""Feature matrices of 4 GiB and more are addressed with 64-bit offsets instead of 32-bit byte offsets
from a scalar base.  That path is exercised here on small inputs (plan option `wide_offsets`), where it
must agree bit for bit with the default path, and once at real size (2.45M x 512 floats = 5.0 GB)."""
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


def _run_spmm(adj, x, P, T):
    import torch
    from featgraph_amd.module import VanillaSpMMhip, placeholder
    m = VanillaSpMMhip(adj, P)
    m.build([placeholder(x.shape)], {'num_feat_partitions': T}, {'num_src_partitions': None})
    return m.run([torch.from_numpy(x).cuda()]).cpu().numpy().copy(), m.lower_to_ir(m._placeholders, {'num_feat_partitions': T}, {'num_src_partitions': None})


@pytest.mark.parametrize("feat_len,P,T", [(4, 1, 0), (32, 1, 0), (64, 3, 0), (100, 1, 0), (128, 2, 2), (512, 4, 8),
                                          (1024, 1, 0), (7, 2, 0)])
def test_spmm_wide_equals_default(oracle, monkeypatch, feat_len, P, T):
    from featgraph_amd import _lib
    rng = np.random.default_rng(feat_len + P)
    adj = _graph(rng)
    x = rng.standard_normal((adj.shape[1], feat_len)).astype("float32")
    base, _ = _run_spmm(adj, x, P, T)
    monkeypatch.setattr(_lib, "plan_opts", _lib.FgPlanOpts(wide_offsets=1))
    wide_out, _ = _run_spmm(adj, x, P, T)
    assert np.array_equal(base, wide_out)
    assert_sum_close(wide_out, oracle.spmm_f64(adj, x), spmm_mass(adj, x), "F=%d P=%d" % (feat_len, P))


@pytest.mark.parametrize("H,D,P,T", [(1, 128, 2, 2), (1, 512, 3, 8), (4, 32, 2, 2), (8, 64, 2, 8), (1, 64, 1, 1)])
def test_sddmm_tiled_wide_equals_default(oracle, monkeypatch, H, D, P, T):
    import torch
    from featgraph_amd import _lib
    from featgraph_amd.module import MultiHeadSDDMMhip, VanillaSDDMMhip, placeholder
    rng = np.random.default_rng(H * 10 + D)
    adj = _graph(rng)
    shp = (H, D) if H > 1 else (D,)
    src = rng.standard_normal((adj.shape[1],) + shp).astype("float32")
    dst = rng.standard_normal((adj.shape[0],) + shp).astype("float32")

    def run():
        m = (MultiHeadSDDMMhip if H > 1 else VanillaSDDMMhip)(adj)
        m.build([placeholder(src.shape), placeholder(dst.shape)], {},
                {'order': 'tiled', 'num_src_partitions': P, 'num_feat_tiles': T})
        return m.run([torch.from_numpy(src).cuda(), torch.from_numpy(dst).cuda()]).cpu().numpy().copy()

    base = run()
    monkeypatch.setattr(_lib, "plan_opts", _lib.FgPlanOpts(wide_offsets=1))
    wide_out = run()
    assert np.array_equal(base, wide_out)
    coo = adj.tocoo()
    ref = oracle.sddmm_multihead_f64(coo.row, coo.col, src, dst) if H > 1 else oracle.sddmm_f64(coo.row, coo.col, src, dst)
    assert_sum_close(wide_out, ref, sddmm_mass(coo.row, coo.col, src, dst), "H=%d D=%d" % (H, D))


def test_five_gigabyte_feature_matrix(oracle):
    """2,450,000 x 512 fp32 = 5.0 GB: past the reach of 32-bit byte offsets.  Sampled rows / edges
    against float64, and the all-ones column sums."""
    import torch
    from featgraph_amd import synthetic
    from featgraph_amd.module import VanillaSpMMhip, VanillaSDDMMhip, placeholder
    indptr, indices = synthetic.make_workload("powerlaw-2.45M")
    n = indptr.shape[0] - 1
    nnz = int(indptr[-1])
    F = 512
    assert n * F * 4 >= 1 << 32
    gen = torch.Generator(device="cuda"); gen.manual_seed(5)
    vals_d = torch.rand(nnz, generator=gen, device="cuda")
    x = torch.randn((n, F), generator=gen, device="cuda")
    vals = vals_d.cpu().numpy()
    adj = sp.csr_matrix((vals, indices, indptr), shape=(n, n))
    m = VanillaSpMMhip(adj)
    m.build([placeholder((n, F))], {}, {})
    out = m.run([x])
    deg = np.diff(indptr)
    rows = [int(np.argmax(deg)), 0, n - 1, n // 2] + list(np.random.default_rng(2).integers(0, n, 40))
    for r in rows:
        b, e = indptr[r], indptr[r + 1]
        cols = torch.from_numpy(indices[b:e].astype(np.int64)).cuda()
        xr = x[cols].double()
        w = vals_d[b:e].double()
        ref = (w[:, None] * xr).sum(0).cpu().numpy()
        mass = (w[:, None] * xr.abs()).sum(0).cpu().numpy()
        assert_sum_close(out[r].cpu().numpy(), ref, mass, "row %d" % r)
    # the last rows of X are reached: every source row is used by its self-loop
    assert torch.isfinite(out).all()
    del m, out
    y = torch.randn((n, F), generator=gen, device="cuda")
    s = VanillaSDDMMhip(adj)
    s.build([placeholder((n, F)), placeholder((n, F))], {}, {})
    sc = s.run([x, y])
    pick = np.random.default_rng(3).integers(0, nnz, 20000)
    pick[:3] = [0, nnz - 1, nnz // 2]
    row_of = np.searchsorted(indptr, pick, side="right") - 1
    pr = torch.from_numpy(row_of.astype(np.int64)).cuda(); pc = torch.from_numpy(indices[pick].astype(np.int64)).cuda()
    prod = x[pc].double() * y[pr].double()
    ref = prod.sum(-1).cpu().numpy(); mass = prod.abs().sum(-1).cpu().numpy()
    assert_sum_close(sc[torch.from_numpy(pick.astype(np.int64)).cuda()].cpu().numpy(), ref, mass, "sampled edges")
