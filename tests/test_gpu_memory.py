"""What the module classes keep on the device: uploads happen at build() and only for what the built configuration
reads, partitioned copies that a re-build no longer uses are freed, and an SDDMM module can run its tiled traversal on an
SpMM module's partitioned copy, plan and scratch (share_layouts) with bit-identical results."""
import numpy as np
import pytest
import scipy.sparse as sp

from helpers import assert_sum_close, spmm_mass, sddmm_mass

pytestmark = pytest.mark.gpu


def _graph(rng, n_rows=400, n_cols=3000):
    a = sp.random(n_rows, n_cols, density=0.02, format="csr", random_state=rng).astype("float32").tolil()
    a[[0, 11], :] = 0
    a[5, rng.choice(n_cols, size=min(2500, n_cols - 20), replace=False)] = 1.0     # longer than the split threshold where the matrix is wide enough
    a = a.tocsr().astype("float32"); a.eliminate_zeros(); a.sort_indices()
    a.data = (rng.random(a.nnz) + 0.1).astype("float32")
    return a


def test_uploads_follow_the_built_configuration(oracle):
    import torch
    from featgraph_amd.module import VanillaSpMMhip, VanillaSDDMMhip, placeholder
    rng = np.random.default_rng(1)
    adj = _graph(rng)
    F = 64
    x = rng.standard_normal((adj.shape[1], F)).astype("float32")
    y = rng.standard_normal((adj.shape[0], F)).astype("float32")
    xd, yd = torch.from_numpy(x).cuda(), torch.from_numpy(y).cuda()

    m = VanillaSpMMhip(adj)
    assert m._layouts == {}                                   # nothing on the device before build()
    m.build([placeholder(x.shape)], {}, {'num_src_partitions': 4})
    assert sorted(m._layouts) == [4]                          # the partitioned copy only: no CSR arrays
    before = m.device_bytes()
    assert before['graph'] > 0 and before['plans'] > 0 and before['buffers'] == 4 * adj.shape[0] * F
    out4 = m.run([xd]).cpu().numpy().copy()
    assert_sum_close(out4, oracle.spmm_f64(adj, x), spmm_mass(adj, x), "P=4")
    m.build([placeholder(x.shape)], {}, {'num_src_partitions': 2})
    assert sorted(m._layouts) == [2]                          # the copy for 4 partitions was freed
    assert_sum_close(m.run([xd]).cpu().numpy(), oracle.spmm_f64(adj, x), spmm_mass(adj, x), "P=2")
    m.build([placeholder(x.shape)], {}, {'num_src_partitions': None})
    assert sorted(m._layouts) == [1]
    assert np.array_equal(m._adj_indices_dev.cpu().numpy(), adj.indices)       # the CSR arrays, bit-exact, on first use
    assert_sum_close(m.run([xd]).cpu().numpy(), oracle.spmm_f64(adj, x), spmm_mass(adj, x), "CSR")
    m.build([placeholder(x.shape)], {}, {'num_src_partitions': 4})
    assert sorted(m._layouts) == [1, 4]                       # the CSR arrays stay once they exist
    assert np.array_equal(m.run([xd]).cpu().numpy(), out4)    # and the rebuilt copy gives the same bits

    s = VanillaSDDMMhip(adj)
    s.build([placeholder(x.shape), placeholder(y.shape)], {}, {'order': 'tiled', 'num_src_partitions': 2, 'num_feat_tiles': 1})
    assert '_row_dev' not in s.__dict__ and '_col_dev' not in s.__dict__      # the tiled traversal reads neither
    coo = adj.tocoo()
    ref, mass = oracle.sddmm_f64(coo.row, coo.col, x, y), sddmm_mass(coo.row, coo.col, x, y)
    assert_sum_close(s.run([xd, yd]).cpu().numpy(), ref, mass, "tiled")
    s.build([placeholder(x.shape), placeholder(y.shape)], {}, {'order': 'coo'})
    assert '_row_dev' in s.__dict__ and '_col_dev' in s.__dict__              # uploaded by build(), not by run()
    assert s._dds == {} or sorted(s._dds) == [2]
    assert_sum_close(s.run([xd, yd]).cpu().numpy(), ref, mass, "coo")


@pytest.mark.parametrize("H", [1, 8])
def test_shared_layouts_give_the_same_bits(oracle, H):
    import torch
    from featgraph_amd.module import VanillaSpMMhip, VanillaSDDMMhip, MultiHeadSDDMMhip, placeholder
    rng = np.random.default_rng(2 + H)
    adj = _graph(rng)
    n_dst, n_src = adj.shape
    D = 64
    shape = (D,) if H == 1 else (H, D)
    x = torch.from_numpy(rng.standard_normal((n_src,) + shape).astype("float32")).cuda()
    y = torch.from_numpy(rng.standard_normal((n_dst,) + shape).astype("float32")).cuda()
    xs = x.reshape(n_src, -1)
    cls = VanillaSDDMMhip if H == 1 else MultiHeadSDDMMhip
    sched = {'order': 'tiled', 'num_src_partitions': 4, 'num_feat_tiles': 1 if H == 1 else H}
    phs = [placeholder(tuple(x.shape)), placeholder(tuple(y.shape))]

    own = cls(adj)
    own.build(phs, {}, sched)
    want = own.run([x, y]).clone()

    spmm = VanillaSpMMhip(adj)
    spmm.build([placeholder(tuple(xs.shape))], {}, {'num_src_partitions': 4})
    agg = spmm.run([xs]).clone()
    shared = cls(adj)
    shared.share_layouts(spmm)
    shared.build(phs, {}, sched)
    d = shared._dds[4]
    assert d['plan'] is spmm._layouts[4]['plan'] and d['idx'] is spmm._layouts[4]['idx']
    assert shared.device_bytes()['plans'] < own.device_bytes()['plans']
    assert shared.device_bytes()['graph'] < own.device_bytes()['graph']
    # the two modules take turns on one scratch
    for _ in range(2):
        assert torch.equal(shared.run([x, y]), want)
        assert torch.equal(spmm.run([xs]), agg)
    # the SpMM module keeps a copy that another module uses, whatever it is re-built for ...
    spmm.build([placeholder(tuple(xs.shape))], {}, {'num_src_partitions': 2})
    assert sorted(spmm._layouts) == [2, 4]
    assert torch.equal(shared.run([x, y]), want)
    # ... and frees it once that module is gone and it builds again
    del shared
    spmm.build([placeholder(tuple(xs.shape))], {}, {'num_src_partitions': 2})
    assert sorted(spmm._layouts) == [2]
    # another structure is refused
    other = sp.csr_matrix(adj.shape, dtype="float32").tolil(); other[1, 2] = 1.0
    with pytest.raises(ValueError):
        cls(other.tocsr()).share_layouts(spmm)
    coo = adj.tocoo()
    p = rng.permutation(coo.nnz)
    with pytest.raises(ValueError):
        cls(sp.coo_matrix((coo.data[p], (coo.row[p], coo.col[p])), shape=coo.shape)).share_layouts(spmm)


def test_graph_modules_share_one_set_of_layouts():
    """featgraph_amd.autograd.Graph: the SpMM-like modules of one orientation (weighted sums of several shapes, per-head
    weights, broadcasting messages, max aggregation) use one set of device layouts and plans, and the SDDMM modules take
    theirs from the forward SpMM module; results as from modules of their own."""
    import torch
    from featgraph_amd.autograd import Graph
    from featgraph_amd.module import GSpMMhip, placeholder
    rng = np.random.default_rng(9)
    adj = _graph(rng, 300, 300)
    g = Graph(adj)
    n, nnz = 300, adj.nnz
    gen = torch.Generator(device="cuda"); gen.manual_seed(4)
    x16 = torch.randn((n, 16), generator=gen, device="cuda", requires_grad=True)
    x64 = torch.randn((n, 64), generator=gen, device="cuda", requires_grad=True)
    xh = torch.randn((n, 4, 16), generator=gen, device="cuda", requires_grad=True)
    w = torch.rand(nnz, generator=gen, device="cuda", requires_grad=True)
    wh = torch.rand((nnz, 4), generator=gen, device="cuda", requires_grad=True)
    outs = [g.spmm(x16, w), g.spmm(x64, w), g.spmm(xh, wh), g.aggregate(x16, 'max'), g.gspmm('u_add_e', x16, w.reshape(-1, 1), 'sum'),
            g.sddmm(x64, x64)]
    sum(o.square().sum() for o in outs).backward()
    fwd = [m for k, m in g._mods.items() if isinstance(m, GSpMMhip) and m._adj_scipy_csr is g._csr]
    bwd = [m for k, m in g._mods.items() if isinstance(m, GSpMMhip) and m._adj_scipy_csr is g._tr]
    assert len(fwd) >= 4 and len(bwd) >= 2
    for mods in (fwd, bwd):
        owner = [m for m in mods if getattr(m, '_layout_owner', None) is None]
        assert len(owner) == 1
        assert all(m._layouts is owner[0]._layouts for m in mods)
        assert sum(m.device_bytes()['plans'] > 0 for m in mods) == 1
    # the same numbers as a module of its own gives
    own = GSpMMhip(adj)
    own.build([placeholder((n, 64)), placeholder((nnz,))], {}, {})
    assert torch.equal(own.run([x64.detach(), w.detach()]), outs[1].detach())
    # the gradient of the first weighted sum against torch autograd on the dense matrix
    dense = torch.zeros((n, n), device="cuda", dtype=torch.float64)
    coo = adj.tocoo()
    rows, cols = torch.from_numpy(coo.row.astype(np.int64)).cuda(), torch.from_numpy(coo.col.astype(np.int64)).cuda()
    x2 = x16.detach().double().requires_grad_()
    w2 = w.detach().double().requires_grad_()
    y = torch.zeros((n, 16), device="cuda", dtype=torch.float64).index_add(0, rows, w2[:, None] * x2[cols])
    g2 = Graph(adj)
    x3 = x16.detach().clone().requires_grad_(); w3 = w.detach().clone().requires_grad_()
    g2.spmm(x3, w3).square().sum().backward()
    y.square().sum().backward()
    assert torch.allclose(x3.grad.double(), x2.grad, rtol=1e-4, atol=1e-4) and torch.allclose(w3.grad.double(), w2.grad, rtol=1e-4, atol=1e-4)
