"""The benchmark's own configurations at full size: 232,965 nodes / ~114.8M edges.

The CPU oracle would need minutes per product here, so the checks are the size-independent ones:
closed forms (dst = ones gives the gathered rows' sums), a 200,000-edge sample against float64
formed on the device, agreement of two different kernels (the tiled traversal over the
source-column-partitioned edge list against the CSR-order kernel), and head sums against the flat
single-head product.  Tolerance: rel 1e-4 / abs 1e-5 plus the rounding allowance 8 * eps32 * sum of
|terms| (the bar of helpers.assert_sum_close, evaluated on the device).
"""
import numpy as np
import pytest
import scipy.sparse as sp

from helpers import RTOL, ATOL, MASS_FACTOR

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def graph():
    import torch
    from featgraph_amd import synthetic
    assert torch.cuda.is_available()
    indptr, indices = synthetic.make_workload("powerlaw-233k")
    n = indptr.shape[0] - 1
    adj = sp.csr_matrix((np.ones(indices.shape[0], "float32"), indices, indptr), shape=(n, n))
    return adj, n, indices.shape[0]


def _close(got, ref64, mass):
    return ((got.double() - ref64).abs() <= ATOL + RTOL * ref64.abs() + MASS_FACTOR * mass).all().item()


@pytest.fixture(scope="module")
def weighted(graph):
    """The benchmark's weighted adjacency (weights U[0, 1), seed 1), one SpMM and one SDDMM module that every
    feature length re-builds, and the graph's arrays on the device."""
    import torch
    from featgraph_amd.module import VanillaSpMMhip, VanillaSDDMMhip
    adj, n, nnz = graph
    g = torch.Generator(device="cuda"); g.manual_seed(1)
    vals_d = torch.rand(nnz, generator=g, device="cuda", dtype=torch.float32)
    wadj = sp.csr_matrix((vals_d.cpu().numpy(), adj.indices, adj.indptr), shape=adj.shape)
    idx_d = torch.from_numpy(adj.indices).cuda().long()
    rows_d = torch.repeat_interleave(torch.arange(n, device="cuda"), torch.from_numpy(np.diff(adj.indptr)).cuda().long())
    return dict(adj=wadj, n=n, nnz=nnz, vals_d=vals_d, idx_d=idx_d, rows_d=rows_d,
                spmm=VanillaSpMMhip(wadj), sddmm=VanillaSDDMMhip(wadj))


# what the cost model picks on this graph (partitions, tiles; SpMM tiles 0 = the kernel's own single tile):
# 16-bit ids and several partitions in flight at F <= 128, the tile-by-tile copy of X from F = 256 on
SPMM_DEFAULTS = {32: (4, 0), 64: (8, 0), 128: (8, 2), 256: (8, 4), 512: (8, 8)}
SDDMM_DEFAULTS = {32: (4, 1), 64: (8, 1), 128: (16, 1), 256: (8, 4), 512: (8, 8)}


@pytest.mark.parametrize("F", [32, 64, 128, 256, 512])
def test_spmm_default_tiling_at_every_benchmark_length(weighted, F):
    """Weighted CSR SpMM at every feature length the benchmark names, in the tiling the library picks there:
    all-ones features give the rows' weight sums in every column, the output's column sums equal the weighted
    out-degree contraction of X (a checksum every stored element enters once), five rows against float64."""
    import torch
    from featgraph_amd.benchmark import verify as chk
    from featgraph_amd.module import placeholder
    w = weighted
    n, m = w['n'], w['spmm']
    m.build([placeholder((n, F))], {}, {})
    assert (m._active['P'], m._num_feat_partitions) == SPMM_DEFAULTS[F], m.lower_to_ir([placeholder((n, F))], {}, {})
    indptr = w['adj'].indptr
    m.out_tvm.fill_(float("nan"))
    assert chk.spmm_ones_failures(m.run([torch.ones((n, F), device="cuda")]), indptr, w['vals_d']) == []
    g = torch.Generator(device="cuda"); g.manual_seed(2)
    x = torch.randn((n, F), generator=g, device="cuda")
    m.out_tvm.fill_(float("nan"))
    out = m.run([x])
    assert chk.spmm_failures(out, indptr, w['idx_d'], w['vals_d'], x) == []
    first = out.clone()
    assert torch.equal(m.run([x]), first)                     # repeatable bit for bit


@pytest.mark.parametrize("F", [32, 64, 128, 256, 512])
def test_sddmm_default_tiling_at_every_benchmark_length(weighted, F):
    """SDDMM over the CSR-ordered edges at every feature length the benchmark names, in the traversal the library
    picks there: dst = ones gives the gathered rows' sums on every edge, 200,000 sampled edges against float64."""
    import torch
    from featgraph_amd.benchmark import verify as chk
    from featgraph_amd.module import placeholder
    w = weighted
    n, m = w['n'], w['sddmm']
    phs = [placeholder((n, F)), placeholder((n, F))]
    m.build(phs, {}, {})
    assert m._tiled is not None and (m._tiled[0]['P'], m._tiled[1]) == SDDMM_DEFAULTS[F], m.lower_to_ir(phs, {}, {})
    g = torch.Generator(device="cuda"); g.manual_seed(5)
    src = torch.randn((n, F), generator=g, device="cuda")
    dst = torch.randn((n, F), generator=g, device="cuda")
    m.out_tvm.fill_(float("nan"))
    assert chk.sddmm_ones_failures(m.run([src, torch.ones((n, F), device="cuda")]), w['idx_d'], src) == []
    m.out_tvm.fill_(float("nan"))
    assert chk.sddmm_failures(m.run([src, dst]), w['rows_d'], w['idx_d'], src, dst) == []


def test_sddmm_coo_order_at_feat_512(weighted):
    """The kernel that walks the stored row / col arrays (`order='coo'`), at the headline feature length."""
    import torch
    from featgraph_amd.benchmark import verify as chk
    from featgraph_amd.module import placeholder
    w = weighted
    n, m, F = w['n'], w['sddmm'], 512
    m.build([placeholder((n, F)), placeholder((n, F))], {}, {'order': 'coo'})
    assert m._tiled is None and not m._use_csr
    g = torch.Generator(device="cuda"); g.manual_seed(6)
    src = torch.randn((n, F), generator=g, device="cuda")
    dst = torch.randn((n, F), generator=g, device="cuda")
    m.out_tvm.fill_(float("nan"))
    assert chk.sddmm_ones_failures(m.run([src, torch.ones((n, F), device="cuda")]), w['idx_d'], src) == []
    m.out_tvm.fill_(float("nan"))
    assert chk.sddmm_failures(m.run([src, dst]), w['rows_d'], w['idx_d'], src, dst) == []


def test_sddmm_shuffled_coo_at_feat_128(weighted):
    """The same edges stored in a random order: `order='auto'` sorts them into the tiled traversal and scatters
    every result back to its stored position; checked against float64 on a sample and, edge by edge, against
    the CSR-ordered module's results permuted the same way."""
    import torch
    from featgraph_amd.benchmark import verify as chk
    from featgraph_amd.module import VanillaSDDMMhip, placeholder
    w = weighted
    n, nnz, F = w['n'], w['nnz'], 128
    perm = torch.randperm(nnz, generator=torch.Generator().manual_seed(3))
    perm_d = perm.cuda()
    rows_s, cols_s = w['rows_d'][perm_d], w['idx_d'][perm_d]
    coo = sp.coo_matrix((np.ones(nnz, np.float32), (rows_s.cpu().numpy().astype(np.int32), cols_s.cpu().numpy().astype(np.int32))),
                        shape=(n, n))
    m = VanillaSDDMMhip(coo)
    del coo
    phs = [placeholder((n, F)), placeholder((n, F))]
    m.build(phs, {}, {})
    assert not m._row_sorted and m._tiled is not None and (m._tiled[0]['P'], m._tiled[1]) == SDDMM_DEFAULTS[F]
    g = torch.Generator(device="cuda"); g.manual_seed(8)
    src = torch.randn((n, F), generator=g, device="cuda")
    dst = torch.randn((n, F), generator=g, device="cuda")
    m.out_tvm.fill_(float("nan"))
    out = m.run([src, dst])
    assert chk.sddmm_failures(out, rows_s, cols_s, src, dst) == []
    ordered = w['sddmm']
    ordered.build(phs, {}, {})
    ref = ordered.run([src, dst])
    # the tiled traversal visits an edge's features in the same order whichever way the edges are stored
    assert torch.equal(out, ref[perm_d])


def test_sddmm_default_at_feat_512(graph):
    """What bench.py times: the tile-by-tile copy of Src, 8 partitions x 8 tiles, the sum over tiles."""
    import torch
    from featgraph_amd.module import VanillaSDDMMhip, placeholder
    adj, n, nnz = graph
    F = 512
    g = torch.Generator(device="cuda"); g.manual_seed(5)
    src = torch.randn((n, F), generator=g, device="cuda")
    dst = torch.randn((n, F), generator=g, device="cuda")
    m = VanillaSDDMMhip(adj)
    m.build([placeholder((n, F)), placeholder((n, F))], {}, {})
    text = m.lower_to_ir([placeholder((n, F)), placeholder((n, F))], {}, {})
    assert m._tiled is not None and m._tiled[1] == 8 and m._tiled[0]['P'] == 8, text
    col_d, row_d = m._adj_col_indices_dev.long(), m._adj_row_indices_dev.long()

    # dst = ones: every edge's result is the sum of its source row
    m.out_tvm.fill_(float("nan"))
    out = m.run([src, torch.ones((n, F), device="cuda")])
    row_sum = src.double().sum(1)
    row_mass = src.double().abs().sum(1)
    assert _close(out, row_sum[col_d], row_mass[col_d])

    # a sample of edges against float64
    m.out_tvm.fill_(float("nan"))
    out = m.run([src, dst])
    assert torch.isfinite(out).all().item()
    pick = torch.randint(0, nnz, (200000,), generator=g, device="cuda")
    pick[0], pick[1] = 0, nnz - 1
    prod = src[col_d[pick]].double() * dst[row_d[pick]].double()
    assert _close(out[pick], prod.sum(1), prod.abs().sum(1))
    del prod

    # the CSR-order kernel (one wavefront per row piece, no tiles, no partial sums) on every edge
    out_tiled = out.clone()
    m2 = VanillaSDDMMhip(adj)
    m2.build([placeholder((n, F)), placeholder((n, F))], {}, {'order': 'csr'})
    assert m2._tiled is None
    out_csr = m2.run([src, dst])
    # two fp32 results, each within the allowance of the exact value; sum |terms| <= |a| |b| (Cauchy-Schwarz)
    bound = src.double().norm(dim=1)[col_d] * dst.double().norm(dim=1)[row_d]
    assert ((out_tiled.double() - out_csr.double()).abs() <= ATOL + RTOL * out_csr.double().abs()
            + 2 * MASS_FACTOR * bound).all().item()
    # repeatable bit for bit
    assert torch.equal(m.run([src, dst]), out_tiled)


@pytest.mark.parametrize("H,D", [(4, 64), (8, 32), (8, 64)])
def test_multihead_shapes(graph, H, D):
    import torch
    from featgraph_amd.module import VanillaSDDMMhip, MultiHeadSDDMMhip, placeholder
    adj, n, nnz = graph
    F = H * D
    g = torch.Generator(device="cuda"); g.manual_seed(H * 100 + D)
    src = torch.randn((n, H, D), generator=g, device="cuda")
    dst = torch.randn((n, H, D), generator=g, device="cuda")
    mh = MultiHeadSDDMMhip(adj)
    mh.build([placeholder((n, H, D)), placeholder((n, H, D))], {}, {})
    assert mh._tiled is not None
    mh.out_tvm.fill_(float("nan"))
    out = mh.run([src, dst])
    assert out.shape == (nnz, H) and torch.isfinite(out).all().item()
    col_d, row_d = mh._adj_col_indices_dev.long(), mh._adj_row_indices_dev.long()
    pick = torch.randint(0, nnz, (200000,), generator=g, device="cuda")
    pick[0], pick[1] = 0, nnz - 1
    prod = src[col_d[pick]].double() * dst[row_d[pick]].double()                        # [S, H, D]
    assert _close(out[pick], prod.sum(2), prod.abs().sum(2))
    del prod
    # the heads' sum is the flat single-head product (another kernel configuration: tile sums)
    flat = VanillaSDDMMhip(adj)
    flat.build([placeholder((n, F)), placeholder((n, F))], {}, {})
    out_flat = flat.run([src.view(n, F), dst.view(n, F)])
    bound = src.view(n, F).double().norm(dim=1)[col_d] * dst.view(n, F).double().norm(dim=1)[row_d]
    head_sum = out.double().sum(1)
    assert ((head_sum - out_flat.double()).abs() <= ATOL + RTOL * out_flat.double().abs()
            + 2 * MASS_FACTOR * bound).all().item()


def test_broadcasting_operators_at_full_size(graph):
    """Closed forms that need no CPU pass over 114.8M edges: the sum of all-ones edge features is the row's degree;
    edge features that repeat one weight per edge give the weighted SpMM; an all-ones edge operand leaves the
    destination rows' features on the edges."""
    import torch
    from featgraph_amd.module import GSpMMhip, GSDDMMhip, VanillaSpMMhip, placeholder
    adj, n, nnz = graph
    F = 16
    g = torch.Generator(device="cuda"); g.manual_seed(7)
    deg = torch.from_numpy(np.diff(adj.indptr).astype(np.float32)).cuda()
    ones = torch.ones((nnz, F), device="cuda")
    m = GSpMMhip(adj)
    m.build([placeholder((nnz, F))], {'msg': 'copy_e', 'reduce': 'sum'}, {})
    m.out_tvm.fill_(float("nan"))
    out = m.run([ones])
    assert torch.equal(out, deg[:, None].expand(n, F))               # integers below 2^24: exact in any order
    m.build([placeholder((nnz, F))], {'msg': 'copy_e', 'reduce': 'max', 'return_arg': True}, {})
    out = m.run([ones])
    assert torch.equal(out, (deg > 0).float()[:, None].expand(n, F))
    first = torch.from_numpy(adj.indptr[:-1].astype(np.int32)).cuda()
    want_arg = torch.where(deg > 0, first, torch.full_like(first, -1))
    assert torch.equal(m.arg_tvm, want_arg[:, None].expand(n, F))     # ties: the row's first edge
    del ones

    w = torch.rand(nnz, generator=g, device="cuda")
    x = torch.randn((n, F), generator=g, device="cuda")
    ef = w[:, None].expand(nnz, F).contiguous()
    m.build([placeholder((n, F)), placeholder((nnz, F))], {'msg': 'u_mul_e', 'reduce': 'sum'}, {})
    out = m.run([x, ef]).clone()
    wadj = sp.csr_matrix((w.cpu().numpy(), adj.indices, adj.indptr), shape=adj.shape)
    plain = VanillaSpMMhip(wadj)
    plain.build([placeholder((n, F))], {}, {})
    ref = plain.run([x])
    mass = VanillaSpMMhip(wadj)
    mass.build([placeholder((n, F))], {}, {})
    row_mass = mass.run([x.abs()]).double()
    assert ((out.double() - ref.double()).abs() <= ATOL + RTOL * ref.double().abs() + 2 * MASS_FACTOR * row_mass).all().item()
    del ef

    y = torch.randn((n, F), generator=g, device="cuda")
    e1 = torch.ones((nnz, 1), device="cuda")
    gs = GSDDMMhip(adj.tocoo())
    gs.build([placeholder((nnz, 1)), placeholder((n, F))], {'op': 'mul', 'lhs_target': 'e', 'rhs_target': 'v'}, {})
    gs.out_tvm.fill_(float("nan"))
    out = gs.run([e1, y])
    rows = gs._adj_row_indices_dev.long()
    pick = torch.randint(0, nnz, (500000,), generator=g, device="cuda")
    pick[0], pick[1] = 0, nnz - 1
    assert torch.equal(out[pick], y[rows[pick]])
    assert torch.isfinite(out).all().item()
