"""GPU parity tests of SDDMM (single- and multi-head): the gfx950 kernels, called through the
module layer and the C ABI, against the CPU oracle and the reference's numpy check
(tests/test_module_sddmm.py:34-37, rtol = atol = 1e-4).  The bar used against the float64
closed form is rel 1e-4 / abs 1e-5 (plus a rounding allowance proportional to the summed
mass, see helpers.assert_sum_close)."""
import numpy as np
import pytest
import scipy.sparse as sp

from helpers import RTOL, ATOL, assert_sum_close, sddmm_mass

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_cuda():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a ROCm device"
    return torch


def _rand_coo(rng, n_rows, n_cols, density, shuffle=False):
    a = sp.random(n_rows, n_cols, density=density, format="csr", random_state=rng).astype("int32")
    a.sort_indices()
    c = a.tocoo()
    if shuffle:
        p = rng.permutation(c.nnz)
        c = sp.coo_matrix((c.data[p], (c.row[p], c.col[p])), shape=c.shape)
    return c


def _run(torch, cls, adj, src, dst, compute_args, schedule_args, *ctor):
    from featgraph_amd.module import placeholder
    m = cls(adj, *ctor)
    m.build([placeholder(src.shape), placeholder(dst.shape)], compute_args, schedule_args)
    out = m.run([torch.from_numpy(src).cuda(), torch.from_numpy(dst).cuda()])
    return m, out


@pytest.mark.parametrize("feat_len,num_feat_partitions,R,C", [(128, 1, 1, 1), (128, 4, 1, 1), (128, 4, 4, 4)])
def test_reference_x86_cases(torch_cuda, oracle, feat_len, num_feat_partitions, R, C):
    """tests/test_module_sddmm.py:39-41 on the reference's 127 x 255, density 0.1 graph."""
    from featgraph.module import VanillaSDDMMx86
    rng = np.random.default_rng(200)
    coo = _rand_coo(rng, 127, 255, 0.1)
    data_before = coo.data.copy()
    src = rng.random((255, feat_len)).astype("float32")      # (num_cols, F), gathered by col
    dst = rng.random((127, feat_len)).astype("float32")      # (num_rows, F), gathered by row
    m, out = _run(torch_cuda, VanillaSDDMMx86, coo, src, dst, {'num_feat_partitions': num_feat_partitions},
                  {'num_feat_partitions': num_feat_partitions}, R, C)
    out = out.cpu().numpy()
    # the reference's knob is honoured: T feature tiles handled by different workgroups
    from featgraph_amd.module import placeholder
    text = m.lower_to_ir([placeholder(src.shape), placeholder(dst.shape)], {'num_feat_partitions': num_feat_partitions},
                         {'num_feat_partitions': num_feat_partitions})
    if num_feat_partitions > 1:
        assert "x %d feature tile(s) of %d floats" % (num_feat_partitions, feat_len // num_feat_partitions) in text, text
    else:
        assert "feature tile(s)" not in text, text
    if R != 1 or C != 1:
        # stored edge order and the mapping are bit-exact with the reference's partitioner
        eid, prow, pcol = oracle.partition_coo_2d(coo, R, C)
        assert np.array_equal(m._adj_row_indices_dev.cpu().numpy(), prow)
        assert np.array_equal(m._adj_col_indices_dev.cpu().numpy(), pcol)
        assert np.array_equal(m.edge_mapping, np.argsort(eid))
        out = out[m.edge_mapping]
    else:
        with pytest.raises(AssertionError):
            m.edge_mapping
    assert np.array_equal(coo.data, data_before)
    expect = (src[coo.col] * dst[coo.row]).sum(axis=-1)
    np.testing.assert_allclose(expect, out, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(out, oracle.sddmm_x86(coo.row, coo.col, src, dst, num_feat_partitions), rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(out, oracle.sddmm_f64(coo.row, coo.col, src, dst), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("num_cuda_blocks", [32, 256])
def test_reference_cuda_cases(torch_cuda, oracle, num_cuda_blocks):
    """tests/test_module_sddmm.py:69-70."""
    from featgraph.module import VanillaSDDMMcuda
    rng = np.random.default_rng(201)
    coo = _rand_coo(rng, 127, 255, 0.1)
    src = rng.random((255, 128)).astype("float32")
    dst = rng.random((127, 128)).astype("float32")
    m, out = _run(torch_cuda, VanillaSDDMMcuda, coo, src, dst, {}, {'num_cuda_blocks': num_cuda_blocks})
    out = out.cpu().numpy()
    expect = (src[coo.col] * dst[coo.row]).sum(axis=-1)
    np.testing.assert_allclose(expect, out, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(out, oracle.sddmm_x86(coo.row, coo.col, src, dst), rtol=RTOL, atol=ATOL)
    with pytest.raises(AssertionError):
        m.edge_mapping
    with pytest.raises(AssertionError):
        m.build(m._placeholders, {}, {'num_cuda_blocks': coo.nnz + 1})


@pytest.mark.parametrize("order", ["csr", "coo", "shuffled"])
@pytest.mark.parametrize("feat_len", [1, 3, 4, 8, 20, 32, 33, 64, 100, 128, 256, 260, 512, 1024, 1028, 2000])
def test_feature_lengths(torch_cuda, oracle, feat_len, order):
    """Every kernel shape in every edge order (row pieces, stored order with and without equal
    rows adjacent), rows longer than the split threshold, rows without edges."""
    from featgraph_amd.module import VanillaSDDMMhip
    rng = np.random.default_rng(1000 + feat_len)
    coo = _rand_coo(rng, 90, 3000, 0.02).tolil()
    coo[[0, 50, 89], :] = 0
    coo[7, rng.choice(3000, 2600, replace=False)] = 1
    coo = coo.tocsr(); coo.eliminate_zeros(); coo.sort_indices(); coo = coo.tocoo()
    if order == "shuffled":
        p = rng.permutation(coo.nnz)
        coo = sp.coo_matrix((coo.data[p], (coo.row[p], coo.col[p])), shape=coo.shape)
    src = rng.standard_normal((3000, feat_len)).astype("float32")
    dst = rng.standard_normal((90, feat_len)).astype("float32")
    sched = {'order': 'coo'} if order != "csr" else {'order': 'csr'}
    m, out = _run(torch_cuda, VanillaSDDMMhip, coo, src, dst, {}, sched)
    assert m._use_csr == (order == "csr")
    assert_sum_close(out.cpu().numpy(), oracle.sddmm_f64(coo.row, coo.col, src, dst),
                     sddmm_mass(coo.row, coo.col, src, dst), "F=%d %s" % (feat_len, order))


@pytest.mark.parametrize("order", ["csr", "coo"])
@pytest.mark.parametrize("H,D", [(1, 32), (4, 32), (4, 64), (8, 32), (8, 64), (2, 8), (16, 16), (16, 64),
                                 (3, 5), (5, 32), (2, 256), (32, 8)])
def test_multihead(torch_cuda, oracle, H, D, order):
    """Out[e, h] = <Src[col[e], h, :], Dst[row[e], h, :]>.  Parity unpinned by the reference (it
    has no multi-head op): checked against the einsum closed form, the oracle, and H == 1 /
    head-sum reductions to the single-head kernel."""
    from featgraph_amd.module import MultiHeadSDDMMhip, VanillaSDDMMhip
    rng = np.random.default_rng(50 * H + D)
    coo = _rand_coo(rng, 150, 400, 0.08)
    src = rng.standard_normal((400, H, D)).astype("float32")
    dst = rng.standard_normal((150, H, D)).astype("float32")
    m, out = _run(torch_cuda, MultiHeadSDDMMhip, coo, src, dst, {}, {'order': order})
    out = out.cpu().numpy()
    assert out.shape == (coo.nnz, H)
    expect = np.einsum("ehd,ehd->eh", src[coo.col].astype("f8"), dst[coo.row].astype("f8"))
    assert_sum_close(out, expect, sddmm_mass(coo.row, coo.col, src, dst), "H=%d D=%d" % (H, D))
    np.testing.assert_allclose(out, oracle.sddmm_multihead(coo.row, coo.col, src, dst), rtol=1e-4, atol=1e-4)
    _, flat = _run(torch_cuda, VanillaSDDMMhip, coo, src.reshape(400, -1), dst.reshape(150, -1), {}, {'order': order})
    np.testing.assert_allclose(out.sum(1), flat.cpu().numpy(), rtol=1e-4, atol=1e-4)
    if H == 1:
        np.testing.assert_allclose(out[:, 0], flat.cpu().numpy(), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("order", ["csr", "shuffled"])
@pytest.mark.parametrize("feat_len,P,T", [(512, 4, 8), (512, 1, 8), (128, 3, 2), (64, 1, 1), (256, 2, 1), (32, 5, 2),
                                           (1024, 2, 8), (2048, 3, 8), (128, 64, 8)])
def test_tiled_traversal(torch_cuda, oracle, feat_len, P, T, order):
    """Source-column-partitioned, feature-tiled traversal (per-tile partial sums added by a second
    kernel): same values, in the stored edge order, for CSR-ordered and arbitrarily ordered edges."""
    from featgraph_amd.module import VanillaSDDMMhip
    rng = np.random.default_rng(31 * feat_len + P)
    coo = _rand_coo(rng, 140, 1500, 0.03).tolil()
    coo[[0, 70, 139], :] = 0
    coo[9, rng.choice(1500, 1400, replace=False)] = 1          # longer than the split threshold
    coo = coo.tocsr(); coo.eliminate_zeros(); coo.sort_indices(); coo = coo.tocoo()
    if order == "shuffled":
        p = rng.permutation(coo.nnz)
        coo = sp.coo_matrix((coo.data[p], (coo.row[p], coo.col[p])), shape=coo.shape)
    src = rng.standard_normal((1500, feat_len)).astype("float32")
    dst = rng.standard_normal((140, feat_len)).astype("float32")
    m, out = _run(torch_cuda, VanillaSDDMMhip, coo, src, dst, {},
                  {'order': 'tiled', 'num_src_partitions': P, 'num_feat_tiles': T})
    assert m._tiled is not None and "tiled" in m.lower_to_ir(m._placeholders, {}, {'order': 'tiled'})
    m.out_tvm.fill_(float("nan"))
    out = m.run([torch_cuda.from_numpy(src).cuda(), torch_cuda.from_numpy(dst).cuda()]).cpu().numpy()
    assert_sum_close(out, oracle.sddmm_f64(coo.row, coo.col, src, dst), sddmm_mass(coo.row, coo.col, src, dst),
                     "F=%d P=%d T=%d %s" % (feat_len, P, T, order))


@pytest.mark.parametrize("H,D,P,T", [(8, 64, 4, 8), (4, 32, 2, 2), (8, 32, 3, 1), (2, 8, 2, 1), (4, 64, 1, 4),
                                     (16, 16, 2, 4), (4, 256, 2, 4),
                                     # one staged head per tile with head counts that are (12) and are not (5, 6) multiples of 4:
                                     # the 128-bit and the one-thread-per-edge form of the last kernel, tiles launched 8 + 4, 4 + 1, 4 + 2
                                     (12, 64, 2, 12), (5, 64, 2, 5), (6, 64, 3, 6), (8, 128, 2, 8),
                                     # all heads in one 256-float tile (16 heads of 16 floats)
                                     (16, 16, 3, 1)])
def test_tiled_multihead(torch_cuda, oracle, H, D, P, T):
    """Whole heads per feature tile: results go straight to out[edge, head], or (one head per tile,
    four heads or more) through a per-tile staging array and a last kernel that writes each edge's heads."""
    from featgraph_amd.module import MultiHeadSDDMMhip
    rng = np.random.default_rng(H * 1000 + D)
    coo = _rand_coo(rng, 150, 900, 0.05, shuffle=True)
    src = rng.standard_normal((900, H, D)).astype("float32")
    dst = rng.standard_normal((150, H, D)).astype("float32")
    m, out = _run(torch_cuda, MultiHeadSDDMMhip, coo, src, dst, {},
                  {'order': 'tiled', 'num_src_partitions': P, 'num_feat_tiles': T})
    assert m._tiled is not None
    expect = np.einsum("ehd,ehd->eh", src[coo.col].astype("f8"), dst[coo.row].astype("f8"))
    assert_sum_close(out.cpu().numpy(), expect, sddmm_mass(coo.row, coo.col, src, dst), "H=%d D=%d" % (H, D))


def test_tiled_rejects_bad_shapes(torch_cuda):
    from featgraph_amd.module import VanillaSDDMMhip, MultiHeadSDDMMhip, placeholder
    rng = np.random.default_rng(1)
    coo = _rand_coo(rng, 20, 30, 0.3)
    torch = torch_cuda
    for cls, shp, T in ((VanillaSDDMMhip, (100,), 1), (VanillaSDDMMhip, (96,), 2), (MultiHeadSDDMMhip, (2, 128), 4),
                        (MultiHeadSDDMMhip, (3, 20), 1)):
        m = cls(coo)
        with pytest.raises(ValueError):          # refused at build(), where the traversal's scratch is sized
            m.build([placeholder((30,) + shp), placeholder((20,) + shp)], {}, {'order': 'tiled', 'num_feat_tiles': T})


@pytest.mark.parametrize("R,C", [(1, 5), (3, 1), (4, 4), (7, 2), (127, 255)])
def test_partitioned_orders(torch_cuda, oracle, R, C):
    """COO order, CSR order and every 2-D partitioned order give the same values after
    edge_mapping; num_col_partitions is honoured."""
    from featgraph_amd.module import VanillaSDDMMhip
    rng = np.random.default_rng(17)
    coo = _rand_coo(rng, 127, 255, 0.1, shuffle=True)
    src = rng.standard_normal((255, 64)).astype("float32")
    dst = rng.standard_normal((127, 64)).astype("float32")
    m, out = _run(torch_cuda, VanillaSDDMMhip, coo, src, dst, {}, {}, R, C)
    eid, prow, pcol = oracle.partition_coo_2d(coo, R, C)
    assert np.array_equal(m._adj_row_indices, prow) and np.array_equal(m._adj_col_indices, pcol)
    got = out.cpu().numpy()[m.edge_mapping]
    assert_sum_close(got, oracle.sddmm_f64(coo.row, coo.col, src, dst), sddmm_mass(coo.row, coo.col, src, dst))
    _, plain = _run(torch_cuda, VanillaSDDMMhip, coo, src, dst, {}, {})
    np.testing.assert_allclose(got, plain.cpu().numpy(), rtol=RTOL, atol=ATOL)


def test_output_overwritten_empty_and_errors(torch_cuda):
    from featgraph_amd.module import VanillaSDDMMhip, MultiHeadSDDMMhip, placeholder
    torch = torch_cuda
    rng = np.random.default_rng(9)
    coo = _rand_coo(rng, 64, 80, 0.2)
    src = rng.standard_normal((80, 24)).astype("float32")
    dst = rng.standard_normal((64, 24)).astype("float32")
    for order in ("csr", "coo"):
        m = VanillaSDDMMhip(coo)
        m.build([placeholder((80, 24)), placeholder((64, 24))], {}, {'order': order})
        m.out_tvm.fill_(float("nan"))
        o1 = m.run([torch.from_numpy(src).cuda(), torch.from_numpy(dst).cuda()])
        assert np.isfinite(o1.cpu().numpy()).all()
        o2 = m.run([torch.from_numpy(src).cuda(), torch.from_numpy(dst).cuda()])
        assert o2 is o1
        np.testing.assert_allclose(o2.cpu().numpy(), (src[coo.col] * dst[coo.row]).sum(-1), rtol=1e-4, atol=1e-4)
    empty = sp.coo_matrix((64, 80), dtype="int32")
    m = VanillaSDDMMhip(empty)
    m.build([placeholder((80, 24)), placeholder((64, 24))], {}, {})
    assert m.run([torch.from_numpy(src).cuda(), torch.from_numpy(dst).cuda()]).shape == (0,)
    m = VanillaSDDMMhip(coo)
    with pytest.raises(AssertionError):
        m.build([placeholder((80, 24)), placeholder((64, 32))], {}, {})       # dimension mismatch
    with pytest.raises(ValueError):
        m.build([placeholder((64, 24)), placeholder((80, 24))], {}, {})       # operands swapped
    with pytest.raises(TypeError):
        m.build([placeholder((80, 24)), placeholder((64, 24))], {}, {'num_threads_per_cuda_block': 32})
    with pytest.raises(ValueError):
        MultiHeadSDDMMhip(coo).build([placeholder((80, 24)), placeholder((64, 24))], {}, {})
    with pytest.raises(AssertionError):
        VanillaSDDMMhip(coo, 0, 1)
    m.build([placeholder((80, 24)), placeholder((64, 24))], {}, {})
    assert 0 < m.measure_average_time([torch.from_numpy(src).cuda(), torch.from_numpy(dst).cuda()], 3) < 1.0
    assert "sddmm" in m.lower_to_ir([placeholder((80, 24)), placeholder((64, 24))], {}, {})


@pytest.mark.parametrize("feat_len", [32, 128, 512])
def test_powerlaw_23k(torch_cuda, oracle, feat_len):
    from featgraph_amd import synthetic
    from featgraph_amd.module import VanillaSDDMMhip
    indptr, indices = synthetic.make_workload("powerlaw-23k")
    n = indptr.shape[0] - 1
    adj = sp.csr_matrix((np.ones(indices.shape[0], "float32"), indices, indptr), shape=(n, n))
    coo = adj.tocoo()
    rng = np.random.default_rng(4)
    src = rng.standard_normal((n, feat_len)).astype("float32")
    dst = rng.standard_normal((n, feat_len)).astype("float32")
    ref = oracle.sddmm_f64(coo.row, coo.col, src, dst)
    mass = sddmm_mass(coo.row, coo.col, src, dst)
    ref32 = oracle.sddmm_x86(coo.row, coo.col, src, dst)
    tiles = max(1, feat_len // 64)
    for sched, ctor in (({'order': 'csr'}, ()), ({'order': 'coo'}, ()), ({}, (8, 8)),
                        ({'order': 'tiled', 'num_src_partitions': 4, 'num_feat_tiles': tiles}, ()),
                        ({'order': 'tiled', 'num_src_partitions': 16, 'num_feat_tiles': tiles}, (3, 3))):
        m, out = _run(torch_cuda, VanillaSDDMMhip, coo, src, dst, {}, sched, *ctor)
        got = out.cpu().numpy()
        if ctor:
            got = got[m.edge_mapping]
        assert_sum_close(got, ref, mass, str(sched))
        assert np.abs(got - ref).max() <= 4 * max(np.abs(ref32 - ref).max(), ATOL)


def test_full_size_properties(torch_cuda):
    """232,965 nodes / ~114.8M edges: properties that need no CPU product.  With dst = ones the
    result is the row sum of the gathered src row; CSR-order and COO-order kernels agree
    bit-for-bit is not required, only within tolerance; multi-head sums to single-head."""
    from featgraph_amd import synthetic
    from featgraph_amd.module import VanillaSDDMMhip, MultiHeadSDDMMhip, placeholder
    torch = torch_cuda
    indptr, indices = synthetic.make_workload("powerlaw-233k")
    n = indptr.shape[0] - 1
    nnz = indices.shape[0]
    adj = sp.csr_matrix((np.ones(nnz, "float32"), indices, indptr), shape=(n, n))
    F = 128
    g = torch.Generator(device="cuda"); g.manual_seed(3)
    src = torch.randn((n, F), generator=g, device="cuda")
    dst = torch.randn((n, F), generator=g, device="cuda")
    m = VanillaSDDMMhip(adj)
    m.build([placeholder((n, F)), placeholder((n, F))], {}, {'order': 'csr'})
    assert np.array_equal(m._adj_col_indices_dev.cpu().numpy(), indices)
    col_d = m._adj_col_indices_dev.long()
    row_d = m._adj_row_indices_dev.long()

    ones = torch.ones((n, F), device="cuda")
    out = m.run([src, ones])
    expect = src.double().sum(1)[col_d]
    assert ((out.double() - expect).abs() <= ATOL + RTOL * expect.abs() + 1e-6 * src.double().abs().sum(1)[col_d]).all()

    out_csr = m.run([src, dst]).clone()
    m3 = VanillaSDDMMhip(adj)
    m3.build([placeholder((n, F)), placeholder((n, F))], {}, {})        # default: tiled traversal at this size
    assert m3._tiled is not None
    out_tiled = m3.run([src, dst])
    assert ((out_csr - out_tiled).abs() <= ATOL + RTOL * out_tiled.abs() + 1e-4).all()
    del m3, out_tiled
    m2 = VanillaSDDMMhip(adj)
    m2.build([placeholder((n, F)), placeholder((n, F))], {}, {'order': 'coo'})
    out_coo = m2.run([src, dst])
    assert ((out_csr - out_coo).abs() <= ATOL + RTOL * out_coo.abs() + 1e-4).all()
    # a sample of edges against float64 on the device
    pick = torch.randint(0, nnz, (200000,), generator=g, device="cuda")
    ref = (src[col_d[pick]].double() * dst[row_d[pick]].double()).sum(1)
    mass = (src[col_d[pick]].double() * dst[row_d[pick]].double()).abs().sum(1)
    assert ((out_csr[pick].double() - ref).abs() <= ATOL + RTOL * ref.abs() + 1e-6 * mass).all()
    # first and last stored edge
    for e in (0, nnz - 1):
        r = (src[col_d[e]].double() * dst[row_d[e]].double()).sum()
        assert abs(out_csr[e].item() - r.item()) <= 1e-3
    del m2, out_coo
    mh = MultiHeadSDDMMhip(adj)
    mh.build([placeholder((n, 4, 32)), placeholder((n, 4, 32))], {}, {})
    out_mh = mh.run([src.view(n, 4, 32), dst.view(n, 4, 32)])
    assert out_mh.shape == (nnz, 4)
    assert ((out_mh.sum(1) - out_csr).abs() <= ATOL + RTOL * out_csr.abs() + 1e-4).all()


@pytest.mark.parametrize("feat_len", [30, 100, 200, 300])
@pytest.mark.parametrize("shuffle", [False, True])
def test_awkward_feature_lengths_run_on_padded_copies(torch_cuda, oracle, feat_len, shuffle):
    """Rows whose length is no multiple of 32 run at the next friendly length on zero-padded copies of both operands
    once the graph is large enough for that to pay: the same dot products, to rounding."""
    from featgraph_amd import tuning
    from featgraph_amd.module import VanillaSDDMMhip
    rng = np.random.default_rng(70 + feat_len)
    coo = _rand_coo(rng, 2500, 4000, 0.07, shuffle=shuffle)
    assert coo.nnz * feat_len >= tuning.PAD_MIN_GATHERED
    src = rng.standard_normal((4000, feat_len)).astype("float32")
    dst = rng.standard_normal((2500, feat_len)).astype("float32")
    ref, mass = oracle.sddmm_f64(coo.row, coo.col, src, dst), sddmm_mass(coo.row, coo.col, src, dst)
    m, out = _run(torch_cuda, VanillaSDDMMhip, coo, src, dst, {}, {})
    assert m._pad_from == feat_len and m._head_len == tuning.padded_feature_len(feat_len)
    got = out.cpu().numpy()
    assert_sum_close(got, ref, mass, "padded F=%d" % feat_len)
    plain, out2 = _run(torch_cuda, VanillaSDDMMhip, coo, src, dst, {}, {'pad_features': False})
    assert plain._pad_from is None
    assert_sum_close(out2.cpu().numpy(), ref, mass, "unpadded F=%d" % feat_len)
    m.out_tvm.fill_(float("nan"))
    assert np.array_equal(m.run([torch_cuda.from_numpy(src).cuda(), torch_cuda.from_numpy(dst).cuda()]).cpu().numpy(), got)


@pytest.mark.parametrize("H,D", [(3, 20), (8, 48), (2, 100)])
def test_awkward_head_lengths_run_on_padded_copies(torch_cuda, oracle, H, D):
    """Heads whose length is neither a power of two nor a multiple of 64 are zero-padded to the next such length."""
    from featgraph_amd import tuning
    from featgraph_amd.module import MultiHeadSDDMMhip
    rng = np.random.default_rng(H * 1000 + D)
    coo = _rand_coo(rng, 2500, 4000, 0.07)
    assert coo.nnz * H * D >= tuning.PAD_MIN_GATHERED
    src = rng.standard_normal((4000, H, D)).astype("float32")
    dst = rng.standard_normal((2500, H, D)).astype("float32")
    m, out = _run(torch_cuda, MultiHeadSDDMMhip, coo, src, dst, {}, {})
    assert m._pad_from == D and m._head_len == tuning.padded_head_len(D) and tuple(out.shape) == (coo.nnz, H)
    assert_sum_close(out.cpu().numpy(), oracle.sddmm_multihead_f64(coo.row, coo.col, src, dst),
                     sddmm_mass(coo.row, coo.col, src, dst), "padded heads %dx%d" % (H, D))
    plain, out2 = _run(torch_cuda, MultiHeadSDDMMhip, coo, src, dst, {}, {'pad_features': False})
    assert plain._pad_from is None
    assert_sum_close(out2.cpu().numpy(), oracle.sddmm_multihead_f64(coo.row, coo.col, src, dst),
                     sddmm_mass(coo.row, coo.col, src, dst), "unpadded heads %dx%d" % (H, D))
