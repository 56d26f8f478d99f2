"""GPU parity tests of SpMM: the gfx950 kernels, called through the module layer and the
C ABI, against the CPU oracle and against scipy (the reference's own check).

Tolerances: the reference's tests use rtol = atol = 1e-4 against csr.dot
(tests/test_module_spmm.py:30); the stricter bar used here is rel 1e-4 / abs 1e-5 against
the float64 product and the fp32 restatement (the summation order differs).
"""
import numpy as np
import pytest
import scipy.sparse as sp

from helpers import RTOL, ATOL, assert_sum_close, spmm_mass

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_cuda():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a ROCm device"
    return torch


def _rand_csr(rng, n_rows, n_cols, density):
    a = sp.random(n_rows, n_cols, density=density, format="csr", random_state=rng,
                  data_rvs=lambda k: rng.random(k)).astype("float32")
    a.sort_indices()
    return a


def _run(torch, cls, adj, x, compute_args, schedule_args, *ctor):
    from featgraph_amd.module import placeholder
    m = cls(adj, *ctor)
    m.build([placeholder(x.shape)], compute_args, schedule_args)
    out = m.run([torch.from_numpy(x).cuda()])
    return m, out


def _adj_with_long_and_empty_rows(rng, n_rows, n_cols, long_len):
    """Random sparse rows + empty rows + one row longer than the split threshold."""
    a = _rand_csr(rng, n_rows, n_cols, 0.02).tolil()
    a[[1, n_rows // 2, n_rows - 1], :] = 0
    cols = rng.choice(n_cols, size=long_len, replace=False)
    a[3, cols] = rng.random(long_len).astype("float32") + 0.1
    a = a.tocsr().astype("float32")
    a.eliminate_zeros()
    a.sort_indices()
    return a


@pytest.mark.parametrize("feat_len,num_col_partitions,num_feat_partitions",
                         [(128, 1, 1), (128, 4, 1), (128, 4, 4)])
def test_reference_x86_cases(torch_cuda, oracle, feat_len, num_col_partitions, num_feat_partitions):
    """tests/test_module_spmm.py:32-34 on the reference's 127 x 255, density 0.1 graph."""
    from featgraph.module import VanillaSpMMx86
    rng = np.random.default_rng(100)
    adj = _rand_csr(rng, 127, 255, 0.1)
    x = rng.random((255, feat_len)).astype("float32")
    m, out = _run(torch_cuda, VanillaSpMMx86, adj, x, {'num_feat_partitions': num_feat_partitions}, {},
                  num_col_partitions)
    out = out.cpu().numpy()
    np.testing.assert_allclose(adj.dot(x), out, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(out, oracle.spmm_f64(adj, x), rtol=RTOL, atol=ATOL)
    if num_col_partitions == 1:
        ref = oracle.spmm_csr_x86(adj.indptr, adj.indices, adj.data, x, num_feat_partitions)
    else:
        s1_pos, s1_idx, vals = oracle.csr_to_dds(adj, num_col_partitions)
        ref = oracle.spmm_dds_x86(s1_pos, s1_idx, vals, x, 127, num_col_partitions, num_feat_partitions)
        # the device copies of the DDS arrays are bit-exact
        assert np.array_equal(m._adj_s1_pos_dev.cpu().numpy(), s1_pos)
        assert np.array_equal(m._adj_s1_idx_dev.cpu().numpy(), s1_idx)
        assert np.array_equal(m._adj_vals_dev.cpu().numpy(), vals)
    np.testing.assert_allclose(out, ref, rtol=RTOL, atol=ATOL)
    assert m.target == 'rocm' and m.ctx.type == 'cuda'


@pytest.mark.parametrize("num_threads_per_cuda_block", [32, 128, None])
def test_reference_cuda_cases(torch_cuda, oracle, num_threads_per_cuda_block):
    """tests/test_module_spmm.py:57-59."""
    from featgraph.module import VanillaSpMMcuda
    rng = np.random.default_rng(101)
    adj = _rand_csr(rng, 127, 255, 0.1)
    x = rng.random((255, 128)).astype("float32")
    m, out = _run(torch_cuda, VanillaSpMMcuda, adj, x, {},
                  {'num_threads_per_cuda_block': num_threads_per_cuda_block})
    out = out.cpu().numpy()
    np.testing.assert_allclose(adj.dot(x), out, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(out, oracle.spmm_csr_rowwise(adj.indptr, adj.indices, adj.data, x), rtol=RTOL, atol=ATOL)
    assert np.array_equal(m._adj_indptr_dev.cpu().numpy(), adj.indptr)
    assert np.array_equal(m._adj_indices_dev.cpu().numpy(), adj.indices)


@pytest.mark.parametrize("feat_len", [1, 2, 3, 4, 5, 12, 17, 32, 36, 64, 100, 128, 200, 256, 257, 512, 600, 1024, 1100])
def test_feature_lengths(torch_cuda, oracle, feat_len):
    """Every kernel shape: vector and scalar lanes, masked tails, 1/2/4 loads per lane, long rows
    split over wavefronts, empty rows."""
    from featgraph_amd.module import VanillaSpMMhip
    rng = np.random.default_rng(feat_len)
    adj = _adj_with_long_and_empty_rows(rng, 300, 4000, 2500)
    x = rng.standard_normal((4000, feat_len)).astype("float32")
    ref64 = oracle.spmm_f64(adj, x)
    m, out = _run(torch_cuda, VanillaSpMMhip, adj, x, {}, {})
    out = out.cpu().numpy()
    assert_sum_close(out, ref64, spmm_mass(adj, x), "F=%d" % feat_len)
    empty = np.diff(adj.indptr) == 0
    assert empty.sum() >= 3 and (out[empty] == 0).all()


@pytest.mark.parametrize("feat_len,T,P", [(512, 8, 1), (512, 2, 1), (512, 16, 3), (96, 3, 1), (96, 96, 2),
                                           (30, 5, 1), (30, 2, 7), (256, 1, 16), (64, 0, 1)])
def test_tilings_and_partitions(torch_cuda, oracle, feat_len, T, P):
    from featgraph_amd.module import VanillaSpMMhip
    rng = np.random.default_rng(7 * feat_len + T + P)
    adj = _adj_with_long_and_empty_rows(rng, 257, 3001, 2900)
    x = rng.standard_normal((3001, feat_len)).astype("float32")
    m, out = _run(torch_cuda, VanillaSpMMhip, adj, x, {'num_feat_partitions': T}, {}, P)
    out = out.cpu().numpy()
    ref64, mass = oracle.spmm_f64(adj, x), spmm_mass(adj, x)
    assert_sum_close(out, ref64, mass, "gpu vs f64")
    if P > 1 and T > 0:
        s1_pos, s1_idx, vals = oracle.csr_to_dds(adj, P)
        ref = oracle.spmm_dds_x86(s1_pos, s1_idx, vals, x, 257, P, T)
        assert_sum_close(ref, ref64, mass, "fp32 restatement vs f64")
        # the GPU's rounding error is of the size of the reference order's own
        assert np.abs(out - ref64).max() <= 4 * max(np.abs(ref - ref64).max(), ATOL)
    text = m.lower_to_ir([__import__("featgraph_amd.module", fromlist=["placeholder"]).placeholder(x.shape)],
                         {'num_feat_partitions': T}, {})
    assert "spmm_items_kernel" in text and "work items" in text


@pytest.mark.parametrize("src_parts", [None, 1, 3, 'auto'])
def test_internal_source_partitions(torch_cuda, oracle, src_parts):
    """The constructor's single partition can be replaced by internal source-column partitions
    at build time; the CSR copy on the device stays bit-exact."""
    from featgraph_amd.module import VanillaSpMMhip
    rng = np.random.default_rng(77)
    adj = _adj_with_long_and_empty_rows(rng, 200, 2500, 1800)
    x = rng.standard_normal((2500, 128)).astype("float32")
    m, out = _run(torch_cuda, VanillaSpMMhip, adj, x, {}, {'num_src_partitions': src_parts})
    assert_sum_close(out.cpu().numpy(), oracle.spmm_f64(adj, x), spmm_mass(adj, x))
    assert np.array_equal(m._adj_indices_dev.cpu().numpy(), adj.indices)
    assert m._active['P'] == (3 if src_parts == 3 else 1)


def test_output_fully_overwritten_and_reused(torch_cuda, oracle):
    """run() returns the same tensor every time and writes every element (no stale data),
    also rows without edges (module/spmm.py:161; te.sum over an empty range is 0)."""
    from featgraph_amd.module import VanillaSpMMhip, placeholder
    torch = torch_cuda
    rng = np.random.default_rng(5)
    adj = _adj_with_long_and_empty_rows(rng, 120, 2000, 1500)
    for P in (1, 3):
        m = VanillaSpMMhip(adj, P)
        m.build([placeholder((2000, 48))], {}, {})
        x1 = rng.standard_normal((2000, 48)).astype("float32")
        x2 = rng.standard_normal((2000, 48)).astype("float32")
        m.out_tvm.fill_(float("nan"))
        o1 = m.run([torch.from_numpy(x1).cuda()])
        r1 = o1.cpu().numpy().copy()
        assert np.isfinite(r1).all()
        m.out_tvm.fill_(1e30)
        o2 = m.run([torch.from_numpy(x2).cuda()])
        assert o2 is o1 and o2.data_ptr() == o1.data_ptr()
        assert_sum_close(r1, oracle.spmm_f64(adj, x1), spmm_mass(adj, x1))
        assert_sum_close(o2.cpu().numpy(), oracle.spmm_f64(adj, x2), spmm_mass(adj, x2))
        # bit-identical on repetition: no atomics, fixed summation order
        again = m.run([torch.from_numpy(x2).cuda()]).cpu().numpy()
        assert np.array_equal(again, o2.cpu().numpy())


def test_exact_special_cases(torch_cuda):
    from featgraph_amd.module import VanillaSpMMhip
    rng = np.random.default_rng(6)
    x = rng.standard_normal((500, 96)).astype("float32")
    eye = sp.identity(500, dtype="float32", format="csr")
    _, out = _run(torch_cuda, VanillaSpMMhip, eye, x, {}, {})
    assert np.array_equal(out.cpu().numpy(), x)
    perm = rng.permutation(500).astype("int32")
    pm = sp.csr_matrix((np.ones(500, "float32"), perm, np.arange(501, dtype="int32")), shape=(500, 500))
    _, out = _run(torch_cuda, VanillaSpMMhip, pm, x, {}, {}, 4)
    assert np.array_equal(out.cpu().numpy(), x[perm])
    # no edges at all, and no rows at all
    zero = sp.csr_matrix((40, 500), dtype="float32")
    _, out = _run(torch_cuda, VanillaSpMMhip, zero, x, {}, {})
    assert out.shape == (40, 96) and (out.cpu().numpy() == 0).all()
    none = sp.csr_matrix((0, 500), dtype="float32")
    _, out = _run(torch_cuda, VanillaSpMMhip, none, x, {}, {})
    assert out.shape == (0, 96)
    # infinities in unrelated source rows must not leak through padded lanes
    xi = x.copy(); xi[0, :] = np.inf
    sel = sp.csr_matrix((np.ones(3, "float32"), np.array([5, 6, 7], "int32"), np.array([0, 3], "int32")), shape=(1, 500))
    _, out = _run(torch_cuda, VanillaSpMMhip, sel, xi, {}, {})
    assert np.isfinite(out.cpu().numpy()).all()


def test_coo_input_and_errors(torch_cuda):
    from featgraph_amd.module import VanillaSpMMhip, VanillaSpMMcuda, placeholder
    torch = torch_cuda
    rng = np.random.default_rng(8)
    adj = _rand_csr(rng, 50, 60, 0.2)
    x = rng.random((60, 16)).astype("float32")
    _, out = _run(torch, VanillaSpMMhip, adj.tocoo(), x, {}, {})
    np.testing.assert_allclose(out.cpu().numpy(), adj.dot(x), rtol=1e-4, atol=1e-4)
    with pytest.raises(AssertionError):
        VanillaSpMMhip(adj, 0)
    with pytest.raises(TypeError):
        VanillaSpMMcuda(adj, 2)
    m = VanillaSpMMhip(adj)
    with pytest.raises(TypeError):
        m.build([placeholder((60, 16))], {'no_such_arg': 1}, {})
    with pytest.raises(ValueError):
        m.build([placeholder((60, 16))], {'num_feat_partitions': 3}, {})
    with pytest.raises(ValueError):
        m.build([placeholder((61, 16))], {}, {})
    with pytest.raises(RuntimeError):
        m.run([torch.from_numpy(x).cuda()])
    m.build([placeholder((60, 16))], {}, {})
    with pytest.raises(ValueError):
        m.run([torch.from_numpy(x)])                      # host tensor
    with pytest.raises(ValueError):
        m.run([torch.from_numpy(x).cuda().double()])
    with pytest.raises(ValueError):
        m.run([torch.from_numpy(np.ascontiguousarray(x.T)).cuda().t()])   # not contiguous
    bad = sp.csr_matrix((np.ones(2, "float32"), np.array([0, 99], "int32"), np.array([0, 2], "int32")), shape=(1, 60))
    bad.has_sorted_indices = True
    with pytest.raises(ValueError):
        VanillaSpMMhip(bad)
    t = m.measure_average_time([torch.from_numpy(x).cuda()], 3)
    assert 0 < t < 1.0


def test_uniform_10k_config(torch_cuda, oracle):
    """10,000 nodes, in-degree 16 + self-loops, weights U(0,1), features 10,000 x 32 ~ N(0,1)."""
    from featgraph_amd import synthetic
    from featgraph_amd.module import VanillaSpMMhip
    indptr, indices = synthetic.make_workload("uniform-10k")
    vals = synthetic.edge_weights(indices.shape[0], 1)
    adj = sp.csr_matrix((vals, indices, indptr), shape=(10000, 10000))
    x = np.random.default_rng(2).standard_normal((10000, 32)).astype("float32")
    m, out = _run(torch_cuda, VanillaSpMMhip, adj, x, {}, {})
    out = out.cpu().numpy()
    np.testing.assert_allclose(out, oracle.spmm_csr_x86(indptr, indices, vals, x, 1, 4), rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(out, oracle.spmm_f64(adj, x), rtol=RTOL, atol=ATOL)
    assert np.array_equal(m._adj_indices_dev.cpu().numpy(), indices)


@pytest.mark.parametrize("feat_len,P,T", [(32, 1, 0), (64, 1, 0), (128, 8, 2), (256, 1, 4), (512, 1, 0), (512, 4, 8)])
def test_powerlaw_23k(torch_cuda, oracle, feat_len, P, T):
    """A 1/10-scale copy of the 233k-node power-law workload (hub rows up to ~1.6k edges)."""
    from featgraph_amd import synthetic
    from featgraph_amd.module import VanillaSpMMhip
    indptr, indices = synthetic.make_workload("powerlaw-23k")
    n = indptr.shape[0] - 1
    vals = synthetic.edge_weights(indices.shape[0], 1)
    adj = sp.csr_matrix((vals, indices, indptr), shape=(n, n))
    x = np.random.default_rng(3).standard_normal((n, feat_len)).astype("float32")
    _, out = _run(torch_cuda, VanillaSpMMhip, adj, x, {'num_feat_partitions': T}, {}, P)
    out = out.cpu().numpy()
    ref64 = oracle.spmm_f64(adj, x)
    assert_sum_close(out, ref64, spmm_mass(adj, x))
    ref32 = oracle.spmm_csr_x86(indptr, indices, vals, x, 1, 4)
    assert np.abs(out - ref64).max() <= 4 * max(np.abs(ref32 - ref64).max(), ATOL)


def test_full_size_properties(torch_cuda):
    """232,965 nodes / ~114.8M edges at F = 512, checked through size-independent properties:
    all-ones features give the weighted in-degree of every row; the column sums of the output
    equal the weighted out-degree contraction of X (a checksum of the whole product)."""
    from featgraph_amd import synthetic
    from featgraph_amd.module import VanillaSpMMhip, placeholder
    torch = torch_cuda
    indptr, indices = synthetic.make_workload("powerlaw-233k")
    n = indptr.shape[0] - 1
    nnz = indices.shape[0]
    g = torch.Generator(device="cuda"); g.manual_seed(1)
    vals_d = torch.rand(nnz, generator=g, device="cuda", dtype=torch.float32)
    vals = vals_d.cpu().numpy()
    adj = sp.csr_matrix((vals, indices, indptr), shape=(n, n))
    m = VanillaSpMMhip(adj)
    F = 512
    m.build([placeholder((n, F))], {}, {})
    assert np.array_equal(m._adj_indptr_dev.cpu().numpy(), indptr)
    assert np.array_equal(m._adj_indices_dev.cpu().numpy(), indices)

    ones = torch.ones((n, F), device="cuda", dtype=torch.float32)
    out = m.run([ones])
    row_sum = np.add.reduceat(vals.astype(np.float64), indptr[:-1])
    got = out.cpu().numpy()
    np.testing.assert_allclose(got[:, 0], row_sum, rtol=RTOL, atol=ATOL)
    assert (got == got[:, :1]).all()

    x = torch.randn((n, F), generator=g, device="cuda", dtype=torch.float32)
    out = m.run([x])
    col_w = torch.zeros(n, device="cuda", dtype=torch.float64)
    col_w.index_add_(0, torch.from_numpy(indices).cuda().long(), vals_d.double())
    expect = (col_w[:, None] * x.double()).sum(0)
    got = out.double().sum(0)
    scale = (col_w[:, None] * x.double().abs()).sum(0)
    assert ((got - expect).abs() <= 1e-5 * scale).all()
    # spot rows against a float64 gather on the host
    xh = x.cpu().numpy()
    outh = out.cpu().numpy()
    deg = np.diff(indptr)
    for v in (int(np.argmax(deg)), int(np.argmin(deg)), 0, n - 1, n // 2):
        e = slice(indptr[v], indptr[v + 1])
        terms = vals[e].astype(np.float64)[:, None] * xh[indices[e]].astype(np.float64)
        assert_sum_close(outh[v], terms.sum(0), np.abs(terms).sum(0), "row %d" % v)


def test_low_degree_large_graph_properties(torch_cuda):
    """2.45M nodes / ~61.9M edges (average degree 25), F = 128: SpMM followed by SDDMM on the same
    edges, checked through a column-sum checksum, all-ones row sums and sampled edges."""
    from featgraph_amd import synthetic
    from featgraph_amd.module import VanillaSpMMhip, VanillaSDDMMhip, placeholder
    torch = torch_cuda
    indptr, indices = synthetic.make_workload("powerlaw-2.45M")
    n = indptr.shape[0] - 1
    nnz = indices.shape[0]
    F = 128
    g = torch.Generator(device="cuda"); g.manual_seed(5)
    vals_d = torch.rand(nnz, generator=g, device="cuda", dtype=torch.float32)
    vals = vals_d.cpu().numpy()
    adj = sp.csr_matrix((vals, indices, indptr), shape=(n, n))
    x = torch.randn((n, F), generator=g, device="cuda")
    y = torch.randn((n, F), generator=g, device="cuda")
    idx_d = torch.from_numpy(indices).cuda().long()

    m = VanillaSpMMhip(adj)
    m.build([placeholder((n, F))], {}, {})
    assert np.array_equal(m._adj_indptr_dev.cpu().numpy(), indptr)
    out = m.run([x])
    col_w = torch.zeros(n, device="cuda", dtype=torch.float64)
    col_w.index_add_(0, idx_d, vals_d.double())
    expect = (col_w[:, None] * x.double()).sum(0)
    scale = (col_w[:, None] * x.double().abs()).sum(0)
    assert ((out.double().sum(0) - expect).abs() <= 1e-5 * scale).all()
    ones = torch.ones((n, F), device="cuda")
    row_sum = np.add.reduceat(vals.astype(np.float64), indptr[:-1])
    got = m.run([ones]).cpu().numpy()
    np.testing.assert_allclose(got[:, 0], row_sum, rtol=RTOL, atol=ATOL)
    assert (got[:, -1] == got[:, 0]).all()

    s = VanillaSDDMMhip(adj)
    s.build([placeholder((n, F)), placeholder((n, F))], {}, {})
    e_out = s.run([x, y])
    pick = torch.randint(0, nnz, (300000,), generator=g, device="cuda")
    r = s._adj_row_indices_dev.long()[pick]
    c = s._adj_col_indices_dev.long()[pick]
    prod = x[c].double() * y[r].double()
    ref = prod.sum(1)
    assert ((e_out[pick].double() - ref).abs() <= ATOL + RTOL * ref.abs() + 1e-6 * prod.abs().sum(1)).all()
    for e in (0, nnz - 1):
        rr, cc = int(s._adj_row_indices[e]), int(s._adj_col_indices[e])
        assert abs(e_out[e].item() - float((x[cc].double() * y[rr].double()).sum())) <= 1e-3


def test_float64_adjacency_with_partitions(torch_cuda, oracle):
    """scipy.sparse.random's default dtype: the values are cast to fp32 once, whatever the partition count."""
    from featgraph_amd.module import VanillaSpMMhip, VanillaSpMMx86
    rng = np.random.default_rng(21)
    adj64 = sp.random(90, 140, density=0.1, format="csr", random_state=rng)
    assert adj64.dtype == np.float64
    adj64.sort_indices()
    x = rng.standard_normal((140, 32)).astype("float32")
    a32 = adj64.astype("float32")
    ref = oracle.spmm_csr_x86(a32.indptr, a32.indices, a32.data, x)
    for cls, ctor, sched in ((VanillaSpMMhip, (), {}), (VanillaSpMMhip, (3,), {}), (VanillaSpMMx86, (4,), {}),
                             (VanillaSpMMhip, (), {'num_src_partitions': 5})):
        _, out = _run(torch_cuda, cls, adj64, x, {}, sched, *ctor)
        np.testing.assert_allclose(out.cpu().numpy(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("feat_len", [30, 100, 200, 300])
def test_awkward_feature_lengths_run_on_padded_copies(torch_cuda, oracle, feat_len):
    """Rows whose length is no multiple of 32 run at the next friendly length on zero-padded copies once the graph is
    large enough for that to pay; the result is that of the unpadded kernels (to rounding: the padded shape has other
    tiles and partitions), every call overwrites all of out, and run() keeps returning the same tensor."""
    from featgraph_amd import tuning
    from featgraph_amd.module import VanillaSpMMhip
    torch = torch_cuda
    rng = np.random.default_rng(feat_len)
    adj = _adj_with_long_and_empty_rows(rng, 3000, 3500, 2600)
    adj = (adj + _rand_csr(rng, 3000, 3500, 0.06)).tocsr().astype("float32"); adj.sort_indices()
    assert adj.nnz * feat_len >= tuning.PAD_MIN_GATHERED
    x = rng.standard_normal((3500, feat_len)).astype("float32")
    m, out = _run(torch, VanillaSpMMhip, adj, x, {}, {})
    assert m._pad_from == feat_len and m._feat_len == tuning.padded_feature_len(feat_len) and tuple(out.shape) == (3000, feat_len)
    got = out.cpu().numpy()
    assert_sum_close(got, oracle.spmm_f64(adj, x), spmm_mass(adj, x), "padded F=%d" % feat_len)
    plain, out2 = _run(torch, VanillaSpMMhip, adj, x, {}, {'pad_features': False})
    assert plain._pad_from is None
    assert_sum_close(out2.cpu().numpy(), oracle.spmm_f64(adj, x), spmm_mass(adj, x), "unpadded F=%d" % feat_len)
    m.out_tvm.fill_(float("nan"))
    again = m.run([torch.from_numpy(x).cuda()])
    assert again is m.out_tvm and np.array_equal(again.cpu().numpy(), got)
    assert "zero-padded" in "".join(m._notes)


def test_padded_feature_lengths():
    from featgraph_amd import tuning
    assert [tuning.padded_feature_len(f) for f in (1, 8, 9, 16, 30, 32, 40, 64, 72, 96, 100, 128, 130, 160, 200, 500, 602, 640)] == \
        [1, 8, 16, 16, 32, 32, 64, 64, 96, 96, 128, 128, 192, 160, 256, 512, 640, 640]
