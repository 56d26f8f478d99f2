"""GPU tests of the generalised SpMM (sum / mean / max / min aggregation, per-head weights,
copy_u).  The reference has no such operator, so parity is unpinned by it; the checks are the
CPU oracle's closed forms (numpy reduceat, see tests/test_oracle.py) and reductions to the plain
SpMM."""
import numpy as np
import pytest
import scipy.sparse as sp

from helpers import assert_sum_close, spmm_mass

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_cuda():
    import torch
    assert torch.cuda.is_available()
    return torch


def _graph(rng, n_rows=260, n_cols=3000, long_len=2700):
    a = sp.random(n_rows, n_cols, density=0.02, format="csr", random_state=rng,
                  data_rvs=lambda k: rng.standard_normal(k)).astype("float32").tolil()
    a[[0, n_rows // 2, n_rows - 1], :] = 0
    cols = rng.choice(n_cols, size=long_len, replace=False)
    a[5, cols] = rng.standard_normal(long_len).astype("float32") + 3.0
    a = a.tocsr().astype("float32"); a.eliminate_zeros(); a.sort_indices()
    return a


@pytest.mark.parametrize("reduce", ["max", "min"])
@pytest.mark.parametrize("feat_len", [1, 4, 7, 32, 64, 100, 128, 256, 512, 1024])
def test_extreme_aggregation(torch_cuda, oracle, reduce, feat_len):
    """max / min are exact: every kernel shape, split hub row, empty rows -> 0, negative weights."""
    from featgraph_amd.module import GSpMMhip, placeholder
    torch = torch_cuda
    rng = np.random.default_rng(feat_len)
    adj = _graph(rng)
    x = rng.standard_normal((3000, feat_len)).astype("float32")
    for msg in ("u_mul_e", "copy_u"):
        m = GSpMMhip(adj)
        m.build([placeholder(x.shape)], {'reduce': reduce, 'msg': msg}, {})
        m.out_tvm.fill_(float("nan"))
        out = m.run([torch.from_numpy(x).cuda()]).cpu().numpy()
        ref = oracle.gspmm(adj.indptr, adj.indices, adj.data if msg == "u_mul_e" else None, x, reduce, 2)
        assert np.array_equal(out, ref), (reduce, msg, feat_len)
        assert (out[np.diff(adj.indptr) == 0] == 0).all()


@pytest.mark.parametrize("reduce,P", [("sum", None), ("sum", 3), ("mean", None), ("mean", 4), ("sum", 'auto')])
def test_sum_and_mean(torch_cuda, oracle, reduce, P):
    from featgraph_amd.module import GSpMMhip, VanillaSpMMhip, placeholder
    torch = torch_cuda
    rng = np.random.default_rng(3)
    adj = _graph(rng)
    x = rng.standard_normal((3000, 96)).astype("float32")
    m = GSpMMhip(adj)
    m.build([placeholder(x.shape)], {'reduce': reduce}, {'num_src_partitions': P})
    out = m.run([torch.from_numpy(x).cuda()]).cpu().numpy()
    ref64 = oracle.spmm_f64(adj, x)
    mass = spmm_mass(adj, x)
    if reduce == "mean":
        deg = np.maximum(np.diff(adj.indptr), 1)[:, None]
        ref64, mass = ref64 / deg, mass / deg
    assert_sum_close(out, ref64, mass, "%s P=%s" % (reduce, P))
    if reduce == "sum" and P is None:
        v = VanillaSpMMhip(adj)
        v.build([placeholder(x.shape)], {}, {'num_src_partitions': None})
        assert np.array_equal(out, v.run([torch.from_numpy(x).cuda()]).cpu().numpy())
    # copy_u mean = plain average of the gathered rows
    m.build([placeholder(x.shape)], {'reduce': 'mean', 'msg': 'copy_u'}, {'num_src_partitions': P})
    out = m.run([torch.from_numpy(x).cuda()]).cpu().numpy()
    ones = sp.csr_matrix((np.ones(adj.nnz, "float32"), adj.indices, adj.indptr), shape=adj.shape)
    deg = np.maximum(np.diff(adj.indptr), 1)[:, None]
    assert_sum_close(out, oracle.spmm_f64(ones, x) / deg, spmm_mass(ones, x) / deg)


@pytest.mark.parametrize("H,D,reduce,P", [(4, 64, "sum", None), (8, 64, "sum", 3), (4, 32, "sum", None), (2, 16, "max", None),
                                          (8, 128, "sum", None), (4, 64, "min", None), (4, 32, "mean", 2), (1, 48, "sum", None),
                                          (8, 8, "sum", None), (8, 8, "sum", 3), (4, 16, "sum", 2), (16, 4, "sum", None),
                                          (2, 32, "sum", 4), (3, 32, "sum", None), (8, 16, "mean", None)])
def test_per_head_weights(torch_cuda, oracle, H, D, reduce, P):
    """out[v,h,:] = reduce_e w[e,h] * x[u,h,:] with weights handed to run() in CSR edge order."""
    from featgraph_amd.module import GSpMMhip, placeholder
    torch = torch_cuda
    rng = np.random.default_rng(H * 100 + D)
    adj = _graph(rng, 200, 1500, 1300)
    x = rng.standard_normal((1500, H, D)).astype("float32")
    w = rng.standard_normal((adj.nnz, H)).astype("float32")
    m = GSpMMhip(adj)
    wshape = (adj.nnz, H) if H > 1 else (adj.nnz,)
    m.build([placeholder(x.shape), placeholder(wshape)], {'reduce': reduce}, {'num_src_partitions': P})
    out = m.run([torch.from_numpy(x).cuda(), torch.from_numpy(w.reshape(wshape)).cuda()]).cpu().numpy()
    assert out.shape == (200, H, D)
    if reduce in ("max", "min"):
        assert np.array_equal(out, oracle.gspmm(adj.indptr, adj.indices, w, x, reduce))
        return
    ref = np.zeros((200, H, D)); mass = np.zeros((200, H, D))
    for h in range(H):
        ah = sp.csr_matrix((w[:, h], adj.indices, adj.indptr), shape=adj.shape)
        ref[:, h] = oracle.spmm_f64(ah, x[:, h]); mass[:, h] = spmm_mass(ah, x[:, h])
    if reduce == "mean":
        deg = np.maximum(np.diff(adj.indptr), 1)[:, None, None]
        ref, mass = ref / deg, mass / deg
    assert_sum_close(out, ref, mass, "H=%d D=%d" % (H, D))
    np.testing.assert_allclose(out, oracle.gspmm(adj.indptr, adj.indices, w, x, "sum") /
                               (np.maximum(np.diff(adj.indptr), 1)[:, None, None] if reduce == "mean" else 1),
                               rtol=1e-3, atol=1e-3)


def test_gspmm_errors(torch_cuda):
    from featgraph_amd.module import GSpMMhip, placeholder
    rng = np.random.default_rng(0)
    adj = _graph(rng, 50, 200, 150)
    m = GSpMMhip(adj)
    with pytest.raises(ValueError):
        m.build([placeholder((200, 8))], {'reduce': 'prod'}, {})
    with pytest.raises(ValueError):
        m.build([placeholder((200, 4, 16))], {}, {})                         # per-head weights missing
    with pytest.raises(ValueError):
        m.build([placeholder((200, 8)), placeholder((7,))], {}, {})          # wrong weight shape
    with pytest.raises(ValueError):
        GSpMMhip(adj, 2).build([placeholder((200, 8))], {'reduce': 'max'}, {})
    with pytest.raises(ValueError):                                          # head length 6 with a tiling of the caller's:
        m.build([placeholder((200, 4, 6)), placeholder((adj.nnz, 4))], {'num_feat_partitions': 2}, {})   # no kernel tile
    m.build([placeholder((200, 4, 6)), placeholder((adj.nnz, 4))], {}, {})       # left alone, the heads are padded to 8
    assert m._pad_from == 6 and m._feat_len == 32


@pytest.mark.parametrize("feat_len", [1, 3, 4, 20, 64, 256, 300, 1024])
@pytest.mark.parametrize("op", ["add", "sub", "mul", "dot"])
def test_gsddmm_elementwise(torch_cuda, op, feat_len):
    """out[e,:] = src[col[e],:] op dst[row[e],:]: bit-exact against numpy (one fp32 operation per
    element); 'dot' falls through to the plain SDDMM."""
    from featgraph_amd.module import GSDDMMhip, placeholder
    torch = torch_cuda
    rng = np.random.default_rng(feat_len)
    coo = sp.random(70, 90, density=0.1, format="coo", random_state=rng).astype("float32")
    p = rng.permutation(coo.nnz)
    coo = sp.coo_matrix((coo.data[p], (coo.row[p], coo.col[p])), shape=coo.shape)
    src = rng.standard_normal((90, feat_len)).astype("float32")
    dst = rng.standard_normal((70, feat_len)).astype("float32")
    for ctor in ((), (3, 2)):
        m = GSDDMMhip(coo, *ctor)
        m.build([placeholder(src.shape), placeholder(dst.shape)], {'op': op}, {})
        m.out_tvm.fill_(float("nan"))
        out = m.run([torch.from_numpy(src).cuda(), torch.from_numpy(dst).cuda()]).cpu().numpy()
        if ctor:
            out = out[m.edge_mapping]
        s, d = src[coo.col], dst[coo.row]
        if op == "dot":
            np.testing.assert_allclose(out, (s.astype("f8") * d).sum(-1), rtol=1e-4, atol=1e-4)
        else:
            expect = {"add": s + d, "sub": s - d, "mul": s * d}[op]
            assert out.shape == expect.shape and np.array_equal(out, expect)


@pytest.mark.parametrize("reduce", ["max", "min"])
@pytest.mark.parametrize("feat_len", [1, 4, 7, 32, 64, 100, 256, 512])
def test_selected_elements(torch_cuda, oracle, reduce, feat_len):
    """return_arg: the stored position of the edge that gave each output, exact against the oracle
    (first occurrence on ties; few distinct values so that ties are frequent; a split hub row)."""
    from featgraph_amd.module import GSpMMhip, placeholder
    torch = torch_cuda
    rng = np.random.default_rng(feat_len + (reduce == "min"))
    adj = _graph(rng)
    adj.data = rng.integers(-2, 3, size=adj.nnz).astype("float32")
    x = rng.integers(-3, 4, size=(3000, feat_len)).astype("float32")
    for msg in ("u_mul_e", "copy_u"):
        m = GSpMMhip(adj)
        m.build([placeholder(x.shape)], {'reduce': reduce, 'msg': msg, 'return_arg': True}, {})
        out = m.run([torch.from_numpy(x).cuda()]).cpu().numpy()
        arg = m.arg_tvm.cpu().numpy()
        ref_out, ref_arg = oracle.gspmm_arg(adj.indptr, adj.indices, adj.data if msg == "u_mul_e" else None, x, reduce, 2)
        assert np.array_equal(out, ref_out), (reduce, msg, feat_len)
        assert np.array_equal(arg, ref_arg), (reduce, msg, feat_len)
        assert (arg[np.diff(adj.indptr) == 0] == -1).all()
    with pytest.raises(ValueError):
        GSpMMhip(adj).build([placeholder(x.shape)], {'reduce': 'sum', 'return_arg': True}, {})


@pytest.mark.parametrize("heads", [1, 3, 4, 8, 16])
@pytest.mark.parametrize("n", [1, 511, 513, 70001])
def test_edge_values_head_major(torch_cuda, heads, n):
    """dst[h, e] = src[pos[e], h]: the relayout of per-head edge weights, through the C ABI; heads of 4, 8 and 16 take
    the kernel with 128-bit loads, the others (and a misaligned source) the scalar one."""
    from featgraph_amd import _lib
    torch = torch_cuda
    g = torch.Generator(device="cuda").manual_seed(n * 31 + heads)
    src = torch.randn((n + 1, heads), device="cuda", generator=g)
    pos = torch.randperm(n, device="cuda", generator=g).to(torch.int32)
    for s, p in ((src[:n], None), (src[:n], pos), (src.reshape(-1)[1:1 + n * heads].reshape(n, heads), pos)):
        dst = torch.full((heads, n), float("nan"), device="cuda")
        _lib.check(_lib.lib().fg_edge_values_head_major_f32(_lib.dev_ptr(s), _lib.dev_ptr(p), n, heads, _lib.dev_ptr(dst), None))
        want = (s if p is None else s[p.long()]).t()
        assert torch.equal(dst, want)


@pytest.mark.parametrize("reduce", ["max", "min"])
@pytest.mark.parametrize("partitions", ['auto', 3])
def test_extreme_of_weighted_messages_with_positions(torch_cuda, oracle, reduce, partitions):
    """max / min of x[col] * w[e] with one weight per edge given to run() (the path over source partitions that finds
    the selected elements in the same sweep): values exact, positions = the oracle's first occurrence."""
    from featgraph_amd.module import GSpMMhip, placeholder
    torch = torch_cuda
    rng = np.random.default_rng(12)
    adj = _graph(rng)
    x = rng.integers(-2, 3, size=(3000, 20)).astype("float32")          # few distinct values: many ties
    w = rng.integers(-2, 3, size=adj.nnz).astype("float32")
    m = GSpMMhip(adj)
    m.build([placeholder(x.shape), placeholder(w.shape)], {'reduce': reduce, 'return_arg': True}, {'num_src_partitions': partitions})
    assert m._bop is not None
    out = m.run([torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()]).cpu().numpy()
    ref = oracle.gspmm(adj.indptr, adj.indices, w, x, reduce)
    assert np.array_equal(out, ref)
    ref_b, ref_arg = oracle.gspmm_bcast(adj.indptr, adj.indices, 'mul', reduce, x, w[:, None], 'u', 'e')
    assert np.array_equal(ref_b, ref) and np.array_equal(m.arg_tvm.cpu().numpy(), ref_arg)


@pytest.mark.parametrize("reduce", ["sum", "mean"])
def test_weights_given_at_run_with_an_awkward_feature_length(torch_cuda, oracle, reduce):
    """One weight per edge given to run(), rows of 100 floats on a graph large enough for the padded copies."""
    from featgraph_amd import tuning
    from featgraph_amd.module import GSpMMhip, placeholder
    torch = torch_cuda
    rng = np.random.default_rng(17)
    adj = sp.random(2500, 3000, density=0.06, format="csr", random_state=rng).astype("float32"); adj.sort_indices()
    F = 100
    assert adj.nnz * F >= tuning.PAD_MIN_GATHERED
    x = rng.standard_normal((3000, F)).astype("float32")
    w = rng.standard_normal(adj.nnz).astype("float32")
    m = GSpMMhip(adj)
    m.build([placeholder(x.shape), placeholder(w.shape)], {'reduce': reduce}, {})
    assert m._pad_from == F and m._feat_len == 128
    m.out_tvm.fill_(float("nan"))
    out = m.run([torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()]).cpu().numpy()
    aw = sp.csr_matrix((w, adj.indices, adj.indptr), shape=adj.shape)
    ref = oracle.spmm_f64(aw, x)
    mass = np.asarray(abs(aw).astype(np.float64).dot(np.abs(x).astype(np.float64)))
    if reduce == "mean":
        deg = np.maximum(np.diff(adj.indptr), 1)[:, None]
        ref, mass = ref / deg, mass / deg
    assert out.shape == (2500, F)
    assert_sum_close(out, ref, mass, "padded weighted %s" % reduce)


@pytest.mark.parametrize("H,D", [(4, 6), (3, 20), (8, 48), (2, 100)])
def test_per_head_weights_with_awkward_head_lengths(torch_cuda, oracle, H, D):
    """Head lengths the kernels have no tile for are zero-padded to the next one they have."""
    from featgraph_amd.module import GSpMMhip, placeholder
    torch = torch_cuda
    rng = np.random.default_rng(H * 100 + D)
    adj = _graph(rng, 200, 1500, 1300)
    x = rng.standard_normal((1500, H, D)).astype("float32")
    w = rng.standard_normal((adj.nnz, H)).astype("float32")
    m = GSpMMhip(adj)
    m.build([placeholder(x.shape), placeholder(w.shape)], {}, {})
    assert m._pad_from == D
    m.out_tvm.fill_(float("nan"))
    out = m.run([torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()]).cpu().numpy()
    assert out.shape == (200, H, D)
    for h in range(H):
        ah = sp.csr_matrix((w[:, h], adj.indices, adj.indptr), shape=adj.shape)
        mass = np.asarray(abs(ah).astype(np.float64).dot(np.abs(x[:, h]).astype(np.float64)))
        assert_sum_close(out[:, h], oracle.spmm_f64(ah, x[:, h]), mass, "head %d of %dx%d" % (h, H, D))
