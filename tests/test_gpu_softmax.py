"""GPU tests of the edge softmax (forward and gradient) and of the attention chain built from it.
The reference has no such operator, so parity is unpinned by it; the checks are the CPU oracle
(itself pinned by scipy.special.softmax and torch autograd in tests/test_oracle.py), float64 closed
forms, and size-independent properties at full size."""
import numpy as np
import pytest
import scipy.sparse as sp

from helpers import RTOL, ATOL

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_cuda():
    import torch
    assert torch.cuda.is_available()
    return torch


def _ragged(rng, kind):
    """CSR structure with empty rows, one-element rows and (kind 'hub') rows long enough to be split."""
    if kind == "short":                      # many rows of a few elements: lane-per-(row, head) path
        lens = rng.integers(0, 9, size=900)
    elif kind == "medium":                   # rows of tens of elements: whole-wavefront path inside multi-row items
        lens = rng.integers(20, 120, size=200)
    else:                                    # single-row items and split rows
        lens = rng.integers(0, 60, size=120)
        lens[7] = 300; lens[40] = 1024; lens[41] = 1025; lens[90] = 5000
        lens[91] = 4096; lens[92] = 4097; lens[93] = 2049; lens[94] = 129     # either side of the workgroups' capacities at H = 8
    lens[::11] = 0
    lens[3] = 1
    indptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    n_cols = int(max(lens.max(), 1))
    indices = np.concatenate([np.sort(rng.choice(n_cols, size=l, replace=False)) for l in lens] + [np.zeros(0, int)])
    adj = sp.csr_matrix((np.ones(indptr[-1], np.float32), indices.astype(np.int32), indptr),
                        shape=(len(lens), n_cols))
    return adj


@pytest.mark.parametrize("kind", ["short", "medium", "hub"])
@pytest.mark.parametrize("H", [1, 2, 3, 4, 6, 8, 12, 33, 64, 65])   # 3, 6, 12, 33: lanes past the largest multiple of H idle; 65: one head at a time
def test_edge_softmax_matches_oracle(torch_cuda, oracle, kind, H):
    from featgraph_amd.module import EdgeSoftmaxhip, placeholder
    torch = torch_cuda
    rng = np.random.default_rng(100 * H + len(kind))
    adj = _ragged(rng, kind)
    nnz = adj.nnz
    shape = (nnz,) if H == 1 else (nnz, H)
    x = (rng.standard_normal(shape) * 4).astype("float32")
    m = EdgeSoftmaxhip(adj)
    m.build([placeholder(shape)])
    m.out_tvm.fill_(float("nan"))
    out = m.run([torch.from_numpy(x).cuda()]).cpu().numpy()
    ref64 = oracle.edge_softmax_f64(adj.indptr, x)
    ref32 = oracle.edge_softmax(adj.indptr, x)
    assert np.isfinite(out).all()                       # every element was written
    np.testing.assert_allclose(out, ref64, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(out, ref32, rtol=RTOL, atol=ATOL)
    # rows sum to one; one-element rows are exactly one
    rows = adj.indptr[:-1][np.diff(adj.indptr) > 0]
    np.testing.assert_allclose(np.add.reduceat(out.astype(np.float64), rows, axis=0), 1.0, atol=2e-5)
    assert (out[adj.indptr[3]:adj.indptr[4]] == 1.0).all()
    # bit-identical on repetition, and in place
    again = m.run([torch.from_numpy(x).cuda()]).cpu().numpy()
    assert np.array_equal(out, again)

    # gradient
    g = rng.standard_normal(shape).astype("float32")
    dx = m.backward(torch.from_numpy(ref32).cuda(), torch.from_numpy(g).cuda()).cpu().numpy()
    a64 = ref32.astype(np.float64)
    ag = a64 * g
    rowsum = np.zeros_like(ag)
    d = np.add.reduceat(ag, rows, axis=0)
    rowsum[...] = np.repeat(d, np.diff(adj.indptr)[np.diff(adj.indptr) > 0], axis=0)
    mass = np.repeat(np.add.reduceat(np.abs(ag), rows, axis=0), np.diff(adj.indptr)[np.diff(adj.indptr) > 0], axis=0)
    ref_dx = a64 * (g - rowsum)
    err = np.abs(dx - ref_dx)
    assert (err <= ATOL + RTOL * np.abs(ref_dx) + 8 * np.finfo(np.float32).eps * mass * np.abs(a64) + 1e-6).all()
    np.testing.assert_allclose(dx, oracle.edge_softmax_backward(adj.indptr, ref32, g), rtol=1e-3, atol=2e-5)


def test_edge_softmax_extremes_and_errors(torch_cuda, oracle):
    from featgraph_amd.module import EdgeSoftmaxhip, placeholder
    torch = torch_cuda
    rng = np.random.default_rng(0)
    adj = _ragged(rng, "hub")
    nnz = adj.nnz
    m = EdgeSoftmaxhip(adj)
    m.build([placeholder((nnz, 4))])
    # large magnitudes do not overflow; a per-row shift changes nothing beyond rounding
    x = (rng.standard_normal((nnz, 4)) * 3).astype("float32")
    base = m.run([torch.from_numpy(x).cuda()]).cpu().numpy().copy()
    shift = np.repeat(rng.standard_normal((adj.shape[0], 4)).astype("float32") * 80, np.diff(adj.indptr), axis=0)
    shifted = m.run([torch.from_numpy(x + shift).cuda()]).cpu().numpy()
    np.testing.assert_allclose(shifted, base, rtol=3e-4, atol=1e-6)
    big = m.run([torch.from_numpy(x * 1e4).cuda()]).cpu().numpy()
    assert np.isfinite(big).all()
    with pytest.raises(ValueError):
        m.run([torch.zeros((nnz, 3), device="cuda")])
    with pytest.raises(ValueError):
        m.build([placeholder((nnz + 1,))])
    with pytest.raises(TypeError):
        m.build([placeholder((nnz,))], {'axis': 0})
    # a graph without edges
    empty = sp.csr_matrix((5, 5), dtype="float32")
    e = EdgeSoftmaxhip(empty)
    e.build([placeholder((0, 2))])
    assert e.run([torch.zeros((0, 2), device="cuda")]).shape == (0, 2)


def test_edge_softmax_full_size(torch_cuda, oracle):
    """232,965 nodes / 114.77M edges, 4 heads: rows sum to one, sampled rows against float64."""
    from featgraph_amd import synthetic
    from featgraph_amd.module import EdgeSoftmaxhip, placeholder
    torch = torch_cuda
    indptr, indices = synthetic.make_workload("powerlaw-233k")
    n = indptr.shape[0] - 1
    nnz = int(indptr[-1])
    adj = sp.csr_matrix((np.ones(nnz, np.float32), indices, indptr), shape=(n, n))
    H = 4
    gen = torch.Generator(device="cuda"); gen.manual_seed(3)
    x = torch.randn((nnz, H), generator=gen, device="cuda") * 3
    m = EdgeSoftmaxhip(adj)
    m.build([placeholder((nnz, H))])
    out = m.run([x])
    row_of = torch.repeat_interleave(torch.arange(n, device="cuda"), torch.from_numpy(np.diff(indptr)).cuda())
    sums = torch.zeros((n, H), dtype=torch.float64, device="cuda").index_add_(0, row_of, out.double())
    assert torch.allclose(sums, torch.ones_like(sums), atol=1e-4)
    deg = np.diff(indptr)
    picks = [int(np.argmax(deg)), int(np.argmin(deg)), 0, n - 1] + list(np.random.default_rng(1).integers(0, n, 60))
    xs = x.cpu().numpy(); os_ = out.cpu().numpy()
    for r in picks:
        b, e = indptr[r], indptr[r + 1]
        ref = oracle.edge_softmax_f64(np.array([0, e - b], np.int32), xs[b:e])
        np.testing.assert_allclose(os_[b:e], ref, rtol=RTOL, atol=ATOL)


def test_attention_chain_gradients(torch_cuda):
    """scores = multi-head SDDMM, a = edge softmax, out = per-head weighted SpMM: values and all
    gradients against the same chain written with gather / index_add / scatter softmax in float64."""
    from featgraph_amd.autograd import Graph
    torch = torch_cuda
    rng = np.random.default_rng(9)
    n_dst, n_src, H, D = 90, 150, 4, 16
    adj = sp.random(n_dst, n_src, density=0.15, format="csr", random_state=rng).astype("float32")
    adj.sort_indices()
    g = Graph(adj)
    coo = adj.tocoo()
    rows = torch.from_numpy(coo.row.astype(np.int64)).cuda()
    cols = torch.from_numpy(coo.col.astype(np.int64)).cuda()
    gen = torch.Generator(device="cuda"); gen.manual_seed(0)
    q = torch.randn((n_dst, H, D), generator=gen, device="cuda", requires_grad=True)
    k = torch.randn((n_src, H, D), generator=gen, device="cuda", requires_grad=True)
    v = torch.randn((n_src, H, D), generator=gen, device="cuda", requires_grad=True)
    up = torch.randn((n_dst, H, D), generator=gen, device="cuda")

    s = g.sddmm(k, q) * (D ** -0.5)
    a = g.edge_softmax(s)
    out = g.spmm(v, a)
    (out * up).sum().backward()

    q64, k64, v64 = (t.detach().double().requires_grad_() for t in (q, k, v))
    s64 = (k64[cols] * q64[rows]).sum(-1) * (D ** -0.5)
    mx = torch.full((n_dst, H), -float("inf"), dtype=torch.float64, device="cuda").scatter_reduce(
        0, rows[:, None].expand(-1, H), s64, reduce="amax")
    ex = torch.exp(s64 - mx[rows])
    den = torch.zeros((n_dst, H), dtype=torch.float64, device="cuda").index_add(0, rows, ex)
    a64 = ex / den[rows]
    out64 = torch.zeros((n_dst, H, D), dtype=torch.float64, device="cuda").index_add(0, rows, a64[:, :, None] * v64[cols])
    (out64 * up.double()).sum().backward()
    assert torch.allclose(a.double(), a64, rtol=1e-4, atol=1e-5)
    assert torch.allclose(out.double(), out64, rtol=1e-4, atol=1e-4)
    for got, ref in ((q.grad, q64.grad), (k.grad, k64.grad), (v.grad, v64.grad)):
        assert torch.allclose(got.double(), ref, rtol=1e-3, atol=1e-4)


@pytest.mark.parametrize("H,D,P", [(1, 32, None), (1, 100, 2), (4, 16, None), (4, 64, 3), (8, 8, None), (2, 128, 'auto'), (3, 32, None)])
def test_fused_softmax_spmm(torch_cuda, oracle, H, D, P):
    """EdgeSoftmaxSpMMhip (statistics + normalise-into-SpMM-layout + SpMM) against float64:
    softmax per row and head (scipy), then the weighted sum per head."""
    from featgraph_amd.module import EdgeSoftmaxSpMMhip, placeholder
    from helpers import assert_sum_close
    torch = torch_cuda
    rng = np.random.default_rng(H * 100 + D)
    adj = _ragged(rng, "hub")
    n_rows, n_cols = adj.shape
    nnz = adj.nnz
    s_shape = (nnz,) if H == 1 else (nnz, H)
    x_shape = (n_cols, D) if H == 1 else (n_cols, H, D)
    s = (rng.standard_normal(s_shape) * 3).astype("float32")
    x = rng.standard_normal(x_shape).astype("float32")
    m = EdgeSoftmaxSpMMhip(adj)
    m.build([placeholder(s_shape), placeholder(x_shape)], {}, {'num_src_partitions': P})
    m.out_tvm.fill_(float("nan"))
    out = m.run([torch.from_numpy(s).cuda(), torch.from_numpy(x).cuda()]).cpu().numpy().reshape(n_rows, H, D)
    a64 = oracle.edge_softmax_f64(adj.indptr, s).reshape(nnz, H)
    x3 = x.reshape(n_cols, H, D).astype(np.float64)
    ref = np.zeros((n_rows, H, D)); mass = np.zeros((n_rows, H, D))
    for h in range(H):
        ah = sp.csr_matrix((a64[:, h], adj.indices, adj.indptr), shape=adj.shape)
        ref[:, h] = ah.dot(x3[:, h]); mass[:, h] = ah.dot(np.abs(x3[:, h]))
    assert np.isfinite(out).all()
    assert_sum_close(out, ref, mass, "H=%d D=%d P=%s" % (H, D, P))
    assert (out[np.diff(adj.indptr) == 0] == 0).all()
