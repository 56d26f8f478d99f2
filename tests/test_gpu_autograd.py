"""Gradients of the differentiable SpMM / SDDMM against torch autograd on the same formulas
written with gather / index_add in float64 (the reference has no autograd layer)."""
import numpy as np
import pytest
import scipy.sparse as sp

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape,feat_len", [((127, 255), 32), ((300, 200), 128), ((64, 64), 7)])
def test_spmm_sddmm_gradients(shape, feat_len):
    import torch
    from featgraph_amd.autograd import Graph
    rng = np.random.default_rng(feat_len)
    adj = sp.random(shape[0], shape[1], density=0.1, format="csr", random_state=rng).astype("float32")
    adj.sort_indices()
    g = Graph(adj)
    coo = adj.tocoo()
    rows = torch.from_numpy(coo.row.astype(np.int64)).cuda()
    cols = torch.from_numpy(coo.col.astype(np.int64)).cuda()
    gen = torch.Generator(device="cuda"); gen.manual_seed(0)
    x = torch.randn((shape[1], feat_len), generator=gen, device="cuda", requires_grad=True)
    d = torch.randn((shape[0], feat_len), generator=gen, device="cuda", requires_grad=True)
    w = torch.rand(adj.nnz, generator=gen, device="cuda", requires_grad=True)
    up = torch.randn((shape[0], feat_len), generator=gen, device="cuda")
    ue = torch.randn(adj.nnz, generator=gen, device="cuda")

    # SpMM
    y = g.spmm(x, w)
    (y * up).sum().backward()
    x64, w64 = x.detach().double().requires_grad_(), w.detach().double().requires_grad_()
    y64 = torch.zeros((shape[0], feat_len), dtype=torch.float64, device="cuda").index_add(0, rows, w64[:, None] * x64[cols])
    (y64 * up.double()).sum().backward()
    assert torch.allclose(y.double(), y64, rtol=1e-4, atol=1e-4)
    assert torch.allclose(x.grad.double(), x64.grad, rtol=1e-4, atol=1e-4)
    assert torch.allclose(w.grad.double(), w64.grad, rtol=1e-4, atol=1e-4)

    # SDDMM
    x.grad = None
    s = g.sddmm(x, d)
    (s * ue).sum().backward()
    x64, d64 = x.detach().double().requires_grad_(), d.detach().double().requires_grad_()
    s64 = (x64[cols] * d64[rows]).sum(-1)
    (s64 * ue.double()).sum().backward()
    assert torch.allclose(s.double(), s64, rtol=1e-4, atol=1e-4)
    assert torch.allclose(x.grad.double(), x64.grad, rtol=1e-4, atol=1e-4)
    assert torch.allclose(d.grad.double(), d64.grad, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("reduce", ["sum", "mean", "max", "min"])
def test_aggregate_gradients(reduce):
    """Graph.aggregate against a dense masked reduction in float64 (continuous random data: no ties)."""
    import torch
    from featgraph_amd.autograd import Graph
    rng = np.random.default_rng(4)
    n_dst, n_src, F = 70, 90, 24
    adj = sp.random(n_dst, n_src, density=0.12, format="csr", random_state=rng).astype("float32").tolil()
    adj[[3, 40], :] = 0                                   # rows without edges
    adj = adj.tocsr(); adj.eliminate_zeros(); adj.sort_indices()
    g = Graph(adj)
    gen = torch.Generator(device="cuda"); gen.manual_seed(1)
    x = torch.randn((n_src, F), generator=gen, device="cuda", requires_grad=True)
    up = torch.randn((n_dst, F), generator=gen, device="cuda")
    y = g.aggregate(x, reduce)
    (y * up).sum().backward()

    mask = torch.from_numpy((adj.toarray() != 0)).cuda()
    x64 = x.detach().double().requires_grad_()
    big = x64[None, :, :].expand(n_dst, -1, -1)
    has = mask.any(1)
    if reduce in ("sum", "mean"):
        y64 = (mask[:, :, None] * big).sum(1)
        if reduce == "mean":
            y64 = y64 / mask.sum(1).clamp(min=1)[:, None]
    else:
        fill = float("-inf") if reduce == "max" else float("inf")
        masked = torch.where(mask[:, :, None], big, torch.full_like(big, fill))
        y64 = masked.max(1).values if reduce == "max" else masked.min(1).values
        y64 = torch.where(has[:, None], y64, torch.zeros_like(y64))
    (y64 * up.double()).sum().backward()
    assert torch.allclose(y.double(), y64, rtol=1e-4, atol=1e-5)
    assert torch.allclose(x.grad.double(), x64.grad, rtol=1e-4, atol=1e-5)


def test_attention_with_and_without_gradients():
    """Graph.attention with and without gradients: same values, and the gradients match float64 torch autograd."""
    import torch
    from featgraph_amd.autograd import Graph
    rng = np.random.default_rng(21)
    adj = sp.random(120, 150, density=0.08, format="csr", random_state=rng).astype("float32")
    adj.sort_indices()
    g = Graph(adj)
    H, D = 4, 32
    q = torch.from_numpy(rng.standard_normal((120, H, D)).astype("float32")).cuda().requires_grad_()
    k = torch.from_numpy(rng.standard_normal((150, H, D)).astype("float32")).cuda().requires_grad_()
    v = torch.from_numpy(rng.standard_normal((150, H, D)).astype("float32")).cuda().requires_grad_()
    with torch.no_grad():
        fused = g.attention(q, k, v)
    chained = g.attention(q, k, v)
    assert chained.requires_grad and not fused.requires_grad
    np.testing.assert_allclose(fused.cpu().numpy(), chained.detach().cpu().numpy(), rtol=2e-4, atol=2e-5)
    chained.square().sum().backward()
    # float64 reference on the dense masked form
    coo = adj.tocoo()
    mask = torch.zeros((120, 150), dtype=torch.bool); mask[coo.row, coo.col] = True
    q64, k64, v64 = (t.detach().cpu().double().requires_grad_() for t in (q, k, v))
    s = torch.einsum("rhd,chd->hrc", q64, k64) / D ** 0.5
    s = s.masked_fill(~mask, float("-inf"))
    a = torch.nan_to_num(torch.softmax(s, dim=-1), nan=0.0)
    ref = torch.einsum("hrc,chd->rhd", a, v64)
    np.testing.assert_allclose(chained.detach().cpu().numpy(), ref.detach().numpy(), rtol=1e-4, atol=2e-5)
    ref.square().sum().backward()
    for got, want in ((q.grad, q64.grad), (k.grad, k64.grad), (v.grad, v64.grad)):
        np.testing.assert_allclose(got.cpu().numpy(), want.numpy(), rtol=1e-3, atol=1e-4)


def test_gat_attention_gradients():
    """Graph.gat_attention (additive scores through a leaky ReLU) against float64 torch autograd."""
    import torch
    from featgraph_amd.autograd import Graph
    rng = np.random.default_rng(22)
    adj = sp.random(90, 140, density=0.1, format="csr", random_state=rng).astype("float32")
    adj.sort_indices()
    g = Graph(adj)
    H, D = 4, 16
    er = torch.from_numpy(rng.standard_normal((90, H)).astype("float32")).cuda().requires_grad_()
    el = torch.from_numpy(rng.standard_normal((140, H)).astype("float32")).cuda().requires_grad_()
    v = torch.from_numpy(rng.standard_normal((140, H, D)).astype("float32")).cuda().requires_grad_()
    out = g.gat_attention(er, el, v, 0.1)
    out.square().sum().backward()
    coo = adj.tocoo()
    mask = torch.zeros((90, 140), dtype=torch.bool); mask[coo.row, coo.col] = True
    er64, el64, v64 = (t.detach().cpu().double().requires_grad_() for t in (er, el, v))
    z = er64.t()[:, :, None] + el64.t()[:, None, :]
    a = torch.nan_to_num(torch.softmax(torch.nn.functional.leaky_relu(z, 0.1).masked_fill(~mask, float("-inf")), dim=-1), nan=0.0)
    ref = torch.einsum("hrc,chd->rhd", a, v64)
    ref.square().sum().backward()
    np.testing.assert_allclose(out.detach().cpu().numpy(), ref.detach().numpy(), rtol=1e-4, atol=2e-5)
    for got, want in ((er.grad, er64.grad), (el.grad, el64.grad), (v.grad, v64.grad)):
        np.testing.assert_allclose(got.cpu().numpy(), want.numpy(), rtol=1e-3, atol=1e-4)


def _dense_pick(t, target, rows, cols):
    import torch
    if target == 'u':
        return t[cols]
    if target == 'v':
        return t[rows]
    return t


def _align(a, b):
    nd = max(a.dim(), b.dim())
    a = a.reshape((a.shape[0],) + (1,) * (nd - a.dim()) + tuple(a.shape[1:]))
    b = b.reshape((b.shape[0],) + (1,) * (nd - b.dim()) + tuple(b.shape[1:]))
    return a, b


_TORCH_OP = {'add': lambda a, b: a + b, 'sub': lambda a, b: a - b, 'mul': lambda a, b: a * b}


@pytest.mark.parametrize("msg,l_shape,r_shape", [
    ("u_mul_e", (24,), (24,)), ("u_mul_e", (4, 8), (4, 1)), ("e_mul_u", (1,), (16,)), ("u_add_e", (8,), (8,)),
    ("u_sub_e", (3, 1), (1, 5)), ("e_sub_u", (6,), (1,)), ("copy_e", (12,), None), ("u_add_e", (), (4,)),
])
@pytest.mark.parametrize("reduce", ["sum", "mean"])
def test_generalised_spmm_gradients(msg, l_shape, r_shape, reduce):
    """Graph.gspmm against torch autograd on the same formula in float64 (gather / index_add)."""
    import torch
    from featgraph_amd.autograd import Graph
    from featgraph_amd.module.general import parse_message
    rng = np.random.default_rng(len(msg) + len(l_shape))
    adj = sp.random(90, 140, density=0.08, format="csr", random_state=rng).astype("float32")
    adj.sort_indices()
    g = Graph(adj)
    coo = adj.tocoo()
    rows = torch.from_numpy(coo.row.astype(np.int64)).cuda()
    cols = torch.from_numpy(coo.col.astype(np.int64)).cuda()
    op, lt, rt = parse_message(msg)
    n_of = {'u': adj.shape[1], 'e': adj.nnz}
    gen = torch.Generator(device="cuda"); gen.manual_seed(1)
    lhs = torch.randn((n_of[lt],) + l_shape, generator=gen, device="cuda", requires_grad=True)
    rhs = torch.randn((n_of[rt],) + r_shape, generator=gen, device="cuda", requires_grad=True) if rt else None
    out = g.gspmm(msg, lhs, rhs, reduce) if rt else g.gspmm(msg, lhs, reduce=reduce)
    up = torch.randn(out.shape, generator=gen, device="cuda")
    (out * up).sum().backward()

    l64 = lhs.detach().double().requires_grad_()
    r64 = rhs.detach().double().requires_grad_() if rt else None
    if rt:
        a, b = _align(_dense_pick(l64, lt, rows, cols), _dense_pick(r64, rt, rows, cols))
        m = _TORCH_OP[op](a, b)
    else:
        m = l64 if len(l_shape) else l64[:, None]
    ref = torch.zeros((adj.shape[0],) + tuple(m.shape[1:]), dtype=torch.float64, device="cuda").index_add(0, rows, m)
    if reduce == "mean":
        deg = torch.from_numpy(np.maximum(np.diff(adj.indptr), 1)).cuda().double()
        ref = ref / deg.reshape((-1,) + (1,) * (ref.dim() - 1))
    assert out.shape == ref.shape
    (ref * up.double()).sum().backward()
    assert torch.allclose(out.double(), ref, rtol=1e-4, atol=1e-4)
    assert torch.allclose(lhs.grad.double(), l64.grad, rtol=1e-4, atol=1e-4)
    if rt:
        assert torch.allclose(rhs.grad.double(), r64.grad, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("op,lt,l_shape,rt,r_shape", [
    ("add", 'u', (16,), 'v', (16,)), ("sub", 'u', (4, 1), 'v', (1, 6)), ("mul", 'u', (12,), 'v', (12,)),
    ("mul", 'v', (4, 8), 'u', (4, 1)), ("mul", 'e', (8,), 'u', (8,)), ("mul", 'e', (1,), 'v', (20,)),
    ("sub", 'e', (5,), 'v', (5,)), ("mul", 'u', (3,), 'e', (3,)), ("add", 'v', (2, 3), 'e', (3,)),
])
def test_generalised_sddmm_gradients(op, lt, l_shape, rt, r_shape):
    import torch
    from featgraph_amd.autograd import Graph
    rng = np.random.default_rng(len(op) + sum(l_shape))
    adj = sp.random(90, 140, density=0.08, format="csr", random_state=rng).astype("float32")
    adj.sort_indices()
    g = Graph(adj)
    coo = adj.tocoo()
    rows = torch.from_numpy(coo.row.astype(np.int64)).cuda()
    cols = torch.from_numpy(coo.col.astype(np.int64)).cuda()
    n_of = {'u': adj.shape[1], 'v': adj.shape[0], 'e': adj.nnz}
    gen = torch.Generator(device="cuda"); gen.manual_seed(2)
    lhs = torch.randn((n_of[lt],) + l_shape, generator=gen, device="cuda", requires_grad=True)
    rhs = torch.randn((n_of[rt],) + r_shape, generator=gen, device="cuda", requires_grad=True)
    out = g.gsddmm(op, lhs, rhs, lt, rt)
    up = torch.randn(out.shape, generator=gen, device="cuda")
    (out * up).sum().backward()
    l64, r64 = lhs.detach().double().requires_grad_(), rhs.detach().double().requires_grad_()
    a, b = _align(_dense_pick(l64, lt, rows, cols), _dense_pick(r64, rt, rows, cols))
    ref = _TORCH_OP[op](a, b)
    assert out.shape == ref.shape
    (ref * up.double()).sum().backward()
    assert torch.allclose(out.double(), ref, rtol=1e-5, atol=1e-5)
    assert torch.allclose(lhs.grad.double(), l64.grad, rtol=1e-4, atol=1e-4)
    assert torch.allclose(rhs.grad.double(), r64.grad, rtol=1e-4, atol=1e-4)


def test_modules_stay_usable_after_the_graph_handed_their_outputs_out():
    """Graph's differentiable calls give the module's output tensor to autograd and the module drops it; a later direct
    run() / measure_average_time() on the same cached module gets a new output tensor instead of a null pointer."""
    import torch
    from featgraph_amd.autograd import Graph
    rng = np.random.default_rng(3)
    adj = sp.random(300, 300, density=0.05, format="csr", random_state=rng).astype("float32")
    adj.sort_indices()
    g = Graph(adj)
    x = torch.randn((300, 16), device="cuda", requires_grad=True)
    w = torch.rand(adj.nnz, device="cuda")
    y = g.spmm(x, w)
    y.sum().backward()
    s = g.sddmm(x.detach(), x.detach())
    a = g.edge_softmax(s)
    for key, mod in list(g._mods.items()):
        if key[0] == 'spmm' and not key[1]:
            assert mod.out_tvm is None
            again = mod.run([x.detach(), w])
            assert torch.equal(again, y.detach())
            assert mod.measure_average_time([x.detach(), w], 2) > 0
        if key[0] == 'sddmm':
            assert torch.equal(mod.run([x.detach(), x.detach()]), s)
        if key[0] == 'softmax':
            assert torch.equal(mod.run([s]), a)
            mod.backward(a, torch.ones_like(a))
