"""featgraph_amd.ops: gspmm / gsddmm with DGL's call signatures, against the same formulas written with gather /
index_add in float64 (values and, where the call is differentiable, gradients).  The reference snapshot has no such
functions (README.md:9-14 points to them); DGL's documented semantics are the specification."""
import numpy as np
import pytest
import scipy.sparse as sp

pytestmark = pytest.mark.gpu

_OP = {'add': lambda a, b: a + b, 'sub': lambda a, b: a - b, 'mul': lambda a, b: a * b, 'div': lambda a, b: a / b}


def _setup(seed=0):
    import torch
    from featgraph_amd.autograd import Graph
    rng = np.random.default_rng(seed)
    adj = sp.random(120, 170, density=0.06, format="csr", random_state=rng).astype("float32").tolil()
    adj[[3, 77], :] = 0
    adj = adj.tocsr().astype("float32"); adj.sort_indices()
    coo = adj.tocoo()
    rows = torch.from_numpy(coo.row.astype(np.int64)).cuda()
    cols = torch.from_numpy(coo.col.astype(np.int64)).cuda()
    return torch, Graph(adj), adj, rows, cols


def _align(a, b):
    nd = max(a.dim(), b.dim())
    a = a.reshape((a.shape[0],) + (1,) * (nd - a.dim()) + tuple(a.shape[1:]))
    b = b.reshape((b.shape[0],) + (1,) * (nd - b.dim()) + tuple(b.shape[1:]))
    return a, b


def _reduce64(torch, m, rows, n_dst, reduce_op, deg):
    if reduce_op in ("sum", "mean"):
        out = torch.zeros((n_dst,) + tuple(m.shape[1:]), dtype=torch.float64, device="cuda").index_add(0, rows, m)
        return out / deg.clamp(min=1).reshape((-1,) + (1,) * (out.dim() - 1)) if reduce_op == "mean" else out
    fill = float("-inf") if reduce_op == "max" else float("inf")
    out = torch.full((n_dst,) + tuple(m.shape[1:]), fill, dtype=torch.float64, device="cuda")
    idx = rows.reshape((-1,) + (1,) * (m.dim() - 1)).expand_as(m)
    out = out.scatter_reduce(0, idx, m, "amax" if reduce_op == "max" else "amin", include_self=True)
    return torch.where(torch.isinf(out), torch.zeros_like(out), out)


@pytest.mark.parametrize("op,reduce_op,l_shape,r_shape", [
    ("mul", "sum", (32,), ()), ("mul", "sum", (4, 8), (4, 1)), ("mul", "sum", (16,), (16,)), ("add", "mean", (8,), (1,)),
    ("sub", "sum", (2, 3), (3,)), ("div", "sum", (8,), (8,)), ("mul", "max", (8,), (8,)), ("add", "min", (5,), (1,)),
    ("div", "mean", (4, 1), (1, 6)), ("div", "max", (6,), (1,)), ("sub", "min", (1,), (7,)), ("mul", "min", (2, 4), (2, 1)),
    ("copy_lhs", "sum", (12,), None), ("copy_lhs", "max", (3, 4), None), ("copy_rhs", "sum", None, (6,)),
    ("copy_rhs", "min", None, (2, 2)), ("copy_lhs", "mean", (), None),
])
def test_gspmm(op, reduce_op, l_shape, r_shape):
    from featgraph_amd import ops
    torch, g, adj, rows, cols = _setup(len(op) + len(reduce_op))
    gen = torch.Generator(device="cuda"); gen.manual_seed(3)
    n_dst, n_src, nnz = adj.shape[0], adj.shape[1], adj.nnz
    deg = torch.from_numpy(np.diff(adj.indptr)).cuda().double()
    differentiable = True

    def make(n, shape):
        if shape is None:
            return None
        t = torch.randn((n,) + shape, generator=gen, device="cuda")
        t = t.abs() + 0.5 if op == "div" else t
        return t.requires_grad_() if differentiable else t

    lhs, rhs = make(n_src, l_shape), make(nnz, r_shape)
    out = ops.gspmm(g, op, reduce_op, lhs, rhs)
    l64 = lhs.detach().double().requires_grad_() if lhs is not None else None
    r64 = rhs.detach().double().requires_grad_() if rhs is not None else None
    if op == "copy_lhs":
        m = l64[cols]
    elif op == "copy_rhs":
        m = r64
    else:
        a, b = _align(l64[cols], r64)
        m = _OP[op](a, b)
    if m.dim() == 1:
        m = m[:, None]
    ref = _reduce64(torch, m, rows, n_dst, reduce_op, deg)
    assert tuple(out.shape) == tuple(ref.shape) or tuple(out.shape) + (1,) == tuple(ref.shape)
    ref = ref.reshape(out.shape)
    assert torch.allclose(out.double(), ref, rtol=1e-4, atol=1e-4)
    if differentiable:
        up = torch.randn(out.shape, generator=gen, device="cuda")
        (out * up).sum().backward()
        (ref * up.double()).sum().backward()
        if lhs is not None:
            assert torch.allclose(lhs.grad.double(), l64.grad, rtol=1e-4, atol=1e-4)
        if rhs is not None:
            assert torch.allclose(rhs.grad.double(), r64.grad, rtol=1e-4, atol=1e-4)
    else:
        with pytest.raises(NotImplementedError):
            ops.gspmm(g, op, reduce_op, lhs.clone().requires_grad_() if lhs is not None else None,
                      rhs.clone().requires_grad_() if rhs is not None else None)


@pytest.mark.parametrize("op,lt,l_shape,rt,r_shape", [
    ("dot", 'u', (24,), 'v', (24,)), ("dot", 'u', (4, 8), 'v', (4, 8)), ("dot", 'v', (16,), 'u', (16,)),
    ("dot", 'e', (2, 4), 'u', (1, 4)), ("add", 'u', (8,), 'v', (8,)), ("mul", 'e', (4, 1), 'v', (4, 8)),
    ("sub", 'v', (3,), 'u', (1,)), ("div", 'u', (6,), 'e', (6,)), ("div", 'e', (2, 3), 'v', (3,)), ("div", 'v', (1,), 'u', (5,)),
    ("copy_lhs", 'u', (5,), 'v', (1,)),
    ("copy_rhs", 'u', (1,), 'v', (2, 3)), ("copy_lhs", 'e', (4,), 'v', (1,)),
])
def test_gsddmm(op, lt, l_shape, rt, r_shape):
    from featgraph_amd import ops
    torch, g, adj, rows, cols = _setup(len(op) + sum(l_shape))
    gen = torch.Generator(device="cuda"); gen.manual_seed(4)
    n_of = {'u': adj.shape[1], 'v': adj.shape[0], 'e': adj.nnz}
    differentiable = op in ("add", "sub", "mul", "div", "copy_lhs", "copy_rhs") or (op == "dot" and {lt, rt} == {'u', 'v'})

    def make(n, shape):
        t = torch.randn((n,) + shape, generator=gen, device="cuda")
        t = t.abs() + 0.5 if op == "div" else t
        return t.requires_grad_() if differentiable else t

    lhs, rhs = make(n_of[lt], l_shape), make(n_of[rt], r_shape)
    out = ops.gsddmm(g, op, lhs, rhs, lt, rt)
    pick = lambda t, target: t[cols] if target == 'u' else t[rows] if target == 'v' else t
    l64, r64 = lhs.detach().double().requires_grad_(), rhs.detach().double().requires_grad_()
    if op == "copy_lhs":
        ref = pick(l64, lt)
    elif op == "copy_rhs":
        ref = pick(r64, rt)
    else:
        a, b = _align(pick(l64, lt), pick(r64, rt))
        ref = (a * b).sum(-1, keepdim=True) if op == "dot" else _OP[op](a, b)
    assert tuple(out.shape) == tuple(ref.shape), (out.shape, ref.shape)
    assert torch.allclose(out.double(), ref, rtol=1e-4, atol=1e-4)
    if differentiable:
        up = torch.randn(out.shape, generator=gen, device="cuda")
        (out * up).sum().backward()
        (ref * up.double()).sum().backward()
        if op != "copy_rhs":
            assert torch.allclose(lhs.grad.double(), l64.grad, rtol=1e-4, atol=1e-4)
        if op != "copy_lhs":
            assert torch.allclose(rhs.grad.double(), r64.grad, rtol=1e-4, atol=1e-4)
    else:
        with pytest.raises(NotImplementedError):
            ops.gsddmm(g, op, lhs.clone().requires_grad_(), rhs, lt, rt)


def test_edge_softmax_shapes():
    from featgraph_amd import ops
    torch, g, adj, rows, cols = _setup(9)
    s = torch.randn((adj.nnz, 4, 1), device="cuda")
    a = ops.edge_softmax(g, s)
    assert a.shape == s.shape
    sums = torch.zeros((adj.shape[0], 4), device="cuda").index_add(0, rows, a[..., 0])
    has = torch.from_numpy(np.diff(adj.indptr) > 0).cuda()
    assert torch.allclose(sums[has], torch.ones_like(sums[has]), atol=1e-5)
