"""The operators allocate nothing after their first call and launch only on the caller's stream, so a
call can be recorded into a HIP graph and replayed.  Each replay is checked against the eager result
of the same inputs, with eager work and synchronisation between the replays."""
import numpy as np
import pytest
import scipy.sparse as sp

from helpers import RTOL

pytestmark = pytest.mark.gpu


def test_spmm_sddmm_softmax_replay():
    import torch
    from featgraph_amd.module import (VanillaSpMMhip, VanillaSDDMMhip, EdgeSoftmaxhip, placeholder)
    rng = np.random.default_rng(3)
    n_dst, n_src, F = 700, 900, 128
    adj = sp.random(n_dst, n_src, density=0.05, format="csr", random_state=rng).astype("float32").tolil()
    cols = rng.choice(n_src, size=850, replace=False)
    adj[11, cols] = 1.0                                    # one long row
    adj = adj.tocsr().astype("float32"); adj.sort_indices()
    adj.data = rng.random(adj.nnz).astype("float32")
    nnz = adj.nnz

    spmm = VanillaSpMMhip(adj, 4)                           # DDS, 4 passes, later ones add in place
    spmm.build([placeholder((n_src, F))], {'num_feat_partitions': 2}, {})
    sddmm = VanillaSDDMMhip(adj)
    sddmm.build([placeholder((n_src, F)), placeholder((n_dst, F))], {},
                {'order': 'tiled', 'num_src_partitions': 2, 'num_feat_tiles': 2})
    soft = EdgeSoftmaxhip(adj)
    soft.build([placeholder((nnz,))])

    x = torch.zeros((n_src, F), device="cuda")
    y = torch.zeros((n_dst, F), device="cuda")

    def chain():
        out = spmm.run([x])
        s = sddmm.run([x, y])
        a = soft.run([s])
        return out, s, a

    chain()                                                # first call: scratch is allocated here
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_out, g_s, g_a = chain()
    gen = torch.Generator(device="cuda")
    for k in range(4):
        gen.manual_seed(10 + k)
        x.copy_(torch.randn((n_src, F), generator=gen, device="cuda"))
        y.copy_(torch.randn((n_dst, F), generator=gen, device="cuda") * 0.1)
        e_out, e_s, e_a = (t.clone() for t in chain())     # eager, same tensors
        torch.cuda.synchronize()
        for t in (spmm.out_tvm, sddmm.out_tvm, soft.out_tvm):
            t.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(g_out, e_out), "SpMM replay %d differs from the eager run" % k
        assert torch.equal(g_s, e_s), "SDDMM replay %d differs from the eager run" % k
        assert torch.equal(g_a, e_a), "edge softmax replay %d differs from the eager run" % k
        ref = adj.astype(np.float64).dot(x.cpu().numpy().astype(np.float64))
        np.testing.assert_allclose(g_out.cpu().numpy(), ref, rtol=RTOL, atol=1e-4)


@pytest.mark.parametrize("scores", ["dot", "additive"])
def test_attention_replay(scores):
    """Forward and gradient kernels of the attention operator recorded once and replayed on new inputs."""
    import torch
    from featgraph_amd.module import GraphAttentionhip, placeholder
    rng = np.random.default_rng(5)
    n_dst, n_src, H, D = 400, 600, 4, 32
    adj = sp.random(n_dst, n_src, density=0.05, format="csr", random_state=rng).astype("float32").tolil()
    adj[3, rng.choice(n_src, size=550, replace=False)] = 1.0
    adj[5, :] = 0
    adj = adj.tocsr().astype("float32"); adj.eliminate_zeros(); adj.sort_indices()
    m = GraphAttentionhip(adj)
    v = torch.zeros((n_src, H, D), device="cuda")
    d = torch.zeros((n_dst, H, D), device="cuda")
    if scores == "additive":
        a = torch.zeros((n_dst, H), device="cuda"); b = torch.zeros((n_src, H), device="cuda")
        m.build([placeholder(a.shape), placeholder(b.shape), placeholder(v.shape)], {'scores': 'additive'},
                {'num_src_partitions': 3, 'num_dst_partitions': 2})
    else:
        a = torch.zeros((n_dst, H, D), device="cuda"); b = torch.zeros((n_src, H, D), device="cuda")
        m.build([placeholder(a.shape), placeholder(b.shape), placeholder(v.shape)], {},
                {'num_src_partitions': 3, 'num_dst_partitions': 2})

    def step():
        out = m.run([a, b, v])
        return (out,) + tuple(m.backward(a, b, v, out, m.state_tvm, d))

    step()                                                 # first call: plans' scratch is allocated here
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        recorded = step()
    gen = torch.Generator(device="cuda")
    for k in range(3):
        gen.manual_seed(20 + k)
        for t in (a, b, v, d):
            t.copy_(torch.randn(t.shape, generator=gen, device="cuda"))
        eager = tuple(t.clone() for t in step())
        torch.cuda.synchronize()
        for t in recorded:
            t.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for i, (r, e) in enumerate(zip(recorded, eager)):
            assert torch.isfinite(e).all()
            assert torch.equal(r, e), "replay %d: result %d differs from the eager run" % (k, i)


def test_scratch_is_reserved_at_build_and_never_grown_under_capture():
    """build() sizes the plan's scratch (fg_spmm_plan_reserve), so the first run() of a module can be the
    recorded one; a direct C-ABI call that would have to grow the scratch while its stream is being
    captured changes nothing and reports FG_ERR_ARG."""
    import ctypes
    import torch
    from featgraph_amd import _lib
    from featgraph_amd.module import VanillaSpMMhip, placeholder
    rng = np.random.default_rng(9)
    n_dst, n_src = 64, 3000
    adj = sp.random(n_dst, n_src, density=0.01, format="csr", random_state=rng).astype("float32").tolil()
    adj[5, rng.choice(n_src, size=2600, replace=False)] = 1.0       # split into pieces: needs scratch
    adj = adj.tocsr().astype("float32"); adj.sort_indices()
    adj.data = rng.random(adj.nnz).astype("float32")
    warm = VanillaSpMMhip(adj)
    warm.build([placeholder((n_src, 8))], {}, {})
    x8 = torch.randn((n_src, 8), device="cuda")
    warm.run([x8])                                                  # the library's kernels are loaded
    torch.cuda.synchronize()

    F = 256
    m = VanillaSpMMhip(adj)
    m.build([placeholder((n_src, F))], {}, {})
    x = torch.randn((n_src, F), device="cuda")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        recorded = m.run([x])                                       # first call of this module
    graph.replay()
    torch.cuda.synchronize()
    ref = adj.astype(np.float64).dot(x.cpu().numpy().astype(np.float64))
    np.testing.assert_allclose(recorded.cpu().numpy(), ref, rtol=RTOL, atol=1e-4)

    # the C ABI without a reservation
    L = _lib.lib()
    plan = ctypes.c_void_p()
    indptr = np.ascontiguousarray(adj.indptr, dtype=np.int32)
    assert L.fg_spmm_plan_create(_lib.host_ptr(indptr), n_dst, n_src, 1, None, ctypes.byref(plan)) == 0
    try:
        ip, ix, vals = (torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (indptr, adj.indices, adj.data))
        out = torch.full((n_dst, F), float("nan"), device="cuda")
        p = _lib.dev_ptr
        g2 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g2):
            s = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            rc = L.fg_spmm_csr_f32(plan, p(ip), p(ix), p(vals), p(x), p(out), F, 0, s)
        assert rc == -1 and b"fg_spmm_plan_reserve" in L.fg_last_error()
        assert L.fg_spmm_plan_reserve(plan, 0, 1, F, 0) == 0
        g3 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g3):
            s = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            rc = L.fg_spmm_csr_f32(plan, p(ip), p(ix), p(vals), p(x), p(out), F, 0, s)
        assert rc == 0
        g3.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, recorded)
        assert L.fg_spmm_plan_reserve(plan, 99, 1, F, 0) == -1
        assert L.fg_spmm_plan_reserve(plan, 2, 1, 24, 1) == -2          # a tile the tiled SDDMM does not take
    finally:
        L.fg_spmm_plan_destroy(plan)


@pytest.mark.parametrize("partitions", [None, 2])
def test_broadcasting_operators_replay_without_a_warm_up_call(partitions):
    """build() reserves the split rows' scratch (and, over source partitions, the partitions' buffers of results), so the
    first run() may already be the recorded one."""
    import torch
    from featgraph_amd.module import GSpMMhip, GSDDMMhip, placeholder
    rng = np.random.default_rng(8)
    n_dst, n_src, F = 300, 2500, 24
    adj = sp.random(n_dst, n_src, density=0.02, format="csr", random_state=rng).astype("float32").tolil()
    adj[7, rng.choice(n_src, size=2200, replace=False)] = 1.0       # a row that is split into pieces
    adj = adj.tocsr().astype("float32"); adj.sort_indices()
    nnz = adj.nnz
    agg = GSpMMhip(adj)
    agg.build([placeholder((n_src, F)), placeholder((nnz, F))], {'msg': 'u_mul_e', 'reduce': 'max', 'return_arg': True},
              {'num_src_partitions': partitions})
    assert agg._active['P'] == (partitions or 1)
    edge = GSDDMMhip(adj.tocoo())
    edge.build([placeholder((nnz, F)), placeholder((n_dst, 1))], {'op': 'add', 'lhs_target': 'e', 'rhs_target': 'v'}, {})
    x = torch.zeros((n_src, F), device="cuda")
    ef = torch.zeros((nnz, F), device="cuda")
    b = torch.zeros((n_dst, 1), device="cuda")

    def chain():
        return agg.run([x, ef]), edge.run([ef, b])

    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_out, g_edge = chain()
    gen = torch.Generator(device="cuda")
    for k in range(3):
        gen.manual_seed(20 + k)
        x.copy_(torch.randn((n_src, F), generator=gen, device="cuda"))
        ef.copy_(torch.randn((nnz, F), generator=gen, device="cuda"))
        b.copy_(torch.randn((n_dst, 1), generator=gen, device="cuda"))
        e_out, e_edge = (t.clone() for t in chain())
        e_arg = agg.arg_tvm.clone()
        torch.cuda.synchronize()
        agg.out_tvm.fill_(float("nan")); agg.arg_tvm.fill_(-7); edge.out_tvm.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(g_out, e_out) and torch.equal(agg.arg_tvm, e_arg), "aggregation replay %d" % k
        assert torch.equal(g_edge, e_edge), "edge operator replay %d" % k
