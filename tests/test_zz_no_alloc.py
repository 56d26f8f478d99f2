"""fg_spmm_csr_noalloc_f32 -- the SpMM entry point that allocates nothing (its split rows' partial sums
live in a fixed array of the library's device image) -- against fg_spmm_csr_f32, called through the C ABI:
bit-identical results on two calls in a row, the second on a smaller input, and a clear refusal beyond the
array's size."""
import ctypes

import numpy as np
import pytest
import scipy.sparse as sp

pytestmark = pytest.mark.gpu


def _graph(rng, n_dst, n_src, long_rows, long_len, density):
    a = sp.random(n_dst, n_src, density=density, format="csr", random_state=rng).astype("float32").tolil()
    for r in long_rows:
        a[r, rng.choice(n_src, size=long_len, replace=False)] = 1.0      # longer than the split threshold
    a[1, :] = 0                                                          # an empty row
    a = a.tocsr().astype("float32"); a.eliminate_zeros(); a.sort_indices()
    a.data = (rng.random(a.nnz) + 0.05).astype("float32")
    return a


def _both(L, lib, adj, x, F, T):
    """(result of fg_spmm_csr_f32, result of fg_spmm_csr_noalloc_f32, status of the latter)."""
    import torch
    indptr = np.ascontiguousarray(adj.indptr, dtype=np.int32)
    plan = ctypes.c_void_p()
    assert L.fg_spmm_plan_create(lib.host_ptr(indptr), adj.shape[0], adj.shape[1], 1, None, ctypes.byref(plan)) == 0
    try:
        ip, ix, vals = (torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (indptr, adj.indices, adj.data))
        p = lib.dev_ptr
        s = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        ref = torch.full((adj.shape[0], F), float("nan"), device="cuda")
        got = torch.full((adj.shape[0], F), float("nan"), device="cuda")
        assert L.fg_spmm_csr_f32(plan, p(ip), p(ix), p(vals), p(x), p(ref), F, T, s) == 0
        rc = L.fg_spmm_csr_noalloc_f32(plan, p(ip), p(ix), p(vals), p(x), p(got), F, T, s)
        torch.cuda.synchronize()
        return ref, got, rc
    finally:
        L.fg_spmm_plan_destroy(plan)


def test_noalloc_matches_the_allocating_entry_point():
    import torch
    from featgraph_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(71)
    # first call: several split rows, 4 feature tiles
    big = _graph(rng, 300, 5000, (3, 40, 41, 250), 4500, 0.01)
    x1 = torch.from_numpy(rng.standard_normal((5000, 256)).astype("float32")).cuda()
    ref, got, rc = _both(L, _lib, big, x1, 256, 4)
    assert rc == 0
    assert torch.isfinite(ref).all() and torch.equal(ref, got)
    exact = big.astype(np.float64).dot(x1.cpu().numpy().astype(np.float64))
    np.testing.assert_allclose(got.cpu().numpy(), exact, rtol=1e-4, atol=2e-4)
    # second call, smaller in every way: the array still holds the first call's pieces
    small = _graph(rng, 40, 1500, (7,), 1300, 0.02)
    x2 = torch.from_numpy(rng.standard_normal((1500, 32)).astype("float32")).cuda()
    ref, got, rc = _both(L, _lib, small, x2, 32, 0)
    assert rc == 0
    assert torch.isfinite(ref).all() and torch.equal(ref, got)
    # no split rows at all, odd feature length
    plain = _graph(rng, 60, 200, (), 0, 0.1)
    x3 = torch.from_numpy(rng.standard_normal((200, 7)).astype("float32")).cuda()
    ref, got, rc = _both(L, _lib, plain, x3, 7, 0)
    assert rc == 0 and torch.equal(ref, got)


def test_noalloc_refuses_what_does_not_fit():
    import torch
    from featgraph_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(72)
    # 200 rows of 2100 elements: 3 pieces each = 600 pieces; at F = 8192 that is 4.9 M floats > 4 Mi
    adj = _graph(rng, 210, 2200, tuple(range(5, 205)), 2100, 0.001)
    x = torch.zeros((2200, 8192), device="cuda")
    ref, got, rc = _both(L, _lib, adj, x, 8192, 0)
    assert rc == -2 and b"fixed buffer" in L.fg_last_error()
    assert torch.isnan(got).all()                       # nothing was launched
    # a plan with column partitions, and a null plan
    s1_pos = np.array([0, 1, 1, 2], dtype=np.int32)
    plan2 = ctypes.c_void_p()
    assert L.fg_spmm_plan_create(_lib.host_ptr(s1_pos), 1, 4, 2, None, ctypes.byref(plan2)) == 0
    try:
        p = _lib.dev_ptr
        assert L.fg_spmm_csr_noalloc_f32(plan2, p(x), p(x), p(x), p(x), p(x), 8, 0, None) == -1
        assert L.fg_spmm_csr_noalloc_f32(None, p(x), p(x), p(x), p(x), p(x), 8, 0, None) == -1
    finally:
        L.fg_spmm_plan_destroy(plan2)


def test_noalloc_allocates_nothing_and_can_be_the_recorded_call():
    """The entry point on a plan whose scratch was never reserved: the plan's device memory and the device's free memory
    are the same before and after, and its very first call may be the one recorded into a HIP graph (the fixed array's
    address is looked up when the plan is created); replays between eager work reproduce the eager result bit for bit."""
    import torch
    from featgraph_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(73)
    adj = _graph(rng, 300, 4000, (3, 40, 250), 3500, 0.01)
    F = 128
    indptr = np.ascontiguousarray(adj.indptr, dtype=np.int32)
    p = _lib.dev_ptr
    x = torch.from_numpy(rng.standard_normal((4000, F)).astype("float32")).cuda()
    ip, ix, vals = (torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (indptr, adj.indices, adj.data))
    ref = torch.full((300, F), float("nan"), device="cuda")
    got = torch.full((300, F), float("nan"), device="cuda")
    plan = ctypes.c_void_p()
    assert L.fg_spmm_plan_create(_lib.host_ptr(indptr), 300, 4000, 1, None, ctypes.byref(plan)) == 0
    plan_ref = ctypes.c_void_p()
    assert L.fg_spmm_plan_create(_lib.host_ptr(indptr), 300, 4000, 1, None, ctypes.byref(plan_ref)) == 0
    try:
        assert L.fg_spmm_csr_f32(plan_ref, p(ip), p(ix), p(vals), p(x), p(ref), F, 2, None) == 0
        torch.cuda.synchronize()
        bytes_before = L.fg_spmm_plan_bytes(plan)
        free_before = torch.cuda.mem_get_info()[0]
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            s = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            rc = L.fg_spmm_csr_noalloc_f32(plan, p(ip), p(ix), p(vals), p(x), p(got), F, 2, s)
        assert rc == 0, L.fg_last_error()
        for k in range(3):
            got.fill_(float("nan"))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(got, ref), "replay %d differs" % k
            # eager work of another shape between the replays shares the fixed array
            small = _graph(rng, 40, 1500, (7,), 1300, 0.02)
            x2 = torch.from_numpy(rng.standard_normal((1500, 32)).astype("float32")).cuda()
            r2, g2, rc2 = _both(L, _lib, small, x2, 32, 0)
            assert rc2 == 0 and torch.equal(r2, g2)
        assert L.fg_spmm_plan_bytes(plan) == bytes_before              # the plan's scratch was never grown
        x.copy_(x * 2)                                                  # new inputs through the same graph
        graph.replay()
        torch.cuda.synchronize()
        assert L.fg_spmm_csr_f32(plan_ref, p(ip), p(ix), p(vals), p(x), p(ref), F, 2, None) == 0
        torch.cuda.synchronize()
        assert torch.equal(got, ref)
        del graph
        assert torch.cuda.mem_get_info()[0] >= free_before - (8 << 20)  # nothing of the operator's size was taken from the device
    finally:
        L.fg_spmm_plan_destroy(plan)
        L.fg_spmm_plan_destroy(plan_ref)
