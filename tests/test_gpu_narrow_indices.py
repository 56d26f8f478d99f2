"""16-bit copy of a layout's column ids (fg_spmm_plan_narrow_indices): the sum SpMM and the tiled SDDMM read it
instead of the int32 array whenever a partition is at most 65,536 columns wide.  The ids are the same, so every
result must agree bit for bit with the int32 stream -- on graphs with empty rows, rows split over wavefronts,
item starts at odd element positions (a 16-bit word is only 2-byte aligned there) and ids up to 65,535."""
import ctypes

import numpy as np
import pytest
import scipy.sparse as sp

from helpers import assert_sum_close, spmm_mass

pytestmark = pytest.mark.gpu


def _graph(rng, n_rows=500, n_cols=4000, long_len=2700):
    a = sp.random(n_rows, n_cols, density=0.012, format="csr", random_state=rng,
                  data_rvs=lambda k: rng.standard_normal(k)).astype("float32").tolil()
    a[[0, 1, n_rows // 2, n_rows - 1], :] = 0
    a[3, :] = 0
    a[3, [n_cols - 1]] = 2.0                                            # one element: later rows start at odd positions
    a[7, rng.choice(n_cols, size=long_len, replace=False)] = 1.5       # longer than the split threshold
    a = a.tocsr().astype("float32"); a.eliminate_zeros(); a.sort_indices()
    return a


def _with(narrow, fn):
    from featgraph_amd.module import common
    old = common.NARROW_INDICES
    common.NARROW_INDICES = narrow
    try:
        return fn()
    finally:
        common.NARROW_INDICES = old


@pytest.mark.parametrize("feat_len,P,T", [(128, 1, 0), (128, 2, 2), (64, 8, 0), (512, 4, 8), (96, 3, 3), (32, 5, 1), (7, 3, 1)])
def test_spmm_bit_identical(oracle, feat_len, P, T):
    import torch
    from featgraph_amd.module import VanillaSpMMhip, placeholder
    rng = np.random.default_rng(100 + feat_len + P)
    adj = _graph(rng)
    x = rng.standard_normal((adj.shape[1], feat_len)).astype("float32")
    xd = torch.from_numpy(x).cuda()

    def run():
        m = VanillaSpMMhip(adj, P)
        m.build([placeholder(x.shape)], {'num_feat_partitions': T}, {'num_src_partitions': None})
        m.out_tvm.fill_(float("nan"))
        return m.run([xd]).cpu().numpy().copy()

    wide, narrow = _with(False, run), _with(True, run)
    assert np.array_equal(wide, narrow)
    assert_sum_close(narrow, oracle.spmm_f64(adj, x), spmm_mass(adj, x), "F=%d P=%d T=%d" % (feat_len, P, T))


def test_per_head_weights_bit_identical():
    import torch
    from featgraph_amd.module import GSpMMhip, placeholder
    rng = np.random.default_rng(5)
    adj = _graph(rng)
    H, D = 4, 32
    x = rng.standard_normal((adj.shape[1], H, D)).astype("float32")
    w = rng.random((adj.nnz, H)).astype("float32")

    def run():
        m = GSpMMhip(adj, 3)
        m.build([placeholder(x.shape), placeholder(w.shape)], {}, {'num_src_partitions': None})
        return m.run([torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()]).cpu().numpy().copy()

    assert np.array_equal(_with(False, run), _with(True, run))


@pytest.mark.parametrize("H,D,P,T", [(1, 128, 2, 2), (1, 512, 3, 8), (1, 64, 4, 1), (4, 32, 2, 2), (8, 64, 2, 8)])
def test_sddmm_tiled_bit_identical(H, D, P, T):
    import torch
    from featgraph_amd.module import VanillaSDDMMhip, MultiHeadSDDMMhip, placeholder
    rng = np.random.default_rng(200 + H * D + P)
    adj = _graph(rng)
    shape_s = (adj.shape[1], D) if H == 1 else (adj.shape[1], H, D)
    shape_d = (adj.shape[0], D) if H == 1 else (adj.shape[0], H, D)
    src = rng.standard_normal(shape_s).astype("float32")
    dst = rng.standard_normal(shape_d).astype("float32")

    def run():
        m = (VanillaSDDMMhip if H == 1 else MultiHeadSDDMMhip)(adj)
        m.build([placeholder(shape_s), placeholder(shape_d)], {}, {'order': 'tiled', 'num_src_partitions': P, 'num_feat_tiles': T})
        m.out_tvm.fill_(float("nan"))
        return m.run([torch.from_numpy(src).cuda(), torch.from_numpy(dst).cuda()]).cpu().numpy().copy()

    wide, narrow = _with(False, run), _with(True, run)
    assert np.array_equal(wide, narrow)
    coo = adj.tocoo()
    ref = np.einsum('e...d,e...d->e...', src[coo.col].astype(np.float64), dst[coo.row].astype(np.float64))
    np.testing.assert_allclose(narrow, ref, rtol=1e-4, atol=1e-3)


def test_ids_up_to_65535_and_other_arrays():
    """C ABI directly: a 65,536-column partition's largest id survives the narrowing; a call that hands the kernels
    another index array than the one that was narrowed reads that array (as int32); releasing the copy works."""
    import torch
    from featgraph_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(9)
    n_dst, n_src, F = 300, 65536, 64
    rows = []
    for r in range(n_dst):
        cols = np.unique(np.concatenate([rng.integers(0, n_src, size=rng.integers(0, 40)), [65535] if r % 3 == 0 else []])).astype(np.int32)
        rows.append(cols)
    indptr = np.zeros(n_dst + 1, np.int32)
    indptr[1:] = np.cumsum([len(c) for c in rows])
    indices = np.concatenate(rows).astype(np.int32)
    vals = rng.random(indices.shape[0]).astype("float32")
    x = rng.standard_normal((n_src, F)).astype("float32")
    ref = sp.csr_matrix((vals.astype(np.float64), indices, indptr), shape=(n_dst, n_src)).dot(x.astype(np.float64))
    plan = ctypes.c_void_p()
    _lib.check(L.fg_spmm_plan_create(_lib.host_ptr(indptr), n_dst, n_src, 1, None, ctypes.byref(plan)))
    try:
        ip, ix, vl, xd = (torch.from_numpy(a).cuda() for a in (indptr, indices, vals, x))
        ix_other = ix.clone()
        out = torch.empty((n_dst, F), device="cuda")
        stream = torch.cuda.current_stream().cuda_stream

        def spmm(idx):
            out.fill_(float("nan"))
            _lib.check(L.fg_spmm_csr_f32(plan, _lib.dev_ptr(ip), _lib.dev_ptr(idx), _lib.dev_ptr(vl), _lib.dev_ptr(xd),
                                         _lib.dev_ptr(out), F, 0, stream))
            return out.cpu().numpy().copy()

        base = spmm(ix)
        _lib.check(L.fg_spmm_plan_narrow_indices(plan, _lib.dev_ptr(ix), stream))
        assert np.array_equal(spmm(ix), base)
        np.testing.assert_allclose(base, ref, rtol=1e-4, atol=1e-4)
        # the narrowed array's contents no longer matter to a call that passes another array
        assert np.array_equal(spmm(ix_other), base)
        _lib.check(L.fg_spmm_plan_narrow_indices(plan, None, stream))
        assert np.array_equal(spmm(ix), base)
    finally:
        L.fg_spmm_plan_destroy(plan)
    # partitions wider than 65,536 columns are refused
    indptr2 = np.zeros(3, np.int32)
    plan2 = ctypes.c_void_p()
    _lib.check(L.fg_spmm_plan_create(_lib.host_ptr(indptr2), 2, 65537, 1, None, ctypes.byref(plan2)))
    try:
        dummy = torch.zeros(4, dtype=torch.int32, device="cuda")
        assert L.fg_spmm_plan_narrow_indices(plan2, _lib.dev_ptr(dummy), None) == -2
        assert b"16 bits" in L.fg_last_error()
    finally:
        L.fg_spmm_plan_destroy(plan2)


@pytest.mark.parametrize("additive", [False, True])
@pytest.mark.parametrize("P", [1, 3])
def test_attention_bit_identical(additive, P):
    """Forward pass and both gradient sweeps (the second one over the transposed adjacency's own layout)."""
    import torch
    from featgraph_amd.module import GraphAttentionhip, placeholder
    rng = np.random.default_rng(31 + P)
    adj = _graph(rng, n_rows=600, n_cols=600, long_len=500)
    n, H, D = 600, 2, 64
    q = torch.from_numpy(rng.standard_normal((n, H) if additive else (n, H, D)).astype("float32")).cuda()
    k = torch.from_numpy(rng.standard_normal((n, H) if additive else (n, H, D)).astype("float32")).cuda()
    v = torch.from_numpy(rng.standard_normal((n, H, D)).astype("float32")).cuda()
    g = torch.from_numpy(rng.standard_normal((n, H, D)).astype("float32")).cuda()

    def run():
        m = GraphAttentionhip(adj)
        m.build([placeholder(tuple(q.shape)), placeholder(tuple(k.shape)), placeholder(tuple(v.shape))],
                {'scores': 'additive'} if additive else {}, {'num_src_partitions': P, 'num_dst_partitions': P})
        out = m.run([q, k, v]).clone()
        grads = m.backward(q, k, v, m.out_tvm, m.state_tvm, g)
        return [out.cpu().numpy()] + [t.cpu().numpy() for t in grads]

    wide, narrow = _with(False, run), _with(True, run)
    for a, b in zip(wide, narrow):
        assert np.isfinite(b).all()
        assert np.array_equal(a, b)


@pytest.mark.parametrize("msg,reduce,P", [("u_add_e", "sum", None), ("u_mul_e", "max", None), ("u_add_e", "sum", 3), ("copy_u", "min", 2)])
def test_broadcasting_spmm_bit_identical(msg, reduce, P):
    import torch
    from featgraph_amd.module import GSpMMhip, placeholder
    rng = np.random.default_rng(77)
    adj = _graph(rng)
    F = 64
    x = rng.standard_normal((adj.shape[1], F)).astype("float32")
    e = rng.standard_normal((adj.nnz, 1)).astype("float32")

    def run():
        m = GSpMMhip(adj)
        phs = [placeholder(x.shape)] + ([placeholder(e.shape)] if msg != "copy_u" else [])
        m.build(phs, {'msg': msg, 'reduce': reduce}, {'num_src_partitions': P})
        ins = [torch.from_numpy(x).cuda()] + ([torch.from_numpy(e).cuda()] if msg != "copy_u" else [])
        return m.run(ins).cpu().numpy().copy()

    wide, narrow = _with(False, run), _with(True, run)
    assert np.isfinite(narrow).all()
    assert np.array_equal(wide, narrow)


def _small_csr(rng, n_dst, n_src, per_row):
    rows = [np.unique(rng.integers(0, n_src, size=per_row)).astype(np.int32) for _ in range(n_dst)]
    indptr = np.zeros(n_dst + 1, np.int32)
    indptr[1:] = np.cumsum([len(c) for c in rows])
    return indptr, np.concatenate(rows).astype(np.int32)


def test_rewritten_ids_need_a_new_copy_and_the_debug_check_sees_stale_ones():
    """C ABI directly.  The 16-bit copy is bound to the int32 array by address: after the array has been overwritten in
    place with other ids (what an allocator that hands the same address out again amounts to), narrowing again gives
    the new product; without it the stale copy would be gathered through -- which fg_debug_checks(1) detects by the
    array's fingerprint, reading the int32 array instead and leaving a message."""
    import torch
    from featgraph_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(12)
    n_dst, n_src, F = 400, 3000, 32
    indptr, idx_a = _small_csr(rng, n_dst, n_src, 20)
    # other ids with the same row lengths (sorted inside each row), different in the first and the last rows as well
    idx_b = np.concatenate([np.sort(rng.choice(n_src, size=indptr[r + 1] - indptr[r], replace=False)) for r in range(n_dst)]).astype(np.int32)
    assert (idx_a[:64] != idx_b[:64]).any() and (idx_a[-64:] != idx_b[-64:]).any()
    vals = rng.random(idx_a.shape[0]).astype("float32")
    x = rng.standard_normal((n_src, F)).astype("float32")
    ref = {k: sp.csr_matrix((vals.astype(np.float64), ix, indptr), shape=(n_dst, n_src)).dot(x.astype(np.float64))
           for k, ix in (("a", idx_a), ("b", idx_b))}
    plan = ctypes.c_void_p()
    _lib.check(L.fg_spmm_plan_create(_lib.host_ptr(indptr), n_dst, n_src, 1, None, ctypes.byref(plan)))
    was = L.fg_debug_checks(0)
    try:
        ip, ix, vl, xd = (torch.from_numpy(a).cuda() for a in (indptr, idx_a, vals, x))
        out = torch.empty((n_dst, F), device="cuda")
        stream = torch.cuda.current_stream().cuda_stream

        def spmm():
            out.fill_(float("nan"))
            _lib.check(L.fg_spmm_csr_f32(plan, _lib.dev_ptr(ip), _lib.dev_ptr(ix), _lib.dev_ptr(vl), _lib.dev_ptr(xd),
                                         _lib.dev_ptr(out), F, 0, stream))
            return out.cpu().numpy().copy()

        _lib.check(L.fg_spmm_plan_narrow_indices(plan, _lib.dev_ptr(ix), stream))
        np.testing.assert_allclose(spmm(), ref["a"], rtol=1e-4, atol=1e-4)
        ix.copy_(torch.from_numpy(idx_b).cuda())                # same address, other ids
        # the debug check notices, the call reads the int32 array and is right; the message says why
        L.fg_debug_checks(1)
        np.testing.assert_allclose(spmm(), ref["b"], rtol=1e-4, atol=1e-4)
        assert b"changed after fg_spmm_plan_narrow_indices" in L.fg_last_error()
        L.fg_debug_checks(0)
        # narrowing again binds the copy to the new contents
        _lib.check(L.fg_spmm_plan_narrow_indices(plan, _lib.dev_ptr(ix), stream))
        narrow_b = spmm()
        np.testing.assert_allclose(narrow_b, ref["b"], rtol=1e-4, atol=1e-4)
        L.fg_debug_checks(1)
        assert np.array_equal(spmm(), narrow_b)                  # fingerprint matches: the copy is used, same bits
        L.fg_debug_checks(0)
        _lib.check(L.fg_spmm_plan_narrow_indices(plan, None, stream))
        assert np.array_equal(spmm(), narrow_b)                  # and the int32 stream gives the same bits
    finally:
        L.fg_debug_checks(was)
        L.fg_spmm_plan_destroy(plan)


def test_ids_outside_the_partition_are_refused():
    """An id that would not survive the cast to 16 bits (or lies outside the partition's width) fails the narrowing
    instead of being truncated."""
    import torch
    from featgraph_amd import _lib
    L = _lib.lib()
    indptr = np.array([0, 2, 3], np.int32)
    plan = ctypes.c_void_p()
    _lib.check(L.fg_spmm_plan_create(_lib.host_ptr(indptr), 2, 1000, 1, None, ctypes.byref(plan)))
    try:
        for bad in (70000, 1000, -1):
            ix = torch.tensor([1, bad, 5], dtype=torch.int32, device="cuda")
            assert L.fg_spmm_plan_narrow_indices(plan, _lib.dev_ptr(ix), None) == -3      # FG_ERR_GRAPH
            assert b"outside [0, 1000)" in L.fg_last_error()
        ix = torch.tensor([1, 999, 5], dtype=torch.int32, device="cuda")
        _lib.check(L.fg_spmm_plan_narrow_indices(plan, _lib.dev_ptr(ix), None))
        assert L.fg_spmm_plan_bytes(plan) >= 3 * 2
    finally:
        L.fg_spmm_plan_destroy(plan)
