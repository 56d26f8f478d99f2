"""Status codes and messages of the device entry points of the C ABI, called directly through ctypes
with raw device pointers (no module layer): bad arguments must come back as negative codes with a
message, never as a launch."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

FG_OK, FG_ERR_ARG, FG_ERR_SHAPE, FG_ERR_GRAPH = 0, -1, -2, -3


@pytest.fixture(scope="module")
def env():
    import torch
    from featgraph_amd import _lib
    L = _lib.lib()
    indptr = np.array([0, 2, 2, 5, 6], dtype=np.int32)
    indices = np.array([0, 3, 1, 2, 4, 0], dtype=np.int32)
    plan = ctypes.c_void_p()
    assert L.fg_spmm_plan_create(_lib.host_ptr(indptr), 4, 5, 1, None, ctypes.byref(plan)) == FG_OK
    s1_pos = np.array([0, 1, 1, 2, 3, 3, 4, 4, 6, 6], dtype=np.int32)        # P = 2 over the same matrix
    plan2 = ctypes.c_void_p()
    assert L.fg_spmm_plan_create(_lib.host_ptr(s1_pos), 4, 5, 2, None, ctypes.byref(plan2)) == FG_OK
    dev = lambda a: torch.from_numpy(a).cuda()
    t = dict(indptr=dev(indptr), indices=dev(indices), vals=torch.ones(6, device="cuda"),
             x=torch.ones((5, 8), device="cuda"), y=torch.ones((4, 8), device="cuda"),
             out=torch.zeros((4, 8), device="cuda"), e=torch.zeros(6, device="cuda"))
    yield L, _lib, plan, plan2, t
    L.fg_spmm_plan_destroy(plan)
    L.fg_spmm_plan_destroy(plan2)


def test_spmm_arguments(env):
    L, lib, plan, plan2, t = env
    p = lib.dev_ptr
    ok = L.fg_spmm_csr_f32(plan, p(t['indptr']), p(t['indices']), p(t['vals']), p(t['x']), p(t['out']), 8, 0, None)
    assert ok == FG_OK
    assert L.fg_spmm_csr_f32(None, p(t['indptr']), p(t['indices']), p(t['vals']), p(t['x']), p(t['out']), 8, 0, None) == FG_ERR_ARG
    assert b"plan" in L.fg_last_error()
    assert L.fg_spmm_csr_f32(plan, p(t['indptr']), None, p(t['vals']), p(t['x']), p(t['out']), 8, 0, None) == FG_ERR_ARG
    assert L.fg_spmm_csr_f32(plan, p(t['indptr']), p(t['indices']), p(t['vals']), p(t['x']), p(t['out']), 0, 0, None) == FG_ERR_SHAPE
    assert L.fg_spmm_csr_f32(plan, p(t['indptr']), p(t['indices']), p(t['vals']), p(t['x']), p(t['out']), 8, 3, None) == FG_ERR_SHAPE
    assert b"divisible" in L.fg_last_error()
    # a plan with column partitions does not fit the CSR entry point
    assert L.fg_spmm_csr_f32(plan2, p(t['indptr']), p(t['indices']), p(t['vals']), p(t['x']), p(t['out']), 8, 0, None) == FG_ERR_ARG
    # max / min aggregation needs one partition; unknown reduce
    assert L.fg_gspmm_f32(plan2, p(t['indptr']), p(t['indices']), p(t['vals']), p(t['x']), p(t['out']), 8, 1, 0, 1, 0, None) == FG_ERR_ARG
    assert L.fg_gspmm_f32(plan, p(t['indptr']), p(t['indices']), p(t['vals']), p(t['x']), p(t['out']), 8, 1, 0, 7, 0, None) == FG_ERR_ARG
    assert L.fg_gspmm_f32(plan, p(t['indptr']), p(t['indices']), p(t['vals']), p(t['x']), p(t['out']), 8, 3, 0, 0, 0, None) == FG_ERR_SHAPE


def test_sddmm_and_softmax_arguments(env):
    L, lib, plan, plan2, t = env
    p = lib.dev_ptr
    assert L.fg_sddmm_csr_f32(plan, p(t['indptr']), p(t['indices']), p(t['x']), p(t['y']), p(t['e']), 1, 8, None) == FG_OK
    assert L.fg_sddmm_csr_f32(plan, p(t['indptr']), p(t['indices']), None, p(t['y']), p(t['e']), 1, 8, None) == FG_ERR_ARG
    assert L.fg_sddmm_csr_f32(plan, p(t['indptr']), p(t['indices']), p(t['x']), p(t['y']), p(t['e']), 0, 8, None) == FG_ERR_SHAPE
    assert L.fg_sddmm_coo_f32(None, p(t['indices']), 6, p(t['x']), p(t['y']), p(t['e']), 1, 8, None) == FG_ERR_ARG
    assert L.fg_sddmm_coo_f32(p(t['indices']), p(t['indices']), -1, p(t['x']), p(t['y']), p(t['e']), 1, 8, None) == FG_ERR_ARG
    # tiled traversal: a tile must be a power of two between 16 and 256 floats
    assert L.fg_sddmm_dds_f32(plan, p(t['indptr']), p(t['indices']), p(t['indices']), p(t['x']), p(t['y']), p(t['e']),
                              1, 8, 1, None) == FG_ERR_SHAPE
    assert L.fg_edge_softmax_f32(plan, p(t['indptr']), p(t['e']), p(t['e']), 1, None) == FG_OK
    assert L.fg_edge_softmax_f32(plan, p(t['indptr']), p(t['e']), p(t['e']), 0, None) == FG_ERR_SHAPE
    assert L.fg_edge_softmax_f32(plan2, p(t['indptr']), p(t['e']), p(t['e']), 1, None) == FG_ERR_ARG
    assert L.fg_edge_softmax_f32(plan, p(t['indptr']), None, p(t['e']), 1, None) == FG_ERR_ARG
    assert L.fg_edge_softmax_backward_f32(plan, p(t['indptr']), p(t['e']), None, p(t['e']), 1, None) == FG_ERR_ARG
    assert L.fg_edge_values_head_major_f32(p(t['e']), None, 6, 0, p(t['e']), None) == FG_ERR_ARG
    assert L.fg_gsddmm_elementwise_f32(p(t['indices']), p(t['indices']), 6, p(t['x']), p(t['y']), p(t['out']), 8, 9, None) == FG_ERR_ARG


def test_plan_rejects_bad_positions(env):
    L, lib, plan, plan2, t = env
    bad = ctypes.c_void_p()
    dec = np.array([0, 3, 2, 5], dtype=np.int32)
    assert L.fg_spmm_plan_create(lib.host_ptr(dec), 3, 4, 1, None, ctypes.byref(bad)) == FG_ERR_GRAPH
    assert not bad.value
    assert L.fg_spmm_plan_create(lib.host_ptr(dec), 3, 4, 0, None, ctypes.byref(bad)) == FG_ERR_ARG
    assert L.fg_spmm_plan_create(None, 3, 4, 1, None, ctypes.byref(bad)) == FG_ERR_ARG


def test_broadcasting_entry_points(env):
    """fg_gspmm_bcast_f32 / fg_gsddmm_bcast_f32 called directly: a correct call, then every refusal."""
    import torch
    L, lib, plan, plan2, t = env
    p = lib.dev_ptr
    U, E, V = 0, 1, 2
    ADD, MUL, COPY_LHS, DOT = 0, 2, 4, 6
    SUM, MAX = 0, 1
    ef = torch.full((6, 8), 2.0, device="cuda")
    out = torch.zeros((4, 8), device="cuda")
    arg = torch.zeros((4, 8), dtype=torch.int32, device="cuda")

    def spmm(pl=plan, op=MUL, red=SUM, lhs=t['x'], lt=U, ll=8, loff=None, rhs=ef, rt=E, rl=8, roff=None, flags=0, o=out, a=None, n=8):
        return L.fg_gspmm_bcast_f32(pl, p(t['indptr']), p(t['indices']), op, red, p(lhs), lt, ll, p(loff), p(rhs), rt, rl, p(roff),
                                    flags, None, p(o), p(a), n, None)

    assert spmm() == FG_OK
    torch.cuda.synchronize()
    deg = torch.tensor([2., 0., 3., 1.], device="cuda")
    assert torch.equal(out, (2 * deg)[:, None].expand(4, 8))          # x = 1, edge features = 2
    assert spmm(red=MAX, a=arg) == FG_OK
    torch.cuda.synchronize()
    assert arg[:, 0].tolist() == [0, -1, 2, 5]                        # first element of every row, -1 for the empty one
    assert spmm(pl=None) == FG_ERR_ARG
    assert spmm(pl=plan2) == FG_ERR_ARG and b"one column partition" in L.fg_last_error()
    assert spmm(op=DOT) == FG_ERR_ARG
    assert spmm(red=5) == FG_ERR_ARG
    assert spmm(a=arg) == FG_ERR_ARG                                  # positions exist for max / min only
    assert spmm(lhs=None) == FG_ERR_ARG and b"lhs" in L.fg_last_error()
    assert spmm(lt=V) == FG_ERR_ARG                                   # destination-node operands: SDDMM only
    assert spmm(ll=4) == FG_ERR_SHAPE                                 # no offset array: the length must be the output's
    assert spmm(n=0) == FG_ERR_SHAPE
    assert spmm(o=None) == FG_ERR_ARG
    assert spmm(op=COPY_LHS, rhs=None, rl=0) == FG_OK                 # the unused operand may be absent

    # the same matrix in two source-column partitions (columns 0-2 and 3-4): fg_gspmm_bcast_dds_f32
    s1_pos = np.array([0, 1, 1, 3, 4, 4, 5, 5, 6, 6], dtype=np.int32)
    s1_idx = torch.tensor([0, 1, 2, 0, 0, 1], dtype=torch.int32, device="cuda")
    edge_pos = torch.tensor([0, 2, 3, 5, 1, 4], dtype=torch.int32, device="cuda")
    plan_dds = ctypes.c_void_p()
    assert L.fg_spmm_plan_create(lib.host_ptr(s1_pos), 4, 5, 2, None, ctypes.byref(plan_dds)) == FG_OK
    pos_dev = torch.from_numpy(s1_pos).cuda()
    ramp = torch.arange(6, dtype=torch.float32, device="cuda")[:, None].expand(6, 8).contiguous()      # edge e holds e

    def dds(pl=plan_dds, red=SUM, ep=edge_pos, a=None, op=COPY_LHS, pos=pos_dev, idx=s1_idx):
        return L.fg_gspmm_bcast_dds_f32(pl, p(pos), p(idx), p(ep), op, red, p(ramp), E, 8, None, None, E, 0, None,
                                        0, None, p(out), p(a), 8, None)

    assert dds() == FG_OK
    torch.cuda.synchronize()
    assert out[:, 0].tolist() == [1.0, 0.0, 9.0, 5.0]                 # sums of the rows' CSR positions: 0+1, -, 2+3+4, 5
    assert dds(red=MAX, a=arg) == FG_OK
    torch.cuda.synchronize()
    assert out[:, 3].tolist() == [1.0, 0.0, 4.0, 5.0] and arg[:, 3].tolist() == [1, -1, 4, 5]     # positions in CSR order
    assert dds(ep=None) == FG_ERR_ARG                                 # several partitions need the stored positions
    assert dds(pl=None) == FG_ERR_ARG
    assert dds(pl=plan, ep=None, pos=t['indptr'], idx=t['indices']) == FG_OK      # one partition: the CSR arrays themselves
    torch.cuda.synchronize()
    assert out[:, 0].tolist() == [1.0, 0.0, 9.0, 5.0]
    L.fg_spmm_plan_destroy(plan_dds)

    row = torch.tensor([0, 0, 2, 2, 2, 3], dtype=torch.int32, device="cuda")
    eo = torch.zeros((6, 8), device="cuda")

    def sddmm(r=row, c=t['indices'], n_edges=6, op=ADD, lhs=t['x'], lt=U, ll=8, rhs=t['y'], rt=V, rl=8, o=eo, n=8, red_len=1):
        return L.fg_gsddmm_bcast_f32(p(r), p(c), n_edges, op, p(lhs), lt, ll, None, p(rhs), rt, rl, None, 0, p(o), n, red_len, None)

    assert sddmm() == FG_OK
    torch.cuda.synchronize()
    assert torch.equal(eo, torch.full((6, 8), 2.0, device="cuda"))
    assert sddmm(op=9) == FG_ERR_ARG
    assert sddmm(n_edges=-1) == FG_ERR_ARG
    assert sddmm(lhs=None) == FG_ERR_ARG
    assert sddmm(c=None) == FG_ERR_ARG                                # an operand on u needs the column ids
    assert sddmm(r=None) == FG_ERR_ARG
    assert sddmm(ll=4) == FG_ERR_SHAPE
    assert sddmm(op=DOT, n=2, red_len=3) == FG_ERR_SHAPE              # 8 is not a multiple of the contracted length
    assert sddmm(op=DOT, n=2, red_len=4, o=eo) == FG_OK
    assert sddmm(n_edges=0, lhs=None, rhs=None) == FG_OK              # nothing to read, nothing refused
