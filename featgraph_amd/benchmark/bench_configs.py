"""Default-configuration timings of every benchmark configuration on one GPU.

    python -m featgraph_amd.benchmark.bench_configs [--quick]

Configurations: weighted CSR SpMM and SDDMM (CSR-ordered and shuffled COO edges) at feature
lengths 32..512 and multi-head SDDMM (H in {4, 8}, D in {32, 64}) on the 232,965-node power-law
graph, plus the other two steps of an attention layer there (edge softmax and its gradient for
H in {1, 4, 8}, per-head weighted SpMM for the same head shapes); SpMM followed by SDDMM at feature
length 128 on the 2.45M-node low-degree graph; SpMM on the 10,000-node uniform graph.  One JSON line per measurement (mean of 5 launches after a warm-up);
the SpMM / SDDMM lines carry `verified`: the output checks of featgraph_amd/benchmark/verify.py on the inputs that were timed.
"""
import argparse
import json

import numpy as np
import scipy.sparse as sp
import torch

from .. import synthetic
from ..module import common
from . import verify as chk
from ..module import (VanillaSpMMhip, VanillaSDDMMhip, MultiHeadSDDMMhip, GSpMMhip, EdgeSoftmaxhip,
                      EdgeSoftmaxSpMMhip, GraphAttentionhip, placeholder)

HBM_PEAK_GBS = 8000.0


def _line(workload, op, knobs, seconds, nnz, feat_len, bytes_model, failures=None):
    out = dict(workload=workload, op=op, **knobs)
    if failures is not None:            # the output of this configuration was checked (featgraph_amd/benchmark/verify.py)
        out["verified"] = not failures
    out.update(ms=round(seconds * 1e3, 4), gflops=round(2.0 * nnz * feat_len / seconds / 1e9, 1),
               compulsory_gb=round(bytes_model / 1e9, 3), compulsory_gbs=round(bytes_model / seconds / 1e9, 1),
               pct_hbm_roofline=round(100.0 * bytes_model / seconds / 1e9 / HBM_PEAK_GBS, 3),
               gathered_tbs=round(4.0 * nnz * feat_len / seconds / 1e12, 2))
    print(json.dumps(out), flush=True)


def _stream_line(workload, op, knobs, seconds, bytes_model):
    """An operator without gathers: bytes that must move / time against the HBM peak."""
    out = dict(workload=workload, op=op, **knobs)
    out.update(ms=round(seconds * 1e3, 4), compulsory_gb=round(bytes_model / 1e9, 3),
               compulsory_gbs=round(bytes_model / seconds / 1e9, 1),
               pct_hbm_roofline=round(100.0 * bytes_model / seconds / 1e9 / HBM_PEAK_GBS, 3))
    print(json.dumps(out), flush=True)


def run_attention_steps(name, adj, softmax_heads, head_shapes):
    n = adj.shape[0]
    nnz = adj.nnz
    gen = torch.Generator(device="cuda")
    sm = EdgeSoftmaxhip(adj)
    for H in softmax_heads:
        gen.manual_seed(4)
        shape = (nnz,) if H == 1 else (nnz, H)
        s = torch.randn(shape, generator=gen, device="cuda")
        sm.build([placeholder(shape)])
        t = sm.measure_average_time([s], 5)
        _stream_line(name, "edge_softmax", {"heads": H}, t, 4 * (n + 1) + 8 * nnz * H)
        a = sm.run([s]).clone()
        t = common.timed_mean_seconds(lambda: sm.backward(a, s), 5)
        _stream_line(name, "edge_softmax_backward", {"heads": H}, t, 4 * (n + 1) + 12 * nnz * H)
        del s, a
    for H, D in head_shapes:
        gen.manual_seed(2)
        x = torch.randn((n, H, D), generator=gen, device="cuda")
        w = torch.rand((nnz, H), generator=gen, device="cuda")
        m = GSpMMhip(adj)
        m.build([placeholder((n, H, D)), placeholder((nnz, H))], {}, {})
        t = m.measure_average_time([x, w], 5)
        _line(name, "spmm_per_head_weights", {"heads": H, "head_len": D, "partitions": m._active['P'],
                                              "tiles": m._num_feat_partitions}, t, nnz, H * D,
              4 * (n + 1) + 4 * nnz + 4 * nnz * H + 8 * n * H * D)
        del m
        # the same aggregation from raw scores, without a stored softmax
        gen.manual_seed(4)
        sc = torch.randn((nnz, H), generator=gen, device="cuda")
        f = EdgeSoftmaxSpMMhip(adj)
        f.build([placeholder((nnz, H)), placeholder((n, H, D))], {}, {})
        t = f.measure_average_time([sc, x], 5)
        _line(name, "edge_softmax_spmm_fused", {"heads": H, "head_len": D, "partitions": f._agg._active['P'],
                                                "tiles": f._agg._num_feat_partitions}, t, nnz, H * D,
              4 * (n + 1) + 4 * nnz + 4 * nnz * H + 8 * n * H * D)
        del f, w, sc
        # scores, softmax and aggregation in one operator (no [nnz, H] array at all)
        gen.manual_seed(5)
        q = torch.randn((n, H, D), generator=gen, device="cuda")
        k = torch.randn((n, H, D), generator=gen, device="cuda")
        g = GraphAttentionhip(adj)
        g.build([placeholder((n, H, D))] * 3, {}, {})
        t = g.measure_average_time([q, k, x], 5)
        # byte model: indices once, Q, K, V and the output once; flops: two gathered operands per edge
        _line(name, "graph_attention", {"heads": H, "head_len": D, "partitions": g._active['P']}, t, nnz, 2 * H * D,
              4 * (n + 1) + 4 * nnz + 16 * n * H * D)
        # the same with the additive scores of GAT layers: only V is gathered
        er = torch.randn((n, H), generator=gen, device="cuda")
        el = torch.randn((n, H), generator=gen, device="cuda")
        g.build([placeholder((n, H)), placeholder((n, H)), placeholder((n, H, D))], {'scores': 'additive'}, {})
        t = g.measure_average_time([er, el, x], 5)
        _line(name, "graph_attention_additive", {"heads": H, "head_len": D, "partitions": g._active['P']}, t, nnz, H * D,
              4 * (n + 1) + 4 * nnz + 8 * n * H + 8 * n * H * D)
        del g, q, k, x, er, el


def run_workload(name, feat_lens, head_shapes, shuffled_coo, softmax_heads=()):
    indptr, indices = synthetic.make_workload(name)
    n = indptr.shape[0] - 1
    nnz = int(indptr[-1])
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1)
    vals = torch.rand(nnz, generator=gen, device="cuda").cpu().numpy()
    adj = sp.csr_matrix((vals, indices, indptr), shape=(n, n))
    vals_d = torch.from_numpy(vals).cuda()
    idx_d = torch.from_numpy(indices).cuda().long()
    rows_d = torch.repeat_interleave(torch.arange(n, device="cuda"), torch.from_numpy(np.diff(indptr)).cuda().long())
    spmm = VanillaSpMMhip(adj)
    sddmm = VanillaSDDMMhip(adj)
    for F in feat_lens:
        gen.manual_seed(2)
        x = torch.randn((n, F), generator=gen, device="cuda")
        y = torch.randn((n, F), generator=gen, device="cuda")
        spmm.build([placeholder((n, F))], {}, {})
        t = spmm.measure_average_time([x], 5)
        _line(name, "spmm", {"feat_len": F, "partitions": spmm._active['P'], "tiles": spmm._num_feat_partitions},
              t, nnz, F, 4 * (n + 1) + 8 * nnz + 8 * n * F, chk.spmm_failures(spmm.run([x]), indptr, idx_d, vals_d, x))
        sddmm.build([placeholder((n, F)), placeholder((n, F))], {}, {})
        t = sddmm.measure_average_time([x, y], 5)
        tiled = (sddmm._tiled[0]['P'], sddmm._tiled[1]) if sddmm._tiled else None
        _line(name, "sddmm_csr_order", {"feat_len": F, "tiled": tiled}, t, nnz, F,
              4 * (n + 1) + 4 * nnz + 8 * n * F + 4 * nnz, chk.sddmm_failures(sddmm.run([x, y]), rows_d, idx_d, x, y))
        del x, y
    for H, D in head_shapes:
        gen.manual_seed(2)
        x = torch.randn((n, H, D), generator=gen, device="cuda")
        y = torch.randn((n, H, D), generator=gen, device="cuda")
        mh = MultiHeadSDDMMhip(adj)
        mh.build([placeholder((n, H, D)), placeholder((n, H, D))], {}, {})
        t = mh.measure_average_time([x, y], 5)
        tiled = (mh._tiled[0]['P'], mh._tiled[1]) if mh._tiled else None
        _line(name, "sddmm_multihead", {"heads": H, "head_len": D, "tiled": tiled}, t, nnz, H * D,
              4 * (n + 1) + 4 * nnz + 8 * n * H * D + 4 * nnz * H, chk.sddmm_failures(mh.run([x, y]), rows_d, idx_d, x, y))
        del mh, x, y
    if softmax_heads:
        run_attention_steps(name, adj, softmax_heads, head_shapes)
    if shuffled_coo:
        coo = adj.tocoo()
        perm = torch.randperm(nnz, generator=torch.Generator().manual_seed(3)).numpy()
        coo = sp.coo_matrix((coo.data[perm], (coo.row[perm], coo.col[perm])), shape=coo.shape)
        perm_d = torch.from_numpy(perm).cuda()
        m = VanillaSDDMMhip(coo)
        for F in shuffled_coo:
            gen.manual_seed(2)
            x = torch.randn((n, F), generator=gen, device="cuda")
            y = torch.randn((n, F), generator=gen, device="cuda")
            for order in ("coo", "auto"):
                m.build([placeholder((n, F)), placeholder((n, F))], {}, {'order': order})
                t = m.measure_average_time([x, y], 5)
                _line(name, "sddmm_shuffled_coo", {"feat_len": F, "order": order}, t, nnz, F, 8 * nnz + 8 * n * F + 4 * nnz,
                      chk.sddmm_failures(m.run([x, y]), rows_d[perm_d], idx_d[perm_d], x, y))
            del x, y


def run_multihead_only(name, H, D, partitions, tiles, runs):
    """One multi-head SDDMM shape on one workload (for profiler runs): a plain device copy of the source operand first
    (the reference point that byte counters are scaled by), then `runs` launches after a warm-up."""
    indptr, indices = synthetic.make_workload(name)
    n = indptr.shape[0] - 1
    nnz = int(indptr[-1])
    adj = sp.csr_matrix((np.ones(nnz, np.float32), indices, indptr), shape=(n, n))
    gen = torch.Generator(device="cuda")
    gen.manual_seed(2)
    x = torch.randn((n, H, D), generator=gen, device="cuda")
    y = torch.randn((n, H, D), generator=gen, device="cuda")
    x_copy = torch.empty_like(x)
    x_copy.copy_(x)
    del x_copy
    mh = MultiHeadSDDMMhip(adj)
    sched = {}
    if partitions:
        sched['num_src_partitions'] = partitions
    if tiles:
        sched['num_feat_tiles'] = tiles
    mh.build([placeholder((n, H, D)), placeholder((n, H, D))], {}, sched)
    t = mh.measure_average_time([x, y], runs)
    tiled = (mh._tiled[0]['P'], mh._tiled[1]) if mh._tiled else None
    _line(name, "sddmm_multihead", {"heads": H, "head_len": D, "tiled": tiled, "copy_bytes": 4 * n * H * D}, t, nnz, H * D,
          4 * (n + 1) + 4 * nnz + 8 * n * H * D + 4 * nnz * H)


if __name__ == '__main__':
    ap = argparse.ArgumentParser()
    ap.add_argument("--quick", action="store_true", help="small graphs only")
    ap.add_argument("--multihead", type=int, nargs=2, metavar=("H", "D"),
                    help="only the multi-head SDDMM of this shape (see --workload, --partitions, --tiles, --runs)")
    ap.add_argument("--workload", default="powerlaw-233k")
    ap.add_argument("--partitions", type=int, default=0, help="source-column partitions (0: the library's choice)")
    ap.add_argument("--tiles", type=int, default=0, help="feature tiles (0: the library's choice)")
    ap.add_argument("--runs", type=int, default=5)
    ap.add_argument("--attention-only", action="store_true",
                    help="only the edge softmax / per-head SpMM steps on the 232,965-node graph")
    args = ap.parse_args()
    if args.multihead:
        run_multihead_only(args.workload, args.multihead[0], args.multihead[1], args.partitions, args.tiles, args.runs)
        raise SystemExit(0)
    if args.attention_only:
        indptr, indices = synthetic.make_workload("powerlaw-233k")
        n = indptr.shape[0] - 1
        adj = sp.csr_matrix((np.ones(int(indptr[-1]), np.float32), indices, indptr), shape=(n, n))
        run_attention_steps("powerlaw-233k", adj, (1, 4, 8), [(4, 64), (8, 64)])
        raise SystemExit(0)
    run_workload("uniform-10k", [32], [], [])
    if args.quick:
        run_workload("powerlaw-23k", [32, 128, 512], [(4, 32), (8, 64)], [128], (1, 4))
    else:
        run_workload("powerlaw-233k", [32, 64, 128, 256, 512], [(4, 32), (4, 64), (8, 32), (8, 64)], [128], (1, 4, 8))
        run_workload("powerlaw-2.45M", [128], [], [])
