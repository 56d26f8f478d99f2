"""Sweep of the SDDMM knobs on one graph, the counterpart of the reference's
benchmark/bench_vanilla_sddmm.py (:18-46 x86 sweep, :49-74 CUDA sweep).

    python -m featgraph_amd.benchmark.bench_vanilla_sddmm --workload powerlaw-233k --feat-len 128
    python -m featgraph_amd.benchmark.bench_vanilla_sddmm --dataset data/reddit_coo_float32.npz

Points: the stored-order kernels, the 2-D partitioned stored orders of the reference's x86 loop
(num_row_partitions x num_col_partitions), and the internal tiled traversal
(num_src_partitions x num_feat_tiles).  One JSON line per point.
"""
import argparse

import torch

from ..module import VanillaSDDMMhip, placeholder
from .common import exp_range, load_adjacency, report


def bench_vanilla_sddmm(adj_scipy_coo, feat_len, max_partitions=8, num_runs=5, src_feat=None, dst_feat=None,
                        collect=None):
    """Times every sweep point.  src_feat / dst_feat: the features to use (default: U[0,1) like the
    reference, bench_vanilla_sddmm.py:31-32); collect: a list that receives (knobs, seconds, output in
    the ORIGINAL stored edge order as a numpy array) per point, for callers that check the results."""
    num_rows, num_cols = adj_scipy_coo.shape
    nnz = adj_scipy_coo.nnz
    if src_feat is None:
        src_feat = torch.rand((num_cols, feat_len), device="cuda", dtype=torch.float32)
    if dst_feat is None:
        dst_feat = torch.rand((num_rows, feat_len), device="cuda", dtype=torch.float32)
    bytes_model = 8 * nnz + 4 * (num_rows + num_cols) * feat_len + 4 * nnz
    phs = [placeholder((num_cols, feat_len)), placeholder((num_rows, feat_len))]

    def run(module, knobs, schedule_args):
        try:
            module.build(phs, {}, schedule_args)
            tcost = module.measure_average_time([src_feat, dst_feat], num_runs)
        except ValueError as e:          # a tile shape the tiled kernel does not take
            print("# skipped %s: %s" % (knobs, e))
            return
        report("sddmm", knobs, tcost, nnz, feat_len, bytes_model)
        if collect is not None:
            out = module.run([src_feat, dst_feat]).cpu().numpy().copy()
            if module._edge_mapping is not None:
                out = out[module.edge_mapping]
            collect.append((knobs, tcost, out))

    module = VanillaSDDMMhip(adj_scipy_coo)
    run(module, {"order": "auto"}, {})
    run(module, {"order": "coo"}, {'order': 'coo'})
    if module._row_sorted:
        run(module, {"order": "csr"}, {'order': 'csr'})
    for p in exp_range(1, 32, 2):
        for t in exp_range(1, max(1, feat_len // 16), 2):
            run(module, {"order": "tiled", "num_src_partitions": p, "num_feat_tiles": t},
                {'order': 'tiled', 'num_src_partitions': p, 'num_feat_tiles': t})
    del module
    for r in exp_range(2, max_partitions, 2):
        for c in exp_range(2, max_partitions, 2):
            module = VanillaSDDMMhip(adj_scipy_coo, r, c)
            run(module, {"num_row_partitions": r, "num_col_partitions": c, "order": "coo"}, {'order': 'coo'})
            del module


if __name__ == '__main__':
    parser = argparse.ArgumentParser()
    parser.add_argument("--dataset", type=str, help="The adjacency matrix in coo format stored as a scipy npz file")
    parser.add_argument("--workload", type=str, default="powerlaw-23k", help="Seeded synthetic graph when no --dataset")
    parser.add_argument("--feat-len", type=int, default=128, help="The feature length")
    parser.add_argument("--max-partitions", type=int, default=8)
    args = parser.parse_args()
    bench_vanilla_sddmm(load_adjacency(args, 'coo'), args.feat_len, args.max_partitions)
