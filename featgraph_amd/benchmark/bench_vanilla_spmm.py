"""Sweep of the SpMM knobs on one graph, the counterpart of the reference's
benchmark/bench_vanilla_spmm.py (:18-41 x86 sweep, :44-68 CUDA sweep).

    python -m featgraph_amd.benchmark.bench_vanilla_spmm --workload powerlaw-233k --feat-len 128
    python -m featgraph_amd.benchmark.bench_vanilla_spmm --dataset data/reddit_csr_float32.npz

Sweeps num_col_partitions x num_feat_partitions like the reference's x86 loop
(exp_range(1, 32, 2) x exp_range(1, feat_len // 16, 2)); both are carried out on the GPU.
Prints one JSON line per point: mean of 5 runs, GFLOP/s, compulsory-model GB/s and % of 8 TB/s.
"""
import argparse

import torch

from ..module import VanillaSpMMhip, placeholder
from .common import exp_range, load_adjacency, report


def bench_vanilla_spmm(adj_scipy_csr, feat_len, max_col_partitions=32, num_runs=5, src_feat=None, collect=None):
    """Times every sweep point.  src_feat: the source features to use (default: U[0,1) like the
    reference's np.random.random, bench_vanilla_spmm.py:29); collect: a list that receives
    (knobs, seconds, output as a numpy array) per point, for callers that check the results."""
    num_rows, num_cols = adj_scipy_csr.shape
    nnz = adj_scipy_csr.nnz
    if src_feat is None:
        src_feat = torch.rand((num_cols, feat_len), device="cuda", dtype=torch.float32)
    bytes_model = 4 * (num_rows + 1) + 8 * nnz + 4 * num_cols * feat_len + 4 * num_rows * feat_len

    def run(module, knobs, compute_args, schedule_args):
        module.build([placeholder((num_cols, feat_len))], compute_args, schedule_args)
        tcost = module.measure_average_time([src_feat], num_runs)
        report("spmm", knobs, tcost, nnz, feat_len, bytes_model)
        if collect is not None:
            collect.append((knobs, tcost, module.run([src_feat]).cpu().numpy().copy()))

    module = VanillaSpMMhip(adj_scipy_csr)
    run(module, {"num_col_partitions": "auto", "num_feat_partitions": "auto"}, {}, {})
    for num_col_partitions in exp_range(1, max_col_partitions, 2):
        module = VanillaSpMMhip(adj_scipy_csr, num_col_partitions)
        for num_feat_partitions in exp_range(1, max(1, feat_len // 16), 2):
            if feat_len % num_feat_partitions:
                continue
            run(module, {"num_col_partitions": num_col_partitions, "num_feat_partitions": num_feat_partitions},
                {'num_feat_partitions': num_feat_partitions}, {'num_src_partitions': None})
        del module


if __name__ == '__main__':
    parser = argparse.ArgumentParser()
    parser.add_argument("--dataset", type=str, help="The adjacency matrix in csr format stored as a scipy npz file")
    parser.add_argument("--workload", type=str, default="powerlaw-23k", help="Seeded synthetic graph when no --dataset")
    parser.add_argument("--feat-len", type=int, default=128, help="The feature length")
    parser.add_argument("--max-col-partitions", type=int, default=32)
    args = parser.parse_args()
    bench_vanilla_spmm(load_adjacency(args, 'csr'), args.feat_len, args.max_col_partitions)
