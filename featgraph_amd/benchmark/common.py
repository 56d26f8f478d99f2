"""Shared pieces of the sweep scripts: dataset loading and result lines."""
import json

import numpy as np
import scipy.sparse

from .. import synthetic

HBM_PEAK_GBS = 8000.0


def exp_range(start, end, mul):
    while start <= end:
        yield start
        start *= mul


def load_adjacency(args, fmt):
    """--dataset: a scipy .npz file as written by the reference's
    benchmark/download_reddit_dataset.py:11-17; otherwise --workload: a seeded synthetic graph."""
    if args.dataset:
        adj = scipy.sparse.load_npz(args.dataset)
        assert adj.format == fmt, "expected a %s matrix in %s" % (fmt, args.dataset)
        return adj.astype(np.float32)
    indptr, indices = synthetic.make_workload(args.workload)
    n = indptr.shape[0] - 1
    n_src = synthetic.WORKLOADS[args.workload]["n"]
    vals = synthetic.edge_weights(indices.shape[0], 1) if indices.shape[0] < 5_000_000 else None
    if vals is None:
        import torch
        g = torch.Generator(device="cuda")
        g.manual_seed(1)
        vals = torch.rand(indices.shape[0], generator=g, device="cuda").cpu().numpy()
    adj = scipy.sparse.csr_matrix((vals, indices, indptr), shape=(n, n_src))
    return adj if fmt == 'csr' else adj.tocoo()


def report(op, knobs, seconds, nnz, feat_len, bytes_model):
    line = dict(op=op, **knobs)
    line.update(ms=round(seconds * 1e3, 4), gflops=round(2.0 * nnz * feat_len / seconds / 1e9, 1),
                compulsory_gbs=round(bytes_model / seconds / 1e9, 1),
                pct_hbm_roofline=round(100.0 * bytes_model / seconds / 1e9 / HBM_PEAK_GBS, 3),
                gathered_tbs=round(4.0 * nnz * feat_len / seconds / 1e12, 2))
    print(json.dumps(line), flush=True)
