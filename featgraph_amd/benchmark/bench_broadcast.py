"""Times the generalised SpMM / SDDMM with broadcasting (GSpMMhip messages, GSDDMMhip operators) on a synthetic
graph or a .npz adjacency.  The reference has no such operators and therefore no benchmark for them; the command
line follows its sweep scripts (benchmark/bench_vanilla_spmm.py:64-79): --dataset / --feat-len, plus --workload.

    python -m featgraph_amd.benchmark.bench_broadcast --workload powerlaw-233k --feat-len 64

One JSON line per operator: time, the algorithmic bytes (index arrays + every operand once + the output once) and
the share of the 8 TB/s HBM peak they amount to.
"""
import argparse
import json

import torch

from ..module import GSpMMhip, GSDDMMhip, placeholder
from .common import load_adjacency, HBM_PEAK_GBS


def _line(op, detail, seconds, nbytes, feat_len):
    print(json.dumps(dict(op=op, detail=detail, feat_len=feat_len, ms=round(seconds * 1e3, 4),
                          algorithmic_gb=round(nbytes / 1e9, 3), algorithmic_gbs=round(nbytes / seconds / 1e9, 1),
                          pct_hbm_roofline=round(100.0 * nbytes / seconds / 1e9 / HBM_PEAK_GBS, 2))), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--dataset", type=str, default=None, help="scipy .npz adjacency (CSR)")
    ap.add_argument("--workload", type=str, default="powerlaw-233k")
    ap.add_argument("--feat-len", type=int, default=64)
    ap.add_argument("--num-runs", type=int, default=5)
    args = ap.parse_args()
    adj = load_adjacency(args, 'csr')
    n_dst, n_src = adj.shape
    nnz, F = adj.nnz, args.feat_len
    x = torch.randn((n_src, F), device="cuda")
    y = torch.randn((n_dst, F), device="cuda")
    ef = torch.randn((nnz, F), device="cuda")
    w = torch.rand((nnz, 1), device="cuda") + 0.5
    index_bytes = 4 * (n_dst + 1) + 4 * nnz

    def nbytes(arrays, out):
        return index_bytes + sum(a.numel() * 4 for a in arrays) + out.numel() * 4

    for msg, arrays in (("u_mul_e", [x, ef]), ("u_add_e", [x, w]), ("copy_e", [ef])):
        for reduce in ("sum", "max"):
            m = GSpMMhip(adj)
            m.build([placeholder(a.shape) for a in arrays], {'msg': msg, 'reduce': reduce}, {})
            t = m.measure_average_time(arrays, args.num_runs)
            _line("gspmm", "%s / %s, operands %s" % (msg, reduce, [tuple(a.shape[1:]) for a in arrays]), t,
                  nbytes(arrays, m.out_tvm), F)
            del m
    coo = adj.tocoo()
    cases = (("add", {}, [x, y]), ("div", {}, [x, y]), ("mul", {'lhs_target': 'e'}, [ef, y]),
             ("mul", {'lhs_target': 'e', 'rhs_target': 'e'}, [w, ef]))
    for op, targets, arrays in cases:
        m = GSDDMMhip(coo)
        m.build([placeholder(a.shape) for a in arrays], dict(targets, op=op), {})
        t = m.measure_average_time(arrays, args.num_runs)
        _line("gsddmm", "%s(%s, %s), operands %s" % (op, targets.get('lhs_target', 'u'), targets.get('rhs_target', 'v'),
                                                     [tuple(a.shape[1:]) for a in arrays]), t,
              4 * nnz + nbytes(arrays, m.out_tvm), F)
        del m


if __name__ == "__main__":
    main()
