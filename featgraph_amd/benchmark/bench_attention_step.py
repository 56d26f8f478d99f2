"""One attention layer, forward and backward, through the autograd layer.

Default: Graph.attention, one operator forward (no stored scores) and two sweeps backward (one over the
adjacency for dQ, one over its transpose for dK and dV).  With --chain: scores = SDDMM(K, Q) per head, softmax
over each destination's edges, out = per-head weighted SpMM of V, whose backward pass is three per-head SpMMs
(two of them on the transposed graph), one multi-head SDDMM and the softmax gradient.

    python -m featgraph_amd.benchmark.bench_attention_step [--workload powerlaw-233k] [--heads 8] [--head-len 64] [--chain | --additive]

Prints one JSON line with the mean times (HIP events on the launch stream) of the steps after the first."""
import argparse
import json

import numpy as np
import scipy.sparse as sp
import torch

from .. import synthetic
from ..autograd import Graph


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="powerlaw-233k", choices=sorted(synthetic.WORKLOADS))
    ap.add_argument("--heads", type=int, default=8)
    ap.add_argument("--head-len", type=int, default=64)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--chain", action="store_true", help="the three operators instead of the single one")
    ap.add_argument("--additive", action="store_true",
                    help="the additive scores of a GAT layer, leaky_relu(el[col] + er[row]), instead of dot products")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("bench_attention_step needs a GPU")
    indptr, indices = synthetic.make_workload(args.workload)
    n, nnz = indptr.shape[0] - 1, int(indptr[-1])
    g = Graph(sp.csr_matrix((np.ones(nnz, np.float32), indices, indptr), shape=(n, n)))
    H, D = args.heads, args.head_len
    gen = torch.Generator(device="cuda"); gen.manual_seed(2)
    q, k, v = (torch.randn((n, H, D), generator=gen, device="cuda").requires_grad_() for _ in range(3))
    er, el = (torch.randn((n, H), generator=gen, device="cuda").requires_grad_() for _ in range(2))
    if args.additive and args.chain:
        raise SystemExit("--additive times the single operator only")

    def mark():
        e = torch.cuda.Event(enable_timing=True)
        e.record()
        return e

    times = []
    for step in range(args.steps + 1):
        e = [mark()]
        if args.chain:
            s = g.sddmm(k, q); e.append(mark())
            a = g.edge_softmax(s * (1.0 / D ** 0.5)); e.append(mark())
            out = g.spmm(v, a); e.append(mark())
        else:
            e += [e[0], e[0]]
            out = g.gat_attention(er, el, v) if args.additive else g.attention(q, k, v); e.append(mark())
        loss = out.square().mean()
        loss.backward(); e.append(mark())
        torch.cuda.synchronize()
        if step > 0:                      # the first step builds the modules and allocates
            times.append([e[i].elapsed_time(e[i + 1]) for i in range(4)])
        q.grad = k.grad = v.grad = er.grad = el.grad = None
    t = np.mean(np.array(times), axis=0)
    line = {"workload": args.workload, "nodes": n, "edges": nnz, "heads": H, "head_len": D,
            "operators": "sddmm + edge_softmax + spmm" if args.chain else ("gat_attention" if args.additive else "attention")}
    if args.chain:
        line.update(sddmm_ms=round(float(t[0]), 3), edge_softmax_ms=round(float(t[1]), 3), spmm_ms=round(float(t[2]), 3))
    else:
        line.update(attention_ms=round(float(t[2]), 3))
    line.update(loss_and_backward_ms=round(float(t[3]), 3), step_ms=round(float(t.sum()), 3), steps=args.steps)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
