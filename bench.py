#!/usr/bin/env python3
"""Benchmark of the SpMM / SDDMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one weighted CSR SpMM followed by one edge-wise SDDMM (edges stored in CSR order), both at
feature length 512 on the seeded 232,965-node / ~114.8M-edge power-law graph, graph and
features resident in HBM, outputs preallocated (the protocol of measure_average_time,
python/featgraph/module/spmm.py:179-186).  Prints ONE JSON line; `value` is
2 * (2 * nnz * F) flops per step over the measured step time.

`roofline` prices the slower of the two operators against the 8 TB/s HBM peak with the
compulsory-traffic byte model (an operator is one C-ABI call; on this graph it is several
launches of one kernel, one per source-column partition, plus a short closing kernel -- the
fix-ups of split rows for SpMM, the sum over feature tiles for SDDMM -- so `achieved` = the
operator's algorithmic bytes / the HIP-event time of all its launches; `kernels` lists them and
`avg_launch_ms` is that time divided by the number of launches of the gather kernel, i.e. it
carries the closing kernel's share as well):
    SpMM  : 4(N+1) + 8 nnz + 4 N F (X once) + 4 N F (out once)
    SDDMM : 4(N+1) + 4 nnz (CSR order; 8 nnz in COO order) + 8 N F + 4 nnz H
`cpu_baseline` times the CPU oracle (a C restatement of the reference's x86 schedules: SpMM
row-parallel, SDDMM serial as in the reference) on a bounded row sample of the same inputs.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# Fabric-side bytes (rocprofv3 FETCH_SIZE x2 + WRITE_SIZE, scaled by the X copy of the same run) moved
# by all launches of the named kernel in one operator call, at the default tiling (the JSON reports
# them per launch as `traffic` and per operator as `op_traffic`); from
# profiles/bench_powerlaw233k_f512_rocprofv3.txt.  Other configurations have no measurement: null.
MEASURED_TRAFFIC = {
    ("spmm", "powerlaw-233k", 512, 8, 8): 72.4e9,      # 8 x spmm_items_kernel + fix-ups (copy: +0.95e9)
    ("sddmm", "powerlaw-233k", 512, 8, 8): 70.9e9,     # 8 x sddmm_tiled_kernel (copy: +0.95e9, tile sum: +4.7e9)
}
METRIC = "SpMM/SDDMM GFLOP/s + achieved HBM GB/s (% roofline), 233k-node graph, feat 512"


def spmm_bytes(n_dst, n_src, nnz, F):
    return 4 * (n_dst + 1) + 8 * nnz + 4 * n_src * F + 4 * n_dst * F


def sddmm_bytes(n, nnz, F, H=1, csr=True):
    idx = 4 * (n + 1) + 4 * nnz if csr else 8 * nnz
    return idx + 8 * n * F + 4 * nnz * H


def cpu_baseline(indptr, indices, vals, x, y, F, budget_s=8.0):
    """Oracle on the host cores over the first rows of the graph (enough rows for roughly
    `budget_s` seconds per op)."""
    import numpy as np
    from oracle import oracle as orc
    threads = orc.max_threads()
    n = indptr.shape[0] - 1

    def rows_for(nnz_target):
        r = int(np.searchsorted(indptr, nnz_target, side="left"))
        return max(1, min(n, r))

    def spmm_on(r):
        ip = indptr[:r + 1]
        e = int(ip[-1])
        t0 = time.perf_counter()
        orc.spmm_csr_x86(ip, indices[:e], vals[:e], x, 1, threads)
        return time.perf_counter() - t0, e

    def sddmm_on(r, parallel):
        e = int(indptr[r])
        rows = np.repeat(np.arange(r, dtype=np.int32), np.diff(indptr[:r + 1]))
        t0 = time.perf_counter()
        orc.sddmm_x86(rows, indices[:e], x, y, 1, parallel, threads)
        return time.perf_counter() - t0, e

    def spmm_variant(r, T, P):
        """Timed SpMM over the first r rows with T feature partitions and P source-column partitions
        (the two knobs the reference's benchmark sweeps, benchmark/bench_vanilla_spmm.py:36-41)."""
        ip = indptr[:r + 1]
        e = int(ip[-1])
        if P == 1:
            t0 = time.perf_counter()
            orc.spmm_csr_x86(ip, indices[:e], vals[:e], x, T, threads)
            return time.perf_counter() - t0
        import scipy.sparse as sp
        sub = sp.csr_matrix((vals[:e], indices[:e], ip), shape=(r, x.shape[0]))
        s1_pos, s1_idx, v = orc.csr_to_dds(sub, P)          # partitioning happens at construction: not timed
        t0 = time.perf_counter()
        orc.spmm_dds_x86(s1_pos, s1_idx, v, x, r, P, T, threads)
        return time.perf_counter() - t0

    # calibrate on ~0.5% of the edges, then size the sample for the budget
    nnz = int(indptr[-1])
    r0 = rows_for(nnz // 200)
    t, e = spmm_on(r0)
    r_spmm = rows_for(min(nnz, int(e * budget_s / 4 / max(t, 1e-6))))
    e_spmm = int(indptr[r_spmm])
    sweep = {(T, P): spmm_variant(r_spmm, T, P) for (T, P) in ((1, 1), (4, 1), (1, 4), (4, 4))}
    best = min(sweep, key=sweep.get)
    t_spmm = sweep[best]
    t, e = sddmm_on(r0, False)
    r_sddmm = rows_for(min(nnz, int(e * budget_s / max(t, 1e-6))))
    t_sddmm, e_sddmm = sddmm_on(r_sddmm, False)
    t_par, e_par = sddmm_on(r_sddmm, True)
    g_spmm = 2.0 * e_spmm * F / t_spmm / 1e9
    g_sddmm = 2.0 * e_sddmm * F / t_sddmm / 1e9
    g_sddmm_par = 2.0 * e_par * F / t_par / 1e9
    # a step runs both ops over the same edges: combined rate = total flops / total time
    combined = 2.0 / (1.0 / g_spmm + 1.0 / g_sddmm)
    return {
        "value": round(combined, 3), "unit": "GFLOP/s", "cores": threads, "kind": "port",
        "sample": "C restatement of the reference x86 schedules (TVM unavailable), F=%d: SpMM row-parallel "
                  "on %d threads over the first %d rows (%d edges), best of (num_feat_partitions, num_col_partitions) "
                  "in {1,4}x{1,4} = %s at %.2f s = %.2f GFLOP/s; SDDMM serial (1 thread, "
                  "as the reference schedule) over the first %d rows (%d edges, %.2f s) = %.2f GFLOP/s; value = "
                  "harmonic combination for one SpMM + one SDDMM over the same edges"
                  % (F, threads, r_spmm, e_spmm, best, t_spmm, g_spmm, r_sddmm, e_sddmm, t_sddmm, g_sddmm),
        "spmm_sweep_seconds": {"T%d_P%d" % k: round(v, 3) for k, v in sweep.items()},
        "spmm_gflops": round(g_spmm, 3), "sddmm_serial_gflops": round(g_sddmm, 3),
        "sddmm_edge_parallel_variant_gflops": round(g_sddmm_par, 3),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="powerlaw-233k")
    ap.add_argument("--feat-len", type=int, default=512)
    ap.add_argument("--num-feat-partitions", type=int, default=0, help="SpMM feature tiles (0 = library default)")
    ap.add_argument("--num-col-partitions", type=int, default=1, help="SpMM source-column partitions")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: both ops are single-device kernels with no collective; "
                 "--gpus %d is not supported (row-sharding across GPUs is design-only)" % args.gpus)

    import numpy as np
    import scipy.sparse as sp
    import torch
    from featgraph_amd import synthetic
    from featgraph_amd.module import VanillaSpMMhip, VanillaSDDMMhip, placeholder

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a ROCm GPU")
    torch.cuda.set_device(0)
    F = args.feat_len
    indptr, indices = synthetic.make_workload(args.workload)
    n = indptr.shape[0] - 1
    nnz = int(indptr[-1])
    deg = np.diff(indptr)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1)
    vals_d = torch.rand(nnz, generator=gen, device="cuda", dtype=torch.float32)       # U[0,1)
    gen.manual_seed(2)
    x_d = torch.randn((n, F), generator=gen, device="cuda", dtype=torch.float32)      # N(0,1)
    y_d = torch.randn((n, F), generator=gen, device="cuda", dtype=torch.float32)
    vals = vals_d.cpu().numpy()
    adj = sp.csr_matrix((vals, indices, indptr), shape=(n, n))

    spmm = VanillaSpMMhip(adj, args.num_col_partitions)
    spmm.build([placeholder((n, F))], {'num_feat_partitions': args.num_feat_partitions}, {})
    sddmm = VanillaSDDMMhip(adj)
    sddmm.build([placeholder((n, F)), placeholder((n, F))], {}, {})
    del adj

    def step(ev=None):
        if ev is not None:
            ev[0].record()
        spmm.run([x_d])
        if ev is not None:
            ev[1].record()
        sddmm.run([x_d, y_d])
        if ev is not None:
            ev[2].record()

    # One plain device copy of X (reads and writes n*F*4 bytes each): the reference point that
    # rocprofv3's FETCH_SIZE / WRITE_SIZE counters of the kernels are scaled by.
    x_copy = torch.empty_like(x_d)
    x_copy.copy_(x_d)
    del x_copy

    for _ in range(args.warmup):
        step()
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        step(evs[k])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    t_spmm = sum(e[0].elapsed_time(e[1]) for e in evs) / args.steps      # ms, HIP events on the launch stream
    t_sddmm = sum(e[1].elapsed_time(e[2]) for e in evs) / args.steps

    def sddmm_launches():
        """Launches of the tiled kernel: with T < 8 tiles, 8 / T partitions share a launch."""
        if not sddmm._tiled:
            return 1
        P, T = sddmm._tiled[0]['P'], sddmm._tiled[1]
        conc = min(8 // T, P) if (T < 8 and 8 % T == 0) else 1
        return (P + conc - 1) // conc

    def copies(n_tiles):
        """Launches of the kernel that makes the tile-by-tile copy of the gathered operand (the library's
        default rule: 4 or more feature tiles, 64 MB or more, 32-bit offsets)."""
        return 1 if (n_tiles >= 4 and (64 << 20) <= 4 * n * F < (1 << 32)) else 0

    flops_op = 2.0 * nnz * F
    b_spmm = spmm_bytes(n, n, nnz, F)
    b_sddmm = sddmm_bytes(n, nnz, F, 1, csr=True)
    ops = {
        "spmm": {"ms": t_spmm, "gflops": flops_op / t_spmm / 1e6, "compulsory_gb": b_spmm / 1e9,
                 "hbm_gbs": b_spmm / t_spmm / 1e6, "gathered_gbs": 4.0 * nnz * F / t_spmm / 1e6,
                 "kernel": "spmm_items_kernel", "launches": spmm._active['P'],
                 "kernels": {"tile_major_kernel": copies(spmm._num_feat_partitions or 1),
                             "spmm_items_kernel": spmm._active['P'], "spmm_fixup_kernel": spmm._active['P']},
                 "num_col_partitions": spmm._active['P'], "num_feat_partitions": spmm._num_feat_partitions},
        "sddmm": {"ms": t_sddmm, "gflops": flops_op / t_sddmm / 1e6, "compulsory_gb": b_sddmm / 1e9,
                  "hbm_gbs": b_sddmm / t_sddmm / 1e6, "gathered_gbs": 4.0 * nnz * F / t_sddmm / 1e6,
                  "kernel": "sddmm_tiled_kernel" if sddmm._tiled else "sddmm_csr_kernel",
                  "launches": sddmm_launches(),
                  "kernels": ({"tile_major_kernel": copies(sddmm._tiled[1]), "sddmm_tiled_kernel": sddmm_launches(),
                               "sddmm_tile_sum_kernel": 1}
                              if sddmm._tiled else {"sddmm_csr_kernel": 1}),
                  "num_src_partitions": sddmm._tiled[0]['P'] if sddmm._tiled else 1,
                  "num_feat_tiles": sddmm._tiled[1] if sddmm._tiled else 1},
    }
    for o in ops.values():
        o["pct_hbm_roofline"] = 100.0 * o["hbm_gbs"] / HBM_PEAK_GBS
    dom = "spmm" if t_spmm >= t_sddmm else "sddmm"
    key = (dom, args.workload, F, ops[dom].get("num_col_partitions", ops[dom].get("num_src_partitions")),
           ops[dom].get("num_feat_partitions", ops[dom].get("num_feat_tiles")))
    op_traffic = MEASURED_TRAFFIC.get(key)
    n_launch = ops[dom]["launches"]
    b_dom = b_spmm if dom == "spmm" else b_sddmm
    # per launch of the gather kernel: algorithmic bytes / launches over op time / launches -- the same
    # ratio as for the whole operator; `traffic` is the measured fabric-side bytes of one such launch
    roofline = {"bound": "hbm", "kernel": ops[dom]["kernel"], "achieved": round(ops[dom]["hbm_gbs"], 2),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(ops[dom]["hbm_gbs"] / HBM_PEAK_GBS, 5),
                "traffic": (round(op_traffic / n_launch) if op_traffic else None), "op_traffic": op_traffic,
                "algorithmic_bytes_per_launch": int(b_dom / n_launch), "algorithmic_bytes": int(b_dom),
                "launches": ops[dom]["launches"], "kernels": ops[dom]["kernels"], "op_ms": round(ops[dom]["ms"], 4),
                "avg_launch_ms": round(ops[dom]["ms"] / ops[dom]["launches"], 4)}

    line = {
        "metric": METRIC, "value": round(2 * flops_op / (ms_per_step * 1e6), 2), "unit": "GFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "%s: weighted CSR SpMM + SDDMM over the same edges, F=%d, fp32, int32 indices" % (args.workload, F),
                   "nodes": n, "edges": nnz, "max_in_degree": int(deg.max()), "median_in_degree": float(np.median(deg)),
                   "feat_len": F, "num_feat_partitions": args.num_feat_partitions,
                   "num_col_partitions": args.num_col_partitions, "seeds": {"graph": 0xFEA7, "weights": 1, "features": 2}},
        "roofline": roofline,
        "ops": {k: {kk: (round(vv, 4) if isinstance(vv, float) else vv) for kk, vv in v.items()} for k, v in ops.items()},
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(indptr, indices, vals, x_d.cpu().numpy(), y_d.cpu().numpy(), F)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
