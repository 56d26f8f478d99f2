#!/usr/bin/env python3
"""Benchmark of the SpMM / SDDMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one weighted CSR SpMM followed by one edge-wise SDDMM (edges stored in CSR order), both at
feature length 512 on the seeded 232,965-node / ~114.8M-edge power-law graph, graph and
features resident in HBM, outputs preallocated (the protocol of measure_average_time,
python/featgraph/module/spmm.py:179-186).  Prints ONE JSON line; `value` is
2 * (2 * nnz * F) flops per step over the measured step time.

`roofline` prices the slower of the two operators against the 8 TB/s HBM peak with the
compulsory-traffic byte model (an operator is one C-ABI call; on this graph it is one launch of
the gather kernel that walks all source-column partitions, preceded by the tile-by-tile copy of the
gathered operand and followed by short closing kernels -- the fix-ups of split rows and the sum of
the passes' buffers for SpMM, the sum over feature tiles for SDDMM -- so `achieved` = the
operator's algorithmic bytes / the HIP-event time of all its launches; `kernels` lists them and
`avg_launch_ms` is that time divided by the number of launches of the gather kernel, i.e. it
carries the other kernels' share as well):
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
# by all launches of the gather kernel in one operator call, at the default tiling (the JSON reports
# them per launch as `traffic` and per operator as `op_traffic`, and names the summary they come from as
# `traffic_source`).  Configurations without a committed summary: null.  tests/test_bench_records.py holds every figure
# to the "Per launch, after calibration" table of the summary it names (read + write GB of the gather kernel, within 1 %).
_PROFILES = "profiles/bench_%s_rocprofv3.txt"
MEASURED_TRAFFIC = {
    # (operator, workload, F, partitions, tiles): (bytes, summary); tiles 0 = the kernel's own single tile
    ("spmm", "powerlaw-233k", 512, 8, 8): (59.2e9, _PROFILES % "powerlaw233k_f512"),     # spmm_items_kernel (copy: +0.95e9, sum of the passes: +4.3e9)
    ("sddmm", "powerlaw-233k", 512, 8, 8): (61.2e9, _PROFILES % "powerlaw233k_f512"),    # sddmm_tiled_kernel (copy: +0.95e9, tile sum: +4.7e9)
    ("spmm", "powerlaw-233k", 64, 8, 0): (8.50e9, _PROFILES % "powerlaw233k_f64"),
    ("sddmm", "powerlaw-233k", 64, 8, 1): (9.30e9, _PROFILES % "powerlaw233k_f64"),
    ("spmm", "powerlaw-233k", 32, 4, 0): (4.72e9, _PROFILES % "powerlaw233k_f32"),
    ("sddmm", "powerlaw-233k", 32, 4, 1): (5.44e9, _PROFILES % "powerlaw233k_f32"),
    ("spmm", "powerlaw-2.45M", 128, 1, 1): (33.15e9, _PROFILES % "powerlaw2450k_f128"),
    ("sddmm", "powerlaw-2.45M", 128, 1, 1): (33.41e9, _PROFILES % "powerlaw2450k_f128"),
}
METRIC = "SpMM/SDDMM GFLOP/s + achieved HBM GB/s (% roofline), 233k-node graph, feat 512"


def spmm_bytes(n_dst, n_src, nnz, F):
    return 4 * (n_dst + 1) + 8 * nnz + 4 * n_src * F + 4 * n_dst * F


def sddmm_bytes(n, nnz, F, H=1, csr=True):
    idx = 4 * (n + 1) + 4 * nnz if csr else 8 * nnz
    return idx + 8 * n * F + 4 * nnz * H


def cpu_baseline(indptr, indices, vals, x, y, F, spmm_run_s=0.25, sddmm_run_s=0.5):
    """The CPU oracle on the host cores over the first rows of the graph, following the reference's
    protocol (mean of 5 runs after one warm-up, python/featgraph/module/spmm.py:179-186, over a grid of
    its two x86 knobs, benchmark/bench_vanilla_spmm.py:36-41, trimmed to {1,4,16} x {1,4,16}).

    Two builds of the same loop nests are timed: one with fused multiply-add and AVX-512 clones, one
    with AVX2 and separately rounded multiply and add (the build the parity tests use); the faster of the
    two per operator goes into `value`, both are listed.

    The row samples are sized so that one SpMM run takes about `spmm_run_s` and one serial SDDMM run
    about `sddmm_run_s` seconds.  An SpMM call re-lays the WHOLE of X whatever the number of rows
    (python/featgraph/op/vanilla_spmm.py:43-44), so a row sample would overweight that fixed part; it is
    timed on its own (a call with zero rows) and the whole-graph time is put together as
    fixed + (sample - fixed) * nnz / sample edges."""
    import numpy as np
    import scipy.sparse as sp
    from oracle import oracle as orc
    threads = orc.max_threads()
    n = indptr.shape[0] - 1
    nnz = int(indptr[-1])

    def rows_for(nnz_target):
        return max(1, min(n, int(np.searchsorted(indptr, nnz_target, side="left"))))

    def mean5(fn):
        fn()                                    # warm-up
        t0 = time.perf_counter()
        for _ in range(5):
            fn()
        return (time.perf_counter() - t0) / 5

    def once(fn):
        t0 = time.perf_counter()
        fn()
        return time.perf_counter() - t0

    # calibrate on ~0.5 % of the edges, then size the samples
    r0 = rows_for(nnz // 200)
    e0 = int(indptr[r0])
    none = np.zeros(1, np.int32)
    t_fix = once(lambda: orc.spmm_csr_x86(none, indices[:0], vals[:0], x, 1, threads, fast=True))
    t = once(lambda: orc.spmm_csr_x86(indptr[:r0 + 1], indices[:e0], vals[:e0], x, 1, threads, fast=True))
    r_spmm = rows_for(min(nnz, int(e0 * spmm_run_s / max(t - t_fix, 1e-6))))
    e_spmm = int(indptr[r_spmm])
    ip = indptr[:r_spmm + 1]
    sub = sp.csr_matrix((vals[:e_spmm], indices[:e_spmm], ip), shape=(r_spmm, x.shape[0]))
    dds = {P: orc.csr_to_dds(sub, P) for P in (4, 16)}      # partitioning happens at construction: not timed

    def spmm_variant(T, P, fast):
        """(seconds for the sample, seconds of the part that does not depend on the rows)"""
        fixed = mean5(lambda: orc.spmm_csr_x86(none, indices[:0], vals[:0], x, T, threads, fast=fast))
        if P == 1:
            return mean5(lambda: orc.spmm_csr_x86(ip, indices[:e_spmm], vals[:e_spmm], x, T, threads, fast=fast)), fixed
        s1_pos, s1_idx, v = dds[P]
        return mean5(lambda: orc.spmm_dds_x86(s1_pos, s1_idx, v, x, r_spmm, P, T, threads, fast=fast)), fixed

    def whole(t_fixed):
        """Whole-graph seconds from (sample seconds, fixed seconds)."""
        return t_fixed[1] + max(t_fixed[0] - t_fixed[1], 1e-9) * nnz / max(e_spmm, 1)

    grid = [(T, P) for T in (1, 4, 16) for P in (1, 4, 16)]
    sweep = {k: spmm_variant(k[0], k[1], True) for k in grid}
    best = min(sweep, key=lambda k: whole(sweep[k]))
    pinned = {k: spmm_variant(k[0], k[1], False) for k in sorted({(1, 1), best})}
    best_pinned = min(pinned, key=lambda k: whole(pinned[k]))

    rows0 = np.repeat(np.arange(r0, dtype=np.int32), np.diff(indptr[:r0 + 1]))
    t = once(lambda: orc.sddmm_x86(rows0, indices[:e0], x, y, 1, False, 1, fast=True))
    r_sddmm = rows_for(min(nnz, int(e0 * sddmm_run_s / max(t, 1e-6))))
    e_sddmm = int(indptr[r_sddmm])
    rows = np.repeat(np.arange(r_sddmm, dtype=np.int32), np.diff(indptr[:r_sddmm + 1]))
    cols = indices[:e_sddmm]
    t_serial = mean5(lambda: orc.sddmm_x86(rows, cols, x, y, 1, False, 1, fast=True))
    t_serial_pinned = mean5(lambda: orc.sddmm_x86(rows, cols, x, y, 1, False, 1, fast=False))
    t_par = mean5(lambda: orc.sddmm_x86(rows, cols, x, y, 1, True, threads, fast=True))

    g_spmm_fast = 2.0 * nnz * F / whole(sweep[best]) / 1e9
    g_spmm_pinned = 2.0 * nnz * F / whole(pinned[best_pinned]) / 1e9
    g_sddmm_fast = 2.0 * e_sddmm * F / t_serial / 1e9           # no fixed part: T = 1 re-lays nothing
    g_sddmm_pinned = 2.0 * e_sddmm * F / t_serial_pinned / 1e9
    g_sddmm_par = 2.0 * e_sddmm * F / t_par / 1e9
    g_spmm, g_sddmm = max(g_spmm_fast, g_spmm_pinned), max(g_sddmm_fast, g_sddmm_pinned)
    # a step runs both ops over the same edges: combined rate = total flops / total time
    combined = 2.0 / (1.0 / g_spmm + 1.0 / g_sddmm)
    fmt = lambda d: {"T%d_P%d" % k: [round(v[0], 4), round(v[1], 4)] for k, v in d.items()}
    return {
        "value": round(combined, 3), "unit": "GFLOP/s", "cores": threads, "kind": "port",
        "sample": "C restatement of the reference x86 schedules (TVM unavailable), F=%d, mean of 5 runs after a warm-up. "
                  "SpMM row-parallel on %d threads over the first %d rows (%d of %d edges) for (num_feat_partitions, "
                  "num_col_partitions) in {1,4,16}x{1,4,16}, put together for the whole graph as re-layout of X (timed "
                  "with zero rows) + per-edge time x edges: best %s = %.2f GFLOP/s. SDDMM serial (1 thread, as the "
                  "reference schedule) over the first %d rows (%d edges, %.3f s) = %.2f GFLOP/s. value = harmonic "
                  "combination for one SpMM + one SDDMM over the same edges, each operator at the faster of two builds "
                  "(fused multiply-add with AVX-512 clones; AVX2 with separately rounded multiply and add, which the "
                  "parity tests use)"
                  % (F, threads, r_spmm, e_spmm, nnz, best if g_spmm_fast >= g_spmm_pinned else best_pinned, g_spmm,
                     r_sddmm, e_sddmm, min(t_serial, t_serial_pinned), g_sddmm),
        "spmm_gflops": round(g_spmm, 3), "sddmm_serial_gflops": round(g_sddmm, 3),
        "sddmm_edge_parallel_variant_gflops": round(g_sddmm_par, 3),
        "fma_avx512_build": {"spmm_gflops": round(g_spmm_fast, 3), "sddmm_serial_gflops": round(g_sddmm_fast, 3),
                             "spmm_sample_and_fixed_seconds": fmt(sweep)},
        "avx2_separate_rounding_build": {"spmm_gflops": round(g_spmm_pinned, 3), "sddmm_serial_gflops": round(g_sddmm_pinned, 3),
                                         "spmm_sample_and_fixed_seconds": fmt(pinned)},
    }


def verify(torch, spmm, sddmm, indptr, indices_d, vals_d, x_d, y_d):
    """Checks the operators' outputs for the benchmark inputs without a CPU product (the checks of
    featgraph_amd/benchmark/verify.py): the SpMM's column sums against the weighted out-degree contraction
    of X, five of its rows (largest, smallest, first, middle, last) and 200,000 sampled SDDMM edges against
    float64 formed on the device.  Returns a list of failures (empty: verified)."""
    from featgraph_amd.benchmark import verify as chk
    failures = chk.spmm_failures(spmm.run([x_d]), indptr, indices_d, vals_d, x_d)
    rows_d = torch.repeat_interleave(torch.arange(indptr.shape[0] - 1, device="cuda"),
                                     torch.from_numpy(indptr[1:] - indptr[:-1]).cuda().long())
    return failures + chk.sddmm_failures(sddmm.run([x_d, y_d]), rows_d, indices_d, x_d, y_d)


VALU_PEAK_GFLOPS = 157300.0      # fp32 vector peak of the part


def config_entry(config, workload, op, shape, tiling, seconds, flops, bytes_model, failures):
    """`tiling`: source-column partitions x feature tiles, or "stored order" for the kernels that walk the edges as stored."""
    gflops = flops / seconds / 1e9
    return {"config": config, "workload": workload, "op": op, "shape": shape, "tiling": tiling,
            "ms_mean_of_5": round(seconds * 1e3, 4), "gflops": round(gflops, 1),
            "compulsory_gb": round(bytes_model / 1e9, 4), "hbm_gbs": round(bytes_model / seconds / 1e9, 1),
            "pct_hbm_roofline": round(100.0 * bytes_model / seconds / 1e9 / HBM_PEAK_GBS, 3),
            "valu_frac": round(gflops / VALU_PEAK_GFLOPS, 4),
            "verified": not failures, **({"failures": failures} if failures else {})}


def sddmm_tiling(m):
    if m._tiled:
        return "%dx%d" % (m._tiled[0]['P'], m._tiled[1])
    return "stored order"


def run_configs(torch, workload, indptr, indices, vals_d, spmm, sddmm, headline_F, skip_low_degree=False):
    """Every other benchmark configuration at the library's defaults, outside the headline's timed region: the
    reference's protocol (mean of 5 back-to-back runs after a warm-up, python/featgraph/module/spmm.py:179-186;
    check of the output, tests/test_module_sddmm.py:34-37) per entry.  cfg2: SpMM at the other feature lengths;
    cfg3: SDDMM at the other feature lengths (edges stored in CSR order, the library's choice of kernel) and at the
    headline length with the kernel that walks the stored row / col arrays (`order='coo'`, forced: the default takes the
    tiled traversal there) and on the same edges stored in a random order (the default); cfg4: multi-head SDDMM;
    cfg5: SpMM then SDDMM on the 2.45M-node low-degree graph."""
    import numpy as np
    import scipy.sparse as sp
    from featgraph_amd import synthetic
    from featgraph_amd.benchmark import verify as chk
    from featgraph_amd.module import VanillaSpMMhip, VanillaSDDMMhip, MultiHeadSDDMMhip, placeholder
    entries = []
    gen = torch.Generator(device="cuda")

    def graph_side(indptr, indices):
        idx_d = torch.from_numpy(indices).cuda().long()
        rows_d = torch.repeat_interleave(torch.arange(indptr.shape[0] - 1, device="cuda"),
                                         torch.from_numpy(np.diff(indptr)).cuda().long())
        return idx_d, rows_d

    def pair(config, name, indptr, idx_d, rows_d, vals_d, spmm, sddmm, F, sddmm_only_order=None):
        n = indptr.shape[0] - 1
        nnz = idx_d.shape[0]
        gen.manual_seed(2)
        x = torch.randn((n, F), generator=gen, device="cuda")
        y = torch.randn((n, F), generator=gen, device="cuda")
        if sddmm_only_order is None:
            spmm.build([placeholder((n, F))], {}, {})
            t = spmm.measure_average_time([x], 5)
            entries.append(config_entry(config.split("/")[0], name, "spmm", "F=%d" % F,
                                        "%dx%d" % (spmm._active['P'], spmm._num_feat_partitions or 1),
                                        t, 2.0 * nnz * F, spmm_bytes(n, n, nnz, F),
                                        chk.spmm_failures(spmm.run([x]), indptr, idx_d, vals_d, x)))
        sa = {} if sddmm_only_order is None else {'order': sddmm_only_order}
        sddmm.build([placeholder((n, F)), placeholder((n, F))], {}, sa)
        t = sddmm.measure_average_time([x, y], 5)
        csr = sddmm_only_order != 'coo'
        entries.append(config_entry(config.split("/")[-1], name, "sddmm" if csr else "sddmm_coo_order", "F=%d" % F,
                                    sddmm_tiling(sddmm), t, 2.0 * nnz * F, sddmm_bytes(n, nnz, F, 1, csr=csr),
                                    chk.sddmm_failures(sddmm.run([x, y]), rows_d, idx_d, x, y)))

    n = indptr.shape[0] - 1
    nnz = indices.shape[0]
    idx_d, rows_d = graph_side(indptr, indices)
    for F in (32, 64, 128, 256, 512):
        if F != headline_F:
            pair("cfg2/cfg3", workload, indptr, idx_d, rows_d, vals_d, spmm, sddmm, F)
    pair("cfg3", workload, indptr, idx_d, rows_d, vals_d, spmm, sddmm, headline_F, sddmm_only_order='coo')
    # the same edges stored in a random order, at the library's default: sorted once at build(), walked by the tiled
    # traversal, every result written back to its stored position
    perm_d = torch.randperm(nnz, generator=torch.Generator().manual_seed(3)).cuda()
    rows_s, cols_s = rows_d[perm_d], idx_d[perm_d]
    shuffled = VanillaSDDMMhip(sp.coo_matrix((np.ones(nnz, np.float32), (rows_s.cpu().numpy().astype(np.int32),
                                                                         cols_s.cpu().numpy().astype(np.int32))), shape=(n, n)))
    F = headline_F
    gen.manual_seed(2)
    x = torch.randn((n, F), generator=gen, device="cuda")
    y = torch.randn((n, F), generator=gen, device="cuda")
    shuffled.build([placeholder((n, F)), placeholder((n, F))], {}, {})
    t = shuffled.measure_average_time([x, y], 5)
    entries.append(config_entry("cfg3", workload, "sddmm_shuffled_coo", "F=%d" % F, sddmm_tiling(shuffled), t, 2.0 * nnz * F,
                                sddmm_bytes(n, nnz, F, 1, csr=False), chk.sddmm_failures(shuffled.run([x, y]), rows_s, cols_s, x, y)))
    del shuffled, x, y, perm_d, rows_s, cols_s
    mh = MultiHeadSDDMMhip(sp.csr_matrix((np.ones(nnz, np.float32), indices, indptr), shape=(n, n)))
    mh.share_layouts(spmm)
    for H, D in ((4, 32), (4, 64), (8, 32), (8, 64)):
        gen.manual_seed(2)
        x = torch.randn((n, H, D), generator=gen, device="cuda")
        y = torch.randn((n, H, D), generator=gen, device="cuda")
        mh.build([placeholder((n, H, D)), placeholder((n, H, D))], {}, {})
        t = mh.measure_average_time([x, y], 5)
        entries.append(config_entry("cfg4", workload, "sddmm_multihead", "H=%d D=%d" % (H, D), sddmm_tiling(mh), t,
                                    2.0 * nnz * H * D, sddmm_bytes(n, nnz, H * D, H, csr=True),
                                    chk.sddmm_failures(mh.run([x, y]), rows_d, idx_d, x, y)))
    del mh, x, y, idx_d, rows_d
    torch.cuda.empty_cache()
    if not skip_low_degree:
        name = "powerlaw-2.45M"
        ip5, ix5 = synthetic.make_workload(name)
        n5, nnz5 = ip5.shape[0] - 1, ix5.shape[0]
        gen.manual_seed(1)
        v5 = torch.rand(nnz5, generator=gen, device="cuda", dtype=torch.float32)
        adj5 = sp.csr_matrix((v5.cpu().numpy(), ix5, ip5), shape=(n5, n5))
        idx_d, rows_d = graph_side(ip5, ix5)
        pair("cfg5", name, ip5, idx_d, rows_d, v5, VanillaSpMMhip(adj5), VanillaSDDMMhip(adj5), 128)
    return entries


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
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the block that times and checks the other benchmark configurations after the headline")
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
    setup = {}
    t0 = time.perf_counter()
    indptr, indices = synthetic.make_workload(args.workload)
    setup["graph_generation_s"] = round(time.perf_counter() - t0, 3)
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

    def timed(key, fn):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        res = fn()
        torch.cuda.synchronize()
        setup[key] = round(time.perf_counter() - t0, 3)
        return res

    # construction: structure checks and host arrays; build(): the cost model's choice, the source-partitioned copy of the
    # adjacency (converted on the host), its work plan, the upload, the 16-bit column ids and the scratch
    spmm = timed("spmm_construct_s", lambda: VanillaSpMMhip(adj, args.num_col_partitions))
    timed("spmm_build_s", lambda: spmm.build([placeholder((n, F))], {'num_feat_partitions': args.num_feat_partitions}, {}))
    sddmm = timed("sddmm_construct_s", lambda: VanillaSDDMMhip(adj))
    sddmm.share_layouts(spmm)           # same adjacency: one partitioned copy, one plan, one scratch for both operators
    timed("sddmm_build_s", lambda: sddmm.build([placeholder((n, F)), placeholder((n, F))], {}, {}))
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
    # outside the timed region: the operators' outputs for these inputs are checked, and the reference's own
    # protocol (mean of 5 back-to-back runs, python/featgraph/module/spmm.py:179-186) is timed as well
    # what the two modules and their inputs hold on the device: the modules' own accounts (graph arrays; plans = the
    # library's own allocations, fg_spmm_plan_bytes; output buffers) and the device's view of the whole process
    free_b, total_b = torch.cuda.mem_get_info()
    gb = lambda b: round(b / 1e9, 3)
    device_mem = {"spmm_module_gb": {k: gb(v) for k, v in spmm.device_bytes().items()},
                  "sddmm_module_gb": {k: gb(v) for k, v in sddmm.device_bytes().items()},
                  "inputs_gb": gb(4 * (2 * n * F + nnz)), "torch_peak_allocated_gb": gb(torch.cuda.max_memory_allocated()),
                  "process_total_gb": gb(total_b - free_b)}
    failures = verify(torch, spmm, sddmm, indptr, torch.from_numpy(indices).cuda().long(), vals_d, x_d, y_d)
    runs5 = {"spmm_ms": round(spmm.measure_average_time([x_d], 5) * 1e3, 4),
             "sddmm_ms": round(sddmm.measure_average_time([x_d, y_d], 5) * 1e3, 4)}
    t_spmm = sum(e[0].elapsed_time(e[1]) for e in evs) / args.steps      # ms, HIP events on the launch stream
    t_sddmm = sum(e[1].elapsed_time(e[2]) for e in evs) / args.steps

    def tile_groups(n_tiles):
        """More than 8 feature tiles are launched 8 at a time (one per XCD)."""
        return n_tiles // 8 if (n_tiles > 8 and n_tiles % 8 == 0) else 1

    def sddmm_launches():
        """Launches of the tiled kernel: one launch walks all partitions (8 / T of them at a time when there are
        fewer than 8 tiles); only beyond 32 such groups does every group get a launch of its own."""
        if not sddmm._tiled:
            return 1
        P, T = sddmm._tiled[0]['P'], sddmm._tiled[1]
        conc = min(8 // T, P) if (T < 8 and 8 % T == 0) else 1
        groups = (P + conc - 1) // conc
        return tile_groups(T) * (1 if groups <= 32 else groups)

    def copies(n_tiles):
        """Launches of the kernel that makes the tile-by-tile copy of the gathered operand (the library's
        default rule: 4 or more feature tiles, 64 MB or more, 32-bit offsets)."""
        return 1 if (n_tiles >= 4 and (64 << 20) <= 4 * n * F < (1 << 32)) else 0

    def pass_sums(n_parts):
        """Launches of the kernel that adds the SpMM passes' own buffers into out (the library's default rule:
        several source partitions and buffers of 8 GiB or less)."""
        return 1 if (n_parts >= 2 and 4 * n * F * n_parts <= (8 << 30)) else 0

    def spmm_launches():
        """Launches of the gather kernel: with buffers per pass one launch walks all partitions, else one per partition."""
        P = spmm._active['P']
        return tile_groups(spmm._num_feat_partitions or 1) * (1 if (P == 1 or pass_sums(P)) else P)

    plain_sddmm = "sddmm_csr_kernel" if sddmm._use_csr else "sddmm_coo_kernel"     # the stored-order kernels
    flops_op = 2.0 * nnz * F
    b_spmm = spmm_bytes(n, n, nnz, F)
    b_sddmm = sddmm_bytes(n, nnz, F, 1, csr=True)
    ops = {
        "spmm": {"ms": t_spmm, "gflops": flops_op / t_spmm / 1e6, "compulsory_gb": b_spmm / 1e9,
                 "hbm_gbs": b_spmm / t_spmm / 1e6, "gathered_gbs": 4.0 * nnz * F / t_spmm / 1e6,
                 "kernel": "spmm_items_kernel", "launches": spmm_launches(),
                 "kernels": {"tile_major_kernel": copies(spmm._num_feat_partitions or 1),
                             "spmm_items_kernel": spmm_launches(),
                             "spmm_fixup_kernel": 1 if pass_sums(spmm._active['P']) else spmm._active['P'],
                             "spmm_pass_sum_kernel": pass_sums(spmm._active['P'])},
                 "num_col_partitions": spmm._active['P'], "num_feat_partitions": spmm._num_feat_partitions},
        "sddmm": {"ms": t_sddmm, "gflops": flops_op / t_sddmm / 1e6, "compulsory_gb": b_sddmm / 1e9,
                  "hbm_gbs": b_sddmm / t_sddmm / 1e6, "gathered_gbs": 4.0 * nnz * F / t_sddmm / 1e6,
                  "kernel": "sddmm_tiled_kernel" if sddmm._tiled else plain_sddmm,
                  "launches": sddmm_launches(),
                  "kernels": ({"tile_major_kernel": copies(sddmm._tiled[1]), "sddmm_tiled_kernel": sddmm_launches(),
                               "sddmm_tile_sum_kernel": 1 if sddmm._tiled[1] > 1 else 0}
                              if sddmm._tiled else {plain_sddmm: 1}),
                  "num_src_partitions": sddmm._tiled[0]['P'] if sddmm._tiled else 1,
                  "num_feat_tiles": sddmm._tiled[1] if sddmm._tiled else 1},
    }
    for o in ops.values():
        o["pct_hbm_roofline"] = 100.0 * o["hbm_gbs"] / HBM_PEAK_GBS
        o["valu_frac"] = o["gflops"] / VALU_PEAK_GFLOPS          # share of the fp32 vector peak (157.3 TFLOP/s)
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
                "valu_frac": round(ops[dom]["valu_frac"], 5),
                "traffic": (round(op_traffic[0] / n_launch) if op_traffic else None),
                "op_traffic": (op_traffic[0] if op_traffic else None),
                # `traffic` is a stored figure from the named rocprofv3 summary (same workload, feature length and
                # tiling as this run), not a counter read in this run
                "traffic_source": (op_traffic[1] if op_traffic else None),
                "algorithmic_bytes_per_launch": int(b_dom / n_launch), "algorithmic_bytes": int(b_dom),
                "launches": ops[dom]["launches"], "kernels": ops[dom]["kernels"], "op_ms": round(ops[dom]["ms"], 4),
                "avg_launch_ms": round(ops[dom]["ms"] / ops[dom]["launches"], 4)}

    line = {
        "metric": METRIC, "value": round(2 * flops_op / (ms_per_step * 1e6), 2), "unit": "GFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "%s: weighted CSR SpMM + SDDMM over the same edges, F=%d, fp32, int32 indices" % (args.workload, F),
                   "nodes": n, "edges": nnz, "max_in_degree": int(deg.max()), "median_in_degree": float(np.median(deg)),
                   "feat_len": F,
                   # what ran (the library's own choice where the command line left the default: 0 tiles / 1 partition)
                   "num_feat_partitions": spmm._num_feat_partitions, "num_col_partitions": spmm._active['P'],
                   "requested": {"num_feat_partitions": args.num_feat_partitions, "num_col_partitions": args.num_col_partitions},
                   "seeds": {"graph": 0xFEA7, "weights": 1, "features": 2}},
        "roofline": roofline,
        "verified": not failures,
        "setup_s": setup,
        "device_mem_gb": device_mem,
        "gpu_mean_of_5_runs": runs5,
        "ops": {k: {kk: (round(vv, 4) if isinstance(vv, float) else vv) for kk, vv in v.items()} for k, v in ops.items()},
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(indptr, indices, vals, x_d.cpu().numpy(), y_d.cpu().numpy(), F)
    if failures:
        line["verification_failures"] = failures
    if not args.no_configs and args.workload == "powerlaw-233k" and F == 512:     # the default invocation only
        del x_d, y_d
        torch.cuda.empty_cache()
        t0 = time.perf_counter()
        entries = run_configs(torch, args.workload, indptr, indices, vals_d, spmm, sddmm, F)
        # one row per configuration (the JSON line stays short; the same table goes to stderr in readable form)
        cols = ["config", "workload", "op", "shape", "tiling", "ms_mean_of_5", "gflops", "compulsory_gb", "hbm_gbs",
                "pct_hbm_roofline", "valu_frac", "verified"]
        line["configs"] = {"columns": cols, "rows": [[e[c] for c in cols] for e in entries]}
        line["configs_verified"] = sum(1 for e in entries if e["verified"])
        line["configs_total"] = len(entries)
        line["configs_seconds"] = round(time.perf_counter() - t0, 1)
        failures = failures + ["%s %s %s: %s" % (e["workload"], e["op"], e["shape"], "; ".join(e["failures"]))
                               for e in entries if not e["verified"]]
        for e in entries:
            print("%-5s %-15s %-19s %-9s %-38s %8.3f ms %7.0f GFLOP/s %6.2f %% of 8 TB/s  %s"
                  % (e["config"], e["workload"], e["op"], e["shape"], e["tiling"], e["ms_mean_of_5"], e["gflops"],
                     e["pct_hbm_roofline"], "verified" if e["verified"] else "FAILED"), file=sys.stderr)
    print(json.dumps(line))
    if failures:
        sys.exit("bench.py: output verification failed: " + "; ".join(failures))


if __name__ == "__main__":
    main()
