"""CPU-only tests of the shipped library's host side: the C ABI loads and exports what the
header declares, the host partitioners are bit-exact with the oracle and the reference's
stored vectors, structural checks reject bad graphs, the generator is deterministic, and the
operator classes refuse to run without a GPU instead of falling back."""
import json
import os
import re

import numpy as np
import pytest
import scipy.sparse as sp

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def fg():
    from featgraph_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from featgraph_amd import build
        build.build(verbose=False)
    _lib.lib()
    return _lib


def test_header_symbols_exported(fg):
    text = open(os.path.join(ROOT, "include", "featgraph_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = set(re.findall(r"\b(fg_[a-z0-9_]+)\s*\(", text))
    assert declared == set(fg.SIGNATURES), declared ^ set(fg.SIGNATURES)
    for name in declared:
        assert hasattr(fg.lib(), name), name
    assert fg.lib().fg_version() >= 100


def test_golden_vectors(fg):
    from featgraph.util import util_convert_csr_to_dds, util_partition_adj_coo_2d
    g = json.load(open(os.path.join(ROOT, "tests", "golden", "util_5x5.json")))
    coo = sp.coo_matrix((np.array(g["data"], dtype="int32"), (g["row"], g["col"])), shape=(5, 5), dtype="int32")
    s1_pos, s1_idx, vals = util_convert_csr_to_dds(coo.tocsr(), g["dds_num_col_partitions"])
    assert vals.tolist() == g["dds_vals"]
    assert s1_idx.tolist() == g["dds_s1_idx"]
    assert s1_pos.tolist() == g["dds_s1_pos"]
    before = coo.data.copy()
    eid, row, col = util_partition_adj_coo_2d(coo, 2, 2)
    assert eid.tolist() == g["part2d_edge_id_list"]
    assert (coo.data == before).all()
    assert eid.dtype == np.int32 and row.dtype == np.int32 and col.dtype == np.int32


@pytest.mark.parametrize("shape,density", [((127, 255), 0.1), ((1000, 40), 0.3), ((3, 5000), 0.05), ((64, 64), 1.0)])
def test_partitioners_match_oracle(fg, oracle, shape, density):
    from featgraph_amd.util import util_convert_csr_to_dds, util_partition_adj_coo_2d
    rng = np.random.default_rng(shape[0])
    a = sp.random(shape[0], shape[1], density=density, format="csr", random_state=rng).astype("float32")
    a.sort_indices()
    for P in (1, 2, 4, 7, 32, shape[1], shape[1] + 3):
        for x, y in zip(util_convert_csr_to_dds(a, P), oracle.csr_to_dds(a, P)):
            assert x.dtype == y.dtype and np.array_equal(x, y)
    coo = a.tocoo()
    perm = rng.permutation(coo.nnz)
    coo = sp.coo_matrix((coo.data[perm], (coo.row[perm], coo.col[perm])), shape=coo.shape)
    for R, C in ((1, 1), (2, 3), (4, 4), (32, 1), (1, 32), (shape[0], shape[1]), (shape[0] + 2, 5)):
        for x, y in zip(util_partition_adj_coo_2d(coo, R, C), oracle.partition_coo_2d(coo, R, C)):
            assert x.dtype == y.dtype and np.array_equal(x, y)


def test_partitioner_edge_cases(fg):
    from featgraph_amd.util import util_convert_csr_to_dds, util_partition_adj_coo_2d
    empty = sp.csr_matrix((4, 6), dtype="float32")
    s1_pos, s1_idx, vals = util_convert_csr_to_dds(empty, 3)
    assert s1_pos.tolist() == [0] * 15 and len(s1_idx) == 0 and len(vals) == 0
    eid, r, c = util_partition_adj_coo_2d(empty.tocoo(), 2, 2)
    assert len(eid) == 0
    with pytest.raises(AssertionError):
        util_convert_csr_to_dds(empty, 0)
    with pytest.raises(AssertionError):
        util_partition_adj_coo_2d(empty.tocoo(), 1, 0)
    dup = sp.coo_matrix((np.ones(3, "int32"), ([0, 0, 1], [1, 1, 0])), shape=(2, 2))
    with pytest.raises(ValueError):
        util_partition_adj_coo_2d(dup, 2, 2)
    f64 = sp.identity(3, dtype="float64", format="csr")
    _, _, v64 = util_convert_csr_to_dds(f64, 2)            # any dtype, as in the reference
    assert v64.dtype == np.float64 and v64.tolist() == [1.0, 1.0, 1.0]
    # unsorted column ids inside a row keep their stored order within each partition
    uns = sp.csr_matrix((np.array([1, 2, 3, 4], "float32"), np.array([3, 0, 2, 1], "int32"), np.array([0, 4], "int32")),
                        shape=(1, 4))
    s1_pos, s1_idx, vals = util_convert_csr_to_dds(uns, 2)
    assert s1_pos.tolist() == [0, 2, 2, 4] and s1_idx.tolist() == [0, 1, 1, 0] and vals.tolist() == [2, 4, 1, 3]


def test_check_csr_host(fg):
    L = fg.lib()
    ok_ptr = np.array([0, 2, 2, 3], dtype=np.int32)
    ok_idx = np.array([0, 4, 1], dtype=np.int32)
    assert L.fg_check_csr_host(3, 5, fg.host_ptr(ok_ptr), fg.host_ptr(ok_idx)) == 0
    assert L.fg_check_csr_host(3, 4, fg.host_ptr(ok_ptr), fg.host_ptr(ok_idx)) == -3
    assert "outside" in fg.last_error()
    bad = np.array([0, 2, 1, 3], dtype=np.int32)
    assert L.fg_check_csr_host(3, 5, fg.host_ptr(bad), fg.host_ptr(ok_idx)) == -3
    bad0 = np.array([1, 2, 2, 3], dtype=np.int32)
    assert L.fg_check_csr_host(3, 5, fg.host_ptr(bad0), fg.host_ptr(ok_idx)) == -3
    assert L.fg_check_csr_host(3, 5, None, None) == -1
    with pytest.raises(ValueError):
        fg.check(-3)


def test_synthetic_graphs(fg):
    from featgraph_amd import synthetic
    a = synthetic.make_workload("powerlaw-23k", num_threads=1)
    b = synthetic.make_workload("powerlaw-23k", num_threads=5)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    indptr, indices = a
    n = indptr.shape[0] - 1
    deg = np.diff(indptr)
    rows = np.repeat(np.arange(n), deg)
    keys = rows.astype(np.int64) * n + indices
    assert (np.diff(keys) > 0).all()                      # sorted, no duplicates
    assert indices.min() >= 0 and indices.max() < n
    loops = np.zeros(n, bool); loops[rows[rows == indices]] = True
    assert loops.all()
    assert 1_000_000 < indptr[-1] < 1_200_000 and deg.max() > 1000
    # fixed checksum: the graph is the same on every host
    assert int(indices.astype(np.int64).sum() % 1000003) == int(b[1].astype(np.int64).sum() % 1000003)
    c = synthetic.make_workload("powerlaw-23k", seed=7)
    assert not np.array_equal(c[1][:1000], indices[:1000])
    u_ptr, u_idx = synthetic.make_workload("uniform-10k")
    assert u_ptr.shape[0] == 10001 and 160000 <= u_ptr[-1] <= 170000
    w = synthetic.edge_weights(1000, 1)
    assert w.dtype == np.float32 and 0 <= w.min() and w.max() < 1 and abs(w.mean() - 0.5) < 0.05


def test_no_cpu_fallback(fg):
    import torch
    if torch.cuda.is_available():
        pytest.skip("this check is for hosts without a GPU")
    from featgraph.module import VanillaSpMMx86, VanillaSDDMMx86
    adj = sp.identity(4, dtype="float32", format="csr")
    with pytest.raises(RuntimeError, match="GPU"):
        VanillaSpMMx86(adj)
    with pytest.raises(RuntimeError, match="GPU"):
        VanillaSDDMMx86(adj)


def test_product_does_not_import_oracle():
    """The shipped package must not reach the CPU oracle in any way."""
    pkg = os.path.join(ROOT, "featgraph_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".cpp", ".h")):
                text = open(os.path.join(base, f)).read()
                assert "oracle" not in text, os.path.join(base, f)


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asking for more ends with a message instead of a run."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr


def test_default_tilings():
    """The defaults the cost model picks for the benchmark shapes (pure arithmetic, no GPU), with and without
    the graph's own statistics, and the model's building blocks."""
    from featgraph_amd import tuning
    n, nnz = 232965, 114766039
    assert tuning.choose_spmm(n, n, nnz, 512) == (8, 8)
    assert tuning.choose_spmm(n, n, nnz, 128) == (8, 2)
    assert tuning.choose_spmm(n, n, nnz, 32) == (4, 0)
    assert tuning.choose_spmm(2450000, 2450000, 61903880, 128) == (1, 1)     # rows too short to partition
    assert tuning.choose_spmm(1000000, 1000000, 64998031, 128) == (1, 1)     # no slice an L2 could hold: plain CSR
    assert tuning.choose_sddmm(n, n, nnz, 1, 512) == (8, 8)
    assert tuning.choose_sddmm(n, n, nnz, 1, 256) == (8, 4)
    assert tuning.choose_sddmm(n, n, nnz, 1, 1024) == (8, 16)
    assert tuning.choose_sddmm(2450000, 2450000, 61903880, 1, 128) is None    # stored-order kernels
    assert tuning.choose_sddmm(2450000, 2450000, 61903880, 1, 512) is None    # no source partitions: stored order, not 1 x 2 tiles
    assert tuning.choose_sddmm(1000000, 1000000, 64998031, 1, 512) is None
    assert tuning.choose_sddmm(n, n, nnz, 8, 64) == (8, 8)                     # one head per tile, results staged per tile
    assert tuning.choose_sddmm(n, n, nnz, 4, 64) == (8, 4)
    assert tuning.choose_sddmm(n, n, nnz, 8, 32) == (32, 1)                    # all 8 heads in one 256-float tile: whole 32-byte runs
    assert tuning.choose_sddmm(n, n, nnz, 4, 32) == (8, 2)
    assert tuning.choose_sddmm(10000, 10000, 170000, 1, 32) is None           # fits the caches: plain kernels
    for F in (32, 64, 96, 128, 256, 512, 2048):
        p, t = tuning.choose_sddmm(n, n, nnz, 1, F)
        assert F % t == 0 and p >= 1 and F // t >= 32
        p, t = tuning.choose_spmm(n, n, nnz, F)
        assert p >= 1 and (t == 0 or F % t == 0)
    # a graph with locality (41 planted communities, ids community-contiguous or relabelled at random): the defaults,
    # from the graph's own statistics, are the points that full sweeps on the GPU found within 2 % of the best
    from featgraph_amd import synthetic
    for name in ("communities-233k", "communities-233k-relabelled"):
        ip, ix = synthetic.make_workload(name)
        st = tuning.GraphStats.from_csr(ip, ix, n)
        assert 112e6 < st.nnz < 117e6
        assert tuning.choose_spmm(n, n, st.nnz, 512, st) == (8, 8) and tuning.choose_spmm(n, n, st.nnz, 128, st) == (8, 2)
        assert tuning.choose_sddmm(n, n, st.nnz, 1, 512, st) == (8, 8) and tuning.choose_sddmm(n, n, st.nnz, 1, 128, st) == (16, 1)
    # hit-rate estimate: monotone in the capacity, 0 for an empty cache, compulsory misses only when all fits
    skew = tuning.GraphStats(1000, 1000, 100000, count_vals=[10, 1000], count_mult=[900, 91], deg_vals=[100], deg_mult=[1000])
    rates = [skew.hit_rate(k) for k in (1, 10, 91, 300, 991, 5000)]
    assert all(a <= b + 1e-12 for a, b in zip(rates, rates[1:])) and rates[0] < 0.05
    assert abs(rates[-1] - (1 - 991 / 100000)) < 1e-9
    assert rates[2] > 0.5                     # the 91 hot columns carry 91 % of the references
    flat = tuning.GraphStats(1000, 1000, 100000)
    assert abs(flat.hit_rate(500) - 0.5) < 0.1
    # row segments: a row of degree d over P partitions
    assert flat.segments(1) == 1000 and abs(flat.segments(4) - 4000) < 1
    short = tuning.GraphStats(1000, 1000, 2000, deg_vals=[2], deg_mult=[1000])
    assert abs(short.segments(8) - 1000 * 8 * (1 - (7 / 8) ** 2)) < 1e-6
    # statistics from a CSR
    ip = np.array([0, 2, 2, 5], np.int32); ix = np.array([0, 3, 3, 1, 0], np.int32)
    st = tuning.GraphStats.from_csr(ip, ix, 4)
    assert (st.n_dst, st.n_src, st.nnz) == (3, 4, 5)
    assert dict(zip(st.count_vals.tolist(), st.count_mult.tolist())) == {1.0: 1.0, 2.0: 2.0}
    # ranked candidates start with the choice
    assert tuning.rank_spmm(tuning.GraphStats(n, n, nnz), 512)[0] == (8, 8)
    # source partitions of a broadcasting message: none without a gathered operand, for an operand that fits the caches
    # or when every partition's buffer of results would not fit 8 GiB together; fewer than for the weighted sum
    assert tuning.choose_gather_partitions(n, n, nnz, 0, 64) == 1
    assert tuning.choose_gather_partitions(10000, 10000, 170000, 32, 32) == 1
    assert tuning.choose_gather_partitions(n, n, nnz, 64, 64) in (2, 4, 8)
    assert tuning.choose_gather_partitions(n, n, nnz, 64, 64) <= tuning.choose_spmm(n, n, nnz, 64)[0]
    assert tuning.choose_gather_partitions(n, n, nnz, 64, 1 << 14) == 1
    assert tuning.choose_gather_partitions(0, n, 0, 64, 64) == 1


def test_partitioners_property_based(fg, oracle):
    """Random small matrices, partition counts and storage orders: the library's partitioners agree with
    the oracle bit for bit, the DDS arrays expand back to the matrix, and the 2-D edge ids are a
    permutation that argsort inverts."""
    from hypothesis import given, settings, strategies as st
    from featgraph_amd.util import util_convert_csr_to_dds, util_partition_adj_coo_2d

    @settings(max_examples=150, deadline=None)
    @given(st.integers(1, 12), st.integers(1, 12), st.integers(0, 2 ** 31 - 1), st.floats(0.0, 1.0),
           st.integers(1, 15), st.integers(1, 15))
    def check(n_rows, n_cols, seed, density, a_parts, b_parts):
        rng = np.random.default_rng(seed)
        mask = rng.random((n_rows, n_cols)) < density
        dense = np.where(mask, rng.integers(1, 1000, size=(n_rows, n_cols)), 0).astype(np.int32)
        csr = sp.csr_matrix(dense)
        csr.sort_indices()
        got = util_convert_csr_to_dds(csr, a_parts)
        for x, y in zip(got, oracle.csr_to_dds(csr, a_parts)):
            assert np.array_equal(x, y)
        s1_pos, s1_idx, vals = got
        width = -(-n_cols // a_parts)
        rebuilt = np.zeros_like(dense)
        for p in range(a_parts):
            for r in range(n_rows):
                for k in range(s1_pos[p * (n_rows + 1) + r], s1_pos[p * (n_rows + 1) + r + 1]):
                    rebuilt[r, s1_idx[k] + p * width] = vals[k]
        assert np.array_equal(rebuilt, dense)
        coo = csr.tocoo()
        perm = rng.permutation(coo.nnz)
        coo = sp.coo_matrix((coo.data[perm], (coo.row[perm], coo.col[perm])), shape=coo.shape)
        eid, row, col = util_partition_adj_coo_2d(coo, a_parts, b_parts)
        for x, y in zip((eid, row, col), oracle.partition_coo_2d(coo, a_parts, b_parts)):
            assert np.array_equal(x, y)
        assert sorted(eid.tolist()) == list(range(1, coo.nnz + 1))
        assert np.array_equal(row, coo.row[eid - 1]) and np.array_equal(col, coo.col[eid - 1])
        mapping = np.argsort(eid)
        assert np.array_equal(eid[mapping], np.arange(1, coo.nnz + 1))

    check()


@pytest.mark.parametrize("dtype", ["float64", "int64", "int16", "complex64"])
def test_dds_values_of_any_width(fg, oracle, dtype):
    """The reference's util keeps the dtype of adj.data (adj_partitioning.py:37-39), e.g. the float64
    of scipy.sparse.random; values that are not 32 bits wide take the host-side permutation."""
    from featgraph_amd.util import util_convert_csr_to_dds
    rng = np.random.default_rng(5)
    a = sp.random(60, 90, density=0.2, format="csr", random_state=rng)
    a.data = (a.data * 1000).astype(dtype)
    a.sort_indices()
    for P in (1, 3, 8):
        s1_pos, s1_idx, vals = util_convert_csr_to_dds(a, P)
        ref_pos, ref_idx, ref_perm = oracle.csr_to_dds(sp.csr_matrix((np.arange(a.nnz, dtype=np.int32), a.indices, a.indptr), shape=a.shape), P)
        assert vals.dtype == a.data.dtype
        assert np.array_equal(s1_pos, ref_pos) and np.array_equal(s1_idx, ref_idx)
        assert np.array_equal(vals, a.data[ref_perm])


@pytest.mark.parametrize("R,C", [(4, 1), (1, 3), (2, 5)])
def test_edge_mapping_restores_stored_order_for_unequal_partition_counts(fg, oracle, R, C):
    """R != C: the reference's SDDMMbase overwrites num_col_partitions with num_row_partitions
    (python/featgraph/module/sddmm.py:37) while this build honours both, so the traversal order
    differs from the reference's there -- but out[edge_mapping] is the unpartitioned result either way."""
    from featgraph_amd.util import util_partition_adj_coo_2d
    rng = np.random.default_rng(R * 10 + C)
    coo = sp.random(50, 70, density=0.15, format="coo", random_state=rng).astype("float32")
    src = rng.standard_normal((70, 24)).astype("float32")
    dst = rng.standard_normal((50, 24)).astype("float32")
    eid, row, col = util_partition_adj_coo_2d(coo, R, C)
    mapping = np.argsort(eid)
    assert sorted(eid.tolist()) == list(range(1, coo.nnz + 1))
    out_part = oracle.sddmm_x86(row, col, src, dst)
    out_plain = oracle.sddmm_x86(coo.row, coo.col, src, dst)
    assert np.array_equal(out_part[mapping], out_plain)
    # blocks in row-major block order: block ids never decrease along the traversal
    rb = row // -(-50 // R)
    cb = col // -(-70 // C)
    assert (np.diff(rb * C + cb) >= 0).all()


def test_sizes_beyond_int32_are_refused():
    """Index arrays are narrowed to int32 at construction; a matrix that does not fit must raise, not wrap."""
    from featgraph_amd.module import common
    common.check_int32_sizes(232965, 232965, 114766039)
    for shape in [(2 ** 31, 10, 5), (10, 2 ** 31 - 1, 5), (10, 10, 2 ** 31 - 1)]:
        with pytest.raises(ValueError, match="int32"):
            common.check_int32_sizes(*shape)


def test_community_graph_generator():
    """fg_synth_community_csr: bit-identical for a seed whatever the thread count, sorted duplicate-free rows with a
    self-loop each, most of a row's sources inside its own community, and the relabelled variant the same kind of
    graph (same size class, no community structure left in the id ranges)."""
    from featgraph_amd import synthetic
    spec = synthetic.WORKLOADS["communities-23k"]
    ip, ix = synthetic.make_workload("communities-23k")
    ip2, ix2 = synthetic.make_workload("communities-23k", num_threads=3)
    assert np.array_equal(ip, ip2) and np.array_equal(ix, ix2)
    n, C = spec["n"], spec["n_comm"]
    assert ip.dtype == np.int32 and ix.dtype == np.int32 and ip[0] == 0 and ip[-1] == ix.shape[0]
    rows = np.repeat(np.arange(n), np.diff(ip))
    inner = np.ones(ix.shape[0], bool); inner[ip[1:-1]] = False
    assert (np.diff(ix)[inner[1:]] > 0).all()                                   # sorted, no duplicates inside a row
    assert (np.diff(ip) >= 1).all()
    has_loop = np.zeros(n, bool); has_loop[rows[ix == rows]] = True
    assert has_loop.all()
    # contiguous ids: community c owns the id range [off[c], off[c + 1]) (ranks r with r % C == c)
    off = np.concatenate([[0], np.cumsum(np.bincount(np.arange(n) % C, minlength=C))])
    same = (np.searchsorted(off, rows, side='right') == np.searchsorted(off, ix, side='right'))
    assert same.mean() > 0.7
    relab = dict(spec, contiguous=False)
    ip3, ix3 = synthetic.community_csr(relab["n"], relab["total_edges"], relab["exponent"], relab["max_degree"], C,
                                       relab["p_in"], False, relab["seed"])
    assert abs(int(ip3[-1]) - int(ip[-1])) < 0.02 * ip[-1]
    rows3 = np.repeat(np.arange(n), np.diff(ip3))
    same3 = (np.searchsorted(off, rows3, side='right') == np.searchsorted(off, ix3, side='right'))
    assert same3.mean() < 0.3
    # bad arguments are refused
    from featgraph_amd import _lib
    assert _lib.lib().fg_synth_community_csr(0, None, None, None, 1, None, None, None, None, 0.5, 1, 0, None, None) == -1
