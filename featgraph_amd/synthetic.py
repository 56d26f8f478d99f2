"""Seeded synthetic graphs of the shapes the benchmarks are quoted on.

The reference benchmarks load the Reddit adjacency saved by
benchmark/download_reddit_dataset.py:9-17, which needs DGL and a network.  These generators
produce graphs of the same size class instead (power-law in-degrees, no duplicate edges,
self-loops, per-row sorted int32 column ids), bit-identical for a given seed on any host.
"""
import numpy as np

from . import _lib

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def _mix64(z):
    """splitmix64 finaliser on a uint64 array (wrapping arithmetic)."""
    with np.errstate(over="ignore"):
        z = (z + np.uint64(0x9E3779B97F4A7C15)) & _M64
        z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _M64
        z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _M64
        return z ^ (z >> np.uint64(31))


def seeded_permutation(n, seed):
    keys = _mix64(np.arange(n, dtype=np.uint64) ^ _mix64(np.full(n, seed, dtype=np.uint64)))
    return np.argsort(keys, kind="stable").astype(np.int32)


def powerlaw_weights(n, total, exponent, max_weight):
    """w_i = max_weight * ((i + i0) / i0) ** (-1 / (exponent - 1)), i = 0..n-1, with i0 chosen by
    bisection so that the weights add up to `total`."""
    alpha = 1.0 / (exponent - 1.0)
    i = np.arange(n, dtype=np.float64)

    def weights(i0):
        return max_weight * ((i + i0) / i0) ** (-alpha)

    lo, hi = 1e-3, float(n) * 1e3
    if weights(hi).sum() < total:
        raise ValueError("max_weight * n is below the requested total")
    for _ in range(200):
        mid = np.sqrt(lo * hi)
        if weights(mid).sum() < total:
            lo = mid
        else:
            hi = mid
    return weights(hi)


def powerlaw_csr(n, total_edges, exponent, max_degree, seed, num_threads=0):
    """Directed power-law graph, rows = destinations.  Returns (indptr, indices), int32.

    Vertex ranks get Chung-Lu weights (see powerlaw_weights) summing to total_edges - n; a
    seeded permutation maps ranks to vertex ids; row v draws round(w[rank(v)]) sources with
    probability proportional to the source's weight; duplicates merge; a self-loop is added.
    """
    w = powerlaw_weights(n, float(total_edges - n), exponent, float(max_degree))
    perm = seeded_permutation(n, seed)                       # rank -> vertex id
    deg_by_rank = np.maximum(np.rint(w), 0).astype(np.int32)
    in_degree = np.empty(n, dtype=np.int32)
    in_degree[perm] = deg_by_rank
    cdf = np.cumsum(w)
    cdf /= cdf[-1]
    cdf[-1] = 1.0
    return _draw(n, in_degree, cdf, perm, seed, num_threads)


def uniform_csr(n, avg_degree, seed, num_threads=0):
    """Uniform-random graph: every row draws `avg_degree` sources uniformly, duplicates merge, a
    self-loop is added."""
    in_degree = np.full(n, int(avg_degree), dtype=np.int32)
    cdf = np.arange(1, n + 1, dtype=np.float64) / n
    cdf[-1] = 1.0
    perm = np.arange(n, dtype=np.int32)
    return _draw(n, in_degree, cdf, perm, seed, num_threads)


def community_csr(n, total_edges, exponent, max_degree, n_comm, p_in, contiguous, seed, num_threads=0):
    """Power-law graph with planted communities (rows = destinations): the degrees and the whole-graph source
    distribution of powerlaw_csr, but every draw of a row stays inside the row's community with probability `p_in`
    (sources then follow the community's own share of the same weights; rows whose degree exceeds half the
    community's size keep that many draws inside it and take the rest from the whole graph).  Rank r belongs to community r % n_comm, so
    every community has its hubs.  `contiguous`: vertex ids are community-major (a community's vertices are
    consecutive ids, in a seeded order inside it), so consecutive rows share their hot columns; otherwise ranks are
    mapped to ids by a seeded permutation of all vertices (the same graph up to relabelling).  The stand-in for the
    Reddit adjacency of benchmark/bench_vanilla_spmm.py:78-79 (41 subreddit communities), which needs a network."""
    w = powerlaw_weights(n, float(total_edges - n), exponent, float(max_degree))
    ranks = np.arange(n, dtype=np.int64)
    comm_of_rank = (ranks % n_comm).astype(np.int32)
    if contiguous:
        keys = _mix64(ranks.astype(np.uint64) ^ _mix64(np.full(n, seed, dtype=np.uint64)))
        order = np.lexsort((keys, comm_of_rank))               # ranks, community by community, seeded order inside
        perm = np.empty(n, dtype=np.int32)
        perm[order] = np.arange(n, dtype=np.int32)             # rank -> vertex id
    else:
        perm = seeded_permutation(n, seed)
    in_degree = np.empty(n, dtype=np.int32)
    in_degree[perm] = np.maximum(np.rint(w), 0).astype(np.int32)
    cdf = np.cumsum(w)
    cdf /= cdf[-1]
    cdf[-1] = 1.0
    comm_of_vertex = np.empty(n, dtype=np.int32)
    comm_of_vertex[perm] = comm_of_rank
    by_comm = np.argsort(comm_of_rank, kind="stable")          # ranks, community by community, ascending rank inside
    comm_off = np.zeros(n_comm + 1, dtype=np.int64)
    np.cumsum(np.bincount(comm_of_rank, minlength=n_comm), out=comm_off[1:])
    comm_member = np.ascontiguousarray(perm[by_comm], dtype=np.int32)
    comm_cdf = np.empty(n, dtype=np.float64)
    for c in range(n_comm):
        part = np.cumsum(w[by_comm[comm_off[c]:comm_off[c + 1]]])
        part /= part[-1]
        part[-1] = 1.0
        comm_cdf[comm_off[c]:comm_off[c + 1]] = part
    L = _lib.lib()
    args = (n, _lib.host_ptr(in_degree), _lib.host_ptr(cdf), _lib.host_ptr(perm), int(n_comm), _lib.host_ptr(comm_of_vertex),
            _lib.host_ptr(comm_off), _lib.host_ptr(comm_member), _lib.host_ptr(comm_cdf), float(p_in), int(seed), int(num_threads))
    indptr = np.zeros(n + 1, dtype=np.int32)
    _lib.check(L.fg_synth_community_csr(*args, _lib.host_ptr(indptr), None))
    indices = np.zeros(int(indptr[-1]), dtype=np.int32)
    _lib.check(L.fg_synth_community_csr(*args, _lib.host_ptr(indptr), _lib.host_ptr(indices)))
    return indptr, indices


def _draw(n, in_degree, cdf, perm, seed, num_threads):
    L = _lib.lib()
    in_degree = np.ascontiguousarray(in_degree, dtype=np.int32)
    cdf = np.ascontiguousarray(cdf, dtype=np.float64)
    perm = np.ascontiguousarray(perm, dtype=np.int32)
    indptr = np.zeros(n + 1, dtype=np.int32)
    _lib.check(L.fg_synth_powerlaw_csr(n, _lib.host_ptr(in_degree), _lib.host_ptr(cdf), _lib.host_ptr(perm),
                                       int(seed), int(num_threads), _lib.host_ptr(indptr), None))
    indices = np.zeros(int(indptr[-1]), dtype=np.int32)
    _lib.check(L.fg_synth_powerlaw_csr(n, _lib.host_ptr(in_degree), _lib.host_ptr(cdf), _lib.host_ptr(perm),
                                       int(seed), int(num_threads), _lib.host_ptr(indptr), _lib.host_ptr(indices)))
    return indptr, indices


def edge_weights(nnz, seed):
    """U[0, 1) float32 weights, one per stored edge."""
    bits = _mix64(np.arange(nnz, dtype=np.uint64) + (_mix64(np.array([seed], dtype=np.uint64))[0]))
    return ((bits >> np.uint64(40)).astype(np.float32) * np.float32(1.0 / (1 << 24))).astype(np.float32)


# Named workloads.  total_edges / max_degree are the draw targets before duplicate sources
# merge; they are set so that the merged graphs come out at about 114.6M edges with largest
# in-degree about 20k (233k nodes) and about 61.9M edges (2.45M nodes).
WORKLOADS = {
    "uniform-10k": dict(kind="uniform", n=10000, avg_degree=16),
    "powerlaw-233k": dict(kind="powerlaw", n=232965, total_edges=120_600_000, exponent=2.1, max_degree=26500),
    "powerlaw-2.45M": dict(kind="powerlaw", n=2_450_000, total_edges=61_970_000, exponent=2.5, max_degree=17600),
    "powerlaw-23k": dict(kind="powerlaw", n=23296, total_edges=1_146_000, exponent=2.1, max_degree=2000),
    # graphs of other shapes, for checking that the tiling defaults carry over (seeds of their own)
    "uniform-1M-deg64": dict(kind="uniform", n=1_000_000, avg_degree=64, seed=11),
    "powerlaw-1M-deg100-g2.5": dict(kind="powerlaw", n=1_000_000, total_edges=100_000_000, exponent=2.5, max_degree=30000, seed=12),
    # planted communities at the benchmark graph's size (41, like Reddit's subreddits; 80 % of a row's draws stay inside
    # its community): once with community-contiguous vertex ids, once with the same kind of graph randomly relabelled
    "communities-233k": dict(kind="community", n=232965, total_edges=139_600_000, exponent=2.1, max_degree=26500,
                             n_comm=41, p_in=0.8, contiguous=True, seed=14),
    "communities-233k-relabelled": dict(kind="community", n=232965, total_edges=139_600_000, exponent=2.1, max_degree=26500,
                                        n_comm=41, p_in=0.8, contiguous=False, seed=14),
    "communities-23k": dict(kind="community", n=23296, total_edges=1_300_000, exponent=2.1, max_degree=2000,
                            n_comm=8, p_in=0.8, contiguous=True, seed=15),
    # non-square: the first 100,000 destination rows of a 1M-node graph, all 1M sources
    "nonsquare-100k-x-1M": dict(kind="powerlaw", n=1_000_000, total_edges=80_000_000, exponent=2.2, max_degree=20000, seed=13,
                                rows=100_000),
}


def make_workload(name, seed=None, num_threads=0):
    """(indptr, indices) of a named workload; the number of source vertices is WORKLOADS[name]['n']."""
    spec = WORKLOADS[name]
    if seed is None:
        seed = spec.get("seed", 0xFEA7)
    if spec["kind"] == "uniform":
        indptr, indices = uniform_csr(spec["n"], spec["avg_degree"], seed, num_threads)
    elif spec["kind"] == "community":
        indptr, indices = community_csr(spec["n"], spec["total_edges"], spec["exponent"], spec["max_degree"], spec["n_comm"],
                                        spec["p_in"], spec["contiguous"], seed, num_threads)
    else:
        indptr, indices = powerlaw_csr(spec["n"], spec["total_edges"], spec["exponent"], spec["max_degree"], seed, num_threads)
    if "rows" in spec:
        indptr = indptr[:spec["rows"] + 1].copy()
        indices = indices[:indptr[-1]].copy()
    return indptr, indices
