"""Default tiling / partitioning choices for gfx950 (MI355X), from a cost model in hardware terms.

What the two knobs do on this part.  The 8 XCDs have 4 MB of L2 each and are dealt workgroups
round-robin, so a feature-tile index that varies fastest with the workgroup id gives every XCD one
slice of the feature axis: T tiles of `tile` floats make a gathered row slice `4 * tile` bytes.
P source-column partitions (the reference's DDS format) bound the source rows one pass touches.
Together they set how many slices an XCD's gathers range over, n_src / P, against how many its L2
holds, L2 / (4 * tile).  The price: every tile re-reads the edge list (T edge visits per edge), every
partition cuts each row into a segment with its own start-up, read of the destination row / earlier
sums and write, and with 4 or more tiles the gathered matrix is first copied tile by tile.

The model adds those terms up for every (P, T) and takes the cheapest:

    gathered bytes  nnz * F * 4, a share h at the L1/L2-hit rate and 1 - h at the miss rate;
        h = hit rate of an LRU cache of (L2 / slice bytes) entries under the graph's own column
        reference counts (Che's approximation), over the columns of one partition;
        misses slow down with the span of memory an XCD's gathers range over;
    row segments    (non-empty (row, partition) pairs, from the degree histogram) * T * seconds each;
    edge visits     nnz * T * seconds each  (index / weight words, staging);
    streamed bytes  the output re-read and re-written per pass (SpMM); destination rows per segment
        and the per-tile partial sums (SDDMM); the tile-by-tile copy of the gathered matrix.

The coefficients are rates of this part -- bytes per second through the L1/L2-hit path, the miss path
and the streaming path, seconds per segment and per edge visit -- fitted to sweeps of P x T on five
graphs (232,965-node and 2.45M-node power-law graphs, a 1M-node uniform graph of degree 64, a 1M-node
power-law graph of degree 100, a 100k x 1M non-square graph; feature lengths 32..512).  On those
sweeps the model's choice is within 7.5 % of the best point (SpMM at F = 512 on the uniform graph:
15 %), 1-2.5 % on average; `autotune` (see the module classes' schedule argument 'tune') times the
model's best few candidates on the graph itself and keeps the fastest.
"""
import math

import numpy as np

N_XCD = 8
L2_BYTES = 4 << 20               # per XCD
COPY_BYTES_PER_S = 6.5e12        # tile_major_kernel: 477 MB read and written in 0.147 ms
MAX_PARTITIONS = 32
MIN_TILE_FLOATS = 32             # 16-float tiles cost 1.6-2x everywhere they were measured
TIE = 0.03                       # predicted times closer than this are equal: fewer tiles / partitions win

# cache: effective L2 capacity as a multiple of L2_BYTES under the independent-reference estimate (the
# gather stream has more locality than independent references, so the 4 MB behave like ~2x);
# hit / miss / stream: bytes per second; span: slow-down of misses per doubling of the gathered span beyond
# 128 MB; seg / edge: seconds per row segment and per edge visit.
SPMM_COEF = dict(cache=2.12, hit=24.0e12, miss=7.07e12, span=0.011, seg=1.64e-11, edge=1.04e-12, stream=4.15e12)
SDDMM_COEF = dict(cache=2.26, hit=23.5e12, miss=6.58e12, span=0.0, seg=3.82e-11, edge=0.0, stream=3.86e12)

# legacy names (attention module): per-XCD slice that two L2s' worth of slices add up to
SPMM_SLICE_BYTES = 7.5e6
SDDMM_SLICE_BYTES = 7.5e6
TILE_FLOATS = 64


class GraphStats(object):
    """What the model needs to know about an adjacency: sizes, how often each source column is
    referenced (as a histogram: `count_vals[i]` references occur for `count_mult[i]` columns) and the
    row degrees (same form)."""

    def __init__(self, n_dst, n_src, nnz, count_vals=None, count_mult=None, deg_vals=None, deg_mult=None):
        self.n_dst, self.n_src, self.nnz = int(n_dst), int(n_src), int(nnz)
        if count_vals is None:          # nothing known: every column referenced equally often
            count_vals, count_mult = [self.nnz / max(1, self.n_src)], [self.n_src]
        if deg_vals is None:
            deg_vals, deg_mult = [self.nnz / max(1, self.n_dst)], [self.n_dst]
        self.count_vals = np.asarray(count_vals, dtype=np.float64)
        self.count_mult = np.asarray(count_mult, dtype=np.float64)
        self.deg_vals = np.asarray(deg_vals, dtype=np.float64)
        self.deg_mult = np.asarray(deg_mult, dtype=np.float64)
        keep = self.count_vals > 0
        self.count_vals, self.count_mult = self.count_vals[keep], self.count_mult[keep]
        self._hits = {}

    @classmethod
    def from_csr(cls, indptr, indices, n_src):
        indptr = np.asarray(indptr)
        nnz = int(indptr[-1]) if len(indptr) else 0
        counts = np.bincount(np.asarray(indices), minlength=int(n_src)) if nnz else np.zeros(int(n_src), np.int64)
        cv, cm = np.unique(counts, return_counts=True)
        dv, dm = np.unique(np.diff(indptr), return_counts=True)
        return cls(len(indptr) - 1, n_src, nnz, cv, cm, dv, dm)

    def segments(self, P):
        """Expected number of non-empty (row, partition) pairs: a row of degree d spreads its elements
        over P equally likely partitions."""
        if P == 1:
            return float((self.deg_mult * (self.deg_vals > 0)).sum())
        return float((self.deg_mult * P * (1.0 - (1.0 - 1.0 / P) ** self.deg_vals)).sum())

    def hit_rate(self, entries):
        """Hit rate of an LRU cache of `entries` column slices under independent references with
        these columns' rates (Che's approximation: a slice stays for a characteristic time t with
        sum_c (1 - exp(-rate_c t)) = entries)."""
        total = float((self.count_vals * self.count_mult).sum())
        if total <= 0:
            return 0.0
        key = round(math.log2(max(entries, 1e-9)), 3)
        if key in self._hits:
            return self._hits[key]
        v, m = self.count_vals, self.count_mult
        if entries >= m.sum():
            h = 1.0 - m.sum() / total                     # only first references miss
        else:
            occupied = lambda t: float((m * -np.expm1(-v * t)).sum())
            lo, hi = 0.0, 1.0 / max(v.max(), 1e-30)
            while occupied(hi) < entries:
                hi *= 2.0
            for _ in range(50):
                mid = 0.5 * (lo + hi)
                if occupied(mid) < entries:
                    lo = mid
                else:
                    hi = mid
            h = float((v * m * -np.expm1(-v * hi)).sum() / total)
        self._hits[key] = h
        return h


def _pow2_floor(v):
    p = 1
    while p * 2 <= v:
        p *= 2
    return p


def feature_tiles(feat_len):
    """Number of feature tiles: tiles of TILE_FLOATS floats when that divides feat_len."""
    if feat_len % TILE_FLOATS == 0:
        return feat_len // TILE_FLOATS
    return 1


def padded_feature_len(feat_len):
    """The feature length the kernels should run at for rows of `feat_len` floats: the same, when it is a multiple of
    32 (tiles of 32 or 64 floats cover it) or too short to matter; else the next length that is -- a power of two up to
    64, a multiple of 32 up to 128, a multiple of 64 beyond.  Rows of any other length leave the kernels one tile and
    scalar accesses (232,965-node graph, SpMM / SDDMM in ms: F=30 1.69 / 2.69 against 0.97 / 1.11 at 32; F=100 4.18 / 6.69
    against 3.17 / 3.58 at 128; F=300 19.8 / 19.1 against 7.67 / 8.41 at 320; F=602 40.8 / 75.9 against 14.7 / 16.6 at 640);
    zero columns change neither the sums nor the dot products."""
    F = int(feat_len)
    if F < 9 or F % 32 == 0:
        return F
    if F <= 64:
        p = 16
        while p < F:
            p *= 2
        return p
    if F <= 128:
        return (F + 31) // 32 * 32
    return (F + 63) // 64 * 64


def padded_head_len(head_len):
    """The head length the multi-head kernels should run at: a power of two up to 64 or a multiple of 64 (a head then
    fills whole lane groups and tiles); other lengths are zero-padded to the next such length (232,965-node graph,
    multi-head SDDMM: 3 heads of 20 floats 26.5 ms, 8 heads of 48 floats 69 ms on the kernel that takes any shape)."""
    D = int(head_len)
    if D % 64 == 0 or (D & (D - 1)) == 0:
        return D
    if D < 64:
        p = 4
        while p < D:
            p *= 2
        return p
    return (D + 63) // 64 * 64


# Padding costs two or three passes over the feature matrices; below this many gathered floats it is not attempted.
PAD_MIN_GATHERED = 1 << 24


def copies_tile_major(n_src, feat_len, n_tiles):
    """The library's rule for gathering from a tile-by-tile copy (fg_plan_opts.tile_major = 0)."""
    xbytes = 4 * n_src * feat_len
    return n_tiles >= 4 and (64 << 20) <= xbytes < (1 << 32)


def _gather_seconds(stats, feat_len, P, T, c):
    tile_bytes = 4.0 * feat_len / T
    h = stats.hit_rate(c['cache'] * L2_BYTES / tile_bytes * P)       # entries counted over all partitions' columns
    tiled = copies_tile_major(stats.n_src, feat_len, T)
    span = stats.n_src * tile_bytes if tiled else 4.0 * stats.n_src * feat_len
    slow = 1.0 + c['span'] * max(0.0, math.log2(span / (128.0 * (1 << 20))))
    gathered = 4.0 * stats.nnz * feat_len
    t = gathered * (h / c['hit'] + (1.0 - h) * slow / c['miss'])
    t += stats.segments(P) * T * c['seg'] + stats.nnz * T * c['edge']
    if tiled:
        t += 2.0 * 4.0 * stats.n_src * feat_len / COPY_BYTES_PER_S
    return t


def predict_spmm(stats, feat_len, P, T, coef=SPMM_COEF):
    """Modelled seconds of one SpMM with P source-column partitions and T feature tiles."""
    t = _gather_seconds(stats, feat_len, P, T, coef)
    # out: one buffer written per pass and read back once by the sum (fitted as (2P - 1) when later passes re-read `out`)
    return t + 4.0 * stats.n_dst * feat_len * (2 * P - 1) / coef['stream']


def predict_sddmm(stats, feat_len, P, T, coef=SDDMM_COEF):
    """Modelled seconds of one single-head SDDMM over the tiled traversal ((1, 1): the row-order kernel)."""
    t = _gather_seconds(stats, feat_len, P, T, coef)
    t += stats.segments(P) * 4.0 * feat_len / coef['stream']                    # destination rows: once per segment
    out_bytes = 4.0 * stats.nnz * ((2 * T + 2) if T > 1 else 1)                 # per-tile partial sums: written, read, scattered
    return t + out_bytes / coef['stream']


def _candidates(feat_len, max_tile=256):
    tiles = sorted({feat_len // w for w in (32, 64, 128, 256) if feat_len % w == 0 and w <= max_tile and feat_len // w >= 1} | {1})
    tiles = [t for t in tiles if t == 1 or feat_len // t >= MIN_TILE_FLOATS]
    parts = [p for p in (1, 2, 4, 8, 16, 32) if p <= MAX_PARTITIONS]
    return [(p, t) for p in parts for t in tiles]


def _rank(stats, feat_len, predict, cands, tie_key):
    timed = sorted(((predict(stats, feat_len, p, t), p, t) for p, t in cands))
    if not timed:
        return []
    best = timed[0][0]
    near = sorted(((s, p, t) for s, p, t in timed if s <= best * (1.0 + TIE)), key=lambda e: tie_key(e[1], e[2]) + (e[0],))
    rest = [(s, p, t) for s, p, t in timed if s > best * (1.0 + TIE)]
    return [(p, t) for s, p, t in near] + [(p, t) for s, p, t in rest]


# predicted times within TIE of the best: SpMM takes fewer tiles (fewer passes over the edge list), SDDMM fewer
# partitions (fewer reads of the destination rows)
_spmm_tie = lambda p, t: (t, p)
_sddmm_tie = lambda p, t: (p, t)


def rank_spmm(stats, feat_len):
    """(num_col_partitions, num_feat_partitions) candidates, most promising first."""
    cands = [(p, t) for p, t in _candidates(feat_len) if p <= max(1, stats.n_src)]
    if feat_len > 256:
        cands = [(p, t) for p, t in cands if t > 1]          # rows wider than 256 floats are always tiled
    return _rank(stats, feat_len, predict_spmm, cands, _spmm_tie)


def rank_sddmm(stats, feat_len):
    """(num_src_partitions, num_feat_tiles) candidates of the tiled traversal, most promising first;
    (1, 1) stands for the plain row-order kernel."""
    cands = [(p, t) for p, t in _candidates(feat_len) if not (t == 1 and p > 1 and feat_len > 256)]
    return _rank(stats, feat_len, predict_sddmm, cands, _sddmm_tie)


def choose_spmm(n_dst, n_src, nnz, feat_len, stats=None):
    """(num_col_partitions, num_feat_partitions) for an SpMM of this size (num_feat_partitions 0:
    the kernel's own single tile).  `stats`: GraphStats of the adjacency; without them every column
    counts as equally referenced and every row as of average degree."""
    if nnz == 0 or n_dst == 0:
        return 1, 0
    if stats is None:
        stats = GraphStats(n_dst, n_src, nnz)
    if feat_len >= 2048 and feat_len % 128 == 0:
        # rows of 8 KB and more: 128-float tiles (measured at F=2048: 57.0 ms against 68.7 ms with 64-float tiles)
        cands = [(p, feat_len // 128) for p in (1, 2, 4, 8, 16, 32)]
        p, t = _rank(stats, feat_len, predict_spmm, cands, _spmm_tie)[0]
        return p, t
    ranked = rank_spmm(stats, feat_len)
    if not ranked:
        return 1, 0
    p, t = ranked[0]
    if p == 1 and t == 1:
        return 1, 1
    return p, (t if t > 1 else 0)


# The broadcasting kernel reduces one row segment after the other, all lane groups on the same segment, where the
# weighted-sum kernel gives short segments a lane group each: a segment costs it a few tenths of a nanosecond of
# machine time more.  With this coefficient the choice was the fastest or within 3 % of it on the 233k-node graph
# (u_add_e with one weight per edge, ms at 1 / 2 / 4 / 8 / 16 partitions: F=32 1.30 / 1.20 / 1.22 / 1.38 / 1.98,
# F=64 3.02 / - / 2.14 / 2.20 / 2.56, F=128 6.58 / 5.95 / 4.99 / 4.14 / 4.38, F=256 15.7 / 14.1 / 12.3 / 10.2 / 8.87;
# u_mul_e with [nnz, F] edge features: F=64 6.87 / - / 6.19 / 6.66 / 7.23, F=128 14.4 / 13.7 / 12.7 / 13.1 / 14.1).
BCAST_COEF = dict(SPMM_COEF, seg=4.5e-10)
# ... and per tile when the feature axis is tiled (u_add_e, F=256 in 4 tiles: 12.8 / 11.2 / 9.21 / 7.83 / 9.54 ms at 1 / 2 / 4 / 8 / 16
# partitions; F=128 in 2 tiles: 6.03 / 5.16 / 4.04 / 4.08 / 4.93)
BCAST_TILED_COEF = dict(SPMM_COEF, seg=2.0e-10)


def choose_gather_partitions(n_dst, n_src, nnz, gathered_len, out_len, stats=None, tiles=1):
    """Source-column partitions for a generalised SpMM whose gathered operand has `gathered_len` floats per source
    node and whose result has `out_len` per destination, with the feature axis in `tiles` tiles (the library's own
    choice: 64-float tiles from 128 features on, when the 128-bit paths apply); every partition's results take a
    buffer of their own (8 GiB at most)."""
    if nnz == 0 or n_dst == 0 or gathered_len < 1:
        return 1
    if stats is None:
        stats = GraphStats(n_dst, n_src, nnz)
    tiles = max(1, int(tiles))
    cands = [(p, tiles) for p in (1, 2, 4, 8, 16, 32)
             if p <= min(MAX_PARTITIONS, max(1, n_src)) and (p == 1 or 4.0 * p * n_dst * out_len <= float(8 << 30))]
    coef = BCAST_TILED_COEF if tiles > 1 else BCAST_COEF
    predict = lambda st, f, p, t: predict_spmm(st, f, p, t, coef)
    return _rank(stats, gathered_len, predict, cands, _spmm_tie)[0][0]


def choose_sddmm(n_rows, n_cols, nnz, heads, head_len, stats=None):
    """(num_src_partitions, num_feat_tiles) for the tiled traversal, or None when the plain
    kernels should be used (small feature matrices, or a shape the tiled kernel does not take)."""
    feat_len = heads * head_len
    if heads == 1:
        if nnz == 0 or feat_len % 4 != 0:
            return None
        if stats is None:
            stats = GraphStats(n_rows, n_cols, nnz)
        if 4.0 * n_cols * feat_len <= N_XCD * L2_BYTES / 4:
            return None                                # the whole operand sits in every L2: nothing to tile
        ranked = [(p, t) for p, t in rank_sddmm(stats, feat_len)
                  if feat_len // t <= 256 and _is_pow2(feat_len // t) and feat_len // t >= 16]
        if not ranked or ranked[0][0] == 1:
            # No source partitions: the stored-order kernels.  Without partitions the traversal has no slice to keep in
            # the L2s and still pays for its partial sums and the scatter to the stored order (measured: 2-8 % behind at
            # 1 x 1; 2.45M-node graph at F = 512: 1 x 2 tiles 22.5 ms, stored order 20.1 ms; uniform 1M-node graph: 23.3 / 22.7 ms).
            return None
        return ranked[0]
    return _choose_sddmm_heads(n_rows, n_cols, nnz, heads, head_len)


def _is_pow2(v):
    return v > 0 and (v & (v - 1)) == 0


def _partitions(n_src, row_bytes, nnz, n_rows, slice_bytes, min_segment):
    """Partitions that bring an XCD's slice of the gathered rows down to `slice_bytes` while row
    segments keep `min_segment` elements on average (the rule the multi-head and attention operators use)."""
    want = (n_src * row_bytes) / slice_bytes
    if want <= 1.0:
        return 1
    p = _pow2_floor(int(want + 0.5)) if want >= 2 else 2
    avg_deg = nnz / max(1, n_rows)
    while p > 1 and avg_deg / p < min_segment:
        p //= 2
    return max(1, min(64, p))


def _choose_sddmm_heads(n_rows, n_cols, nnz, heads, head_len):
    """Several heads per edge.  What an (edge, tile) pair writes decides the tile: the memory system writes whole 32-byte
    sectors, so a tile that holds fewer than 8 heads and scatters them to `out` pays a sector for its 8 or 16 bytes
    (232,965-node graph, counted at the fabric: 8.0 GB written for 3.67 GB of results at H=8, D=32 with 128-float tiles,
    16.2 GB at H=8, D=64).  Hence
      * heads of up to 32 floats, 8 or more of them: 256-float tiles (8 or more heads, 32 bytes or more per edge and
        tile, written where they belong) -- H=8, D=32: 8.64 -> 7.71 ms with one tile x 32 partitions;
      * longer heads: one head per tile, each tile's results kept in traversal order (whole runs) and every edge's H
        results written as one run by a last kernel -- H=8, D=64: 15.2 -> 13.4 ms with 8 tiles x 8 partitions;
      * fewer than 8 short heads: 64-float tiles as before (H=4, D=32: one 128-float tile is no faster).
    Partitions: two L2s' worth of slices per XCD, segments of 24 elements or more (12 for the 256-float tiles, whose
    slices need four times the partitions: 7.7 ms at 32 partitions against 8.4 at 16)."""
    feat_len = heads * head_len
    if head_len % 4 != 0 or head_len < 8 or (head_len & (head_len - 1)) != 0:
        return None
    min_segment = 24
    if head_len <= 32 and heads >= 8 and feat_len % 256 == 0:
        tile, min_segment = 256, 12
    elif head_len in (64, 128) and feat_len >= 256:
        tile = head_len
    else:
        tile = None
        for cand in (64, 128, 256, 32, 16):
            if feat_len % cand == 0 and (cand % head_len == 0 or head_len == cand):
                tile = cand
                break
        if tile is None:
            return None
    t = feat_len // tile
    row_bytes = 4 * feat_len / t          # more than 8 tiles are launched 8 at a time: one tile's slice per XCD
    if n_cols * row_bytes <= SDDMM_SLICE_BYTES:
        return None
    p = _partitions(n_cols, row_bytes, nnz, n_rows, SDDMM_SLICE_BYTES, min_segment=min_segment)
    if p > 1 and t < 8 and 8 % t == 0 and p < 8 // t:
        # at least one partition per XCD (a single launch covers them all) -- unless that leaves the segments too short
        p = 8 // t if nnz / max(1, n_rows) / (8 // t) >= min_segment else 1
    if p == 1:
        if feat_len <= 256 and (feat_len & (feat_len - 1)) == 0 and feat_len >= 16 and feat_len % head_len == 0:
            return 1, 1
        if t == 1:
            return None
    return p, t
