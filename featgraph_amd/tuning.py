"""Default tiling / partitioning choices for gfx950 (MI355X: 8 XCDs, 4 MB of L2 each).

A gathered feature row is useful to an XCD only through that XCD's L2, and workgroups are
dealt to XCDs round-robin, so a kernel tile index that varies fastest with the workgroup id
gives every XCD its own slice of the feature axis.  Source-column partitions then bound how
many source rows an XCD touches per pass.  The numbers below come from sweeps on the
232,965-node / 114.8M-edge power-law graph (feature lengths 32..512).
"""

TILE_FLOATS = 64                 # feature tile per workgroup: 256 B of every gathered row
SPMM_SLICE_BYTES = 7.5e6         # per-XCD slice of X per pass (out is re-read every pass, so few passes)
SDDMM_SLICE_BYTES = 7.5e6        # same optimum measured for SDDMM: shorter row segments cost more than misses
MAX_PARTITIONS = 64


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


def _partitions(n_src, row_bytes, nnz, n_rows, slice_bytes, min_segment):
    want = (n_src * row_bytes) / slice_bytes
    if want <= 1.0:
        return 1
    p = _pow2_floor(int(want + 0.5)) if want >= 2 else 2
    # keep row segments long enough to amortise the per-row work
    avg_deg = nnz / max(1, n_rows)
    while p > 1 and avg_deg / p < min_segment:
        p //= 2
    return max(1, min(MAX_PARTITIONS, p))


def choose_spmm(n_dst, n_src, nnz, feat_len):
    """(num_col_partitions, num_feat_partitions) for an SpMM of this size."""
    t = feature_tiles(feat_len)
    if feat_len >= 2048 and feat_len % 128 == 0:
        # rows of 8 KB and more: 128-float tiles (measured at F=2048: 57.0 ms against 68.7 ms with 64-float tiles)
        t = feat_len // 128
    # more than 8 tiles are launched 8 at a time, so an XCD never holds more than one tile's slice
    row_bytes = 4 * feat_len / t if t > 1 else 4 * feat_len
    p = _partitions(n_src, row_bytes, nnz, n_dst, SPMM_SLICE_BYTES, min_segment=24)
    if p == 1 and feat_len <= 256:
        # rows too short to partition: nothing is reused through the L2 anyway, and whole rows per
        # wavefront cost the fewest index reads (measured on the 2.45M-node / 61.9M-edge graph)
        return 1, 1
    return p, (t if t > 1 else 0)


def choose_sddmm(n_rows, n_cols, nnz, heads, head_len):
    """(num_src_partitions, num_feat_tiles) for the tiled traversal, or None when the plain
    kernels should be used (small feature matrices, or a shape the tiled kernel does not take)."""
    feat_len = heads * head_len
    tile = None
    # One result per edge: 64-float tiles.  With 4 or more tiles the kernel gathers from a tile-by-tile
    # copy of the source features, and 8 partitions of 64-float tiles then beat 16 partitions of
    # 128-float tiles (232,965-node graph: 13.7 against 13.8 ms at F=512, 6.8 against 7.3 ms at F=256).
    # Several heads: a tile's results are scattered per edge, so wider tiles (more heads per write) win
    # (H=8, D=32: 8.8 ms with 128-float tiles, 9.3 ms with 64; H=8, D=64: 16.0 against 16.8 ms) unless
    # that leaves fewer than 4 tiles of whole 64-float heads (H=4, D=64: 7.7 ms, 7.3 ms with 64-float tiles).
    if heads == 1:
        order = (64, 128, 256, 32, 16)
    elif feat_len >= 256 and not (head_len >= 64 and feat_len // 128 < 4):
        order = (128, 64, 256, 32, 16)
    else:
        order = (64, 128, 256, 32, 16)
    for cand in order:
        if feat_len % cand != 0:
            continue
        if heads == 1 or cand % head_len == 0 or (head_len == cand):
            if heads > 1 and (head_len % 4 != 0 or head_len < 8 or (head_len & (head_len - 1)) != 0):
                continue
            tile = cand
            break
    if tile is None:
        return None
    t = feat_len // tile
    row_bytes = 4 * feat_len / t          # more than 8 tiles are launched 8 at a time: one tile's slice per XCD
    if n_cols * row_bytes <= SDDMM_SLICE_BYTES:
        return None
    p = _partitions(n_cols, row_bytes, nnz, n_rows, SDDMM_SLICE_BYTES, min_segment=24)
    if p > 1 and t < 8 and 8 % t == 0:
        p = max(p, 8 // t)          # at least one partition per XCD: a single launch covers them all
    if p == 1:
        # rows too short to partition: one tile per edge when the kernel takes the whole row
        if feat_len <= 256 and (feat_len & (feat_len - 1)) == 0 and feat_len >= 16 and \
                (heads == 1 or feat_len % head_len == 0):
            return 1, 1
        if t == 1:
            return None
    return p, t
