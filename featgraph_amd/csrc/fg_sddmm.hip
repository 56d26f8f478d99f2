// Edge-wise dot products (SDDMM) for gfx950, single- and multi-head:
//   out[e, h] = sum_{d<D} src[col[e], h, d] * dst[row[e], h, d]
//
// Edge-parallel: a wavefront owns a run of consecutive stored edges.  A group of L lanes
// covers one edge's F = H*D floats with K vector loads per operand, the 64/L groups work on
// different edges at once, and each head's products are added across its lanes with a
// butterfly of cross-lane shuffles.  Row/column ids are staged in LDS (up to 256 edges per
// wavefront), results are collected in registers and written back as dense runs.  When the
// stored order keeps equal row ids together (CSR order, 2-D partitioned order) the dst row
// already held in registers is reused instead of fetched again.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "fg_common.h"
#include "fg_device.h"

using fg::fail;
using fg::Item;
using fg::dpp_move;
using fg::wave_lds_sync;

namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kBlock = 64 * kWavesPerBlock;
constexpr int kEdgesPerWave = 256;       // COO kernel: stored edges per wavefront
constexpr int kMaxHeadsFast = 16;        // most heads the lane layouts below cover (4 loads x 4 heads)

template <int V> struct Vec;
template <> struct Vec<4> { using type = float4; };
template <> struct Vec<1> { using type = float; };

__device__ __forceinline__ float vdot(const float4 &a, const float4 &b) {
    return a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w;
}
__device__ __forceinline__ float vdot(const float &a, const float &b) { return a * b; }
__device__ __forceinline__ float4 vzero4() { return make_float4(0.f, 0.f, 0.f, 0.f); }

// Sum over the RW consecutive lanes of a head segment; every lane of the segment gets it.
// Inside a 16-lane row the butterfly runs on DPP moves: swap neighbours, swap pairs, mirror
// the half row (the other quad's sum), mirror the row (the other half's sum); only the 32- and
// 64-lane steps go through the LDS crossbar.
template <int RW>
__device__ __forceinline__ float segment_sum(float v) {
    if (RW >= 2) v += dpp_move<0xB1>(v);     // quad_perm [1,0,3,2]
    if (RW >= 4) v += dpp_move<0x4E>(v);     // quad_perm [2,3,0,1]
    if (RW >= 8) v += dpp_move<0x141>(v);    // row_half_mirror
    if (RW >= 16) v += dpp_move<0x140>(v);   // row_mirror
    if (RW >= 32) v += __shfl_xor(v, 16);
    if (RW >= 64) v += __shfl_xor(v, 32);
    return v;
}

struct SddmmArgs {
    const int32_t *row;     // COO kernel: row id per stored edge
    const int32_t *col;     // column id per stored edge
    const Item *items;      // CSR kernel: plan items
    int64_t n_items;
    const int32_t *pos;     // CSR kernel: row boundaries (indptr)
    int64_t n_edges;
    const float *src;       // gathered by col
    const float *dst;       // gathered by row
    float *out;             // [E, H]
    int F;                  // H * D
};

// Layout of one edge over its group of L lanes: lane li, load k covers floats
// [k*L*V + li*V, +V).  A head is RW lanes wide inside one load (KH == 1, L/RW heads per
// load) or spans KH whole loads (RW == L).  Heads per edge: (L / RW) * (K / KH).
template <int V, int L, int K, int RW, int KH>
struct Shape {
    using vec = typename Vec<V>::type;
    static constexpr int G = 64 / L;
    static constexpr int HPL = L / RW;          // heads per load
    static constexpr int NH = K / KH;           // head groups along k
    static constexpr int H = HPL * NH;
};

// dot products of one edge's operands, reduced per head; result valid in every lane of the
// head's segment, for head group kk in q[kk].
template <int V, int L, int K, int RW, int KH, bool FULL>
__device__ __forceinline__ void edge_heads(const typename Vec<V>::type (&s)[K], const typename Vec<V>::type (&d)[K],
                                           const bool (&on)[K], float (&q)[K / KH]) {
#pragma unroll
    for (int kk = 0; kk < K / KH; ++kk) {
        float p = 0.f;
#pragma unroll
        for (int k = kk * KH; k < (kk + 1) * KH; ++k)
            if (FULL || on[k]) p += vdot(s[k], d[k]);
        q[kk] = segment_sum<RW>(p);
    }
}

// Dot products of the staged edges [0, n) of `edge` (x = column id, y = row id); results go to
// out[j * H + head] for staged edge j.  The G lane groups take edges g, g+G, ...; U steps' src
// loads are issued back to back.  Per-head results are collected in registers -- the lane
// whose position in its head segment equals the step number (mod RW) keeps that step's value
// -- and written out every RW steps as one dense run of RW*G*H floats.
template <int V, int L, int K, int RW, int KH, bool FULL>
__device__ __forceinline__ void sddmm_staged(const int2 *edge, int n, int g, int li, const float *sb,
                                             const float *db, int64_t F, const bool (&on)[K], float *out,
                                             int32_t &held_row, typename Vec<V>::type (&dv)[K]) {
    using S = Shape<V, L, K, RW, KH>;
    using vec = typename S::vec;
    constexpr int G = S::G, H = S::H, NH = S::NH;
    constexpr int U = (K >= 2) ? 2 : 4;
    const int seg_pos = li % RW, head0 = li / RW;
    (void)held_row;
    float res[NH];
#pragma unroll
    for (int kk = 0; kk < NH; ++kk) res[kk] = 0.f;
    const int nsteps = (n + G - 1) / G;
    for (int s0 = 0; s0 < nsteps; s0 += U) {
        int2 rc[U];
        vec sv[U][K], dw[U][K];
        // no load sits under a branch: a group without an edge in this step re-reads the last edge
        // (its result is not stored), and both operands are fetched for every edge -- when the row
        // repeats, the destination row comes from the cache
#pragma unroll
        for (int u = 0; u < U; ++u) rc[u] = edge[min((s0 + u) * G + g, n - 1)];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int k = 0; k < K; ++k)
                if (FULL || on[k]) {
                    sv[u][k] = *reinterpret_cast<const vec *>(sb + (int64_t)rc[u].x * F + k * L * V);
                    dw[u][k] = *reinterpret_cast<const vec *>(db + (int64_t)rc[u].y * F + k * L * V);
                }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int step = s0 + u;
            if (step < nsteps) {                       // uniform
#pragma unroll
                for (int k = 0; k < K; ++k) dv[k] = dw[u][k];
                float q[NH];
                edge_heads<V, L, K, RW, KH, FULL>(sv[u], dv, on, q);
                if ((step % RW) == seg_pos) {
#pragma unroll
                    for (int kk = 0; kk < NH; ++kk) res[kk] = q[kk];
                }
                if ((step % RW) == RW - 1 || step == nsteps - 1) {   // uniform: write the collected block
                    const int my_step = (step / RW) * RW + seg_pos;
                    const int j = my_step * G + g;
                    if (my_step <= step && j < n) {
#pragma unroll
                        for (int kk = 0; kk < NH; ++kk) out[(int64_t)j * H + kk * S::HPL + head0] = res[kk];
                    }
                }
            }
        }
    }
}

// Stored-order (COO) kernel: a wavefront takes kEdgesPerWave consecutive stored edges.
template <int V, int L, int K, int RW, int KH, bool FULL>
__global__ __launch_bounds__(kBlock) void sddmm_coo_kernel(const SddmmArgs a) {
    using S = Shape<V, L, K, RW, KH>;
    using vec = typename S::vec;
    constexpr int H = S::H;
    static_assert(kEdgesPerWave <= fg::kItemEdges, "staging row too small");
    __shared__ int2 s_edge[kWavesPerBlock][fg::kItemEdges];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane / L, li = lane % L;
    const int64_t e_begin = ((int64_t)blockIdx.x * kWavesPerBlock + wave) * kEdgesPerWave;
    if (e_begin >= a.n_edges) return;
    const int n = (int)min((int64_t)kEdgesPerWave, a.n_edges - e_begin);
    bool on[K];
#pragma unroll
    for (int k = 0; k < K; ++k) on[k] = FULL || (k * L * V + li * V < a.F);
    int2 *edge = s_edge[wave];
    for (int t = lane; t < n; t += 64) edge[t] = make_int2(a.col[e_begin + t], a.row[e_begin + t]);
    wave_lds_sync();
    int32_t held_row = -1;
    vec dv[K];
#pragma unroll
    for (int k = 0; k < K; ++k) dv[k] = vec();
    sddmm_staged<V, L, K, RW, KH, FULL>(edge, n, g, li, a.src + li * V, a.dst + li * V, a.F, on,
                                        a.out + e_begin * H, held_row, dv);
}

// CSR-order kernel over plan items: a run of whole rows, one row, or a piece of a long row.
template <int V, int L, int K, int RW, int KH, bool FULL>
__global__ __launch_bounds__(kBlock) void sddmm_csr_kernel(const SddmmArgs a) {
    using S = Shape<V, L, K, RW, KH>;
    using vec = typename S::vec;
    constexpr int H = S::H;
    __shared__ int2 s_edge[kWavesPerBlock][fg::kItemEdges];
    __shared__ int32_t s_end[kWavesPerBlock][fg::kItemRows];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane / L, li = lane % L;
    const int64_t item_id = (int64_t)blockIdx.x * kWavesPerBlock + wave;
    if (item_id >= a.n_items) return;
    const Item it = a.items[item_id];
    if (it.len == 0) return;
    bool on[K];
#pragma unroll
    for (int k = 0; k < K; ++k) on[k] = FULL || (k * L * V + li * V < a.F);
    int2 *edge = s_edge[wave];
    int32_t held_row = -1;
    vec dv[K];
#pragma unroll
    for (int k = 0; k < K; ++k) dv[k] = vec();
    const float *sb = a.src + li * V, *db = a.dst + li * V;

    if (it.info < -1) {
        // several whole rows: the row of staged edge t is the first row whose end exceeds t
        const int nrows = -it.info;
        if (lane < nrows) s_end[wave][lane] = a.pos[it.row + lane + 1] - it.start;
        wave_lds_sync();
        for (int t = lane; t < it.len; t += 64) {
            int lo = 0, hi = nrows - 1;
            while (lo < hi) { const int mid = (lo + hi) >> 1; if (s_end[wave][mid] > t) hi = mid; else lo = mid + 1; }
            edge[t] = make_int2(a.col[it.start + t], it.row + lo);
        }
        wave_lds_sync();
        sddmm_staged<V, L, K, RW, KH, FULL>(edge, it.len, g, li, sb, db, a.F, on, a.out + (int64_t)it.start * H,
                                            held_row, dv);
        return;
    }
    for (int32_t base = 0; base < it.len; base += fg::kItemEdges) {
        const int n = min(fg::kItemEdges, it.len - base);
        wave_lds_sync();
        for (int t = lane; t < n; t += 64) edge[t] = make_int2(a.col[it.start + base + t], it.row);
        wave_lds_sync();
        sddmm_staged<V, L, K, RW, KH, FULL>(edge, n, g, li, sb, db, a.F, on,
                                            a.out + ((int64_t)it.start + base) * H, held_row, dv);
    }
}

// ---- feature-tiled, source-column-partitioned traversal ---------------------------------------
//
// For graphs whose feature matrices do not fit the L2 caches.  The edge list is a DDS copy of
// the adjacency (column partition by column partition, CSR inside a partition) and the feature
// axis is cut into tiles of L*K*4 floats; workgroup id = item block * n_tiles + tile, so the 8
// XCDs (dealt workgroups round-robin) work on the same edges but different tiles and each L2
// holds one tile's slice of one partition's src rows.  A head (RW lanes) must lie inside a tile.
// One head per edge in total means the tiles hold partial dot products: they go to
// partial[tile][e'] and sddmm_tile_sum_kernel adds them; with whole heads per tile the results
// go straight to out.  Results are scattered to the caller's edge order through edge_pos.

constexpr int kMaxGroups = 32;
struct SddmmTiledArgs {
    const Item *items;        // all partitions' items
    const int64_t *item_off;  // [n_parts + 1]: partition p owns items [item_off[p], item_off[p + 1])
    const int32_t *pos;       // row boundaries, one array of pos_stride entries per partition
    int64_t pos_stride;
    const int32_t *col;       // partition-local column ids, DDS order
    const uint16_t *col16;    // the plan's 16-bit copy of `col`, read instead of it (null: none)
    const int32_t *edge_pos;  // DDS position -> position in the caller's edge order
    const float *src;         // partition p's first src row is src + p * src_stride
    int64_t src_stride;
    // 32-bit offsets only.  Bytes between consecutive src rows, and, when the tiles of src are
    // stored one after the other ([tile][row][tile floats]), the bytes from one tile's block to
    // the next; 0: rows of F floats that hold all tiles.
    uint32_t src_row_bytes;
    uint32_t src_tile_bytes;
    int first_part, conc, n_parts;   // this launch works on partitions [first_part, first_part + conc)
    // n_groups > 0: one launch walks all partitions, `conc` of them at a time: group g holds partitions
    // [g * conc, (g + 1) * conc) and the item blocks [group_off[g], group_off[g + 1]) of the grid
    int n_groups;
    int64_t group_off[kMaxGroups + 1];
    int tile_base;                   // ... and on tiles [tile_base, tile_base + n_tiles)
    const float *dst;
    float *out;               // out (direct mode) or partial (tile-sum mode)
    int64_t out_edge_stride;  // floats between consecutive edges in out
    int64_t out_tile_stride;  // floats between consecutive tiles in out
    int F;
    int n_tiles;
};

// One batch: U edges of one row for this lane group (edge j0 + u*jstride, u < U, those below
// `e`), all U*K src loads issued back to back; lanes without an edge re-read edge e-1.  Every
// head's U results end up one per lane (lane position u of the head segment keeps result u) and
// are stored by those lanes.
constexpr int kTilePad = 8;   // staging slots past the last edge that the unclamped walk may read
// STAGE: a result goes to a word of its edge's staging slot instead of to `out`, and the kernel writes the item's results
// from there in whole runs: 1 = the .y word (results in traversal order; the positions are not needed), 2 = the .x word
// (the column word, which is dead once the batch's gathers are issued; .y keeps the position the result goes to).
template <int L, int K, int RW, int KH, int U, bool SCATTER, bool OFF32, bool CLAMP, bool ALLVALID = false, int STAGE = 0>
__device__ __forceinline__ void sddmm_tile_batch(const int2 *edge, int j0, int jstride, int e, const float *src,
                                                 uint32_t lane_bytes, int64_t F, const float4 (&dv)[K], float *out,
                                                 int64_t estride, int64_t e_base, int seg_pos) {
    static_assert(U <= RW, "one result per lane of a head segment");
    constexpr int NH = K / KH, HPL = L / RW;
    int2 ce[U];
    float4 sv[U][K];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int j = j0 + u * jstride;
        // !CLAMP (consecutive edges): slots past the row's end hold later rows' edges or the
        // padding -- loadable, and their results are not stored
        ce[u] = edge[(!CLAMP || ALLVALID || j < e) ? j : e - 1];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const char *base = reinterpret_cast<const char *>(src);
#pragma unroll
        for (int k = 0; k < K; ++k)
            sv[u][k] = OFF32 ? *reinterpret_cast<const float4 *>(base + ((uint32_t)ce[u].x + lane_bytes) + k * L * 16)
                             : *reinterpret_cast<const float4 *>(base + (int64_t)ce[u].x * F * 4 + lane_bytes + k * L * 16);
    }
    if constexpr (RW == 16 && U == 8 && K == 1 && KH == 1) {
        // Eight dot products over 16 lanes with 22 operations instead of 8 x 4: at every step a
        // lane keeps half of its values and hands the other half to its partner (lanes 15-i,
        // 7-i, i^2, then i^1), so the result of edge u ends in the two lanes whose position in
        // the segment is 2u and 2u+1.
        float p[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) p[u] = vdot(sv[u][0], dv[0]);
        const bool k3 = (seg_pos & 8) != 0, k2 = (seg_pos & 4) != 0, k1 = (seg_pos & 2) != 0;
        float q[4], r[2];
#pragma unroll
        for (int i = 0; i < 4; ++i) q[i] = (k3 ? p[4 + i] : p[i]) + dpp_move<0x140>(k3 ? p[i] : p[4 + i]);   // row_mirror
#pragma unroll
        for (int i = 0; i < 2; ++i) r[i] = (k2 ? q[2 + i] : q[i]) + dpp_move<0x141>(k2 ? q[i] : q[2 + i]);   // row_half_mirror
        float t = (k1 ? r[1] : r[0]) + dpp_move<0x4E>(k1 ? r[0] : r[1]);                                    // quad_perm [2,3,0,1]
        t += dpp_move<0xB1>(t);                                                                             // quad_perm [1,0,3,2]
        const int u_mine = seg_pos >> 1;
        const int ju = j0 + u_mine * jstride;
        if ((seg_pos & 1) == 0 && (ALLVALID || ju < e)) {
            if constexpr (STAGE == 1) {
                const_cast<int2 *>(edge)[ju].y = __float_as_int(t);
            } else if constexpr (STAGE == 2) {
                const_cast<int2 *>(edge)[ju].x = __float_as_int(t);
            } else {
                const int64_t at = SCATTER ? (int64_t)edge[ju].y : e_base + ju;
                out[at * estride] = t;
            }
        }
        return;
    }
    float mine[NH];
    int my_pos = 0;
#pragma unroll
    for (int kk = 0; kk < NH; ++kk) mine[kk] = 0.f;
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int kk = 0; kk < NH; ++kk) {
            float p = 0.f;
#pragma unroll
            for (int k = kk * KH; k < (kk + 1) * KH; ++k) p += vdot(sv[u][k], dv[k]);
            p = segment_sum<RW>(p);
            if (seg_pos == u) mine[kk] = p;
        }
        if (seg_pos == u) my_pos = ce[u].y;
    }
    const int ju = j0 + seg_pos * jstride;
    if (seg_pos < U && (ALLVALID || ju < e)) {
        if constexpr (STAGE == 1) {
            static_assert(STAGE != 1 || (NH == 1 && HPL == 1 && !SCATTER), "one result per edge and tile");
            const_cast<int2 *>(edge)[ju].y = __float_as_int(mine[0]);
        } else if constexpr (STAGE == 2) {
            static_assert(STAGE != 2 || (NH == 1 && HPL == 1 && SCATTER), "one result per edge");
            const_cast<int2 *>(edge)[ju].x = __float_as_int(mine[0]);
        } else {
            const int64_t at = SCATTER ? (int64_t)my_pos : e_base + ju;
#pragma unroll
            for (int kk = 0; kk < NH; ++kk) out[at * estride + kk * HPL] = mine[kk];
        }
    }
}

// The last, partly filled batch of a row: exactly `nu` steps (1 <= nu <= U, uniform over the
// wavefront) are loaded and reduced, instead of U steps padded with re-reads of the last edge --
// a re-read costs the same cache bandwidth as a gather.
template <int L, int K, int RW, int KH, int NU, bool SCATTER, bool OFF32, int STAGE = 0>
__device__ __forceinline__ void sddmm_tile_tail(int nu, const int2 *edge, int j0, int jstride, int e, const float *src,
                                                uint32_t lane_bytes, int64_t F, const float4 (&dv)[K], float *out,
                                                int64_t estride, int64_t e_base, int seg_pos) {
    if (nu >= NU) {
        sddmm_tile_batch<L, K, RW, KH, NU, SCATTER, OFF32, true, false, STAGE>(edge, j0, jstride, e, src, lane_bytes, F, dv, out, estride,
                                                                  e_base, seg_pos);
        return;
    }
    if constexpr (NU > 1)
        sddmm_tile_tail<L, K, RW, KH, NU - 1, SCATTER, OFF32, STAGE>(nu, edge, j0, jstride, e, src, lane_bytes, F, dv, out, estride,
                                                              e_base, seg_pos);
}

// L lanes x K loads cover one tile of L*K*4 floats of an edge's operands; RW lanes per head inside
// one load (KH == 1) or a head spanning KH loads (RW == L).
template <int L, int K, int RW, int KH, bool SCATTER, bool OFF32>
__global__ __launch_bounds__(kBlock) void sddmm_tiled_kernel(const SddmmTiledArgs a) {
    constexpr int G = 64 / L;
    constexpr int U = (RW < 8 ? RW : 8) / (K >= 2 ? 2 : 1) > 0 ? (RW < 8 ? RW : 8) / (K >= 2 ? 2 : 1) : 1;
    // One result per edge and tile, written in traversal order: the results of an item (or of 256 elements of a long row)
    // are collected in the staging row's unused position words and written from there as whole runs of consecutive floats,
    // instead of 4 bytes per lane from every batch (which reached memory as partly filled 64-byte blocks).
    // Results that are scattered to stored positions take the column words instead, where the whole wavefront walks one row
    // at a time; where lane groups walk rows of their own a group may still read a later row's column words, so those items
    // keep storing 4 bytes per lane.
    constexpr bool ONE = K == KH && RW == L;
    constexpr int STAGE = ONE ? (SCATTER ? 2 : 1) : 0;
    constexpr int STAGE_OWN_ROWS = STAGE == 1 ? 1 : 0;
    static_assert(U <= kTilePad, "unclamped reads must stay inside the padded staging row");
    __shared__ __align__(16) int2 s_edge[kWavesPerBlock][fg::kItemEdges + kTilePad];     // x = column word, y = edge_pos
    __shared__ int32_t s_end[kWavesPerBlock][fg::kItemRows];
    __shared__ int32_t s_next[kWavesPerBlock];
    __shared__ __align__(16) float4 s_dst[kWavesPerBlock][128 * K];      // destination slices of an item with few rows

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane / L, li = lane % L;
    // workgroup id = (item block, partition in flight, tile), tile fastest: with n_tiles * conc == 8
    // every XCD works on one tile of one partition
    const unsigned per = (unsigned)(a.n_tiles * a.conc);
    const int slot = (int)(blockIdx.x % per);
    const int tile = a.tile_base + slot % a.n_tiles;
    int part = a.first_part + slot / a.n_tiles;
    int64_t item_block = blockIdx.x / per;
    if (a.n_groups > 0) {
        // the group of partitions this workgroup belongs to (uniform): groups follow each other in the grid
        int grp = 0;
        while (grp + 1 < a.n_groups && item_block >= a.group_off[grp + 1]) ++grp;
        part = grp * a.conc + slot / a.n_tiles;
        item_block -= a.group_off[grp];
    }
    if (part >= a.n_parts) return;
    const int64_t i0 = a.item_off[part];
    const int64_t item_id = item_block * kWavesPerBlock + wave;
    if (item_id >= a.item_off[part + 1] - i0) return;
    const Item it = a.items[i0 + item_id];
    const int32_t *pos = a.pos + part * a.pos_stride;
    const float *src = a.src + part * a.src_stride;
    if (it.len == 0) return;
    const int64_t F = a.F;
    const int f_lo = tile * (L * K * 4) + li * 4;
    const uint32_t lane_bytes = (OFF32 && a.src_tile_bytes) ? (uint32_t)tile * a.src_tile_bytes + (uint32_t)li * 16u
                                                            : (uint32_t)f_lo * 4u;
    const uint32_t scale = OFF32 ? a.src_row_bytes : 1u;
    const float *db = a.dst + f_lo;
    const int seg_pos = li % RW;
    float *out = a.out + (int64_t)tile * a.out_tile_stride + li / RW;
    int2 *edge = s_edge[wave];
    float4 dv[K];

    auto stage = [&](int64_t base, int n) {
        // lane l holds edges 4l .. 4l + 3 (past the end: the last edge again)
        int32_t c[4], at[4] = {0, 0, 0, 0};
        fg::load_four_ids(a.col, a.col16, base, n, lane, c);
        if (SCATTER) fg::load_four(a.edge_pos + base, n, lane, 1, at);
#pragma unroll
        for (int i = 0; i < 4; ++i) c[i] = (int)((uint32_t)c[i] * scale);
        int4 *e4 = reinterpret_cast<int4 *>(edge);
        e4[2 * lane] = make_int4(c[0], at[0], c[1], at[1]);
        e4[2 * lane + 1] = make_int4(c[2], at[2], c[3], at[3]);
        if (lane < kTilePad) edge[fg::kItemEdges + lane] = make_int2(c[3], at[3]);
    };
    // the staged results of elements [0, n) of the staging row go to out[e_base ..]
    auto flush = [&](int64_t e_base, int n) {
        wave_lds_sync();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int j = lane + 64 * i;
            if (j < n) {
                const int2 w = edge[j];
                if (STAGE == 2) out[(int64_t)w.y * a.out_edge_stride] = __int_as_float(w.x);
                else out[(e_base + j) * a.out_edge_stride] = __int_as_float(w.y);
            }
        }
    };
    auto load_dst = [&](int64_t row) {
#pragma unroll
        for (int k = 0; k < K; ++k) dv[k] = *reinterpret_cast<const float4 *>(db + row * F + k * L * 4);
    };

    if (it.info < -1) {
        const int nrows = -it.info;
        if (nrows < 2 * G) {
            // Few, longer rows: all lane groups share each row in turn.  The rows' destination slices (fewer than
            // 128 * K 128-bit words) are read once here, together with the staging loads, and kept in LDS: a slice
            // fetched at the moment its row starts would sit in front of that row's gathers (loads return in order),
            // and one that was only touched here has left the L2 again by the time a later row of the item needs it.
            constexpr int RV = L * K;                    // 128-bit words per row slice
            float4 held[2 * K];
            // With one partition in flight nobody else reads these slices before they have left the caches: non-temporal
            // loads then keep them from displacing the gathered operand's rows (232,965-node graph, F=512, 8 tiles: 13.22 ->
            // 13.03 ms).  With several partitions in flight (fewer than 8 tiles) the other partitions' workgroups read the same
            // rows at about the same time, through the memory-side cache, and plain loads are 1-2.5 % faster.
            const bool stream_dst = a.conc == 1;
            typedef float f4 __attribute__((ext_vector_type(4)));
#pragma unroll
            for (int i = 0; i < 2 * K; ++i) {
                const int t = lane + 64 * i;
                const int r = min(t / RV, nrows - 1);
                const float *at = a.dst + (int64_t)(it.row + r) * F + tile * (RV * 4) + (t % RV) * 4;
                if (stream_dst) {
                    const f4 hv = __builtin_nontemporal_load(reinterpret_cast<const f4 *>(at));
                    held[i] = make_float4(hv.x, hv.y, hv.z, hv.w);
                } else {
                    held[i] = *reinterpret_cast<const float4 *>(at);
                }
            }
            stage(it.start, it.len);
            s_end[wave][lane] = pos[it.row + min(lane, nrows - 1) + 1] - it.start;
#pragma unroll
            for (int i = 0; i < 2 * K; ++i) s_dst[wave][lane + 64 * i] = held[i];
            wave_lds_sync();
            int b = 0;
            for (int q = 0; q < nrows; ++q) {
                const int e = __builtin_amdgcn_readfirstlane(s_end[wave][q]);
                if (e > b) {
#pragma unroll
                    for (int k = 0; k < K; ++k) dv[k] = s_dst[wave][q * RV + k * L + li];
                    int s0 = b;
                    for (; s0 + G * U <= e; s0 += G * U)
                        sddmm_tile_batch<L, K, RW, KH, U, SCATTER, OFF32, false, true, STAGE>(edge, s0 + g, G, e, src, lane_bytes, F, dv,
                                                                                 out, a.out_edge_stride, it.start, seg_pos);
                    if (s0 < e)
                        sddmm_tile_tail<L, K, RW, KH, U, SCATTER, OFF32, STAGE>((e - s0 + G - 1) / G, edge, s0 + g, G, e, src, lane_bytes,
                                                                         F, dv, out, a.out_edge_stride, it.start, seg_pos);
                }
                b = e;
            }
            if constexpr (STAGE != 0) flush(it.start, it.len);
            return;
        }
        // Many short rows.  Their destination slices are touched once here, one word per 128 bytes, while the
        // edges are on their way, so that all rows' misses overlap each other and the staging loads and the
        // reads at the rows' starts hit the cache.
        constexpr int kLines = (L * K * 16 + 127) / 128;
        constexpr int kTouch = (fg::kItemRows * kLines + 63) / 64;
        float touched[kTouch];
#pragma unroll
        for (int i = 0; i < kTouch; ++i) {
            const int t = lane + 64 * i;
            const int r = min(t / kLines, nrows - 1);
            const int f = min((t % kLines) * 32, L * K * 4 - 1);
            touched[i] = a.dst[(int64_t)(it.row + r) * F + tile * (L * K * 4) + f];
        }
        stage(it.start, it.len);
        s_end[wave][lane] = pos[it.row + min(lane, nrows - 1) + 1] - it.start;
        if (lane == 0) s_next[wave] = 0;
        wave_lds_sync();
#pragma unroll
        for (int i = 0; i < kTouch; ++i) asm volatile("" ::"v"(touched[i]));    // keeps the loads
        // many short rows: every lane group walks rows of its own
        int q = -1, j = 0, e = 0;
        bool done = false;
#pragma unroll
        for (int k = 0; k < K; ++k) dv[k] = vzero4();
        for (;;) {
            if (!done && j >= e) {
                int qn = 0;
                if (li == 0) qn = atomicAdd(&s_next[wave], 1);
                q = __shfl(qn, g * L);
                if (q >= nrows) {
                    done = true;
                } else {
                    j = q ? s_end[wave][q - 1] : 0;
                    e = s_end[wave][q];
                    if (e > j) load_dst(it.row + q);
                }
            }
            if (__all(done)) break;
            if (!done && j < e) {
                sddmm_tile_batch<L, K, RW, KH, U, SCATTER, OFF32, false, false, STAGE_OWN_ROWS>(edge, j, 1, e, src, lane_bytes, F, dv, out,
                                                                  a.out_edge_stride, it.start, seg_pos);
                j += U;
            }
        }
        if constexpr (STAGE_OWN_ROWS != 0) flush(it.start, it.len);
        return;
    }
    // one row, or one piece of a long row
    load_dst(it.row);
    for (int32_t base = 0; base < it.len; base += fg::kItemEdges) {
        const int n = min(fg::kItemEdges, it.len - base);
        wave_lds_sync();
        stage((int64_t)it.start + base, n);
        wave_lds_sync();
        int s0 = 0;
        for (; s0 + G * U <= n; s0 += G * U)
            sddmm_tile_batch<L, K, RW, KH, U, SCATTER, OFF32, false, true, STAGE>(edge, s0 + g, G, n, src, lane_bytes, F, dv, out,
                                                                     a.out_edge_stride, (int64_t)it.start + base, seg_pos);
        if (s0 < n)
            sddmm_tile_tail<L, K, RW, KH, U, SCATTER, OFF32, STAGE>((n - s0 + G - 1) / G, edge, s0 + g, G, n, src, lane_bytes, F, dv, out,
                                                             a.out_edge_stride, (int64_t)it.start + base, seg_pos);
        if constexpr (STAGE != 0) flush((int64_t)it.start + base, n);
    }
}

// out[edge_pos[e']] = sum over tiles of partial[tile][e'], tiles added in ascending order.  Four
// edges per lane: the tiles' arrays start `stride` floats apart (a multiple of 4, 16-byte aligned)
// and are read as 128-bit non-temporal loads (each word is read once: 13.24 -> 13.16 ms at F=512 on the 232,965-node graph).
__global__ __launch_bounds__(256) void sddmm_tile_sum_kernel(const float *partial, const int32_t *edge_pos,
                                                             float *out, int64_t n_edges, int64_t stride, int n_tiles) {
    const int64_t e = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (e >= n_edges) return;
    if (e + 4 <= n_edges) {
        typedef float f4 __attribute__((ext_vector_type(4)));
        f4 s = __builtin_nontemporal_load(reinterpret_cast<const f4 *>(partial + e));
        for (int t = 1; t < n_tiles; ++t) s += __builtin_nontemporal_load(reinterpret_cast<const f4 *>(partial + (int64_t)t * stride + e));
        const int4 at = *reinterpret_cast<const int4 *>(edge_pos + e);
        out[at.x] = s.x; out[at.y] = s.y; out[at.z] = s.z; out[at.w] = s.w;
        return;
    }
    for (int64_t i = e; i < n_edges; ++i) {
        float s = partial[i];
        for (int t = 1; t < n_tiles; ++t) s += partial[(int64_t)t * stride + i];
        out[edge_pos[i]] = s;
    }
}

// out[edge_pos[e'], t * hpt + h] = staged[t][e'][h]: the heads of every edge, computed tile by tile
// in traversal order, written as one run of H floats at the edge's stored position.
__global__ __launch_bounds__(256) void sddmm_tile_heads_kernel(const float *staged, const int32_t *edge_pos,
                                                               float *out, int64_t n_edges, int64_t tile_stride, int n_tiles, int hpt) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n_edges) return;
    float *o = out + (int64_t)edge_pos[e] * n_tiles * hpt;
    for (int t = 0; t < n_tiles; ++t) {
        const float *s = staged + (int64_t)t * tile_stride + e * hpt;
        for (int h = 0; h < hpt; ++h) o[t * hpt + h] = s[h];
    }
}

// The same for head counts that are multiples of 4: a lane owns four consecutive heads of one edge (four loads, one from
// each of their tiles' arrays, and one 128-bit store), and consecutive lanes take an edge's groups of four and then the
// next edge's, so that a wavefront reads runs of consecutive edges from each tile's array and writes whole runs of H
// floats per edge.  232,965-node graph, H=8, D=64: 2.3 ms with one thread per edge and scalar stores (3.4 TB/s), 1.5 ms
// this way (5.2 TB/s); plain loads (non-temporal ones: +0.2 ms), one edge group per lane (four: no change).
__global__ __launch_bounds__(256) void sddmm_tile_heads_vec_kernel(const float *staged, const int32_t *edge_pos,
                                                                   float *out, int64_t n_edges, int64_t tile_stride, int H) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    const int per_edge = H / 4;
    const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t e = id / per_edge;
    if (e >= n_edges) return;
    const int q = (int)(id - e * per_edge);                 // heads 4q .. 4q + 3
    const float *s = staged + (int64_t)(4 * q) * tile_stride + e;
    f4 v;
    v.x = s[0];
    v.y = s[tile_stride];
    v.z = s[2 * tile_stride];
    v.w = s[3 * tile_stride];
    *reinterpret_cast<f4 *>(out + (int64_t)edge_pos[e] * H + 4 * q) = v;
}

template <int L, int K, int RW, int KH, bool SCATTER>
void launch_tiled_off(bool off32, dim3 grid, hipStream_t st, const SddmmTiledArgs &a) {
    if (off32) hipLaunchKernelGGL((sddmm_tiled_kernel<L, K, RW, KH, SCATTER, true>), grid, dim3(kBlock), 0, st, a);
    else hipLaunchKernelGGL((sddmm_tiled_kernel<L, K, RW, KH, SCATTER, false>), grid, dim3(kBlock), 0, st, a);
}

// heads narrower than one load: RW lanes per head, KH == 1
template <int L, int K, bool SCATTER>
bool launch_tiled_rw(int RW, bool off32, dim3 grid, hipStream_t st, const SddmmTiledArgs &a) {
    switch (RW) {
        case 2: if constexpr (L >= 2) { launch_tiled_off<L, K, 2, 1, SCATTER>(off32, grid, st, a); return true; } break;
        case 4: if constexpr (L >= 4) { launch_tiled_off<L, K, 4, 1, SCATTER>(off32, grid, st, a); return true; } break;
        case 8: if constexpr (L >= 8) { launch_tiled_off<L, K, 8, 1, SCATTER>(off32, grid, st, a); return true; } break;
        case 16: if constexpr (L >= 16) { launch_tiled_off<L, K, 16, 1, SCATTER>(off32, grid, st, a); return true; } break;
        case 32: if constexpr (L >= 32) { launch_tiled_off<L, K, 32, 1, SCATTER>(off32, grid, st, a); return true; } break;
    }
    return false;
}

// KH: loads per head (0 = heads narrower than a load, RW lanes each)
template <int L, int K, bool SCATTER>
bool launch_tiled_lk(int RW, int KH, bool off32, dim3 grid, hipStream_t st, const SddmmTiledArgs &a) {
    if (KH == 0) return launch_tiled_rw<L, K, SCATTER>(RW, off32, grid, st, a);
    if (KH == 1) { launch_tiled_off<L, K, L, 1, SCATTER>(off32, grid, st, a); return true; }
    if constexpr (K >= 2) { if (KH == 2) { launch_tiled_off<L, K, L, 2, SCATTER>(off32, grid, st, a); return true; } }
    return false;
}

template <bool SCATTER>
bool launch_tiled_l(int L, int K, int RW, int KH, bool off32, dim3 grid, hipStream_t st, const SddmmTiledArgs &a) {
    if (K == 1) {
        switch (L) {
            case 4: return launch_tiled_lk<4, 1, SCATTER>(RW, KH, off32, grid, st, a);
            case 8: return launch_tiled_lk<8, 1, SCATTER>(RW, KH, off32, grid, st, a);
            case 16: return launch_tiled_lk<16, 1, SCATTER>(RW, KH, off32, grid, st, a);
        }
    } else if (K == 2) {
        switch (L) {
            case 16: return launch_tiled_lk<16, 2, SCATTER>(RW, KH, off32, grid, st, a);
            case 32: return launch_tiled_lk<32, 2, SCATTER>(RW, KH, off32, grid, st, a);
        }
    }
    return false;
}

// Any H, D (odd lengths, unaligned pointers): one edge at a time per wavefront, lanes stride
// over the head's D floats, full-wavefront reduction per head.
__global__ __launch_bounds__(kBlock) void sddmm_generic_kernel(const int32_t *row, const int32_t *col,
                                                               const int32_t *indptr, int64_t n_rows,
                                                               int64_t n_edges, const float *src,
                                                               const float *dst, float *out, int H, int D) {
    const int lane = threadIdx.x & 63;
    const int64_t wave_id = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t e0 = wave_id * 64;
    const int64_t F = (int64_t)H * D;
    for (int64_t e = e0; e < min(e0 + 64, n_edges); ++e) {
        int64_t r;
        if (row) r = row[e];
        else {                                   // CSR order: last row with indptr[r] <= e
            int64_t lo = 0, hi = n_rows;
            while (hi - lo > 1) { const int64_t mid = (lo + hi) >> 1; if (indptr[mid] <= e) lo = mid; else hi = mid; }
            r = lo;
        }
        const float *s = src + (int64_t)col[e] * F;
        const float *d = dst + r * F;
        for (int h = 0; h < H; ++h) {
            float p = 0.f;
            for (int k = lane; k < D; k += 64) p += s[h * D + k] * d[h * D + k];
            p = segment_sum<64>(p);
            if (lane == 0) out[e * H + h] = p;
        }
    }
}

struct SddmmConfig { int V, L, K, RW, KH; bool full; bool generic; };

int pow2_ceil(int v) { int p = 1; while (p < v) p <<= 1; return p; }
bool is_pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }

void choose_config(int H, int D, bool aligned16, SddmmConfig *c) {
    const int F = H * D;
    c->generic = true;
    c->full = false;
    if (H == 1) {
        c->V = (aligned16 && F % 4 == 0) ? 4 : 1;
        const int lanes = (F + c->V - 1) / c->V;
        if (lanes <= 64) { c->L = pow2_ceil(lanes) < 4 ? 4 : pow2_ceil(lanes); c->K = 1; }
        else if (lanes <= 128) { c->L = 64; c->K = 2; }
        else if (lanes <= 256) { c->L = 64; c->K = 4; }
        else return;
        c->RW = c->L; c->KH = c->K;
        c->full = (F == c->V * c->L * c->K);
        c->generic = false;
        return;
    }
    if (!aligned16 || D % 4 != 0 || H > kMaxHeadsFast) return;
    const int rw = D / 4;                       // lanes per head
    if (!is_pow2(rw) || rw > 64 || rw < 2) return;
    const int lanes = H * rw;
    c->V = 4; c->RW = rw; c->KH = 1;
    if (lanes <= 64) {
        if (!is_pow2(lanes)) return;
        c->L = lanes < 4 ? 4 : lanes; c->K = 1;
        if (c->L != lanes) return;
    } else {
        if (lanes != 128 && lanes != 256) return;
        c->L = 64; c->K = lanes / 64;
    }
    c->full = true;
    c->generic = false;
}

template <int V, int L, int K, int RW, int KH>
void launch_one(bool csr, bool full, dim3 grid, hipStream_t st, const SddmmArgs &a) {
    if (csr) {
        if (full) hipLaunchKernelGGL((sddmm_csr_kernel<V, L, K, RW, KH, true>), grid, dim3(kBlock), 0, st, a);
        else hipLaunchKernelGGL((sddmm_csr_kernel<V, L, K, RW, KH, false>), grid, dim3(kBlock), 0, st, a);
    } else {
        if (full) hipLaunchKernelGGL((sddmm_coo_kernel<V, L, K, RW, KH, true>), grid, dim3(kBlock), 0, st, a);
        else hipLaunchKernelGGL((sddmm_coo_kernel<V, L, K, RW, KH, false>), grid, dim3(kBlock), 0, st, a);
    }
}

// single head: the head spans the whole lane group and all K loads
template <int V>
bool launch_vanilla(const SddmmConfig &c, bool csr, dim3 grid, hipStream_t st, const SddmmArgs &a) {
    if (c.K == 1) {
        switch (c.L) {
            case 4: launch_one<V, 4, 1, 4, 1>(csr, c.full, grid, st, a); return true;
            case 8: launch_one<V, 8, 1, 8, 1>(csr, c.full, grid, st, a); return true;
            case 16: launch_one<V, 16, 1, 16, 1>(csr, c.full, grid, st, a); return true;
            case 32: launch_one<V, 32, 1, 32, 1>(csr, c.full, grid, st, a); return true;
            case 64: launch_one<V, 64, 1, 64, 1>(csr, c.full, grid, st, a); return true;
        }
    } else if (c.K == 2) { launch_one<V, 64, 2, 64, 2>(csr, c.full, grid, st, a); return true; }
    else if (c.K == 4) { launch_one<V, 64, 4, 64, 4>(csr, c.full, grid, st, a); return true; }
    return false;
}

template <int L, int K>
bool launch_heads_lk(const SddmmConfig &c, bool csr, dim3 grid, hipStream_t st, const SddmmArgs &a) {
    switch (c.RW) {
        case 2: if constexpr (L >= 2) { launch_one<4, L, K, 2, 1>(csr, true, grid, st, a); return true; } break;
        case 4: if constexpr (L >= 4) { launch_one<4, L, K, 4, 1>(csr, true, grid, st, a); return true; } break;
        case 8: if constexpr (L >= 8) { launch_one<4, L, K, 8, 1>(csr, true, grid, st, a); return true; } break;
        case 16: if constexpr (L >= 16) { launch_one<4, L, K, 16, 1>(csr, true, grid, st, a); return true; } break;
        case 32: if constexpr (L >= 32) { launch_one<4, L, K, 32, 1>(csr, true, grid, st, a); return true; } break;
        case 64: if constexpr (L >= 64) { launch_one<4, L, K, 64, 1>(csr, true, grid, st, a); return true; } break;
    }
    return false;
}

bool launch_heads(const SddmmConfig &c, bool csr, dim3 grid, hipStream_t st, const SddmmArgs &a) {
    if (c.K == 1) {
        switch (c.L) {
            case 4: return launch_heads_lk<4, 1>(c, csr, grid, st, a);
            case 8: return launch_heads_lk<8, 1>(c, csr, grid, st, a);
            case 16: return launch_heads_lk<16, 1>(c, csr, grid, st, a);
            case 32: return launch_heads_lk<32, 1>(c, csr, grid, st, a);
            case 64: return launch_heads_lk<64, 1>(c, csr, grid, st, a);
        }
    } else if (c.K == 2) return launch_heads_lk<64, 2>(c, csr, grid, st, a);
    else if (c.K == 4) return launch_heads_lk<64, 4>(c, csr, grid, st, a);
    return false;
}

int sddmm_run(const fg_spmm_plan *pl, const int32_t *row, const int32_t *col, const int32_t *indptr,
              int64_t n_rows, int64_t n_edges, const float *src, const float *dst, float *out, int H,
              int D, void *stream) {
    if (H < 1 || D < 1) return fail(FG_ERR_SHAPE, "heads and head length must be positive, got H=%d D=%d", H, D);
    if (n_edges < 0) return fail(FG_ERR_ARG, "negative edge count");
    if (n_edges == 0) return FG_OK;
    if (!col || !src || !dst || !out || (!row && !pl) || (pl && !indptr)) return fail(FG_ERR_ARG, "null device pointer");
    if ((int64_t)H * D > INT32_MAX) return fail(FG_ERR_SHAPE, "H*D too large");
    hipStream_t st = (hipStream_t)stream;
    const bool aligned16 = (((uintptr_t)src | (uintptr_t)dst) & 15) == 0;
    SddmmConfig c;
    choose_config(H, D, aligned16, &c);
    SddmmArgs a;
    a.row = row; a.col = col; a.items = pl ? pl->items_dev : nullptr; a.n_items = pl ? pl->n_items : 0;
    a.pos = indptr;
    a.n_edges = n_edges; a.src = src; a.dst = dst; a.out = out; a.F = H * D;
    const bool csr = pl != nullptr;
    bool launched = false;
    if (!c.generic) {
        const int64_t waves = csr ? pl->n_items : (n_edges + kEdgesPerWave - 1) / kEdgesPerWave;
        const int64_t blocks = (waves + kWavesPerBlock - 1) / kWavesPerBlock;
        if (blocks > 0x7fffffffLL) return fail(FG_ERR_SHAPE, "grid too large");
        const dim3 grid((unsigned)blocks);
        if (H == 1) launched = (c.V == 4) ? launch_vanilla<4>(c, csr, grid, st, a) : launch_vanilla<1>(c, csr, grid, st, a);
        else launched = launch_heads(c, csr, grid, st, a);
    }
    if (!launched) {
        const int64_t waves = (n_edges + 63) / 64;
        const int64_t blocks = (waves + kWavesPerBlock - 1) / kWavesPerBlock;
        if (blocks > 0x7fffffffLL) return fail(FG_ERR_SHAPE, "grid too large");
        hipLaunchKernelGGL(sddmm_generic_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, st, row, col, indptr,
                           n_rows, n_edges, src, dst, out, H, D);
    }
    FG_HIP_TRY(hipGetLastError());
    return FG_OK;
}

}  // namespace

extern "C" int fg_sddmm_coo_f32(const int32_t *row_dev, const int32_t *col_dev, int64_t n_edges,
                                const float *src_dev, const float *dst_dev, float *out_dev, int H,
                                int D, void *stream) {
    if (n_edges > 0 && !row_dev) return fail(FG_ERR_ARG, "row_dev is null");
    return sddmm_run(nullptr, row_dev, col_dev, nullptr, 0, n_edges, src_dev, dst_dev, out_dev, H, D, stream);
}

extern "C" int fg_sddmm_csr_f32(const fg_spmm_plan *plan, const int32_t *indptr_dev,
                                const int32_t *indices_dev, const float *src_dev, const float *dst_dev,
                                float *out_dev, int H, int D, void *stream) {
    if (!plan) return fail(FG_ERR_ARG, "plan is null");
    if (int drc = fg::check_device(plan)) return drc;
    if (plan->num_col_partitions != 1) return fail(FG_ERR_ARG, "fg_sddmm_csr_f32 needs a plan with one column partition");
    return sddmm_run(plan, nullptr, indices_dev, indptr_dev, plan->n_dst, plan->nnz, src_dev, dst_dev,
                     out_dev, H, D, stream);
}

namespace {
// How the tiled traversal covers H heads of D floats with T feature tiles.
struct TiledShape {
    int F, T, tile_w;
    int L, K;          // tile = L lanes x K loads x 4 floats
    int RW, KH;        // lanes per head inside a load / loads per head (0: head narrower than a load)
    int hpt;           // whole heads per tile (1 when a head spans one or more tiles)
    bool tile_sum;     // tiles hold partial sums of one head
    bool staged;       // several heads, one per tile: results staged per tile, written per edge by a last kernel
    bool off32, tile_major;
};

int resolve_tiled(const fg_spmm_plan *pl, int H, int D, int T, bool src_aligned16, TiledShape *ts) {
    if (H < 1 || D < 1) return fail(FG_ERR_SHAPE, "heads and head length must be positive, got H=%d D=%d", H, D);
    const int64_t F64 = (int64_t)H * D;
    if (F64 > INT32_MAX) return fail(FG_ERR_SHAPE, "H*D too large");
    const int F = (int)F64;
    if (T < 1 || F % T != 0) return fail(FG_ERR_SHAPE, "feature length %d is not divisible by num_feat_partitions %d", F, T);
    const int tile_w = F / T;
    if (tile_w % 4 != 0 || tile_w > 256 || !is_pow2(tile_w / 4) || tile_w < 16)
        return fail(FG_ERR_SHAPE, "feature tile of %d floats: need a power of two between 16 and 256", tile_w);
    // tile = L lanes x K loads x 4 floats: two loads per lane from 128 floats up, so that a lane's own
    // share of the dot product is longer and the cross-lane sum is paid once per 8 floats
    const int K = tile_w >= 128 ? 2 : 1;
    const int L = tile_w / 4 / K;
    const int load_w = L * 4;     // floats covered by one load of the lane group
    int RW, KH;
    bool tile_sum;
    if (D >= tile_w) {
        if (D % tile_w != 0) return fail(FG_ERR_SHAPE, "head length %d is not a multiple of the %d-float tile", D, tile_w);
        if (D > tile_w && H != 1) return fail(FG_ERR_SHAPE, "a head spanning several tiles needs H == 1");
        RW = L; KH = K; tile_sum = D > tile_w;
    } else {
        if (tile_w % D != 0 || D % 4 != 0 || !is_pow2(D / 4) || D < 8)
            return fail(FG_ERR_SHAPE, "head length %d does not pack into a %d-float tile", D, tile_w);
        if (D >= load_w) { RW = L; KH = D / load_w; }
        else { RW = D / 4; KH = 0; }
        tile_sum = false;
    }
    ts->F = F; ts->T = T; ts->tile_w = tile_w; ts->L = L; ts->K = K; ts->RW = RW; ts->KH = KH;
    ts->hpt = D >= tile_w ? 1 : tile_w / D;
    ts->tile_sum = tile_sum;
    // Several heads: a tile's results, 4 or 8 bytes per edge, would land H floats apart in out.  They
    // are kept per tile in traversal order instead and a last kernel writes each edge's H results
    // as one run.
    // (Measured on the 232,965-node graph: 20.2 -> 18.4 ms at H=8, D=64; with several heads per tile the
    // direct writes are wider and staging them costs more than it saves.)
    ts->staged = !tile_sum && ts->hpt == 1 && H >= 4 && T > 1;
    ts->off32 = !pl->wide_offsets && (uint64_t)pl->n_src * (uint64_t)F * 4u < (1ull << 32);
    // The gathers of an XCD touch one tile's slice of every src row, F * 4 bytes apart; from a copy
    // that stores each tile's slices back to back the same working set is cached better
    // (232,965-node graph, F=512: 14.5 -> 13.7 ms with 4 tiles x 16 partitions, 14.9 -> 13.5 ms with
    // 8 x 8, before the 0.15 ms of the copy).  The destination rows gain nothing from it.
    ts->tile_major = ts->off32 && pl->nnz > 0 && src_aligned16 &&
                     fg::wants_tile_major(pl, T, (uint64_t)pl->n_src * (uint64_t)F * 4u);
    return FG_OK;
}

// floats between two tiles' arrays of staged results: whole 128-byte lines, so that no line holds two tiles' results
int64_t staged_stride(int64_t nnz, int hpt) { return (nnz * hpt + 31) / 32 * 32; }

fg::ScratchNeed tiled_need(const fg_spmm_plan *pl, const TiledShape &ts, int H) {
    fg::ScratchNeed need;
    if (ts.tile_sum) need.partial = (size_t)ts.T * (size_t)((pl->nnz + 3) & ~(int64_t)3);
    else if (ts.staged) need.partial = (size_t)ts.T * (size_t)staged_stride(pl->nnz, ts.hpt);
    if (ts.tile_major) need.tiled = (size_t)pl->n_src * (size_t)ts.F;
    return need;
}
}  // namespace

namespace fg {
int sddmm_dds_scratch_need(const fg_spmm_plan *pl, int H, int D, int T, ScratchNeed *need) {
    TiledShape ts;
    if (int rc = resolve_tiled(pl, H, D, T, true, &ts)) return rc;
    *need = tiled_need(pl, ts, H);
    return FG_OK;
}
}  // namespace fg

extern "C" int fg_sddmm_dds_f32(fg_spmm_plan *pl, const int32_t *s1_pos_dev, const int32_t *s1_idx_dev,
                                const int32_t *edge_pos_dev, const float *src_dev, const float *dst_dev,
                                float *out_dev, int H, int D, int num_feat_partitions, void *stream) {
    if (!pl) return fail(FG_ERR_ARG, "plan is null");
    if (int drc = fg::check_device(pl)) return drc;
    TiledShape ts;
    int rc = resolve_tiled(pl, H, D, num_feat_partitions, (((uintptr_t)src_dev) & 15) == 0, &ts);
    if (rc != FG_OK) return rc;
    if (pl->nnz == 0) return FG_OK;
    if (!s1_pos_dev || !s1_idx_dev || !edge_pos_dev || !src_dev || !dst_dev || !out_dev)
        return fail(FG_ERR_ARG, "null device pointer");
    if ((((uintptr_t)src_dev | (uintptr_t)dst_dev) & 15) != 0) return fail(FG_ERR_ARG, "src/dst must be 16-byte aligned");
    if (ts.tile_sum && ((uintptr_t)edge_pos_dev & 15)) return fail(FG_ERR_ARG, "edge_pos must be 16-byte aligned");
    if ((rc = fg::ensure_scratch(pl, tiled_need(pl, ts, H), stream)) != FG_OK) return rc;
    const int F = ts.F, T = ts.T, tile_w = ts.tile_w, L = ts.L, K = ts.K, RW = ts.RW, KH = ts.KH, hpt = ts.hpt;
    const bool tile_sum = ts.tile_sum, staged = ts.staged, off32 = ts.off32;
    hipStream_t st = (hipStream_t)stream;
    SddmmTiledArgs a;
    a.col = s1_idx_dev; a.col16 = fg::narrow_indices(pl, s1_idx_dev); a.edge_pos = edge_pos_dev; a.dst = dst_dev; a.F = F; a.n_tiles = T;
    if (tile_sum) {
        a.out = pl->partial_dev; a.out_edge_stride = 1; a.out_tile_stride = (pl->nnz + 3) & ~(int64_t)3;
    } else if (staged) {
        a.out = pl->partial_dev; a.out_edge_stride = hpt; a.out_tile_stride = staged_stride(pl->nnz, hpt);
    } else {
        a.out = out_dev; a.out_edge_stride = H; a.out_tile_stride = tile_w / D;
    }
    const int P = pl->num_col_partitions;
    const int64_t width = (pl->n_src + P - 1) / P;
    a.items = pl->items_dev; a.item_off = pl->item_off_dev;
    a.pos = s1_pos_dev; a.pos_stride = pl->n_dst + 1;
    a.src = src_dev; a.src_stride = width * F; a.n_parts = P;
    a.src_row_bytes = (uint32_t)F * 4u; a.src_tile_bytes = 0;
    if (ts.tile_major) {
        if ((rc = fg::make_tile_major(pl, src_dev, pl->n_src, F, tile_w, stream)) != FG_OK) return rc;
        a.src = pl->tiled_dev; a.src_stride = width * tile_w;
        a.src_row_bytes = (uint32_t)tile_w * 4u; a.src_tile_bytes = (uint32_t)((uint64_t)pl->n_src * tile_w * 4u);
    }
    // The tiles go out 8, 4, 2 or 1 per launch: counts that divide the 8 XCDs, so that workgroup id % slots always puts
    // a tile on the same XCDs (10 tiles: 8 + 2; with all 10 in one launch every L2 would see every tile's slice).
    // Fewer than 8 tiles in a launch: 8 / tiles partitions at a time, so that every XCD still has one tile of one
    // partition to itself (no two L2s hold the same slice) and a partition's slice can be smaller at the same number
    // of launches; edges of different partitions write different results.
    // (232,965-node graph: 3.93 -> 3.71 ms at F=128, 7.89 -> 7.56 ms at F=256, 1.96 -> 1.82 ms at F=64.)
    for (int tb = 0, per_launch; tb < T; tb += per_launch) {
        const int left = T - tb;
        per_launch = left >= 8 ? 8 : left >= 4 ? 4 : left >= 2 ? 2 : 1;
        const int conc = std::max(1, std::min(8 / per_launch, P));
        a.conc = conc; a.n_tiles = per_launch; a.tile_base = tb;
        // Nothing orders the passes over the partitions: one launch walks all groups of `conc` partitions, group after
        // group in workgroup order; the next group's first workgroups fill the compute units that the previous one's
        // last workgroups leave idle (232,965-node graph, F=512: 13.64 -> 13.51 ms).
        const int n_groups = (P + conc - 1) / conc;
        a.n_groups = 0;
        a.first_part = 0;
        if (n_groups > 1 && n_groups <= kMaxGroups) {
            a.n_groups = n_groups;
            a.group_off[0] = 0;
            for (int g = 0; g < n_groups; ++g) {
                int64_t most = 0;
                for (int p = g * conc; p < std::min(P, (g + 1) * conc); ++p) most = std::max(most, pl->item_off[p + 1] - pl->item_off[p]);
                a.group_off[g + 1] = a.group_off[g] + (most + kWavesPerBlock - 1) / kWavesPerBlock;
            }
            const int64_t blocks = a.group_off[n_groups] * per_launch * conc;
            if (blocks > 0x7fffffffLL) return fail(FG_ERR_SHAPE, "grid too large");
            if (blocks > 0) {
                const bool ok = (tile_sum || staged) ? launch_tiled_l<false>(L, K, RW, KH, off32, dim3((unsigned)blocks), st, a)
                                                     : launch_tiled_l<true>(L, K, RW, KH, off32, dim3((unsigned)blocks), st, a);
                if (!ok) return fail(FG_ERR_SHAPE, "no tiled SDDMM kernel for L=%d K=%d RW=%d KH=%d", L, K, RW, KH);
            }
            continue;
        }
        for (int p0 = 0; p0 < P; p0 += conc) {
            int64_t most = 0;
            for (int p = p0; p < std::min(P, p0 + conc); ++p) most = std::max(most, pl->item_off[p + 1] - pl->item_off[p]);
            if (most == 0) continue;
            a.first_part = p0;
            const int64_t blocks = ((most + kWavesPerBlock - 1) / kWavesPerBlock) * per_launch * conc;
            if (blocks > 0x7fffffffLL) return fail(FG_ERR_SHAPE, "grid too large");
            const bool ok = (tile_sum || staged) ? launch_tiled_l<false>(L, K, RW, KH, off32, dim3((unsigned)blocks), st, a)
                                                 : launch_tiled_l<true>(L, K, RW, KH, off32, dim3((unsigned)blocks), st, a);
            if (!ok) return fail(FG_ERR_SHAPE, "no tiled SDDMM kernel for L=%d K=%d RW=%d KH=%d", L, K, RW, KH);
        }
    }
    if (tile_sum) {
        const unsigned blocks = (unsigned)((pl->nnz + 1023) / 1024);
        hipLaunchKernelGGL(sddmm_tile_sum_kernel, dim3(blocks), dim3(256), 0, st, pl->partial_dev, edge_pos_dev,
                           out_dev, pl->nnz, (pl->nnz + 3) & ~(int64_t)3, T);
    } else if (staged) {
        const int64_t blocks_vec = (pl->nnz * (H / 4) + 255) / 256;
        const int64_t tstride = staged_stride(pl->nnz, hpt);
        if (H % 4 == 0 && hpt == 1 && (((uintptr_t)out_dev) & 15) == 0 && blocks_vec <= 0x7fffffffLL) {
            hipLaunchKernelGGL(sddmm_tile_heads_vec_kernel, dim3((unsigned)blocks_vec), dim3(256), 0, st, pl->partial_dev,
                               edge_pos_dev, out_dev, pl->nnz, tstride, H);
        } else {
            const unsigned blocks = (unsigned)((pl->nnz + 255) / 256);
            hipLaunchKernelGGL(sddmm_tile_heads_kernel, dim3(blocks), dim3(256), 0, st, pl->partial_dev, edge_pos_dev,
                               out_dev, pl->nnz, tstride, T, hpt);
        }
    }
    FG_HIP_TRY(hipGetLastError());
    return FG_OK;
}

// ---- element-wise edge operators ---------------------------------------------------------------
//
// out[e, f] = src[col[e], f] (+ | - | *) dst[row[e], f]: the broadcasting kernel of fg_general.hip with both
// operands in the output's layout (no reduction, F results per edge: bound by writing out).

extern "C" int fg_gsddmm_elementwise_f32(const int32_t *row_dev, const int32_t *col_dev, int64_t n_edges,
                                         const float *src_dev, const float *dst_dev, float *out_dev, int F,
                                         int op, void *stream) {
    if (op != FG_EDGE_ADD && op != FG_EDGE_SUB && op != FG_EDGE_MUL) return fail(FG_ERR_ARG, "unknown edge operator %d", op);
    const int bin = op == FG_EDGE_ADD ? FG_BIN_ADD : op == FG_EDGE_SUB ? FG_BIN_SUB : FG_BIN_MUL;
    return fg_gsddmm_bcast_f32(row_dev, col_dev, n_edges, bin, src_dev, FG_TARGET_U, F, nullptr, dst_dev, FG_TARGET_V, F,
                               nullptr, 0, out_dev, F, 1, stream);
}
