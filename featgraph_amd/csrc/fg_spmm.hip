// CSR / DDS SpMM for gfx950: out[v, :] = sum_e vals[e] * X[indices[e], :].
//
// One wavefront per plan item (a run of short rows, one row, or a piece of a long row).  The feature axis is
// spread over lanes in vectors of V floats: a group of L lanes covers V*L*K consecutive
// floats of one source row with K coalesced vector loads, and the 64/L groups of the
// wavefront take different elements of the row at the same time.  Column ids and weights
// are staged in LDS (up to 256 elements per wavefront) by coalesced loads and read back as
// broadcasts, so no lane re-reads them from global memory.  Wide rows are cut into feature
// tiles; the tile index is the fastest-varying part of the workgroup id, so consecutive
// workgroups (which the dispatcher deals round-robin to the 8 XCDs) work on the same
// elements but different feature tiles, and every XCD's L2 holds only its tiles' slice of X.
#include <hip/hip_runtime.h>

#include <climits>
#include <mutex>
#include <string>

#include "fg_common.h"
#include "fg_device.h"

using fg::fail;
using fg::Fixup;
using fg::Item;
using fg::wave_lds_sync;

namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kBlock = 64 * kWavesPerBlock;
constexpr int kPad = 8;

template <int V> struct Vec;
template <> struct Vec<4> { using type = float4; };
template <> struct Vec<1> { using type = float; };

__device__ __forceinline__ float4 vzero(float4) { return make_float4(0.f, 0.f, 0.f, 0.f); }
__device__ __forceinline__ float vzero(float) { return 0.f; }
__device__ __forceinline__ void vfma(float4 &a, float w, const float4 &x) {
    a.x += w * x.x; a.y += w * x.y; a.z += w * x.z; a.w += w * x.w;
}
__device__ __forceinline__ void vfma(float &a, float w, const float &x) { a += w * x; }
__device__ __forceinline__ void vadd(float4 &a, const float4 &b) { a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w; }
__device__ __forceinline__ void vadd(float &a, const float &b) { a += b; }
__device__ __forceinline__ float4 vshfl_xor(const float4 &a, int off) {
    return make_float4(__shfl_xor(a.x, off), __shfl_xor(a.y, off), __shfl_xor(a.z, off), __shfl_xor(a.w, off));
}
__device__ __forceinline__ float vshfl_xor(const float &a, int off) { return __shfl_xor(a, off); }
// a where `keep`, else zeros
__device__ __forceinline__ float4 vkeep(bool keep, const float4 &a) {
    return make_float4(keep ? a.x : 0.f, keep ? a.y : 0.f, keep ? a.z : 0.f, keep ? a.w : 0.f);
}
__device__ __forceinline__ float vkeep(bool keep, const float &a) { return keep ? a : 0.f; }

struct SpmmArgs {
    const Item *items;
    int64_t n_items;
    const int32_t *pos;    // this partition's position array (row boundaries), n_dst + 1 entries
    const int32_t *indices;
    const uint16_t *indices16 = nullptr;   // the plan's 16-bit copy of `indices` (null: none), read by the sum kernel
    const float *vals;
    const float *x;        // already offset to the partition's first source row
    // Sum, max and min kernels, 32-bit offsets only.  Bytes between consecutive source rows, and, when the
    // kernel tiles of x are stored one after the other ([tile][row][tile floats]), the bytes from
    // one tile's block to the next; 0: rows of F floats that hold all tiles.
    uint32_t x_row_bytes;
    uint32_t x_tile_bytes;
    float *out;
    float *partial;
    int F;                 // row stride of x / out in floats
    int tile_w;            // floats per requested feature tile (F / num_feat_partitions)
    int sub_per_tile;      // kernel tiles (V*L*K floats each) per requested tile
    int n_ftiles;          // kernel tiles handled by this launch (consecutive, starting at tile_base)
    int tile_base;
    int accumulate;        // add to out instead of overwriting it
    int heads;             // weights are [nnz, heads]; a kernel tile lies inside one head
    int head_len;          // floats per head (F / heads)
    int32_t *arg;          // arg kernel: stored position of the element that gave out[v, f]
    int vstride;           // weight of element t, head h: vals[t * vstride + h * head_stride]
    int64_t head_stride;
    // One launch over the items of all source partitions (sum kernel, every pass into a buffer of its own): the
    // plan's item_off on the device (n_parts + 1 entries; null: the launch holds one partition's items and the
    // strides are unused) and the distance from one partition's pos / x / out / partial to the next, in elements.
    const int64_t *item_off = nullptr;
    int n_parts = 1;
    int64_t pos_stride = 0, x_stride = 0, out_stride = 0, partial_stride = 0;
};


// Address of this lane's part of a staged source row.  OFF32: the staged word is the row's byte
// offset from the (wave-uniform) start of X and fits 32 bits, so the load takes a scalar base
// plus a 32-bit lane offset and no 64-bit multiply is left in the loop; otherwise it is the
// column id.
template <bool OFF32>
__device__ __forceinline__ const float *row_ptr(const float *x, uint32_t lane_bytes, int64_t F, int staged) {
    if (OFF32) return reinterpret_cast<const float *>(reinterpret_cast<const char *>(x) + ((uint32_t)staged + lane_bytes));
    return reinterpret_cast<const float *>(reinterpret_cast<const char *>(x + (int64_t)staged * F) + lane_bytes);
}

// The last, partly filled batch of gather_rows: exactly `nu` steps (1 <= nu <= NU, uniform over
// the wavefront), so that no step is spent re-reading the row's last element; inside the last
// step a lane without an element still re-reads it (no load under a branch) and replaces what it
// loaded by zeros -- a select, not a product with weight zero, so that a non-finite source row
// only ever reaches the rows that reference it.
template <int V, int L, int K, bool FULL, int NU, bool OFF32, int HPT>
__device__ __forceinline__ void gather_tail(int nu, const int2 *s_edge, const float *wrow, int s0, int e, int g,
                                            const float *x, uint32_t lane_bytes, int64_t F, const bool (&on)[K],
                                            typename Vec<V>::type (&acc)[K]) {
    using vec = typename Vec<V>::type;
    constexpr int G = 64 / L;
    if (nu < NU) {
        if constexpr (NU > 1) gather_tail<V, L, K, FULL, NU - 1, OFF32, HPT>(nu, s_edge, wrow, s0, e, g, x, lane_bytes, F, on, acc);
        return;
    }
    int2 cw[NU];
    vec xv[NU][K];
#pragma unroll
    for (int u = 0; u < NU; ++u) {
        const int j = s0 + u * G + g;
        cw[u] = s_edge[j < e ? j : e - 1];
        if (HPT > 1) cw[u].y = __float_as_int(wrow[j < e ? j : e - 1]);
        if (j >= e) cw[u].y = 0;
    }
#pragma unroll
    for (int u = 0; u < NU; ++u)
#pragma unroll
        for (int k = 0; k < K; ++k)
            if (FULL || on[k])
                xv[u][k] = *reinterpret_cast<const vec *>(row_ptr<OFF32>(x, lane_bytes, F, cw[u].x) + k * L * V);
    const bool last_has = s0 + (NU - 1) * G + g < e;      // steps before the last are full
#pragma unroll
    for (int u = 0; u < NU; ++u)
#pragma unroll
        for (int k = 0; k < K; ++k)
            if (FULL || on[k]) {
                if (u == NU - 1) xv[u][k] = vkeep(last_has, xv[u][k]);
                vfma(acc[k], __int_as_float(cw[u].y), xv[u][k]);
            }
}

// Adds vals * X rows for the staged elements [b, e) of s_edge (x = staged column word, y =
// weight bits) into acc.  The G lane groups take elements b+g, b+g+G, ...; U steps' loads are
// issued back to back before the first use.  No load sits under a branch: in the last, partly
// filled batch a lane without an element re-reads the row's last element and discards it.
// HPT > 1: the kernel tile holds HPT heads and the lane's weight is wrow[slot] (its head's staged
// weights) instead of the word staged next to the column.
template <int V, int L, int K, bool FULL, int U, bool OFF32, int HPT>
__device__ __forceinline__ void gather_rows(const int2 *s_edge, const float *wrow, int b, int e, int g, const float *x,
                                            uint32_t lane_bytes, int64_t F, const bool (&on)[K],
                                            typename Vec<V>::type (&acc)[K]) {
    using vec = typename Vec<V>::type;
    constexpr int G = 64 / L;
    int s0 = b;
    for (; s0 + G * U <= e; s0 += G * U) {
        int2 cw[U];
        vec xv[U][K];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            cw[u] = s_edge[s0 + u * G + g];
            if (HPT > 1) cw[u].y = __float_as_int(wrow[s0 + u * G + g]);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int k = 0; k < K; ++k)
                if (FULL || on[k])
                    xv[u][k] = *reinterpret_cast<const vec *>(row_ptr<OFF32>(x, lane_bytes, F, cw[u].x) + k * L * V);
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int k = 0; k < K; ++k)
                if (FULL || on[k]) vfma(acc[k], __int_as_float(cw[u].y), xv[u][k]);
    }
    if (s0 < e)                            // uniform: fewer than G*U elements left
        gather_tail<V, L, K, FULL, U, OFF32, HPT>((e - s0 + G - 1) / G, s_edge, wrow, s0, e, g, x, lane_bytes, F, on, acc);
}

// Adds the lane groups' sums (group 0 gets the total) and stores one output row; `old` is what
// the row held before (only read when ADD).
template <int V, int L, int K, bool FULL, bool ADD>
__device__ __forceinline__ void finish_row(typename Vec<V>::type (&acc)[K], const typename Vec<V>::type (&old)[K],
                                           int g, const bool (&on)[K], float *dst) {
    using vec = typename Vec<V>::type;
#pragma unroll
    for (int off = L; off < 64; off <<= 1)
#pragma unroll
        for (int k = 0; k < K; ++k) vadd(acc[k], vshfl_xor(acc[k], off));
    if (g == 0) {
#pragma unroll
        for (int k = 0; k < K; ++k)
            if (FULL || on[k]) {
                vec r = acc[k];
                if (ADD) vadd(r, old[k]);
                if constexpr (V == 4 && !ADD) {
                    // written once, read back by another kernel: a non-temporal store leaves the L2 to the gathered rows
                    // (232,965-node graph: 11.24 -> 11.17 ms at F=512, 5.75 -> 5.72 ms at F=256)
                    typedef float f4 __attribute__((ext_vector_type(4)));
                    f4 t; t.x = r.x; t.y = r.y; t.z = r.z; t.w = r.w;
                    __builtin_nontemporal_store(t, reinterpret_cast<f4 *>(dst + k * L * V));
                } else {
                    *reinterpret_cast<vec *>(dst + k * L * V) = r;
                }
            }
    }
}

// Loads elements [base, base + min(n, 256)) of (indices, vals) into registers, lane l holding
// elements 4l .. 4l + 3.  n >= 1.
// `scale` turns a column id into the staged word: the row's byte size (OFF32) or 1.  The weight of
// element t is vals[t * vstride + voff] (one weight per head), or 1 when there are no weights.
// indices16 (uniform; null: none): the same ids as 16-bit words, read instead of `indices`.
__device__ __forceinline__ void stage_load(const int32_t *indices, const uint16_t *indices16, const float *vals, int64_t base, int n,
                                           int lane, uint32_t scale, int vstride, int64_t voff, int2 (&r)[4]) {
    int32_t c[4];
    float w[4] = {1.0f, 1.0f, 1.0f, 1.0f};
    fg::load_four_ids(indices, indices16, base, n, lane, c);
    if (vals) fg::load_four(vals + base * vstride + voff, n, lane, vstride, w);
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = make_int2((int)((uint32_t)c[i] * scale), __float_as_int(w[i]));
}
// Writes the staged words to the wavefront's staging row (16-byte aligned), two elements per store.
__device__ __forceinline__ void stage_store(int2 *edge, int lane, const int2 (&r)[4]) {
    int4 *e4 = reinterpret_cast<int4 *>(edge);
    e4[2 * lane] = make_int4(r[0].x, r[0].y, r[1].x, r[1].y);
    e4[2 * lane + 1] = make_int4(r[2].x, r[2].y, r[3].x, r[3].y);
    if (lane < kPad) edge[fg::kItemEdges + lane] = r[3];      // a valid element: slots past the end stay loadable
}

// The same for the weights of the HPT heads of a kernel tile (head h of the tile: vals[t * vstride + voff + h * hstride]).
template <int HPT>
__device__ __forceinline__ void stage_load_w(const float *vals, int64_t base, int n, int lane, int vstride,
                                             int64_t voff, int64_t hstride, float (&w)[HPT][4]) {
#pragma unroll
    for (int h = 0; h < HPT; ++h) {
        if (vals) {
            fg::load_four(vals + base * vstride + voff + h * hstride, n, lane, vstride, w[h]);
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) w[h][i] = 1.0f;
        }
    }
}
template <int HPT, int ROW>
__device__ __forceinline__ void stage_store_w(float (*rows)[ROW], int lane, const float (&w)[HPT][4]) {
#pragma unroll
    for (int h = 0; h < HPT; ++h) {
        *reinterpret_cast<float4 *>(&rows[h][4 * lane]) = make_float4(w[h][0], w[h][1], w[h][2], w[h][3]);
        if (lane < kPad) rows[h][fg::kItemEdges + lane] = w[h][3];
    }
}

// V: floats per lane per load; L: lanes per source row; K: loads per lane per source row;
// FULL: every lane's columns are inside the tile (no masking needed); ACC: add to out;
// OFF32: X spans less than 4 GiB, rows are addressed by 32-bit byte offsets; HPT: heads (with
// their own weights) per kernel tile, each covered by L / HPT lanes.
template <int V, int L, int K, bool FULL, bool ACC, bool OFF32, int HPT = 1>
__device__ __forceinline__ void spmm_items_body(const SpmmArgs &a) {
    using vec = typename Vec<V>::type;
    static_assert(fg::kItemEdges == 256, "stage_load/stage_store move 4 x 64 elements");
    constexpr int FT = V * L * K;          // floats per kernel tile
    constexpr int G = 64 / L;              // lane groups per wavefront
    constexpr int U = (K >= 2) ? 2 : 4;   // steps whose loads are issued back to back
    static_assert(U <= kPad, "reads past a row's end must stay inside the padded staging row");
    // kPad extra slots: the lane-group-per-row walk may read up to U - 1 slots past a row's end
    __shared__ __align__(16) int2 s_edge[kWavesPerBlock][fg::kItemEdges + kPad];
    __shared__ int32_t s_end[kWavesPerBlock][fg::kItemRows];
    __shared__ int32_t s_next[kWavesPerBlock];
    constexpr int kWRow = HPT > 1 ? fg::kItemEdges + kPad : 1;
    __shared__ __align__(16) float s_w[kWavesPerBlock][HPT][kWRow];
    static_assert(HPT == 1 || (L % HPT == 0 && K == 1 && FULL), "heads of a tile split its lanes evenly");

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int tile = a.tile_base + (int)(blockIdx.x % (unsigned)a.n_ftiles);
    const int64_t item_id = (int64_t)(blockIdx.x / (unsigned)a.n_ftiles) * kWavesPerBlock + wave;
    if (item_id >= a.n_items) return;      // uniform per wavefront; no workgroup barriers below
    const Item it = a.items[item_id];
    // the partition this item belongs to (uniform per wavefront): selects its position array, its slice of x,
    // its output buffer and its share of the split rows' scratch
    int part = 0;
    if (a.item_off) {
        const int64_t id = ((int64_t)__builtin_amdgcn_readfirstlane((int)(item_id >> 32)) << 32) |
                           (uint32_t)__builtin_amdgcn_readfirstlane((int)item_id);
        while (part + 1 < a.n_parts && id >= a.item_off[part + 1]) ++part;
    }
    const int32_t *const pos_p = a.pos + part * a.pos_stride;
    const float *const x_p = a.x + part * a.x_stride;
    float *const out_p = a.out + part * a.out_stride;
    float *const partial_p = a.partial + part * a.partial_stride;
    const int g = lane / L, li = lane % L;

    const int rt = tile / a.sub_per_tile, st = tile % a.sub_per_tile;
    const int f_end = (rt + 1) * a.tile_w;
    const int f_lo = rt * a.tile_w + st * FT + li * V;      // first column of this lane, k = 0
    bool on[K];
#pragma unroll
    for (int k = 0; k < K; ++k) on[k] = FULL || (f_lo + k * L * V < f_end);
    const uint32_t lane_bytes = (OFF32 && a.x_tile_bytes) ? (uint32_t)tile * a.x_tile_bytes + (uint32_t)(li * V) * 4u
                                                          : (uint32_t)f_lo * 4u;
    const uint32_t scale = OFF32 ? a.x_row_bytes : 1u;
    const int64_t voff = (int64_t)((rt * a.tile_w + st * FT) / a.head_len) * a.head_stride;     // head of this kernel tile
    const int64_t F = a.F;
    int2 *edge = s_edge[wave];
    const float *wrow = s_w[wave][HPT > 1 ? (lane % L) / (L / HPT) : 0];
    const float *col_vals = HPT > 1 ? nullptr : a.vals;     // HPT > 1: weights are staged per head instead
    vec acc[K], old[K];
    int2 regs[4];
    float wregs[HPT][4];

    if (it.info < -1) {
        // Several whole rows: stage all their elements once.
        const int nrows = -it.info;
        // ACC: the rows this item adds to are read once here, one word per 128 bytes, while the
        // elements are on their way.  Loads return in order, so a row of `out` fetched from memory
        // at the moment it is needed would hold up every gather issued after it; fetched here, all
        // rows' misses overlap each other and the staging loads, and the later reads hit the cache.
        constexpr int kLines = (FT * 4 + 127) / 128;
        constexpr int kTouch = ACC ? (fg::kItemRows * kLines + 63) / 64 : 1;
        float touched[kTouch];
        if (ACC) {
            const int f_tile = rt * a.tile_w + st * FT;
            const int f_last = min(f_tile + FT, f_end) - 1;
#pragma unroll
            for (int i = 0; i < kTouch; ++i) {
                const int t = lane + 64 * i;
                const int r = min(t / kLines, nrows - 1);
                const int f = min(f_tile + (t % kLines) * 32, f_last);
                touched[i] = out_p[(int64_t)(it.row + r) * F + f];
            }
        }
        if (it.len > 0) {
            stage_load(a.indices, a.indices16, col_vals, it.start, it.len, lane, scale, a.vstride, voff, regs);
            if (HPT > 1) stage_load_w<HPT>(a.vals, it.start, it.len, lane, a.vstride, voff, a.head_stride, wregs);
            stage_store(edge, lane, regs);
            if (HPT > 1) stage_store_w<HPT>(s_w[wave], lane, wregs);
        }
        s_end[wave][lane] = pos_p[it.row + min(lane, nrows - 1) + 1] - it.start;
        if (lane == 0) s_next[wave] = 0;
        wave_lds_sync();
        if (ACC) {
#pragma unroll
            for (int i = 0; i < kTouch; ++i) asm volatile("" ::"v"(touched[i]));    // keeps the loads
        }
        if (nrows < 2 * G) {
            // Few, longer rows: all lane groups share each row in turn.
            int b = 0;
            for (int q = 0; q < nrows; ++q) {
                const int e = __builtin_amdgcn_readfirstlane(s_end[wave][q]);
                if (e > b || !ACC) {
                    float *dst = out_p + (int64_t)(it.row + q) * F + f_lo;
                    if (ACC) {
#pragma unroll
                        for (int k = 0; k < K; ++k)
                            if (FULL || on[k]) old[k] = *reinterpret_cast<const vec *>(dst + k * L * V);
                    }
#pragma unroll
                    for (int k = 0; k < K; ++k) acc[k] = vzero(vec());
                    gather_rows<V, L, K, FULL, U, OFF32, HPT>(edge, wrow, b, e, g, x_p, lane_bytes, F, on, acc);
                    finish_row<V, L, K, FULL, ACC>(acc, old, g, on, dst);
                }
                b = e;
            }
            return;
        }
        // Many short rows: every lane group takes rows of its own (next free row from a counter
        // in LDS), walks each row's elements U at a time and writes the row itself, so G rows
        // are in flight per wavefront and no sums cross lane groups.
        int q = -1, j = 0, e = 0;
        bool done = false, nonempty = false;
        for (;;) {
            if (!done && j >= e) {
                if (q >= 0 && (!ACC || nonempty)) {       // the row this group just finished
                    float *dst = out_p + (int64_t)(it.row + q) * F + f_lo;
#pragma unroll
                    for (int k = 0; k < K; ++k)
                        if (FULL || on[k]) {
                            vec r = acc[k];
                            if (ACC) vadd(r, old[k]);
                            *reinterpret_cast<vec *>(dst + k * L * V) = r;
                        }
                }
                int qn = 0;
                if (li == 0) qn = atomicAdd(&s_next[wave], 1);
                q = __shfl(qn, g * L);
                if (q >= nrows) {
                    done = true;
                } else {
                    j = q ? s_end[wave][q - 1] : 0;
                    e = s_end[wave][q];
                    nonempty = e > j;
#pragma unroll
                    for (int k = 0; k < K; ++k) acc[k] = vzero(vec());
                    if (ACC && nonempty) {
                        const float *src = out_p + (int64_t)(it.row + q) * F + f_lo;
#pragma unroll
                        for (int k = 0; k < K; ++k)
                            if (FULL || on[k]) old[k] = *reinterpret_cast<const vec *>(src + k * L * V);
                    }
                }
            }
            if (__all(done)) break;
            if (!done && j < e) {
                int2 cw[U];
                vec xv[U][K];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    // past the row's end this is a later row's element (or the padding): a loadable
                    // source row whose values are replaced by zeros below
                    cw[u] = edge[j + u];
                    if (HPT > 1) cw[u].y = __float_as_int(wrow[j + u]);
                    if (j + u >= e) cw[u].y = 0;
                }
#pragma unroll
                for (int u = 0; u < U; ++u)
#pragma unroll
                    for (int k = 0; k < K; ++k)
                        if (FULL || on[k])
                            xv[u][k] = *reinterpret_cast<const vec *>(row_ptr<OFF32>(x_p, lane_bytes, F, cw[u].x) + k * L * V);
#pragma unroll
                for (int u = 0; u < U; ++u)
#pragma unroll
                    for (int k = 0; k < K; ++k)
                        if (FULL || on[k]) {
                            // u == 0 is always the row's own element (j < e)
                            if (u > 0) xv[u][k] = vkeep(j + u < e, xv[u][k]);
                            vfma(acc[k], __int_as_float(cw[u].y), xv[u][k]);
                        }
                j += U;
            }
        }
        return;
    }

    // one row, or one piece of a long row: 256 elements at a time, the next 256 on their way
    // while the current ones are used
    float *dst = (it.info < 0 ? out_p + (int64_t)it.row * F : partial_p + (int64_t)it.info * F) + f_lo;
    const bool add = ACC && it.info < 0;
#pragma unroll
    for (int k = 0; k < K; ++k) acc[k] = vzero(vec());
    if (it.len > 0) {
        stage_load(a.indices, a.indices16, col_vals, it.start, it.len, lane, scale, a.vstride, voff, regs);
        if (HPT > 1) stage_load_w<HPT>(a.vals, it.start, it.len, lane, a.vstride, voff, a.head_stride, wregs);
    }
    if (ACC) {
#pragma unroll
        for (int k = 0; k < K; ++k)
            if (FULL || on[k]) old[k] = add ? *reinterpret_cast<const vec *>(dst + k * L * V) : vzero(vec());
    }
    for (int32_t base = 0; base < it.len; base += fg::kItemEdges) {
        const int n = min(fg::kItemEdges, it.len - base);
        wave_lds_sync();                   // earlier reads of the staging row are done
        stage_store(edge, lane, regs);
        if (HPT > 1) stage_store_w<HPT>(s_w[wave], lane, wregs);
        wave_lds_sync();
        if (base + fg::kItemEdges < it.len) {
            stage_load(a.indices, a.indices16, col_vals, (int64_t)it.start + base + fg::kItemEdges,
                       it.len - base - fg::kItemEdges, lane, scale, a.vstride, voff, regs);
            if (HPT > 1)
                stage_load_w<HPT>(a.vals, (int64_t)it.start + base + fg::kItemEdges, it.len - base - fg::kItemEdges,
                                  lane, a.vstride, voff, a.head_stride, wregs);
        }
        gather_rows<V, L, K, FULL, U, OFF32, HPT>(edge, wrow, 0, n, g, x_p, lane_bytes, F, on, acc);
    }
    finish_row<V, L, K, FULL, ACC>(acc, old, g, on, dst);
}

// The kernels proper.  One load per lane and source row (K == 1) fits 64 registers without spilling
// and is held to 8 wavefronts per SIMD; wider rows per lane and tiles of several heads keep the
// compiler's own register budget.
template <int V, int L, int K, bool FULL, bool ACC, bool OFF32>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(8, 8))) void spmm_items_kernel(const SpmmArgs a) {
    static_assert(K == 1, "wider rows use spmm_items_wide_kernel");
    spmm_items_body<V, L, K, FULL, ACC, OFF32, 1>(a);
}
template <int V, int L, int K, bool FULL, bool ACC, bool OFF32, int HPT>
__global__ __launch_bounds__(kBlock) void spmm_items_wide_kernel(const SpmmArgs a) {
    spmm_items_body<V, L, K, FULL, ACC, OFF32, HPT>(a);
}

// ---- max / min aggregation ------------------------------------------------------------------------
//
// out[v, f] = max (or min) over the row's elements of vals[e] * X[indices[e], f]; a row without
// elements gives 0.  Same items, staging and lane layout as the sum kernel; all lane groups share
// each row in turn and a lane without an element in the last batch keeps its running extreme.

template <bool IS_MAX> __device__ __forceinline__ float ext_identity() { return IS_MAX ? -INFINITY : INFINITY; }
// a NaN message beats every number (it reaches the result, as through a sum); once the running extreme is a NaN it stays
template <bool IS_MAX> __device__ __forceinline__ float ext_op(float a, float b) { return ((IS_MAX ? b > a : b < a) || b != b) ? b : a; }
template <bool IS_MAX> __device__ __forceinline__ void vext(float4 &a, const float4 &b) {
    a.x = ext_op<IS_MAX>(a.x, b.x); a.y = ext_op<IS_MAX>(a.y, b.y);
    a.z = ext_op<IS_MAX>(a.z, b.z); a.w = ext_op<IS_MAX>(a.w, b.w);
}
template <bool IS_MAX> __device__ __forceinline__ void vext(float &a, const float &b) { a = ext_op<IS_MAX>(a, b); }
__device__ __forceinline__ float4 vscale(float w, const float4 &x) { return make_float4(w * x.x, w * x.y, w * x.z, w * x.w); }
__device__ __forceinline__ float vscale(float w, const float &x) { return w * x; }
__device__ __forceinline__ float4 vsplat(float4, float v) { return make_float4(v, v, v, v); }
__device__ __forceinline__ float vsplat(float, float v) { return v; }
__device__ __forceinline__ float4 vpick(bool c, const float4 &a, const float4 &b) {
    return make_float4(c ? a.x : b.x, c ? a.y : b.y, c ? a.z : b.z, c ? a.w : b.w);
}
__device__ __forceinline__ float vpick(bool c, const float &a, const float &b) { return c ? a : b; }

template <int V, int L, int K, bool FULL, bool OFF32, bool IS_MAX>
__global__ __launch_bounds__(kBlock) void gspmm_extreme_kernel(const SpmmArgs a) {
    using vec = typename Vec<V>::type;
    constexpr int FT = V * L * K;
    constexpr int G = 64 / L;
    constexpr int U = (K >= 2) ? 2 : 4;
    __shared__ __align__(16) int2 s_edge[kWavesPerBlock][fg::kItemEdges + kPad];
    __shared__ int32_t s_end[kWavesPerBlock][fg::kItemRows];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int tile = a.tile_base + (int)(blockIdx.x % (unsigned)a.n_ftiles);
    const int64_t item_id = (int64_t)(blockIdx.x / (unsigned)a.n_ftiles) * kWavesPerBlock + wave;
    if (item_id >= a.n_items) return;
    const Item it = a.items[item_id];
    const int g = lane / L, li = lane % L;
    const int rt = tile / a.sub_per_tile, st = tile % a.sub_per_tile;
    const int f_end = (rt + 1) * a.tile_w;
    const int f_lo = rt * a.tile_w + st * FT + li * V;
    bool on[K];
#pragma unroll
    for (int k = 0; k < K; ++k) on[k] = FULL || (f_lo + k * L * V < f_end);
    const uint32_t lane_bytes = (OFF32 && a.x_tile_bytes) ? (uint32_t)tile * a.x_tile_bytes + (uint32_t)(li * V) * 4u
                                                          : (uint32_t)f_lo * 4u;
    const uint32_t scale = OFF32 ? a.x_row_bytes : 1u;
    const int64_t voff = (int64_t)((rt * a.tile_w + st * FT) / a.head_len) * a.head_stride;
    const int64_t F = a.F;
    int2 *edge = s_edge[wave];
    int2 regs[4];
    vec acc[K];

    // running extreme over staged elements [b, e)
    auto walk = [&](int b, int e) {
        for (int s0 = b; s0 < e; s0 += G * U) {
            int2 cw[U];
            bool ok[U];
            vec xv[U][K];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int j = s0 + u * G + g;
                ok[u] = j < e;
                cw[u] = edge[ok[u] ? j : e - 1];
            }
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int k = 0; k < K; ++k)
                    if (FULL || on[k])
                        xv[u][k] = *reinterpret_cast<const vec *>(row_ptr<OFF32>(a.x, lane_bytes, F, cw[u].x) + k * L * V);
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int k = 0; k < K; ++k)
                    if (FULL || on[k]) {
                        vec m = acc[k];
                        vext<IS_MAX>(m, vscale(__int_as_float(cw[u].y), xv[u][k]));
                        acc[k] = vpick(ok[u], m, acc[k]);
                    }
        }
    };
    auto reset = [&]() {
#pragma unroll
        for (int k = 0; k < K; ++k) acc[k] = vsplat(vec(), ext_identity<IS_MAX>());
    };
    // combine the lane groups, store (an empty row stores 0)
    auto finish = [&](float *dst, bool empty) {
#pragma unroll
        for (int off = L; off < 64; off <<= 1)
#pragma unroll
            for (int k = 0; k < K; ++k) vext<IS_MAX>(acc[k], vshfl_xor(acc[k], off));
        if (g == 0) {
#pragma unroll
            for (int k = 0; k < K; ++k)
                if (FULL || on[k]) *reinterpret_cast<vec *>(dst + k * L * V) = empty ? vzero(vec()) : acc[k];
        }
    };

    if (it.info < -1) {
        const int nrows = -it.info;
        if (it.len > 0) {
            stage_load(a.indices, nullptr, a.vals, it.start, it.len, lane, scale, a.vstride, voff, regs);
            stage_store(edge, lane, regs);
        }
        s_end[wave][lane] = a.pos[it.row + min(lane, nrows - 1) + 1] - it.start;
        wave_lds_sync();
        int b = 0;
        for (int q = 0; q < nrows; ++q) {
            const int e = __builtin_amdgcn_readfirstlane(s_end[wave][q]);
            reset();
            walk(b, e);
            finish(a.out + (int64_t)(it.row + q) * F + f_lo, e == b);
            b = e;
        }
        return;
    }
    reset();
    for (int32_t base = 0; base < it.len; base += fg::kItemEdges) {
        const int n = min(fg::kItemEdges, it.len - base);
        wave_lds_sync();
        stage_load(a.indices, nullptr, a.vals, (int64_t)it.start + base, n, lane, scale, a.vstride, voff, regs);
        stage_store(edge, lane, regs);
        wave_lds_sync();
        walk(0, n);
    }
    float *dst = (it.info < 0 ? a.out + (int64_t)it.row * F : a.partial + (int64_t)it.info * F) + f_lo;
    finish(dst, it.len == 0);
}

// out[row, :] = max / min over the row's pieces.
template <int V, bool IS_MAX>
__global__ __launch_bounds__(256) void gspmm_extreme_fixup_kernel(const Fixup *fixups, int64_t n_fixups,
                                                                  const float *partial, float *out, int F) {
    using vec = typename Vec<V>::type;
    const int per_row = F / V;
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_fixups * per_row) return;
    const Fixup fx = fixups[t / per_row];
    const int f = (int)(t % per_row) * V;
    vec m = *reinterpret_cast<const vec *>(partial + (int64_t)fx.slot0 * F + f);
    for (int p = 1; p < fx.n_pieces; ++p)
        vext<IS_MAX>(m, *reinterpret_cast<const vec *>(partial + (int64_t)(fx.slot0 + p) * F + f));
    *reinterpret_cast<vec *>(out + (int64_t)fx.row * F + f) = m;
}

// ---- which element gave the extreme -------------------------------------------------------------
//
// arg[v, f] = stored position of the first element e of row v with vals[e] * X[indices[e], f] ==
// out[v, f] (out as written by the max / min kernel; -1 for a row without elements).  Same items
// and lane layout; the products are formed by the same multiplication, so the comparison is exact.
// Pieces of split rows combine through atomicMin on arg (set to INT_MAX beforehand).

// equal, or both NaN (a NaN extreme is matched by the first NaN message)
__device__ __forceinline__ bool same_value(float m, float t) { return m == t || (m != m && t != t); }
__device__ __forceinline__ int4 imin4(const int4 &a, const int4 &b) {
    return make_int4(min(a.x, b.x), min(a.y, b.y), min(a.z, b.z), min(a.w, b.w));
}
__device__ __forceinline__ int imin4(const int &a, const int &b) { return min(a, b); }
__device__ __forceinline__ int4 imatch(const float4 &m, const float4 &t, int e, const int4 &cur) {
    return make_int4(same_value(m.x, t.x) ? min(cur.x, e) : cur.x, same_value(m.y, t.y) ? min(cur.y, e) : cur.y,
                     same_value(m.z, t.z) ? min(cur.z, e) : cur.z, same_value(m.w, t.w) ? min(cur.w, e) : cur.w);
}
__device__ __forceinline__ int imatch(const float &m, const float &t, int e, const int &cur) { return same_value(m, t) ? min(cur, e) : cur; }
__device__ __forceinline__ int4 ishfl_xor(const int4 &a, int off) {
    return make_int4(__shfl_xor(a.x, off), __shfl_xor(a.y, off), __shfl_xor(a.z, off), __shfl_xor(a.w, off));
}
__device__ __forceinline__ int ishfl_xor(const int &a, int off) { return __shfl_xor(a, off); }
__device__ __forceinline__ int4 isplat(int4, int v) { return make_int4(v, v, v, v); }
__device__ __forceinline__ int isplat(int, int v) { return v; }
__device__ __forceinline__ int4 inone(const int4 &a) {      // INT_MAX (no match) -> -1
    return make_int4(a.x == INT_MAX ? -1 : a.x, a.y == INT_MAX ? -1 : a.y, a.z == INT_MAX ? -1 : a.z, a.w == INT_MAX ? -1 : a.w);
}
__device__ __forceinline__ int inone(const int &a) { return a == INT_MAX ? -1 : a; }
__device__ __forceinline__ void iatomic_min(int32_t *p, const int4 &a) {
    atomicMin(p, a.x); atomicMin(p + 1, a.y); atomicMin(p + 2, a.z); atomicMin(p + 3, a.w);
}
__device__ __forceinline__ void iatomic_min(int32_t *p, const int &a) { atomicMin(p, a); }
template <int V> struct IVec;
template <> struct IVec<4> { using type = int4; };
template <> struct IVec<1> { using type = int; };

template <int V, int L, int K, bool FULL>
__global__ __launch_bounds__(kBlock) void gspmm_arg_kernel(const SpmmArgs a) {
    using vec = typename Vec<V>::type;
    using ivec = typename IVec<V>::type;
    constexpr int FT = V * L * K;
    constexpr int G = 64 / L;
    constexpr int U = (K >= 2) ? 2 : 4;
    __shared__ __align__(16) int2 s_edge[kWavesPerBlock][fg::kItemEdges + kPad];
    __shared__ int32_t s_end[kWavesPerBlock][fg::kItemRows];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int tile = a.tile_base + (int)(blockIdx.x % (unsigned)a.n_ftiles);
    const int64_t item_id = (int64_t)(blockIdx.x / (unsigned)a.n_ftiles) * kWavesPerBlock + wave;
    if (item_id >= a.n_items) return;
    const Item it = a.items[item_id];
    const int g = lane / L, li = lane % L;
    const int rt = tile / a.sub_per_tile, st = tile % a.sub_per_tile;
    const int f_end = (rt + 1) * a.tile_w;
    const int f_lo = rt * a.tile_w + st * FT + li * V;
    bool on[K];
#pragma unroll
    for (int k = 0; k < K; ++k) on[k] = FULL || (f_lo + k * L * V < f_end);
    const uint32_t lane_bytes = (uint32_t)f_lo * 4u;
    const int64_t voff = (int64_t)((rt * a.tile_w + st * FT) / a.head_len) * a.head_stride;
    const int64_t F = a.F;
    int2 *edge = s_edge[wave];
    int2 regs[4];
    vec target[K];
    ivec acc[K];

    // `first` = stored position of staged element 0
    auto walk = [&](int b, int e, int first) {
        for (int s0 = b; s0 < e; s0 += G * U) {
            int2 cw[U];
            bool ok[U];
            vec xv[U][K];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int j = s0 + u * G + g;
                ok[u] = j < e;
                cw[u] = edge[ok[u] ? j : e - 1];
            }
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int k = 0; k < K; ++k)
                    if (FULL || on[k])
                        xv[u][k] = *reinterpret_cast<const vec *>(row_ptr<false>(a.x, lane_bytes, F, cw[u].x) + k * L * V);
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int k = 0; k < K; ++k)
                    if ((FULL || on[k]) && ok[u])
                        acc[k] = imatch(vscale(__int_as_float(cw[u].y), xv[u][k]), target[k], first + s0 + u * G + g, acc[k]);
        }
    };
    auto begin_row = [&](int64_t row) {
#pragma unroll
        for (int k = 0; k < K; ++k) {
            acc[k] = isplat(ivec(), INT_MAX);
            if (FULL || on[k]) target[k] = *reinterpret_cast<const vec *>(a.out + row * F + f_lo + k * L * V);
        }
    };
    auto combine = [&]() {
#pragma unroll
        for (int off = L; off < 64; off <<= 1)
#pragma unroll
            for (int k = 0; k < K; ++k) acc[k] = imin4(acc[k], ishfl_xor(acc[k], off));
    };

    if (it.info < -1) {
        const int nrows = -it.info;
        if (it.len > 0) {
            stage_load(a.indices, nullptr, a.vals, it.start, it.len, lane, 1u, a.vstride, voff, regs);
            stage_store(edge, lane, regs);
        }
        s_end[wave][lane] = a.pos[it.row + min(lane, nrows - 1) + 1] - it.start;
        wave_lds_sync();
        int b = 0;
        for (int q = 0; q < nrows; ++q) {
            const int e = __builtin_amdgcn_readfirstlane(s_end[wave][q]);
            begin_row(it.row + q);
            walk(b, e, it.start);
            combine();
            if (g == 0) {
#pragma unroll
                for (int k = 0; k < K; ++k)
                    if (FULL || on[k])
                        *reinterpret_cast<ivec *>(a.arg + (int64_t)(it.row + q) * F + f_lo + k * L * V) = inone(acc[k]);
            }
            b = e;
        }
        return;
    }
    begin_row(it.row);
    for (int32_t base = 0; base < it.len; base += fg::kItemEdges) {
        const int n = min(fg::kItemEdges, it.len - base);
        wave_lds_sync();
        stage_load(a.indices, nullptr, a.vals, (int64_t)it.start + base, n, lane, 1u, a.vstride, voff, regs);
        stage_store(edge, lane, regs);
        wave_lds_sync();
        walk(0, n, it.start + base);
    }
    combine();
    if (g == 0) {
        int32_t *dst = a.arg + (int64_t)it.row * F + f_lo;
#pragma unroll
        for (int k = 0; k < K; ++k)
            if (FULL || on[k]) {
                if (it.info < 0) *reinterpret_cast<ivec *>(dst + k * L * V) = inone(acc[k]);
                else iatomic_min(dst + k * L * V, acc[k]);       // a piece: the row's other pieces add theirs
            }
    }
}

// arg rows of split rows start at INT_MAX so that their pieces can take the minimum.
__global__ __launch_bounds__(256) void gspmm_arg_init_kernel(const Fixup *fixups, int64_t n_fixups, int32_t *arg, int F) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_fixups * F) return;
    arg[(int64_t)fixups[t / F].row * F + t % F] = INT_MAX;
}

template <int V, int L, int K>
void launch_arg_vlk(bool full, dim3 grid, hipStream_t st, const SpmmArgs &a) {
    if (full) hipLaunchKernelGGL((gspmm_arg_kernel<V, L, K, true>), grid, dim3(kBlock), 0, st, a);
    else hipLaunchKernelGGL((gspmm_arg_kernel<V, L, K, false>), grid, dim3(kBlock), 0, st, a);
}

template <int V>
int launch_arg_v(int L, int K, bool full, dim3 grid, hipStream_t st, const SpmmArgs &a) {
    if (K == 1) {
        switch (L) {
            case 4: launch_arg_vlk<V, 4, 1>(full, grid, st, a); return FG_OK;
            case 8: launch_arg_vlk<V, 8, 1>(full, grid, st, a); return FG_OK;
            case 16: launch_arg_vlk<V, 16, 1>(full, grid, st, a); return FG_OK;
            case 32: launch_arg_vlk<V, 32, 1>(full, grid, st, a); return FG_OK;
            case 64: launch_arg_vlk<V, 64, 1>(full, grid, st, a); return FG_OK;
        }
    } else if (L == 64 && K == 2) { launch_arg_vlk<V, 64, 2>(full, grid, st, a); return FG_OK; }
    else if (L == 64 && K == 4) { launch_arg_vlk<V, 64, 4>(full, grid, st, a); return FG_OK; }
    return FG_ERR_SHAPE;
}

// out[row, :] (+)= sum of the row's pieces, in piece order.  One lane per V columns.
// part_stride / out_stride (floats; 0 for a launch over one partition's fix-ups): with every pass in a buffer of
// its own, partition p's pieces start at partial + p * part_stride and its rows at out + p * out_stride.
template <int V>
__global__ __launch_bounds__(256) void spmm_fixup_kernel(const Fixup *fixups, int64_t n_fixups,
                                                         const float *partial, float *out, int F,
                                                         int accumulate, int64_t part_stride, int64_t out_stride) {
    using vec = typename Vec<V>::type;
    const int per_row = F / V;
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_fixups * per_row) return;
    const Fixup fx = fixups[t / per_row];
    const int f = (int)(t % per_row) * V;
    partial += fx.part * part_stride;
    out += fx.part * out_stride;
    vec sum = *reinterpret_cast<const vec *>(partial + (int64_t)fx.slot0 * F + f);
    for (int p = 1; p < fx.n_pieces; ++p)
        vadd(sum, *reinterpret_cast<const vec *>(partial + (int64_t)(fx.slot0 + p) * F + f));
    vec *o = reinterpret_cast<vec *>(out + (int64_t)fx.row * F + f);
    if (accumulate) vadd(sum, *o);
    *o = sum;
}

// out = buf[0] + buf[1] + ... + buf[P - 1], in that order (the order in which the passes would have added to out).
// Every word is read once and written once: non-temporal accesses, which leave the caches to the next operator's gathers
// (232,965-node graph, F=512: SpMM 11.39 -> 11.33 ms).
__global__ __launch_bounds__(256) void spmm_pass_sum_kernel(const float4 *buf, float4 *out, size_t words, int P) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= words) return;
    typedef float f4 __attribute__((ext_vector_type(4)));
    const f4 *b = reinterpret_cast<const f4 *>(buf);
    f4 s = __builtin_nontemporal_load(b + i);
    for (int p = 1; p < P; ++p) s += __builtin_nontemporal_load(b + (size_t)p * words + i);
    __builtin_nontemporal_store(s, reinterpret_cast<f4 *>(out) + i);
}

struct SpmmConfig {
    int V, L, K;
    int tile_w, sub_per_tile, n_ftiles;
    bool full;
    bool off32;     // every source row starts less than 4 GiB into X
    int hpt = 1;    // heads (with their own weights) per kernel tile
};

int pow2_ceil(int v) { int p = 1; while (p < v) p <<= 1; return p; }

// Picks vector width, lanes per row and loads per lane for feature length F cut into T
// requested tiles (T == 0: one tile).  `aligned16`: x and out are 16-byte aligned.
int choose_config(int F, int T, bool aligned16, SpmmConfig *c) {
    if (F < 1) return fail(FG_ERR_SHAPE, "feature length must be positive, got %d", F);
    if (T < 0) return fail(FG_ERR_ARG, "num_feat_partitions must be >= 0, got %d", T);
    if (T == 0) T = 1;
    if (F % T != 0) return fail(FG_ERR_SHAPE, "feature length %d is not divisible by num_feat_partitions %d", F, T);
    const int Fp = F / T;
    c->V = (aligned16 && F % 4 == 0 && Fp % 4 == 0) ? 4 : 1;
    const int lanes = Fp / c->V;
    if (lanes <= 64) { c->L = pow2_ceil(lanes) < 4 ? 4 : pow2_ceil(lanes); c->K = 1; }
    else { c->L = 64; c->K = (lanes >= 256 && c->V == 1) ? 4 : 2; }
    const int ft = c->V * c->L * c->K;
    c->tile_w = Fp;
    c->sub_per_tile = (Fp + ft - 1) / ft;
    c->n_ftiles = T * c->sub_per_tile;
    c->full = (Fp % ft == 0);
    return FG_OK;
}

template <int V, int L, int K, bool FULL, bool ACC>
void launch_off(bool off32, dim3 grid, hipStream_t st, const SpmmArgs &a) {
    if constexpr (K == 1) {
        if (off32) hipLaunchKernelGGL((spmm_items_kernel<V, L, K, FULL, ACC, true>), grid, dim3(kBlock), 0, st, a);
        else hipLaunchKernelGGL((spmm_items_kernel<V, L, K, FULL, ACC, false>), grid, dim3(kBlock), 0, st, a);
    } else {
        if (off32) hipLaunchKernelGGL((spmm_items_wide_kernel<V, L, K, FULL, ACC, true, 1>), grid, dim3(kBlock), 0, st, a);
        else hipLaunchKernelGGL((spmm_items_wide_kernel<V, L, K, FULL, ACC, false, 1>), grid, dim3(kBlock), 0, st, a);
    }
}

// tiles of HPT heads: 128-bit lanes, one load per lane, no masking
template <int L, int HPT>
void launch_hpt(bool off32, dim3 grid, hipStream_t st, const SpmmArgs &a) {
    if (a.accumulate) {
        if (off32) hipLaunchKernelGGL((spmm_items_wide_kernel<4, L, 1, true, true, true, HPT>), grid, dim3(kBlock), 0, st, a);
        else hipLaunchKernelGGL((spmm_items_wide_kernel<4, L, 1, true, true, false, HPT>), grid, dim3(kBlock), 0, st, a);
    } else {
        if (off32) hipLaunchKernelGGL((spmm_items_wide_kernel<4, L, 1, true, false, true, HPT>), grid, dim3(kBlock), 0, st, a);
        else hipLaunchKernelGGL((spmm_items_wide_kernel<4, L, 1, true, false, false, HPT>), grid, dim3(kBlock), 0, st, a);
    }
}

template <int V, int L, int K>
void launch_vlk(bool full, bool off32, dim3 grid, hipStream_t st, const SpmmArgs &a) {
    if (a.accumulate) {
        if (full) launch_off<V, L, K, true, true>(off32, grid, st, a);
        else launch_off<V, L, K, false, true>(off32, grid, st, a);
    } else {
        if (full) launch_off<V, L, K, true, false>(off32, grid, st, a);
        else launch_off<V, L, K, false, false>(off32, grid, st, a);
    }
}

template <int V>
int launch_v(const SpmmConfig &c, dim3 grid, hipStream_t st, const SpmmArgs &a) {
    if (c.hpt > 1) {
        if (V == 4 && c.K == 1 && c.full) {
            if (c.L == 16 && c.hpt == 2) { launch_hpt<16, 2>(c.off32, grid, st, a); return FG_OK; }
            if (c.L == 16 && c.hpt == 4) { launch_hpt<16, 4>(c.off32, grid, st, a); return FG_OK; }
            if (c.L == 8 && c.hpt == 4) { launch_hpt<8, 4>(c.off32, grid, st, a); return FG_OK; }
            if (c.L == 4 && c.hpt == 4) { launch_hpt<4, 4>(c.off32, grid, st, a); return FG_OK; }
        }
        return fail(FG_ERR_SHAPE, "no SpMM kernel for %d heads per tile with V=%d L=%d K=%d", c.hpt, V, c.L, c.K);
    }
    if (c.K == 1) {
        switch (c.L) {
            case 4: launch_vlk<V, 4, 1>(c.full, c.off32, grid, st, a); return FG_OK;
            case 8: launch_vlk<V, 8, 1>(c.full, c.off32, grid, st, a); return FG_OK;
            case 16: launch_vlk<V, 16, 1>(c.full, c.off32, grid, st, a); return FG_OK;
            case 32: launch_vlk<V, 32, 1>(c.full, c.off32, grid, st, a); return FG_OK;
            case 64: launch_vlk<V, 64, 1>(c.full, c.off32, grid, st, a); return FG_OK;
        }
    } else if (c.L == 64 && c.K == 2) { launch_vlk<V, 64, 2>(c.full, c.off32, grid, st, a); return FG_OK; }
    else if (c.L == 64 && c.K == 4) { launch_vlk<V, 64, 4>(c.full, c.off32, grid, st, a); return FG_OK; }
    return fail(FG_ERR_SHAPE, "no SpMM kernel for V=%d L=%d K=%d", V, c.L, c.K);
}

template <int V, int L, int K, bool IS_MAX>
void launch_ext_vlk(const SpmmConfig &c, dim3 grid, hipStream_t st, const SpmmArgs &a) {
    if (c.full) {
        if (c.off32) hipLaunchKernelGGL((gspmm_extreme_kernel<V, L, K, true, true, IS_MAX>), grid, dim3(kBlock), 0, st, a);
        else hipLaunchKernelGGL((gspmm_extreme_kernel<V, L, K, true, false, IS_MAX>), grid, dim3(kBlock), 0, st, a);
    } else {
        if (c.off32) hipLaunchKernelGGL((gspmm_extreme_kernel<V, L, K, false, true, IS_MAX>), grid, dim3(kBlock), 0, st, a);
        else hipLaunchKernelGGL((gspmm_extreme_kernel<V, L, K, false, false, IS_MAX>), grid, dim3(kBlock), 0, st, a);
    }
}

template <int V, bool IS_MAX>
int launch_ext_v(const SpmmConfig &c, dim3 grid, hipStream_t st, const SpmmArgs &a) {
    if (c.K == 1) {
        switch (c.L) {
            case 4: launch_ext_vlk<V, 4, 1, IS_MAX>(c, grid, st, a); return FG_OK;
            case 8: launch_ext_vlk<V, 8, 1, IS_MAX>(c, grid, st, a); return FG_OK;
            case 16: launch_ext_vlk<V, 16, 1, IS_MAX>(c, grid, st, a); return FG_OK;
            case 32: launch_ext_vlk<V, 32, 1, IS_MAX>(c, grid, st, a); return FG_OK;
            case 64: launch_ext_vlk<V, 64, 1, IS_MAX>(c, grid, st, a); return FG_OK;
        }
    } else if (c.L == 64 && c.K == 2) { launch_ext_vlk<V, 64, 2, IS_MAX>(c, grid, st, a); return FG_OK; }
    else if (c.L == 64 && c.K == 4) { launch_ext_vlk<V, 64, 4, IS_MAX>(c, grid, st, a); return FG_OK; }
    return fail(FG_ERR_SHAPE, "no max/min kernel for V=%d L=%d K=%d", V, c.L, c.K);
}

// Whether the sum / max / min kernels of this configuration gather from a tile-by-tile copy of X.
bool gathers_tile_major(const fg_spmm_plan *pl, const SpmmConfig &c, int F) {
    return c.off32 && c.V == 4 && c.K == 1 && c.full && c.sub_per_tile == 1 && pl->nnz > 0 &&
           fg::wants_tile_major(pl, c.n_ftiles, (uint64_t)pl->n_src * (uint64_t)F * 4u);
}

// The kernel configuration of one call: feature length F in `heads` heads, T requested tiles (0 = choose).
// heads > 1: every kernel tile must hold whole heads or lie inside one.
int resolve_config(const fg_spmm_plan *pl, int F, int T, int heads, int reduce, bool aligned16, SpmmConfig *c) {
    if (reduce != FG_REDUCE_SUM && reduce != FG_REDUCE_MAX && reduce != FG_REDUCE_MIN)
        return fail(FG_ERR_ARG, "unknown reduce op %d", reduce);
    if (reduce != FG_REDUCE_SUM && pl->num_col_partitions != 1)
        return fail(FG_ERR_ARG, "max / min aggregation needs a plan with one column partition");
    if (F < 1) return fail(FG_ERR_SHAPE, "feature length must be positive, got %d", F);
    if (heads < 1 || F % heads != 0) return fail(FG_ERR_SHAPE, "feature length %d is not divisible by %d heads", F, heads);
    int hpt = 1;
    if (heads > 1) {
        // A kernel tile holds whole heads or lies inside one: 64 floats when the head length divides
        // or is a multiple of 64, else (short heads) 4 heads; the sum kernel stages one weight per
        // head of the tile.
        const int D = F / heads;
        if (D % 4 != 0 || !aligned16) return fail(FG_ERR_SHAPE, "per-head weights need a head length that is a multiple of 4 and 16-byte aligned arrays, got %d", D);
        int tile;
        if (T == 0) {
            if (D % 64 == 0) tile = 64;
            else if ((D & (D - 1)) != 0) return fail(FG_ERR_SHAPE, "per-head weights need a head length that is a power of two or a multiple of 64, got %d", D);
            else if (D >= 16) tile = (reduce == FG_REDUCE_SUM && 64 % D == 0 && F % 64 == 0) ? 64 : D;
            else tile = (reduce == FG_REDUCE_SUM && heads % 4 == 0) ? 4 * D : 0;
            if (tile == 0) return fail(FG_ERR_SHAPE, "no kernel for %d heads of %d floats with this aggregation", heads, D);
            T = F / tile;
        } else {
            if (T < 1 || F % T != 0) return fail(FG_ERR_SHAPE, "feature length %d is not divisible by num_feat_partitions %d", F, T);
            tile = F / T;
        }
        if ((tile & (tile - 1)) != 0 || tile > 256 || tile < 16 || !(tile % D == 0 || D % tile == 0))
            return fail(FG_ERR_SHAPE, "num_feat_partitions %d does not cut %d-float heads into power-of-two tiles of 16..256 floats", T, D);
        if (tile > D) {
            hpt = tile / D;
            if (reduce != FG_REDUCE_SUM || !(hpt == 2 || hpt == 4) || tile > 64 || (tile == 64 ? false : hpt != 4))
                return fail(FG_ERR_SHAPE, "no kernel for tiles of %d floats holding %d heads", tile, hpt);
        }
    }
    int rc = choose_config(F, T, aligned16, c);
    if (rc != FG_OK) return rc;
    c->hpt = hpt;
    c->off32 = !pl->wide_offsets && (uint64_t)pl->n_src * (uint64_t)F * 4u < (1ull << 32);
    return FG_OK;
}

// Floats of split-row pieces at the start of the plan's scratch (a multiple of 4: what follows stays 16-byte aligned).
size_t piece_floats(const fg_spmm_plan *pl, int F) {
    return (((size_t)pl->max_slots_in_partition * (size_t)F) + 3) & ~(size_t)3;
}

// Whether the passes over the source partitions write buffers of their own that one last kernel adds up,
// instead of every later pass reading and rewriting `out`.  A wavefront's loads return in order, so a row of
// `out` that has to come from memory holds up the gathers issued behind it; without those reads a pass over
// the 232,965-node graph takes 1.37 instead of 1.52 ms at F = 512 and the sum of the 8 buffers 0.77 ms.  Passes
// that do not read each other's results need no ordering either, so one launch walks all partitions' items.
// Together (232,965-node graph): 12.11 -> 11.53 ms at F = 512, 6.19 -> 5.90 ms at F = 256, 3.13 -> 3.03 ms at F = 128,
// 1.76 -> 1.66 ms at F = 64, 0.93 -> 0.90 ms at F = 32.  Same sums in the same order: bit-identical results.
// The buffers take P times the output's size; beyond 8 GiB the passes add to `out` in place.
bool uses_pass_buffers(const fg_spmm_plan *pl, const SpmmConfig &c, int F, int reduce) {
    const int P = pl->num_col_partitions;
    if (P < 2 || reduce != FG_REDUCE_SUM || c.V != 4 || pl->pass_buffers == 2) return false;
    if (pl->pass_buffers == 1) return true;
    const uint64_t out_bytes = (uint64_t)pl->n_dst * (uint64_t)F * 4u;
    return out_bytes * (uint64_t)P <= (8ull << 30);
}

fg::ScratchNeed scratch_need(const fg_spmm_plan *pl, const SpmmConfig &c, int F, int reduce) {
    fg::ScratchNeed need;
    need.partial = piece_floats(pl, F);                                  // one row of F floats per piece of a split row
    if (uses_pass_buffers(pl, c, F, reduce))                             // every pass: pieces and a buffer of its own
        need.partial = (size_t)pl->num_col_partitions * (need.partial + (size_t)pl->n_dst * (size_t)F);
    if (gathers_tile_major(pl, c, F)) need.tiled = (size_t)pl->n_src * (size_t)F;
    return need;
}

// Kernel tiles per launch: 8, 4, 2 or 1 -- counts that divide the 8 XCDs, so that workgroup id % tiles-per-launch
// always puts a tile on the same XCDs and an L2 serves one tile's slice at a time (10 tiles: 8 + 2; 5: 4 + 1).  With
// any other count every XCD would see every tile (232,965-node graph, F=640: 27.4 ms with 10 tiles in one launch).
int tiles_this_launch(int remaining) {
    return remaining >= 8 ? 8 : remaining >= 4 ? 4 : remaining >= 2 ? 2 : 1;
}

// reduce: FG_REDUCE_SUM / MAX / MIN.  heads > 1: vals is [nnz, heads] (or [heads, nnz] when
// head_major).  vals == nullptr with allow_no_vals: every weight is 1.
int spmm_run(fg_spmm_plan *pl, const int32_t *pos, const int32_t *idx, const float *vals,
             const float *x, float *out, int F, int T, void *stream, int heads = 1,
             int reduce = FG_REDUCE_SUM, bool allow_no_vals = false, bool head_major = false,
             int32_t *arg_out = nullptr, float *fixed_partial = nullptr, size_t fixed_partial_floats = 0) {
    if (!pl) return fail(FG_ERR_ARG, "plan is null");
    if (arg_out && reduce == FG_REDUCE_SUM) return fail(FG_ERR_ARG, "positions of the selected elements exist for max / min only");
    if (int drc = fg::check_device(pl)) return drc;
    if (pl->n_dst == 0) return FG_OK;
    if (!out || !pos || (pl->nnz > 0 && (!idx || (!vals && !allow_no_vals) || !x)))
        return fail(FG_ERR_ARG, "null device pointer");
    const bool aligned16 = (((uintptr_t)x | (uintptr_t)out | (uintptr_t)arg_out) & 15) == 0;
    SpmmConfig c;
    int rc = resolve_config(pl, F, T, heads, reduce, aligned16, &c);
    if (rc != FG_OK) return rc;
    // fixed_partial: the split rows' partial sums go to this buffer of fixed size instead of the plan's,
    // X is gathered from the caller's matrix (no tile-by-tile copy), and nothing is allocated.
    fg::ScratchNeed need = scratch_need(pl, c, F, reduce);
    if (fixed_partial) {
        need.partial = piece_floats(pl, F);
        if (need.partial > fixed_partial_floats)
            return fail(FG_ERR_SHAPE, "the split rows of this plan need %zu floats of scratch at feature length %d; "
                        "the fixed buffer of this entry point holds %zu", need.partial, F, fixed_partial_floats);
        need.tiled = 0;
    } else if ((rc = fg::ensure_scratch(pl, need, stream)) != FG_OK) {
        return rc;
    }
    float *const partial = fixed_partial ? fixed_partial : pl->partial_dev;
    // per-pass buffers [P][n_dst][F] behind the pieces (every row of every buffer is written by its pass:
    // the plan holds an item or a fix-up for every row of every partition)
    const int P = pl->num_col_partitions;
    const size_t piece = piece_floats(pl, F);
    float *const pass_buf = (!fixed_partial && uses_pass_buffers(pl, c, F, reduce)) ? pl->partial_dev + (size_t)P * piece : nullptr;
    const size_t pass_stride = (size_t)pl->n_dst * (size_t)F;
    hipStream_t st = (hipStream_t)stream;
    const int64_t width = (pl->n_src + P - 1) / P;
    // With several feature tiles an XCD gathers one tile's 256 bytes (or less) out of every source
    // row, F * 4 bytes apart.  Gathered from a copy that stores each tile's slices back to back, the
    // same working set is cached markedly better (232,965-node graph, 8 partitions: 13.5 -> 11.9 ms
    // at F=512, 6.8 -> 6.1 ms at F=256, before the 0.25 / 0.13 ms that the copy takes); the sums
    // are the same, in the same order.
    const int ft = c.V * c.L * c.K;
    const bool tiled = need.tiled > 0;
    if (tiled && (rc = fg::make_tile_major(pl, x, pl->n_src, F, ft, stream)) != FG_OK) return rc;
    if (pass_buf && pl->n_items > 0) {
        // The passes are independent (each writes a buffer and pieces of its own), so one launch walks the items of all
        // partitions, partition by partition in workgroup order: the next partition's first workgroups fill the
        // compute units that the previous one's last workgroups leave idle, and seven launch gaps go away.
        SpmmArgs a;
        a.items = pl->items_dev; a.n_items = pl->n_items;
        a.item_off = pl->item_off_dev; a.n_parts = P;
        a.pos = pos; a.pos_stride = pl->n_dst + 1;
        a.indices = idx; a.indices16 = fg::narrow_indices(pl, idx); a.vals = vals;
        a.x = tiled ? pl->tiled_dev : x; a.x_stride = width * (tiled ? ft : F);
        a.x_row_bytes = (uint32_t)(tiled ? ft : F) * 4u;
        a.x_tile_bytes = tiled ? (uint32_t)((uint64_t)pl->n_src * ft * 4u) : 0u;
        a.out = pass_buf; a.out_stride = (int64_t)pass_stride;
        a.partial = partial; a.partial_stride = (int64_t)piece;
        a.F = F; a.tile_w = c.tile_w; a.sub_per_tile = c.sub_per_tile;
        a.heads = heads; a.head_len = F / heads;
        a.vstride = head_major ? 1 : heads; a.head_stride = head_major ? pl->nnz : 1;
        a.accumulate = 0;
        for (int tb = 0, per_launch; tb < c.n_ftiles; tb += per_launch) {
            per_launch = tiles_this_launch(c.n_ftiles - tb);
            a.n_ftiles = per_launch; a.tile_base = tb;
            const int64_t blocks = ((pl->n_items + kWavesPerBlock - 1) / kWavesPerBlock) * per_launch;
            if (blocks > 0x7fffffffLL) return fail(FG_ERR_SHAPE, "grid of %lld workgroups is too large", (long long)blocks);
            rc = (c.V == 4) ? launch_v<4>(c, dim3((unsigned)blocks), st, a) : launch_v<1>(c, dim3((unsigned)blocks), st, a);
            if (rc != FG_OK) return rc;
        }
    }
    if (pass_buf && pl->n_fixups > 0) {
        // the split rows of all partitions in one launch, each into its partition's buffer
        const int fv = (aligned16 && F % 4 == 0) ? 4 : 1;
        const int64_t threads = pl->n_fixups * (F / fv);
        const unsigned blocks = (unsigned)((threads + 255) / 256);
        if (fv == 4) hipLaunchKernelGGL(spmm_fixup_kernel<4>, dim3(blocks), dim3(256), 0, st, pl->fixups_dev, pl->n_fixups, partial, pass_buf, F, 0, (int64_t)piece, (int64_t)pass_stride);
        else hipLaunchKernelGGL(spmm_fixup_kernel<1>, dim3(blocks), dim3(256), 0, st, pl->fixups_dev, pl->n_fixups, partial, pass_buf, F, 0, (int64_t)piece, (int64_t)pass_stride);
    }
    for (int p = 0; p < P && !pass_buf; ++p) {
        const int64_t i0 = pl->item_off[p], i1 = pl->item_off[p + 1];
        if (i1 > i0) {
            SpmmArgs a;
            a.items = pl->items_dev + i0; a.n_items = i1 - i0;
            a.pos = pos + (int64_t)p * (pl->n_dst + 1);
            a.indices = idx; a.indices16 = fg::narrow_indices(pl, idx); a.vals = vals;
            a.x = tiled ? pl->tiled_dev + (int64_t)p * width * ft : x + (int64_t)p * width * F;
            a.x_row_bytes = (uint32_t)(tiled ? ft : F) * 4u;
            a.x_tile_bytes = tiled ? (uint32_t)((uint64_t)pl->n_src * ft * 4u) : 0u;
            a.out = out; a.partial = partial;
            a.F = F; a.tile_w = c.tile_w; a.sub_per_tile = c.sub_per_tile;
            a.heads = heads; a.head_len = F / heads;
            a.vstride = head_major ? 1 : heads; a.head_stride = head_major ? pl->nnz : 1;
            a.accumulate = p > 0;
            // More than 8 tiles: 8 at a time (one per XCD), so that an XCD's L2 serves one tile's
            // slice of this partition per launch; the partition's index arrays stay in the
            // memory-side cache between the launches.
            for (int tb = 0, per_launch; tb < c.n_ftiles; tb += per_launch) {
                per_launch = tiles_this_launch(c.n_ftiles - tb);
                a.n_ftiles = per_launch; a.tile_base = tb;
                const int64_t blocks = ((i1 - i0 + kWavesPerBlock - 1) / kWavesPerBlock) * per_launch;
                if (blocks > 0x7fffffffLL) return fail(FG_ERR_SHAPE, "grid of %lld workgroups is too large", (long long)blocks);
                const dim3 grid((unsigned)blocks);
                if (reduce == FG_REDUCE_SUM) rc = (c.V == 4) ? launch_v<4>(c, grid, st, a) : launch_v<1>(c, grid, st, a);
                else if (reduce == FG_REDUCE_MAX) rc = (c.V == 4) ? launch_ext_v<4, true>(c, grid, st, a) : launch_ext_v<1, true>(c, grid, st, a);
                else rc = (c.V == 4) ? launch_ext_v<4, false>(c, grid, st, a) : launch_ext_v<1, false>(c, grid, st, a);
                if (rc != FG_OK) return rc;
            }
        }
        const int64_t x0 = pl->fixup_off[p], x1 = pl->fixup_off[p + 1];
        if (x1 > x0) {
            const int fv = (aligned16 && F % 4 == 0) ? 4 : 1;
            const int64_t threads = (x1 - x0) * (F / fv);
            const unsigned blocks = (unsigned)((threads + 255) / 256);
            const Fixup *fx = pl->fixups_dev + x0;
            if (reduce == FG_REDUCE_SUM) {
                const int add = p > 0 ? 1 : 0;
                if (fv == 4) hipLaunchKernelGGL(spmm_fixup_kernel<4>, dim3(blocks), dim3(256), 0, st, fx, x1 - x0, partial, out, F, add, (int64_t)0, (int64_t)0);
                else hipLaunchKernelGGL(spmm_fixup_kernel<1>, dim3(blocks), dim3(256), 0, st, fx, x1 - x0, partial, out, F, add, (int64_t)0, (int64_t)0);
            } else if (reduce == FG_REDUCE_MAX) {
                if (fv == 4) hipLaunchKernelGGL((gspmm_extreme_fixup_kernel<4, true>), dim3(blocks), dim3(256), 0, st, fx, x1 - x0, partial, out, F);
                else hipLaunchKernelGGL((gspmm_extreme_fixup_kernel<1, true>), dim3(blocks), dim3(256), 0, st, fx, x1 - x0, partial, out, F);
            } else {
                if (fv == 4) hipLaunchKernelGGL((gspmm_extreme_fixup_kernel<4, false>), dim3(blocks), dim3(256), 0, st, fx, x1 - x0, partial, out, F);
                else hipLaunchKernelGGL((gspmm_extreme_fixup_kernel<1, false>), dim3(blocks), dim3(256), 0, st, fx, x1 - x0, partial, out, F);
            }
        }
    }
    if (pass_buf) {
        const size_t words = pass_stride / 4;
        hipLaunchKernelGGL(spmm_pass_sum_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, st,
                           reinterpret_cast<const float4 *>(pass_buf), reinterpret_cast<float4 *>(out), words, P);
    }
    if (arg_out) {
        // second sweep over the same items: which element equals the extreme that was just written
        SpmmArgs a;
        a.items = pl->items_dev; a.n_items = pl->n_items; a.pos = pos; a.indices = idx; a.vals = vals;
        a.x = x; a.out = out; a.partial = nullptr; a.arg = arg_out;
        a.F = F; a.tile_w = c.tile_w; a.sub_per_tile = c.sub_per_tile; a.n_ftiles = c.n_ftiles; a.tile_base = 0;
        a.accumulate = 0; a.heads = heads; a.head_len = F / heads;
        a.vstride = head_major ? 1 : heads; a.head_stride = head_major ? pl->nnz : 1;
        if (pl->n_fixups > 0) {
            const int64_t threads = pl->n_fixups * (int64_t)F;
            hipLaunchKernelGGL(gspmm_arg_init_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st,
                               pl->fixups_dev, pl->n_fixups, arg_out, F);
        }
        const int64_t blocks = ((pl->n_items + kWavesPerBlock - 1) / kWavesPerBlock) * c.n_ftiles;
        if (blocks > 0x7fffffffLL) return fail(FG_ERR_SHAPE, "grid of %lld workgroups is too large", (long long)blocks);
        if (blocks > 0) {
            rc = (c.V == 4) ? launch_arg_v<4>(c.L, c.K, c.full, dim3((unsigned)blocks), st, a)
                            : launch_arg_v<1>(c.L, c.K, c.full, dim3((unsigned)blocks), st, a);
            if (rc != FG_OK) return fail(FG_ERR_SHAPE, "no arg kernel for V=%d L=%d K=%d", c.V, c.L, c.K);
        }
    }
    FG_HIP_TRY(hipGetLastError());
    return FG_OK;
}

}  // namespace

namespace fg {
int spmm_scratch_need(const fg_spmm_plan *pl, int F, int heads, int reduce, int T, ScratchNeed *need) {
    SpmmConfig c;
    if (int rc = resolve_config(pl, F, T, heads, reduce, true, &c)) return rc;
    *need = scratch_need(pl, c, F, reduce);
    return FG_OK;
}
std::string spmm_launch_text(const fg_spmm_plan *pl, int F, int T) {
    SpmmConfig c;
    if (choose_config(F, T, true, &c) != FG_OK) return std::string("  launch           : ") + fg_last_error() + "\n";
    char b[512];
    const int64_t per_part = pl->item_off.size() > 1 ? pl->item_off[1] - pl->item_off[0] : 0;
    snprintf(b, sizeof(b),
             "  feature length   : %d, %d requested tile(s) of %d, %d kernel tile(s) of %d floats\n"
             "  kernel           : %s<V=%d, L=%d, K=%d, FULL=%d, ACC=pass>0>; %d element(s) per step\n"
             "  launch           : %d pass(es); first pass grid %lld x block %d; fixup rows %lld\n",
             F, c.n_ftiles / c.sub_per_tile, c.tile_w, c.n_ftiles, c.V * c.L * c.K,
             c.K == 1 ? "spmm_items_kernel" : "spmm_items_wide_kernel", c.V, c.L, c.K,
             (int)c.full, 64 / c.L, pl->num_col_partitions,
             (long long)(((per_part + kWavesPerBlock - 1) / kWavesPerBlock) * c.n_ftiles), kBlock,
             (long long)pl->n_fixups);
    std::string text = b;
    c.off32 = !pl->wide_offsets && (uint64_t)pl->n_src * (uint64_t)F * 4u < (1ull << 32);
    text += gathers_tile_major(pl, c, F) ? "  source features  : gathered from a tile-by-tile copy made at the start of every call\n"
                                         : "  source features  : gathered from the caller's row-major matrix\n";
    if (pl->num_col_partitions > 1)
        text += uses_pass_buffers(pl, c, F, FG_REDUCE_SUM) ? "  passes           : one launch walks all partitions, each into a buffer of its own; one last kernel adds the buffers into out\n"
                                                           : "  passes           : later passes add to out in place\n";
    return text;
}
}  // namespace fg

extern "C" int fg_spmm_csr_f32(fg_spmm_plan *plan, const int32_t *indptr_dev,
                               const int32_t *indices_dev, const float *vals_dev, const float *x_dev,
                               float *out_dev, int F, int num_feat_partitions, void *stream) {
    if (plan && plan->num_col_partitions != 1)
        return fail(FG_ERR_ARG, "fg_spmm_csr_f32 needs a plan with one column partition; use fg_spmm_dds_f32");
    return spmm_run(plan, indptr_dev, indices_dev, vals_dev, x_dev, out_dev, F, num_feat_partitions, stream);
}

// ---- an SpMM entry point that allocates nothing ------------------------------------------------
//
// The split rows' partial sums (one row of F floats per piece) live in a file-scope device array
// instead of plan-owned memory.  Every device the library runs on holds its own copy of the array
// until the process ends; its address on a device is looked up once, with that device current.
namespace {
constexpr size_t kFixedScratchFloats = (size_t)4 << 20;          // 16 MiB
static __device__ __align__(256) float scratch[kFixedScratchFloats];

constexpr int kMaxDevices = 64;
float *g_scratch_ptr[kMaxDevices];                                // address of `scratch` per device, once known
std::mutex g_scratch_mutex;

// The device address of `scratch` on the current device `dev` (the array's name is a host-side
// handle, never an address a kernel could use).
int fixed_scratch(int dev, float **ptr) {
    if (dev < 0 || dev >= kMaxDevices) return fail(FG_ERR_ARG, "device %d: at most %d devices are supported", dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return fail(FG_ERR_HIP, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = static_cast<float *>(p);
    }
    *ptr = g_scratch_ptr[dev];
    return FG_OK;
}
}  // namespace

namespace fg {
// Called by fg_spmm_plan_create (never under stream capture), so that fg_spmm_csr_noalloc_f32 finds the address known
// when its first call on this device is being recorded into a graph.  A failure here is reported by that call instead.
void prepare_fixed_scratch(int dev) {
    float *ptr = nullptr;
    (void)fixed_scratch(dev, &ptr);
}
}  // namespace fg

extern "C" int fg_spmm_csr_noalloc_f32(const fg_spmm_plan *plan, const int32_t *indptr_dev,
                                       const int32_t *indices_dev, const float *vals_dev, const float *x_dev,
                                       float *out_dev, int F, int num_feat_partitions, void *stream) {
    if (!plan) return fail(FG_ERR_ARG, "plan is null");
    if (plan->num_col_partitions != 1)
        return fail(FG_ERR_ARG, "fg_spmm_csr_noalloc_f32 needs a plan with one column partition");
    if (int drc = fg::check_device(plan)) return drc;        // the plan's device is the current one
    float *ptr = nullptr;
    if (int rc = fixed_scratch(plan->device, &ptr)) return rc;
    // The plan is only read here: every buffer the kernels write is the caller's or the fixed array.
    return spmm_run(const_cast<fg_spmm_plan *>(plan), indptr_dev, indices_dev, vals_dev, x_dev, out_dev, F,
                    num_feat_partitions, stream, 1, FG_REDUCE_SUM, false, false, nullptr, ptr, kFixedScratchFloats);
}

extern "C" int fg_spmm_dds_f32(fg_spmm_plan *plan, const int32_t *s1_pos_dev,
                               const int32_t *s1_idx_dev, const float *vals_dev, const float *x_dev,
                               float *out_dev, int F, int num_feat_partitions, void *stream) {
    return spmm_run(plan, s1_pos_dev, s1_idx_dev, vals_dev, x_dev, out_dev, F, num_feat_partitions, stream);
}

extern "C" int fg_gspmm_f32(fg_spmm_plan *plan, const int32_t *pos_dev, const int32_t *idx_dev,
                            const float *vals_dev, const float *x_dev, float *out_dev, int F, int heads,
                            int vals_head_major, int reduce, int num_feat_partitions, void *stream) {
    return spmm_run(plan, pos_dev, idx_dev, vals_dev, x_dev, out_dev, F, num_feat_partitions, stream, heads,
                    reduce, /*allow_no_vals=*/true, vals_head_major != 0);
}

extern "C" int fg_gspmm_arg_f32(fg_spmm_plan *plan, const int32_t *indptr_dev, const int32_t *indices_dev,
                                const float *vals_dev, const float *x_dev, float *out_dev, int32_t *arg_dev, int F,
                                int heads, int vals_head_major, int reduce, int num_feat_partitions, void *stream) {
    if (!arg_dev) return fail(FG_ERR_ARG, "fg_gspmm_arg_f32: arg_dev is null");
    return spmm_run(plan, indptr_dev, indices_dev, vals_dev, x_dev, out_dev, F, num_feat_partitions, stream, heads,
                    reduce, /*allow_no_vals=*/true, vals_head_major != 0, arg_dev);
}

namespace {
// dst[h, e] = src[pos[e], h] (pos == nullptr: src[e, h]): one lane per element, the element's
// heads are read together and written to the heads' own contiguous arrays.
__global__ __launch_bounds__(256) void edge_values_head_major_kernel(const float *src, const int32_t *pos,
                                                                     int64_t n, int H, float *dst) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n) return;
    const float *s = src + (pos ? (int64_t)pos[e] : e) * H;
    for (int h = 0; h < H; ++h) dst[(int64_t)h * n + e] = s[h];
}
// One head, weights in another order: dst[e] = src[pos[e]], four consecutive elements per lane (their positions by one
// 128-bit load, the results by one 128-bit store; pos and dst 16-byte aligned).
__global__ __launch_bounds__(256) void edge_values_permute_kernel(const float *src, const int32_t *pos, int64_t n, float *dst) {
    const int64_t e = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (e >= n) return;
    if (e + 4 <= n) {
        const int4 p = *reinterpret_cast<const int4 *>(pos + e);
        *reinterpret_cast<float4 *>(dst + e) = make_float4(src[p.x], src[p.y], src[p.z], src[p.w]);
    } else {
        for (int64_t i = e; i < n; ++i) dst[i] = src[pos[i]];
    }
}
// The same for H = 4 * Q heads and a 16-byte aligned src: an element's heads by Q 128-bit loads, two elements per lane
// (a block apart, so that every store of a wavefront still covers 64 consecutive elements of one head).
template <int Q>
__global__ __launch_bounds__(256) void edge_values_head_major_vec_kernel(const float *src, const int32_t *pos,
                                                                         int64_t n, float *dst) {
    constexpr int H = 4 * Q;
    const int64_t e0 = (int64_t)blockIdx.x * 512 + threadIdx.x;
    float4 v[2][Q];
    bool ok[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int64_t e = e0 + 256 * j;
        ok[j] = e < n;
        const int64_t ec = ok[j] ? e : n - 1;                  // clamped: no branch around the loads
        const float4 *s = reinterpret_cast<const float4 *>(src + (pos ? (int64_t)pos[ec] : ec) * H);
#pragma unroll
        for (int q = 0; q < Q; ++q) v[j][q] = s[q];
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        if (!ok[j]) continue;
        float *d = dst + e0 + 256 * j;
#pragma unroll
        for (int q = 0; q < Q; ++q) {
            d[(int64_t)(4 * q + 0) * n] = v[j][q].x;
            d[(int64_t)(4 * q + 1) * n] = v[j][q].y;
            d[(int64_t)(4 * q + 2) * n] = v[j][q].z;
            d[(int64_t)(4 * q + 3) * n] = v[j][q].w;
        }
    }
}
}  // namespace

extern "C" int fg_edge_values_head_major_f32(const float *src_dev, const int32_t *edge_pos_dev, int64_t n_edges,
                                             int heads, float *dst_dev, void *stream) {
    if (n_edges < 0 || heads < 1) return fail(FG_ERR_ARG, "fg_edge_values_head_major_f32: bad size");
    if (n_edges == 0) return FG_OK;
    if (!src_dev || !dst_dev) return fail(FG_ERR_ARG, "null device pointer");
    const int64_t blocks = (n_edges + 255) / 256;
    if (blocks > 0x7fffffffLL) return fail(FG_ERR_SHAPE, "too many edges for one grid");
    hipStream_t st = (hipStream_t)stream;
    const dim3 wide((unsigned)((n_edges + 511) / 512));
    const bool aligned = ((uintptr_t)src_dev & 15) == 0;
    if (heads == 1 && edge_pos_dev && (((uintptr_t)edge_pos_dev | (uintptr_t)dst_dev) & 15) == 0)
        hipLaunchKernelGGL(edge_values_permute_kernel, dim3((unsigned)((n_edges + 1023) / 1024)), dim3(256), 0, st,
                           src_dev, edge_pos_dev, n_edges, dst_dev);
    else if (aligned && heads == 4)
        hipLaunchKernelGGL(edge_values_head_major_vec_kernel<1>, wide, dim3(256), 0, st, src_dev, edge_pos_dev, n_edges, dst_dev);
    else if (aligned && heads == 8)
        hipLaunchKernelGGL(edge_values_head_major_vec_kernel<2>, wide, dim3(256), 0, st, src_dev, edge_pos_dev, n_edges, dst_dev);
    else if (aligned && heads == 16)
        hipLaunchKernelGGL(edge_values_head_major_vec_kernel<4>, wide, dim3(256), 0, st, src_dev, edge_pos_dev, n_edges, dst_dev);
    else
        hipLaunchKernelGGL(edge_values_head_major_kernel, dim3((unsigned)blocks), dim3(256), 0, st,
                           src_dev, edge_pos_dev, n_edges, heads, dst_dev);
    FG_HIP_TRY(hipGetLastError());
    return FG_OK;
}
