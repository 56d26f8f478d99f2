// Dot-product attention over the edges of a graph, in one sweep per source-column partition:
//
//   s[e, h]   = scale * <K[col e, h, :], Q[row e, h, :]>
//   a[e, h]   = softmax of s[., h] over the edges of row(e)
//   out[v, h, :] = sum over the edges e of row v of a[e, h] * V[col e, h, :]
//
// i.e. multi-head SDDMM, edge softmax and per-head weighted SpMM without ever storing the [nnz, H]
// scores: every lane group keeps a running maximum, a running sum of exponentials and the running
// weighted sum of its row (rescaled whenever the maximum grows), and source-column partitions are
// merged the same way through `out` and a small [n_dst, H, 2] state array.  Not in the reference (no
// attention operator exists there); the result is defined by the composition of the three operators.
//
// Layout of the work: one head (16, 32 or 64 floats) per kernel tile, the tile index fastest in the
// workgroup id so that every XCD gathers one head's slices of K and V; items, staging and the
// tile-by-tile copies of the gathered operands are those of the SpMM kernels.
#include <hip/hip_runtime.h>

#include <cmath>

#include "fg_common.h"
#include "fg_device.h"

using fg::fail;
using fg::Item;
using fg::group_sum;
using fg::wave_lds_sync;

namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kBlock = 64 * kWavesPerBlock;
constexpr int kPad = 8;
constexpr int kU = 4;                  // elements per lane group whose gathers are issued back to back

struct AttnArgs {
    const Item *items;
    int64_t n_items;
    const int32_t *pos;       // this partition's row boundaries
    const int32_t *indices;   // partition-local column ids
    const uint16_t *indices16 = nullptr;   // the plan's 16-bit copy of them, read instead (null: none)
    const float *q;           // [n_dst, F]
    const float *k, *v;       // offset to the partition's first source row
    uint32_t kv_row_bytes;    // bytes between consecutive rows of k / v
    uint32_t kv_tile_bytes;   // k / v stored head by head: bytes from one head's block to the next; 0: rows of F floats
    float *out;               // [n_dst, F]: running weighted sums (divided by the sum of exponentials at the end)
    float *state;             // [n_dst, H, 2]: running maximum and sum of exponentials
    int F, H;
    int n_heads, head_base;   // heads of this launch
    float scale;
    // additive scores: q = er [H, n_dst] and k = el [H, n_src] (k offset to the partition's first source), one
    // scalar per vertex and head; floats from one head's block to the next; negative slope of the leaky ReLU
    int64_t q_head_floats, k_head_floats;
    float slope;
    // One launch over the items of all source partitions, every partition into buffers of its own (FIRST in every
    // pass): the plan's item_off on the device (n_parts + 1 entries; null: one partition's items, strides unused) and
    // the distance from one partition's pos / k / v / out / state to the next, in elements.
    const int64_t *item_off = nullptr;
    int n_parts = 1;
    int64_t pos_stride = 0, k_stride = 0, v_stride = 0, out_stride = 0, state_stride = 0;
};

// Running softmax-weighted sum of one lane group: maximum, sum of exponentials, weighted sum.
struct Running {
    float m, l;
    float4 acc;
};

__device__ __forceinline__ Running running_empty() { return {-INFINITY, 0.f, make_float4(0.f, 0.f, 0.f, 0.f)}; }

// r <- r and s merged (both relative to their own maxima).
__device__ __forceinline__ void running_merge(Running &r, const Running &s) {
    const float m = fmaxf(r.m, s.m);
    if (m == -INFINITY) return;               // both empty
    const float fr = __expf(r.m - m), fs = __expf(s.m - m);      // exp(-inf) = 0 for the empty side
    r.acc.x = r.acc.x * fr + s.acc.x * fs; r.acc.y = r.acc.y * fr + s.acc.y * fs;
    r.acc.z = r.acc.z * fr + s.acc.z * fs; r.acc.w = r.acc.w * fr + s.acc.w * fs;
    r.l = r.l * fr + s.l * fs;
    r.m = m;
}

// What is staged per element: the byte offset of its row in K / V, and, for additive scores, its scalar
// el[col, h] as well (gathered once per item, 64 elements per load, instead of once per step).
template <bool ADD> struct Staged;
template <> struct Staged<false> { using type = int32_t; };
template <> struct Staged<true> { using type = int2; };
__device__ __forceinline__ uint32_t slice_off(int32_t c) { return (uint32_t)c; }
__device__ __forceinline__ uint32_t slice_off(const int2 &c) { return (uint32_t)c.x; }
__device__ __forceinline__ float staged_scalar(int32_t) { return 0.f; }
__device__ __forceinline__ float staged_scalar(const int2 &c) { return __int_as_float(c.y); }

// NU elements of one row, those with valid[u] counted: all gathers are issued before the first is used,
// then the scores and the running update.
//   ADD == false: score = scale * <K[c, h, :], q>  (k: the K slices, this lane's 16 bytes at lane_bytes);
//   ADD == true : score = leaky_relu(el + q.x) with negative slope `scale`  (el: the element's staged scalar).
template <int L, int NU, bool ADD, typename S>
__device__ __forceinline__ void update(const S (&c)[NU], const bool (&valid)[NU], const float *k, const float *v,
                                       uint32_t lane_bytes, const float4 &q, float scale, Running &r) {
    float4 kk[NU], vv[NU];
    float ev[NU];
#pragma unroll
    for (int u = 0; u < NU; ++u) {
        if constexpr (ADD) ev[u] = staged_scalar(c[u]);
        else kk[u] = *reinterpret_cast<const float4 *>(reinterpret_cast<const char *>(k) + (slice_off(c[u]) + lane_bytes));
        vv[u] = *reinterpret_cast<const float4 *>(reinterpret_cast<const char *>(v) + (slice_off(c[u]) + lane_bytes));
    }
    float s[NU];
    float m = r.m;
#pragma unroll
    for (int u = 0; u < NU; ++u) {
        float t;
        if constexpr (ADD) {
            const float z = ev[u] + q.x;
            t = z > 0.f ? z : z * scale;
        } else {
            const float d = kk[u].x * q.x + kk[u].y * q.y + kk[u].z * q.z + kk[u].w * q.w;
            t = group_sum<L>(d) * scale;                // every lane takes part in the cross-lane sum
        }
        s[u] = valid[u] ? t : -INFINITY;
        m = fmaxf(m, s[u]);
    }
    if (m == -INFINITY) return;             // nothing finite so far (uniform inside a lane group)
    const float f = __expf(r.m - m);
    r.acc.x *= f; r.acc.y *= f; r.acc.z *= f; r.acc.w *= f;
    r.l *= f;
    r.m = m;
#pragma unroll
    for (int u = 0; u < NU; ++u) {
        const float p = __expf(s[u] - m);      // 0 for a slot without an element
        r.l += p;
        // such a slot's V slice (a re-read or a later row's element) is dropped by a select: a product
        // with p = 0 would turn a non-finite row of V into NaN in rows that do not reference it
        const float4 w = valid[u] ? vv[u] : make_float4(0.f, 0.f, 0.f, 0.f);
        r.acc.x += p * w.x; r.acc.y += p * w.y; r.acc.z += p * w.z; r.acc.w += p * w.w;
    }
}

// NU steps of one row for this lane group: staged elements s0 + g, s0 + g + G, ...; every step but the
// last lies wholly below e, and in the last one (unless ALLVALID) a group whose element would be e or
// beyond re-reads element e - 1 and gives it no weight.
template <int L, int NU, bool ALLVALID, bool ADD, typename S>
__device__ __forceinline__ void walk_batch(const S *cols, int s0, int e, int g, const float *k, const float *v,
                                           uint32_t lane_bytes, const float4 &q, float scale, Running &r) {
    constexpr int G = 64 / L;
    const bool last_valid = ALLVALID || s0 + (NU - 1) * G + g < e;
    S c[NU];
    bool valid[NU];
#pragma unroll
    for (int u = 0; u < NU; ++u) {
        valid[u] = u < NU - 1 || last_valid;
        c[u] = cols[valid[u] ? s0 + u * G + g : e - 1];
    }
    update<L, NU, ADD>(c, valid, k, v, lane_bytes, q, scale, r);
}

// Staged elements [b, e) of one row, shared by the G lane groups; the last batch is issued with exactly
// the steps it has left.
template <int L, bool ADD, typename S>
__device__ __forceinline__ void walk(const S *cols, int b, int e, int g, const float *k, const float *v,
                                     uint32_t lane_bytes, const float4 &q, float scale, Running &r) {
    constexpr int G = 64 / L;
    int s0 = b;
    for (; s0 + G * kU <= e; s0 += G * kU) walk_batch<L, kU, true, ADD>(cols, s0, e, g, k, v, lane_bytes, q, scale, r);
    if (s0 >= e) return;
    const int nu = (e - s0 + G - 1) / G;    // uniform: 1 .. kU
    static_assert(kU == 4, "the tail below lists the step counts");
    if (nu == 1) walk_batch<L, 1, false, ADD>(cols, s0, e, g, k, v, lane_bytes, q, scale, r);
    else if (nu == 2) walk_batch<L, 2, false, ADD>(cols, s0, e, g, k, v, lane_bytes, q, scale, r);
    else if (nu == 3) walk_batch<L, 3, false, ADD>(cols, s0, e, g, k, v, lane_bytes, q, scale, r);
    else walk_batch<L, 4, false, ADD>(cols, s0, e, g, k, v, lane_bytes, q, scale, r);
}

// kU consecutive staged elements j .. j + kU - 1 of this lane group's own row (those below e count; the
// slots behind them hold later rows' elements or the padding: loadable, given no weight).
template <int L, bool ADD, typename S>
__device__ __forceinline__ void own_batch(const S *cols, int j, int e, const float *k, const float *v,
                                          uint32_t lane_bytes, const float4 &q, float scale, Running &r) {
    S c[kU];
    bool valid[kU];
#pragma unroll
    for (int u = 0; u < kU; ++u) {
        c[u] = cols[j + u];
        valid[u] = j + u < e;
    }
    update<L, kU, ADD>(c, valid, k, v, lane_bytes, q, scale, r);
}

// What the earlier partitions left for a row (read before the row's gathers are issued).
template <bool FIRST>
__device__ __forceinline__ Running load_state(const float *out_row, const float *state_row) {
    Running old = running_empty();
    if (!FIRST) {
        old.m = state_row[0]; old.l = state_row[1];
        old.acc = *reinterpret_cast<const float4 *>(out_row);
    }
    return old;
}

// Merges the lane groups' running sums (every group ends with the row's), then, in later passes, the
// row's state from the earlier partitions, and stores the row.
template <int L, bool FIRST>
__device__ __forceinline__ void finish_row(Running r, const Running &old, int g, int li, float *out_row, float *state_row) {
#pragma unroll
    for (int off = L; off < 64; off <<= 1) {
        Running o;
        o.m = __shfl_xor(r.m, off); o.l = __shfl_xor(r.l, off);
        o.acc = make_float4(__shfl_xor(r.acc.x, off), __shfl_xor(r.acc.y, off), __shfl_xor(r.acc.z, off), __shfl_xor(r.acc.w, off));
        running_merge(r, o);
    }
    if (g != 0) return;
    if (!FIRST) running_merge(r, old);
    if constexpr (FIRST) {
        // written once and read back by another kernel (or a later pass): a non-temporal store leaves the L2 to the gathered rows
        typedef float f4 __attribute__((ext_vector_type(4)));
        f4 t; t.x = r.acc.x; t.y = r.acc.y; t.z = r.acc.z; t.w = r.acc.w;
        __builtin_nontemporal_store(t, reinterpret_cast<f4 *>(out_row));
    } else {
        *reinterpret_cast<float4 *>(out_row) = r.acc;
    }
    if (li == 0) { state_row[0] = r.m; state_row[1] = r.l; }
}

// L lanes x 128 bits cover one head.  FIRST: the pass writes every row's state -- the first partition's pass, or
// every partition's when each has buffers of its own (one launch over all partitions, merged afterwards);
// otherwise later passes merge into the stored state and skip rows without elements in their partition.
// ADD: scores are leaky_relu(el[col e, h] + er[row e, h]) (a.k = el and a.q = er, one scalar per vertex and head,
// head by head) instead of scaled dot products of K and Q slices.
template <int L, bool FIRST, bool ADD>
__global__ __launch_bounds__(kBlock) void attention_items_kernel(const AttnArgs a) {
    constexpr int G = 64 / L, D = 4 * L;
    using S = typename Staged<ADD>::type;
    __shared__ __align__(16) S s_col[kWavesPerBlock][fg::kItemEdges + kPad];
    __shared__ int32_t s_end[kWavesPerBlock][fg::kItemRows];
    __shared__ int32_t s_next[kWavesPerBlock];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int head = a.head_base + (int)(blockIdx.x % (unsigned)a.n_heads);
    const int64_t item_id = (int64_t)(blockIdx.x / (unsigned)a.n_heads) * kWavesPerBlock + wave;
    if (item_id >= a.n_items) return;
    const Item it = a.items[item_id];
    // the partition this item belongs to (uniform per wavefront)
    int part = 0;
    if (a.item_off) {
        const int64_t id = ((int64_t)__builtin_amdgcn_readfirstlane((int)(item_id >> 32)) << 32) |
                           (uint32_t)__builtin_amdgcn_readfirstlane((int)item_id);
        while (part + 1 < a.n_parts && id >= a.item_off[part + 1]) ++part;
    }
    const int32_t *const pos_p = a.pos + part * a.pos_stride;
    const float *const k_p = a.k + part * a.k_stride;
    const float *const v_p = a.v + part * a.v_stride;
    float *const out_p = a.out + part * a.out_stride;
    float *const state_p = a.state + part * a.state_stride;
    const int g = lane / L, li = lane % L;
    const int f_lo = head * D + li * 4;
    const uint32_t lane_bytes = a.kv_tile_bytes ? (uint32_t)head * a.kv_tile_bytes + (uint32_t)li * 16u : (uint32_t)f_lo * 4u;
    const int64_t F = a.F;
    S *cols = s_col[wave];
    // ADD: this head's scalars; the score's second parameter is the negative slope
    const float *kptr = ADD ? k_p + (int64_t)head * a.k_head_floats : k_p;
    const float *q_head = a.q + (int64_t)head * a.q_head_floats;
    const float sparam = ADD ? a.slope : a.scale;

    auto stage = [&](int64_t base, int n) {
        int32_t c[4];
        fg::load_four_ids(a.indices, a.indices16, base, n, lane, c);
        uint32_t b[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) b[i] = (uint32_t)c[i] * a.kv_row_bytes;
        if constexpr (ADD) {
            int ev[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) ev[i] = __float_as_int(kptr[c[i]]);
            int4 *c4 = reinterpret_cast<int4 *>(cols);
            c4[2 * lane] = make_int4((int)b[0], ev[0], (int)b[1], ev[1]);
            c4[2 * lane + 1] = make_int4((int)b[2], ev[2], (int)b[3], ev[3]);
            if (lane < kPad) cols[fg::kItemEdges + lane] = make_int2((int)b[3], ev[3]);
        } else {
            *reinterpret_cast<int4 *>(cols + 4 * lane) = make_int4((int)b[0], (int)b[1], (int)b[2], (int)b[3]);
            if (lane < kPad) cols[fg::kItemEdges + lane] = (int)b[3];
        }
    };
    // the row's own operand: its slice of Q, or (ADD) its scalar in .x
    auto own_q = [&](int64_t row) {
        if constexpr (ADD) return make_float4(q_head[row], 0.f, 0.f, 0.f);
        else return *reinterpret_cast<const float4 *>(a.q + row * F + f_lo);
    };
    auto out_row = [&](int64_t row) { return out_p + row * F + f_lo; };
    auto state_row = [&](int64_t row) { return state_p + (row * a.H + head) * 2; };

    if (it.info < -1) {
        // several whole rows, at most 256 elements: staged once
        const int nrows = -it.info;
        // The rows of Q (and, in later passes, the rows' earlier sums) are read once here, one word per row
        // and 128 bytes, while the column ids are on their way: loads return in order, so a row fetched
        // from memory when it is needed would hold up every gather behind it.
        float touched = 0.f;
        constexpr int kLines = (D * 4 + 127) / 128;
        static_assert(fg::kItemRows * kLines <= 128, "two touches per lane cover an item's rows");
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int t = lane + 64 * i;
            const int64_t at = (int64_t)(it.row + min(t / kLines, nrows - 1)) * F + head * D + min((t % kLines) * 32, D - 1);
            if (!ADD) touched += a.q[at];
            if (!FIRST) touched += out_p[at];
        }
        if (it.len > 0) stage(it.start, it.len);
        s_end[wave][lane] = pos_p[it.row + min(lane, nrows - 1) + 1] - it.start;
        if (lane == 0) s_next[wave] = 0;
        wave_lds_sync();
        asm volatile("" ::"v"(touched));      // keeps the loads
        if (nrows >= 2 * G && it.len <= nrows * 2 * kU) {
            // Many rows of a few elements: every lane group takes rows of its own (next free row from a
            // counter in LDS), walks the row's elements kU at a time and stores the row itself, so G rows are
            // in flight per wavefront and nothing crosses lane groups.  (Rows of 30 elements are faster
            // shared: 26.7 against 27.6 ms at H=8, D=64 on the 232,965-node graph with 16 partitions.)
            int r = -1, j = 0, e = 0;
            bool done = false, live = false;
            float4 q = make_float4(0.f, 0.f, 0.f, 0.f);
            Running run = running_empty(), old = running_empty();
            for (;;) {
                if (!done && j >= e) {
                    if (live) {                      // the row this group just finished
                        if (!FIRST) running_merge(run, old);
                        *reinterpret_cast<float4 *>(out_row(it.row + r)) = run.acc;
                        if (li == 0) { float *st = state_row(it.row + r); st[0] = run.m; st[1] = run.l; }
                    }
                    int rn = 0;
                    if (li == 0) rn = atomicAdd(&s_next[wave], 1);
                    r = __shfl(rn, g * L);
                    if (r >= nrows) {
                        done = true;
                    } else {
                        j = r ? s_end[wave][r - 1] : 0;
                        e = s_end[wave][r];
                        live = FIRST || e > j;
                        if (live) {
                            q = own_q(it.row + r);
                            old = load_state<FIRST>(out_row(it.row + r), state_row(it.row + r));
                            run = running_empty();
                        }
                    }
                }
                if (__all(done)) break;
                if (!done && j < e) {
                    own_batch<L, ADD>(cols, j, e, kptr, v_p, lane_bytes, q, sparam, run);
                    j += kU;
                }
            }
            return;
        }
        int b = 0;
        for (int r = 0; r < nrows; ++r) {
            const int e = __builtin_amdgcn_readfirstlane(s_end[wave][r]);
            if (e > b || FIRST) {
                const float4 q = own_q(it.row + r);
                const Running old = load_state<FIRST>(out_row(it.row + r), state_row(it.row + r));
                Running run = running_empty();
                walk<L, ADD>(cols, b, e, g, kptr, v_p, lane_bytes, q, sparam, run);
                finish_row<L, FIRST>(run, old, g, li, out_row(it.row + r), state_row(it.row + r));
            }
            b = e;
        }
        return;
    }
    // one row of any length: 256 elements at a time
    const float4 q = own_q(it.row);
    const Running old = load_state<FIRST>(out_row(it.row), state_row(it.row));
    Running run = running_empty();
    for (int32_t base = 0; base < it.len; base += fg::kItemEdges) {
        const int n = min(fg::kItemEdges, it.len - base);
        wave_lds_sync();
        stage((int64_t)it.start + base, n);
        wave_lds_sync();
        walk<L, ADD>(cols, 0, n, g, kptr, v_p, lane_bytes, q, sparam, run);
    }
    if (it.len > 0 || FIRST) finish_row<L, FIRST>(run, old, g, li, out_row(it.row), state_row(it.row));
}

// out[v, h, :] /= state[v, h].sum (rows without edges: 0).
__global__ __launch_bounds__(256) void attention_finish_kernel(float4 *out, const float *state, uint32_t n_words,
                                                               uint32_t row_words, uint32_t head_words, int H) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= n_words) return;
    const uint32_t r = i / row_words, h = (i - r * row_words) / head_words;
    const float l = state[((uint64_t)r * H + h) * 2 + 1];
    float4 o = out[i];
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    o.x *= inv; o.y *= inv; o.z *= inv; o.w *= inv;
    out[i] = l > 0.f ? o : make_float4(0.f, 0.f, 0.f, 0.f);
}

// The partitions' buffers merged, partition after partition, and the row divided by its sum of exponentials:
// out[r, h, :] and state[r, h] = (maximum, sum) from buf_out [P][n_dst][F] and buf_state [P][n_dst][H][2].
__global__ __launch_bounds__(256) void attention_merge_kernel(float4 *out, float *state, const float4 *buf_out,
                                                              const float *buf_state, uint32_t n_words, uint32_t row_words,
                                                              uint32_t head_words, int H, int P) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= n_words) return;
    const uint32_t r = i / row_words, w = i - r * row_words, h = w / head_words;
    const uint64_t srow = ((uint64_t)r * H + h) * 2, sstride = (uint64_t)(n_words / row_words) * H * 2;
    // the row's maximum over the partitions first, so that every buffer enters with one factor and the loads of the
    // running sums do not wait for each other
    float m = -INFINITY;
    for (int p = 0; p < P; ++p) m = fmaxf(m, buf_state[p * sstride + srow]);
    Running run = running_empty();
    if (m != -INFINITY) {
        run.m = m;
#pragma unroll 4
        for (int p = 0; p < P; ++p) {
            const float f = __expf(buf_state[p * sstride + srow] - m);      // exp(-inf) = 0 for a partition without elements
            typedef float f4 __attribute__((ext_vector_type(4)));
            const f4 a = __builtin_nontemporal_load(reinterpret_cast<const f4 *>(buf_out) + (uint64_t)p * n_words + i);   // read once
            run.acc.x += a.x * f; run.acc.y += a.y * f; run.acc.z += a.z * f; run.acc.w += a.w * f;
            run.l += buf_state[p * sstride + srow + 1] * f;
        }
    }
    const float inv = run.l > 0.f ? 1.0f / run.l : 0.f;
    out[i] = run.l > 0.f ? make_float4(run.acc.x * inv, run.acc.y * inv, run.acc.z * inv, run.acc.w * inv)
                         : make_float4(0.f, 0.f, 0.f, 0.f);
    if (w == h * head_words) { state[srow] = run.m; state[srow + 1] = run.l; }
}

template <int L, bool ADD>
void launch(bool first, dim3 grid, hipStream_t st, const AttnArgs &a) {
    if (first) hipLaunchKernelGGL((attention_items_kernel<L, true, ADD>), grid, dim3(kBlock), 0, st, a);
    else hipLaunchKernelGGL((attention_items_kernel<L, false, ADD>), grid, dim3(kBlock), 0, st, a);
}

// The passes over the source partitions.  ADD == false: q / k are the [n, F] operands of the dot products and
// `param` their scale; ADD == true: q = er [H, n_dst], k = el [H, n_src] and `param` the leaky ReLU's slope.
template <bool ADD>
int run_forward(fg_spmm_plan *pl, const int32_t *pos_dev, const int32_t *idx_dev, const float *q_dev,
                const float *k_dev, const float *v_dev, float *out_dev, float *row_state_dev, int heads,
                int head_len, float param, void *stream) {
    if (!pl) return fail(FG_ERR_ARG, "plan is null");
    if (int drc = fg::check_device(pl)) return drc;
    if (heads < 1 || !(head_len == 16 || head_len == 32 || head_len == 64))
        return fail(FG_ERR_SHAPE, "attention takes heads of 16, 32 or 64 floats, got %d heads of %d", heads, head_len);
    if (pl->n_fixups > 0)
        return fail(FG_ERR_ARG, "attention needs a plan without split rows (fg_plan_opts.split_threshold = INT32_MAX)");
    if (pl->n_dst == 0) return FG_OK;
    if (!pos_dev || !q_dev || !out_dev || (pl->nnz > 0 && (!idx_dev || !k_dev || !v_dev)))
        return fail(FG_ERR_ARG, "null device pointer");
    if ((((uintptr_t)v_dev | (uintptr_t)out_dev | (ADD ? 0 : ((uintptr_t)q_dev | (uintptr_t)k_dev))) & 15) != 0)
        return fail(FG_ERR_ARG, "attention needs 16-byte aligned arrays");
    const int F = heads * head_len;
    if ((uint64_t)pl->n_src * (uint64_t)F * 4u >= (1ull << 32) || (uint64_t)pl->n_dst * (uint64_t)F >= (1ull << 32))
        return fail(FG_ERR_SHAPE, "attention operands of 4 GiB and more are not supported");
    fg::ScratchNeed need;
    int rc = fg::attention_scratch_need(pl, heads, head_len, ADD, !row_state_dev, &need);
    if (rc == FG_OK) rc = fg::ensure_scratch(pl, need, stream);
    if (rc != FG_OK) return rc;
    if (!row_state_dev) row_state_dev = pl->partial_dev;
    hipStream_t st = (hipStream_t)stream;
    const int P = pl->num_col_partitions;
    const int64_t width = (pl->n_src + P - 1) / P;
    // the gathered [n_src, F] operands head by head, as the SpMM kernels gather X tile by tile
    const bool tiled = need.tiled > 0;
    const float *k = k_dev, *v = v_dev;
    if (tiled) {
        const int slots = ADD ? 1 : 2;
        if ((rc = fg::make_tile_major(pl, v_dev, pl->n_src, F, head_len, stream, 0, slots)) != FG_OK) return rc;
        v = pl->tiled_dev;
        if (!ADD) {
            if ((rc = fg::make_tile_major(pl, k_dev, pl->n_src, F, head_len, stream, 1, slots)) != FG_OK) return rc;
            k = pl->tiled_dev + (size_t)pl->n_src * F;
        }
    }
    const int row_floats = tiled ? head_len : F;
    const size_t own_state = row_state_dev == pl->partial_dev ? (size_t)pl->n_dst * heads * 2 : 0;
    const size_t buf_out_floats = (size_t)pl->n_dst * F, buf_state_floats = (size_t)pl->n_dst * heads * 2;
    if (fg::attention_pass_buffers(pl, heads, head_len) && pl->n_items > 0) {
        // Every partition into buffers of its own (no reads of the rows' earlier state inside the gather kernel, no
        // order between the passes): one launch walks all partitions' items, one kernel merges the buffers.
        float *buf_out = pl->partial_dev + ((own_state + 3) & ~(size_t)3);
        float *buf_state = buf_out + (size_t)P * buf_out_floats;
        AttnArgs a;
        a.items = pl->items_dev; a.n_items = pl->n_items; a.item_off = pl->item_off_dev; a.n_parts = P;
        a.pos = pos_dev; a.pos_stride = pl->n_dst + 1;
        a.indices = idx_dev; a.indices16 = fg::narrow_indices(pl, idx_dev); a.q = q_dev;
        a.k = k; a.k_stride = ADD ? width : width * row_floats;
        a.v = v; a.v_stride = width * row_floats;
        a.kv_row_bytes = (uint32_t)row_floats * 4u;
        a.kv_tile_bytes = tiled ? (uint32_t)((uint64_t)pl->n_src * head_len * 4u) : 0u;
        a.out = buf_out; a.out_stride = (int64_t)buf_out_floats;
        a.state = buf_state; a.state_stride = (int64_t)buf_state_floats;
        a.F = F; a.H = heads; a.scale = param; a.slope = param;
        a.q_head_floats = ADD ? pl->n_dst : 0; a.k_head_floats = ADD ? pl->n_src : 0;
        const int per_launch = (heads > 8 && heads % 8 == 0) ? 8 : heads;
        for (int hb = 0; hb < heads; hb += per_launch) {
            a.n_heads = per_launch; a.head_base = hb;
            const int64_t blocks = ((pl->n_items + kWavesPerBlock - 1) / kWavesPerBlock) * per_launch;
            if (blocks > 0x7fffffffLL) return fail(FG_ERR_SHAPE, "grid of %lld workgroups is too large", (long long)blocks);
            const dim3 grid((unsigned)blocks);
            if (head_len == 64) launch<16, ADD>(true, grid, st, a);
            else if (head_len == 32) launch<8, ADD>(true, grid, st, a);
            else launch<4, ADD>(true, grid, st, a);
        }
        const uint32_t n_words = (uint32_t)((uint64_t)pl->n_dst * F / 4);
        hipLaunchKernelGGL(attention_merge_kernel, dim3((n_words + 255u) / 256u), dim3(256), 0, st,
                           reinterpret_cast<float4 *>(out_dev), row_state_dev, reinterpret_cast<const float4 *>(buf_out), buf_state,
                           n_words, (uint32_t)(F / 4), (uint32_t)(head_len / 4), heads, P);
        FG_HIP_TRY(hipGetLastError());
        return FG_OK;
    }
    for (int p = 0; p < P; ++p) {
        const int64_t i0 = pl->item_off[p], i1 = pl->item_off[p + 1];
        if (i1 == i0) continue;
        AttnArgs a;
        a.items = pl->items_dev + i0; a.n_items = i1 - i0;
        a.pos = pos_dev + (int64_t)p * (pl->n_dst + 1);
        a.indices = idx_dev; a.indices16 = fg::narrow_indices(pl, idx_dev); a.q = q_dev;
        a.k = ADD ? k + (int64_t)p * width : k + (int64_t)p * width * row_floats;
        a.v = v + (int64_t)p * width * row_floats;
        a.kv_row_bytes = (uint32_t)row_floats * 4u;
        a.kv_tile_bytes = tiled ? (uint32_t)((uint64_t)pl->n_src * head_len * 4u) : 0u;
        a.out = out_dev; a.state = row_state_dev; a.F = F; a.H = heads; a.scale = param; a.slope = param;
        a.q_head_floats = ADD ? pl->n_dst : 0; a.k_head_floats = ADD ? pl->n_src : 0;
        const int per_launch = (heads > 8 && heads % 8 == 0) ? 8 : heads;
        for (int hb = 0; hb < heads; hb += per_launch) {
            a.n_heads = per_launch; a.head_base = hb;
            const int64_t blocks = ((i1 - i0 + kWavesPerBlock - 1) / kWavesPerBlock) * per_launch;
            if (blocks > 0x7fffffffLL) return fail(FG_ERR_SHAPE, "grid of %lld workgroups is too large", (long long)blocks);
            const dim3 grid((unsigned)blocks);
            if (head_len == 64) launch<16, ADD>(p == 0, grid, st, a);
            else if (head_len == 32) launch<8, ADD>(p == 0, grid, st, a);
            else launch<4, ADD>(p == 0, grid, st, a);
        }
    }
    const uint32_t n_words = (uint32_t)((uint64_t)pl->n_dst * F / 4);
    hipLaunchKernelGGL(attention_finish_kernel, dim3((n_words + 255u) / 256u), dim3(256), 0, st,
                       reinterpret_cast<float4 *>(out_dev), row_state_dev, n_words, (uint32_t)(F / 4),
                       (uint32_t)(head_len / 4), heads);
    FG_HIP_TRY(hipGetLastError());
    return FG_OK;
}

}  // namespace

namespace fg {
// Whether the forward passes over the source partitions write buffers of their own ([P][n_dst][F] running sums and
// [P][n_dst][H][2] maxima / sums of exponentials) that one kernel merges: several partitions, unless the plan's
// pass_buffers option says never or the buffers would take more than 8 GiB.
bool attention_pass_buffers(const fg_spmm_plan *pl, int heads, int head_len) {
    const int P = pl->num_col_partitions;
    if (P < 2 || pl->pass_buffers == 2) return false;
    const uint64_t floats = (uint64_t)pl->n_dst * heads * (head_len + 2);
    return floats * 4u * (uint64_t)P <= (8ull << 30);
}
// The rows' (max, sum) state when the caller passes none, and the head-by-head copies of the gathered
// operands (V, and K for dot-product scores); the gradient kernels need the same copies and no state.
int attention_scratch_need(const fg_spmm_plan *pl, int heads, int head_len, bool additive, bool own_row_state,
                           ScratchNeed *need, bool forward) {
    if (heads < 1 || !(head_len == 16 || head_len == 32 || head_len == 64))
        return fail(FG_ERR_SHAPE, "attention takes heads of 16, 32 or 64 floats, got %d heads of %d", heads, head_len);
    const uint64_t F = (uint64_t)heads * head_len;
    need->partial = own_row_state ? (size_t)pl->n_dst * heads * 2 : 0;
    if (forward && attention_pass_buffers(pl, heads, head_len))
        need->partial = ((need->partial + 3) & ~(size_t)3) +
                        (size_t)pl->num_col_partitions * ((size_t)pl->n_dst * F + (size_t)pl->n_dst * heads * 2);
    need->tiled = 0;
    if (pl->nnz > 0 && wants_tile_major(pl, heads, (uint64_t)pl->n_src * F * 4u))
        need->tiled = (size_t)pl->n_src * F * (additive ? 1 : 2);
    return FG_OK;
}
}  // namespace fg

extern "C" int fg_graph_attention_f32(fg_spmm_plan *pl, const int32_t *pos_dev, const int32_t *idx_dev,
                                      const float *q_dev, const float *k_dev, const float *v_dev, float *out_dev,
                                      float *row_state_dev, int heads, int head_len, float scale, void *stream) {
    return run_forward<false>(pl, pos_dev, idx_dev, q_dev, k_dev, v_dev, out_dev, row_state_dev, heads, head_len, scale, stream);
}

extern "C" int fg_graph_attention_additive_f32(fg_spmm_plan *pl, const int32_t *pos_dev, const int32_t *idx_dev,
                                               const float *er_dev, const float *el_dev, const float *v_dev,
                                               float *out_dev, float *row_state_dev, int heads, int head_len,
                                               float negative_slope, void *stream) {
    return run_forward<true>(pl, pos_dev, idx_dev, er_dev, el_dev, v_dev, out_dev, row_state_dev, heads, head_len,
                             negative_slope, stream);
}
