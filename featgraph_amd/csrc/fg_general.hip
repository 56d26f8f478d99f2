// Generalised SpMM / SDDMM with broadcasting, for gfx950: the two operands of the message may live on the
// source nodes (u: indexed by the element's column), the destination nodes (v: its row) or the stored
// elements themselves (e), and their feature shapes may differ as long as they broadcast against each
// other.  The caller describes the broadcast by two index arrays: output feature f takes operand feature
// lhs_off[f] and rhs_off[f] (a null array is the identity).
//
//   SpMM : out[v, f]  = reduce over the elements e of row v of  lhs[.., lhs_off[f]] op rhs[.., rhs_off[f]]
//   SDDMM: out[e, f]  = lhs[.., lhs_off[f]] op rhs[.., rhs_off[f]]           (element-wise operators)
//          out[e, f]  = sum_{i < R} lhs[.., lhs_off[f] * R + i] * rhs[.., rhs_off[f] * R + i]   (dot)
//
// No counterpart in the reference, whose operators are the weighted sum (python/featgraph/op/vanilla_spmm.py)
// and the dot product (python/featgraph/op/vanilla_sddmm.py); the message / reduce vocabulary is the one its
// README.md:9-11 names ("generalized SpMM and SDDMM").
//
// The SpMM kernel walks the plan's work items, one wavefront each, like the weighted-sum kernel.  A lane holds
// V output features (V = 4 with 128-bit accesses when the shapes allow it, else 1); a group of L lanes
// (L = the power of two that covers the F / V vectors, at most 64) takes one element at a time and the
// 64 / L groups take different elements of the row, several steps in flight (in an item of many short rows
// every group takes a row of its own instead); feature axes of 128 floats and more, in multiples of 64, are cut
// into 64-float tiles for different workgroups when an operand is gathered (each L2 then holds one tile's slice of
// the gathered rows); other long axes are walked 64 vectors at a time.  With one group (64 vectors or more, no
// tiles), and for rows that a group has to itself, a row's sum is formed in the stored element order.  The edge operand, when there is one, is the dominant stream ([nnz, len] floats read once,
// coalesced, past the caches); the node operand is gathered, through column words that the wavefront has staged
// in LDS for the whole item.
//
// Over a plan with several source-column partitions (fg_gspmm_bcast_dds_f32) one launch walks all partitions'
// items in partition order, so that the gathered operand's rows of the current partition stay in the L2s: a
// partition's row segments are reduced into a buffer of its own and a closing kernel combines the buffers in
// partition order.  The elements then come in the partitioned layout's order and reach the operands on the edges
// (and the reported positions) through the layout's element -> stored position array.
#include <hip/hip_runtime.h>

#include <climits>
#include <type_traits>

#include "fg_common.h"
#include "fg_device.h"

using fg::fail;
using fg::Fixup;
using fg::Item;
using fg::wave_lds_sync;

// Every message is one correctly rounded float32 operation and every sum adds the rounded messages one by
// one, so that max / min, the selected positions and (with one lane group per row) the sums in stored
// order can be compared bit for bit with a sequential float32 evaluation.  This file is therefore compiled
// with -ffp-contract=off (featgraph_amd/build.py); a pragma alone does not stop the back end from fusing
// when the command line says -ffp-contract=fast.

namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kBlock = 64 * kWavesPerBlock;
constexpr int kStage = 256;             // elements whose index words a wavefront keeps in LDS at a time

struct GenArgs {
    const Item *items;
    int64_t n_items;
    const int32_t *indptr;
    const int32_t *indices;
    const uint16_t *indices16;   // the plan's 16-bit copy of `indices`, read instead of it (null: none)
    const float *lhs, *rhs;
    const int32_t *lhs_off, *rhs_off;
    int lhs_len, rhs_len;
    int lhs_target, rhs_target;
    float sign;                  // -1: the launch computes a minimum as the negated maximum of the negated messages; else 1
    const float *row_scale;      // out[v, :] *= row_scale[v] (null: 1), applied where a row is completed
    float *out;
    int32_t *arg;                // optional: stored position of the selected element (max / min)
    float *partial;              // pieces of split rows: [slot][F] values
    int32_t *partial_arg;        //                       [slot][F] positions
    int F, L;
    // PART: the elements are not addressed by their own positions -- several source-column partitions (indptr /
    // indices are the partitioned layout's position and local column arrays, item_off the plan's item ranges per
    // partition, out / arg the partitions' buffers; strides in elements, per partition), or edge operands that the
    // caller keeps in another order: edge_pos gives every element's row in the edge operands (and the position that
    // is reported for it).
    const int64_t *item_off;
    const int32_t *edge_pos;
    int n_parts;
    int n_tiles, tile_vecs;      // the feature axis in n_tiles tiles of tile_vecs vectors (V floats each), one per workgroup
    int final;                   // the kernel's rows are results (one partition), not a partition's share of them
    int64_t pos_stride, col_width, out_stride, partial_stride;
};

// The operand features of a lane's V outputs: V consecutive ones (CONTIG: one 128-bit load) or one value V times.
// NT: a non-temporal load, for an operand on the stored elements, which is read once from end to end and should not
// displace the gathered operand's rows from the L2.
typedef float nt_f4 __attribute__((ext_vector_type(4)));
template <int V, bool CONTIG, bool NT = false>
__device__ __forceinline__ void load_operand(const float *p, float (&o)[V]) {
    if (V == 4 && CONTIG && NT) {
        const nt_f4 t = __builtin_nontemporal_load(reinterpret_cast<const nt_f4 *>(p));
        o[0] = t.x; o[1 % V] = t.y; o[2 % V] = t.z; o[3 % V] = t.w;
    } else if (V == 4 && CONTIG) {
        const float4 t = *reinterpret_cast<const float4 *>(p);
        o[0] = t.x; o[1 % V] = t.y; o[2 % V] = t.z; o[3 % V] = t.w;
    } else {
        const float s = *p;
#pragma unroll
        for (int i = 0; i < V; ++i) o[i] = s;
    }
}

template <int OP> __device__ __forceinline__ float binary(float l, float r) {
    return OP == FG_BIN_ADD ? l + r : OP == FG_BIN_SUB ? l - r : OP == FG_BIN_MUL ? l * r
         : OP == FG_BIN_DIV ? l / r : OP == FG_BIN_COPY_LHS ? l : r;
}
template <int OP> constexpr bool kUsesLhs = OP != FG_BIN_COPY_RHS;
template <int OP> constexpr bool kUsesRhs = OP != FG_BIN_COPY_LHS;

template <int RED> __device__ __forceinline__ float identity() {
    return RED == FG_REDUCE_SUM ? 0.f : RED == FG_REDUCE_MAX ? -INFINITY : INFINITY;
}
// Max / min treat a NaN message as beating every number, so that it reaches the row's result the way it does through
// a sum (what numpy's maximum / minimum reductions and argmax / argmin do): the running extreme of (acc, m).
template <int RED> __device__ __forceinline__ float extreme(float acc, float m) {
    // once acc is a NaN no comparison with it holds and it stays; a NaN m enters through m != m
    return ((RED == FG_REDUCE_MAX ? m > acc : m < acc) || m != m) ? m : acc;
}
// Whether candidate (m, at element em) replaces (acc, at element ea): the better value (a NaN is better than any
// number), or the same value (two NaNs count as the same) at an earlier element; the first value always enters.
template <int RED> __device__ __forceinline__ bool replaces(float m, int em, float acc, int ea) {
    const bool m_nan = m != m, acc_nan = acc != acc;
    const bool better = m_nan ? !acc_nan : (!acc_nan && (RED == FG_REDUCE_MAX ? m > acc : m < acc));
    const bool same = m_nan ? acc_nan : m == acc;
    return em != INT_MAX && (ea == INT_MAX || better || (same && em < ea));
}

// LC / RC (V == 4 only): the operand's 4 features are consecutive (one 128-bit load), else one value 4 times.
// No branch stands between the loads of a step: one around a load would make the wavefront wait for everything
// issued before it.
// PART: see GenArgs; with several partitions (a.final == 0) a row segment without elements keeps the reduction's
// identity and no row is scaled, both being the combining kernel's business.
// LNT / RNT: see load_operand.  RED: FG_REDUCE_SUM or FG_REDUCE_MAX; a minimum runs as the maximum of the negated
// messages (a.sign = -1; negation is exact, so values, ties and selected positions are those of the minimum).
template <int OP, int RED, bool ARG, int V, bool LC, bool RC, bool LNT, bool RNT, bool PART>
__global__ __launch_bounds__(kBlock) void gspmm_bcast_kernel(const GenArgs a) {
    static_assert(RED == FG_REDUCE_SUM || RED == FG_REDUCE_MAX, "a minimum is a maximum with a.sign = -1");
    constexpr bool kLhs = kUsesLhs<OP>, kRhs = kUsesRhs<OP>;
    const float sign = RED == FG_REDUCE_SUM ? 1.f : a.sign;
    const bool final = !PART || a.final != 0;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    // workgroup id = item block * n_tiles + tile: the XCDs, dealt workgroups in turn, work on different feature tiles
    // of the same items, so that each L2 holds one tile's slice of the gathered rows
    const int tile = (int)(blockIdx.x % (unsigned)a.n_tiles);
    const int64_t item_id = (int64_t)(blockIdx.x / (unsigned)a.n_tiles) * kWavesPerBlock + wave;
    if (item_id >= a.n_items) return;
    const Item it = a.items[item_id];
    const int L = a.L, G = 64 / L, g = lane / L, li = lane % L;
    const int F = a.F, FV = F / V;
    const int fv_lo = tile * a.tile_vecs, fv_hi = min(FV, fv_lo + a.tile_vecs);
    int part = 0;
    if (PART) {
        const int64_t id = ((int64_t)__builtin_amdgcn_readfirstlane((int)(item_id >> 32)) << 32) |
                           (uint32_t)__builtin_amdgcn_readfirstlane((int)item_id);
        while (part + 1 < a.n_parts && id >= a.item_off[part + 1]) ++part;
    }
    const int32_t *const pos_p = a.indptr + (PART ? part * a.pos_stride : 0);
    const int64_t ubase = PART ? part * a.col_width : 0;       // the partition's first column
    float *const out_p = a.out + (PART ? part * a.out_stride : 0);
    int32_t *const arg_p = ARG ? a.arg + (PART ? part * a.out_stride : 0) : nullptr;
    float *const partial_p = a.partial + (PART ? part * a.partial_stride : 0);
    int32_t *const partial_arg_p = ARG ? a.partial_arg + (PART ? part * a.partial_stride : 0) : nullptr;
    const bool l_on_e = a.lhs_target == FG_TARGET_E, r_on_e = a.rhs_target == FG_TARGET_E;
    constexpr int U = V == 4 ? 4 : 8;     // elements in flight per lane group: the loads of a step are issued before its sums

    // The column and the stored position of up to kStage consecutive elements, read once with coalesced loads: the
    // gathers of a step then wait for LDS, not for a load of their own index words.
    __shared__ int2 s_el[kWavesPerBlock][kStage];
    int2 *const el = s_el[wave];
    auto stage = [&](int64_t c0, int n) {
        for (int t = lane; t < n; t += 64) {
            const int col = a.indices16 ? (int)a.indices16[c0 + t] : a.indices[c0 + t];      // uniform choice
            el[t] = make_int2(col + (int)ubase, PART ? a.edge_pos[c0 + t] : (int)(c0 + t));
        }
        wave_lds_sync();
    };

    // the elements [e0, e1) of output row v: reduce and store to (dst_v, dst_a); `done`: the row is complete.
    // staged_at >= 0: the range lies inside the elements staged from that position on; else it is staged here, kStage
    // elements at a time (a lane group keeps its elements and their order: kStage is a multiple of the groups).
    // own (a std::bool_constant): false = the wavefront's lane groups share the row, taking every G-th element each, and
    // their results are combined; true = every lane group has a row of its own (e0, e1, v and the destinations differ
    // from group to group, `mine` says whether the group has a row at all), walks it element by element in stored
    // order and stores it itself -- for items of many short rows, whose elements are all staged.
    auto reduce_range = [&](auto own, bool mine, int64_t e0, int64_t e1, int64_t staged_at, int v, float *dst_v, int32_t *dst_a,
                            bool done) {
        constexpr bool OWN = decltype(own)::value;
        const int first = OWN ? 0 : g, step = OWN ? 1 : G;
        for (int f0 = fv_lo; f0 < fv_hi; f0 += L) {
            const bool active = f0 + li < fv_hi;
            const int fc = (active ? f0 + li : fv_hi - 1) * V;       // the lane's first output feature
            const int fl = kLhs ? (a.lhs_off ? a.lhs_off[fc] : fc) : 0;
            const int fr = kRhs ? (a.rhs_off ? a.rhs_off[fc] : fc) : 0;
            float acc[V];
            int at[V];
#pragma unroll
            for (int i = 0; i < V; ++i) { acc[i] = identity<RED>(); at[i] = INT_MAX; }
            for (int64_t c0 = e0; c0 < e1; c0 += kStage) {
            const int64_t c1 = min(c0 + kStage, e1);
            int64_t base = staged_at;
            if (!OWN && staged_at < 0) {
                wave_lds_sync();          // the reads of what was staged before
                stage(c0, (int)(c1 - c0));
                base = c0;
            }
            const int t1 = (int)(c1 - base);       // positions in the staged window
            for (int tb = (int)(c0 - base) + first; tb < t1; tb += step * U) {
                float m[U][V];
                bool ok[U];
                int stored[U];          // the element's position in the caller's edge order
#pragma unroll
                for (int k = 0; k < U; ++k) {
                    const int t = tb + k * step;
                    ok[k] = t < t1;
                    const int2 w = el[ok[k] ? t : tb];
                    const int64_t u = w.x, ee = w.y;
                    stored[k] = w.y;
                    float l[V], r[V];
                    if (kLhs) load_operand<V, LC, LNT>(a.lhs + (l_on_e ? ee : u) * a.lhs_len + fl, l);
                    if (kRhs) load_operand<V, RC, RNT>(a.rhs + (r_on_e ? ee : u) * a.rhs_len + fr, r);
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        m[k][i] = binary<OP>(kLhs ? l[i] : 0.f, kRhs ? r[i] : 0.f);
                        if (RED != FG_REDUCE_SUM) m[k][i] *= sign;
                    }
                }
#pragma unroll
                for (int k = 0; k < U; ++k) {
                    const int e = stored[k];
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        if (RED == FG_REDUCE_SUM) {
                            acc[i] += ok[k] ? m[k][i] : 0.f;      // a select: what a slot without an element loaded is discarded
                        } else if (ARG) {
                            if (ok[k] && replaces<RED>(m[k][i], e, acc[i], at[i])) { acc[i] = m[k][i]; at[i] = e; }
                        } else if (ok[k]) {
                            acc[i] = extreme<RED>(acc[i], m[k][i]);
                        }
                    }
                }
            }
            }
            for (int off = L; !OWN && off < 64; off <<= 1) {
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    const float o = __shfl_xor(acc[i], off);
                    if (RED == FG_REDUCE_SUM) acc[i] += o;
                    else if (ARG) {
                        const int oa = __shfl_xor(at[i], off);
                        if (replaces<RED>(o, oa, acc[i], at[i])) { acc[i] = o; at[i] = oa; }
                    } else acc[i] = extreme<RED>(acc[i], o);
                }
            }
            if ((OWN ? mine : g == 0) && active) {
                const bool empty = e1 <= e0;
                const float scale = (done && a.row_scale) ? a.row_scale[v] : 1.f;
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    if (RED != FG_REDUCE_SUM) acc[i] *= sign;
                    acc[i] = (RED != FG_REDUCE_SUM && empty && final) ? 0.f : acc[i];
                    if (done && a.row_scale) acc[i] *= scale;
                    if (ARG) at[i] = (at[i] == INT_MAX) ? -1 : at[i];
                }
                if (V == 4) {
                    *reinterpret_cast<float4 *>(dst_v + fc) = make_float4(acc[0], acc[1 % V], acc[2 % V], acc[3 % V]);
                    if (ARG) *reinterpret_cast<int4 *>(dst_a + fc) = make_int4(at[0], at[1 % V], at[2 % V], at[3 % V]);
                } else {
                    dst_v[fc] = acc[0];
                    if (ARG) dst_a[fc] = at[0];
                }
            }
        }
    };

    if (it.info < 0) {
        const int nrows = -it.info;
        const bool fits = it.len <= kStage;       // always, for an item of several rows
        if (fits) stage(it.start, it.len);
        if (fits && nrows >= 2 * G) {
            // many short rows: a lane group per row, G rows at a time
            for (int q0 = 0; q0 < nrows; q0 += G) {
                const bool mine = q0 + g < nrows;
                const int v = it.row + min(q0 + g, nrows - 1);
                const int64_t e0 = pos_p[v], e1 = mine ? pos_p[v + 1] : e0;
                reduce_range(std::true_type{}, mine, e0, e1, it.start, v, out_p + (int64_t)v * F,
                             ARG ? arg_p + (int64_t)v * F : nullptr, final);
            }
            return;
        }
        for (int q = 0; q < nrows; ++q) {
            const int v = it.row + q;
            const int64_t e0 = pos_p[v], e1 = pos_p[v + 1];
            reduce_range(std::false_type{}, true, e0, e1, fits ? (int64_t)it.start : -1, v, out_p + (int64_t)v * F,
                         ARG ? arg_p + (int64_t)v * F : nullptr, final);
        }
        return;
    }
    reduce_range(std::false_type{}, true, it.start, (int64_t)it.start + it.len, -1, it.row, partial_p + (int64_t)it.info * F,
                 ARG ? partial_arg_p + (int64_t)it.info * F : nullptr, false);
}

// The pieces of a split row, combined in stored order.
// partial_stride / out_stride: per source partition (0 with one partition); the split segment's partition is fx.part.
template <int RED, bool ARG>
__global__ __launch_bounds__(256) void gspmm_bcast_fixup_kernel(const Fixup *fixups, int64_t n_fixups, const float *partial,
                                                                const int32_t *partial_arg, const float *row_scale,
                                                                float *out, int32_t *arg, int F, int64_t partial_stride,
                                                                int64_t out_stride) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_fixups * F) return;
    const Fixup fx = fixups[t / F];
    const int f = (int)(t % F);
    const int64_t from = fx.part * partial_stride, to = fx.part * out_stride;
    float acc = identity<RED>();
    int at = INT_MAX;
    for (int p = 0; p < fx.n_pieces; ++p) {
        const float m = partial[from + (int64_t)(fx.slot0 + p) * F + f];
        if (RED == FG_REDUCE_SUM) acc = p == 0 ? m : acc + m;
        else if (ARG) {
            const int am = partial_arg[from + (int64_t)(fx.slot0 + p) * F + f];
            if (am >= 0 && replaces<RED>(m, am, acc, at)) { acc = m; at = am; }
        } else acc = extreme<RED>(acc, m);
    }
    if (row_scale) acc *= row_scale[fx.row];
    out[to + (int64_t)fx.row * F + f] = acc;
    if (ARG) arg[to + (int64_t)fx.row * F + f] = (at == INT_MAX) ? -1 : at;
}

// out[v, f] = the partitions' results for row v combined in partition order (buf[p * buf_stride + v * F + f], positions abuf likewise, with -1
// for "none"); a row without elements in any partition gives 0 for max / min; rows are scaled here.
template <int RED, bool ARG>
__global__ __launch_bounds__(256) void gspmm_bcast_combine_kernel(const float *buf, const int32_t *abuf, const int32_t *pos,
                                                                  int n_parts, int64_t pos_stride, int64_t buf_stride,
                                                                  int64_t n_rows, int F, const float *row_scale, float *out,
                                                                  int32_t *arg) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_rows * F) return;
    const int64_t v = t / F;
    float acc = identity<RED>();
    int at = INT_MAX;
    bool any = false;
    for (int p = 0; p < n_parts; ++p) {
        const float m = buf[p * buf_stride + t];
        if (RED == FG_REDUCE_SUM) acc = p == 0 ? m : acc + m;
        else {
            any = any || pos[p * pos_stride + v + 1] > pos[p * pos_stride + v];
            if (ARG) {
                const int am = abuf[p * buf_stride + t];
                if (am >= 0 && replaces<RED>(m, am, acc, at)) { acc = m; at = am; }
            } else acc = extreme<RED>(acc, m);
        }
    }
    if (RED != FG_REDUCE_SUM && !any) acc = 0.f;
    if (row_scale) acc *= row_scale[v];
    out[t] = acc;
    if (ARG) arg[t] = (at == INT_MAX) ? -1 : at;
}

// vec: 0 = one feature per lane; else 4 per lane with (lhs, rhs) read as 1 = (consecutive, consecutive),
// 2 = (consecutive, one value), 3 = (one value, consecutive); lnt / rnt: that operand streams from the stored elements
template <int OP, int RED, bool ARG, bool PART>
void launch_spmm_variant(int vec, bool lnt, bool rnt, dim3 grid, hipStream_t st, const GenArgs &a) {
    constexpr int USES = (kUsesLhs<OP> ? 1 : 0) | (kUsesRhs<OP> ? 2 : 0);
#define FG_GO(V, LC, RC, LNT, RNT) \
    hipLaunchKernelGGL((gspmm_bcast_kernel<OP, RED, ARG, V, LC, RC, LNT, RNT, PART>), grid, dim3(kBlock), 0, st, a)
    if (vec == 0) { FG_GO(1, true, true, false, false); return; }
    const bool lc = vec != 3, rc = vec != 2;
    lnt = lnt && lc; rnt = rnt && rc;
    if constexpr (USES == 1) {             // the right operand is not read: one instantiation stands for all its modes
        if (!lc) FG_GO(4, false, true, false, false);
        else if (lnt) FG_GO(4, true, true, true, false);
        else FG_GO(4, true, true, false, false);
    } else if constexpr (USES == 2) {
        if (!rc) FG_GO(4, true, false, false, false);
        else if (rnt) FG_GO(4, true, true, false, true);
        else FG_GO(4, true, true, false, false);
    } else {
        if (lc && rc) {
            if (lnt && rnt) FG_GO(4, true, true, true, true);
            else if (lnt) FG_GO(4, true, true, true, false);
            else if (rnt) FG_GO(4, true, true, false, true);
            else FG_GO(4, true, true, false, false);
        } else if (lc) {
            if (lnt) FG_GO(4, true, false, true, false);
            else FG_GO(4, true, false, false, false);
        } else {
            if (rnt) FG_GO(4, false, true, false, true);
            else FG_GO(4, false, true, false, false);
        }
    }
#undef FG_GO
}
template <int OP, int RED, bool ARG>
void launch_spmm_ora(int vec, bool lnt, bool rnt, dim3 grid, hipStream_t st, const GenArgs &a) {
    if (a.n_parts > 1 || a.edge_pos) launch_spmm_variant<OP, RED, ARG, true>(vec, lnt, rnt, grid, st, a);
    else launch_spmm_variant<OP, RED, ARG, false>(vec, lnt, rnt, grid, st, a);
}
template <int OP>
void launch_spmm_o(int reduce, bool with_arg, int vec, bool lnt, bool rnt, dim3 grid, hipStream_t st, const GenArgs &a) {
    if (reduce == FG_REDUCE_SUM) launch_spmm_ora<OP, FG_REDUCE_SUM, false>(vec, lnt, rnt, grid, st, a);
    else if (with_arg) launch_spmm_ora<OP, FG_REDUCE_MAX, true>(vec, lnt, rnt, grid, st, a);       // max, or min by a.sign
    else launch_spmm_ora<OP, FG_REDUCE_MAX, false>(vec, lnt, rnt, grid, st, a);
}
void launch_spmm(int op, int reduce, bool with_arg, int vec, bool lnt, bool rnt, dim3 grid, hipStream_t st, const GenArgs &a) {
    switch (op) {
        case FG_BIN_ADD: launch_spmm_o<FG_BIN_ADD>(reduce, with_arg, vec, lnt, rnt, grid, st, a); break;
        case FG_BIN_SUB: launch_spmm_o<FG_BIN_SUB>(reduce, with_arg, vec, lnt, rnt, grid, st, a); break;
        case FG_BIN_MUL: launch_spmm_o<FG_BIN_MUL>(reduce, with_arg, vec, lnt, rnt, grid, st, a); break;
        case FG_BIN_DIV: launch_spmm_o<FG_BIN_DIV>(reduce, with_arg, vec, lnt, rnt, grid, st, a); break;
        case FG_BIN_COPY_LHS: launch_spmm_o<FG_BIN_COPY_LHS>(reduce, with_arg, vec, lnt, rnt, grid, st, a); break;
        default: launch_spmm_o<FG_BIN_COPY_RHS>(reduce, with_arg, vec, lnt, rnt, grid, st, a); break;
    }
}

// How one operand can be read when a lane holds 4 consecutive output features: 1 = 4 consecutive features by one
// 128-bit load, 2 = one feature 4 times, 0 = neither (scalar kernel).  Without an offset array the operand has the
// output's layout; with one, the caller's flags say which pattern every aligned group of 4 follows.
int vector_mode(bool used, const float *p, int len, const int32_t *off, int flags, int vec_flag, int splat_flag) {
    if (!used) return 1;
    if (!off || (flags & vec_flag)) return (len % 4 == 0 && ((uintptr_t)p & 15) == 0) ? 1 : 0;
    return (flags & splat_flag) ? 2 : 0;
}
// The launchers' `vec` from the two operands' modes (0: scalar kernel).
int vector_variant(bool can_vec, int lmode, int rmode) {
    if (!can_vec || !lmode || !rmode) return 0;
    if (lmode == 1 && rmode == 1) return 1;
    if (lmode == 1 && rmode == 2) return 2;
    if (lmode == 2 && rmode == 1) return 3;
    return 0;       // both operands repeat one value over every group of 4: nothing to gain
}

int lanes_for(int F) {
    int L = 1;
    while (L < F && L < 64) L <<= 1;
    return L;
}

// rows: how many rows the operand has in this call (an operand without rows may be a null pointer)
int check_operand(const char *name, bool used, const float *p, int64_t rows, int len, int target, bool allow_v) {
    if (!used) return FG_OK;
    if (!p && rows > 0) return fail(FG_ERR_ARG, "%s is null", name);
    if (len < 1) return fail(FG_ERR_SHAPE, "%s feature length must be positive, got %d", name, len);
    if (!(target == FG_TARGET_U || target == FG_TARGET_E || (allow_v && target == FG_TARGET_V)))
        return fail(FG_ERR_ARG, "%s target %d is not valid here", name, target);
    return FG_OK;
}

// Scratch of one call, in floats: per partition the pieces of its split rows ([slot][F], rounded up to 16 bytes) and,
// with several partitions, a buffer of [n_dst][F] results; the selected positions, when wanted, take as much again.
struct BcastScratch {
    size_t pieces = 0;      // per partition
    size_t buffers = 0;     // per partition (0 with one partition)
    size_t half = 0;        // all partitions' values; the positions follow
    size_t total = 0;
};
BcastScratch bcast_scratch(const fg_spmm_plan *pl, int F, bool with_arg) {
    BcastScratch b;
    const size_t P = (size_t)pl->num_col_partitions;
    b.pieces = (((size_t)pl->max_slots_in_partition * (size_t)F) + 3) & ~(size_t)3;
    b.buffers = P > 1 ? (((size_t)pl->n_dst * (size_t)F) + 3) & ~(size_t)3 : 0;
    b.half = P * (b.pieces + b.buffers);
    b.total = with_arg ? 2 * b.half : b.half;
    return b;
}
constexpr size_t kMaxBufferBytes = (size_t)8 << 30;     // all partitions' result buffers together

// ---- SDDMM ------------------------------------------------------------------------------------------

struct EdgeArgs {
    const int32_t *lhs_index, *rhs_index;   // per edge: the operand's row (col for u, row for v; any valid array for e)
    int64_t n_edges;
    const float *lhs, *rhs;
    const int32_t *lhs_off, *rhs_off;
    int lhs_len, rhs_len;
    int lhs_target, rhs_target;
    float *out;
    int F, L, R;
};

// 64 edges per wavefront; a group of L lanes writes one edge's F results (coalesced, V per lane), 64 / L edges at
// a time and U such steps in flight.  No branch between the loads of a step.
template <int OP, int V, bool LC, bool RC>
__global__ __launch_bounds__(kBlock) void gsddmm_bcast_kernel(const EdgeArgs a) {
    const int lane = threadIdx.x & 63;
    const int64_t wave_id = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int L = a.L, G = 64 / L, g = lane / L, li = lane % L;
    const int FV = a.F / V;
    const int64_t e0 = wave_id * 64;
    const int64_t e1 = min(e0 + 64, a.n_edges);
    const bool l_on_e = a.lhs_target == FG_TARGET_E, r_on_e = a.rhs_target == FG_TARGET_E;
    constexpr int U = 4;
    for (int fv = li; fv < FV; fv += L) {
        const int fc = fv * V;
        const int fl = kUsesLhs<OP> ? (a.lhs_off ? a.lhs_off[fc] : fc) : 0;
        const int fr = kUsesRhs<OP> ? (a.rhs_off ? a.rhs_off[fc] : fc) : 0;
        for (int64_t eb = e0 + g; eb < e1; eb += (int64_t)G * U) {
            float m[U][V];
            bool ok[U];
#pragma unroll
            for (int k = 0; k < U; ++k) {
                const int64_t e = eb + (int64_t)k * G;
                ok[k] = e < e1;
                const int64_t ec = ok[k] ? e : eb;
                const int64_t il = kUsesLhs<OP> ? (int64_t)a.lhs_index[ec] : 0, ir = kUsesRhs<OP> ? (int64_t)a.rhs_index[ec] : 0;
                const float *lp = a.lhs + (l_on_e ? ec : il) * a.lhs_len;
                const float *rp = a.rhs + (r_on_e ? ec : ir) * a.rhs_len;
                if (OP == FG_BIN_DOT) {
                    const float *l = lp + (int64_t)fl * a.R, *r = rp + (int64_t)fr * a.R;
                    float sum = 0.f;
                    for (int i = 0; i < a.R; ++i) sum += l[i] * r[i];
                    m[k][0] = sum;
                } else {
                    float l[V], r[V];
                    if (kUsesLhs<OP>) load_operand<V, LC>(lp + fl, l);
                    if (kUsesRhs<OP>) load_operand<V, RC>(rp + fr, r);
#pragma unroll
                    for (int i = 0; i < V; ++i) m[k][i] = binary<OP>(kUsesLhs<OP> ? l[i] : 0.f, kUsesRhs<OP> ? r[i] : 0.f);
                }
            }
#pragma unroll
            for (int k = 0; k < U; ++k) {
                if (!ok[k]) continue;
                float *o = a.out + (eb + (int64_t)k * G) * a.F + fc;
                if (V == 4) { nt_f4 t4; t4.x = m[k][0]; t4.y = m[k][1 % V]; t4.z = m[k][2 % V]; t4.w = m[k][3 % V]; __builtin_nontemporal_store(t4, reinterpret_cast<nt_f4 *>(o)); }
                else *o = m[k][0];
            }
        }
    }
}

// Dot products over a contracted axis of R floats (R a multiple of 4, operands 16-byte aligned): a group of L lanes
// (4 L >= R up to 64 lanes) reads the two operands' R floats of one (edge, output feature) pair with 128-bit loads and
// adds its products up with shuffles; the 64 / L groups take different pairs of the wavefront's 64 edges, U pairs in
// flight each.  (gsddmm_bcast_kernel<FG_BIN_DOT> walks the axis lane by lane and serves every other shape.)
template <int L>
__global__ __launch_bounds__(kBlock) void gsddmm_dot_kernel(const EdgeArgs a) {
    constexpr int G = 64 / L, U = 4;
    const int lane = threadIdx.x & 63, g = lane / L, li = lane % L;
    const int64_t wave_id = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t e0 = wave_id * 64;
    if (e0 >= a.n_edges) return;
    const int n_e = (int)min((int64_t)64, a.n_edges - e0);
    const int F = a.F, R = a.R;
    const int n_pairs = n_e * F;
    const bool l_on_e = a.lhs_target == FG_TARGET_E, r_on_e = a.rhs_target == FG_TARGET_E;
    for (int pb = g; pb < n_pairs; pb += G * U) {
        float s[U];
        bool ok[U];
#pragma unroll
        for (int k = 0; k < U; ++k) {
            const int p = pb + k * G;
            ok[k] = p < n_pairs;
            const int pc = ok[k] ? p : pb;
            const int64_t e = e0 + pc / F;
            const int f = pc % F;
            const int64_t il = a.lhs_index[e], ir = a.rhs_index[e];
            const int fl = a.lhs_off ? a.lhs_off[f] : f, fr = a.rhs_off ? a.rhs_off[f] : f;
            const float *lp = a.lhs + (l_on_e ? e : il) * a.lhs_len + (int64_t)fl * R;
            const float *rp = a.rhs + (r_on_e ? e : ir) * a.rhs_len + (int64_t)fr * R;
            float acc = 0.f;
            for (int c = li * 4; c < R; c += L * 4) {
                const float4 x = *reinterpret_cast<const float4 *>(lp + c), y = *reinterpret_cast<const float4 *>(rp + c);
                acc += (x.x * y.x + x.y * y.y) + (x.z * y.z + x.w * y.w);
            }
            s[k] = acc;
        }
#pragma unroll
        for (int k = 0; k < U; ++k) {
            for (int off = 1; off < L; off <<= 1) s[k] += __shfl_xor(s[k], off);
            const int p = pb + k * G;
            if (li == 0 && ok[k]) a.out[(e0 + p / F) * F + p % F] = s[k];
        }
    }
}

template <int OP>
void launch_sddmm(int vec, dim3 grid, hipStream_t st, const EdgeArgs &a) {
    if (vec == 1) hipLaunchKernelGGL((gsddmm_bcast_kernel<OP, 4, true, true>), grid, dim3(kBlock), 0, st, a);
    else if (vec == 2) hipLaunchKernelGGL((gsddmm_bcast_kernel<OP, 4, true, false>), grid, dim3(kBlock), 0, st, a);
    else if (vec == 3) hipLaunchKernelGGL((gsddmm_bcast_kernel<OP, 4, false, true>), grid, dim3(kBlock), 0, st, a);
    else hipLaunchKernelGGL((gsddmm_bcast_kernel<OP, 1, true, true>), grid, dim3(kBlock), 0, st, a);
}

}  // namespace

namespace fg {
int gspmm_bcast_scratch_need(const fg_spmm_plan *pl, int F, bool with_arg, ScratchNeed *need) {
    if (F < 1) return fail(FG_ERR_SHAPE, "feature length must be positive, got %d", F);
    const BcastScratch b = bcast_scratch(pl, F, with_arg);
    if ((size_t)pl->num_col_partitions * b.buffers * 4 * (with_arg ? 2 : 1) > kMaxBufferBytes)
        return fail(FG_ERR_SHAPE, "%d source partitions of [%lld, %d] results need more than 8 GiB of buffers; use fewer partitions",
                    pl->num_col_partitions, (long long)pl->n_dst, F);
    need->partial = b.total;
    need->tiled = 0;
    return FG_OK;
}
}  // namespace fg

namespace {

// pos / idx: indptr / indices of the CSR arrays with one partition, else the partitioned layout's position and local
// column arrays; edge_pos (required with several partitions): the row of each element in the edge operands.
int gspmm_bcast_run(fg_spmm_plan *pl, const int32_t *pos_dev, const int32_t *idx_dev, const int32_t *edge_pos_dev, int op,
                    int reduce, const float *lhs_dev, int lhs_target, int lhs_len, const int32_t *lhs_off_dev,
                    const float *rhs_dev, int rhs_target, int rhs_len, const int32_t *rhs_off_dev, int flags,
                    const float *row_scale_dev, float *out_dev, int32_t *arg_dev, int out_len, void *stream) {
    if (op < FG_BIN_ADD || op > FG_BIN_COPY_RHS) return fail(FG_ERR_ARG, "unknown message operator %d", op);
    if (reduce != FG_REDUCE_SUM && reduce != FG_REDUCE_MAX && reduce != FG_REDUCE_MIN)
        return fail(FG_ERR_ARG, "unknown reduce op %d", reduce);
    if (arg_dev && reduce == FG_REDUCE_SUM) return fail(FG_ERR_ARG, "positions of the selected elements exist for max / min only");
    fg::ScratchNeed need;
    if (int rc = fg::gspmm_bcast_scratch_need(pl, out_len, arg_dev != nullptr, &need)) return rc;
    const int P = pl->num_col_partitions;
    const bool uses_l = op != FG_BIN_COPY_RHS, uses_r = op != FG_BIN_COPY_LHS;
    if (int rc = check_operand("lhs", uses_l, lhs_dev, lhs_target == FG_TARGET_E ? pl->nnz : pl->n_src, lhs_len, lhs_target, false)) return rc;
    if (int rc = check_operand("rhs", uses_r, rhs_dev, rhs_target == FG_TARGET_E ? pl->nnz : pl->n_src, rhs_len, rhs_target, false)) return rc;
    if ((uses_l && !lhs_off_dev && lhs_len != out_len) || (uses_r && !rhs_off_dev && rhs_len != out_len))
        return fail(FG_ERR_SHAPE, "an operand without an offset array must have the output's feature length %d", out_len);
    if (pl->n_dst == 0) return FG_OK;
    if (!out_dev || !pos_dev || (pl->nnz > 0 && (!idx_dev || (P > 1 && !edge_pos_dev)))) return fail(FG_ERR_ARG, "null device pointer");
    if (int rc = fg::ensure_scratch(pl, need, stream)) return rc;
    hipStream_t st = (hipStream_t)stream;
    const BcastScratch b = bcast_scratch(pl, out_len, arg_dev != nullptr);
    const int lmode = vector_mode(uses_l, lhs_dev, lhs_len, lhs_off_dev, flags, FG_BCAST_LHS_VEC4, FG_BCAST_LHS_SPLAT4);
    const int rmode = vector_mode(uses_r, rhs_dev, rhs_len, rhs_off_dev, flags, FG_BCAST_RHS_VEC4, FG_BCAST_RHS_SPLAT4);
    const int vec = vector_variant(out_len % 4 == 0 && (((uintptr_t)out_dev | (uintptr_t)arg_dev) & 15) == 0, lmode, rmode);
    const int V = vec ? 4 : 1;
    float *const values = pl->partial_dev;                                          // [P][pieces] then [P][buffers]
    int32_t *const positions = reinterpret_cast<int32_t *>(pl->partial_dev + b.half);
    float *const buf = values + (size_t)P * b.pieces;
    int32_t *const abuf = positions + (size_t)P * b.pieces;
    GenArgs a;
    a.items = pl->items_dev; a.n_items = pl->n_items;
    a.indptr = pos_dev; a.indices = idx_dev; a.indices16 = fg::narrow_indices(pl, idx_dev);
    a.lhs = lhs_dev; a.rhs = rhs_dev; a.lhs_off = lhs_off_dev; a.rhs_off = rhs_off_dev;
    a.lhs_len = lhs_len; a.rhs_len = rhs_len; a.lhs_target = lhs_target; a.rhs_target = rhs_target;
    a.sign = reduce == FG_REDUCE_MIN ? -1.f : 1.f;
    a.row_scale = P > 1 ? nullptr : row_scale_dev;
    a.out = P > 1 ? buf : out_dev;
    a.arg = P > 1 ? (arg_dev ? abuf : nullptr) : arg_dev;
    a.partial = values; a.partial_arg = positions;
    // Feature tiles of 64 floats over the workgroups (as for the weighted sum) when an operand is gathered from the
    // source nodes and the 128-bit paths apply: a partition's slice of a tile is what an L2 has to hold.
    // (Not with the positions of the selected elements, whose kernels hold too many registers to gain from it --
    // F=256: 17.1 ms tiled against 14.7 ms -- nor with an operand streamed from the edges, which sets the time.)
    const bool gathers = (uses_l && lhs_target == FG_TARGET_U) || (uses_r && rhs_target == FG_TARGET_U);
    const bool streams = (uses_l && lhs_target == FG_TARGET_E && lmode == 1) || (uses_r && rhs_target == FG_TARGET_E && rmode == 1);
    const int T = (V == 4 && gathers && !streams && !arg_dev && out_len >= 128 && out_len % 64 == 0) ? out_len / 64 : 1;
    a.n_tiles = T; a.tile_vecs = T > 1 ? 16 : (out_len + V - 1) / V;
    a.F = out_len; a.L = lanes_for(T > 1 ? 16 : out_len / V);
    a.item_off = pl->item_off_dev; a.edge_pos = edge_pos_dev; a.n_parts = P; a.final = P == 1;
    a.pos_stride = pl->n_dst + 1; a.col_width = (pl->n_src + P - 1) / P;
    a.out_stride = (int64_t)b.buffers; a.partial_stride = (int64_t)b.pieces;
    const int64_t blocks = ((pl->n_items + kWavesPerBlock - 1) / kWavesPerBlock) * T;
    if (blocks > 0x7fffffffLL) return fail(FG_ERR_SHAPE, "grid of %lld workgroups is too large", (long long)blocks);
    // an operand on the stored elements that is read with 128-bit loads streams past the caches
    const bool lnt = uses_l && lhs_target == FG_TARGET_E && lmode == 1, rnt = uses_r && rhs_target == FG_TARGET_E && rmode == 1;
    if (blocks > 0) launch_spmm(op, reduce, arg_dev != nullptr, vec, lnt, rnt, dim3((unsigned)blocks), st, a);
    const int which = reduce == FG_REDUCE_SUM ? 0 : (reduce == FG_REDUCE_MAX ? 1 : 3) + (arg_dev ? 1 : 0);
    if (pl->n_fixups > 0) {
        const int64_t threads = pl->n_fixups * (int64_t)out_len;
        const dim3 grid((unsigned)((threads + 255) / 256));
#define FG_FIXUP(RED, ARG) hipLaunchKernelGGL((gspmm_bcast_fixup_kernel<RED, ARG>), grid, dim3(256), 0, st, pl->fixups_dev, pl->n_fixups, \
                                              a.partial, a.partial_arg, a.row_scale, a.out, a.arg, out_len, a.partial_stride, a.out_stride)
        switch (which) {
            case 0: FG_FIXUP(FG_REDUCE_SUM, false); break;
            case 1: FG_FIXUP(FG_REDUCE_MAX, false); break;
            case 2: FG_FIXUP(FG_REDUCE_MAX, true); break;
            case 3: FG_FIXUP(FG_REDUCE_MIN, false); break;
            default: FG_FIXUP(FG_REDUCE_MIN, true); break;
        }
#undef FG_FIXUP
    }
    if (P > 1) {
        const int64_t threads = pl->n_dst * (int64_t)out_len;
        if ((threads + 255) / 256 > 0x7fffffffLL) return fail(FG_ERR_SHAPE, "output of %lld values is too large", (long long)threads);
        const dim3 grid((unsigned)((threads + 255) / 256));
#define FG_COMBINE(RED, ARG) hipLaunchKernelGGL((gspmm_bcast_combine_kernel<RED, ARG>), grid, dim3(256), 0, st, buf, abuf, pos_dev, P, \
                                                a.pos_stride, a.out_stride, pl->n_dst, out_len, row_scale_dev, out_dev, arg_dev)
        switch (which) {
            case 0: FG_COMBINE(FG_REDUCE_SUM, false); break;
            case 1: FG_COMBINE(FG_REDUCE_MAX, false); break;
            case 2: FG_COMBINE(FG_REDUCE_MAX, true); break;
            case 3: FG_COMBINE(FG_REDUCE_MIN, false); break;
            default: FG_COMBINE(FG_REDUCE_MIN, true); break;
        }
#undef FG_COMBINE
    }
    FG_HIP_TRY(hipGetLastError());
    return FG_OK;
}

}  // namespace

extern "C" int fg_gspmm_bcast_f32(fg_spmm_plan *pl, const int32_t *indptr_dev, const int32_t *indices_dev, int op,
                                  int reduce, const float *lhs_dev, int lhs_target, int lhs_len,
                                  const int32_t *lhs_off_dev, const float *rhs_dev, int rhs_target, int rhs_len,
                                  const int32_t *rhs_off_dev, int flags, const float *row_scale_dev, float *out_dev,
                                  int32_t *arg_dev, int out_len, void *stream) {
    if (!pl) return fail(FG_ERR_ARG, "plan is null");
    if (int drc = fg::check_device(pl)) return drc;
    if (pl->num_col_partitions != 1)
        return fail(FG_ERR_ARG, "fg_gspmm_bcast_f32 takes a plan with one column partition (fg_gspmm_bcast_dds_f32: several)");
    return gspmm_bcast_run(pl, indptr_dev, indices_dev, nullptr, op, reduce, lhs_dev, lhs_target, lhs_len, lhs_off_dev, rhs_dev,
                           rhs_target, rhs_len, rhs_off_dev, flags, row_scale_dev, out_dev, arg_dev, out_len, stream);
}

extern "C" int fg_gspmm_bcast_dds_f32(fg_spmm_plan *pl, const int32_t *s1_pos_dev, const int32_t *s1_idx_dev,
                                      const int32_t *edge_pos_dev, int op, int reduce, const float *lhs_dev, int lhs_target,
                                      int lhs_len, const int32_t *lhs_off_dev, const float *rhs_dev, int rhs_target,
                                      int rhs_len, const int32_t *rhs_off_dev, int flags, const float *row_scale_dev,
                                      float *out_dev, int32_t *arg_dev, int out_len, void *stream) {
    if (!pl) return fail(FG_ERR_ARG, "plan is null");
    if (int drc = fg::check_device(pl)) return drc;
    return gspmm_bcast_run(pl, s1_pos_dev, s1_idx_dev, edge_pos_dev, op, reduce, lhs_dev, lhs_target, lhs_len, lhs_off_dev, rhs_dev,
                           rhs_target, rhs_len, rhs_off_dev, flags, row_scale_dev, out_dev, arg_dev, out_len, stream);
}

extern "C" int fg_gsddmm_bcast_f32(const int32_t *row_dev, const int32_t *col_dev, int64_t n_edges, int op,
                                   const float *lhs_dev, int lhs_target, int lhs_len, const int32_t *lhs_off_dev,
                                   const float *rhs_dev, int rhs_target, int rhs_len, const int32_t *rhs_off_dev,
                                   int flags, float *out_dev, int out_len, int reduce_len, void *stream) {
    if (op < FG_BIN_ADD || op > FG_BIN_DOT) return fail(FG_ERR_ARG, "unknown edge operator %d", op);
    if (n_edges < 0) return fail(FG_ERR_ARG, "negative edge count");
    if (out_len < 1) return fail(FG_ERR_SHAPE, "feature length must be positive, got %d", out_len);
    const bool uses_l = op != FG_BIN_COPY_RHS, uses_r = op != FG_BIN_COPY_LHS;
    // with edges every operand has rows to read; without, nothing is read
    if (int rc = check_operand("lhs", uses_l, lhs_dev, n_edges, lhs_len, lhs_target, true)) return rc;
    if (int rc = check_operand("rhs", uses_r, rhs_dev, n_edges, rhs_len, rhs_target, true)) return rc;
    const int R = op == FG_BIN_DOT ? reduce_len : 1;
    if (R < 1) return fail(FG_ERR_SHAPE, "the contracted length must be positive, got %d", reduce_len);
    if (op == FG_BIN_DOT && (lhs_len % R != 0 || rhs_len % R != 0))
        return fail(FG_ERR_SHAPE, "operand lengths %d and %d are not multiples of the contracted length %d", lhs_len, rhs_len, R);
    if ((uses_l && !lhs_off_dev && lhs_len != (int64_t)out_len * R) || (uses_r && !rhs_off_dev && rhs_len != (int64_t)out_len * R))
        return fail(FG_ERR_SHAPE, "an operand without an offset array must have the output's feature length %d (times the contracted length)", out_len);
    if (n_edges == 0) return FG_OK;
    const bool any_u = (uses_l && lhs_target == FG_TARGET_U) || (uses_r && rhs_target == FG_TARGET_U);
    const bool any_v = (uses_l && lhs_target == FG_TARGET_V) || (uses_r && rhs_target == FG_TARGET_V);
    if (!out_dev || (any_u && !col_dev) || (any_v && !row_dev)) return fail(FG_ERR_ARG, "null device pointer");
    const int lmode = vector_mode(uses_l, lhs_dev, lhs_len, lhs_off_dev, flags, FG_BCAST_LHS_VEC4, FG_BCAST_LHS_SPLAT4);
    const int rmode = vector_mode(uses_r, rhs_dev, rhs_len, rhs_off_dev, flags, FG_BCAST_RHS_VEC4, FG_BCAST_RHS_SPLAT4);
    const int vec = vector_variant(op != FG_BIN_DOT && out_len % 4 == 0 && ((uintptr_t)out_dev & 15) == 0, lmode, rmode);
    const int V = vec ? 4 : 1;
    // every lane reads its operands' row indices without a branch: an operand on the edges reads (and discards) an
    // index array that exists, or the start of out when the call has none
    const int32_t *some = col_dev ? col_dev : row_dev ? row_dev : reinterpret_cast<const int32_t *>(out_dev);
    EdgeArgs a;
    a.lhs_index = lhs_target == FG_TARGET_U ? col_dev : lhs_target == FG_TARGET_V ? row_dev : some;
    a.rhs_index = rhs_target == FG_TARGET_U ? col_dev : rhs_target == FG_TARGET_V ? row_dev : some;
    a.n_edges = n_edges;
    a.lhs = lhs_dev; a.rhs = rhs_dev; a.lhs_off = lhs_off_dev; a.rhs_off = rhs_off_dev;
    a.lhs_len = lhs_len; a.rhs_len = rhs_len; a.lhs_target = lhs_target; a.rhs_target = rhs_target;
    a.out = out_dev; a.F = out_len; a.L = lanes_for(out_len / V); a.R = R;
    const int64_t waves = (n_edges + 63) / 64;
    const int64_t blocks = (waves + kWavesPerBlock - 1) / kWavesPerBlock;
    if (blocks > 0x7fffffffLL) return fail(FG_ERR_SHAPE, "grid of %lld workgroups is too large", (long long)blocks);
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)blocks);
    switch (op) {
        case FG_BIN_ADD: launch_sddmm<FG_BIN_ADD>(vec, grid, st, a); break;
        case FG_BIN_SUB: launch_sddmm<FG_BIN_SUB>(vec, grid, st, a); break;
        case FG_BIN_MUL: launch_sddmm<FG_BIN_MUL>(vec, grid, st, a); break;
        case FG_BIN_DIV: launch_sddmm<FG_BIN_DIV>(vec, grid, st, a); break;
        case FG_BIN_COPY_LHS: launch_sddmm<FG_BIN_COPY_LHS>(vec, grid, st, a); break;
        case FG_BIN_COPY_RHS: launch_sddmm<FG_BIN_COPY_RHS>(vec, grid, st, a); break;
        default: {
            const bool wide = R % 4 == 0 && lhs_len % 4 == 0 && rhs_len % 4 == 0 && (((uintptr_t)lhs_dev | (uintptr_t)rhs_dev) & 15) == 0;
            if (!wide) hipLaunchKernelGGL((gsddmm_bcast_kernel<FG_BIN_DOT, 1, true, true>), grid, dim3(kBlock), 0, st, a);
            else if (R <= 16) hipLaunchKernelGGL(gsddmm_dot_kernel<4>, grid, dim3(kBlock), 0, st, a);
            else if (R <= 32) hipLaunchKernelGGL(gsddmm_dot_kernel<8>, grid, dim3(kBlock), 0, st, a);
            else if (R <= 64) hipLaunchKernelGGL(gsddmm_dot_kernel<16>, grid, dim3(kBlock), 0, st, a);
            else if (R <= 128) hipLaunchKernelGGL(gsddmm_dot_kernel<32>, grid, dim3(kBlock), 0, st, a);
            else hipLaunchKernelGGL(gsddmm_dot_kernel<64>, grid, dim3(kBlock), 0, st, a);
            break;
        }
    }
    FG_HIP_TRY(hipGetLastError());
    return FG_OK;
}
