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
// 64 / L groups take different elements of the row, several steps in flight; longer feature axes are walked
// 64 vectors at a time.  With one group (64 vectors or more) a row's sum is formed in the stored element
// order.  The edge operand, when there is one, is the dominant stream ([nnz, len] floats read once,
// coalesced); the node operand is gathered.
#include <hip/hip_runtime.h>

#include <climits>

#include "fg_common.h"
#include "fg_device.h"

using fg::fail;
using fg::Fixup;
using fg::Item;

// Every message is one correctly rounded float32 operation and every sum adds the rounded messages one by
// one, so that max / min, the selected positions and (with one lane group per row) the sums in stored
// order can be compared bit for bit with a sequential float32 evaluation.  This file is therefore compiled
// with -ffp-contract=off (featgraph_amd/build.py); a pragma alone does not stop the back end from fusing
// when the command line says -ffp-contract=fast.

namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kBlock = 64 * kWavesPerBlock;

struct GenArgs {
    const Item *items;
    int64_t n_items;
    const int32_t *indptr;
    const int32_t *indices;
    const float *lhs, *rhs;
    const int32_t *lhs_off, *rhs_off;
    int lhs_len, rhs_len;
    int lhs_target, rhs_target;
    const float *row_scale;      // out[v, :] *= row_scale[v] (null: 1), applied where a row is completed
    float *out;
    int32_t *arg;                // optional: stored position of the selected element (max / min)
    float *partial;              // pieces of split rows: [slot][F] values
    int32_t *partial_arg;        //                       [slot][F] positions
    int F, L;
};

// The operand features of a lane's V outputs: V consecutive ones (CONTIG: one 128-bit load) or one value V times.
template <int V, bool CONTIG>
__device__ __forceinline__ void load_operand(const float *p, float (&o)[V]) {
    if (V == 4 && CONTIG) {
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
// Whether candidate (m, at element em) replaces (acc, at element ea): the better value, or the same value at an
// earlier element; the first value that is not a NaN always enters.
template <int RED> __device__ __forceinline__ bool replaces(float m, int em, float acc, int ea) {
    const bool better = RED == FG_REDUCE_MAX ? m > acc : m < acc;
    return em != INT_MAX && m == m && (ea == INT_MAX || better || (m == acc && em < ea));
}

// LC / RC (V == 4 only): the operand's 4 features are consecutive (one 128-bit load), else one value 4 times.
// No branch stands between the loads of a step: one around a load would make the wavefront wait for everything
// issued before it.
template <int OP, int RED, bool ARG, int V, bool LC, bool RC>
__global__ __launch_bounds__(kBlock) void gspmm_bcast_kernel(const GenArgs a) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t item_id = (int64_t)blockIdx.x * kWavesPerBlock + wave;
    if (item_id >= a.n_items) return;
    const Item it = a.items[item_id];
    const int L = a.L, G = 64 / L, g = lane / L, li = lane % L;
    const int F = a.F, FV = F / V;
    const bool l_on_e = a.lhs_target == FG_TARGET_E, r_on_e = a.rhs_target == FG_TARGET_E;
    constexpr int U = V == 4 ? 4 : 8;     // elements in flight per lane group: the loads of a step are issued before its sums

    // the elements [e0, e1) of output row v: reduce and store to (dst_v, dst_a); `done`: the row is complete
    auto reduce_range = [&](int64_t e0, int64_t e1, int v, float *dst_v, int32_t *dst_a, bool done) {
        for (int f0 = 0; f0 < FV; f0 += L) {
            const bool active = f0 + li < FV;
            const int fc = (active ? f0 + li : FV - 1) * V;       // the lane's first output feature
            const int fl = kUsesLhs<OP> ? (a.lhs_off ? a.lhs_off[fc] : fc) : 0;
            const int fr = kUsesRhs<OP> ? (a.rhs_off ? a.rhs_off[fc] : fc) : 0;
            float acc[V];
            int at[V];
#pragma unroll
            for (int i = 0; i < V; ++i) { acc[i] = identity<RED>(); at[i] = INT_MAX; }
            for (int64_t eb = e0 + g; eb < e1; eb += (int64_t)G * U) {
                float m[U][V];
                bool ok[U];
#pragma unroll
                for (int k = 0; k < U; ++k) {
                    const int64_t e = eb + (int64_t)k * G;
                    ok[k] = e < e1;
                    const int64_t ec = ok[k] ? e : eb;
                    const int64_t u = a.indices[ec];          // read also when no operand lives on u: no branch
                    float l[V], r[V];
                    if (kUsesLhs<OP>) load_operand<V, LC>(a.lhs + (l_on_e ? ec : u) * a.lhs_len + fl, l);
                    if (kUsesRhs<OP>) load_operand<V, RC>(a.rhs + (r_on_e ? ec : u) * a.rhs_len + fr, r);
#pragma unroll
                    for (int i = 0; i < V; ++i) m[k][i] = binary<OP>(kUsesLhs<OP> ? l[i] : 0.f, kUsesRhs<OP> ? r[i] : 0.f);
                }
#pragma unroll
                for (int k = 0; k < U; ++k) {
                    const int e = (int)(eb + (int64_t)k * G);
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        if (RED == FG_REDUCE_SUM) {
                            acc[i] += ok[k] ? m[k][i] : 0.f;      // a select: what a slot without an element loaded is discarded
                        } else if (ARG) {
                            if (ok[k] && replaces<RED>(m[k][i], e, acc[i], at[i])) { acc[i] = m[k][i]; at[i] = e; }
                        } else if (ok[k]) {
                            acc[i] = RED == FG_REDUCE_MAX ? fmaxf(acc[i], m[k][i]) : fminf(acc[i], m[k][i]);
                        }
                    }
                }
            }
            for (int off = L; off < 64; off <<= 1) {
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    const float o = __shfl_xor(acc[i], off);
                    if (RED == FG_REDUCE_SUM) acc[i] += o;
                    else if (ARG) {
                        const int oa = __shfl_xor(at[i], off);
                        if (replaces<RED>(o, oa, acc[i], at[i])) { acc[i] = o; at[i] = oa; }
                    } else acc[i] = RED == FG_REDUCE_MAX ? fmaxf(acc[i], o) : fminf(acc[i], o);
                }
            }
            if (g == 0 && active) {
                const bool empty = e1 <= e0;
                const float scale = (done && a.row_scale) ? a.row_scale[v] : 1.f;
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    acc[i] = (RED != FG_REDUCE_SUM && empty) ? 0.f : acc[i];
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
        for (int q = 0; q < nrows; ++q) {
            const int v = it.row + q;
            const int64_t e0 = a.indptr[v], e1 = a.indptr[v + 1];
            reduce_range(e0, e1, v, a.out + (int64_t)v * F, ARG ? a.arg + (int64_t)v * F : nullptr, true);
        }
        return;
    }
    reduce_range(it.start, (int64_t)it.start + it.len, it.row, a.partial + (int64_t)it.info * F,
                 ARG ? a.partial_arg + (int64_t)it.info * F : nullptr, false);
}

// The pieces of a split row, combined in stored order.
template <int RED, bool ARG>
__global__ __launch_bounds__(256) void gspmm_bcast_fixup_kernel(const Fixup *fixups, int64_t n_fixups, const float *partial,
                                                                const int32_t *partial_arg, const float *row_scale,
                                                                float *out, int32_t *arg, int F) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_fixups * F) return;
    const Fixup fx = fixups[t / F];
    const int f = (int)(t % F);
    float acc = identity<RED>();
    int at = INT_MAX;
    for (int p = 0; p < fx.n_pieces; ++p) {
        const float m = partial[(int64_t)(fx.slot0 + p) * F + f];
        if (RED == FG_REDUCE_SUM) acc = p == 0 ? m : acc + m;
        else if (ARG) {
            const int am = partial_arg[(int64_t)(fx.slot0 + p) * F + f];
            if (am >= 0 && replaces<RED>(m, am, acc, at)) { acc = m; at = am; }
        } else acc = RED == FG_REDUCE_MAX ? fmaxf(acc, m) : fminf(acc, m);
    }
    if (row_scale) acc *= row_scale[fx.row];
    out[(int64_t)fx.row * F + f] = acc;
    if (ARG) arg[(int64_t)fx.row * F + f] = (at == INT_MAX) ? -1 : at;
}

// vec: 0 = one feature per lane; else 4 per lane with (lhs, rhs) read as 1 = (consecutive, consecutive),
// 2 = (consecutive, one value), 3 = (one value, consecutive)
template <int OP, int RED, bool ARG>
void launch_spmm_ora(int vec, dim3 grid, hipStream_t st, const GenArgs &a) {
    if (vec == 1) hipLaunchKernelGGL((gspmm_bcast_kernel<OP, RED, ARG, 4, true, true>), grid, dim3(kBlock), 0, st, a);
    else if (vec == 2) hipLaunchKernelGGL((gspmm_bcast_kernel<OP, RED, ARG, 4, true, false>), grid, dim3(kBlock), 0, st, a);
    else if (vec == 3) hipLaunchKernelGGL((gspmm_bcast_kernel<OP, RED, ARG, 4, false, true>), grid, dim3(kBlock), 0, st, a);
    else hipLaunchKernelGGL((gspmm_bcast_kernel<OP, RED, ARG, 1, true, true>), grid, dim3(kBlock), 0, st, a);
}
template <int OP>
void launch_spmm_o(int reduce, bool with_arg, int vec, dim3 grid, hipStream_t st, const GenArgs &a) {
    if (reduce == FG_REDUCE_SUM) launch_spmm_ora<OP, FG_REDUCE_SUM, false>(vec, grid, st, a);
    else if (reduce == FG_REDUCE_MAX && with_arg) launch_spmm_ora<OP, FG_REDUCE_MAX, true>(vec, grid, st, a);
    else if (reduce == FG_REDUCE_MAX) launch_spmm_ora<OP, FG_REDUCE_MAX, false>(vec, grid, st, a);
    else if (with_arg) launch_spmm_ora<OP, FG_REDUCE_MIN, true>(vec, grid, st, a);
    else launch_spmm_ora<OP, FG_REDUCE_MIN, false>(vec, grid, st, a);
}
void launch_spmm(int op, int reduce, bool with_arg, int vec, dim3 grid, hipStream_t st, const GenArgs &a) {
    switch (op) {
        case FG_BIN_ADD: launch_spmm_o<FG_BIN_ADD>(reduce, with_arg, vec, grid, st, a); break;
        case FG_BIN_SUB: launch_spmm_o<FG_BIN_SUB>(reduce, with_arg, vec, grid, st, a); break;
        case FG_BIN_MUL: launch_spmm_o<FG_BIN_MUL>(reduce, with_arg, vec, grid, st, a); break;
        case FG_BIN_DIV: launch_spmm_o<FG_BIN_DIV>(reduce, with_arg, vec, grid, st, a); break;
        case FG_BIN_COPY_LHS: launch_spmm_o<FG_BIN_COPY_LHS>(reduce, with_arg, vec, grid, st, a); break;
        default: launch_spmm_o<FG_BIN_COPY_RHS>(reduce, with_arg, vec, grid, st, a); break;
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

size_t gspmm_piece_floats(const fg_spmm_plan *pl, int F, bool with_arg) {
    const size_t per = (((size_t)pl->max_slots_in_partition * (size_t)F) + 3) & ~(size_t)3;
    return with_arg ? 2 * per : per;
}

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
                if (V == 4) *reinterpret_cast<float4 *>(o) = make_float4(m[k][0], m[k][1 % V], m[k][2 % V], m[k][3 % V]);
                else *o = m[k][0];
            }
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
    if (pl->num_col_partitions != 1) return fail(FG_ERR_ARG, "the broadcasting SpMM needs a plan with one column partition");
    if (F < 1) return fail(FG_ERR_SHAPE, "feature length must be positive, got %d", F);
    need->partial = gspmm_piece_floats(pl, F, with_arg);
    need->tiled = 0;
    return FG_OK;
}
}  // namespace fg

extern "C" int fg_gspmm_bcast_f32(fg_spmm_plan *pl, const int32_t *indptr_dev, const int32_t *indices_dev, int op,
                                  int reduce, const float *lhs_dev, int lhs_target, int lhs_len,
                                  const int32_t *lhs_off_dev, const float *rhs_dev, int rhs_target, int rhs_len,
                                  const int32_t *rhs_off_dev, int flags, const float *row_scale_dev, float *out_dev,
                                  int32_t *arg_dev, int out_len, void *stream) {
    if (!pl) return fail(FG_ERR_ARG, "plan is null");
    if (int drc = fg::check_device(pl)) return drc;
    if (op < FG_BIN_ADD || op > FG_BIN_COPY_RHS) return fail(FG_ERR_ARG, "unknown message operator %d", op);
    if (reduce != FG_REDUCE_SUM && reduce != FG_REDUCE_MAX && reduce != FG_REDUCE_MIN)
        return fail(FG_ERR_ARG, "unknown reduce op %d", reduce);
    if (arg_dev && reduce == FG_REDUCE_SUM) return fail(FG_ERR_ARG, "positions of the selected elements exist for max / min only");
    fg::ScratchNeed need;
    if (int rc = fg::gspmm_bcast_scratch_need(pl, out_len, arg_dev != nullptr, &need)) return rc;
    const bool uses_l = op != FG_BIN_COPY_RHS, uses_r = op != FG_BIN_COPY_LHS;
    if (int rc = check_operand("lhs", uses_l, lhs_dev, lhs_target == FG_TARGET_E ? pl->nnz : pl->n_src, lhs_len, lhs_target, false)) return rc;
    if (int rc = check_operand("rhs", uses_r, rhs_dev, rhs_target == FG_TARGET_E ? pl->nnz : pl->n_src, rhs_len, rhs_target, false)) return rc;
    if ((uses_l && !lhs_off_dev && lhs_len != out_len) || (uses_r && !rhs_off_dev && rhs_len != out_len))
        return fail(FG_ERR_SHAPE, "an operand without an offset array must have the output's feature length %d", out_len);
    if (pl->n_dst == 0) return FG_OK;
    if (!out_dev || !indptr_dev || (pl->nnz > 0 && !indices_dev)) return fail(FG_ERR_ARG, "null device pointer");
    if (int rc = fg::ensure_scratch(pl, need, stream)) return rc;
    hipStream_t st = (hipStream_t)stream;
    const int lmode = vector_mode(uses_l, lhs_dev, lhs_len, lhs_off_dev, flags, FG_BCAST_LHS_VEC4, FG_BCAST_LHS_SPLAT4);
    const int rmode = vector_mode(uses_r, rhs_dev, rhs_len, rhs_off_dev, flags, FG_BCAST_RHS_VEC4, FG_BCAST_RHS_SPLAT4);
    const int vec = vector_variant(out_len % 4 == 0 && (((uintptr_t)out_dev | (uintptr_t)arg_dev) & 15) == 0, lmode, rmode);
    const int V = vec ? 4 : 1;
    GenArgs a;
    a.items = pl->items_dev; a.n_items = pl->n_items;
    a.indptr = indptr_dev; a.indices = indices_dev;
    a.lhs = lhs_dev; a.rhs = rhs_dev; a.lhs_off = lhs_off_dev; a.rhs_off = rhs_off_dev;
    a.lhs_len = lhs_len; a.rhs_len = rhs_len; a.lhs_target = lhs_target; a.rhs_target = rhs_target;
    a.row_scale = row_scale_dev;
    a.out = out_dev; a.arg = arg_dev;
    a.partial = pl->partial_dev;
    a.partial_arg = reinterpret_cast<int32_t *>(pl->partial_dev + need.partial / 2);
    a.F = out_len; a.L = lanes_for(out_len / V);
    const int64_t blocks = (pl->n_items + kWavesPerBlock - 1) / kWavesPerBlock;
    if (blocks > 0x7fffffffLL) return fail(FG_ERR_SHAPE, "grid of %lld workgroups is too large", (long long)blocks);
    if (blocks > 0) launch_spmm(op, reduce, arg_dev != nullptr, vec, dim3((unsigned)blocks), st, a);
    if (pl->n_fixups > 0) {
        const int64_t threads = pl->n_fixups * (int64_t)out_len;
        const dim3 grid((unsigned)((threads + 255) / 256));
        if (reduce == FG_REDUCE_SUM)
            hipLaunchKernelGGL((gspmm_bcast_fixup_kernel<FG_REDUCE_SUM, false>), grid, dim3(256), 0, st, pl->fixups_dev, pl->n_fixups,
                               a.partial, a.partial_arg, row_scale_dev, out_dev, arg_dev, out_len);
        else if (reduce == FG_REDUCE_MAX && arg_dev)
            hipLaunchKernelGGL((gspmm_bcast_fixup_kernel<FG_REDUCE_MAX, true>), grid, dim3(256), 0, st, pl->fixups_dev, pl->n_fixups,
                               a.partial, a.partial_arg, row_scale_dev, out_dev, arg_dev, out_len);
        else if (reduce == FG_REDUCE_MAX)
            hipLaunchKernelGGL((gspmm_bcast_fixup_kernel<FG_REDUCE_MAX, false>), grid, dim3(256), 0, st, pl->fixups_dev, pl->n_fixups,
                               a.partial, a.partial_arg, row_scale_dev, out_dev, arg_dev, out_len);
        else if (arg_dev)
            hipLaunchKernelGGL((gspmm_bcast_fixup_kernel<FG_REDUCE_MIN, true>), grid, dim3(256), 0, st, pl->fixups_dev, pl->n_fixups,
                               a.partial, a.partial_arg, row_scale_dev, out_dev, arg_dev, out_len);
        else
            hipLaunchKernelGGL((gspmm_bcast_fixup_kernel<FG_REDUCE_MIN, false>), grid, dim3(256), 0, st, pl->fixups_dev, pl->n_fixups,
                               a.partial, a.partial_arg, row_scale_dev, out_dev, arg_dev, out_len);
    }
    FG_HIP_TRY(hipGetLastError());
    return FG_OK;
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
        default: hipLaunchKernelGGL((gsddmm_bcast_kernel<FG_BIN_DOT, 1, true, true>), grid, dim3(kBlock), 0, st, a); break;
    }
    FG_HIP_TRY(hipGetLastError());
    return FG_OK;
}
