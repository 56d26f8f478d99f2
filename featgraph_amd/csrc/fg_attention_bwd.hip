// Gradients of the graph attention operator (fg_attention.hip), without any [nnz, H] array.
//
// With s[e, h] = scale * <K[c, h, :], Q[r, h, :]>, a[e, h] = exp(s - m[r, h]) / l[r, h] (m, l: the row's
// maximum and sum of exponentials, kept by the forward pass) and out[r, h, :] = sum_e a * V[c, h, :]:
//
//   da[e, h] = <dout[r, h, :], V[c, h, :]>
//   ds[e, h] = a * (da - delta[r, h]),   delta[r, h] = sum_e a * da = <dout[r, h, :], out[r, h, :]>
//   dQ[r]   += scale * ds * K[c]          (a sum over the row's edges: the forward pass's traversal)
//   dV[c]   += a * dout[r],  dK[c] += scale * ds * Q[r]      (sums over a column's edges: the same
//                                                            traversal of the transposed adjacency)
//
// Both kernels form s again from Q and K, read (m + log l, delta) per row and head, and gather two
// operands per edge, as the forward pass does.  Not in the reference.
#include <hip/hip_runtime.h>

#include <cmath>
#include <type_traits>

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

__device__ __forceinline__ float dot4(const float4 &a, const float4 &b) { return a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w; }
__device__ __forceinline__ void fma4(float4 &acc, float w, const float4 &x) {
    acc.x += w * x.x; acc.y += w * x.y; acc.z += w * x.z; acc.w += w * x.w;
}
__device__ __forceinline__ float4 zero4() { return make_float4(0.f, 0.f, 0.f, 0.f); }
__device__ __forceinline__ void shfl_add(float4 &a, int off) {
    a.x += __shfl_xor(a.x, off); a.y += __shfl_xor(a.y, off); a.z += __shfl_xor(a.z, off); a.w += __shfl_xor(a.w, off);
}

// What is staged per element of a row: the byte offset of the far row's slices and, gathered once per item
// (64 elements per load) rather than once per step, the far side's scalars:
//   rows, dot products : nothing more                       rows, additive scores   : el[c, h]
//   columns            : the destination's (m + log l, delta), and with additive scores its er[r, h]
template <bool BY_COLUMN, bool ADD> struct FarStaged { using type = int4; };
template <> struct FarStaged<false, false> { using type = int32_t; };
template <> struct FarStaged<false, true> { using type = int2; };
__device__ __forceinline__ uint32_t far_off(int32_t w) { return (uint32_t)w; }
__device__ __forceinline__ uint32_t far_off(const int2 &w) { return (uint32_t)w.x; }
__device__ __forceinline__ uint32_t far_off(const int4 &w) { return (uint32_t)w.x; }

// One traversal serves both kernels.  The "own" side is the row of the traversed matrix, the "far" side is
// what its elements point at:
//   BY_COLUMN == false (adjacency, rows = destinations): own = (Q[r], dout[r], coef[r]), far = (K[c], V[c]);
//     result A = dQ[r].
//   BY_COLUMN == true (transposed adjacency, rows = sources): own = (K[c], V[c]), far = (Q[r], dout[r],
//     coef[r]); results A = dK[c], B = dV[c].
struct BwdArgs {
    const Item *items;
    int64_t n_items;
    const int32_t *pos;
    const int32_t *indices;   // partition-local ids of the far side
    const uint16_t *indices16 = nullptr;   // the plan's 16-bit copy of them, read instead (null: none)
    const float *own0, *own1; // [n_own, F]: (Q, dout) or (K, V)
    const float *far0, *far1; // offset to the partition's first far row: (K, V) or (Q, dout)
    uint32_t far_row_bytes, far_tile_bytes;
    const float *coef;        // [H, n_dst, 2]: (m + log l, delta), head by head; BY_COLUMN: offset to the partition's first far row
    int64_t coef_head_floats; // floats from one head's block of coef to the next (2 * n_dst)
    float *res0, *res1;       // [n_own, F]: dQ, or dK and dV
    int F, H;
    int n_heads, head_base;
    float scale;
    // Additive scores leaky_relu(el[c] + er[r]) (ADD): no far0 / own0 slices; instead
    //   rows:    far_s = el [H, n_src] (4 bytes per element), coef holds (m + log l, delta, er[r], 0) per row;
    //   columns: own_s = el [H, n_src], far_s = that 16-byte coef of the destinations;
    // res_s = d_er (rows) or d_el (columns), [H, n_own]; all head by head, *_head_floats apart.
    const float *own_s, *far_s;
    float *res_s;
    int64_t own_s_head_floats, far_s_head_floats;
    float slope;
};

template <int L, bool BY_COLUMN, bool ACC, bool ADD>
__global__ __launch_bounds__(kBlock) void attention_backward_kernel(const BwdArgs a) {
    constexpr int G = 64 / L, D = 4 * L;
    constexpr int KU = kU;   // (two steps in flight by column lower the registers from 95 to 74 and change no time)
    using W = typename FarStaged<BY_COLUMN, ADD>::type;
    __shared__ __align__(16) W s_far[kWavesPerBlock][fg::kItemEdges + kPad];
    __shared__ int32_t s_end[kWavesPerBlock][fg::kItemRows];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int head = a.head_base + (int)(blockIdx.x % (unsigned)a.n_heads);
    const int64_t item_id = (int64_t)(blockIdx.x / (unsigned)a.n_heads) * kWavesPerBlock + wave;
    if (item_id >= a.n_items) return;
    const Item it = a.items[item_id];
    const int g = lane / L, li = lane % L;
    const int f_lo = head * D + li * 4;
    const uint32_t lane_bytes = a.far_tile_bytes ? (uint32_t)head * a.far_tile_bytes + (uint32_t)li * 16u : (uint32_t)f_lo * 4u;
    const int64_t F = a.F;
    W *far = s_far[wave];
    const float *coef_head = a.coef + (int64_t)head * a.coef_head_floats;
    const float *far_s_head = ADD ? a.far_s + (int64_t)head * a.far_s_head_floats : nullptr;
    const float *own_s_head = (ADD && BY_COLUMN) ? a.own_s + (int64_t)head * a.own_s_head_floats : nullptr;
    float *res_s_head = ADD ? a.res_s + (int64_t)head * a.own_s_head_floats : nullptr;

    auto stage = [&](int64_t base, int n) {
        int32_t c[4];
        fg::load_four_ids(a.indices, a.indices16, base, n, lane, c);
        W w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int off = (int)((uint32_t)c[i] * a.far_row_bytes);
            if constexpr (BY_COLUMN && ADD) {
                const float4 cf = *reinterpret_cast<const float4 *>(far_s_head + (int64_t)c[i] * 4);
                w[i] = make_int4(off, __float_as_int(cf.x), __float_as_int(cf.y), __float_as_int(cf.z));
            } else if constexpr (BY_COLUMN) {
                const float2 cf = *reinterpret_cast<const float2 *>(coef_head + (int64_t)c[i] * 2);
                w[i] = make_int4(off, __float_as_int(cf.x), __float_as_int(cf.y), 0);
            } else if constexpr (ADD) {
                w[i] = make_int2(off, __float_as_int(far_s_head[c[i]]));
            } else {
                w[i] = off;
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) far[4 * lane + i] = w[i];
        if (lane < kPad) far[fg::kItemEdges + lane] = w[3];
    };

    // NU steps of one row for this lane group (elements s0 + g, s0 + g + G, ...; only the last step may have
    // groups without an element, which re-read element e - 1 and discard it).
    auto batch = [&](auto nu_tag, auto allvalid_tag, int s0, int e, const float4 &o0, const float4 &o1, float c1, float delta,
                     float4 &accA, float4 &accB, float &accS) {
        constexpr int NU = decltype(nu_tag)::value;
        constexpr bool ALLVALID = decltype(allvalid_tag)::value;
        const bool last_valid = ALLVALID || s0 + (NU - 1) * G + g < e;
        W w[NU];
#pragma unroll
        for (int u = 0; u < NU; ++u) w[u] = far[(u < NU - 1 || last_valid) ? s0 + u * G + g : e - 1];
        float4 f0[NU], f1[NU];
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            if constexpr (!ADD) f0[u] = *reinterpret_cast<const float4 *>(reinterpret_cast<const char *>(a.far0) + (far_off(w[u]) + lane_bytes));
            f1[u] = *reinterpret_cast<const float4 *>(reinterpret_cast<const char *>(a.far1) + (far_off(w[u]) + lane_bytes));
        }
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            // rows: o0 = Q[r], o1 = dout[r], f0 = K[c], f1 = V[c];  columns: o0 = K[c], o1 = V[c], f0 = Q[r], f1 = dout[r]
            // ADD: o0.x = the own scalar (er[r] | el[c]); the far one (el[c] | er[r]) was staged with the offsets
            float s, gate = 1.f, cc = c1, dd = delta;
            if constexpr (BY_COLUMN) { cc = __int_as_float(w[u].y); dd = __int_as_float(w[u].z); }
            if constexpr (ADD) {
                float far_scalar;
                if constexpr (BY_COLUMN) far_scalar = __int_as_float(w[u].w);
                else far_scalar = __int_as_float(w[u].y);
                const float z = o0.x + far_scalar;
                gate = z > 0.f ? 1.f : a.slope;
                s = z * gate;
            } else {
                s = group_sum<L>(dot4(f0[u], o0)) * a.scale;
            }
            const float da = group_sum<L>(dot4(f1[u], o1));
            float p = __expf(s - cc);                       // the softmax value; cc = +inf for rows without edges
            float ds = p * (da - dd);
            if (!(u < NU - 1 || last_valid)) {
                // a group without an element: nothing of what it re-read may reach the sums (selects, not
                // products with zero, so that non-finite operands stay in the rows that reference them)
                p = 0.f; ds = 0.f;
                if constexpr (!ADD) f0[u] = zero4();
                f1[u] = zero4();
            }
            if constexpr (ADD) {
                accS += ds * gate;                                                  // d_er[r] | d_el[c]
                if (BY_COLUMN) fma4(accB, p, f1[u]);                                // dV += a * dout[r]
            } else {
                if (BY_COLUMN) { fma4(accA, ds, f0[u]); fma4(accB, p, f1[u]); }     // dK += ds * Q[r], dV += a * dout[r]
                else fma4(accA, ds, f0[u]);                                         // dQ += ds * K[c]
            }
        }
    };
    auto walk = [&](int b, int e, const float4 &o0, const float4 &o1, float c1, float delta, float4 &accA, float4 &accB, float &accS) {
        using std::integral_constant;
        int s0 = b;
        for (; s0 + G * KU <= e; s0 += G * KU)
            batch(integral_constant<int, KU>(), integral_constant<bool, true>(), s0, e, o0, o1, c1, delta, accA, accB, accS);
        if (s0 >= e) return;
        const int nu = (e - s0 + G - 1) / G;
        static_assert(KU == 2 || KU == 4, "the tail below lists the step counts");
        if (nu == 1) batch(integral_constant<int, 1>(), integral_constant<bool, false>(), s0, e, o0, o1, c1, delta, accA, accB, accS);
        else if (KU == 2 || nu == 2) batch(integral_constant<int, 2>(), integral_constant<bool, false>(), s0, e, o0, o1, c1, delta, accA, accB, accS);
        else if (nu == 3) batch(integral_constant<int, 3>(), integral_constant<bool, false>(), s0, e, o0, o1, c1, delta, accA, accB, accS);
        else batch(integral_constant<int, 4>(), integral_constant<bool, false>(), s0, e, o0, o1, c1, delta, accA, accB, accS);
    };
    // sums the lane groups' parts, scales what carries the score's scale, and stores (ACC: adds to) the row
    auto finish = [&](int64_t row, float4 accA, float4 accB, float accS, const float4 &oldA, const float4 &oldB, float oldS) {
#pragma unroll
        for (int off = L; off < 64; off <<= 1) {
            if (!ADD) shfl_add(accA, off);
            if (BY_COLUMN) shfl_add(accB, off);
            if (ADD) accS += __shfl_xor(accS, off);
        }
        if (g != 0) return;
        if constexpr (ADD) {
            if (li == 0) res_s_head[row] = ACC ? accS + oldS : accS;
        } else {
            accA.x *= a.scale; accA.y *= a.scale; accA.z *= a.scale; accA.w *= a.scale;
            if (ACC) { accA.x += oldA.x; accA.y += oldA.y; accA.z += oldA.z; accA.w += oldA.w; }
            *reinterpret_cast<float4 *>(a.res0 + row * F + f_lo) = accA;
        }
        if (BY_COLUMN) {
            if (ACC) { accB.x += oldB.x; accB.y += oldB.y; accB.z += oldB.z; accB.w += oldB.w; }
            *reinterpret_cast<float4 *>(a.res1 + row * F + f_lo) = accB;
        }
    };
    auto row_inputs = [&](int64_t row, float4 &o0, float4 &o1, float &c1, float &delta, float4 &oldA, float4 &oldB, float &oldS) {
        o1 = *reinterpret_cast<const float4 *>(a.own1 + row * F + f_lo);
        c1 = 0.f; delta = 0.f;
        if constexpr (ADD) {
            if (BY_COLUMN) {
                o0 = make_float4(own_s_head[row], 0.f, 0.f, 0.f);
            } else {
                const float4 cf = *reinterpret_cast<const float4 *>(coef_head + row * 4);
                c1 = cf.x; delta = cf.y;
                o0 = make_float4(cf.z, 0.f, 0.f, 0.f);
            }
        } else {
            o0 = *reinterpret_cast<const float4 *>(a.own0 + row * F + f_lo);
            if (!BY_COLUMN) {
                const float2 cf = *reinterpret_cast<const float2 *>(coef_head + row * 2);
                c1 = cf.x; delta = cf.y;
            }
        }
        oldA = zero4(); oldB = zero4(); oldS = 0.f;
        if (ACC) {
            if (ADD) oldS = res_s_head[row];
            else oldA = *reinterpret_cast<const float4 *>(a.res0 + row * F + f_lo);
            if (BY_COLUMN) oldB = *reinterpret_cast<const float4 *>(a.res1 + row * F + f_lo);
        }
    };

    float4 o0, o1, oldA, oldB;
    float c1, delta, oldS;
    if (it.info < -1) {
        const int nrows = -it.info;
        // own rows read once while the ids are on their way (loads return in order)
        float touched = 0.f;
        constexpr int kLines = (D * 4 + 127) / 128;
        static_assert(fg::kItemRows * kLines <= 128, "two touches per lane cover an item's rows");
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int t = lane + 64 * i;
            const int64_t at = (int64_t)(it.row + min(t / kLines, nrows - 1)) * F + head * D + min((t % kLines) * 32, D - 1);
            touched += a.own1[at];
            if (!ADD) touched += a.own0[at];
            if (ACC && !ADD) touched += a.res0[at];
            if (ACC && BY_COLUMN) touched += a.res1[at];
        }
        if (it.len > 0) stage(it.start, it.len);
        s_end[wave][lane] = a.pos[it.row + min(lane, nrows - 1) + 1] - it.start;
        wave_lds_sync();
        asm volatile("" ::"v"(touched));      // keeps the loads
        int b = 0;
        for (int r = 0; r < nrows; ++r) {
            const int e = __builtin_amdgcn_readfirstlane(s_end[wave][r]);
            if (e > b || !ACC) {
                row_inputs(it.row + r, o0, o1, c1, delta, oldA, oldB, oldS);
                float4 accA = zero4(), accB = zero4();
                float accS = 0.f;
                walk(b, e, o0, o1, c1, delta, accA, accB, accS);
                finish(it.row + r, accA, accB, accS, oldA, oldB, oldS);
            }
            b = e;
        }
        return;
    }
    // one row of any length: 256 elements at a time
    row_inputs(it.row, o0, o1, c1, delta, oldA, oldB, oldS);
    float4 accA = zero4(), accB = zero4();
    float accS = 0.f;
    for (int32_t base = 0; base < it.len; base += fg::kItemEdges) {
        const int n = min(fg::kItemEdges, it.len - base);
        wave_lds_sync();
        stage((int64_t)it.start + base, n);
        wave_lds_sync();
        walk(0, n, o0, o1, c1, delta, accA, accB, accS);
    }
    if (it.len > 0 || !ACC) finish(it.row, accA, accB, accS, oldA, oldB, oldS);
}

// coef[h, r] = (m + log l, <dout[r, h, :], out[r, h, :]>), head by head so that the gathers of one head stay
// inside 8 * n_dst bytes; rows without edges (l == 0): (+inf, 0), so that
// every softmax value formed from them is 0.  One lane group of head_len / 4 lanes per (row, head).
template <int L>
__global__ __launch_bounds__(256) void attention_coef_kernel(const float *out, const float *dout, const float *state,
                                                             const float *er, float *coef, int64_t n_pairs,
                                                             int64_t n_rows, int H) {
    const int64_t pair = ((int64_t)blockIdx.x * 256 + threadIdx.x) / L;
    const int li = threadIdx.x % L;
    const bool on = pair < n_pairs;
    const int64_t at = (on ? pair : 0) * (4 * L) + li * 4;
    const float4 o = *reinterpret_cast<const float4 *>(out + at), d = *reinterpret_cast<const float4 *>(dout + at);
    const float delta = group_sum<L>(dot4(o, d));
    if (on && li == 0) {
        const float m = state[pair * 2], l = state[pair * 2 + 1];
        const int64_t r = pair / H, h = pair - r * H;
        const float c1 = l > 0.f ? m + __logf(l) : INFINITY, dl = l > 0.f ? delta : 0.f;
        if (er) {       // additive scores: the row's own scalar rides along, 16 bytes per row and head
            *reinterpret_cast<float4 *>(coef + (h * n_rows + r) * 4) = make_float4(c1, dl, er[h * n_rows + r], 0.f);
        } else {
            float *c = coef + (h * n_rows + r) * 2;             // head by head
            c[0] = c1; c[1] = dl;
        }
    }
}

template <int L, bool BY_COLUMN, bool ADD>
void launch(bool acc, dim3 grid, hipStream_t st, const BwdArgs &a) {
    if (acc) hipLaunchKernelGGL((attention_backward_kernel<L, BY_COLUMN, true, ADD>), grid, dim3(kBlock), 0, st, a);
    else hipLaunchKernelGGL((attention_backward_kernel<L, BY_COLUMN, false, ADD>), grid, dim3(kBlock), 0, st, a);
}

int check_common(const fg_spmm_plan *pl, int heads, int head_len, int64_t n_far_rows) {
    if (!pl) return fail(FG_ERR_ARG, "plan is null");
    if (int drc = fg::check_device(pl)) return drc;
    if (heads < 1 || !(head_len == 16 || head_len == 32 || head_len == 64))
        return fail(FG_ERR_SHAPE, "attention takes heads of 16, 32 or 64 floats, got %d heads of %d", heads, head_len);
    if (pl->n_fixups > 0)
        return fail(FG_ERR_ARG, "attention needs a plan without split rows (fg_plan_opts.split_threshold = INT32_MAX)");
    const uint64_t F = (uint64_t)heads * head_len;
    if ((uint64_t)n_far_rows * F * 4u >= (1ull << 32) || (uint64_t)pl->n_dst * F >= (1ull << 32) ||
        (uint64_t)n_far_rows * 8u >= (1ull << 32))
        return fail(FG_ERR_SHAPE, "attention operands of 4 GiB and more are not supported");
    return FG_OK;
}

// The passes over the source-column partitions of `pl`; far0 / far1 are gathered through its column ids.
// ADD (additive scores): far0 / own0 are not used; own_s / far_s / res_s as described at BwdArgs, coef_dev is
// the 16-byte form.
template <bool BY_COLUMN, bool ADD>
int run_backward(fg_spmm_plan *pl, const int32_t *pos_dev, const int32_t *idx_dev, const float *own0,
                 const float *own1, const float *far0_dev, const float *far1_dev, const float *coef_dev,
                 float *res0, float *res1, int heads, int head_len, float param, void *stream,
                 const float *own_s = nullptr, const float *far_s = nullptr, float *res_s = nullptr) {
    const int F = heads * head_len;
    hipStream_t st = (hipStream_t)stream;
    const int P = pl->num_col_partitions;
    const int64_t width = (pl->n_src + P - 1) / P;
    fg::ScratchNeed need;
    int rc = fg::attention_scratch_need(pl, heads, head_len, ADD, false, &need, false);
    if (rc == FG_OK) rc = fg::ensure_scratch(pl, need, stream);
    if (rc != FG_OK) return rc;
    const bool tiled = need.tiled > 0;
    const float *far0 = far0_dev, *far1 = far1_dev;
    if (tiled) {
        const int slots = ADD ? 1 : 2;
        if ((rc = fg::make_tile_major(pl, far1_dev, pl->n_src, F, head_len, stream, 0, slots)) != FG_OK) return rc;
        far1 = pl->tiled_dev;
        if (!ADD) {
            if ((rc = fg::make_tile_major(pl, far0_dev, pl->n_src, F, head_len, stream, 1, slots)) != FG_OK) return rc;
            far0 = pl->tiled_dev + (size_t)pl->n_src * F;
        }
    }
    const int row_floats = tiled ? head_len : F;
    const int far_s_floats = BY_COLUMN ? 4 : 1;          // ADD: floats per far element in far_s
    for (int p = 0; p < P; ++p) {
        const int64_t i0 = pl->item_off[p], i1 = pl->item_off[p + 1];
        if (i1 == i0) continue;
        BwdArgs a;
        a.items = pl->items_dev + i0; a.n_items = i1 - i0;
        a.pos = pos_dev + (int64_t)p * (pl->n_dst + 1);
        a.indices = idx_dev; a.indices16 = fg::narrow_indices(pl, idx_dev);
        a.own0 = own0; a.own1 = own1;
        a.far0 = ADD ? nullptr : far0 + (int64_t)p * width * row_floats; a.far1 = far1 + (int64_t)p * width * row_floats;
        a.far_row_bytes = (uint32_t)row_floats * 4u;
        a.far_tile_bytes = tiled ? (uint32_t)((uint64_t)pl->n_src * head_len * 4u) : 0u;
        if (ADD) {
            a.coef = coef_dev; a.coef_head_floats = 4 * pl->n_dst;       // rows only: the own rows' 16-byte coef
            a.own_s = own_s; a.own_s_head_floats = pl->n_dst; a.res_s = res_s;
            a.far_s = far_s + (int64_t)p * width * far_s_floats; a.far_s_head_floats = (int64_t)far_s_floats * pl->n_src;
        } else {
            a.coef = BY_COLUMN ? coef_dev + (int64_t)p * width * 2 : coef_dev;
            a.coef_head_floats = 2 * (BY_COLUMN ? pl->n_src : pl->n_dst);
            a.own_s = a.far_s = nullptr; a.res_s = nullptr; a.own_s_head_floats = a.far_s_head_floats = 0;
        }
        a.res0 = res0; a.res1 = res1; a.F = F; a.H = heads; a.scale = param; a.slope = param;
        const int per_launch = (heads > 8 && heads % 8 == 0) ? 8 : heads;
        for (int hb = 0; hb < heads; hb += per_launch) {
            a.n_heads = per_launch; a.head_base = hb;
            const int64_t blocks = ((i1 - i0 + kWavesPerBlock - 1) / kWavesPerBlock) * per_launch;
            if (blocks > 0x7fffffffLL) return fail(FG_ERR_SHAPE, "grid of %lld workgroups is too large", (long long)blocks);
            const dim3 grid((unsigned)blocks);
            if (head_len == 64) launch<16, BY_COLUMN, ADD>(p > 0, grid, st, a);
            else if (head_len == 32) launch<8, BY_COLUMN, ADD>(p > 0, grid, st, a);
            else launch<4, BY_COLUMN, ADD>(p > 0, grid, st, a);
        }
    }
    FG_HIP_TRY(hipGetLastError());
    return FG_OK;
}

int run_coef(const float *out_dev, const float *dout_dev, const float *row_state_dev, const float *er_dev,
             float *row_coef_dev, int64_t n_dst, int heads, int head_len, void *stream) {
    if (n_dst < 0 || heads < 1 || !(head_len == 16 || head_len == 32 || head_len == 64))
        return fail(FG_ERR_SHAPE, "attention takes heads of 16, 32 or 64 floats, got %d heads of %d", heads, head_len);
    if (n_dst == 0) return FG_OK;
    if (!out_dev || !dout_dev || !row_state_dev || !row_coef_dev) return fail(FG_ERR_ARG, "null device pointer");
    if ((((uintptr_t)out_dev | (uintptr_t)dout_dev | (uintptr_t)row_coef_dev) & 15) != 0)
        return fail(FG_ERR_ARG, "attention needs 16-byte aligned arrays");
    const int64_t n_pairs = n_dst * heads;
    const int L = head_len / 4;
    const int64_t threads = n_pairs * L;
    const dim3 grid((unsigned)((threads + 255) / 256));
    hipStream_t st = (hipStream_t)stream;
    if (L == 16) hipLaunchKernelGGL(attention_coef_kernel<16>, grid, dim3(256), 0, st, out_dev, dout_dev, row_state_dev, er_dev, row_coef_dev, n_pairs, n_dst, heads);
    else if (L == 8) hipLaunchKernelGGL(attention_coef_kernel<8>, grid, dim3(256), 0, st, out_dev, dout_dev, row_state_dev, er_dev, row_coef_dev, n_pairs, n_dst, heads);
    else hipLaunchKernelGGL(attention_coef_kernel<4>, grid, dim3(256), 0, st, out_dev, dout_dev, row_state_dev, er_dev, row_coef_dev, n_pairs, n_dst, heads);
    FG_HIP_TRY(hipGetLastError());
    return FG_OK;
}

}  // namespace

extern "C" int fg_graph_attention_coef_f32(const float *out_dev, const float *dout_dev, const float *row_state_dev,
                                           float *row_coef_dev, int64_t n_dst, int heads, int head_len, void *stream) {
    return run_coef(out_dev, dout_dev, row_state_dev, nullptr, row_coef_dev, n_dst, heads, head_len, stream);
}

extern "C" int fg_graph_attention_backward_q_f32(fg_spmm_plan *pl, const int32_t *pos_dev, const int32_t *idx_dev,
                                                 const float *q_dev, const float *k_dev, const float *v_dev,
                                                 const float *dout_dev, const float *row_coef_dev, float *dq_dev,
                                                 int heads, int head_len, float scale, void *stream) {
    if (pl == nullptr) return fail(FG_ERR_ARG, "plan is null");
    if (int rc = check_common(pl, heads, head_len, pl->n_src)) return rc;
    if (pl->n_dst == 0) return FG_OK;
    if (!pos_dev || !q_dev || !dout_dev || !row_coef_dev || !dq_dev || (pl->nnz > 0 && (!idx_dev || !k_dev || !v_dev)))
        return fail(FG_ERR_ARG, "null device pointer");
    if ((((uintptr_t)q_dev | (uintptr_t)k_dev | (uintptr_t)v_dev | (uintptr_t)dout_dev | (uintptr_t)dq_dev) & 15) != 0)
        return fail(FG_ERR_ARG, "attention needs 16-byte aligned arrays");
    return run_backward<false, false>(pl, pos_dev, idx_dev, q_dev, dout_dev, k_dev, v_dev, row_coef_dev, dq_dev, nullptr,
                               heads, head_len, scale, stream);
}

extern "C" int fg_graph_attention_backward_kv_f32(fg_spmm_plan *pl, const int32_t *pos_t_dev, const int32_t *idx_t_dev,
                                                  const float *q_dev, const float *dout_dev, const float *k_dev,
                                                  const float *v_dev, const float *row_coef_dev, float *dk_dev,
                                                  float *dv_dev, int heads, int head_len, float scale, void *stream) {
    if (pl == nullptr) return fail(FG_ERR_ARG, "plan is null");
    if (int rc = check_common(pl, heads, head_len, pl->n_src)) return rc;
    if (pl->n_dst == 0) return FG_OK;
    if (!pos_t_dev || !k_dev || !v_dev || !dk_dev || !dv_dev || (pl->nnz > 0 && (!idx_t_dev || !q_dev || !dout_dev || !row_coef_dev)))
        return fail(FG_ERR_ARG, "null device pointer");
    if ((((uintptr_t)q_dev | (uintptr_t)k_dev | (uintptr_t)v_dev | (uintptr_t)dout_dev | (uintptr_t)dk_dev | (uintptr_t)dv_dev) & 15) != 0 ||
        ((uintptr_t)row_coef_dev & 7) != 0)
        return fail(FG_ERR_ARG, "attention needs 16-byte aligned arrays");
    return run_backward<true, false>(pl, pos_t_dev, idx_t_dev, k_dev, v_dev, q_dev, dout_dev, row_coef_dev, dk_dev, dv_dev,
                              heads, head_len, scale, stream);
}

extern "C" int fg_graph_attention_additive_coef_f32(const float *out_dev, const float *dout_dev, const float *row_state_dev,
                                                    const float *er_dev, float *row_coef_dev, int64_t n_dst, int heads,
                                                    int head_len, void *stream) {
    if (!er_dev) return fail(FG_ERR_ARG, "null device pointer");
    return run_coef(out_dev, dout_dev, row_state_dev, er_dev, row_coef_dev, n_dst, heads, head_len, stream);
}

extern "C" int fg_graph_attention_additive_backward_er_f32(fg_spmm_plan *pl, const int32_t *pos_dev,
                                                           const int32_t *idx_dev, const float *el_dev, const float *v_dev,
                                                           const float *dout_dev, const float *row_coef_dev,
                                                           float *der_dev, int heads, int head_len,
                                                           float negative_slope, void *stream) {
    if (pl == nullptr) return fail(FG_ERR_ARG, "plan is null");
    if (int rc = check_common(pl, heads, head_len, pl->n_src)) return rc;
    if (pl->n_dst == 0) return FG_OK;
    if (!pos_dev || !dout_dev || !row_coef_dev || !der_dev || (pl->nnz > 0 && (!idx_dev || !el_dev || !v_dev)))
        return fail(FG_ERR_ARG, "null device pointer");
    if ((((uintptr_t)v_dev | (uintptr_t)dout_dev | (uintptr_t)row_coef_dev) & 15) != 0)
        return fail(FG_ERR_ARG, "attention needs 16-byte aligned arrays");
    return run_backward<false, true>(pl, pos_dev, idx_dev, nullptr, dout_dev, nullptr, v_dev, row_coef_dev, nullptr, nullptr,
                                     heads, head_len, negative_slope, stream, nullptr, el_dev, der_dev);
}

extern "C" int fg_graph_attention_additive_backward_elv_f32(fg_spmm_plan *pl, const int32_t *pos_t_dev,
                                                            const int32_t *idx_t_dev, const float *dout_dev,
                                                            const float *el_dev, const float *v_dev,
                                                            const float *row_coef_dev, float *del_dev, float *dv_dev,
                                                            int heads, int head_len, float negative_slope, void *stream) {
    if (pl == nullptr) return fail(FG_ERR_ARG, "plan is null");
    if (int rc = check_common(pl, heads, head_len, pl->n_src)) return rc;
    if ((uint64_t)pl->n_src * 16u >= (1ull << 32)) return fail(FG_ERR_SHAPE, "attention operands of 4 GiB and more are not supported");
    if (pl->n_dst == 0) return FG_OK;
    if (!pos_t_dev || !el_dev || !v_dev || !del_dev || !dv_dev || (pl->nnz > 0 && (!idx_t_dev || !dout_dev || !row_coef_dev)))
        return fail(FG_ERR_ARG, "null device pointer");
    if ((((uintptr_t)v_dev | (uintptr_t)dout_dev | (uintptr_t)dv_dev | (uintptr_t)row_coef_dev) & 15) != 0)
        return fail(FG_ERR_ARG, "attention needs 16-byte aligned arrays");
    return run_backward<true, true>(pl, pos_t_dev, idx_t_dev, nullptr, v_dev, nullptr, dout_dev, row_coef_dev, nullptr, dv_dev,
                                    heads, head_len, negative_slope, stream, el_dev, row_coef_dev, del_dev);
}
