// Softmax over the stored elements of every CSR row, per head, and its gradient (gfx950).
//
//   forward : y[e, h] = exp(x[e, h] - m[v, h]) / sum_{e' in row v} exp(x[e', h] - m[v, h]),  m = row maximum
//   backward: dx[e, h] = a[e, h] * (g[e, h] - sum_{e' in row v} a[e', h] * g[e', h])
//
// x, y are [nnz, H] row-major, so a row's values are one contiguous run of len * H floats.  The
// work is cut by the same plan items as SpMM: one wavefront per run of short rows, per row, or
// per piece of a long row.  A row of up to 1024 floats is read once and finished in registers, a
// run of short rows is finished in LDS, a longer row is swept twice (statistics, then result).  Pieces of a split row write
// (max, sum) per head, a small kernel merges them per row, and a second launch of the main
// kernel normalises the pieces.  Both operators move 2 * nnz * H * 4 bytes at best (read + write;
// the gradient reads two arrays): they are bound by HBM bandwidth.
#include <hip/hip_runtime.h>

#include <cmath>

#include "fg_common.h"
#include "fg_device.h"

using fg::fail;
using fg::Fixup;
using fg::Item;
using fg::wave_lds_sync;

namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kBlock = 64 * kWavesPerBlock;
constexpr int kStage = 1024;          // floats of a multi-row item staged in LDS per wavefront

struct SoftmaxArgs {
    const Item *items;
    int64_t n_items;
    const int32_t *indptr;
    const float *x;       // forward: scores; backward: the softmax output a
    const float *g;       // backward: dL/da
    float *y;
    float2 *stats;        // per (piece, head): forward (max, sum of exp); backward (sum of a * g, 0)
    int H;
    int W;                // lanes of a wavefront in use when lanes are tied to heads: the largest multiple of H <= 64
};

// Combines `v` over the lanes that hold the same head (lane % H, H a power of two <= 64), or over
// the whole wavefront when H == 1.
template <bool IS_MAX>
__device__ __forceinline__ float head_reduce(float v, int H) {
    for (int off = 32; off >= H; off >>= 1) {
        const float o = __shfl_xor(v, off);
        v = IS_MAX ? fmaxf(v, o) : v + o;
    }
    return v;
}

// The same for any H <= 64: the lanes below W (the largest multiple of H that a wavefront holds) carry head
// lane % H, the others carry nothing.  Windows of doubling length are folded towards the lanes below H, which
// then hand every lane the result of its head.
template <bool IS_MAX>
__device__ __forceinline__ float head_reduce_any(float v, int H, int W, int lane) {
    for (int off = H; off < W; off <<= 1) {
        const float o = __shfl_down(v, off);
        if (lane + off < W) v = IS_MAX ? fmaxf(v, o) : v + o;
    }
    return __shfl(v, lane % H);
}

// MODE 1: H a power of two, all 64 lanes in use; MODE 2: any H <= 64, W lanes in use.
template <bool IS_MAX, int MODE>
__device__ __forceinline__ float lanes_reduce(float v, int H, int W, int lane) {
    return MODE == 2 ? head_reduce_any<IS_MAX>(v, H, W, lane) : head_reduce<IS_MAX>(v, H);
}


// A whole row of n <= 64 * R floats (H a power of two <= 64, so lane i always meets head i % H):
// every lane's R loads are issued back to back, the row is read from memory once and the result
// is formed in registers.  No load sits under a branch: lanes past the end re-read the last float.
// l0: the lane's first index (its lane number; past every run for a lane that is not in use), W: lanes in use.
template <bool BWD, int R, int MODE>
__device__ __forceinline__ void row_in_registers(const float *x, const float *g, float *y, int n, int lane, int l0, int W, int H) {
    float v[R], w[BWD ? R : 1];
#pragma unroll
    for (int k = 0; k < R; ++k) {
        const int i = min(l0 + W * k, n - 1);
        v[k] = x[i];
        if (BWD) w[k] = g[i];
    }
    if (!BWD) {
        float m = -INFINITY;
#pragma unroll
        for (int k = 0; k < R; ++k) m = (l0 + W * k < n) ? fmaxf(m, v[k]) : m;
        m = lanes_reduce<true, MODE>(m, H, W, lane);
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < R; ++k) {
            v[k] = (l0 + W * k < n) ? __expf(v[k] - m) : 0.f;
            s += v[k];
        }
        s = lanes_reduce<false, MODE>(s, H, W, lane);
        const float inv = 1.0f / s;
#pragma unroll
        for (int k = 0; k < R; ++k)
            if (l0 + W * k < n) y[l0 + W * k] = v[k] * inv;
    } else {
        float d = 0.f;
#pragma unroll
        for (int k = 0; k < R; ++k) d += (l0 + W * k < n) ? v[k] * w[k] : 0.f;
        d = lanes_reduce<false, MODE>(d, H, W, lane);
#pragma unroll
        for (int k = 0; k < R; ++k)
            if (l0 + W * k < n) y[l0 + W * k] = v[k] * (w[k] - d);
    }
}

// One run of `len` elements starting at element e0, all lanes together.
//   LANEHEAD 1: H divides 64, lane i always meets head i % H, values are read as one coalesced run.
//   LANEHEAD 2: any H <= 64: the same with the first W lanes (the largest multiple of H), the rest idle.
//   LANEHEAD 0: one head at a time, lanes stride over the elements.
// STATS_ONLY: write (max, sum) / (dot, 0) to stats[slot * H + h] instead of the result.
// NORMALISE : the row statistics come from stats[slot * H + h] (merged over the row's pieces).
template <bool BWD, int LANEHEAD, bool STATS_ONLY, bool NORMALISE>
__device__ __forceinline__ void run_together(const SoftmaxArgs &a, int64_t e0, int len, int lane, int slot) {
    const int H = a.H;
    const int64_t base = e0 * H;
    const float *x = a.x + base;
    const float *g = BWD ? a.g + base : nullptr;
    float *y = a.y + base;
    if (LANEHEAD) {
        const int n = len * H;
        const int W = LANEHEAD == 2 ? a.W : 64;
        const int l0 = (LANEHEAD == 2 && lane >= W) ? (1 << 29) : lane;
        if (!STATS_ONLY && !NORMALISE) {
            if (n <= W * 2) { row_in_registers<BWD, 2, LANEHEAD>(x, g, y, n, lane, l0, W, H); return; }
            if (n <= W * 4) { row_in_registers<BWD, 4, LANEHEAD>(x, g, y, n, lane, l0, W, H); return; }
            if (n <= W * 8) { row_in_registers<BWD, 8, LANEHEAD>(x, g, y, n, lane, l0, W, H); return; }
        }
        // longer runs: sweeps of 8 loads per lane issued back to back (lanes past the end re-read
        // the last float, so no load sits under a branch)
        constexpr int U = 8;
        const int h = LANEHEAD == 2 ? lane % H : lane & (H - 1);
        float m = 0.f, s = 0.f;
        if (NORMALISE) {
            const float2 st = a.stats[(int64_t)slot * H + h];
            m = st.x; s = st.y;
        } else if (!BWD) {
            // one sweep: running maximum, the sum rescaled whenever the maximum grows
            m = -INFINITY;
            for (int i0 = l0, b0 = 0; b0 < n; i0 += W * U, b0 += W * U) {
                float v[U];
#pragma unroll
                for (int k = 0; k < U; ++k) v[k] = x[min(i0 + W * k, n - 1)];
#pragma unroll
                for (int k = 0; k < U; ++k) {
                    const float vk = (i0 + W * k < n) ? v[k] : -INFINITY;
                    const float mn = fmaxf(m, vk);
                    s = (m == mn ? s : s * __expf(m - mn)) + (vk == -INFINITY ? 0.f : __expf(vk - mn));
                    m = mn;
                }
            }
            const float mw = lanes_reduce<true, LANEHEAD>(m, H, W, lane);
            s = (m == -INFINITY) ? 0.f : s * __expf(m - mw);
            m = mw;
            s = lanes_reduce<false, LANEHEAD>(s, H, W, lane);
        } else {
            for (int i0 = l0, b0 = 0; b0 < n; i0 += W * U, b0 += W * U) {
                float v[U], w[U];
#pragma unroll
                for (int k = 0; k < U; ++k) { const int i = min(i0 + W * k, n - 1); v[k] = x[i]; w[k] = g[i]; }
#pragma unroll
                for (int k = 0; k < U; ++k) m += (i0 + W * k < n) ? v[k] * w[k] : 0.f;
            }
            m = lanes_reduce<false, LANEHEAD>(m, H, W, lane);
        }
        if (STATS_ONLY) {
            if (lane < H) a.stats[(int64_t)slot * H + lane] = make_float2(m, s);
            return;
        }
        if (!BWD) {
            const float inv = 1.0f / s;
            for (int i0 = l0, b0 = 0; b0 < n; i0 += W * U, b0 += W * U) {
                float v[U];
#pragma unroll
                for (int k = 0; k < U; ++k) v[k] = x[min(i0 + W * k, n - 1)];
#pragma unroll
                for (int k = 0; k < U; ++k)
                    if (i0 + W * k < n) y[i0 + W * k] = __expf(v[k] - m) * inv;
            }
        } else {
            for (int i0 = l0, b0 = 0; b0 < n; i0 += W * U, b0 += W * U) {
                float v[U], w[U];
#pragma unroll
                for (int k = 0; k < U; ++k) { const int i = min(i0 + W * k, n - 1); v[k] = x[i]; w[k] = g[i]; }
#pragma unroll
                for (int k = 0; k < U; ++k)
                    if (i0 + W * k < n) y[i0 + W * k] = v[k] * (w[k] - m);
            }
        }
        return;
    }
    for (int h = 0; h < H; ++h) {
        float m = 0.f, s = 0.f;
        if (NORMALISE) {
            const float2 st = a.stats[(int64_t)slot * H + h];
            m = st.x; s = st.y;
        } else if (!BWD) {
            m = -INFINITY;
            for (int j = lane; j < len; j += 64) m = fmaxf(m, x[(int64_t)j * H + h]);
            m = head_reduce<true>(m, 1);
            for (int j = lane; j < len; j += 64) s += __expf(x[(int64_t)j * H + h] - m);
            s = head_reduce<false>(s, 1);
        } else {
            for (int j = lane; j < len; j += 64) m += x[(int64_t)j * H + h] * g[(int64_t)j * H + h];
            m = head_reduce<false>(m, 1);
        }
        if (STATS_ONLY) {
            if (lane == 0) a.stats[(int64_t)slot * H + h] = make_float2(m, s);
            continue;
        }
        if (!BWD) {
            const float inv = 1.0f / s;
            for (int j = lane; j < len; j += 64) y[(int64_t)j * H + h] = __expf(x[(int64_t)j * H + h] - m) * inv;
        } else {
            for (int j = lane; j < len; j += 64) y[(int64_t)j * H + h] = x[(int64_t)j * H + h] * (g[(int64_t)j * H + h] - m);
        }
    }
}

// PIECES == false: rows held whole by an item are finished, pieces write their statistics.
// PIECES == true : pieces only, normalised with the merged statistics of their row.
template <bool BWD, int LANEHEAD, bool PIECES>
__device__ __forceinline__ void edge_softmax_body(const SoftmaxArgs &a) {
    __shared__ float s_x[kWavesPerBlock][kStage];
    __shared__ float s_g[BWD ? kWavesPerBlock : 1][BWD ? kStage : 1];
    const int lane = threadIdx.x & 63;
    const int64_t item_id = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (item_id >= a.n_items) return;         // uniform per wavefront; no workgroup barriers below
    const Item it = a.items[item_id];
    if (it.len == 0) return;
    if (it.info >= 0) {
        if (PIECES) run_together<BWD, LANEHEAD, false, true>(a, it.start, it.len, lane, it.info);
        else run_together<BWD, LANEHEAD, true, false>(a, it.start, it.len, lane, it.info);
        return;
    }
    if (PIECES) return;
    if (it.info == -1) {
        run_together<BWD, LANEHEAD, false, false>(a, it.start, it.len, lane, 0);
        return;
    }
    // several whole rows: lane q keeps the end of row q
    const int nrows = -it.info;
    const int H = a.H;
    const int ends = a.indptr[it.row + min(lane, nrows - 1) + 1];
    const int nf = it.len * H;
    if (nf <= kStage) {
        // The item's values are one contiguous run: copy it to LDS with coalesced loads, let one
        // lane per (row, head) work on its row there, and copy the result out the same way.
        float *sx = s_x[threadIdx.x >> 6];
        float *sg = s_g[BWD ? (threadIdx.x >> 6) : 0];
        const int64_t base = (int64_t)it.start * H;
        for (int i0 = 0; i0 < nf; i0 += 256) {
            float v[4], w[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int i = min(i0 + lane + 64 * k, nf - 1);
                v[k] = a.x[base + i];
                if (BWD) w[k] = a.g[base + i];
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int i = i0 + lane + 64 * k;
                if (i < nf) { sx[i] = v[k]; if (BWD) sg[i] = w[k]; }
            }
        }
        wave_lds_sync();
        const int tasks = nrows * H;
        for (int t0 = 0; t0 < tasks; t0 += 64) {
            const int t = min(t0 + lane, tasks - 1);
            const int q = t / H, h = t - q * H;
            const int prev = __shfl(ends, max(q - 1, 0));
            const int e = __shfl(ends, q) - it.start;
            const int b = q ? prev - it.start : 0;
            if (t0 + lane < tasks && e > b) {
                float *r = sx + b * H + h;
                const int len = e - b;
                if (!BWD) {
                    float m = r[0];
                    for (int j = 1; j < len; ++j) m = fmaxf(m, r[j * H]);
                    float sum = 0.f;
                    for (int j = 0; j < len; ++j) { const float ex = __expf(r[j * H] - m); r[j * H] = ex; sum += ex; }
                    const float inv = 1.0f / sum;
                    for (int j = 0; j < len; ++j) r[j * H] *= inv;
                } else {
                    const float *gr = sg + b * H + h;
                    float d = 0.f;
                    for (int j = 0; j < len; ++j) d += r[j * H] * gr[j * H];
                    for (int j = 0; j < len; ++j) r[j * H] *= gr[j * H] - d;
                }
            }
        }
        wave_lds_sync();
        for (int i = lane; i < nf; i += 64) a.y[base + i] = sx[i];
        return;
    }
    if ((int64_t)it.len * H >= 32 * (int64_t)nrows) {
        // long enough rows: the wavefront takes them one after the other
        int b = it.start;
        for (int q = 0; q < nrows; ++q) {
            const int e = __shfl(ends, q);
            if (e > b) run_together<BWD, LANEHEAD, false, false>(a, b, e - b, lane, 0);
            b = e;
        }
        return;
    }
    // short rows: one lane per (row, head), walking that row's values for its head
    const int tasks = nrows * H;
    for (int t0 = 0; t0 < tasks; t0 += 64) {
        const int t = min(t0 + lane, tasks - 1);
        const int q = t / H, h = t - q * H;
        const int prev = __shfl(ends, max(q - 1, 0));
        const int e = __shfl(ends, q);
        const int b = q ? prev : it.start;
        if (t0 + lane < tasks && e > b) {
            const float *x = a.x + (int64_t)b * H + h;
            float *y = a.y + (int64_t)b * H + h;
            const int len = e - b;
            if (!BWD) {
                float m = x[0];
                for (int j = 1; j < len; ++j) m = fmaxf(m, x[(int64_t)j * H]);
                float s = 0.f;
                for (int j = 0; j < len; ++j) s += __expf(x[(int64_t)j * H] - m);
                const float inv = 1.0f / s;
                for (int j = 0; j < len; ++j) y[(int64_t)j * H] = __expf(x[(int64_t)j * H] - m) * inv;
            } else {
                const float *g = a.g + (int64_t)b * H + h;
                float d = 0.f;
                for (int j = 0; j < len; ++j) d += x[(int64_t)j * H] * g[(int64_t)j * H];
                for (int j = 0; j < len; ++j) y[(int64_t)j * H] = x[(int64_t)j * H] * (g[(int64_t)j * H] - d);
            }
        }
    }
}

// The forward kernel is held to 64 registers (8 wavefronts per SIMD); the gradient kernel is bound
// by its two LDS staging rows per wavefront instead.
template <int LANEHEAD, bool PIECES>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(8, 8))) void edge_softmax_kernel(const SoftmaxArgs a) {
    edge_softmax_body<false, LANEHEAD, PIECES>(a);
}
template <int LANEHEAD, bool PIECES>
__global__ __launch_bounds__(kBlock) void edge_softmax_backward_kernel(const SoftmaxArgs a) {
    edge_softmax_body<true, LANEHEAD, PIECES>(a);
}

// Merges the pieces' statistics of every split row, in piece order, and writes the row's
// statistics back to each of its pieces.  One lane per (split row, head).
template <bool BWD>
__global__ __launch_bounds__(256) void edge_softmax_merge_kernel(const Fixup *fixups, int64_t n_fixups,
                                                                 float2 *stats, int H) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_fixups * H) return;
    const Fixup fx = fixups[t / H];
    const int h = (int)(t % H);
    float2 *s = stats + (int64_t)fx.slot0 * H + h;
    float m, sum = 0.f;
    if (!BWD) {
        m = s[0].x;
        for (int p = 1; p < fx.n_pieces; ++p) m = fmaxf(m, s[(int64_t)p * H].x);
        for (int p = 0; p < fx.n_pieces; ++p) sum += s[(int64_t)p * H].y * __expf(s[(int64_t)p * H].x - m);
    } else {
        m = 0.f;
        for (int p = 0; p < fx.n_pieces; ++p) m += s[(int64_t)p * H].x;
    }
    for (int p = 0; p < fx.n_pieces; ++p) s[(int64_t)p * H] = make_float2(m, sum);
}

// ---- statistics only, and the fused normalise-and-relayout step ------------------------------------
//
// For attention without a stored softmax: row_stats[v, h] = (max, sum of exp(x - max)) over row v, then
// edge_softmax_head_major_kernel writes exp(x - max) / sum straight into the head-major, traversal-ordered
// weight array that the per-head SpMM streams -- the [nnz, H] softmax array is never written or re-read.

template <int LANEHEAD>
__global__ __launch_bounds__(kBlock) void edge_softmax_stats_kernel(const SoftmaxArgs a, float2 *row_stats) {
    const int lane = threadIdx.x & 63;
    const int64_t item_id = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (item_id >= a.n_items) return;         // uniform per wavefront; no workgroup barriers below
    const Item it = a.items[item_id];
    if (it.len == 0) return;
    if (it.info >= 0) {                       // a piece: its statistics go to the plan's scratch, merged later
        run_together<false, LANEHEAD, true, false>(a, it.start, it.len, lane, it.info);
        return;
    }
    SoftmaxArgs rows = a;
    rows.stats = row_stats;                   // whole rows write their own entry, slot = row
    const int nrows = -it.info;
    const int ends = a.indptr[it.row + min(lane, nrows - 1) + 1];
    int b = it.start;
    for (int q = 0; q < nrows; ++q) {
        const int e = __shfl(ends, q);
        if (e > b) run_together<false, LANEHEAD, true, false>(rows, b, e - b, lane, it.row + q);
        b = e;
    }
}

// Merges the pieces of every split row and writes the row's entry of row_stats.
__global__ __launch_bounds__(256) void edge_softmax_stats_merge_kernel(const Fixup *fixups, int64_t n_fixups,
                                                                       const float2 *stats, float2 *row_stats, int H) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_fixups * H) return;
    const Fixup fx = fixups[t / H];
    const int h = (int)(t % H);
    const float2 *s = stats + (int64_t)fx.slot0 * H + h;
    float m = s[0].x, sum = 0.f;
    for (int p = 1; p < fx.n_pieces; ++p) m = fmaxf(m, s[(int64_t)p * H].x);
    for (int p = 0; p < fx.n_pieces; ++p) sum += s[(int64_t)p * H].y * __expf(s[(int64_t)p * H].x - m);
    row_stats[(int64_t)fx.row * H + h] = make_float2(m, sum);
}

// dst[h, e'] = exp(x[pos[e'], h] - max) / sum with the statistics of the row of stored element pos[e'].
__global__ __launch_bounds__(256) void edge_softmax_head_major_kernel(const float *x, const float2 *row_stats,
                                                                      const int32_t *edge_row, const int32_t *pos,
                                                                      int64_t n, int H, float *dst) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n) return;
    const int64_t at = pos ? (int64_t)pos[e] : e;
    const float *xs = x + at * H;
    const float2 *st = row_stats + (int64_t)edge_row[at] * H;
    for (int h = 0; h < H; ++h) dst[(int64_t)h * n + e] = __expf(xs[h] - st[h].x) / st[h].y;
}

// The same for H = 4 * Q heads and 16-byte aligned arrays: an element's scores by Q 128-bit loads and its row's
// statistics by 2 Q, two elements per lane (a block apart: every store of a wavefront covers 64 consecutive elements
// of one head); exp and division as in the kernel above, so both give the same bits.
template <int Q>
__global__ __launch_bounds__(256) void edge_softmax_head_major_vec_kernel(const float *x, const float2 *row_stats,
                                                                          const int32_t *edge_row, const int32_t *pos,
                                                                          int64_t n, float *dst) {
    constexpr int H = 4 * Q;
    const int64_t e0 = (int64_t)blockIdx.x * 512 + threadIdx.x;
    float4 xs[2][Q], st[2][2 * Q];
    bool ok[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int64_t e = e0 + 256 * j;
        ok[j] = e < n;
        const int64_t ec = ok[j] ? e : n - 1;                   // clamped: no branch around the loads
        const int64_t at = pos ? (int64_t)pos[ec] : ec;
        const float4 *xp = reinterpret_cast<const float4 *>(x + at * H);
        const float4 *sp = reinterpret_cast<const float4 *>(row_stats + (int64_t)edge_row[at] * H);
#pragma unroll
        for (int q = 0; q < Q; ++q) xs[j][q] = xp[q];
#pragma unroll
        for (int q = 0; q < 2 * Q; ++q) st[j][q] = sp[q];       // (max, sum) of heads 2q and 2q + 1
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        if (!ok[j]) continue;
        float *d = dst + e0 + 256 * j;
#pragma unroll
        for (int q = 0; q < Q; ++q) {
            d[(int64_t)(4 * q + 0) * n] = __expf(xs[j][q].x - st[j][2 * q].x) / st[j][2 * q].y;
            d[(int64_t)(4 * q + 1) * n] = __expf(xs[j][q].y - st[j][2 * q].z) / st[j][2 * q].w;
            d[(int64_t)(4 * q + 2) * n] = __expf(xs[j][q].z - st[j][2 * q + 1].x) / st[j][2 * q + 1].y;
            d[(int64_t)(4 * q + 3) * n] = __expf(xs[j][q].w - st[j][2 * q + 1].z) / st[j][2 * q + 1].w;
        }
    }
}

template <bool BWD, int LANEHEAD>
void launch_both(const fg_spmm_plan *pl, const SoftmaxArgs &a, hipStream_t st) {
    const dim3 grid((unsigned)((pl->n_items + kWavesPerBlock - 1) / kWavesPerBlock));
    if (BWD) hipLaunchKernelGGL((edge_softmax_backward_kernel<LANEHEAD, false>), grid, dim3(kBlock), 0, st, a);
    else hipLaunchKernelGGL((edge_softmax_kernel<LANEHEAD, false>), grid, dim3(kBlock), 0, st, a);
    if (pl->n_fixups > 0) {
        const int64_t threads = pl->n_fixups * a.H;
        hipLaunchKernelGGL(edge_softmax_merge_kernel<BWD>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st,
                           pl->fixups_dev, pl->n_fixups, a.stats, a.H);
        if (BWD) hipLaunchKernelGGL((edge_softmax_backward_kernel<LANEHEAD, true>), grid, dim3(kBlock), 0, st, a);
        else hipLaunchKernelGGL((edge_softmax_kernel<LANEHEAD, true>), grid, dim3(kBlock), 0, st, a);
    }
}

// How a wavefront's lanes meet the heads: 1: H divides 64; 2: any other H <= 64 (the lanes past the largest multiple of
// H stay idle); 0: more heads than lanes, one head at a time.
int lane_mode(int H) { return H > 64 ? 0 : (H & (H - 1)) == 0 ? 1 : 2; }

int softmax_run(fg_spmm_plan *pl, const int32_t *indptr, const float *x, const float *g, float *y,
                int H, void *stream, bool bwd) {
    if (!pl) return fail(FG_ERR_ARG, "plan is null");
    if (int drc = fg::check_device(pl)) return drc;
    if (pl->num_col_partitions != 1) return fail(FG_ERR_ARG, "edge softmax needs a plan with one column partition");
    if (H < 1) return fail(FG_ERR_SHAPE, "number of heads must be positive, got %d", H);
    if (pl->nnz == 0 || pl->n_items == 0) return FG_OK;
    if (!indptr || !x || !y || (bwd && !g)) return fail(FG_ERR_ARG, "null device pointer");
    if ((pl->n_items + kWavesPerBlock - 1) / kWavesPerBlock > 0x7fffffffLL)
        return fail(FG_ERR_SHAPE, "too many work items for one grid");
    fg::ScratchNeed need;
    int rc = fg::softmax_scratch_need(pl, H, &need);
    if (rc == FG_OK) rc = fg::ensure_scratch(pl, need, stream);
    if (rc != FG_OK) return rc;
    SoftmaxArgs a;
    a.items = pl->items_dev; a.n_items = pl->n_items; a.indptr = indptr;
    a.x = x; a.g = g; a.y = y; a.stats = reinterpret_cast<float2 *>(pl->partial_dev); a.H = H;
    hipStream_t st = (hipStream_t)stream;
    const int mode = lane_mode(H);
    a.W = H <= 64 ? 64 / H * H : 64;
    if (bwd) {
        if (mode == 1) launch_both<true, 1>(pl, a, st);
        else if (mode == 2) launch_both<true, 2>(pl, a, st);
        else launch_both<true, 0>(pl, a, st);
    } else {
        if (mode == 1) launch_both<false, 1>(pl, a, st);
        else if (mode == 2) launch_both<false, 2>(pl, a, st);
        else launch_both<false, 0>(pl, a, st);
    }
    FG_HIP_TRY(hipGetLastError());
    return FG_OK;
}

}  // namespace

namespace fg {
// (max, sum) per head for every piece of a split row
int softmax_scratch_need(const fg_spmm_plan *pl, int heads, ScratchNeed *need) {
    if (heads < 1) return fail(FG_ERR_SHAPE, "number of heads must be positive, got %d", heads);
    need->partial = (size_t)pl->max_slots_in_partition * 2 * (size_t)heads;
    need->tiled = 0;
    return FG_OK;
}
}  // namespace fg

extern "C" int fg_edge_softmax_f32(fg_spmm_plan *plan, const int32_t *indptr_dev, const float *scores_dev,
                                   float *out_dev, int heads, void *stream) {
    return softmax_run(plan, indptr_dev, scores_dev, nullptr, out_dev, heads, stream, false);
}

extern "C" int fg_edge_softmax_stats_f32(fg_spmm_plan *pl, const int32_t *indptr_dev, const float *scores_dev,
                                         float *row_stats_dev, int heads, void *stream) {
    if (!pl) return fail(FG_ERR_ARG, "plan is null");
    if (int drc = fg::check_device(pl)) return drc;
    if (pl->num_col_partitions != 1) return fail(FG_ERR_ARG, "edge softmax needs a plan with one column partition");
    if (heads < 1) return fail(FG_ERR_SHAPE, "number of heads must be positive, got %d", heads);
    if (pl->nnz == 0 || pl->n_items == 0) return FG_OK;
    if (!indptr_dev || !scores_dev || !row_stats_dev) return fail(FG_ERR_ARG, "null device pointer");
    if (((uintptr_t)row_stats_dev & 7) != 0) return fail(FG_ERR_ARG, "row_stats must be 8-byte aligned");
    fg::ScratchNeed need;
    int rc = fg::softmax_scratch_need(pl, heads, &need);
    if (rc == FG_OK) rc = fg::ensure_scratch(pl, need, stream);
    if (rc != FG_OK) return rc;
    SoftmaxArgs a;
    a.items = pl->items_dev; a.n_items = pl->n_items; a.indptr = indptr_dev;
    a.x = scores_dev; a.g = nullptr; a.y = nullptr; a.stats = reinterpret_cast<float2 *>(pl->partial_dev); a.H = heads;
    hipStream_t st = (hipStream_t)stream;
    float2 *row_stats = reinterpret_cast<float2 *>(row_stats_dev);
    const dim3 grid((unsigned)((pl->n_items + kWavesPerBlock - 1) / kWavesPerBlock));
    a.W = heads <= 64 ? 64 / heads * heads : 64;
    const int mode = lane_mode(heads);
    if (mode == 1) hipLaunchKernelGGL(edge_softmax_stats_kernel<1>, grid, dim3(kBlock), 0, st, a, row_stats);
    else if (mode == 2) hipLaunchKernelGGL(edge_softmax_stats_kernel<2>, grid, dim3(kBlock), 0, st, a, row_stats);
    else hipLaunchKernelGGL(edge_softmax_stats_kernel<0>, grid, dim3(kBlock), 0, st, a, row_stats);
    if (pl->n_fixups > 0) {
        const int64_t threads = pl->n_fixups * heads;
        hipLaunchKernelGGL(edge_softmax_stats_merge_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st,
                           pl->fixups_dev, pl->n_fixups, a.stats, row_stats, heads);
    }
    FG_HIP_TRY(hipGetLastError());
    return FG_OK;
}

extern "C" int fg_edge_softmax_head_major_f32(const float *scores_dev, const float *row_stats_dev,
                                              const int32_t *edge_row_dev, const int32_t *edge_pos_dev, int64_t n_edges,
                                              int heads, float *dst_dev, void *stream) {
    if (n_edges < 0 || heads < 1) return fail(FG_ERR_ARG, "fg_edge_softmax_head_major_f32: bad size");
    if (n_edges == 0) return FG_OK;
    if (!scores_dev || !row_stats_dev || !edge_row_dev || !dst_dev) return fail(FG_ERR_ARG, "null device pointer");
    const int64_t blocks = (n_edges + 255) / 256;
    if (blocks > 0x7fffffffLL) return fail(FG_ERR_SHAPE, "too many edges for one grid");
    hipStream_t st = (hipStream_t)stream;
    const float2 *stats = reinterpret_cast<const float2 *>(row_stats_dev);
    const dim3 wide((unsigned)((n_edges + 511) / 512));
    const bool aligned = (((uintptr_t)scores_dev | (uintptr_t)row_stats_dev) & 15) == 0;
    if (aligned && heads == 4)
        hipLaunchKernelGGL(edge_softmax_head_major_vec_kernel<1>, wide, dim3(256), 0, st, scores_dev, stats, edge_row_dev,
                           edge_pos_dev, n_edges, dst_dev);
    else if (aligned && heads == 8)
        hipLaunchKernelGGL(edge_softmax_head_major_vec_kernel<2>, wide, dim3(256), 0, st, scores_dev, stats, edge_row_dev,
                           edge_pos_dev, n_edges, dst_dev);
    else
        hipLaunchKernelGGL(edge_softmax_head_major_kernel, dim3((unsigned)blocks), dim3(256), 0, st,
                           scores_dev, stats, edge_row_dev, edge_pos_dev, n_edges, heads, dst_dev);
    FG_HIP_TRY(hipGetLastError());
    return FG_OK;
}

extern "C" int fg_edge_softmax_backward_f32(fg_spmm_plan *plan, const int32_t *indptr_dev,
                                            const float *softmax_dev, const float *grad_softmax_dev,
                                            float *grad_scores_dev, int heads, void *stream) {
    return softmax_run(plan, indptr_dev, softmax_dev, grad_softmax_dev, grad_scores_dev, heads, stream, true);
}
