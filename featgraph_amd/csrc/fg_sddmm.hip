// Edge-wise dot products (SDDMM) for gfx950, single- and multi-head:
//   out[e, h] = sum_{d<D} src[col[e], h, d] * dst[row[e], h, d]
//
// Edge-parallel: a wavefront owns a run of consecutive stored edges.  A group of L lanes
// covers one edge's F = H*D floats with K vector loads per operand, the 64/L groups work on
// different edges at once, and each head's products are added across its lanes with a
// butterfly of cross-lane shuffles.  Row/column ids are staged 64 at a time in LDS, results
// are collected in LDS and written back as one coalesced run per 64 edges.  When the stored
// order keeps equal row ids together (CSR order, 2-D partitioned order) the dst row already
// held in registers is reused instead of fetched again.
#include <hip/hip_runtime.h>

#include "fg_common.h"

using fg::fail;
using fg::Item;

namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kBlock = 64 * kWavesPerBlock;
constexpr int kEdgesPerWave = 256;       // COO kernel: stored edges per wavefront
constexpr int kMaxHeadsFast = 16;        // LDS result staging holds 64 * H floats per wavefront

template <int V> struct Vec;
template <> struct Vec<4> { using type = float4; };
template <> struct Vec<1> { using type = float; };

__device__ __forceinline__ float vdot(const float4 &a, const float4 &b) {
    return a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w;
}
__device__ __forceinline__ float vdot(const float &a, const float &b) { return a * b; }
__device__ __forceinline__ float4 vzero4() { return make_float4(0.f, 0.f, 0.f, 0.f); }

__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Sum over the RW consecutive lanes of a head segment; every lane of the segment gets it.
template <int RW>
__device__ __forceinline__ float segment_sum(float v) {
#pragma unroll
    for (int off = 1; off < RW; off <<= 1) v += __shfl_xor(v, off);
    return v;
}

struct SddmmArgs {
    const int32_t *row;     // COO kernel: row id per stored edge
    const int32_t *col;     // column id per stored edge
    const Item *items;      // CSR kernel: row pieces
    int64_t n_items;
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

// Stored-order (COO) kernel.
template <int V, int L, int K, int RW, int KH, bool FULL>
__global__ __launch_bounds__(kBlock) void sddmm_coo_kernel(const SddmmArgs a) {
    using S = Shape<V, L, K, RW, KH>;
    using vec = typename S::vec;
    constexpr int G = S::G, H = S::H;
    constexpr int U = (K >= 2) ? 2 : 4;
    __shared__ int32_t s_row[kWavesPerBlock][64];
    __shared__ int32_t s_col[kWavesPerBlock][64];
    __shared__ float s_out[kWavesPerBlock][64 * H];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane / L, li = lane % L;
    const int64_t e_begin = ((int64_t)blockIdx.x * kWavesPerBlock + wave) * kEdgesPerWave;
    if (e_begin >= a.n_edges) return;
    const int64_t e_end = min(e_begin + (int64_t)kEdgesPerWave, a.n_edges);
    const int64_t F = a.F;
    bool on[K];
#pragma unroll
    for (int k = 0; k < K; ++k) on[k] = FULL || (k * L * V + li * V < a.F);
    const float *sb = a.src + li * V;
    const float *db = a.dst + li * V;

    int32_t held_row = -1;                 // row whose dst vectors are in dv[]
    vec dv[K];
#pragma unroll
    for (int k = 0; k < K; ++k) dv[k] = vec();

    for (int64_t base = e_begin; base < e_end; base += 64) {
        const int n = (int)min((int64_t)64, e_end - base);
        int32_t r = 0, c = 0;
        if (lane < n) { r = a.row[base + lane]; c = a.col[base + lane]; }
        wave_lds_sync();
        s_row[wave][lane] = r;
        s_col[wave][lane] = c;
        wave_lds_sync();

        const int nsteps = (n + G - 1) / G;
        for (int s0 = 0; s0 < nsteps; s0 += U) {
            int32_t er[U], ec[U];
            bool live[U];
            vec sv[U][K];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int j = (s0 + u) * G + g;
                live[u] = j < n;
                er[u] = live[u] ? s_row[wave][j] : -1;
                ec[u] = live[u] ? s_col[wave][j] : 0;
            }
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int k = 0; k < K; ++k)
                    if (live[u] && on[k]) sv[u][k] = *reinterpret_cast<const vec *>(sb + (int64_t)ec[u] * F + k * L * V);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (live[u] && er[u] != held_row) {
#pragma unroll
                    for (int k = 0; k < K; ++k)
                        if (on[k]) dv[k] = *reinterpret_cast<const vec *>(db + (int64_t)er[u] * F + k * L * V);
                    held_row = er[u];
                }
                float q[K / KH];
                edge_heads<V, L, K, RW, KH, FULL>(sv[u], dv, on, q);
                if (live[u] && (li % RW) == 0) {
                    const int j = (s0 + u) * G + g;
#pragma unroll
                    for (int kk = 0; kk < K / KH; ++kk) s_out[wave][j * H + kk * S::HPL + li / RW] = q[kk];
                }
            }
        }
        wave_lds_sync();
        for (int t = lane; t < n * H; t += 64) a.out[base * H + t] = s_out[wave][t];
    }
}

// CSR-order kernel over plan items: edges [start, start+len) all belong to row `row`.
template <int V, int L, int K, int RW, int KH, bool FULL>
__global__ __launch_bounds__(kBlock) void sddmm_csr_kernel(const SddmmArgs a) {
    using S = Shape<V, L, K, RW, KH>;
    using vec = typename S::vec;
    constexpr int G = S::G, H = S::H;
    constexpr int U = (K >= 2) ? 2 : 4;
    __shared__ int32_t s_col[kWavesPerBlock][64];
    __shared__ float s_out[kWavesPerBlock][64 * H];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane / L, li = lane % L;
    const int64_t item_id = (int64_t)blockIdx.x * kWavesPerBlock + wave;
    if (item_id >= a.n_items) return;
    const Item it = a.items[item_id];
    if (it.len == 0) return;
    const int64_t F = a.F;
    bool on[K];
#pragma unroll
    for (int k = 0; k < K; ++k) on[k] = FULL || (k * L * V + li * V < a.F);
    const float *sb = a.src + li * V;
    vec dv[K];
#pragma unroll
    for (int k = 0; k < K; ++k)
        if (on[k]) dv[k] = *reinterpret_cast<const vec *>(a.dst + (int64_t)it.row * F + k * L * V + li * V);

    for (int32_t base = 0; base < it.len; base += 64) {
        const int n = min(64, it.len - base);
        int32_t c = 0;
        if (lane < n) c = a.col[it.start + base + lane];
        wave_lds_sync();
        s_col[wave][lane] = c;
        wave_lds_sync();
        const int nsteps = (n + G - 1) / G;
        for (int s0 = 0; s0 < nsteps; s0 += U) {
            int32_t ec[U];
            bool live[U];
            vec sv[U][K];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int j = (s0 + u) * G + g;
                live[u] = j < n;
                ec[u] = live[u] ? s_col[wave][j] : 0;
            }
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int k = 0; k < K; ++k)
                    if (live[u] && on[k]) sv[u][k] = *reinterpret_cast<const vec *>(sb + (int64_t)ec[u] * F + k * L * V);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float q[K / KH];
                edge_heads<V, L, K, RW, KH, FULL>(sv[u], dv, on, q);
                if (live[u] && (li % RW) == 0) {
                    const int j = (s0 + u) * G + g;
#pragma unroll
                    for (int kk = 0; kk < K / KH; ++kk) s_out[wave][j * H + kk * S::HPL + li / RW] = q[kk];
                }
            }
        }
        wave_lds_sync();
        for (int t = lane; t < n * H; t += 64) a.out[((int64_t)it.start + base) * H + t] = s_out[wave][t];
    }
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
    if (!col || !src || !dst || !out || (!row && !pl)) return fail(FG_ERR_ARG, "null device pointer");
    if ((int64_t)H * D > INT32_MAX) return fail(FG_ERR_SHAPE, "H*D too large");
    hipStream_t st = (hipStream_t)stream;
    const bool aligned16 = (((uintptr_t)src | (uintptr_t)dst) & 15) == 0;
    SddmmConfig c;
    choose_config(H, D, aligned16, &c);
    SddmmArgs a;
    a.row = row; a.col = col; a.items = pl ? pl->items_dev : nullptr; a.n_items = pl ? pl->n_items : 0;
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
        if (csr && !indptr) return fail(FG_ERR_ARG, "indptr_dev is needed for this shape");
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
    if (plan->num_col_partitions != 1) return fail(FG_ERR_ARG, "fg_sddmm_csr_f32 needs a plan with one column partition");
    return sddmm_run(plan, nullptr, indices_dev, indptr_dev, plan->n_dst, plan->nnz, src_dev, dst_dev,
                     out_dev, H, D, stream);
}
