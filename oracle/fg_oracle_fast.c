/*
 * Timing-only copies of the oracle's three hot loop nests.  TEST INFRASTRUCTURE ONLY.
 *
 * fg_oracle.c is compiled for AVX2 with multiply and add kept separately rounded, because it is the
 * bit-pinned checker.  A CPU time printed beside the GPU's should not carry that handicap, so the
 * same loop nests are restated here with fused multiply-add allowed and with the per-row / per-edge
 * inner kernels cloned for AVX-512 (chosen at load time by the CPU that runs them):
 *   orcf_spmm_csr_x86   ~ orc_spmm_csr_x86   (python/featgraph/op/vanilla_spmm.py:6-62, schedule :65-80)
 *   orcf_spmm_dds_x86   ~ orc_spmm_dds_x86   (vanilla_spmm.py:149-224, schedule :227-246)
 *   orcf_sddmm_x86      ~ orc_sddmm_x86      (python/featgraph/op/vanilla_sddmm.py:6-63, schedule :66-74)
 * Same arguments, loop order and threading as the pinned functions.  Their results are NOT a parity
 * reference (fusing changes the last bits); tests/test_oracle.py only checks that they stay within
 * the fp32 tolerance of the pinned ones.  bench.py's cpu_baseline times both sets and says which is which.
 */
#include <stdint.h>
#include <stdlib.h>

#define ORC_OK 0
#define ORC_EARG -1
#define ORC_ENOMEM -2

/* Versions for AVX-512 and for the build's baseline (AVX2 + FMA); the loader picks one per process. */
#define ORC_CLONES __attribute__((target_clones("avx512f", "default"), noinline))

static void relayout_in(const float *x, float *rx, int64_t n, int F, int T, int nthreads) {
    const int Fp = F / T;
    for (int fo = 0; fo < T; ++fo) {
#pragma omp parallel for num_threads(nthreads) schedule(static)
        for (int64_t v = 0; v < n; ++v)
            for (int fi = 0; fi < Fp; ++fi)
                rx[((int64_t)fo * n + v) * Fp + fi] = x[v * F + fo * Fp + fi];
    }
}

static void relayout_out(const float *ro, float *out, int64_t n, int F, int T, int nthreads) {
    const int Fp = F / T;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int64_t v = 0; v < n; ++v)
        for (int f = 0; f < F; ++f)
            out[v * F + f] = ro[((int64_t)(f / Fp) * n + v) * Fp + (f % Fp)];
}

/* o[0..Fp) (+)= sum over elements [b, e) of vals * rows of rxf; the functions called from inside the
 * parallel regions are the cloned ones (the regions' own bodies are compiled once). */
ORC_CLONES static void row_sum(float *restrict o, int Fp, int32_t b, int32_t e, const int32_t *restrict idx,
                               const float *restrict vals, const float *restrict rxf, int64_t col0, int add) {
    float acc[Fp];
    for (int fi = 0; fi < Fp; ++fi) acc[fi] = 0.0f;
    for (int32_t k = b; k < e; ++k) {
        const float w = vals[k];
        const float *xr = rxf + ((int64_t)idx[k] + col0) * Fp;
        for (int fi = 0; fi < Fp; ++fi) acc[fi] += w * xr[fi];
    }
    if (add) for (int fi = 0; fi < Fp; ++fi) o[fi] += acc[fi];
    else for (int fi = 0; fi < Fp; ++fi) o[fi] = acc[fi];
}

int orcf_spmm_csr_x86(int64_t n_dst, int64_t n_src, int F, const int32_t *indptr, const int32_t *indices,
                      const float *vals, const float *x, float *out, int num_feat_partitions, int nthreads) {
    const int T = num_feat_partitions;
    if (T < 1 || F < 1 || F % T != 0 || nthreads < 1) return ORC_EARG;
    const int Fp = F / T;
    float *rx = (float *)malloc(sizeof(float) * (size_t)(n_src ? n_src : 1) * F);
    float *ro = (float *)malloc(sizeof(float) * (size_t)(n_dst ? n_dst : 1) * F);
    if (!rx || !ro) { free(rx); free(ro); return ORC_ENOMEM; }
    relayout_in(x, rx, n_src, F, T, nthreads);
    for (int fo = 0; fo < T; ++fo) {
        const float *rxf = rx + (int64_t)fo * n_src * Fp;
        float *rof = ro + (int64_t)fo * n_dst * Fp;
#pragma omp parallel for num_threads(nthreads) schedule(dynamic, 64)
        for (int64_t row = 0; row < n_dst; ++row)
            row_sum(rof + row * Fp, Fp, indptr[row], indptr[row + 1], indices, vals, rxf, 0, 0);
    }
    relayout_out(ro, out, n_dst, F, T, nthreads);
    free(rx); free(ro);
    return ORC_OK;
}

int orcf_spmm_dds_x86(int64_t n_dst, int64_t n_src, int F, int P, const int32_t *s1_pos, const int32_t *s1_idx,
                      const float *vals, const float *x, float *out, int num_feat_partitions, int nthreads) {
    const int T = num_feat_partitions;
    if (T < 1 || P < 1 || F < 1 || F % T != 0 || nthreads < 1) return ORC_EARG;
    const int Fp = F / T;
    const int64_t d2 = n_dst + 1;
    const int64_t cols_per_part = (n_src + P - 1) / P;
    float *rx = (float *)malloc(sizeof(float) * (size_t)(n_src ? n_src : 1) * F);
    float *ro = (float *)malloc(sizeof(float) * (size_t)(n_dst ? n_dst : 1) * F);
    if (!rx || !ro) { free(rx); free(ro); return ORC_ENOMEM; }
    relayout_in(x, rx, n_src, F, T, nthreads);
    for (int fo = 0; fo < T; ++fo) {
        const float *rxf = rx + (int64_t)fo * n_src * Fp;
        float *rof = ro + (int64_t)fo * n_dst * Fp;
        for (int p = 0; p < P; ++p) {
            const int32_t *pos = s1_pos + (int64_t)p * d2;
#pragma omp parallel for num_threads(nthreads) schedule(dynamic, 64)
            for (int64_t row = 0; row < n_dst; ++row)
                row_sum(rof + row * Fp, Fp, pos[row], pos[row + 1], s1_idx, vals, rxf, (int64_t)p * cols_per_part, p > 0);
        }
    }
    relayout_out(ro, out, n_dst, F, T, nthreads);
    free(rx); free(ro);
    return ORC_OK;
}

/* out[e] (+)= <s rows gathered by col, d rows gathered by row> for edges [e0, e1), Fp floats each */
ORC_CLONES static void edge_dots(float *restrict out, int64_t e0, int64_t e1, const int32_t *restrict row,
                                 const int32_t *restrict col, const float *restrict s, const float *restrict d,
                                 int Fp, int add) {
    for (int64_t e = e0; e < e1; ++e) {
        const float *sr = s + (int64_t)col[e] * Fp;
        const float *dr = d + (int64_t)row[e] * Fp;
        float acc = add ? out[e] : 0.0f;
        for (int k = 0; k < Fp; ++k) acc += sr[k] * dr[k];
        out[e] = acc;
    }
}

int orcf_sddmm_x86(int64_t n_edges, int64_t n_src_rows, int64_t n_dst_rows, int F, const int32_t *row,
                   const int32_t *col, const float *src, const float *dst, float *out, int num_feat_partitions,
                   int parallel_edges, int nthreads) {
    const int T = num_feat_partitions;
    if (T < 1 || F < 1 || F % T != 0 || nthreads < 1) return ORC_EARG;
    const int nt = parallel_edges ? nthreads : 1;
    const int64_t chunk = 4096;
    const int64_t n_chunks = (n_edges + chunk - 1) / chunk;
    const int Fp = F / T;
    float *rs = NULL, *rd = NULL;
    if (T > 1) {
        rs = (float *)malloc(sizeof(float) * (size_t)(n_src_rows ? n_src_rows : 1) * F);
        rd = (float *)malloc(sizeof(float) * (size_t)(n_dst_rows ? n_dst_rows : 1) * F);
        if (!rs || !rd) { free(rs); free(rd); return ORC_ENOMEM; }
        relayout_in(src, rs, n_src_rows, F, T, 1);
        relayout_in(dst, rd, n_dst_rows, F, T, 1);
    }
    for (int fo = 0; fo < T; ++fo) {
        const float *sf = T > 1 ? rs + (int64_t)fo * n_src_rows * Fp : src;
        const float *df = T > 1 ? rd + (int64_t)fo * n_dst_rows * Fp : dst;
        if (nt == 1) {
            edge_dots(out, 0, n_edges, row, col, sf, df, Fp, fo > 0);
        } else {
#pragma omp parallel for num_threads(nt) schedule(static)
            for (int64_t c = 0; c < n_chunks; ++c)
                edge_dots(out, c * chunk, (c + 1) * chunk < n_edges ? (c + 1) * chunk : n_edges, row, col, sf, df, Fp, fo > 0);
        }
    }
    free(rs); free(rd);
    return ORC_OK;
}
