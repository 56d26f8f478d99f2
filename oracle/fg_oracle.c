/*
 * CPU oracle for the FeatGraph SpMM / SDDMM path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the loop nests that the reference describes
 * as TVM compute + x86 schedule pairs, plus its two host-side graph
 * partitioners.  It is the checker that the HIP kernels are compared against
 * and the "port" CPU baseline that the benchmark times; nothing in the shipped
 * package links, loads or calls it.
 *
 * The reference executes these loop nests through Apache TVM (unpinned, not
 * vendored, absent here), so this is a restatement of the loop structure the
 * schedules fix, not a build of reference code.
 *
 * How each function is pinned (see tests/test_oracle.py):
 *   orc_spmm_csr_x86, orc_spmm_dds_x86, orc_spmm_csr_rowwise
 *       scipy.sparse csr.dot (the reference's own check,
 *       tests/test_module_spmm.py:29-30) and a float64 product; identity and
 *       empty-row special cases; bit-invariance under num_feat_partitions.
 *   orc_sddmm_x86
 *       numpy gather-multiply-sum (tests/test_module_sddmm.py:34-37), float64
 *       einsum; operand-swap symmetry; bit-invariance under feature tiling.
 *   orc_csr_to_dds, orc_partition_coo_2d
 *       the reference's stored vectors (tests/test_util.py:22-24, :43), scipy
 *       sub-matrix slicing on random matrices, brute-force invariants.
 *   orc_gspmm
 *       PARITY UNPINNED by the reference: max / min / per-head-weighted aggregation is what
 *       README.md:9-11 points to ("generalized SpMM") but the snapshot holds no code, test or
 *       vector for it.  Pinned by numpy maximum/minimum.reduceat closed forms, by reduce == sum
 *       with H == 1 equalling orc_spmm_csr_rowwise bit-exactly, and by brute force on tiny inputs.
 *   orc_gspmm_arg
 *       PARITY UNPINNED by the reference (no such operator).  Pinned by numpy argmax / argmin over the
 *       gathered messages on inputs with many ties, and by its values equalling orc_gspmm's.
 *   orc_edge_softmax, orc_edge_softmax_backward
 *       PARITY UNPINNED by the reference: the snapshot has no attention / softmax operator at all.
 *       Pinned by scipy.special.softmax per row in float64, rows summing to 1, invariance under a
 *       per-row shift, one-element rows giving 1, and for the backward pass by torch's float64
 *       autograd of a dense masked softmax and by central finite differences.
 *   orc_sddmm_multihead
 *       PARITY UNPINNED by the reference: the reference snapshot holds no
 *       multi-head op, test or vector (python/featgraph/op/__init__.py:1-5).
 *       It is pinned only by its closed form (einsum 'ehd,ehd->eh'), by H=1
 *       reducing to orc_sddmm_x86, and by head sums equalling the flat SDDMM.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_OK 0
#define ORC_EARG -1
#define ORC_ENOMEM -2
#define ORC_EDUP -3

int orc_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ReshapedSrcFeat[fo, n, fi] = SrcFeat[n, fo*Fp + fi]
 * (python/featgraph/op/vanilla_spmm.py:43-44; parallel over n, :76). */
static void relayout_in(const float *x, float *rx, int64_t n, int F, int T, int nthreads) {
    const int Fp = F / T;
    for (int fo = 0; fo < T; ++fo) {
#pragma omp parallel for num_threads(nthreads) schedule(static)
        for (int64_t v = 0; v < n; ++v)
            for (int fi = 0; fi < Fp; ++fi)
                rx[((int64_t)fo * n + v) * Fp + fi] = x[v * F + fo * Fp + fi];
    }
}

/* Out[n, f] = ReshapedOut[f / Fp, n, f % Fp]
 * (python/featgraph/op/vanilla_spmm.py:58-60; parallel over n, :78). */
static void relayout_out(const float *ro, float *out, int64_t n, int F, int T, int nthreads) {
    const int Fp = F / T;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int64_t v = 0; v < n; ++v)
        for (int f = 0; f < F; ++f)
            out[v * F + f] = ro[((int64_t)(f / Fp) * n + v) * Fp + (f % Fp)];
}

/*
 * Feature-tiled CSR SpMM on x86: compute python/featgraph/op/vanilla_spmm.py:6-62,
 * schedule :65-80.  Loop order fo -> row (parallel) -> elem -> fi; each output
 * element accumulates sequentially in stored CSR element order, starting at 0.
 * The two re-layout stages are inside the built function, so they are inside
 * this one too and a timing of it pays for them as the reference does.
 */
int orc_spmm_csr_x86(int64_t n_dst, int64_t n_src, int F, const int32_t *indptr,
                     const int32_t *indices, const float *vals, const float *x,
                     float *out, int num_feat_partitions, int nthreads) {
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
        for (int64_t row = 0; row < n_dst; ++row) {
            float *o = rof + row * Fp;
            for (int fi = 0; fi < Fp; ++fi) o[fi] = 0.0f;
            for (int32_t e = indptr[row]; e < indptr[row + 1]; ++e) {
                const float w = vals[e];
                const float *xr = rxf + (int64_t)indices[e] * Fp;
                for (int fi = 0; fi < Fp; ++fi) o[fi] += w * xr[fi];
            }
        }
    }
    relayout_out(ro, out, n_dst, F, T, nthreads);
    free(rx); free(ro);
    return ORC_OK;
}

/*
 * CSR SpMM without layout transformation: the math of the CUDA compute
 * python/featgraph/op/vanilla_spmm.py:83-125 (Out[row, ff] = sum over the row's
 * elements of vals[e] * SrcFeat[indices[e], ff]), evaluated on the host with a
 * sequential per-element sum.
 */
int orc_spmm_csr_rowwise(int64_t n_dst, int F, const int32_t *indptr,
                         const int32_t *indices, const float *vals, const float *x,
                         float *out, int nthreads) {
    if (F < 1 || nthreads < 1) return ORC_EARG;
#pragma omp parallel for num_threads(nthreads) schedule(dynamic, 64)
    for (int64_t row = 0; row < n_dst; ++row) {
        float *o = out + row * F;
        for (int f = 0; f < F; ++f) o[f] = 0.0f;
        for (int32_t e = indptr[row]; e < indptr[row + 1]; ++e) {
            const float w = vals[e];
            const float *xr = x + (int64_t)indices[e] * F;
            for (int f = 0; f < F; ++f) o[f] += w * xr[f];
        }
    }
    return ORC_OK;
}

/*
 * Generalised aggregation.  NOT IN THE REFERENCE (parity unpinned, see the header):
 *   out[v, h, d] = reduce over the row's elements e of w(e, h) * X[indices[e], h, d]
 * reduce: 0 sum, 1 max, 2 min; w(e, h) = vals[e * H + h], or 1 when vals is NULL; a row without
 * elements gives 0 for every reduce.  Elements are visited in stored order.
 */
int orc_gspmm(int64_t n_dst, int F, int H, const int32_t *indptr, const int32_t *indices,
              const float *vals, const float *x, float *out, int reduce, int nthreads) {
    if (F < 1 || H < 1 || F % H != 0 || reduce < 0 || reduce > 2 || nthreads < 1) return ORC_EARG;
    const int D = F / H;
#pragma omp parallel for num_threads(nthreads) schedule(dynamic, 64)
    for (int64_t row = 0; row < n_dst; ++row) {
        float *o = out + row * F;
        const int32_t b = indptr[row], e = indptr[row + 1];
        for (int f = 0; f < F; ++f) o[f] = 0.0f;
        for (int32_t k = b; k < e; ++k) {
            const float *xr = x + (int64_t)indices[k] * F;
            for (int f = 0; f < F; ++f) {
                const float w = vals ? vals[(int64_t)k * H + f / D] : 1.0f;
                const float m = w * xr[f];
                /* max / min: a NaN message beats every number and stays (numpy's maximum / minimum reductions) */
                if (reduce == 0) o[f] += m;
                else if (k == b) o[f] = m;
                else if (o[f] == o[f] && ((reduce == 1 ? m > o[f] : m < o[f]) || m != m)) o[f] = m;
            }
        }
    }
    return ORC_OK;
}

/*
 * orc_gspmm for max (reduce 1) / min (reduce 2) that also reports the selected element.  NOT IN THE
 * REFERENCE (parity unpinned, see the header): arg[v, f] = stored position of the first element of
 * row v whose message equals the extreme, -1 for a row without elements.  Pinned by numpy argmax /
 * argmin over the gathered messages (first occurrence on ties).
 */
int orc_gspmm_arg(int64_t n_dst, int F, int H, const int32_t *indptr, const int32_t *indices,
                  const float *vals, const float *x, float *out, int32_t *arg, int reduce, int nthreads) {
    if (F < 1 || H < 1 || F % H != 0 || reduce < 1 || reduce > 2 || nthreads < 1) return ORC_EARG;
    const int D = F / H;
#pragma omp parallel for num_threads(nthreads) schedule(dynamic, 64)
    for (int64_t row = 0; row < n_dst; ++row) {
        float *o = out + row * F;
        int32_t *a = arg + row * F;
        const int32_t b = indptr[row], e = indptr[row + 1];
        for (int f = 0; f < F; ++f) { o[f] = 0.0f; a[f] = -1; }
        for (int32_t k = b; k < e; ++k) {
            const float *xr = x + (int64_t)indices[k] * F;
            for (int f = 0; f < F; ++f) {
                const float w = vals ? vals[(int64_t)k * H + f / D] : 1.0f;
                const float m = w * xr[f];
                /* the first NaN message, if there is one, is the selected element (numpy's argmax / argmin) */
                if (k == b || (o[f] == o[f] && ((reduce == 1 ? m > o[f] : m < o[f]) || m != m))) { o[f] = m; a[f] = k; }
            }
        }
    }
    return ORC_OK;
}

/*
 * Softmax over each row's stored elements, separately per head.  NOT IN THE REFERENCE (parity
 * unpinned, see the header):
 *   out[e, h] = exp(x[e, h] - m[v, h]) / sum over the row's e' of exp(x[e', h] - m[v, h]),
 *   m[v, h] = max over the row's elements, v = the row of e.
 * Elements are visited in stored order; a row without elements writes nothing.
 */
int orc_edge_softmax(int64_t n_rows, int H, const int32_t *indptr, const float *x, float *out,
                     int nthreads) {
    if (H < 1 || nthreads < 1) return ORC_EARG;
#pragma omp parallel for num_threads(nthreads) schedule(dynamic, 64)
    for (int64_t row = 0; row < n_rows; ++row) {
        const int64_t b = indptr[row], e = indptr[row + 1];
        for (int h = 0; h < H; ++h) {
            if (e <= b) continue;
            float m = x[b * H + h];
            for (int64_t k = b + 1; k < e; ++k) m = x[k * H + h] > m ? x[k * H + h] : m;
            float s = 0.0f;
            for (int64_t k = b; k < e; ++k) s += expf(x[k * H + h] - m);
            for (int64_t k = b; k < e; ++k) out[k * H + h] = expf(x[k * H + h] - m) / s;
        }
    }
    return ORC_OK;
}

/*
 * Gradient of orc_edge_softmax with respect to x, given a = its output and g = dL/da:
 *   dx[e, h] = a[e, h] * (g[e, h] - sum over the row's e' of a[e', h] * g[e', h]).
 */
int orc_edge_softmax_backward(int64_t n_rows, int H, const int32_t *indptr, const float *a,
                              const float *g, float *dx, int nthreads) {
    if (H < 1 || nthreads < 1) return ORC_EARG;
#pragma omp parallel for num_threads(nthreads) schedule(dynamic, 64)
    for (int64_t row = 0; row < n_rows; ++row) {
        const int64_t b = indptr[row], e = indptr[row + 1];
        for (int h = 0; h < H; ++h) {
            float d = 0.0f;
            for (int64_t k = b; k < e; ++k) d += a[k * H + h] * g[k * H + h];
            for (int64_t k = b; k < e; ++k) dx[k * H + h] = a[k * H + h] * (g[k * H + h] - d);
        }
    }
    return ORC_OK;
}

/*
 * Feature-tiled, source-column-partitioned SpMM on x86 over the DDS format:
 * compute python/featgraph/op/vanilla_spmm.py:149-224, schedule :227-246.
 * Loop order fo -> p -> row (parallel) -> elem -> fi.  Intermediate[fo,p,row,:]
 * is a fresh sequential sum over partition p's elements of the row (:201-213),
 * and ReshapedOut[fo,row,:] is the running sum of the Intermediates in
 * ascending p (:215-218, Intermediate computed at the p loop, :238).
 * s1_idx holds partition-local column ids; the global one adds
 * p * ceil(n_src / P) (:196, :209-210).
 */
int orc_spmm_dds_x86(int64_t n_dst, int64_t n_src, int F, int P, const int32_t *s1_pos,
                     const int32_t *s1_idx, const float *vals, const float *x, float *out,
                     int num_feat_partitions, int nthreads) {
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
        for (int64_t i = 0; i < n_dst * Fp; ++i) rof[i] = 0.0f;
        for (int p = 0; p < P; ++p) {
            const int32_t *pos = s1_pos + (int64_t)p * d2;
            const int64_t col0 = (int64_t)p * cols_per_part;
#pragma omp parallel for num_threads(nthreads) schedule(dynamic, 64)
            for (int64_t row = 0; row < n_dst; ++row) {
                float inter[Fp];
                for (int fi = 0; fi < Fp; ++fi) inter[fi] = 0.0f;
                for (int32_t e = pos[row]; e < pos[row + 1]; ++e) {
                    const float w = vals[e];
                    const float *xr = rxf + ((int64_t)s1_idx[e] + col0) * Fp;
                    for (int fi = 0; fi < Fp; ++fi) inter[fi] += w * xr[fi];
                }
                float *o = rof + row * Fp;
                for (int fi = 0; fi < Fp; ++fi) o[fi] += inter[fi];
            }
        }
    }
    relayout_out(ro, out, n_dst, F, T, nthreads);
    free(rx); free(ro);
    return ORC_OK;
}

/*
 * Edge-wise dot product on x86: compute python/featgraph/op/vanilla_sddmm.py:6-63,
 * schedule :66-74.  Out[e] = sum_k Src[col[e], k] * Dst[row[e], k]: Src is
 * indexed by the COLUMN index and Dst by the ROW index (:47; the reference's
 * tests size Src as (num_cols, F) and Dst as (num_rows, F),
 * tests/test_module_sddmm.py:18-19).  With T > 1 both operands are re-laid
 * [T, n, Fp] (:52-57) and the loop order is fo -> edge -> fi (:71-72); k stays
 * ascending per edge, so the rounding equals T == 1.  The reference schedule
 * has no parallel axis (:11, :66-74): parallel_edges == 0 is that serial
 * schedule; parallel_edges != 0 is a labelled variant that splits the edge
 * loop over threads and changes no per-edge arithmetic.
 */
int orc_sddmm_x86(int64_t n_edges, int64_t n_src_rows, int64_t n_dst_rows, int F,
                  const int32_t *row, const int32_t *col, const float *src,
                  const float *dst, float *out, int num_feat_partitions,
                  int parallel_edges, int nthreads) {
    const int T = num_feat_partitions;
    if (T < 1 || F < 1 || F % T != 0 || nthreads < 1) return ORC_EARG;
    const int nt = parallel_edges ? nthreads : 1;
    if (T == 1) {
#pragma omp parallel for num_threads(nt) schedule(static) if (nt > 1)
        for (int64_t e = 0; e < n_edges; ++e) {
            const float *s = src + (int64_t)col[e] * F;
            const float *d = dst + (int64_t)row[e] * F;
            float acc = 0.0f;
            for (int k = 0; k < F; ++k) acc += s[k] * d[k];
            out[e] = acc;
        }
        return ORC_OK;
    }
    const int Fp = F / T;
    float *rs = (float *)malloc(sizeof(float) * (size_t)(n_src_rows ? n_src_rows : 1) * F);
    float *rd = (float *)malloc(sizeof(float) * (size_t)(n_dst_rows ? n_dst_rows : 1) * F);
    if (!rs || !rd) { free(rs); free(rd); return ORC_ENOMEM; }
    relayout_in(src, rs, n_src_rows, F, T, 1);
    relayout_in(dst, rd, n_dst_rows, F, T, 1);
    for (int64_t e = 0; e < n_edges; ++e) out[e] = 0.0f;
    for (int fo = 0; fo < T; ++fo) {
        const float *rsf = rs + (int64_t)fo * n_src_rows * Fp;
        const float *rdf = rd + (int64_t)fo * n_dst_rows * Fp;
#pragma omp parallel for num_threads(nt) schedule(static) if (nt > 1)
        for (int64_t e = 0; e < n_edges; ++e) {
            const float *s = rsf + (int64_t)col[e] * Fp;
            const float *d = rdf + (int64_t)row[e] * Fp;
            float acc = out[e];
            for (int fi = 0; fi < Fp; ++fi) acc += s[fi] * d[fi];
            out[e] = acc;
        }
    }
    free(rs); free(rd);
    return ORC_OK;
}

/*
 * Multi-head edge-wise dot product.  NOT IN THE REFERENCE (parity unpinned, see
 * the header): Out[e, h] = sum_{d<D} Src[col[e], h, d] * Dst[row[e], h, d] with
 * Src/Dst contiguous [n, H, D] and Out row-major [E, H].  Same operand/index
 * pairing as orc_sddmm_x86 (python/featgraph/op/vanilla_sddmm.py:47), so H == 1
 * is that function.
 */
int orc_sddmm_multihead(int64_t n_edges, int H, int D, const int32_t *row,
                        const int32_t *col, const float *src, const float *dst,
                        float *out, int nthreads) {
    if (H < 1 || D < 1 || nthreads < 1) return ORC_EARG;
    const int64_t F = (int64_t)H * D;
#pragma omp parallel for num_threads(nthreads) schedule(static) if (nthreads > 1)
    for (int64_t e = 0; e < n_edges; ++e) {
        const float *s = src + (int64_t)col[e] * F;
        const float *d = dst + (int64_t)row[e] * F;
        for (int h = 0; h < H; ++h) {
            float acc = 0.0f;
            for (int k = 0; k < D; ++k) acc += s[h * D + k] * d[h * D + k];
            out[e * H + h] = acc;
        }
    }
    return ORC_OK;
}

/*
 * CSR -> DDS (1-D source-column partitioning):
 * python/featgraph/util/adj_partitioning.py:29-57.  For partition p the
 * reference column-slices the CSR to [p*c, (p+1)*c), c = ceil(n_cols / P)
 * (:42), the last slice open-ended (:44-47), and appends the slice's data to
 * vals, its slice-local indices to s1_idx and its indptr plus the running
 * element count to s1_pos[p*d2 : (p+1)*d2] (:48-52).  A column slice keeps a
 * row's stored element order.  Values are moved as opaque 32-bit words, so
 * int32 edge ids (the reference's test data) and float32 weights both work.
 */
int orc_csr_to_dds(int64_t n_rows, int64_t n_cols, const int32_t *indptr,
                   const int32_t *indices, const uint32_t *data, int P,
                   int32_t *s1_pos, int32_t *s1_idx, uint32_t *vals) {
    if (P < 1) return ORC_EARG;
    const int64_t d2 = n_rows + 1;
    const int64_t c = (n_cols + P - 1) / P;
    int64_t counter = 0;
    for (int p = 0; p < P; ++p) {
        const int64_t lo = (int64_t)p * c;
        const int64_t hi = (p == P - 1) ? n_cols : (int64_t)(p + 1) * c;
        int32_t *pos = s1_pos + (int64_t)p * d2;
        pos[0] = (int32_t)counter;
        for (int64_t r = 0; r < n_rows; ++r) {
            for (int32_t e = indptr[r]; e < indptr[r + 1]; ++e) {
                const int64_t cidx = indices[e];
                if (cidx >= lo && cidx < hi) {
                    s1_idx[counter] = (int32_t)(cidx - lo);
                    vals[counter] = data[e];
                    ++counter;
                }
            }
            pos[r + 1] = (int32_t)counter;
        }
    }
    return counter == indptr[n_rows] ? ORC_OK : ORC_EARG;
}

typedef struct { int32_t r, c, id; } orc_edge;

static int edge_cmp(const void *a, const void *b) {
    const orc_edge *x = (const orc_edge *)a, *y = (const orc_edge *)b;
    if (x->r != y->r) return x->r < y->r ? -1 : 1;
    if (x->c != y->c) return x->c < y->c ? -1 : 1;
    return 0;
}

/*
 * 2-D COO partitioning: python/featgraph/util/adj_partitioning.py:85-128.
 * Edges get ids 1..nnz in stored COO order (:92); the matrix is converted to
 * CSR (:95), which orders each row's entries by column; blocks are visited in
 * row-major block order (:103-104) with R' = ceil(rows / R), C' = ceil(cols / C)
 * (:100-101) and open-ended last blocks; each block is emitted in row-major,
 * column-ascending order with global row/col ids (:119-126).
 * Duplicate (row, col) pairs make the reference's CSR conversion add edge ids
 * together; that input is rejected here (ORC_EDUP).
 */
int orc_partition_coo_2d(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *row,
                         const int32_t *col, int R, int C, int32_t *edge_id,
                         int32_t *out_row, int32_t *out_col) {
    if (R < 1 || C < 1) return ORC_EARG;
    orc_edge *ed = (orc_edge *)malloc(sizeof(orc_edge) * (size_t)(nnz ? nnz : 1));
    int64_t *rowptr = (int64_t *)calloc((size_t)n_rows + 1, sizeof(int64_t));
    if (!ed || !rowptr) { free(ed); free(rowptr); return ORC_ENOMEM; }
    for (int64_t e = 0; e < nnz; ++e) {
        ed[e].r = row[e]; ed[e].c = col[e]; ed[e].id = (int32_t)(e + 1);
        rowptr[row[e] + 1]++;
    }
    qsort(ed, (size_t)nnz, sizeof(orc_edge), edge_cmp);
    for (int64_t e = 1; e < nnz; ++e)
        if (ed[e].r == ed[e - 1].r && ed[e].c == ed[e - 1].c) { free(ed); free(rowptr); return ORC_EDUP; }
    for (int64_t r = 0; r < n_rows; ++r) rowptr[r + 1] += rowptr[r];
    const int64_t rp = (n_rows + R - 1) / R, cp = (n_cols + C - 1) / C;
    int64_t counter = 0;
    for (int rb = 0; rb < R; ++rb) {
        const int64_t r0 = (int64_t)rb * rp;
        const int64_t r1 = (rb == R - 1) ? n_rows : (int64_t)(rb + 1) * rp;
        for (int cb = 0; cb < C; ++cb) {
            const int64_t c0 = (int64_t)cb * cp;
            const int64_t c1 = (cb == C - 1) ? n_cols : (int64_t)(cb + 1) * cp;
            for (int64_t r = r0; r < r1 && r < n_rows; ++r)
                for (int64_t k = rowptr[r]; k < rowptr[r + 1]; ++k)
                    if (ed[k].c >= c0 && ed[k].c < c1) {
                        edge_id[counter] = ed[k].id;
                        out_row[counter] = ed[k].r;
                        out_col[counter] = ed[k].c;
                        ++counter;
                    }
        }
    }
    free(ed); free(rowptr);
    return counter == nnz ? ORC_OK : ORC_EARG;
}
