// Host-side parts of libfeatgraph_hip.so: error reporting, graph partitioners, structural
// checks and the seeded synthetic-graph generator.  No device code in this file.
#include <algorithm>
#include <atomic>
#include <cstring>
#include <numeric>
#include <thread>

#include "fg_common.h"

namespace fg {

static thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

// Runs fn(t, begin, end) over [0, n) cut into `nt` contiguous ranges on `nt` threads.
template <class Fn>
static void parallel_ranges(int64_t n, int nt, Fn fn) {
    nt = (int)std::max<int64_t>(1, std::min<int64_t>(nt, n));
    if (nt == 1) { fn(0, (int64_t)0, n); return; }
    std::vector<std::thread> th;
    for (int t = 0; t < nt; ++t)
        th.emplace_back([=] { fn(t, n * t / nt, n * (t + 1) / nt); });
    for (auto &x : th) x.join();
}

static int default_threads() {
    unsigned hc = std::thread::hardware_concurrency();
    return (int)std::max(1u, std::min(hc, 16u));
}

}  // namespace fg

using fg::fail;

extern "C" int fg_version(void) { return 100; }
extern "C" const char *fg_last_error(void) { return fg::g_err; }

extern "C" int fg_check_csr_host(int64_t n_rows, int64_t n_cols, const int32_t *indptr,
                                 const int32_t *indices) {
    if (!indptr || n_rows < 0 || n_cols < 0) return fail(FG_ERR_ARG, "fg_check_csr_host: bad argument");
    if (indptr[0] != 0) return fail(FG_ERR_GRAPH, "indptr[0] = %d, expected 0", indptr[0]);
    for (int64_t r = 0; r < n_rows; ++r)
        if (indptr[r + 1] < indptr[r])
            return fail(FG_ERR_GRAPH, "indptr decreases at row %lld", (long long)r);
    const int64_t nnz = indptr[n_rows];
    if (nnz > 0 && !indices) return fail(FG_ERR_ARG, "fg_check_csr_host: indices is null");
    for (int64_t e = 0; e < nnz; ++e)
        if (indices[e] < 0 || indices[e] >= n_cols)
            return fail(FG_ERR_GRAPH, "indices[%lld] = %d outside [0, %lld)", (long long)e,
                        indices[e], (long long)n_cols);
    return FG_OK;
}

// One pass counts each (partition, row) cell, a prefix sum over cells in partition-major
// order gives s1_pos, a second pass scatters.  O(nnz + P * n_rows); a row's elements keep
// their stored order inside each partition, which is what a column slice of the row gives.
extern "C" int fg_csr_to_dds(int64_t n_rows, int64_t n_cols, const int32_t *indptr,
                             const int32_t *indices, const void *data32, int P,
                             int32_t *s1_pos, int32_t *s1_idx, void *vals32) {
    if (P < 1) return fail(FG_ERR_ARG, "num_col_partitions should be larger than or equal to 1");
    if (!indptr || !s1_pos || n_rows < 0 || n_cols < 0) return fail(FG_ERR_ARG, "fg_csr_to_dds: bad argument");
    const int64_t nnz = indptr[n_rows];
    if (nnz > 0 && (!indices || !data32 || !s1_idx || !vals32)) return fail(FG_ERR_ARG, "fg_csr_to_dds: null array");
    const uint32_t *data = static_cast<const uint32_t *>(data32);
    uint32_t *vals = static_cast<uint32_t *>(vals32);
    const int64_t d2 = n_rows + 1;
    const int64_t width = (n_cols + P - 1) / P;          // columns per partition
    if (n_cols >= INT32_MAX) return fail(FG_ERR_SHAPE, "fg_csr_to_dds: column count does not fit int32");
    const uint32_t w32 = (uint32_t)std::max<int64_t>(width, 1);
    auto part_of = [&](int32_t c) { return (int64_t)((uint32_t)c / w32); };
    const int nt = fg::default_threads();

    // cursor[p*d2 + r] = number of elements of row r in partition p, then their offsets.  Rows are
    // independent in both passes (a cell belongs to one row), so they run over row ranges in parallel.
    std::vector<int64_t> cursor((size_t)P * d2, 0);
    std::vector<int64_t> bad_at((size_t)nt, -1);
    fg::parallel_ranges(n_rows, nt, [&](int t, int64_t r0, int64_t r1) {
        for (int64_t r = r0; r < r1; ++r)
            for (int32_t e = indptr[r]; e < indptr[r + 1]; ++e) {
                const int32_t c = indices[e];
                if (c < 0 || c >= n_cols) { if (bad_at[t] < 0) bad_at[t] = e; continue; }
                cursor[part_of(c) * d2 + r]++;
            }
    });
    for (int64_t e : bad_at)
        if (e >= 0) return fail(FG_ERR_GRAPH, "indices[%lld] = %d outside [0, %lld)", (long long)e, indices[e], (long long)n_cols);
    int64_t run = 0;
    for (int p = 0; p < P; ++p) {
        for (int64_t r = 0; r < n_rows; ++r) {
            const int64_t cnt = cursor[p * d2 + r];
            s1_pos[p * d2 + r] = (int32_t)run;
            cursor[p * d2 + r] = run;
            run += cnt;
        }
        s1_pos[p * d2 + n_rows] = (int32_t)run;
    }
    fg::parallel_ranges(n_rows, nt, [&](int, int64_t r0, int64_t r1) {
        for (int64_t r = r0; r < r1; ++r)
            for (int32_t e = indptr[r]; e < indptr[r + 1]; ++e) {
                const int32_t c = indices[e];
                const int64_t p = part_of(c);
                const int64_t at = cursor[p * d2 + r]++;
                s1_idx[at] = (int32_t)(c - p * width);
                vals[at] = data[e];
            }
    });
    return FG_OK;
}

// Traversal order = sort by (row block, col block, row, col).  Edges are bucketed by row with
// a counting sort, each row is sorted by column, then a stable counting sort by block id
// keeps that (row, col) order inside every block.  O(nnz log(deg) + R*C).
extern "C" int fg_partition_coo_2d(int64_t n_rows, int64_t n_cols, int64_t nnz,
                                   const int32_t *row, const int32_t *col, int R, int C,
                                   int32_t *edge_id, int32_t *out_row, int32_t *out_col) {
    if (R < 1) return fail(FG_ERR_ARG, "num_row_partitions should be larger than or equal to 1");
    if (C < 1) return fail(FG_ERR_ARG, "num_col_partitions should be larger than or equal to 1");
    if (n_rows < 0 || n_cols < 0 || nnz < 0) return fail(FG_ERR_ARG, "fg_partition_coo_2d: negative size");
    if (nnz == 0) return FG_OK;
    if (!row || !col || !edge_id || !out_row || !out_col) return fail(FG_ERR_ARG, "fg_partition_coo_2d: null array");
    if (nnz >= INT32_MAX) return fail(FG_ERR_SHAPE, "fg_partition_coo_2d: nnz does not fit int32 edge ids");
    const int nt = fg::default_threads();

    std::vector<int64_t> rowptr((size_t)n_rows + 1, 0);
    for (int64_t e = 0; e < nnz; ++e) {
        if (row[e] < 0 || row[e] >= n_rows || col[e] < 0 || col[e] >= n_cols)
            return fail(FG_ERR_GRAPH, "edge %lld = (%d, %d) outside the %lld x %lld matrix",
                        (long long)e, row[e], col[e], (long long)n_rows, (long long)n_cols);
        rowptr[row[e] + 1]++;
    }
    for (int64_t r = 0; r < n_rows; ++r) rowptr[r + 1] += rowptr[r];
    // (col, id) pairs grouped by row
    std::vector<uint64_t> byrow((size_t)nnz);
    {
        std::vector<int64_t> cur(rowptr.begin(), rowptr.end() - 1);
        for (int64_t e = 0; e < nnz; ++e)
            byrow[cur[row[e]]++] = ((uint64_t)(uint32_t)col[e] << 32) | (uint32_t)(e + 1);
    }
    std::atomic<bool> dup{false};     // set by any worker thread
    fg::parallel_ranges(n_rows, nt, [&](int, int64_t r0, int64_t r1) {
        for (int64_t r = r0; r < r1; ++r) {
            std::sort(byrow.begin() + rowptr[r], byrow.begin() + rowptr[r + 1]);
            for (int64_t k = rowptr[r] + 1; k < rowptr[r + 1]; ++k)
                if ((byrow[k] >> 32) == (byrow[k - 1] >> 32)) dup.store(true, std::memory_order_relaxed);
        }
    });
    if (dup.load()) return fail(FG_ERR_GRAPH, "duplicate (row, col) pairs: edge ids would be ambiguous");

    const int64_t rp = (n_rows + R - 1) / R, cp = (n_cols + C - 1) / C;
    const int64_t n_blocks = (int64_t)R * C;
    std::vector<int64_t> boff((size_t)n_blocks + 1, 0);
    for (int64_t r = 0; r < n_rows; ++r) {
        const int64_t rb = r / rp;
        for (int64_t k = rowptr[r]; k < rowptr[r + 1]; ++k)
            boff[rb * C + (int64_t)(byrow[k] >> 32) / cp + 1]++;
    }
    for (int64_t b = 0; b < n_blocks; ++b) boff[b + 1] += boff[b];
    for (int64_t r = 0; r < n_rows; ++r) {
        const int64_t rb = r / rp;
        for (int64_t k = rowptr[r]; k < rowptr[r + 1]; ++k) {
            const int32_t c = (int32_t)(byrow[k] >> 32);
            const int64_t at = boff[rb * C + c / cp]++;
            edge_id[at] = (int32_t)(byrow[k] & 0xffffffffu);
            out_row[at] = (int32_t)r;
            out_col[at] = c;
        }
    }
    return FG_OK;
}

// ---- synthetic power-law graph ------------------------------------------------------------

namespace {

inline uint64_t mix64(uint64_t z) {          // splitmix64 finaliser
    z += 0x9e3779b97f4a7c15ull;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

// Sources of row v: in_degree draws through the inverse CDF, keyed by (seed, v, k) only.
void draw_row(int64_t v, int64_t n, int32_t deg, const double *cdf, const int32_t *perm,
              uint64_t seed, std::vector<int32_t> &buf) {
    buf.clear();
    buf.push_back((int32_t)v);                               // self-loop
    const uint64_t key = mix64(seed ^ mix64((uint64_t)v));
    for (int32_t k = 0; k < deg; ++k) {
        const uint64_t bits = mix64(key + (uint64_t)k * 0xd1342543de82ef95ull);
        const double u = (double)(bits >> 11) * (1.0 / 9007199254740992.0);   // [0, 1)
        int64_t rank = std::upper_bound(cdf, cdf + n, u) - cdf;
        if (rank >= n) rank = n - 1;
        buf.push_back(perm[rank]);
    }
    std::sort(buf.begin(), buf.end());
    buf.erase(std::unique(buf.begin(), buf.end()), buf.end());
}

// The same with planted communities: each draw stays inside the row's own community with probability p_in (its
// sources then come from that community's own distribution) and is a draw from the whole graph otherwise.
struct Communities {
    const int32_t *of_vertex;   // [n]
    const int64_t *off;         // [n_comm + 1] into member / cdf
    const int32_t *member;      // vertex ids, community by community
    const double *cdf;          // per community, non-decreasing, last element 1
    double p_in;
};

void draw_row_communities(int64_t v, int64_t n, int32_t deg, const double *cdf, const int32_t *perm, const Communities &cm,
                          uint64_t seed, std::vector<int32_t> &buf) {
    buf.clear();
    buf.push_back((int32_t)v);                               // self-loop
    const uint64_t key = mix64(seed ^ mix64((uint64_t)v));
    const int32_t c = cm.of_vertex[v];
    const double *ccdf = cm.cdf + cm.off[c];
    const int64_t csize = cm.off[c + 1] - cm.off[c];
    // a row that asks for more than half of its community keeps that many draws inside and takes the rest from the
    // whole graph (a hub's neighbours are not confined to its community, and repeated draws would merge)
    const double p_in = (double)deg * 2.0 <= (double)csize ? cm.p_in : cm.p_in * ((double)csize / 2.0) / (double)deg;
    for (int32_t k = 0; k < deg; ++k) {
        const uint64_t bits = mix64(key + (uint64_t)k * 0xd1342543de82ef95ull);
        const double u = (double)(bits >> 11) * (1.0 / 9007199254740992.0);   // [0, 1)
        const uint64_t bits2 = mix64(bits ^ 0xa0761d6478bd642full);
        const double where = (double)(bits2 >> 11) * (1.0 / 9007199254740992.0);
        if (where < p_in && csize > 0) {
            int64_t at = std::upper_bound(ccdf, ccdf + csize, u) - ccdf;
            if (at >= csize) at = csize - 1;
            buf.push_back(cm.member[cm.off[c] + at]);
        } else {
            int64_t rank = std::upper_bound(cdf, cdf + n, u) - cdf;
            if (rank >= n) rank = n - 1;
            buf.push_back(perm[rank]);
        }
    }
    std::sort(buf.begin(), buf.end());
    buf.erase(std::unique(buf.begin(), buf.end()), buf.end());
}

template <typename Draw>
int synth_csr(int64_t n, int num_threads, int32_t *indptr, int32_t *indices, const char *what, Draw draw) {
    const int nt = num_threads > 0 ? num_threads : fg::default_threads();
    if (!indices) {
        // first call: row lengths only
        fg::parallel_ranges(n, nt, [&](int, int64_t v0, int64_t v1) {
            std::vector<int32_t> buf;
            for (int64_t v = v0; v < v1; ++v) {
                draw(v, buf);
                indptr[v + 1] = (int32_t)buf.size();
            }
        });
        int64_t run = 0;
        indptr[0] = 0;
        for (int64_t v = 0; v < n; ++v) {
            run += indptr[v + 1];
            if (run >= INT32_MAX) return fail(FG_ERR_SHAPE, "graph has more than 2^31-1 edges");
            indptr[v + 1] = (int32_t)run;
        }
        return FG_OK;
    }
    std::atomic<bool> bad{false};     // set by any worker thread
    fg::parallel_ranges(n, nt, [&](int, int64_t v0, int64_t v1) {
        std::vector<int32_t> buf;
        for (int64_t v = v0; v < v1; ++v) {
            draw(v, buf);
            if ((int64_t)buf.size() != indptr[v + 1] - indptr[v]) { bad.store(true, std::memory_order_relaxed); continue; }
            std::copy(buf.begin(), buf.end(), indices + indptr[v]);
        }
    });
    if (bad.load()) return fail(FG_ERR_ARG, "%s: indptr does not match this seed", what);
    return FG_OK;
}

}  // namespace

extern "C" int fg_synth_community_csr(int64_t n, const int32_t *in_degree, const double *cdf, const int32_t *perm,
                                      int n_comm, const int32_t *comm_of_vertex, const int64_t *comm_off,
                                      const int32_t *comm_member, const double *comm_cdf, double p_in, uint64_t seed,
                                      int num_threads, int32_t *indptr, int32_t *indices) {
    if (n < 1 || !in_degree || !cdf || !perm || !indptr || n_comm < 1 || !comm_of_vertex || !comm_off || !comm_member ||
        !comm_cdf || !(p_in >= 0.0 && p_in <= 1.0))
        return fail(FG_ERR_ARG, "fg_synth_community_csr: bad argument");
    if (comm_off[0] != 0 || comm_off[n_comm] != n) return fail(FG_ERR_ARG, "fg_synth_community_csr: communities must cover the n vertices");
    for (int64_t v = 0; v < n; ++v)
        if (comm_of_vertex[v] < 0 || comm_of_vertex[v] >= n_comm) return fail(FG_ERR_ARG, "fg_synth_community_csr: community id out of range");
    for (int64_t i = 0; i < n; ++i)
        if (comm_member[i] < 0 || comm_member[i] >= n) return fail(FG_ERR_ARG, "fg_synth_community_csr: member id out of range");
    const Communities cm{comm_of_vertex, comm_off, comm_member, comm_cdf, p_in};
    return synth_csr(n, num_threads, indptr, indices, "fg_synth_community_csr", [&](int64_t v, std::vector<int32_t> &buf) {
        draw_row_communities(v, n, in_degree[v], cdf, perm, cm, seed, buf);
    });
}

extern "C" int fg_synth_powerlaw_csr(int64_t n, const int32_t *in_degree, const double *cdf,
                                     const int32_t *perm, uint64_t seed, int num_threads,
                                     int32_t *indptr, int32_t *indices) {
    if (n < 1 || !in_degree || !cdf || !perm || !indptr)
        return fail(FG_ERR_ARG, "fg_synth_powerlaw_csr: bad argument");
    return synth_csr(n, num_threads, indptr, indices, "fg_synth_powerlaw_csr", [&](int64_t v, std::vector<int32_t> &buf) {
        draw_row(v, n, in_degree[v], cdf, perm, seed, buf);
    });
}
