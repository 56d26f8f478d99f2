// Load-balance plan of one adjacency: the list of per-wavefront work items that both the
// SpMM kernels and the CSR-order SDDMM kernel walk.  Built on the host from the position
// array, kept on the device.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstring>
#include <string>

#include "fg_common.h"

using fg::fail;
using fg::Fixup;
using fg::Item;

namespace {
constexpr int kDefaultSplit = 1024;   // elements per wavefront piece of a long row
}

extern "C" int fg_spmm_plan_create(const int32_t *pos, int64_t n_dst, int64_t n_src, int P,
                                   const fg_plan_opts *opts, fg_spmm_plan **plan_out) {
    if (!plan_out) return fail(FG_ERR_ARG, "fg_spmm_plan_create: plan_out is null");
    *plan_out = nullptr;
    if (!pos || n_dst < 0 || n_src < 0) return fail(FG_ERR_ARG, "fg_spmm_plan_create: bad argument");
    if (P < 1) return fail(FG_ERR_ARG, "num_col_partitions should be larger than or equal to 1");
    if (n_dst >= INT32_MAX || n_src >= INT32_MAX) return fail(FG_ERR_SHAPE, "vertex count does not fit int32");
    int split = (opts && opts->split_threshold > 0) ? opts->split_threshold : kDefaultSplit;
    int item_edges = (opts && opts->item_edges > 0) ? opts->item_edges : fg::kItemEdges;
    if (item_edges > fg::kItemEdges) item_edges = fg::kItemEdges;
    if (item_edges > split) item_edges = split;
    const int64_t d2 = n_dst + 1;

    // structure check: one non-decreasing run of positions across all partitions
    int64_t prev = 0;
    for (int p = 0; p < P; ++p)
        for (int64_t r = 0; r <= n_dst; ++r) {
            const int64_t v = pos[p * d2 + r];
            if ((p == 0 && r == 0 && v != 0) || v < prev || (r == 0 && v != prev))
                return fail(FG_ERR_GRAPH, "position array is not a monotone run at partition %d row %lld",
                            p, (long long)r);
            prev = v;
        }

    auto *pl = new fg_spmm_plan();
    pl->n_dst = n_dst; pl->n_src = n_src; pl->nnz = prev;
    pl->num_col_partitions = P; pl->split_threshold = split; pl->item_edges = item_edges;
    pl->wide_offsets = opts && opts->wide_offsets != 0;
    pl->tile_major = opts ? opts->tile_major : 0;
    pl->pass_buffers = opts ? opts->pass_buffers : 0;
    std::vector<Item> items;
    std::vector<Fixup> fixups;
    items.reserve((size_t)(n_dst + n_dst / 8 + 16));
    pl->item_off.push_back(0);
    pl->fixup_off.push_back(0);
    for (int p = 0; p < P; ++p) {
        int32_t slot = 0;
        const int32_t *pp = pos + p * d2;
        int64_t r = 0;
        while (r < n_dst) {
            const int32_t start = pp[r];
            const int32_t len = pp[r + 1] - start;
            pl->max_len = std::max<int64_t>(pl->max_len, len);
            if (len > split) {
                const int32_t pieces = (len + split - 1) / split;
                // equal pieces, rounded up to whole 64-element staging rounds
                const int32_t piece_len = (((len + pieces - 1) / pieces) + 63) / 64 * 64;
                int32_t made = 0;
                for (int32_t s = 0; s < len; s += piece_len, ++made)
                    items.push_back({start + s, std::min(piece_len, len - s), (int32_t)r, slot + made});
                fixups.push_back({(int32_t)r, slot, made, (int32_t)p});
                slot += made;
                pl->n_split_rows++;
                ++r;
                continue;
            }
            if (len > item_edges) {            // one whole row, too long to share an item
                items.push_back({start, len, (int32_t)r, -1});
                ++r;
                continue;
            }
            // a run of short rows: at most item_edges elements and kItemRows rows
            const int64_t r0 = r;
            int32_t total = 0;
            while (r < n_dst && r - r0 < fg::kItemRows) {
                const int32_t l = pp[r + 1] - pp[r];
                if (l > item_edges || total + l > item_edges) break;
                if (l == 0 && p == 0) pl->n_empty++;
                pl->max_len = std::max<int64_t>(pl->max_len, l);
                total += l;
                ++r;
            }
            if (r == r0) {                      // item_edges < 1 row: cannot happen, len <= item_edges
                items.push_back({start, len, (int32_t)r, -1});
                ++r;
                continue;
            }
            // (runs of empty segments keep their item in later partitions too: a pass that writes a buffer
            // of its own must write every row of it, and a pass that adds in place skips them in the kernel)
            items.push_back({start, total, (int32_t)r0, -(int32_t)(r - r0)});
            if (r - r0 > 1) pl->n_multi_items++;
        }
        pl->item_off.push_back((int64_t)items.size());
        pl->fixup_off.push_back((int64_t)fixups.size());
        pl->n_slots += slot;
        pl->max_slots_in_partition = std::max<int64_t>(pl->max_slots_in_partition, slot);
    }
    pl->n_items = (int64_t)items.size();
    pl->n_fixups = (int64_t)fixups.size();

    hipError_t e = hipGetDevice(&pl->device);
    if (e == hipSuccess && P == 1) fg::prepare_fixed_scratch(pl->device);
    if (e == hipSuccess && pl->n_items) e = hipMalloc((void **)&pl->items_dev, sizeof(Item) * items.size());
    if (e == hipSuccess && pl->n_items)
        e = hipMemcpy(pl->items_dev, items.data(), sizeof(Item) * items.size(), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMalloc((void **)&pl->item_off_dev, sizeof(int64_t) * pl->item_off.size());
    if (e == hipSuccess)
        e = hipMemcpy(pl->item_off_dev, pl->item_off.data(), sizeof(int64_t) * pl->item_off.size(), hipMemcpyHostToDevice);
    if (e == hipSuccess && pl->n_fixups) e = hipMalloc((void **)&pl->fixups_dev, sizeof(Fixup) * fixups.size());
    if (e == hipSuccess && pl->n_fixups)
        e = hipMemcpy(pl->fixups_dev, fixups.data(), sizeof(Fixup) * fixups.size(), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        fg_spmm_plan_destroy(pl);
        return fail(FG_ERR_HIP, "fg_spmm_plan_create: %s", hipGetErrorString(e));
    }
    *plan_out = pl;
    return FG_OK;
}

extern "C" void fg_spmm_plan_destroy(fg_spmm_plan *pl) {
    if (!pl) return;
    if (pl->items_dev) (void)hipFree(pl->items_dev);
    if (pl->item_off_dev) (void)hipFree(pl->item_off_dev);
    if (pl->fixups_dev) (void)hipFree(pl->fixups_dev);
    if (pl->partial_dev) (void)hipFree(pl->partial_dev);
    if (pl->tiled_dev) (void)hipFree(pl->tiled_dev);
    if (pl->idx16_dev) (void)hipFree(pl->idx16_dev);
    if (pl->idx16_words_dev) (void)hipFree(pl->idx16_words_dev);
    delete pl;
}

namespace {
// One 16-byte word per lane: word i of the row-major matrix goes to its tile's block.
__global__ __launch_bounds__(256) void tile_major_kernel(const float4 *x, float4 *dst, uint32_t n_rows,
                                                         uint32_t row_words, uint32_t tile_words, uint32_t n_words) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= n_words) return;
    const uint32_t r = i / row_words, c = i - r * row_words;
    const uint32_t t = c / tile_words, w = c - t * tile_words;
    dst[((uint64_t)t * n_rows + r) * tile_words + w] = x[i];
}
}  // namespace

namespace fg {
bool wants_tile_major(const fg_spmm_plan *pl, int n_tiles, uint64_t x_bytes) {
    if (pl->tile_major == 2 || n_tiles < 2) return false;
    if (pl->tile_major == 1) return true;
    // Measured on the 232,965-node graph (238 / 477 MB): nothing at 2 tiles, 10-12 % at 4 and 8 tiles;
    // on a 23,296-node graph (47 MB, mostly cache-resident) the copy only costs its own time.
    return n_tiles >= 4 && x_bytes >= (64ull << 20);
}
int make_tile_major(const fg_spmm_plan *pl, const float *x, int64_t n_rows, int F, int tile, void *stream, int slot, int n_slots) {
    const uint64_t floats = (uint64_t)n_rows * (uint64_t)F;
    if (slot < 0 || slot >= n_slots) return fail(FG_ERR_ARG, "tile-major copy: slot %d of %d", slot, n_slots);
    if (F % 4 != 0 || tile % 4 != 0 || F % tile != 0 || floats >= (1ull << 32) || ((uintptr_t)x & 15) != 0)
        return fail(FG_ERR_SHAPE, "tile-major copy of a %lld x %d matrix in tiles of %d floats", (long long)n_rows, F, tile);
    if (floats * (uint64_t)n_slots > pl->tiled_floats)
        return fail(FG_ERR_ARG, "tile-major copy: the plan's buffer holds %zu floats, %llu needed", pl->tiled_floats,
                    (unsigned long long)(floats * n_slots));
    const uint32_t n_words = (uint32_t)(floats / 4);
    if (n_words == 0) return FG_OK;
    hipLaunchKernelGGL(tile_major_kernel, dim3((n_words + 255u) / 256u), dim3(256), 0, (hipStream_t)stream,
                       reinterpret_cast<const float4 *>(x), reinterpret_cast<float4 *>(pl->tiled_dev + floats * slot),
                       (uint32_t)n_rows, (uint32_t)(F / 4), (uint32_t)(tile / 4), n_words);
    FG_HIP_TRY(hipGetLastError());
    return FG_OK;
}
int check_device(const fg_spmm_plan *pl) {
    int dev = -1;
    FG_HIP_TRY(hipGetDevice(&dev));
    if (dev != pl->device)
        return fail(FG_ERR_ARG, "the plan lives on device %d but the current device is %d", pl->device, dev);
    return FG_OK;
}
namespace {
int grow(float **buf, size_t *have, size_t need, void *stream, const char *what) {
    if (need <= *have) return FG_OK;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    // (the NULL stream cannot be captured, and querying it while another stream is being captured would
    // invalidate that capture)
    if (stream && hipStreamIsCapturing((hipStream_t)stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone)
        return fail(FG_ERR_ARG, "the plan's %s holds %zu floats and this call needs %zu, but the stream is being captured: "
                    "call fg_spmm_plan_reserve (or run the call once) before capturing", what, *have, need);
    if (*buf) FG_HIP_TRY(hipFree(*buf));
    *buf = nullptr; *have = 0;
    if (hipMalloc((void **)buf, need * sizeof(float)) != hipSuccess) {
        (void)hipGetLastError();
        *buf = nullptr;
        return fail(FG_ERR_NOMEM, "cannot allocate %zu bytes for the plan's %s", need * sizeof(float), what);
    }
    *have = need;
    return FG_OK;
}
}  // namespace
int ensure_scratch(fg_spmm_plan *pl, const ScratchNeed &need, void *stream) {
    if (int rc = grow(&pl->partial_dev, &pl->partial_floats, need.partial, stream, "scratch buffer")) return rc;
    return grow(&pl->tiled_dev, &pl->tiled_floats, need.tiled, stream, "tile-by-tile copy buffer");
}
// Declared in fg_spmm.hip: text of the launch the SpMM entry points would use.
std::string spmm_launch_text(const fg_spmm_plan *plan, int F, int num_feat_partitions);
}

namespace {
// dst[i] = (uint16_t)src[i], four elements per lane (the tail one by one); *bad is set when an id lies outside [0, width).
__global__ __launch_bounds__(256) void narrow_indices_kernel(const int32_t *src, uint16_t *dst, int64_t n, int32_t width, int32_t *bad) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= n) return;
    bool out_of_range = false;
    for (int k = 0; k < 4 && i + k < n; ++k) {
        const int32_t c = src[i + k];
        out_of_range |= (c < 0 || c >= width);
        dst[i + k] = (uint16_t)c;
    }
    if (out_of_range) atomicOr(bad, 1);
}

__device__ __forceinline__ uint64_t mix64_dev(uint64_t z) {          // splitmix64 finaliser
    z += 0x9e3779b97f4a7c15ull;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

// A cheap fingerprint of an id array: the sum of a hash of (position, id) over the first and the last kPrintIds ids.
constexpr int kPrintIds = 1024;
__global__ __launch_bounds__(256) void fingerprint_kernel(const int32_t *src, int64_t n, unsigned long long *out) {
    unsigned long long h = 0;
    for (int64_t j = threadIdx.x; j < 2 * kPrintIds; j += 256) {
        const int64_t i = j < kPrintIds ? j : n - 2 * kPrintIds + j;      // the last kPrintIds positions
        if (i < 0 || i >= n || (j >= kPrintIds && i < kPrintIds)) continue;
        h += mix64_dev(((uint64_t)i << 32) ^ (uint32_t)src[i]);
    }
    if (h) atomicAdd(out, h);
}

// words_dev[0] holds the range flag of narrow_indices_kernel, words_dev[1] the fingerprint; read back synchronously
int fingerprint(const int32_t *idx_dev, int64_t n, hipStream_t st, unsigned long long *words_dev, uint64_t *out) {
    FG_HIP_TRY(hipMemsetAsync(words_dev + 1, 0, sizeof(unsigned long long), st));
    hipLaunchKernelGGL(fingerprint_kernel, dim3(1), dim3(256), 0, st, idx_dev, n, words_dev + 1);
    FG_HIP_TRY(hipGetLastError());
    unsigned long long h = 0;
    FG_HIP_TRY(hipMemcpyAsync(&h, words_dev + 1, sizeof(h), hipMemcpyDeviceToHost, st));
    FG_HIP_TRY(hipStreamSynchronize(st));
    *out = (uint64_t)h + (uint64_t)n;
    return FG_OK;
}

std::atomic<int> g_debug_checks{0};
}  // namespace

extern "C" int fg_debug_checks(int on) { return g_debug_checks.exchange(on ? 1 : 0); }

namespace fg {
const uint16_t *narrow_indices(const fg_spmm_plan *plan, const int32_t *idx) {
    if (!plan->idx16_dev || !idx || idx != plan->idx16_src) return nullptr;
    if (g_debug_checks.load(std::memory_order_relaxed)) {
        // the array at this address must still be the one the copy was made from
        uint64_t now = 0;
        if (fingerprint(idx, plan->nnz, nullptr, plan->idx16_words_dev, &now) != FG_OK) return nullptr;
        if (now != plan->idx16_fingerprint) {
            fail(FG_ERR_ARG, "the int32 column ids at %p changed after fg_spmm_plan_narrow_indices copied them; the int32 array is read instead",
                 (const void *)idx);
            return nullptr;
        }
    }
    return plan->idx16_dev;
}
}  // namespace fg

extern "C" int fg_spmm_plan_narrow_indices(fg_spmm_plan *pl, const int32_t *idx_dev, void *stream) {
    if (!pl) return fail(FG_ERR_ARG, "plan is null");
    if (int drc = fg::check_device(pl)) return drc;
    auto forget = [&]() {
        if (pl->idx16_dev) (void)hipFree(pl->idx16_dev);
        pl->idx16_dev = nullptr; pl->idx16_src = nullptr; pl->idx16_fingerprint = 0;
    };
    if (!idx_dev) {                                  // forget the copy
        forget();
        return FG_OK;
    }
    const int64_t width = (pl->n_src + pl->num_col_partitions - 1) / pl->num_col_partitions;
    if (width > 65536)
        return fail(FG_ERR_SHAPE, "column ids of partitions %lld columns wide do not fit 16 bits", (long long)width);
    forget();
    if (pl->nnz == 0) return FG_OK;
    if (!pl->idx16_words_dev && hipMalloc((void **)&pl->idx16_words_dev, 2 * sizeof(unsigned long long)) != hipSuccess) {
        (void)hipGetLastError();
        pl->idx16_words_dev = nullptr;
        return fail(FG_ERR_NOMEM, "cannot allocate the 16-bit column ids' check words");
    }
    if (hipMalloc((void **)&pl->idx16_dev, (size_t)pl->nnz * sizeof(uint16_t)) != hipSuccess) {
        (void)hipGetLastError();
        pl->idx16_dev = nullptr;
        return fail(FG_ERR_NOMEM, "cannot allocate %zu bytes for the 16-bit column ids", (size_t)pl->nnz * sizeof(uint16_t));
    }
    hipStream_t st = (hipStream_t)stream;
    int32_t *bad_dev = reinterpret_cast<int32_t *>(pl->idx16_words_dev);
    hipError_t e = hipMemsetAsync(bad_dev, 0, sizeof(int32_t), st);
    if (e == hipSuccess) {
        const int64_t blocks = (pl->nnz + 1023) / 1024;
        hipLaunchKernelGGL(narrow_indices_kernel, dim3((unsigned)blocks), dim3(256), 0, st, idx_dev, pl->idx16_dev, pl->nnz,
                           (int32_t)std::max<int64_t>(width, 1), bad_dev);
        e = hipGetLastError();
    }
    int32_t bad = 0;
    if (e == hipSuccess) e = hipMemcpyAsync(&bad, bad_dev, sizeof(bad), hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess) {
        forget();
        return fail(FG_ERR_HIP, "fg_spmm_plan_narrow_indices: %s", hipGetErrorString(e));
    }
    if (bad) {
        forget();
        return fail(FG_ERR_GRAPH, "fg_spmm_plan_narrow_indices: a column id lies outside [0, %lld)", (long long)width);
    }
    if (int rc = fingerprint(idx_dev, pl->nnz, st, pl->idx16_words_dev, &pl->idx16_fingerprint)) {
        forget();
        return rc;
    }
    pl->idx16_src = idx_dev;
    return FG_OK;
}

extern "C" int64_t fg_spmm_plan_bytes(const fg_spmm_plan *pl) {
    if (!pl) return 0;
    int64_t b = 0;
    b += (int64_t)pl->n_items * (int64_t)sizeof(Item) + (int64_t)pl->n_fixups * (int64_t)sizeof(Fixup);
    b += (int64_t)(pl->num_col_partitions + 1) * (int64_t)sizeof(int64_t);
    b += (int64_t)pl->partial_floats * 4 + (int64_t)pl->tiled_floats * 4;
    if (pl->idx16_dev) b += pl->nnz * 2;
    if (pl->idx16_words_dev) b += 16;
    return b;
}

extern "C" int fg_spmm_plan_reserve(fg_spmm_plan *pl, int op, int heads, int head_len, int num_feat_partitions) {
    if (!pl) return fail(FG_ERR_ARG, "plan is null");
    if (int drc = fg::check_device(pl)) return drc;
    if (heads < 1 || head_len < 1 || (int64_t)heads * head_len > INT32_MAX)
        return fail(FG_ERR_SHAPE, "heads and head length must be positive, got %d x %d", heads, head_len);
    fg::ScratchNeed need;
    int rc;
    switch (op) {
        case FG_OP_SPMM_SUM: rc = fg::spmm_scratch_need(pl, heads * head_len, heads, FG_REDUCE_SUM, num_feat_partitions, &need); break;
        case FG_OP_SPMM_EXTREME: rc = fg::spmm_scratch_need(pl, heads * head_len, heads, FG_REDUCE_MAX, num_feat_partitions, &need); break;
        case FG_OP_SDDMM_DDS: rc = fg::sddmm_dds_scratch_need(pl, heads, head_len, num_feat_partitions, &need); break;
        case FG_OP_EDGE_SOFTMAX: rc = fg::softmax_scratch_need(pl, heads, &need); break;
        case FG_OP_ATTENTION: rc = fg::attention_scratch_need(pl, heads, head_len, false, true, &need); break;
        case FG_OP_ATTENTION_ADDITIVE: rc = fg::attention_scratch_need(pl, heads, head_len, true, true, &need); break;
        case FG_OP_GSPMM_BCAST: rc = fg::gspmm_bcast_scratch_need(pl, heads * head_len, false, &need); break;
        case FG_OP_GSPMM_BCAST_ARG: rc = fg::gspmm_bcast_scratch_need(pl, heads * head_len, true, &need); break;
        default: return fail(FG_ERR_ARG, "fg_spmm_plan_reserve: unknown operator %d", op);
    }
    if (rc != FG_OK) return rc;
    return fg::ensure_scratch(pl, need, nullptr);
}

extern "C" int fg_spmm_plan_describe(const fg_spmm_plan *pl, int F, int T, char *buf, size_t buf_len) {
    if (!pl || !buf || buf_len == 0) return fail(FG_ERR_ARG, "fg_spmm_plan_describe: bad argument");
    char head[800];
    snprintf(head, sizeof(head),
             "featgraph-hip plan (gfx950)\n"
             "  adjacency        : %lld dst x %lld src, nnz %lld, %d source-column partition(s)\n"
             "  work items       : %lld (one wavefront each; 4 per workgroup), %lld hold several rows (<= %d elements)\n"
             "  split threshold  : %d elements; %lld row segment(s) split into %lld piece(s)\n"
             "  longest segment  : %lld elements; %lld empty row(s)\n",
             (long long)pl->n_dst, (long long)pl->n_src, (long long)pl->nnz, pl->num_col_partitions,
             (long long)pl->n_items, (long long)pl->n_multi_items, pl->item_edges, pl->split_threshold, (long long)pl->n_split_rows,
             (long long)pl->n_slots, (long long)pl->max_len, (long long)pl->n_empty);
    std::string s = head;
    if (pl->idx16_dev) s += "  column ids       : a 16-bit copy is streamed by the sum SpMM and the tiled SDDMM\n";
    if (F > 0) s += fg::spmm_launch_text(pl, F, T);
    const size_t n = std::min(s.size(), buf_len - 1);
    memcpy(buf, s.data(), n);
    buf[n] = 0;
    return (int)n;
}
