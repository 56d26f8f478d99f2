// Shared internals of libfeatgraph_hip.so: error reporting and the plan layout.
#pragma once

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <vector>

#include "../../include/featgraph_hip.h"

namespace fg {

// Records a message for fg_last_error() and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define FG_HIP_TRY(expr)                                                              \
    do {                                                                              \
        hipError_t _e = (expr);                                                       \
        if (_e != hipSuccess)                                                         \
            return ::fg::fail(FG_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(_e)); \
    } while (0)

// One unit of wavefront work: `len` consecutive stored elements starting at `start`.
//   info >= 0 : a piece of a row segment longer than the split threshold; all elements belong
//               to output row `row`, the piece's sum goes to partial[info] and a second kernel
//               adds the pieces.
//   info <  0 : -info whole consecutive row segments, rows [row, row - info); the wavefront
//               writes those rows itself.  Row boundaries come from the position array.
struct Item {
    int32_t start;
    int32_t len;
    int32_t row;
    int32_t info;
};

constexpr int kItemEdges = 256;   // elements staged in LDS per wavefront at a time
constexpr int kItemRows = 64;     // most rows one multi-row item may hold

// A row segment that was split: pieces partial[slot0 .. slot0 + n_pieces) add up to it.
struct Fixup {
    int32_t row;
    int32_t slot0;
    int32_t n_pieces;
    int32_t pad;
};

}  // namespace fg

struct fg_spmm_plan {
    int64_t n_dst = 0, n_src = 0, nnz = 0;
    int num_col_partitions = 1;
    int split_threshold = 0;
    int item_edges = 0;              // element budget of a multi-row item
    bool wide_offsets = false;       // never use 32-bit byte offsets into the feature matrices
    int tile_major = 0;              // fg_plan_opts.tile_major
    int device = 0;
    // per partition: [item_begin, item_end) and [fixup_begin, fixup_end)
    std::vector<int64_t> item_off, fixup_off;
    int64_t n_items = 0, n_fixups = 0, n_slots = 0, max_slots_in_partition = 0;
    fg::Item *items_dev = nullptr;
    int64_t *item_off_dev = nullptr;     // item_off on the device (num_col_partitions + 1 entries)
    fg::Fixup *fixups_dev = nullptr;
    // partial sums of split rows; grown on demand to max_slots_in_partition * F floats
    mutable float *partial_dev = nullptr;
    mutable size_t partial_floats = 0;
    // tile-by-tile copy of the source features of the call in progress; grown on demand
    mutable float *tiled_dev = nullptr;
    mutable size_t tiled_floats = 0;
    // statistics for fg_spmm_plan_describe
    int64_t max_len = 0, n_empty = 0, n_split_rows = 0, n_multi_items = 0;
};

namespace fg {
// Makes plan->partial_dev hold at least floats_per_piece floats for every piece of split rows of
// one partition (grown on demand, never shrunk).
int ensure_partial(const fg_spmm_plan *plan, size_t floats_per_piece);
// Whether a call with n_tiles feature tiles over a source matrix of x_bytes gathers from a
// tile-by-tile copy (the plan's tile_major option; the kernel-side conditions are the caller's).
bool wants_tile_major(const fg_spmm_plan *plan, int n_tiles, uint64_t x_bytes);
// plan->tiled_dev[(t * n_rows + r) * tile + i] = x[r * F + t * tile + i] for the F / tile tiles of
// an [n_rows, F] matrix (F and tile multiples of 4, x 16-byte aligned, fewer than 2^32 floats),
// on `stream`.  The buffer is grown on demand and never shrunk.
// With n_slots > 1 the buffer holds that many copies of this size one after the other and the call fills
// copy `slot` (fill slot 0 first: growing the buffer discards what it held).
int make_tile_major(const fg_spmm_plan *plan, const float *x, int64_t n_rows, int F, int tile, void *stream,
                    int slot = 0, int n_slots = 1);
// Makes plan->partial_dev hold at least `floats` floats (grown on demand, never shrunk).
int ensure_scratch(const fg_spmm_plan *plan, size_t floats);
// FG_OK when the calling thread's current device is the one the plan was created on.
int check_device(const fg_spmm_plan *plan);
}  // namespace fg
