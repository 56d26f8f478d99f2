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
    int32_t part;     // the source partition the segment belongs to
};

}  // namespace fg

struct fg_spmm_plan {
    int64_t n_dst = 0, n_src = 0, nnz = 0;
    int num_col_partitions = 1;
    int split_threshold = 0;
    int item_edges = 0;              // element budget of a multi-row item
    bool wide_offsets = false;       // never use 32-bit byte offsets into the feature matrices
    int tile_major = 0;              // fg_plan_opts.tile_major
    int pass_buffers = 0;            // fg_plan_opts.pass_buffers
    int device = 0;
    // per partition: [item_begin, item_end) and [fixup_begin, fixup_end)
    std::vector<int64_t> item_off, fixup_off;
    int64_t n_items = 0, n_fixups = 0, n_slots = 0, max_slots_in_partition = 0;
    fg::Item *items_dev = nullptr;
    int64_t *item_off_dev = nullptr;     // item_off on the device (num_col_partitions + 1 entries)
    fg::Fixup *fixups_dev = nullptr;
    // Scratch that the operator calls fill and read (partial sums of split rows, per-tile partial scores,
    // softmax statistics, attention row state); grown by fg_spmm_plan_reserve or by the first call that
    // needs more, never shrunk.
    float *partial_dev = nullptr;
    size_t partial_floats = 0;
    // tile-by-tile copy of the gathered operand(s) of the call in progress; grown the same way
    float *tiled_dev = nullptr;
    size_t tiled_floats = 0;
    // 16-bit copy of the layout's (partition-local) column ids, made by fg_spmm_plan_narrow_indices and owned by the
    // plan: the kernels that can read it do so whenever a call hands them the int32 array it was made from.
    uint16_t *idx16_dev = nullptr;
    const int32_t *idx16_src = nullptr;
    uint64_t idx16_fingerprint = 0;               // of idx16_src's contents when the copy was made (fg_debug_checks re-checks it)
    unsigned long long *idx16_words_dev = nullptr; // two device words: the range flag and the fingerprint under construction
    // statistics for fg_spmm_plan_describe
    int64_t max_len = 0, n_empty = 0, n_split_rows = 0, n_multi_items = 0;
};

namespace fg {
// Device scratch one operator call needs from its plan, in floats.
struct ScratchNeed {
    size_t partial = 0;   // plan->partial_dev
    size_t tiled = 0;     // plan->tiled_dev
};
// Makes the plan's two scratch buffers hold at least `need` (grown on demand, never shrunk).  Growing
// frees and allocates device memory, which synchronises the device and cannot be recorded: when `stream`
// is being captured into a graph and a buffer is too small, nothing is changed and FG_ERR_ARG is returned
// (reserve the scratch with fg_spmm_plan_reserve, or run the call once, before capturing).
int ensure_scratch(fg_spmm_plan *plan, const ScratchNeed &need, void *stream);
// Whether a call with n_tiles feature tiles over a source matrix of x_bytes gathers from a
// tile-by-tile copy (the plan's tile_major option; the kernel-side conditions are the caller's).
bool wants_tile_major(const fg_spmm_plan *plan, int n_tiles, uint64_t x_bytes);
// plan->tiled_dev[(t * n_rows + r) * tile + i] = x[r * F + t * tile + i] for the F / tile tiles of
// an [n_rows, F] matrix (F and tile multiples of 4, x 16-byte aligned, fewer than 2^32 floats),
// on `stream`.  With n_slots > 1 the buffer holds that many copies of this size one after the other and
// the call fills copy `slot`.  The buffer must already be large enough (ensure_scratch).
int make_tile_major(const fg_spmm_plan *plan, const float *x, int64_t n_rows, int F, int tile, void *stream,
                    int slot = 0, int n_slots = 1);
// The plan's 16-bit copy of `idx` when it has one of exactly this array (same address), else null.  With
// fg_debug_checks(1) the array's fingerprint is compared as well (a device round trip per call): an array that was
// rewritten or replaced at the same address is then read as int32 and the mismatch is left in fg_last_error().
const uint16_t *narrow_indices(const fg_spmm_plan *plan, const int32_t *idx);
// Looks up, once per device, the address of the fixed array that fg_spmm_csr_noalloc_f32 keeps its partial sums in.
void prepare_fixed_scratch(int dev);
// FG_OK when the calling thread's current device is the one the plan was created on.
int check_device(const fg_spmm_plan *plan);

// What one call of each operator needs (the same functions size the buffers inside the calls).
// Each returns FG_OK or the status the call itself would return for that shape.
int spmm_scratch_need(const fg_spmm_plan *plan, int F, int heads, int reduce, int num_feat_partitions, ScratchNeed *need);
int sddmm_dds_scratch_need(const fg_spmm_plan *plan, int H, int D, int num_feat_partitions, ScratchNeed *need);
int softmax_scratch_need(const fg_spmm_plan *plan, int heads, ScratchNeed *need);
int gspmm_bcast_scratch_need(const fg_spmm_plan *plan, int out_len, bool with_arg, ScratchNeed *need);
bool attention_pass_buffers(const fg_spmm_plan *plan, int heads, int head_len);
// forward: the call is the forward pass (whose partitions may write buffers of their own); the gradient sweeps need
// only the head-by-head copies of the gathered operands.
int attention_scratch_need(const fg_spmm_plan *plan, int heads, int head_len, bool additive, bool own_row_state,
                           ScratchNeed *need, bool forward = true);
}  // namespace fg
