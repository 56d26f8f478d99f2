"""Edge softmax: softmax of per-edge scores over the incoming edges of every destination row,
per head.  The reference snapshot has no such operator; the class follows the build()/run()
conventions of the reference's modules (python/featgraph/module/spmm.py:81-161) and sits between
the multi-head SDDMM (scores) and the per-head weighted SpMM (aggregation) of an attention layer."""
import ctypes

import numpy as np
import torch

from .. import _lib
from . import common


class EdgeSoftmaxhip(object):
    """out[e, h] = softmax over the edges e' of e's row of Scores[e', h].

    Scores is (nnz,) or (nnz, H), float32, in the adjacency's CSR edge order (rows are
    destinations).  Rows without edges contribute nothing.  run() returns the same preallocated
    tensor on every call; backward(softmax, grad_softmax) returns the gradient with respect to
    the scores in a second preallocated tensor.
    """

    def __init__(self, adj_scipy):
        adj = adj_scipy if adj_scipy.format == 'csr' else adj_scipy.tocsr()
        self._num_rows, self._num_cols = adj.shape
        self._target = 'rocm'
        self._ctx = common.device()
        self._indptr = np.ascontiguousarray(adj.indptr, dtype=np.int32)
        indices = np.ascontiguousarray(adj.indices, dtype=np.int32)
        _lib.check(_lib.lib().fg_check_csr_host(self._num_rows, self._num_cols, _lib.host_ptr(self._indptr),
                                                _lib.host_ptr(indices)))
        self._nnz = int(self._indptr[-1])
        self._indptr_dev = common.to_device_i32(self._indptr, self._ctx)
        self._plan = ctypes.c_void_p()
        with torch.cuda.device(self._ctx):
            _lib.check(_lib.lib().fg_spmm_plan_create(_lib.host_ptr(self._indptr), self._num_rows, self._num_cols,
                                                      1, _lib.plan_opts_ptr(), ctypes.byref(self._plan)))
        self._placeholders = None
        self._heads = None
        self.out_tvm = None
        self.grad_tvm = None

    def __del__(self):
        plan = getattr(self, "_plan", None)
        if plan is not None and plan.value:
            try:
                _lib.lib().fg_spmm_plan_destroy(plan)
            except Exception:
                pass
            self._plan = None

    def build(self, input_placeholders, compute_args=None, schedule_args=None):
        """input_placeholders: [Scores (nnz,) or (nnz, H)]; no compute or schedule arguments."""
        common.take_args(compute_args or {}, (), "compute_func")
        common.take_args(schedule_args or {}, (), "schedule_func")
        if len(input_placeholders) != 1:
            raise ValueError("edge softmax takes one input (Scores), got %d" % len(input_placeholders))
        ph = input_placeholders[0]
        if len(ph.shape) not in (1, 2) or ph.shape[0] != self._nnz:
            raise ValueError("Scores must have shape (nnz=%d,) or (nnz, H), got %s" % (self._nnz, ph.shape))
        self._placeholders = [ph]
        self._heads = int(ph.shape[1]) if len(ph.shape) == 2 else 1
        if self._heads < 1:
            raise ValueError("number of heads must be positive")
        common.reserve(self._plan, common.OP_EDGE_SOFTMAX, self._heads, 1, 0, self._ctx)
        self.out_tvm = torch.zeros(tuple(ph.shape), dtype=torch.float32, device=self._ctx)
        self.grad_tvm = None

    def lower_to_ir(self, input_placeholders, compute_args=None, schedule_args=None):
        buf = ctypes.create_string_buffer(4096)
        _lib.check(_lib.lib().fg_spmm_plan_describe(self._plan, 0, 0, buf, len(buf)))
        return buf.value.decode() + "  kernel           : edge_softmax_kernel over the plan's items; pieces of split rows merged per row\n"

    def _forward(self, scores, out):
        _lib.check(_lib.lib().fg_edge_softmax_f32(self._plan, _lib.dev_ptr(self._indptr_dev), _lib.dev_ptr(scores),
                                                  _lib.dev_ptr(out), self._heads, common.stream_ptr()))

    def run(self, input_tvm_ndarrays):
        """[Scores] -> self.out_tvm (the same tensor on every call); nothing is synchronised."""
        if self._placeholders is None:
            raise RuntimeError("call build() before run()")
        common.ensure_output(self)
        common.check_inputs(input_tvm_ndarrays, self._placeholders, self._ctx)
        self._forward(input_tvm_ndarrays[0], self.out_tvm)
        return self.out_tvm

    def backward(self, softmax, grad_softmax):
        """Gradient with respect to the scores, given run()'s output and dL/d(output)."""
        if self._placeholders is None:
            raise RuntimeError("call build() before backward()")
        common.check_inputs([softmax], self._placeholders, self._ctx)
        common.check_inputs([grad_softmax], self._placeholders, self._ctx)
        if self.grad_tvm is None:
            self.grad_tvm = torch.zeros_like(softmax)
        _lib.check(_lib.lib().fg_edge_softmax_backward_f32(self._plan, _lib.dev_ptr(self._indptr_dev),
                                                           _lib.dev_ptr(softmax), _lib.dev_ptr(grad_softmax),
                                                           _lib.dev_ptr(self.grad_tvm), self._heads,
                                                           common.stream_ptr()))
        return self.grad_tvm

    def measure_average_time(self, input_tvm_ndarrays, num_runs):
        if self._placeholders is None:
            raise RuntimeError("call build() before measure_average_time()")
        common.ensure_output(self)
        common.check_inputs(input_tvm_ndarrays, self._placeholders, self._ctx)
        x = input_tvm_ndarrays[0]
        return common.timed_mean_seconds(lambda: self._forward(x, self.out_tvm), num_runs)

    @property
    def ctx(self):
        return self._ctx

    @property
    def target(self):
        return self._target


class EdgeSoftmaxSpMMhip(object):
    """Attention aggregation without a stored softmax:

        out[v, h, :] = sum over the edges e into v of softmax_v(Scores)[e, h] * SrcFeat[col e, h, :]

    Scores is (nnz,) or (nnz, H) in the adjacency's CSR edge order, SrcFeat (num_cols, F) or
    (num_cols, H, D).  Three launches: the rows' (max, sum of exp) per head, a pass that writes
    exp(score - max) / sum directly in the order and layout the per-head weighted SpMM streams, and that
    SpMM; the normalised [nnz, H] array of EdgeSoftmaxhip is never written or read back.  The reference
    has neither operator; conventions as in its modules (python/featgraph/module/spmm.py:81-161).
    """

    def __init__(self, adj_scipy):
        from .gspmm import GSpMMhip
        self._agg = GSpMMhip(adj_scipy)
        self._ctx = self._agg.ctx
        self._target = self._agg.target
        indptr = self._agg._adj_indptr
        self._nnz = int(indptr[-1])
        self._num_rows = self._agg._num_rows
        rows = np.repeat(np.arange(self._num_rows, dtype=np.int32), np.diff(indptr))
        self._edge_row = common.to_device_i32(rows, self._ctx)
        self._placeholders = None
        self.out_tvm = None

    def build(self, input_placeholders, compute_args=None, schedule_args=None):
        """input_placeholders: [Scores, SrcFeat]; schedule_args as for GSpMMhip ('num_src_partitions')."""
        common.take_args(compute_args or {}, ('num_feat_partitions',), "compute_func")
        if len(input_placeholders) != 2:
            raise ValueError("takes two inputs (Scores, SrcFeat), got %d" % len(input_placeholders))
        s_ph, x_ph = input_placeholders
        heads = x_ph.shape[1] if len(x_ph.shape) == 3 else 1
        want = ((self._nnz,), (self._nnz, 1)) if heads == 1 else ((self._nnz, heads),)
        if tuple(s_ph.shape) not in want:
            raise ValueError("Scores must have shape %s, got %s" % (want[-1], s_ph.shape))
        w_shape = (self._nnz,) if heads == 1 else (self._nnz, heads)
        self._agg.build([x_ph, common.placeholder(w_shape)], dict(compute_args or {}), dict(schedule_args or {}))
        self._heads = heads
        common.reserve(self._agg._layout(1)['plan'], common.OP_EDGE_SOFTMAX, heads, 1, 0, self._ctx)
        self._placeholders = [s_ph, x_ph]
        self._row_stats = torch.zeros((self._num_rows, heads, 2), dtype=torch.float32, device=self._ctx)
        self._weights = torch.empty((heads, self._nnz), dtype=torch.float32, device=self._ctx)
        self.out_tvm = self._agg.out_tvm

    def _launch(self, scores, x):
        agg, L, s = self._agg, _lib.lib(), common.stream_ptr()
        csr = agg._layout(1)
        lay = agg._active
        _lib.check(L.fg_edge_softmax_stats_f32(csr['plan'], _lib.dev_ptr(csr['pos']), _lib.dev_ptr(scores),
                                               _lib.dev_ptr(self._row_stats), self._heads, s))
        pos = lay['edge_pos32'] if lay['P'] > 1 else None
        _lib.check(L.fg_edge_softmax_head_major_f32(_lib.dev_ptr(scores), _lib.dev_ptr(self._row_stats),
                                                    _lib.dev_ptr(self._edge_row), _lib.dev_ptr(pos), self._nnz,
                                                    self._heads, _lib.dev_ptr(self._weights), s))
        _lib.check(L.fg_gspmm_f32(lay['plan'], _lib.dev_ptr(lay['pos']), _lib.dev_ptr(lay['idx']),
                                  _lib.dev_ptr(self._weights), _lib.dev_ptr(x), _lib.dev_ptr(self.out_tvm),
                                  agg._feat_len, self._heads, 1, 0, agg._num_feat_partitions, s))

    def run(self, input_tvm_ndarrays):
        """[Scores, SrcFeat] -> self.out_tvm (the same tensor on every call); nothing is synchronised."""
        if self._placeholders is None:
            raise RuntimeError("call build() before run()")
        common.ensure_output(self)
        common.check_inputs(input_tvm_ndarrays, self._placeholders, self._ctx)
        self._launch(input_tvm_ndarrays[0], input_tvm_ndarrays[1])
        return self.out_tvm

    def measure_average_time(self, input_tvm_ndarrays, num_runs):
        if self._placeholders is None:
            raise RuntimeError("call build() before measure_average_time()")
        common.ensure_output(self)
        common.check_inputs(input_tvm_ndarrays, self._placeholders, self._ctx)
        s, x = input_tvm_ndarrays
        return common.timed_mean_seconds(lambda: self._launch(s, x), num_runs)

    @property
    def ctx(self):
        return self._ctx

    @property
    def target(self):
        return self._target
