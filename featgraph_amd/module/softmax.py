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
            self.grad_tvm = torch.zeros_like(self.out_tvm)
        _lib.check(_lib.lib().fg_edge_softmax_backward_f32(self._plan, _lib.dev_ptr(self._indptr_dev),
                                                           _lib.dev_ptr(softmax), _lib.dev_ptr(grad_softmax),
                                                           _lib.dev_ptr(self.grad_tvm), self._heads,
                                                           common.stream_ptr()))
        return self.grad_tvm

    def measure_average_time(self, input_tvm_ndarrays, num_runs):
        if self._placeholders is None:
            raise RuntimeError("call build() before measure_average_time()")
        common.check_inputs(input_tvm_ndarrays, self._placeholders, self._ctx)
        x = input_tvm_ndarrays[0]
        return common.timed_mean_seconds(lambda: self._forward(x, self.out_tvm), num_runs)

    @property
    def ctx(self):
        return self._ctx

    @property
    def target(self):
        return self._target
