"""Dot-product attention over a graph's edges in one operator: multi-head SDDMM, edge softmax and per-head
weighted SpMM without the [nnz, H] scores ever being stored.  The reference has no such operator; the
class follows the build()/run() conventions of its modules (python/featgraph/module/spmm.py:81-161)."""
import ctypes

import numpy as np
import torch

from .. import _lib
from .. import tuning
from ..util import util_convert_csr_to_dds
from . import common

_INT32_MAX = 2 ** 31 - 1


class GraphAttentionhip(object):
    """out[v, h, :] = sum over the edges e into v of softmax_v(scale * <K[col e, h, :], Q[v, h, :]>) * V[col e, h, :]

    Q is (num_rows, H, D), K and V are (num_cols, H, D), D in {16, 32, 64}; rows without edges give 0.
    compute_args: 'scale' (default 1 / sqrt(D)); 'scores': 'dot' (default) | 'additive' -- the attention of GAT
    layers, scores leaky_relu(El[col e, h] + Er[v, h]) with 'negative_slope' (default 0.2); the inputs are then
    [Er (num_rows, H), El (num_cols, H), V (num_cols, H, D)].  schedule_args: 'num_src_partitions': 'auto' (default: chosen
    for the L2 size, as for SpMM) | int | None (plain CSR); 'num_dst_partitions': the same for the transposed
    adjacency that backward() sweeps.
    Equal, within rounding, to MultiHeadSDDMMhip -> EdgeSoftmaxhip -> GSpMMhip with per-head weights.
    """

    def __init__(self, adj_scipy):
        csr = adj_scipy.tocsr() if adj_scipy.format != 'csr' else adj_scipy
        self._num_rows, self._num_cols = csr.shape
        self._target = 'rocm'
        self._ctx = common.device()
        self._indptr = np.ascontiguousarray(csr.indptr, dtype=np.int32)
        self._indices = np.ascontiguousarray(csr.indices, dtype=np.int32)
        _lib.check(_lib.lib().fg_check_csr_host(self._num_rows, self._num_cols, _lib.host_ptr(self._indptr),
                                                _lib.host_ptr(self._indices)))
        self._csr = csr
        self._layouts = {}
        self._placeholders = None
        self.out_tvm = None

    def _layout(self, P):
        """Device arrays and a plan without split rows for P source-column partitions (built once per P)."""
        if P in self._layouts:
            return self._layouts[P]
        if P > 1:
            pos, idx, _ = util_convert_csr_to_dds(self._csr, P)
        else:
            pos, idx = self._indptr, self._indices
        lay = {'P': P, 'pos': common.to_device_i32(pos, self._ctx), 'idx': common.to_device_i32(idx, self._ctx),
               'plan': ctypes.c_void_p()}
        base = _lib.plan_opts
        opts = _lib.FgPlanOpts(split_threshold=_INT32_MAX, item_edges=base.item_edges if base is not None else 0,
                               wide_offsets=0, tile_major=base.tile_major if base is not None else 0)
        with torch.cuda.device(self._ctx):
            _lib.check(_lib.lib().fg_spmm_plan_create(_lib.host_ptr(np.ascontiguousarray(pos, dtype=np.int32)),
                                                      self._num_rows, self._num_cols, P, ctypes.byref(opts),
                                                      ctypes.byref(lay['plan'])))
        common.narrow_indices(lay['plan'], lay['idx'], self._num_cols, P, self._ctx)
        self._layouts[P] = lay
        return lay

    def __del__(self):
        for lay in getattr(self, "_layouts", {}).values():
            plan = lay.get('plan')
            if plan is not None and plan.value:
                try:
                    _lib.lib().fg_spmm_plan_destroy(plan)
                except Exception:
                    pass
                lay['plan'] = None

    def build(self, input_placeholders, compute_args=None, schedule_args=None):
        """input_placeholders: [Q (num_rows, H, D), K (num_cols, H, D), V (num_cols, H, D)]."""
        compute_args = common.take_args(compute_args or {}, ('scale', 'scores', 'negative_slope'), "compute_func")
        self._additive = compute_args.get('scores', 'dot') == 'additive'
        if compute_args.get('scores', 'dot') not in ('dot', 'additive'):
            raise ValueError("scores must be 'dot' or 'additive'")
        if self._additive:
            return self._build_additive(input_placeholders, compute_args, schedule_args)
        schedule_args = common.take_args(schedule_args or {}, ('num_src_partitions', 'num_dst_partitions'), "schedule_func")
        if len(input_placeholders) != 3:
            raise ValueError("attention takes three inputs (Q, K, V), got %d" % len(input_placeholders))
        q_ph, k_ph, v_ph = input_placeholders
        if len(q_ph.shape) != 3 or q_ph.shape[0] != self._num_rows:
            raise ValueError("Q must be (num_rows=%d, H, D), got %s" % (self._num_rows, q_ph.shape))
        heads, head_len = int(q_ph.shape[1]), int(q_ph.shape[2])
        for name, ph in (("K", k_ph), ("V", v_ph)):
            if tuple(ph.shape) != (self._num_cols, heads, head_len):
                raise ValueError("%s must be (num_cols=%d, %d, %d), got %s" % (name, self._num_cols, heads, head_len, ph.shape))
        if head_len not in (16, 32, 64):
            raise ValueError("heads of 16, 32 or 64 floats, got %d" % head_len)
        P = self._partitions(schedule_args, 2 * 4 * head_len)
        self._heads, self._head_len = heads, head_len
        t_parts = schedule_args.get('num_dst_partitions')       # backward(): partitions of the transposed adjacency
        self._t_parts = None if t_parts in (None, 'auto') else int(t_parts)
        self._scale = float(compute_args.get('scale', 1.0 / np.sqrt(head_len)))
        self._active = self._layout(P)
        common.reserve(self._active['plan'], common.OP_ATTENTION, heads, head_len, 0, self._ctx)
        self._placeholders = [q_ph, k_ph, v_ph]
        self.out_tvm = torch.zeros((self._num_rows, heads, head_len), dtype=torch.float32, device=self._ctx)
        # every row's maximum score and sum of exponentials, per head: what backward() starts from
        self.state_tvm = torch.zeros((self._num_rows, heads, 2), dtype=torch.float32, device=self._ctx)
        self._coef = None

    def _partitions(self, schedule_args, slice_row_bytes):
        """Source partitions: one head per XCD, whose L2 holds the head's slices of the gathered operands."""
        src_parts = schedule_args.get('num_src_partitions', 'auto')
        if src_parts is None:
            return 1
        if src_parts == 'auto':
            return tuning._partitions(self._num_cols, slice_row_bytes, self._indices.shape[0], self._num_rows,
                                      tuning.SPMM_SLICE_BYTES, min_segment=24)
        if int(src_parts) < 1:
            raise ValueError("num_src_partitions must be >= 1")
        return int(src_parts)

    def _build_additive(self, input_placeholders, compute_args, schedule_args):
        schedule_args = common.take_args(schedule_args or {}, ('num_src_partitions', 'num_dst_partitions'), "schedule_func")
        if len(input_placeholders) != 3:
            raise ValueError("additive attention takes three inputs (Er, El, V), got %d" % len(input_placeholders))
        er_ph, el_ph, v_ph = input_placeholders
        if len(v_ph.shape) != 3 or v_ph.shape[0] != self._num_cols:
            raise ValueError("V must be (num_cols=%d, H, D), got %s" % (self._num_cols, v_ph.shape))
        heads, head_len = int(v_ph.shape[1]), int(v_ph.shape[2])
        if tuple(er_ph.shape) != (self._num_rows, heads) or tuple(el_ph.shape) != (self._num_cols, heads):
            raise ValueError("Er must be (num_rows=%d, %d) and El (num_cols=%d, %d), got %s and %s"
                             % (self._num_rows, heads, self._num_cols, heads, er_ph.shape, el_ph.shape))
        if head_len not in (16, 32, 64):
            raise ValueError("heads of 16, 32 or 64 floats, got %d" % head_len)
        self._heads, self._head_len = heads, head_len
        self._slope = float(compute_args.get('negative_slope', 0.2))
        self._scale = 1.0
        t_parts = schedule_args.get('num_dst_partitions')
        self._t_parts = None if t_parts in (None, 'auto') else int(t_parts)
        self._active = self._layout(self._partitions(schedule_args, 4 * head_len))
        common.reserve(self._active['plan'], common.OP_ATTENTION_ADDITIVE, heads, head_len, 0, self._ctx)
        self._placeholders = [er_ph, el_ph, v_ph]
        self.out_tvm = torch.zeros((self._num_rows, heads, head_len), dtype=torch.float32, device=self._ctx)
        self.state_tvm = torch.zeros((self._num_rows, heads, 2), dtype=torch.float32, device=self._ctx)
        self._coef = None

    def _launch_additive(self, er, el, v):
        lay = self._active
        self._er_t, self._el_t = er.t().contiguous(), el.t().contiguous()      # head by head
        _lib.check(_lib.lib().fg_graph_attention_additive_f32(
            lay['plan'], _lib.dev_ptr(lay['pos']), _lib.dev_ptr(lay['idx']), _lib.dev_ptr(self._er_t),
            _lib.dev_ptr(self._el_t), _lib.dev_ptr(v), _lib.dev_ptr(self.out_tvm), _lib.dev_ptr(self.state_tvm),
            self._heads, self._head_len, ctypes.c_float(self._slope), common.stream_ptr()))

    def _launch(self, q, k, v):
        if self._additive:
            return self._launch_additive(q, k, v)
        lay = self._active
        _lib.check(_lib.lib().fg_graph_attention_f32(lay['plan'], _lib.dev_ptr(lay['pos']), _lib.dev_ptr(lay['idx']),
                                                     _lib.dev_ptr(q), _lib.dev_ptr(k), _lib.dev_ptr(v),
                                                     _lib.dev_ptr(self.out_tvm), _lib.dev_ptr(self.state_tvm),
                                                     self._heads, self._head_len,
                                                     ctypes.c_float(self._scale), common.stream_ptr()))

    def run(self, input_tvm_ndarrays):
        """[Q, K, V] -> self.out_tvm (the same tensor on every call); nothing is synchronised."""
        if self._placeholders is None:
            raise RuntimeError("call build() before run()")
        common.ensure_output(self)
        common.check_inputs(input_tvm_ndarrays, self._placeholders, self._ctx)
        self._launch(*input_tvm_ndarrays)
        return self.out_tvm

    def _layout_t(self, P):
        """The transposed adjacency (rows = sources) with P partitions over the destinations."""
        key = ('t', P)
        if key in self._layouts:
            return self._layouts[key]
        tr = self._csr.T.tocsr()
        tr.sort_indices()
        if P > 1:
            pos, idx, _ = util_convert_csr_to_dds(tr, P)
        else:
            pos, idx = tr.indptr, tr.indices
        pos = np.ascontiguousarray(pos, dtype=np.int32)
        lay = {'P': P, 'pos': common.to_device_i32(pos, self._ctx),
               'idx': common.to_device_i32(np.ascontiguousarray(idx, dtype=np.int32), self._ctx), 'plan': ctypes.c_void_p()}
        base = _lib.plan_opts
        opts = _lib.FgPlanOpts(split_threshold=_INT32_MAX, item_edges=base.item_edges if base is not None else 0,
                               wide_offsets=0, tile_major=base.tile_major if base is not None else 0)
        with torch.cuda.device(self._ctx):
            _lib.check(_lib.lib().fg_spmm_plan_create(_lib.host_ptr(pos), self._num_cols, self._num_rows, P,
                                                      ctypes.byref(opts), ctypes.byref(lay['plan'])))
        common.narrow_indices(lay['plan'], lay['idx'], self._num_rows, P, self._ctx)      # the transposed graph gathers from the rows
        self._layouts[key] = lay
        return lay

    def backward(self, q, k, v, out, state, grad_out):
        """(dQ, dK, dV) for dL/d(out) = grad_out, given the inputs, the output and the row state
        (out_tvm / state_tvm as they were after run() on these inputs).  The scores are formed again from Q
        and K; dQ comes from a sweep like the forward pass, dK and dV from the same sweep over the
        transposed adjacency.  Returns new tensors."""
        if self._placeholders is None:
            raise RuntimeError("call build() before backward()")
        common.check_inputs([q, k, v], self._placeholders, self._ctx)
        if self._additive:
            return self._backward_additive(q, k, v, out, state, grad_out)
        common.check_inputs([out, grad_out], [self._placeholders[0]] * 2, self._ctx)
        L, s = _lib.lib(), common.stream_ptr()
        coef = torch.empty_like(state)
        _lib.check(L.fg_graph_attention_coef_f32(_lib.dev_ptr(out), _lib.dev_ptr(grad_out), _lib.dev_ptr(state),
                                                 _lib.dev_ptr(coef), self._num_rows, self._heads, self._head_len, s))
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        lay = self._active
        _lib.check(L.fg_graph_attention_backward_q_f32(lay['plan'], _lib.dev_ptr(lay['pos']), _lib.dev_ptr(lay['idx']),
                                                       _lib.dev_ptr(q), _lib.dev_ptr(k), _lib.dev_ptr(v),
                                                       _lib.dev_ptr(grad_out), _lib.dev_ptr(coef), _lib.dev_ptr(dq),
                                                       self._heads, self._head_len, ctypes.c_float(self._scale), s))
        # partitions over the destinations, sized like the forward pass's over the sources
        lt = self._layout_t(self._dst_partitions(2 * 4 * self._head_len))
        _lib.check(L.fg_graph_attention_backward_kv_f32(lt['plan'], _lib.dev_ptr(lt['pos']), _lib.dev_ptr(lt['idx']),
                                                        _lib.dev_ptr(q), _lib.dev_ptr(grad_out), _lib.dev_ptr(k),
                                                        _lib.dev_ptr(v), _lib.dev_ptr(coef), _lib.dev_ptr(dk),
                                                        _lib.dev_ptr(dv), self._heads, self._head_len,
                                                        ctypes.c_float(self._scale), s))
        self._coef = coef
        return dq, dk, dv

    def _dst_partitions(self, slice_row_bytes):
        if self._t_parts is not None:
            return self._t_parts
        if self._active['P'] == 1:
            return 1
        return max(1, tuning._partitions(self._num_rows, slice_row_bytes, self._indices.shape[0], self._num_cols,
                                         tuning.SPMM_SLICE_BYTES, min_segment=24))

    def _backward_additive(self, er, el, v, out, state, grad_out):
        """(dEr, dEl, dV) of the additive-score operator."""
        out_ph = common.placeholder((self._num_rows, self._heads, self._head_len))
        common.check_inputs([out, grad_out], [out_ph] * 2, self._ctx)
        L, s = _lib.lib(), common.stream_ptr()
        H, D = self._heads, self._head_len
        er_t, el_t = er.t().contiguous(), el.t().contiguous()
        coef = torch.empty((H, self._num_rows, 4), dtype=torch.float32, device=self._ctx)
        _lib.check(L.fg_graph_attention_additive_coef_f32(_lib.dev_ptr(out), _lib.dev_ptr(grad_out), _lib.dev_ptr(state),
                                                          _lib.dev_ptr(er_t), _lib.dev_ptr(coef), self._num_rows, H, D, s))
        der_t = torch.empty_like(er_t)
        del_t = torch.empty_like(el_t)
        dv = torch.empty_like(v)
        lay = self._active
        _lib.check(L.fg_graph_attention_additive_backward_er_f32(
            lay['plan'], _lib.dev_ptr(lay['pos']), _lib.dev_ptr(lay['idx']), _lib.dev_ptr(el_t), _lib.dev_ptr(v),
            _lib.dev_ptr(grad_out), _lib.dev_ptr(coef), _lib.dev_ptr(der_t), H, D, ctypes.c_float(self._slope), s))
        lt = self._layout_t(self._dst_partitions(4 * D))
        _lib.check(L.fg_graph_attention_additive_backward_elv_f32(
            lt['plan'], _lib.dev_ptr(lt['pos']), _lib.dev_ptr(lt['idx']), _lib.dev_ptr(grad_out), _lib.dev_ptr(el_t),
            _lib.dev_ptr(v), _lib.dev_ptr(coef), _lib.dev_ptr(del_t), _lib.dev_ptr(dv), H, D,
            ctypes.c_float(self._slope), s))
        self._coef = coef
        return der_t.t().contiguous(), del_t.t().contiguous(), dv

    def measure_average_time(self, input_tvm_ndarrays, num_runs):
        if self._placeholders is None:
            raise RuntimeError("call build() before measure_average_time()")
        common.ensure_output(self)
        common.check_inputs(input_tvm_ndarrays, self._placeholders, self._ctx)
        q, k, v = input_tvm_ndarrays
        return common.timed_mean_seconds(lambda: self._launch(q, k, v), num_runs)

    @property
    def ctx(self):
        return self._ctx

    @property
    def target(self):
        return self._target
