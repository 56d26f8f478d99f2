"""Generalised SpMM: aggregation by sum / mean / max / min, with one weight per edge, one weight
per edge and head, or none.  The reference snapshot has no such operator (its README.md:9-11
points to a branch with "generalized SpMM"); the class follows the build()/run() conventions of
the reference's SpMM modules (python/featgraph/module/spmm.py:81-161)."""
import ctypes

import numpy as np
import scipy.sparse
import torch

from .. import _lib
from ..util import util_convert_csr_to_dds
from .. import tuning
from . import common
from . import general
from .spmm import VanillaSpMMhip

_REDUCE = {'sum': 0, 'mean': 0, 'max': 1, 'min': 2}


class GSpMMhip(VanillaSpMMhip):
    """out[v, h, :] = reduce_{e in row v} w[e, h] * SrcFeat[indices[e], h, :].

    compute_args: 'reduce' in {'sum', 'mean', 'max', 'min'} (default 'sum'); 'msg' in
    {'u_mul_e', 'copy_u'} (default 'u_mul_e': the adjacency values, or the edge weights given
    to run(); 'copy_u': weight 1); 'num_feat_partitions' as for VanillaSpMMhip.
    SrcFeat is (num_cols, F) or (num_cols, H, D); with H > 1 the weights are (nnz, H) and must
    be passed to run() as a second input, in the adjacency's CSR edge order.
    Rows without edges give 0 for every reduce.
    'return_arg': True (max / min only) also fills self.arg_tvm, int32 of out's shape: the position, in
    the adjacency's CSR edge order, of the edge whose message was selected (-1 for rows without edges).

    Any other message goes to the library's broadcasting kernel: 'msg' = '<lhs>_<op>_<rhs>' with
    lhs, rhs in {'u', 'e'} and op in {'add', 'sub', 'mul', 'div'}, or 'copy_e'; the inputs are the two
    operands in that order ('u': (num_cols, ...), 'e': (nnz, ...) in CSR edge order), whose feature shapes
    broadcast against each other the numpy way, e.g. 'u_mul_e' with (num_cols, H, D) and (nnz, H, 1), or
    'u_add_e' with (num_cols, F) and (nnz, F).  out[v] = reduce over row v's edges of the message; out
    has the broadcast feature shape.  (With 'u_mul_e', a second input of shape (nnz,) or (nnz, H) keeps
    its meaning of one weight per edge, or per edge and head; compute_args {'broadcast': True} makes every message
    follow numpy broadcasting instead, as DGL's gspmm does -- the two readings differ only for SrcFeat (num_cols, H, D)
    with D == H and a second input (nnz, H).)  schedule_args {'num_src_partitions': 'auto' | int |
    None} cuts the source columns into partitions as for the weighted sum (default 'auto': chosen from the size of the
    operand that is gathered from the source nodes); operands on the edges and the reported positions stay in CSR order.
    """
    _compute_keys = ('num_feat_partitions', 'reduce', 'msg', 'return_arg', 'broadcast')

    def build(self, input_placeholders, compute_args, schedule_args):
        compute_args = dict(compute_args)
        reduce = compute_args.pop('reduce', 'sum')
        msg = compute_args.pop('msg', 'u_mul_e')
        return_arg = bool(compute_args.pop('return_arg', False))
        force = bool(compute_args.pop('broadcast', False))
        if return_arg and reduce not in ('max', 'min'):
            raise ValueError("return_arg is defined for reduce='max' / 'min' only")
        if reduce not in _REDUCE:
            raise ValueError("reduce must be one of %s" % sorted(_REDUCE))
        self._bop = None
        if self._is_broadcast_message(msg, input_placeholders, reduce, force):
            return self._build_broadcast(input_placeholders, compute_args, schedule_args, msg, reduce, return_arg)
        if len(input_placeholders) not in (1, 2):
            raise ValueError("GSpMM takes SrcFeat and optionally the edge weights")
        src_ph = input_placeholders[0]
        if len(src_ph.shape) not in (2, 3) or src_ph.shape[0] != self._num_cols:
            raise ValueError("SrcFeat must be (num_cols=%d, F) or (num_cols, H, D), got %s" % (self._num_cols, src_ph.shape))
        heads = src_ph.shape[1] if len(src_ph.shape) == 3 else 1
        feat_len = int(np.prod(src_ph.shape[1:]))
        nnz = self._adj_indices.shape[0]
        weights_at_run = len(input_placeholders) == 2
        if weights_at_run:
            want = (nnz,) if heads == 1 else (nnz, heads)
            if tuple(input_placeholders[1].shape) not in (want, (nnz, heads)):
                raise ValueError("edge weights must have shape %s, got %s" % (want, input_placeholders[1].shape))
            if msg == 'copy_u':
                raise ValueError("msg='copy_u' takes no edge weights")
        elif heads > 1 and msg == 'u_mul_e':
            raise ValueError("per-head weights (nnz, H) must be passed to run() as a second input")
        if reduce in ('max', 'min'):
            schedule_args = dict(schedule_args, num_src_partitions=None)
            if self._num_col_partitions != 1:
                raise ValueError("max / min aggregation needs num_col_partitions == 1")
        # rows of an awkward length run at the next friendly one, on zero-padded copies (tuning.padded_feature_len)
        self._pad_from = None
        if heads == 1 and len(src_ph.shape) == 2 and not return_arg and schedule_args.get('pad_features', True) \
                and not compute_args.get('num_feat_partitions'):
            want = tuning.padded_feature_len(feat_len)
            if want != feat_len and nnz * feat_len >= tuning.PAD_MIN_GATHERED:
                self._pad_from, feat_len = feat_len, want
        elif heads > 1 and not return_arg and not compute_args.get('num_feat_partitions'):
            # several heads: a head length the kernels have no tile for is padded to the next one they have
            D0 = feat_len // heads
            want = tuning.padded_head_len(D0)
            if want != D0:
                self._pad_from, feat_len = D0, heads * want
        schedule_args = {k: v for k, v in schedule_args.items() if k != 'pad_features'}
        flat = common.placeholder((self._num_cols, feat_len))
        _, _, T, P, notes = self._resolve([flat], compute_args, schedule_args)
        if self._pad_from is not None:
            notes.append("rows (heads) of %d floats run as rows of %d on zero-padded copies" % (self._pad_from, feat_len // heads))
        self._placeholders = list(input_placeholders)
        self._feat_len, self._heads, self._num_feat_partitions = feat_len, heads, (0 if heads > 1 and 'num_feat_partitions' not in compute_args else T)
        self._reduce, self._msg, self._weights_at_run, self._notes = reduce, msg, weights_at_run, notes
        self._active = self._glayout(P)
        self._func = _lib.lib().fg_gspmm_f32
        common.reserve(self._active['plan'], common.OP_SPMM_SUM if _REDUCE[reduce] == 0 else common.OP_SPMM_EXTREME,
                       heads, feat_len // heads, self._num_feat_partitions, self._ctx)
        self._return_arg = return_arg
        self._inv_deg_edge = None
        self._w_head_major = None
        self._w_static = None
        if reduce == 'mean':
            deg = np.diff(self._adj_indptr).astype(np.float32)
            inv = np.where(deg > 0, 1.0 / np.maximum(deg, 1), 0).astype(np.float32)
            self._inv_deg_edge = common.to_device_f32(np.repeat(inv, np.diff(self._adj_indptr)), self._ctx)
        self._x_pad = self._out_pad = None
        if self._pad_from is not None:
            tail = (feat_len,) if heads == 1 else (heads, feat_len // heads)
            self._x_pad = torch.zeros((self._num_cols,) + tail, dtype=torch.float32, device=self._ctx)
            self._out_pad = torch.zeros((self._num_rows,) + tail, dtype=torch.float32, device=self._ctx)
        self.out_tvm = torch.zeros((self._num_rows,) + tuple(src_ph.shape[1:]), dtype=torch.float32, device=self._ctx)
        self.arg_tvm = torch.full(self.out_tvm.shape, -1, dtype=torch.int32, device=self._ctx) if return_arg else None
        if not weights_at_run:
            self._weights(None)          # the adjacency's own values, laid out for the kernel now: run() uploads nothing

    def _is_broadcast_message(self, msg, input_placeholders, reduce='sum', force=False):
        if msg not in ('u_mul_e', 'copy_u'):
            return True
        if force and len(input_placeholders) == 2:
            # numpy broadcasting throughout; what the weighted-sum kernels also compute stays with them
            src_ph, e_ph = input_placeholders
            nnz = self._adj_indices.shape[0]
            one_weight = tuple(e_ph.shape) == (nnz,) and len(src_ph.shape) == 2
            if not (msg == 'u_mul_e' and reduce in ('sum', 'mean') and one_weight):
                return True
        if reduce in ('max', 'min') and self._num_col_partitions == 1:
            # the broadcasting kernel takes source partitions and finds the selected elements in the same sweep
            # (232,965-node graph, F=64: 2.0 ms against 3.0 ms, 4.1 against 6.1 ms with the positions)
            if msg == 'copy_u' and len(input_placeholders) == 1:
                return True
            if msg == 'u_mul_e' and len(input_placeholders) == 2 and len(input_placeholders[0].shape) == 2 \
                    and tuple(input_placeholders[1].shape) == (self._adj_indices.shape[0],):
                return True                   # one weight per edge, given to run()
            if msg == 'u_mul_e' and len(input_placeholders) == 1 and len(input_placeholders[0].shape) == 2:
                return True                   # ... or the adjacency's own values
        if len(input_placeholders) >= 1 and len(input_placeholders[0].shape) not in (2, 3):
            return True                   # the weighted-sum kernels take (num_cols, F) or (num_cols, H, D)
        if msg == 'u_mul_e' and len(input_placeholders) == 2:
            src_ph, e_ph = input_placeholders
            heads = src_ph.shape[1] if len(src_ph.shape) == 3 else 1
            nnz = self._adj_indices.shape[0]
            return tuple(e_ph.shape) != ((nnz,) if heads == 1 else (nnz, heads))
        return False

    def _build_broadcast(self, input_placeholders, compute_args, schedule_args, msg, reduce, return_arg):
        """Messages with vector edge features or broadcasting between the operands."""
        common.take_args(compute_args, self._compute_keys, "compute_func")
        common.take_args(schedule_args, self._schedule_keys, "schedule_func")
        op, lt, rt = general.parse_message(msg)
        nnz = self._adj_indices.shape[0]
        self._pad_from = None
        # 'u_mul_e' with SrcFeat alone: the adjacency's own values are the edge operand (CSR order, already on the device)
        self._static_rhs = None
        if msg == 'u_mul_e' and len(input_placeholders) == 1:
            self._static_rhs = self._layout(1)['vals']
            input_placeholders = [input_placeholders[0], common.placeholder((nnz,))]
        if len(input_placeholders) != (1 if rt is None else 2):
            raise ValueError("message %r takes %d input(s), got %d" % (msg, 1 if rt is None else 2, len(input_placeholders)))
        lhs_ph = input_placeholders[0]
        rhs_ph = input_placeholders[1] if rt is not None else None
        self._bop = general.BroadcastOp(op, lt, rt, lhs_ph, rhs_ph, self._num_rows, self._num_cols, nnz, self._ctx, allow_v=False)
        self._placeholders = list(input_placeholders[:1] if self._static_rhs is not None else input_placeholders)
        self._feat_len, self._heads, self._num_feat_partitions = self._bop.out_len, 1, 0
        self._reduce, self._msg, self._return_arg = reduce, msg, return_arg
        self._notes = [self._bop.describe()]
        P = self._broadcast_partitions(schedule_args, return_arg)
        if P > 1:
            self._notes.append("%d source-column partitions, one buffer of results each, combined in partition order" % P)
        if compute_args.get('num_feat_partitions') or any(k != 'num_src_partitions' for k in schedule_args):
            self._notes.append("the feature axis of this message is not tiled; tiling knobs ignored")
        self._active = self._glayout(P)
        self._func = _lib.lib().fg_gspmm_bcast_dds_f32 if P > 1 else _lib.lib().fg_gspmm_bcast_f32
        common.reserve(self._active['plan'], common.OP_GSPMM_BCAST_ARG if return_arg else common.OP_GSPMM_BCAST,
                       1, self._bop.out_len, 0, self._ctx)
        self._row_scale = None
        if reduce == 'mean':
            deg = np.diff(self._adj_indptr).astype(np.float32)
            self._row_scale = common.to_device_f32(np.where(deg > 0, 1.0 / np.maximum(deg, 1), 0), self._ctx)
        self.out_tvm = torch.zeros((self._num_rows,) + self._bop.out_shape, dtype=torch.float32, device=self._ctx)
        self.arg_tvm = torch.full(self.out_tvm.shape, -1, dtype=torch.int32, device=self._ctx) if return_arg else None

    def _broadcast_partitions(self, schedule_args, return_arg):
        """Source-column partitions of a broadcasting message: the constructor's count when it was given, else
        schedule_args['num_src_partitions'] ('auto', the default: chosen for the operand gathered from the source
        nodes, if there is one; None: the CSR arrays as they are)."""
        if self._num_col_partitions != 1:
            return self._num_col_partitions
        want = schedule_args.get('num_src_partitions', 'auto')
        if want is None:
            return 1
        if want != 'auto':
            if int(want) < 1:
                raise ValueError("num_src_partitions must be >= 1")
            return int(want)
        bop = self._bop
        if bop.gathered_len() == 0:
            return 1
        return tuning.choose_gather_partitions(self._num_rows, self._num_cols, self._adj_indices.shape[0], bop.gathered_len(),
                                               bop.out_len * (2 if return_arg else 1), self._graph_stats(), bop.feature_tiles(return_arg))

    def _launch_broadcast(self, inputs):
        lay = self._active
        lhs = inputs[0]
        rhs = inputs[1] if len(inputs) > 1 else self._static_rhs
        # where each element of the layout lies in the edge operands (None: at its own position); the adjacency's own
        # values are in CSR order whatever order was announced for operands given to run()
        own = len(inputs) == 1 and self._static_rhs is not None
        pos = (lay['edge_pos32'] if lay['P'] > 1 else None) if own else self._given_pos(lay)
        self._bop.run_spmm(lay['plan'], lay['pos'], lay['idx'], _REDUCE[self._reduce], lhs, rhs, self._row_scale,
                           self.out_tvm, self.arg_tvm, edge_pos_dev=pos)

    def lower_to_ir(self, input_placeholders, compute_args, schedule_args):
        compute_args = dict(compute_args)
        msg = compute_args.get('msg', 'u_mul_e')
        if self._is_broadcast_message(msg, input_placeholders, compute_args.get('reduce', 'sum'), bool(compute_args.get('broadcast'))):
            op, lt, rt = general.parse_message(msg)
            nnz = self._adj_indices.shape[0]
            if msg == 'u_mul_e' and len(input_placeholders) == 1:
                input_placeholders = [input_placeholders[0], common.placeholder((nnz,))]       # the adjacency's own values
            bop = general.BroadcastOp(op, lt, rt, input_placeholders[0], input_placeholders[1] if rt is not None else None,
                                      self._num_rows, self._num_cols, nnz, self._ctx, allow_v=False)
            self._bop, keep = bop, self._bop
            try:
                P = self._broadcast_partitions(common.take_args(schedule_args, self._schedule_keys, "schedule_func"),
                                               bool(compute_args.get('return_arg', False)))
            finally:
                self._bop = keep
            buf = ctypes.create_string_buffer(4096)
            _lib.check(_lib.lib().fg_spmm_plan_describe(self._layout(P)['plan'], 0, 0, buf, len(buf)))
            return buf.value.decode() + "  kernel           : gspmm_bcast_kernel, one wavefront per work item\n  note             : %s\n" % bop.describe()
        for k in ('reduce', 'msg', 'return_arg', 'broadcast'):
            compute_args.pop(k, None)
        flat = common.placeholder((self._num_cols, int(np.prod(input_placeholders[0].shape[1:]))))
        return super(GSpMMhip, self).lower_to_ir([flat], compute_args, schedule_args)

    def _glayout(self, P):
        """Layout for P source partitions plus, for P > 1, each DDS element's CSR position (so that
        weights given in CSR order can be brought into DDS order on the device)."""
        lay = self._layout(P)
        if P > 1 and 'edge_pos32' not in lay:
            nnz = self._adj_indices.shape[0]
            csr = scipy.sparse.csr_matrix((np.arange(nnz, dtype=np.int32), self._adj_indices, self._adj_indptr),
                                          shape=(self._num_rows, self._num_cols))
            _, _, edge_pos = util_convert_csr_to_dds(csr, P)
            lay['edge_pos32'] = torch.from_numpy(edge_pos.astype(np.int32)).to(self._ctx)
        return lay

    def _weights(self, given):
        """(device weights in the active layout's element order or None for weight 1, head-major flag).
        One weight per edge: a 1-D array in element order.  One weight per edge and head: the
        library's relayout kernel writes them head-major (each head contiguous) in element order."""
        lay = self._active
        if given is None and self._w_static is not None:
            return self._w_static          # the adjacency's own values: laid out once per build
        if self._msg == 'copy_u':
            w = None
        elif given is not None:
            w = given.reshape(given.shape[0], -1)
        else:
            w = self._layouts[1]['vals'].reshape(-1, 1) if 1 in self._layouts else None
            if w is None:
                w = common.to_device_f32(self._adj_scipy_csr.data, self._ctx).reshape(-1, 1)
        if self._inv_deg_edge is not None:
            if given is not None and getattr(self, '_weight_perm', None) is not None:
                raise ValueError("reduce='mean' with weights in another edge order is not supported")
            w = self._inv_deg_edge.reshape(-1, 1) if w is None else w * self._inv_deg_edge.reshape(-1, 1)
        if w is None:
            return None, 0
        if given is None:
            self._w_static = self._weights_in_layout(w, lay)
            if self._w_static[0] is self._w_head_major:
                self._w_head_major = None          # kept; weights given to later runs get a buffer of their own
            return self._w_static
        return self._weights_in_layout(w, lay, given=True)

    def set_weight_order(self, position_of_edge):
        """Weights and edge operands given to run() are stored in another edge order: position_of_edge[i] is
        where the weight (or operand row) of this adjacency's i-th edge (CSR order) lies in the given array (int
        array of nnz entries, or None for CSR order).  The library's relayout kernel, or the broadcasting kernel's
        own addressing, follows it: no separate permutation pass.  Positions reported by 'return_arg' then refer
        to the given order too (broadcasting messages)."""
        if position_of_edge is None:
            self._weight_perm = None
        else:
            perm = torch.as_tensor(position_of_edge, device=self._ctx).to(torch.int32).contiguous()
            if perm.shape != (self._adj_indices.shape[0],):
                raise ValueError("position_of_edge must have nnz = %d entries" % self._adj_indices.shape[0])
            self._weight_perm = perm
        self._perm_pos = {}

    def _given_pos(self, lay):
        """Element of the active layout -> position in the array given to run() (None: identity)."""
        perm = getattr(self, '_weight_perm', None)
        pos = lay['edge_pos32'] if lay['P'] > 1 else None
        if perm is None:
            return pos
        if pos is None:
            return perm
        cache = self.__dict__.setdefault('_perm_pos', {})
        if lay['P'] not in cache:
            cache[lay['P']] = perm[pos.long()].contiguous()
        return cache[lay['P']]

    def _weights_in_layout(self, w, lay, given=False):
        pos = self._given_pos(lay) if given else (lay['edge_pos32'] if lay['P'] > 1 else None)
        if w.shape[1] > 1 or pos is not None:
            w = w.contiguous()
            if self._w_head_major is None or self._w_head_major.shape != (w.shape[1], w.shape[0]):
                self._w_head_major = torch.empty((w.shape[1], w.shape[0]), dtype=torch.float32, device=self._ctx)
            _lib.check(_lib.lib().fg_edge_values_head_major_f32(_lib.dev_ptr(w), _lib.dev_ptr(pos), w.shape[0],
                                                                w.shape[1], _lib.dev_ptr(self._w_head_major),
                                                                common.stream_ptr()))
            return self._w_head_major, 1
        return w.contiguous(), 0

    def _launch(self, src_feat, weights=None):
        lay = self._active
        w, head_major = self._weights(weights)
        heads = w.shape[0] if head_major else 1
        self._w_keepalive = w
        if self._return_arg:
            _lib.check(_lib.lib().fg_gspmm_arg_f32(lay['plan'], _lib.dev_ptr(lay['pos']), _lib.dev_ptr(lay['idx']),
                                                   _lib.dev_ptr(w), _lib.dev_ptr(src_feat), _lib.dev_ptr(self.out_tvm),
                                                   _lib.dev_ptr(self.arg_tvm), self._feat_len, heads, head_major,
                                                   _REDUCE[self._reduce], self._num_feat_partitions, common.stream_ptr()))
            return
        out = self.out_tvm
        if getattr(self, '_pad_from', None) is not None:
            self._x_pad[..., :self._pad_from].copy_(src_feat)       # the padding columns stay zero
            src_feat, out = self._x_pad, self._out_pad
        _lib.check(self._func(lay['plan'], _lib.dev_ptr(lay['pos']), _lib.dev_ptr(lay['idx']), _lib.dev_ptr(w),
                              _lib.dev_ptr(src_feat), _lib.dev_ptr(out), self._feat_len, heads, head_major,
                              _REDUCE[self._reduce], self._num_feat_partitions, common.stream_ptr()))
        if out is not self.out_tvm:
            self.out_tvm.copy_(out[..., :self._pad_from])

    def run(self, input_tvm_ndarrays):
        """[SrcFeat] or [SrcFeat, edge_weights]; returns self.out_tvm (overwritten in place)."""
        if self._func is None:
            raise RuntimeError("call build() before run()")
        common.ensure_output(self)
        common.check_inputs(input_tvm_ndarrays, self._placeholders, self._ctx)
        if self._bop is not None:
            self._launch_broadcast(input_tvm_ndarrays)
        else:
            self._launch(input_tvm_ndarrays[0], input_tvm_ndarrays[1] if self._weights_at_run else None)
        return self.out_tvm

    def measure_average_time(self, input_tvm_ndarrays, num_runs):
        if self._func is None:
            raise RuntimeError("call build() before measure_average_time()")
        common.ensure_output(self)
        common.check_inputs(input_tvm_ndarrays, self._placeholders, self._ctx)
        if self._bop is not None:
            return common.timed_mean_seconds(lambda: self._launch_broadcast(input_tvm_ndarrays), num_runs)
        x = input_tvm_ndarrays[0]
        w = input_tvm_ndarrays[1] if self._weights_at_run else None
        return common.timed_mean_seconds(lambda: self._launch(x, w), num_runs)
