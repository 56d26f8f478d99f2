"""Differentiable SpMM / SDDMM / edge softmax built from the forward kernels.

The backward passes are the same two operators on the transposed graph:
  y = A(w) x            dx = A(w)^T dy          dw[e] = <dy[row e], x[col e]>       (an SDDMM)
  s[e] = <src[col e], dst[row e]>    ddst = A(ds) src    dsrc = A(ds)^T dst         (two SpMMs)
(with heads: x, src, dst are (n, H, D), w and s are (nnz, H), and every identity holds per head);
  a = edge_softmax(s)   ds = a * (da - sum over the row of a * da)
so `Graph` keeps plans for the adjacency in CSR order and for its transpose, and the permutation
between the two edge orders.  The reference has no autograd layer; this is the consumer-side API
its README (README.md:13-14, DGL integration) points at.
"""
import numpy as np
import scipy.sparse
import torch

from .module import (EdgeSoftmaxhip, GraphAttentionhip, GSDDMMhip, GSpMMhip, MultiHeadSDDMMhip, VanillaSDDMMhip,
                     placeholder)
from .module.general import parse_message


class Graph(object):
    """Structure of one adjacency (rows = destinations, columns = sources) for differentiable ops.

    Edge weights and edge outputs are (nnz,) tensors, or (nnz, H) with heads, in the adjacency's CSR
    edge order.
    """

    def __init__(self, adj_scipy):
        csr = adj_scipy.tocsr().astype(np.float32)
        csr.sort_indices()
        self.shape = csr.shape
        self.nnz = csr.nnz
        pos = scipy.sparse.csr_matrix((np.arange(1, csr.nnz + 1, dtype=np.int64), csr.indices, csr.indptr),
                                      shape=csr.shape)
        tr = pos.T.tocsr()
        tr.sort_indices()
        self._csr = csr
        self._tr = scipy.sparse.csr_matrix((np.ones(csr.nnz, np.float32), tr.indices.astype(np.int32),
                                            tr.indptr.astype(np.int32)), shape=tr.shape)
        self._tr_pos_host = (tr.data - 1).astype(np.int64)      # transposed edge order -> CSR position
        self._mods = {}
        # the first SpMM-like module of each orientation owns the device layouts (partitioned copies of the adjacency, plans,
        # scratch); later ones of the same orientation use them too: every operator of a Graph runs on the caller's one
        # stream, one after the other, so one scratch per orientation is enough
        self._layout_owner = {}

    def _gspmm_module(self, transposed):
        m = GSpMMhip(self._tr if transposed else self._csr)
        owner = self._layout_owner.get(transposed)
        if owner is None:
            self._layout_owner[transposed] = m
        else:
            m.share_layouts_with(owner)
        return m

    def _spmm_mod(self, transposed, tail, w_heads):
        key = ('spmm', transposed, tail, w_heads)
        if key not in self._mods:
            adj = self._tr if transposed else self._csr
            m = self._gspmm_module(transposed)
            w_shape = (self.nnz,) if w_heads == 0 else (self.nnz, w_heads)
            m.build([placeholder((adj.shape[1],) + tail), placeholder(w_shape)], {}, {})
            if transposed:
                m.set_weight_order(self._tr_pos_host)      # weights arrive in this graph's CSR edge order
            self._mods[key] = m
        return self._mods[key]

    def _sddmm_mod(self, tail):
        key = ('sddmm', tail)
        if key not in self._mods:
            m = (MultiHeadSDDMMhip if len(tail) == 2 else VanillaSDDMMhip)(self._csr)
            # one partitioned copy of the adjacency, one plan and one scratch with a forward SpMM module, if there is one
            # (every operator of a Graph runs on the caller's one stream, one after the other)
            for k, other in self._mods.items():
                if k[0] == 'spmm' and not k[1]:
                    m.share_layouts(other)
                    break
            m.build([placeholder((self.shape[1],) + tail), placeholder((self.shape[0],) + tail)], {}, {})
            self._mods[key] = m
        return self._mods[key]

    def _softmax_mod(self, shape):
        key = ('softmax', shape)
        if key not in self._mods:
            m = EdgeSoftmaxhip(self._csr)
            m.build([placeholder(shape)])
            self._mods[key] = m
        return self._mods[key]

    # raw (non-differentiable) building blocks; each returns a fresh tensor
    def _spmm_raw(self, x, w, transposed=False):
        x = x.contiguous()
        if x.dim() == 3 and (w.dim() != 2 or w.shape[1] != x.shape[1]):
            raise ValueError("with x of shape (n, H, D) the weights must be (nnz, H)")
        if x.dim() == 2 and w.dim() != 1:
            raise ValueError("with x of shape (n, F) the weights must be (nnz,)")
        mod = self._spmm_mod(transposed, tuple(x.shape[1:]), 0 if w.dim() == 1 else w.shape[1])
        return _fresh_run(mod, [x, w.contiguous()])

    def _sddmm_raw(self, src, dst):
        return _fresh_run(self._sddmm_mod(tuple(src.shape[1:])), [src.contiguous(), dst.contiguous()])

    def spmm(self, x, w):
        """y[v,:] = sum_e w[e] x[col e,:]; x (num_cols, F) with w (nnz,), or x (num_cols, H, D) with
        w (nnz, H); differentiable in both."""
        return _SpMM.apply(self, x, w)

    def sddmm(self, src, dst):
        """s[e] = <src[col e,:], dst[row e,:]>; src (num_cols, F), dst (num_rows, F) -> (nnz,), or
        (n, H, D) operands -> (nnz, H)."""
        return _SDDMM.apply(self, src, dst)

    def aggregate(self, x, reduce="sum"):
        """y[v,:] = reduce over the edges e into v of x[col e,:], reduce in {'sum', 'mean', 'max', 'min'}
        (rows without edges give 0); x (num_cols, F); differentiable in x."""
        if reduce not in ("sum", "mean", "max", "min"):
            raise ValueError("reduce must be 'sum', 'mean', 'max' or 'min'")
        return _Aggregate.apply(self, x, reduce)

    def _aggregate_mod(self, feat_len, reduce):
        key = ('aggregate', feat_len, reduce)
        if key not in self._mods:
            m = self._gspmm_module(False)
            args = {'reduce': reduce, 'msg': 'copy_u'}
            if reduce in ('max', 'min'):
                args['return_arg'] = True
            m.build([placeholder((self.shape[1], feat_len))], args, {})
            self._mods[key] = m
        return self._mods[key]

    def _mean_weights(self, device):
        if getattr(self, "_inv_deg", None) is None or self._inv_deg.device != device:
            deg = np.diff(self._csr.indptr).astype(np.float32)
            inv = np.where(deg > 0, 1.0 / np.maximum(deg, 1), 0).astype(np.float32)
            self._inv_deg = torch.from_numpy(np.repeat(inv, np.diff(self._csr.indptr))).to(device)
            self._ones = torch.ones(self.nnz, device=device)
            self._cols = torch.from_numpy(self._csr.indices.astype(np.int64)).to(device)
        return self._inv_deg

    def attention(self, q, k, v, scale=None):
        """out[r, h, :] = sum over the edges e into r of softmax_r(scale * <k[col e, h, :], q[r, h, :]>) * v[col e, h, :];
        q (num_rows, H, D), k and v (num_cols, H, D), scale 1 / sqrt(D) unless given.  With D in {16, 32, 64}
        this is one operator that stores no scores, and its backward pass forms them again (two sweeps, one
        of them over the transposed adjacency); otherwise the differentiable chain sddmm -> edge_softmax ->
        spmm."""
        if scale is None:
            scale = 1.0 / float(q.shape[-1]) ** 0.5
        if q.dim() == 3 and q.shape[-1] in (16, 32, 64):
            return _Attention.apply(self, q, k, v, float(scale))
        return self.spmm(v, self.edge_softmax(self.sddmm(k, q) * scale))

    def gat_attention(self, er, el, v, negative_slope=0.2):
        """The attention of a GAT layer: out[r, h, :] = sum over the edges e into r of
        softmax_r(leaky_relu(el[col e, h] + er[r, h])) * v[col e, h, :]; er (num_rows, H), el (num_cols, H),
        v (num_cols, H, D) with D in {16, 32, 64}.  One operator forward, two sweeps backward; no per-edge
        array is stored."""
        return _GatAttention.apply(self, er, el, v, float(negative_slope))

    def _gat_mod(self, er, el, v, slope):
        key = ('gat', tuple(v.shape[1:]), slope)
        if key not in self._mods:
            m = GraphAttentionhip(self._csr)
            m.build([placeholder(tuple(er.shape)), placeholder(tuple(el.shape)), placeholder(tuple(v.shape))],
                    {'scores': 'additive', 'negative_slope': slope}, {})
            self._mods[key] = m
        return self._mods[key]

    def _attention_mod(self, q, k, v, scale):
        key = ('attention', tuple(q.shape[1:]), scale)
        if key not in self._mods:
            m = GraphAttentionhip(self._csr)
            m.build([placeholder(tuple(q.shape)), placeholder(tuple(k.shape)), placeholder(tuple(v.shape))],
                    {'scale': scale}, {})
            self._mods[key] = m
        return self._mods[key]

    # ---- generalised operators with broadcasting -------------------------------------------------------

    def gspmm(self, msg, lhs, rhs=None, reduce="sum"):
        """out[v] = reduce over the edges e into v of the message msg = '<u|e>_<add|sub|mul|div>_<u|e>' or 'copy_e'
        (DGL's names), reduce in {'sum', 'mean', 'max', 'min'}: operands on 'u' are (num_cols, ...), on 'e' (nnz, ...) in
        CSR edge order, and their feature shapes broadcast the numpy way.  Differentiable in both operands (max / min:
        the gradient goes to the selected edge's operands).  ('u_mul_e' with one weight per edge or per edge and head
        is spmm(); 'copy_u' is aggregate().)"""
        op, lt, rt = parse_message(msg)
        if reduce not in ("sum", "mean", "max", "min") or op not in ("add", "sub", "mul", "div", "copy_lhs") \
                or "v" in (lt, rt) or lt == rt:
            raise ValueError("differentiable here: sum / mean / max / min of add, sub, mul, div between an operand on 'u' "
                             "and one on 'e', or copy_e")
        fn = _GSpMM if reduce in ("sum", "mean") else _GSpMMExtreme
        if rt is None:
            return fn.apply(self, msg, reduce, lhs)
        return fn.apply(self, msg, reduce, lhs, rhs)

    def gsddmm(self, op, lhs, rhs, lhs_target="u", rhs_target="v"):
        """out[e] = lhs[..] op rhs[..] per edge, op in {'add', 'sub', 'mul', 'div'}, operands on 'u' (num_cols, ...), 'v'
        (num_rows, ...) or 'e' (nnz, ...), feature shapes broadcasting the numpy way; out is (nnz, ...) in CSR edge
        order.  Differentiable in both operands.  (The dot product is sddmm().)"""
        if op not in ("add", "sub", "mul", "div") or lhs_target == rhs_target or not {lhs_target, rhs_target} <= {"u", "v", "e"}:
            raise ValueError("differentiable here: add, sub, mul, div between operands on two different targets of u / v / e")
        return _GSDDMM.apply(self, op, lhs_target, rhs_target, lhs, rhs)

    def _bcast_spmm_raw(self, msg, arrays, reduce="sum", transposed=False, return_arg=False):
        """Generalised SpMM over the adjacency or its transpose; edge operands in this graph's CSR edge order either
        way (over the transpose the kernel addresses them through the transposed edges' CSR positions);
        return_arg (max / min): also the CSR position of the selected edge per output, as a tensor of the caller's own."""
        arrays = [a.contiguous() for a in arrays]
        key = ('gspmm', msg, reduce, transposed, return_arg) + tuple(tuple(a.shape) for a in arrays)
        if key not in self._mods:
            m = self._gspmm_module(transposed)
            args = {'msg': msg, 'reduce': reduce, 'broadcast': True}      # numpy broadcasting, whatever the shapes
            if return_arg:
                args['return_arg'] = True
            m.build([placeholder(tuple(a.shape)) for a in arrays], args, {})
            if transposed:
                m.set_weight_order(self._tr_pos_host)
            self._mods[key] = m
        mod = self._mods[key]
        if return_arg:
            mod.arg_tvm = torch.empty(mod._fresh_like[0] if getattr(mod, '_fresh_like', None) else mod.out_tvm.shape,
                                      dtype=torch.int32, device=mod._ctx)
            return _fresh_run(mod, arrays), mod.arg_tvm
        return _fresh_run(mod, arrays)

    def _bcast_sddmm_raw(self, op, lt, rt, arrays):
        arrays = [a.contiguous() for a in arrays]
        key = ('gsddmm', op, lt, rt) + tuple(tuple(a.shape) for a in arrays)
        if key not in self._mods:
            m = GSDDMMhip(self._csr)
            args = {'op': op}
            if lt is not None:
                args['lhs_target'] = lt
            if rt is not None:
                args['rhs_target'] = rt
            m.build([placeholder(tuple(a.shape)) for a in arrays], args, {})
            self._mods[key] = m
        return _fresh_run(self._mods[key], arrays)

    def _to_edges(self, x, target):
        """x on 'v' or 'u' copied to the edges (CSR order); x on 'e' as it is."""
        if target == "e":
            return x
        return self._bcast_sddmm_raw('copy_lhs', target, None, [x])

    def _from_edges(self, m, target):
        """Sum of the per-edge array m (CSR order) over the edges of each node of `target`; 'e': m itself."""
        if target == "e":
            return m
        if target == "v":
            return self._bcast_spmm_raw('copy_e', [m])
        return self._bcast_spmm_raw('copy_e', [m], transposed=True)

    def _edge_product_sum(self, m, q, tq, target, op="mul"):
        """For every node of `target` ('v' or 'u'): the sum over its edges of m[e] * q(e) (op='div': m[e] / q(e)), m per
        edge (CSR order), q on `tq`; the messages are formed inside the aggregation, no per-edge array is written."""
        if target == "v":               # rows of the adjacency: q on 'u' or 'e'
            if tq == "v":
                raise ValueError("both operands on the same target")
            return self._bcast_spmm_raw('e_%s_%s' % (op, tq), [m, q])
        if tq == "u":                   # rows of the transpose: its 'u' are this graph's 'v'
            raise ValueError("both operands on the same target")
        if tq == "v":
            return self._bcast_spmm_raw('e_%s_u' % op, [m, q], transposed=True)
        return self._bcast_spmm_raw('e_%s_e' % op, [m, q], transposed=True)

    def edge_softmax(self, scores):
        """Softmax of scores, (nnz,) or (nnz, H), over the edges of each destination row, per head."""
        return _EdgeSoftmax.apply(self, scores)


def _fresh_run(mod, inputs):
    """run() into a tensor of the caller's own: the module's output buffer (every element of which a run
    overwrites) is replaced first, so nothing has to be copied out of it, and the module lets go of it
    afterwards -- autograd takes a gradient it alone refers to as it is, and clones one that is shared."""
    like = getattr(mod, '_fresh_like', None)
    if like is None:
        like = mod._fresh_like = (tuple(mod.out_tvm.shape), mod.out_tvm.dtype, mod.out_tvm.device)
    mod.out_tvm = torch.empty(like[0], dtype=like[1], device=like[2])
    out = mod.run(inputs)
    mod.out_tvm = None
    return out


class _SpMM(torch.autograd.Function):
    @staticmethod
    def forward(ctx, g, x, w):
        ctx.g = g
        ctx.save_for_backward(x, w)
        return g._spmm_raw(x, w)

    @staticmethod
    def backward(ctx, dy):
        g = ctx.g
        x, w = ctx.saved_tensors
        dx = g._spmm_raw(dy, w, transposed=True) if ctx.needs_input_grad[1] else None
        dw = g._sddmm_raw(x, dy) if ctx.needs_input_grad[2] else None
        return None, dx, dw


class _SDDMM(torch.autograd.Function):
    @staticmethod
    def forward(ctx, g, src, dst):
        ctx.g = g
        ctx.save_for_backward(src, dst)
        return g._sddmm_raw(src, dst)

    @staticmethod
    def backward(ctx, ds):
        g = ctx.g
        src, dst = ctx.saved_tensors
        dsrc = g._spmm_raw(dst, ds, transposed=True) if ctx.needs_input_grad[1] else None
        ddst = g._spmm_raw(src, ds) if ctx.needs_input_grad[2] else None
        return None, dsrc, ddst


class _Attention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, g, q, k, v, scale):
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        mod = g._attention_mod(q, k, v, scale)
        mod.state_tvm = torch.empty_like(mod.state_tvm)        # handed to backward with the output
        out = _fresh_run(mod, [q, k, v])
        ctx.g, ctx.scale = g, scale
        ctx.save_for_backward(q, k, v, out, mod.state_tvm)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, state = ctx.saved_tensors
        dq, dk, dv = ctx.g._attention_mod(q, k, v, ctx.scale).backward(q, k, v, out, state, dout.contiguous())
        return None, dq, dk, dv, None


class _GatAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, g, er, el, v, slope):
        er, el, v = er.contiguous(), el.contiguous(), v.contiguous()
        mod = g._gat_mod(er, el, v, slope)
        mod.state_tvm = torch.empty_like(mod.state_tvm)
        out = _fresh_run(mod, [er, el, v])
        ctx.g, ctx.slope = g, slope
        ctx.save_for_backward(er, el, v, out, mod.state_tvm)
        return out

    @staticmethod
    def backward(ctx, dout):
        er, el, v, out, state = ctx.saved_tensors
        der, del_, dv = ctx.g._gat_mod(er, el, v, ctx.slope).backward(er, el, v, out, state, dout.contiguous())
        return None, der, del_, dv, None


class _EdgeSoftmax(torch.autograd.Function):
    @staticmethod
    def forward(ctx, g, scores):
        ctx.g = g
        a = _fresh_run(g._softmax_mod(tuple(scores.shape)), [scores.contiguous()])
        ctx.save_for_backward(a)
        return a

    @staticmethod
    def backward(ctx, da):
        (a,) = ctx.saved_tensors
        mod = ctx.g._softmax_mod(tuple(a.shape))
        mod.grad_tvm = torch.empty_like(a)          # handed to the caller; the module takes a new one next time
        grad = mod.backward(a, da.contiguous())
        mod.grad_tvm = None
        return None, grad


def _reduce_to(full, shape):
    """Sums `full` (rows, *broadcast feature shape) over the axes along which an operand of `shape` was broadcast."""
    shape = tuple(shape)
    lead = full.dim() - len(shape)
    if lead > 0:
        full = full.sum(dim=tuple(range(1, 1 + lead)))
    return full.sum_to_size(shape) if tuple(full.shape) != shape else full


class _GSpMM(torch.autograd.Function):
    @staticmethod
    def forward(ctx, g, msg, reduce, lhs, rhs=None):
        ctx.g, ctx.msg, ctx.reduce = g, msg, reduce
        arrays = [lhs] if rhs is None else [lhs, rhs]
        ctx.save_for_backward(*arrays)
        return g._bcast_spmm_raw(msg, arrays, reduce)

    @staticmethod
    def backward(ctx, dout):
        g = ctx.g
        op, lt, rt = parse_message(ctx.msg)
        arrays = ctx.saved_tensors
        dout = dout.contiguous()
        if ctx.reduce == "mean":
            deg = torch.from_numpy(np.maximum(np.diff(g._csr.indptr), 1).astype(np.float32)).to(dout.device)
            dout = dout / deg.reshape((-1,) + (1,) * (dout.dim() - 1))
        grads = []
        targets = [lt] if rt is None else [lt, rt]
        for i, (p, tp) in enumerate(zip(arrays, targets)):
            if not ctx.needs_input_grad[3 + i]:
                grads.append(None)
                continue
            if op in ("add", "sub", "copy_lhs"):
                # the message is linear in p with coefficient +-1: reduce dout to p's feature shape first
                d = _reduce_to(dout, (dout.shape[0],) + tuple(p.shape[1:]))
                full = g._to_edges(d, "v") if tp == "e" else _sum_over_out_edges(g, d)
                if op == "sub" and i == 1:
                    full = -full
                grads.append(full.reshape(p.shape))
            else:
                # mul: d message / d p = the other operand q;  div: 1 / q for the numerator, -l / p^2 for the denominator
                q, tq = arrays[1 - i], targets[1 - i]
                inner = "div" if (op == "div" and i == 0) else "mul"
                if tp == "u":       # sum over the edges that leave u of dout[row e] (* or /) q[e]
                    full = g._bcast_spmm_raw('u_%s_e' % inner, [dout, q], transposed=True)
                else:               # per edge: dout[row e] (* or /) q[col e]
                    full = g._bcast_sddmm_raw(inner, 'v', tq, [dout, q])
                if op == "div" and i == 1:
                    full = -full / _align_features(p, full) ** 2
                grads.append(_reduce_to(full, p.shape))
        return (None, None, None) + tuple(grads)


def _align_features(x, like):
    """View of x (rows, *feat) with its feature axes right-aligned to those of `like` (rows, *broadcast feat)."""
    return x.reshape((x.shape[0],) + (1,) * (like.dim() - x.dim()) + tuple(x.shape[1:]))


class _GSpMMExtreme(torch.autograd.Function):
    """max / min aggregation of a generalised message: the gradient of out[v, f] goes to the operands of the edge
    that was selected (the first one on ties, as the kernel reports it)."""

    @staticmethod
    def forward(ctx, g, msg, reduce, lhs, rhs=None):
        arrays = [lhs] if rhs is None else [lhs, rhs]
        out, arg = g._bcast_spmm_raw(msg, arrays, reduce, return_arg=True)
        ctx.g, ctx.msg = g, msg
        ctx.save_for_backward(arg, *arrays)
        ctx.mark_non_differentiable(arg)
        return out

    @staticmethod
    def backward(ctx, dout):
        g = ctx.g
        op, lt, rt = parse_message(ctx.msg)
        arg, *arrays = ctx.saved_tensors
        targets = [lt] if rt is None else [lt, rt]
        n_dst, out_shape = dout.shape[0], tuple(dout.shape[1:])
        n_out = int(np.prod(out_shape)) if out_shape else 1
        g._mean_weights(dout.device)                                   # makes g._cols
        e = arg.reshape(n_dst, n_out).long()
        valid = e >= 0
        e = e.clamp(min=0)
        rows_of = {"u": g._cols[e], "e": e}                            # operand row per output element

        def spread(x):      # (rows, *feat) -> (rows, n_out): the operand feature every output feature reads
            return _align_features(x, dout).expand((x.shape[0],) + out_shape).reshape(x.shape[0], n_out)

        picked = [spread(x).gather(0, rows_of[t]) for x, t in zip(arrays, targets)]
        d = dout.reshape(n_dst, n_out) * valid
        grads = []
        for i, (p, tp) in enumerate(zip(arrays, targets)):
            if not ctx.needs_input_grad[3 + i]:
                grads.append(None)
                continue
            if op in ("add", "copy_lhs") or (op == "sub" and i == 0):
                c = d
            elif op == "sub":
                c = -d
            elif op == "mul":
                c = d * picked[1 - i]
            elif i == 0:                                               # div, numerator
                c = d / picked[1]
            else:                                                      # div, denominator
                c = -d * picked[0] / picked[1] ** 2
            c = torch.where(valid, c, torch.zeros_like(c))
            full = torch.zeros((p.shape[0], n_out), dtype=dout.dtype, device=dout.device).scatter_add_(0, rows_of[tp], c)
            grads.append(_reduce_to(full.reshape((p.shape[0],) + out_shape), p.shape))
        return (None, None, None) + tuple(grads)


def _sum_over_out_edges(g, d):
    """For every source node: the sum of d[row e] over the edges that leave it (d on the destination nodes)."""
    return g._bcast_spmm_raw('copy_u', [d.reshape(d.shape[0], -1)], transposed=True).reshape((g.shape[1],) + tuple(d.shape[1:]))


class _GSDDMM(torch.autograd.Function):
    @staticmethod
    def forward(ctx, g, op, lt, rt, lhs, rhs):
        ctx.g, ctx.op, ctx.targets = g, op, (lt, rt)
        ctx.save_for_backward(lhs, rhs)
        return g._bcast_sddmm_raw(op, lt, rt, [lhs, rhs])

    @staticmethod
    def backward(ctx, dout):
        g, op = ctx.g, ctx.op
        arrays, targets = ctx.saved_tensors, ctx.targets
        dout = dout.contiguous()
        grads = []
        for i, (p, tp) in enumerate(zip(arrays, targets)):
            if not ctx.needs_input_grad[4 + i]:
                grads.append(None)
                continue
            if op in ("add", "sub"):
                d = _reduce_to(dout, (dout.shape[0],) + tuple(p.shape[1:]))
                full = g._from_edges(d.reshape(d.shape[0], -1), tp).reshape(p.shape)
                grads.append(-full if (op == "sub" and i == 1) else full)
            else:
                # mul: d out / d p = q;  div: 1 / q for the numerator, -l / p^2 for the denominator
                q, tq = arrays[1 - i], targets[1 - i]
                inner = "div" if (op == "div" and i == 0) else "mul"
                if tp == "e":
                    full = g._bcast_sddmm_raw(inner, 'e', tq, [dout, q])
                else:
                    full = g._edge_product_sum(dout, q, tq, tp, inner)
                if op == "div" and i == 1:
                    full = -full / _align_features(p, full) ** 2
                grads.append(_reduce_to(full, p.shape))
        return (None, None, None, None) + tuple(grads)


class _Aggregate(torch.autograd.Function):
    @staticmethod
    def forward(ctx, g, x, reduce):
        ctx.g, ctx.reduce = g, reduce
        x = x.contiguous()
        mod = g._aggregate_mod(x.shape[1], reduce)
        y = mod.run([x]).clone()
        if reduce in ("max", "min"):
            ctx.save_for_backward(mod.arg_tvm.clone())
        ctx.x_shape = tuple(x.shape)
        return y

    @staticmethod
    def backward(ctx, dy):
        g, reduce = ctx.g, ctx.reduce
        dy = dy.contiguous()
        if reduce in ("sum", "mean"):
            w = g._mean_weights(dy.device)
            return None, g._spmm_raw(dy, w if reduce == "mean" else g._ones, transposed=True), None
        (arg,) = ctx.saved_tensors
        g._mean_weights(dy.device)
        n_src, F = ctx.x_shape
        valid = arg >= 0
        src = g._cols[arg.clamp(min=0).long()]                               # source vertex of the selected edge
        flat = (src * F + torch.arange(F, device=dy.device)[None, :])[valid]
        dx = torch.zeros(n_src * F, dtype=dy.dtype, device=dy.device)
        dx.index_add_(0, flat, dy[valid])
        return None, dx.view(n_src, F), None
