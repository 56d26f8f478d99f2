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

from .module import (EdgeSoftmaxhip, GraphAttentionhip, GSpMMhip, MultiHeadSDDMMhip, VanillaSDDMMhip,
                     placeholder)


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

    def _spmm_mod(self, transposed, tail, w_heads):
        key = ('spmm', transposed, tail, w_heads)
        if key not in self._mods:
            adj = self._tr if transposed else self._csr
            m = GSpMMhip(adj)
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
            m = GSpMMhip(self._csr)
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

    def edge_softmax(self, scores):
        """Softmax of scores, (nnz,) or (nnz, H), over the edges of each destination row, per head."""
        return _EdgeSoftmax.apply(self, scores)


def _fresh_run(mod, inputs):
    """run() into a tensor of the caller's own: the module's output buffer (every element of which a run
    overwrites) is replaced first, so nothing has to be copied out of it."""
    mod.out_tvm = torch.empty_like(mod.out_tvm)
    return mod.run(inputs)


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
        return None, mod.backward(a, da.contiguous())


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
