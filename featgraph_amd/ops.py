"""gspmm / gsddmm with the call signatures of DGL's `dgl.ops`, over a `featgraph_amd.autograd.Graph`.

The reference's README (README.md:9-14) points to generalised SpMM / SDDMM kernels and to their integration
into DGL, whose message-passing layer calls exactly these two functions; the reference snapshot itself holds
neither.  Operand conventions are DGL's: node features of the source nodes are `(num_src, ...)`, of the
destination nodes `(num_dst, ...)`, edge features `(nnz, ...)` in the graph's CSR edge order, and the feature
shapes of two operands broadcast against each other the numpy way.

Gradients: every call routes to a differentiable operator (weighted sums; sum / mean / max / min of add / sub /
mul / div messages and copies; per-edge add / sub / mul / div and dot products of node features); what is left --
operators between two operands on the same target, dot products that involve edge features or broadcasting --
runs forward only and refuses inputs that require grad.
"""
import torch

_BINARY = ("add", "sub", "mul", "div")


def _no_grad_inputs(what, *tensors):
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors):
        raise NotImplementedError("%s has no gradient here; detach the inputs or run under torch.no_grad()" % what)


def gspmm(g, op, reduce_op, lhs_data, rhs_data):
    """out[v] = reduce_op over the edges e = (u -> v) of  lhs_data[u] op rhs_data[e].

    op: 'add' | 'sub' | 'mul' | 'div' | 'copy_lhs' | 'copy_rhs'; reduce_op: 'sum' | 'mean' | 'max' | 'min'
    (rows without edges give 0).  lhs_data lives on the source nodes, rhs_data on the edges; the operand a
    copy does not use may be None."""
    if reduce_op not in ("sum", "mean", "max", "min"):
        raise ValueError("reduce_op must be 'sum', 'mean', 'max' or 'min'")
    if op == "copy_lhs":
        x = lhs_data
        if x.dim() == 1:
            return g.aggregate(x[:, None], reduce_op)[:, 0]
        return g.aggregate(x.reshape(x.shape[0], -1), reduce_op).reshape((g.shape[0],) + tuple(x.shape[1:]))
    if op == "copy_rhs":
        return g.gspmm("copy_e", rhs_data, reduce=reduce_op)
    if op not in _BINARY:
        raise ValueError("op must be one of %s, 'copy_lhs', 'copy_rhs'" % (_BINARY,))
    if op == "mul" and reduce_op == "sum" and lhs_data.dim() in (2, 3):
        # one weight per edge (or per edge and head): the weighted-sum kernels with their source partitions
        heads = lhs_data.shape[1] if lhs_data.dim() == 3 else 1
        if rhs_data.dim() == 1 and lhs_data.dim() == 2:
            return g.spmm(lhs_data, rhs_data)
        if lhs_data.dim() == 3 and tuple(rhs_data.shape[1:]) == (heads, 1):
            return g.spmm(lhs_data, rhs_data[:, :, 0])
        if lhs_data.dim() == 2 and tuple(rhs_data.shape[1:]) == (1,):
            return g.spmm(lhs_data, rhs_data[:, 0])
    return g.gspmm("u_%s_e" % op, lhs_data, rhs_data, reduce_op)


def gsddmm(g, op, lhs_data, rhs_data, lhs_target="u", rhs_target="v"):
    """out[e] = lhs_data[lhs_target of e] op rhs_data[rhs_target of e] for every edge e.

    op: 'add' | 'sub' | 'mul' | 'div' | 'dot' | 'copy_lhs' | 'copy_rhs'; targets: 'u' (source node), 'v'
    (destination node), 'e' (the edge).  'dot' contracts the last feature axis and keeps it with length 1,
    as DGL does.  out is (nnz, ...) in the graph's CSR edge order."""
    if op == "copy_lhs":
        return _copy_to_edges(g, lhs_data, lhs_target)
    if op == "copy_rhs":
        return _copy_to_edges(g, rhs_data, rhs_target)
    if op == "dot":
        same = (lhs_target, rhs_target) == ("u", "v") and lhs_data.shape[1:] == rhs_data.shape[1:]
        if same and lhs_data.dim() in (2, 3):
            return g.sddmm(lhs_data, rhs_data).unsqueeze(-1)
        if (lhs_target, rhs_target) == ("v", "u") and lhs_data.shape[1:] == rhs_data.shape[1:] and lhs_data.dim() in (2, 3):
            return g.sddmm(rhs_data, lhs_data).unsqueeze(-1)
        _no_grad_inputs("a dot product between these targets / shapes", lhs_data, rhs_data)
        return g._bcast_sddmm_raw("dot", lhs_target, rhs_target, [lhs_data, rhs_data]).unsqueeze(-1)
    if op not in _BINARY:
        raise ValueError("op must be one of %s, 'dot', 'copy_lhs', 'copy_rhs'" % (_BINARY,))
    if lhs_target != rhs_target:
        return g.gsddmm(op, lhs_data, rhs_data, lhs_target, rhs_target)
    _no_grad_inputs("gsddmm(%s) between '%s' and '%s'" % (op, lhs_target, rhs_target), lhs_data, rhs_data)
    return g._bcast_sddmm_raw(op, lhs_target, rhs_target, [lhs_data, rhs_data])


def _copy_to_edges(g, x, target):
    if target == "e":
        return x
    # a copy is the per-edge sum of x with zeros on the edges: differentiable through gsddmm
    zeros = torch.zeros((g.nnz,) + (1,) * (x.dim() - 1), dtype=x.dtype, device=x.device)
    return g.gsddmm("add", x, zeros, target, "e")


def edge_softmax(g, scores):
    """Softmax of the edge scores over the edges of each destination node, per head (dgl.ops.edge_softmax with
    norm_by='dst')."""
    squeeze = scores.dim() == 3 and scores.shape[-1] == 1
    a = g.edge_softmax(scores[..., 0] if squeeze else scores)
    return a.unsqueeze(-1) if squeeze else a
