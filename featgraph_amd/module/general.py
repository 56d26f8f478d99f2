"""Broadcasting between the two operands of a generalised SpMM / SDDMM message, and the launch of the
library's broadcasting kernels.  The reference snapshot has no such operators (README.md:9-11 names
"generalized SpMM and SDDMM" on another branch); operand targets and operator names follow DGL's
gspmm / gsddmm vocabulary: u = source node (column), v = destination node (row), e = stored element."""
import re

import numpy as np
import torch

from .. import _lib
from . import common

BINARY = {'add': 0, 'sub': 1, 'mul': 2, 'div': 3, 'copy_lhs': 4, 'copy_rhs': 5, 'dot': 6}
TARGET = {'u': 0, 'e': 1, 'v': 2}
_MSG = re.compile(r'^([uev])_(add|sub|mul|div|dot)_([uev])$')


def parse_message(msg):
    """'u_mul_e' -> ('mul', 'u', 'e'); 'copy_u' / 'copy_e' / 'copy_v' -> ('copy_lhs', target, None)."""
    if msg in ('copy_u', 'copy_e', 'copy_v'):
        return 'copy_lhs', msg[-1], None
    m = _MSG.match(msg)
    if not m:
        raise ValueError("message %r is not '<u|e|v>_<add|sub|mul|div|dot>_<u|e|v>' or 'copy_<u|e|v>'" % (msg,))
    return m.group(2), m.group(1), m.group(3)


def broadcast_plan(lhs_shape, rhs_shape, dot=False):
    """Feature shapes of the operands (without the leading row axis; None for an absent operand) ->
    (out_shape, lhs_off, rhs_off, reduce_len): numpy broadcasting of the two shapes, as index arrays that
    give, for every flattened output feature, the flattened operand feature it reads (None where that is
    the identity).  dot=True: the last axis (equal in both) is contracted and the arrays index the rest."""
    def norm(s):
        return (1,) if s is not None and len(s) == 0 else s
    lhs_shape, rhs_shape = norm(lhs_shape), norm(rhs_shape)
    reduce_len = 1
    if dot:
        if lhs_shape is None or rhs_shape is None or lhs_shape[-1] != rhs_shape[-1]:
            raise ValueError("'dot' contracts the last axis, which must be equal: %s vs %s" % (lhs_shape, rhs_shape))
        reduce_len = int(lhs_shape[-1])
        lhs_shape, rhs_shape = tuple(lhs_shape[:-1]), tuple(rhs_shape[:-1])
    shapes = [tuple(s) for s in (lhs_shape, rhs_shape) if s is not None]
    try:
        out_shape = np.broadcast_shapes(*shapes)
    except ValueError:
        raise ValueError("operand feature shapes %s and %s do not broadcast" % (lhs_shape, rhs_shape))
    n_out = int(np.prod(out_shape))

    def offsets(shape):
        if shape is None:
            return None
        n = int(np.prod(shape))
        if n == n_out:
            return None          # same number of features and broadcastable: the identity
        return np.ascontiguousarray(np.broadcast_to(np.arange(n, dtype=np.int32).reshape(shape), out_shape).reshape(-1))
    return tuple(int(s) for s in out_shape), offsets(lhs_shape), offsets(rhs_shape), reduce_len


def vector_flags(off, out_len, vec_flag, splat_flag):
    """The library's FG_BCAST_* flag for one offset array: whether every aligned group of 4 output features
    reads 4 consecutive operand features that start at a multiple of 4, or one feature 4 times."""
    if off is None or out_len % 4 != 0:
        return 0
    groups = off.reshape(-1, 4)
    if (groups == groups[:, :1]).all():
        return splat_flag
    if (groups[:, 0] % 4 == 0).all() and (groups == groups[:, :1] + np.arange(4)).all():
        return vec_flag
    return 0


def rows_of(target, num_rows, num_cols, nnz):
    return {'u': num_cols, 'v': num_rows, 'e': nnz}[target]


def check_operand_shape(ph, target, num_rows, num_cols, nnz, what):
    want = rows_of(target, num_rows, num_cols, nnz)
    if len(ph.shape) < 1 or ph.shape[0] != want:
        raise ValueError("%s lives on '%s' and must have %d rows, got shape %s" % (what, target, want, ph.shape))
    return tuple(ph.shape[1:])


class BroadcastOp(object):
    """One resolved message: operator, targets, offset arrays on the device, output feature shape."""

    def __init__(self, op, lhs_target, rhs_target, lhs_ph, rhs_ph, num_rows, num_cols, nnz, dev, allow_v):
        if op not in BINARY:
            raise ValueError("operator must be one of %s" % sorted(BINARY))
        for t in (lhs_target, rhs_target):
            if t is not None and (t not in TARGET or (t == 'v' and not allow_v)):
                raise ValueError("operand target %r is not valid here" % (t,))
        self.op = op
        self.lhs_target, self.rhs_target = lhs_target, rhs_target
        l_shape = check_operand_shape(lhs_ph, lhs_target, num_rows, num_cols, nnz, "the left operand") if lhs_ph is not None else None
        r_shape = check_operand_shape(rhs_ph, rhs_target, num_rows, num_cols, nnz, "the right operand") if rhs_ph is not None else None
        self.out_shape, lo, ro, self.reduce_len = broadcast_plan(l_shape, r_shape, dot=(op == 'dot'))
        self.out_len = int(np.prod(self.out_shape))
        self.lhs_len = int(np.prod(l_shape)) if l_shape is not None else 0
        self.rhs_len = int(np.prod(r_shape)) if r_shape is not None else 0
        self.flags = vector_flags(lo, self.out_len, 1, 2) | vector_flags(ro, self.out_len, 4, 8)
        self.lhs_off = None if lo is None else torch.from_numpy(lo).to(dev)
        self.rhs_off = None if ro is None else torch.from_numpy(ro).to(dev)

    def describe(self):
        return ("message %s(%s, %s): operand lengths %d / %d -> %d output feature(s)%s%s"
                % (self.op, self.lhs_target, self.rhs_target, self.lhs_len, self.rhs_len, self.out_len,
                   "" if self.reduce_len == 1 else ", %d contracted" % self.reduce_len,
                   "" if self.lhs_off is None and self.rhs_off is None else ", broadcast through offset arrays"))

    def feature_tiles(self, return_arg=False):
        """The number of 64-float feature tiles the library's SpMM kernel will cut this message into (it does so from
        128 output features on, when an operand is gathered from the source nodes, none is streamed from the edges
        with 4 consecutive features per lane, no positions are asked for and 4 features per lane are possible: every
        operand's groups of 4 consecutive or equal)."""
        def wide(off, length, vec_flag, splat_flag):
            if length == 0:
                return 1                                    # operand not used
            if off is None or (self.flags & vec_flag):
                return 1 if length % 4 == 0 else 0
            return 2 if (self.flags & splat_flag) else 0
        l, r = wide(self.lhs_off, self.lhs_len, 1, 2), wide(self.rhs_off, self.rhs_len, 4, 8)
        vec = self.out_len % 4 == 0 and l and r and not (l == 2 and r == 2)
        streams = (self.lhs_target == 'e' and self.lhs_len > 0 and l == 1) or (self.rhs_target == 'e' and self.rhs_len > 0 and r == 1)
        if vec and not streams and not return_arg and self.gathered_len() > 0 and self.out_len >= 128 and self.out_len % 64 == 0:
            return self.out_len // 64
        return 1

    def gathered_len(self):
        """Feature length of the operand that is gathered from the source nodes (0: none is)."""
        return max(self.lhs_len if self.lhs_target == 'u' else 0, self.rhs_len if self.rhs_target == 'u' else 0)

    def run_spmm(self, plan, pos_dev, idx_dev, reduce, lhs, rhs, row_scale, out, arg, edge_pos_dev=None):
        """pos_dev / idx_dev: indptr / indices, or the arrays of a source-partitioned layout; edge_pos_dev: where each
        of their elements lies in the edge operands (required with partitions; None: at its own position)."""
        operands = (BINARY[self.op], reduce,
                    _lib.dev_ptr(lhs), TARGET[self.lhs_target or 'u'], self.lhs_len, _lib.dev_ptr(self.lhs_off),
                    _lib.dev_ptr(rhs), TARGET[self.rhs_target or 'e'], self.rhs_len, _lib.dev_ptr(self.rhs_off), self.flags,
                    _lib.dev_ptr(row_scale), _lib.dev_ptr(out), _lib.dev_ptr(arg), self.out_len, common.stream_ptr())
        if edge_pos_dev is None:
            _lib.check(_lib.lib().fg_gspmm_bcast_f32(plan, _lib.dev_ptr(pos_dev), _lib.dev_ptr(idx_dev), *operands))
        else:
            _lib.check(_lib.lib().fg_gspmm_bcast_dds_f32(plan, _lib.dev_ptr(pos_dev), _lib.dev_ptr(idx_dev),
                                                         _lib.dev_ptr(edge_pos_dev), *operands))

    def run_sddmm(self, row_dev, col_dev, n_edges, lhs, rhs, out):
        _lib.check(_lib.lib().fg_gsddmm_bcast_f32(
            _lib.dev_ptr(row_dev), _lib.dev_ptr(col_dev), n_edges, BINARY[self.op],
            _lib.dev_ptr(lhs), TARGET[self.lhs_target or 'u'], self.lhs_len, _lib.dev_ptr(self.lhs_off),
            _lib.dev_ptr(rhs), TARGET[self.rhs_target or 'v'], self.rhs_len, _lib.dev_ptr(self.rhs_off), self.flags,
            _lib.dev_ptr(out), self.out_len, self.reduce_len, common.stream_ptr()))
