"""Pieces shared by the SpMM and SDDMM module classes."""
import numpy as np
import torch

from .. import _lib


class placeholder(object):
    """Shape/dtype record of a dense input, standing where the reference's callers pass
    ``te.placeholder(shape)`` to ``build`` (tests/test_module_spmm.py:18-19)."""

    def __init__(self, shape, dtype="float32", name="placeholder"):
        self.shape = tuple(int(s) for s in shape)
        self.dtype = str(dtype)
        self.name = name
        if self.dtype != "float32":
            raise ValueError("only float32 features are supported, got %s" % self.dtype)

    def __repr__(self):
        return "placeholder(%s, shape=%s, dtype=%s)" % (self.name, self.shape, self.dtype)


def device():
    """The GPU every module object lives on.  Fails loudly without one: there is no CPU path."""
    if not torch.cuda.is_available():
        raise RuntimeError("featgraph_amd needs a ROCm GPU (gfx950); torch.cuda.is_available() is False")
    return torch.device("cuda", torch.cuda.current_device())


def check_int32_sizes(num_rows, num_cols, nnz):
    """The kernels address vertices and stored elements with int32 (every benchmark configuration fits); a larger
    matrix would wrap around silently when its index arrays are narrowed, so it is refused here."""
    limit = 2 ** 31 - 1
    if num_rows >= limit or num_cols >= limit or nnz >= limit:
        raise ValueError("a %d x %d adjacency with %d stored elements does not fit the kernels' int32 indices"
                         % (num_rows, num_cols, nnz))


def to_device_i32(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int32)).to(dev)


def to_device_f32(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dev)


def stream_ptr():
    import ctypes
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def check_inputs(tensors, placeholders, dev):
    if len(tensors) != len(placeholders):
        raise ValueError("expected %d input array(s), got %d" % (len(placeholders), len(tensors)))
    for t, ph in zip(tensors, placeholders):
        if not isinstance(t, torch.Tensor):
            raise TypeError("inputs must be torch tensors on the module's device, got %s" % type(t))
        if t.device != dev:
            raise ValueError("input is on %s, the module lives on %s" % (t.device, dev))
        if t.dtype != torch.float32:
            raise ValueError("input dtype must be float32, got %s" % t.dtype)
        if tuple(t.shape) != ph.shape:
            raise ValueError("input shape %s does not match the built shape %s" % (tuple(t.shape), ph.shape))
        if not t.is_contiguous():
            raise ValueError("inputs must be contiguous (row-major)")


def ensure_output(mod):
    """A module that handed its output tensor out for good (featgraph_amd.autograd does: the gradient machinery keeps
    the tensor, the module drops it) gets a new one of the built shape before its next direct run()."""
    like = getattr(mod, '_fresh_like', None)
    if getattr(mod, 'out_tvm', None) is None and like is not None:
        mod.out_tvm = torch.empty(like[0], dtype=like[1], device=like[2])
    if hasattr(mod, 'arg_tvm') and mod.arg_tvm is None and getattr(mod, '_return_arg', False) and mod.out_tvm is not None:
        mod.arg_tvm = torch.full(mod.out_tvm.shape, -1, dtype=torch.int32, device=mod.out_tvm.device)


def timed_mean_seconds(fn, num_runs):
    """Mean seconds of `num_runs` back-to-back launches between two events on the current
    stream, after one untimed call (the protocol of Module.time_evaluator(number=num_runs)
    used at python/featgraph/module/spmm.py:179-186, plus a warm-up)."""
    assert num_runs >= 1
    fn()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(num_runs):
        fn()
    end.record()
    end.synchronize()
    return start.elapsed_time(end) * 1e-3 / num_runs


# fg_op of include/featgraph_hip.h
(OP_SPMM_SUM, OP_SPMM_EXTREME, OP_SDDMM_DDS, OP_EDGE_SOFTMAX, OP_ATTENTION, OP_ATTENTION_ADDITIVE,
 OP_GSPMM_BCAST, OP_GSPMM_BCAST_ARG) = range(8)


def reserve(plan, op, heads, head_len, num_feat_partitions, dev):
    """Sizes the plan's device scratch at build() time, so that run() allocates nothing (and can be
    captured into a HIP graph without a warm-up call)."""
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().fg_spmm_plan_reserve(plan, op, int(heads), int(head_len), int(num_feat_partitions)))


# Tests switch this off to compare the kernels' 16-bit and 32-bit index streams.
NARROW_INDICES = True


def narrow_indices(plan, idx_dev, num_cols, num_partitions, dev):
    """Gives the plan a 16-bit copy of the layout's column ids whenever a partition is at most 65,536 columns wide
    (232,965-node graph, 8 partitions: SpMM 11.5 -> 11.3 ms at F=512, 3.10 -> 2.96 ms at F=128, 1.73 -> 1.63 ms at
    F=64); the kernels read it instead of `idx_dev` on every call that hands them this tensor."""
    if not NARROW_INDICES or idx_dev.numel() == 0:
        return
    if (int(num_cols) + int(num_partitions) - 1) // int(num_partitions) > 65536:
        return
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().fg_spmm_plan_narrow_indices(plan, _lib.dev_ptr(idx_dev), stream_ptr()))
        # the copy is made on the current stream, once, at construction; run() may be called under any other stream
        torch.cuda.current_stream().synchronize()


def take_args(args, allowed, what):
    """Mirrors the reference's ``**args`` unpacking: an unknown key is a TypeError."""
    for k in args:
        if k not in allowed:
            raise TypeError("%s got an unexpected keyword argument '%s'" % (what, k))
    return dict(args)
