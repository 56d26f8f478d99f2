"""SpMM module classes: the build()/run() surface of the reference's
python/featgraph/module/spmm.py, executing hand-written gfx950 kernels."""
import ctypes

import numpy as np
import torch

from .. import _lib
from ..util import util_convert_csr_to_dds
from . import common


class SpMMbase(object):
    """The base class for SpMM-like computation kernels (python/featgraph/module/spmm.py:12-194)."""

    def __init__(self, adj_scipy, num_col_partitions=1):
        """Doing 1D graph partitioning (src vertex partitioning) during init.

        Parameters
        ----------
        adj_scipy : scipy.sparse.coo_matrix or scipy.sparse.csr_matrix
            The input scipy sparse matrix; rows are destinations, columns are sources.

        num_col_partitions : int
            Number of partitions along the col dimension (src vertices)
        """
        if adj_scipy.format != 'csr':
            adj_scipy_csr = adj_scipy.tocsr()
        else:
            adj_scipy_csr = adj_scipy
        self._num_rows = adj_scipy_csr.shape[0]
        self._num_cols = adj_scipy_csr.shape[1]
        assert num_col_partitions >= 1, "num_col_partitions should be larger than or equal to 1"
        self._num_col_partitions = num_col_partitions
        self._target = None
        self._ctx = None
        self._register()
        L = _lib.lib()
        indptr = np.ascontiguousarray(adj_scipy_csr.indptr, dtype=np.int32)
        indices = np.ascontiguousarray(adj_scipy_csr.indices, dtype=np.int32)
        _lib.check(L.fg_check_csr_host(self._num_rows, self._num_cols, _lib.host_ptr(indptr),
                                       _lib.host_ptr(indices)))
        self._plan = ctypes.c_void_p()
        # 1D graph partitioning
        if self._num_col_partitions > 1:
            adj_s1_pos, adj_s1_idx, adj_vals = self._preprocess_adj(adj_scipy_csr, self._num_col_partitions)
            self._adj_s1_pos = adj_s1_pos
            self._adj_s1_idx = adj_s1_idx
            self._adj_vals = np.ascontiguousarray(adj_vals, dtype=np.float32)
            self._adj_s1_pos_dev = common.to_device_i32(self._adj_s1_pos, self._ctx)
            self._adj_s1_idx_dev = common.to_device_i32(self._adj_s1_idx, self._ctx)
            self._adj_vals_dev = common.to_device_f32(self._adj_vals, self._ctx)
            self._adj_d1_size = self._num_col_partitions
            self._adj_d2_size = self._num_rows + 1
            pos_host = self._adj_s1_pos
        else:
            self._adj_indptr = indptr
            self._adj_indices = indices
            self._adj_vals = np.ascontiguousarray(adj_scipy_csr.data, dtype=np.float32)
            self._adj_indptr_dev = common.to_device_i32(self._adj_indptr, self._ctx)
            self._adj_indices_dev = common.to_device_i32(self._adj_indices, self._ctx)
            self._adj_vals_dev = common.to_device_f32(self._adj_vals, self._ctx)
            pos_host = self._adj_indptr
        with torch.cuda.device(self._ctx):
            _lib.check(L.fg_spmm_plan_create(_lib.host_ptr(pos_host), self._num_rows, self._num_cols,
                                             self._num_col_partitions, None, ctypes.byref(self._plan)))
        # To be updated in self.build
        self._func = None
        self._placeholders = None
        self._feat_len = None
        self._num_feat_partitions = 0
        self._notes = []
        # To be updated in self.build; the same tensor is returned by every run()
        self.out_tvm = None

    def __del__(self):
        plan = getattr(self, "_plan", None)
        if plan is not None and plan.value:
            try:
                _lib.lib().fg_spmm_plan_destroy(plan)
            except Exception:
                pass
            self._plan = None

    def _preprocess_adj(self, adj_scipy_csr, num_col_partitions=1):
        return util_convert_csr_to_dds(adj_scipy_csr, num_col_partitions)

    def _register(self):
        raise NotImplementedError("Please register target and ctx.")

    def _resolve(self, input_placeholders, compute_args, schedule_args):
        compute_args = common.take_args(compute_args, self._compute_keys, "compute_func")
        schedule_args = common.take_args(schedule_args, self._schedule_keys, "schedule_func")
        if len(input_placeholders) != 1:
            raise ValueError("SpMM takes one dense input (SrcFeat), got %d" % len(input_placeholders))
        ph = input_placeholders[0]
        if len(ph.shape) != 2 or ph.shape[0] != self._num_cols:
            raise ValueError("SrcFeat must have shape (num_cols=%d, feat_len), got %s" % (self._num_cols, ph.shape))
        feat_len = ph.shape[1]
        notes = []
        T = compute_args.get('num_feat_partitions', 0)
        if T is None:
            T = 0
        if T == 0 and schedule_args.get('num_threads_per_cuda_block'):
            # the reference splits the feature axis by this factor (vanilla_spmm.py:140-141)
            t = int(schedule_args['num_threads_per_cuda_block'])
            if feat_len % t == 0:
                T = feat_len // t
            else:
                notes.append("num_threads_per_cuda_block=%d does not divide feat_len; ignored" % t)
        if schedule_args.get('num_cuda_blocks') is not None:
            notes.append("num_cuda_blocks has no counterpart: work items, not row blocks, are balanced")
        if T < 0 or (T > 0 and feat_len % T != 0):
            raise ValueError("feat_len %d is not divisible by num_feat_partitions %d" % (feat_len, T))
        return ph, feat_len, int(T), notes

    def build(self, input_placeholders, compute_args, schedule_args):
        """Fix the feature length and kernel variant, allocate the output once.

        Parameters
        ----------
        input_placeholders : list of placeholder
            The dense inputs other than adj: [SrcFeat (num_cols, feat_len)]

        compute_args : dict
            e.g. {'num_feat_partitions': T}: feature tiles handled by different workgroups

        schedule_args : dict
            The reference's CUDA keys 'num_cuda_blocks' / 'num_threads_per_cuda_block' are accepted
        """
        ph, feat_len, T, notes = self._resolve(input_placeholders, compute_args, schedule_args)
        self._placeholders = [ph]
        self._feat_len = feat_len
        self._num_feat_partitions = T
        self._notes = notes
        self._func = (_lib.lib().fg_spmm_dds_f32 if self._num_col_partitions > 1
                      else _lib.lib().fg_spmm_csr_f32)
        self.out_tvm = torch.zeros((self._num_rows, feat_len), dtype=torch.float32, device=self._ctx)

    def lower_to_ir(self, input_placeholders, compute_args, schedule_args):
        """Return a text description of the plan and launch. This can be useful for debug."""
        _, feat_len, T, notes = self._resolve(input_placeholders, compute_args, schedule_args)
        buf = ctypes.create_string_buffer(4096)
        _lib.check(_lib.lib().fg_spmm_plan_describe(self._plan, feat_len, T, buf, len(buf)))
        text = buf.value.decode()
        for n in notes:
            text += "  note             : %s\n" % n
        return text

    def _launch(self, src_feat):
        if self._num_col_partitions > 1:
            pos, idx = self._adj_s1_pos_dev, self._adj_s1_idx_dev
        else:
            pos, idx = self._adj_indptr_dev, self._adj_indices_dev
        _lib.check(self._func(self._plan, _lib.dev_ptr(pos), _lib.dev_ptr(idx), _lib.dev_ptr(self._adj_vals_dev),
                              _lib.dev_ptr(src_feat), _lib.dev_ptr(self.out_tvm), self._feat_len,
                              self._num_feat_partitions, common.stream_ptr()))

    def run(self, input_tvm_ndarrays):
        """Run the built func with the given inputs.

        Parameters
        ----------
        input_tvm_ndarrays : list of torch.Tensor
            [SrcFeat], float32, contiguous, on the module's device

        Returns
        -------
        self.out_tvm: torch.Tensor
            The output tensor (the same one on every call, overwritten in place).  The launch
            is enqueued on torch's current stream; nothing is synchronised here.
        """
        if self._func is None:
            raise RuntimeError("call build() before run()")
        common.check_inputs(input_tvm_ndarrays, self._placeholders, self._ctx)
        self._launch(input_tvm_ndarrays[0])
        return self.out_tvm

    def measure_average_time(self, input_tvm_ndarrays, num_runs):
        """Average run time in seconds over `num_runs` back-to-back launches."""
        if self._func is None:
            raise RuntimeError("call build() before measure_average_time()")
        common.check_inputs(input_tvm_ndarrays, self._placeholders, self._ctx)
        x = input_tvm_ndarrays[0]
        return common.timed_mean_seconds(lambda: self._launch(x), num_runs)

    @property
    def ctx(self):
        return self._ctx

    @property
    def target(self):
        return self._target


class VanillaSpMMhip(SpMMbase):
    """CSR (or, with num_col_partitions > 1, DDS) SpMM on gfx950."""
    _compute_keys = ('num_feat_partitions',)
    _schedule_keys = ('num_cuda_blocks', 'num_threads_per_cuda_block')

    def __init__(self, adj_scipy, num_col_partitions=1):
        super(VanillaSpMMhip, self).__init__(adj_scipy, num_col_partitions)

    def _register(self):
        self._target = 'rocm'
        self._ctx = common.device()


class VanillaSpMMx86(VanillaSpMMhip):
    """Constructor and knobs of the reference's VanillaSpMMx86
    (python/featgraph/module/spmm.py:197-209): source-column partitions at init,
    'num_feat_partitions' at build.  Both partitionings are carried out on the GPU."""
    _schedule_keys = ()


class VanillaSpMMcuda(VanillaSpMMhip):
    """Constructor and knobs of the reference's VanillaSpMMcuda
    (python/featgraph/module/spmm.py:212-220): no partitioning arguments."""
    _compute_keys = ()

    def __init__(self, adj_scipy):
        super(VanillaSpMMcuda, self).__init__(adj_scipy, num_col_partitions=1)
