"""SpMM module classes: the build()/run() surface of the reference's
python/featgraph/module/spmm.py, executing hand-written gfx950 kernels."""
import ctypes

import numpy as np
import torch

from .. import _lib
from .. import tuning
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
        if adj_scipy_csr.dtype != np.float32:
            # the kernels compute in fp32 whatever the matrix holds (e.g. scipy.sparse.random's float64)
            adj_scipy_csr = adj_scipy_csr.astype(np.float32)
        self._num_rows = adj_scipy_csr.shape[0]
        self._num_cols = adj_scipy_csr.shape[1]
        common.check_int32_sizes(self._num_rows, self._num_cols, adj_scipy_csr.nnz)
        assert num_col_partitions >= 1, "num_col_partitions should be larger than or equal to 1"
        self._num_col_partitions = num_col_partitions
        self._target = None
        self._ctx = None
        self._register()
        indptr = np.ascontiguousarray(adj_scipy_csr.indptr, dtype=np.int32)
        indices = np.ascontiguousarray(adj_scipy_csr.indices, dtype=np.int32)
        _lib.check(_lib.lib().fg_check_csr_host(self._num_rows, self._num_cols, _lib.host_ptr(indptr),
                                                _lib.host_ptr(indices)))
        self._adj_scipy_csr = adj_scipy_csr
        self._adj_indptr = indptr
        self._adj_indices = indices
        self._adj_vals = np.ascontiguousarray(adj_scipy_csr.data, dtype=np.float32)
        # device layouts by number of source-column partitions: 1 = CSR, P > 1 = DDS
        self._layouts = {}
        # 1D graph partitioning
        if self._num_col_partitions > 1:
            lay = self._layout(self._num_col_partitions)
            self._adj_s1_pos, self._adj_s1_idx, self._adj_vals = lay['host']
            self._adj_s1_pos_dev, self._adj_s1_idx_dev = lay['pos'], lay['idx']
            self.__dict__['_adj_vals_dev'] = lay['vals']
            self._adj_d1_size = self._num_col_partitions
            self._adj_d2_size = self._num_rows + 1
        # (one partition: the CSR arrays go to the device when something first needs them -- see _adj_indptr_dev below --
        # so a module whose build() picks source partitions holds the partitioned copy only)
        # To be updated in self.build
        self._func = None
        self._active = None
        self._placeholders = None
        self._feat_len = None
        self._num_feat_partitions = 0
        self._notes = []
        # To be updated in self.build; the same tensor is returned by every run()
        self.out_tvm = None

    def _layout(self, P):
        """Device arrays + load-balance plan for P source-column partitions (built once per P)."""
        if P in self._layouts:
            return self._layouts[P]
        if P > 1:
            pos, idx, vals = self._preprocess_adj(self._adj_scipy_csr, P)
            vals = np.ascontiguousarray(vals, dtype=np.float32)
        else:
            pos, idx, vals = self._adj_indptr, self._adj_indices, self._adj_vals
        lay = {'P': P, 'host': (pos, idx, vals),
               'pos': common.to_device_i32(pos, self._ctx), 'idx': common.to_device_i32(idx, self._ctx),
               'vals': common.to_device_f32(vals, self._ctx), 'plan': ctypes.c_void_p()}
        with torch.cuda.device(self._ctx):
            _lib.check(_lib.lib().fg_spmm_plan_create(_lib.host_ptr(pos), self._num_rows, self._num_cols, P, _lib.plan_opts_ptr(),
                                                      ctypes.byref(lay['plan'])))
        common.narrow_indices(lay['plan'], lay['idx'], self._num_cols, P, self._ctx)
        self._layouts[P] = lay
        return lay

    # The CSR layout's device arrays, for modules constructed with one partition (uploaded on first use).
    @property
    def _adj_indptr_dev(self):
        return self.__dict__['_adj_indptr_dev'] if '_adj_indptr_dev' in self.__dict__ else self._layout(1)['pos']

    @property
    def _adj_indices_dev(self):
        return self.__dict__['_adj_indices_dev'] if '_adj_indices_dev' in self.__dict__ else self._layout(1)['idx']

    @property
    def _adj_vals_dev(self):
        return self.__dict__['_adj_vals_dev'] if '_adj_vals_dev' in self.__dict__ else self._layout(1)['vals']

    @staticmethod
    def _destroy_layout(lay):
        plan = lay.get('plan')
        if plan is not None and plan.value:
            try:
                _lib.lib().fg_spmm_plan_destroy(plan)
            except Exception:
                pass
            lay['plan'] = None

    def share_layouts_with(self, other):
        """Uses the device layouts of `other` -- another SpMM-like module built on the same adjacency (same structure and
        values) -- instead of making its own: every partitioned copy, plan, 16-bit id copy and scratch exists once for the
        two (the scratch as large as the larger need).  To be called before build().  Their run() calls must follow each other
        on one stream, as two calls on one module must.  Keeps `other` alive; `other` stops freeing layouts on re-builds."""
        same = (self._num_rows, self._num_cols) == (other._num_rows, other._num_cols) \
            and np.array_equal(self._adj_indptr, other._adj_indptr) and np.array_equal(self._adj_indices, other._adj_indices) \
            and np.array_equal(self._adj_scipy_csr.data, other._adj_scipy_csr.data)
        if not same:
            raise ValueError("share_layouts_with needs a module built on the same adjacency")
        if self._layouts:
            raise RuntimeError("share_layouts_with must be called before the first build()")
        owner = getattr(other, '_layout_owner', None) or other
        owner._layout_sharers = getattr(owner, '_layout_sharers', 0) + 1
        self._layout_owner = owner
        self._layouts = owner._layouts

    def _release_unused_layouts(self):
        """Frees the partitioned copies (device arrays, plan, scratch) that the built configuration does not use; a
        later build() that wants one of them makes it again.  The constructor's own layout and the CSR arrays stay."""
        if getattr(self, '_layout_owner', None) is not None or getattr(self, '_layout_sharers', 0):
            return                  # the layouts serve several modules
        keep = {1, self._num_col_partitions, self._active['P']}
        for P in [P for P in self._layouts if P not in keep and not self._layouts[P].get('users')]:
            self._destroy_layout(self._layouts.pop(P))

    def device_bytes(self):
        """Device memory this module holds: {'graph': the adjacency's arrays in every layout kept, 'plans': work items,
        scratch, tile-by-tile copy and 16-bit ids of their plans (fg_spmm_plan_bytes), 'buffers': output and padding};
        layouts taken over from another module (share_layouts_with) are counted there."""
        graph = plans = 0
        for lay in ({} if getattr(self, '_layout_owner', None) is not None else self._layouts).values():
            graph += sum(t.numel() * t.element_size() for t in lay.values() if isinstance(t, torch.Tensor))
            plans += int(_lib.lib().fg_spmm_plan_bytes(lay['plan']))
        bufs = sum(t.numel() * t.element_size() for t in (self.out_tvm, getattr(self, '_x_pad', None), getattr(self, '_out_pad', None))
                   if isinstance(t, torch.Tensor))
        return {'graph': graph, 'plans': plans, 'buffers': bufs}

    def __del__(self):
        owner = getattr(self, '_layout_owner', None)
        if owner is not None:
            owner._layout_sharers = max(0, getattr(owner, '_layout_sharers', 1) - 1)
            return
        for lay in getattr(self, "_layouts", {}).values():
            self._destroy_layout(lay)

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
        # Source-column partitions: the constructor's count when it was given, else chosen for
        # the L2 size (the product is the same; the partitions' results are summed in partition order).
        P = self._num_col_partitions
        src_parts = schedule_args.get('num_src_partitions', 'auto')
        if P == 1 and src_parts is not None:
            auto_p, auto_t = tuning.choose_spmm(self._num_rows, self._num_cols, self._adj_indices.shape[0], feat_len,
                                                self._graph_stats())
            P = auto_p if src_parts == 'auto' else int(src_parts)
            if P < 1:
                raise ValueError("num_src_partitions must be >= 1")
            if T == 0:
                T = auto_t
            if P > 1:
                notes.append("%d source-column partitions chosen for the L2 size" % P)
        elif T == 0 and tuning.feature_tiles(feat_len) > 1:
            # the caller fixed the partitions but not the tiles: 64-float tiles across the XCDs
            # (tiling changes which workgroup computes a column, not the sums)
            T = tuning.feature_tiles(feat_len)
        return ph, feat_len, int(T), P, notes

    def _graph_stats(self):
        """Column reference counts and row degrees of the adjacency, as the tuning model reads them (once per object)."""
        if getattr(self, '_stats', None) is None:
            self._stats = tuning.GraphStats.from_csr(self._adj_indptr, self._adj_indices, self._num_cols)
        return self._stats

    def _tune(self, ph, compute_args, schedule_args, how_many):
        """Times the model's `how_many` most promising (partitions, tiles) on this graph (zero features:
        the kernels' time does not depend on the values) and returns the fastest as schedule / compute arguments."""
        feat_len = ph.shape[1]
        cands = tuning.rank_spmm(self._graph_stats(), feat_len)[:max(1, how_many)]
        x = torch.zeros(ph.shape, dtype=torch.float32, device=self._ctx)
        timed = []
        self._tuning = True             # candidates' layouts are kept until the choice is built
        try:
            for p, t in cands:
                ca = dict(compute_args, num_feat_partitions=t)
                sa = dict(schedule_args, num_src_partitions=(p if p > 1 else None))
                sa.pop('tune', None)
                self.build([ph], ca, sa)
                timed.append((self.measure_average_time([x], 3), p, t, ca, sa))
        finally:
            self._tuning = False
        timed.sort(key=lambda e: e[0])
        self._tuned = [(round(s * 1e3, 4), p, t) for s, p, t, _, _ in timed]
        return timed[0][3], timed[0][4]

    def build(self, input_placeholders, compute_args, schedule_args):
        """Fix the feature length and kernel variant, allocate the output once.

        Parameters
        ----------
        input_placeholders : list of placeholder
            The dense inputs other than adj: [SrcFeat (num_cols, feat_len)]

        compute_args : dict
            e.g. {'num_feat_partitions': T}: feature tiles handled by different workgroups

        schedule_args : dict
            The reference's CUDA keys 'num_cuda_blocks' / 'num_threads_per_cuda_block' are accepted.
            'num_src_partitions': 'auto' (default) | int | None -- source-column partitions used
            when the constructor was left at one partition (None: plain CSR).
            'tune': k -- time the cost model's k most promising (partitions, tiles) on this graph
            and keep the fastest (True: 6), in the manner of the reference's own sweeps
            (benchmark/bench_vanilla_spmm.py:36-41); only when neither knob was given.
        """
        tune = schedule_args.get('tune') if isinstance(schedule_args, dict) else None
        if tune and self._num_col_partitions == 1 and not compute_args.get('num_feat_partitions') \
                and schedule_args.get('num_src_partitions', 'auto') == 'auto' and len(input_placeholders) == 1:
            compute_args, schedule_args = self._tune(input_placeholders[0], dict(compute_args), dict(schedule_args),
                                                     6 if tune is True else int(tune))
        schedule_args = {k: v for k, v in schedule_args.items() if k != 'tune'}
        # Rows of an awkward length run at the next friendly one, on zero-padded copies (tuning.padded_feature_len)
        self._pad_from = None
        ph0 = input_placeholders[0] if len(input_placeholders) == 1 else None
        if ph0 is not None and len(ph0.shape) == 2 and schedule_args.get('pad_features', True) \
                and not compute_args.get('num_feat_partitions') and not schedule_args.get('num_threads_per_cuda_block'):
            want = tuning.padded_feature_len(ph0.shape[1])
            if want != ph0.shape[1] and self._adj_indices.shape[0] * ph0.shape[1] >= tuning.PAD_MIN_GATHERED:
                self._pad_from = ph0.shape[1]
                input_placeholders = [common.placeholder((ph0.shape[0], want))]
        schedule_args = {k: v for k, v in schedule_args.items() if k != 'pad_features'}
        ph, feat_len, T, P, notes = self._resolve(input_placeholders, compute_args, schedule_args)
        if self._pad_from is not None:
            notes.append("rows of %d floats run as rows of %d on zero-padded copies" % (self._pad_from, feat_len))
            ph = ph0
        self._placeholders = [ph]
        self._feat_len = feat_len
        self._num_feat_partitions = T
        self._notes = notes
        self._active = self._layout(P)
        if not getattr(self, '_tuning', False):
            self._release_unused_layouts()
        self._func = _lib.lib().fg_spmm_dds_f32 if P > 1 else _lib.lib().fg_spmm_csr_f32
        common.reserve(self._active['plan'], common.OP_SPMM_SUM, 1, feat_len, T, self._ctx)
        self._x_pad = self._out_pad = None
        if self._pad_from is not None:
            self._x_pad = torch.zeros((self._num_cols, feat_len), dtype=torch.float32, device=self._ctx)
            self._out_pad = torch.zeros((self._num_rows, feat_len), dtype=torch.float32, device=self._ctx)
        self.out_tvm = torch.zeros((self._num_rows, self._pad_from or feat_len), dtype=torch.float32, device=self._ctx)

    def lower_to_ir(self, input_placeholders, compute_args, schedule_args):
        """Return a text description of the plan and launch. This can be useful for debug."""
        _, feat_len, T, P, notes = self._resolve(input_placeholders, compute_args, schedule_args)
        buf = ctypes.create_string_buffer(4096)
        _lib.check(_lib.lib().fg_spmm_plan_describe(self._layout(P)['plan'], feat_len, T, buf, len(buf)))
        text = buf.value.decode()
        for n in notes:
            text += "  note             : %s\n" % n
        return text

    def _launch(self, src_feat):
        lay = self._active
        out = self.out_tvm
        if getattr(self, '_pad_from', None) is not None:
            self._x_pad[:, :self._pad_from].copy_(src_feat)         # the padding columns stay zero
            src_feat, out = self._x_pad, self._out_pad
        _lib.check(self._func(lay['plan'], _lib.dev_ptr(lay['pos']), _lib.dev_ptr(lay['idx']), _lib.dev_ptr(lay['vals']),
                              _lib.dev_ptr(src_feat), _lib.dev_ptr(out), self._feat_len,
                              self._num_feat_partitions, common.stream_ptr()))
        if out is not self.out_tvm:
            self.out_tvm.copy_(out[:, :self._pad_from])

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
        common.ensure_output(self)
        common.check_inputs(input_tvm_ndarrays, self._placeholders, self._ctx)
        self._launch(input_tvm_ndarrays[0])
        return self.out_tvm

    def measure_average_time(self, input_tvm_ndarrays, num_runs):
        """Average run time in seconds over `num_runs` back-to-back launches."""
        if self._func is None:
            raise RuntimeError("call build() before measure_average_time()")
        common.ensure_output(self)
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
    _schedule_keys = ('num_cuda_blocks', 'num_threads_per_cuda_block', 'num_src_partitions', 'tune', 'pad_features')

    def __init__(self, adj_scipy, num_col_partitions=1):
        super(VanillaSpMMhip, self).__init__(adj_scipy, num_col_partitions)

    def _register(self):
        self._target = 'rocm'
        self._ctx = common.device()


class VanillaSpMMx86(VanillaSpMMhip):
    """Constructor and knobs of the reference's VanillaSpMMx86
    (python/featgraph/module/spmm.py:197-209): source-column partitions at init,
    'num_feat_partitions' at build.  Both partitionings are carried out on the GPU."""
    _schedule_keys = ('num_src_partitions', 'tune', 'pad_features')


class VanillaSpMMcuda(VanillaSpMMhip):
    """Constructor and knobs of the reference's VanillaSpMMcuda
    (python/featgraph/module/spmm.py:212-220): no partitioning arguments."""
    _compute_keys = ()

    def __init__(self, adj_scipy):
        super(VanillaSpMMcuda, self).__init__(adj_scipy, num_col_partitions=1)
