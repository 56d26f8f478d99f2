"""SDDMM module classes: the build()/run() surface of the reference's
python/featgraph/module/sddmm.py, executing hand-written gfx950 kernels."""
import ctypes

import numpy as np
import torch

from .. import _lib
from .. import tuning
from ..util import util_convert_csr_to_dds, util_partition_adj_coo_2d
from . import common
from . import general


class SDDMMbase(object):
    """The base class for SDDMM-like computation kernels (python/featgraph/module/sddmm.py:11-165)."""

    def __init__(self, adj_scipy, num_row_partitions=1, num_col_partitions=1):
        """Doing 2D graph partitioning during init.

        Parameters
        ----------
        adj_scipy : scipy.sparse.coo_matrix or scipy.sparse.csr_matrix
            The input scipy sparse matrix (only its structure is used)

        num_row_partitions : int
            Number of partitions along the row dimension

        num_col_partitions : int
            Number of partitions along the col dimension (honoured; the reference overwrites
            it with num_row_partitions, python/featgraph/module/sddmm.py:37)
        """
        if adj_scipy.format != 'coo':
            adj_scipy_coo = adj_scipy.tocoo()
        else:
            adj_scipy_coo = adj_scipy
        self._num_rows = adj_scipy_coo.shape[0]
        self._num_cols = adj_scipy_coo.shape[1]
        common.check_int32_sizes(self._num_rows, self._num_cols, adj_scipy_coo.nnz)
        assert num_row_partitions >= 1, "num_row_partitions should be larger than or equal to 1"
        assert num_col_partitions >= 1, "num_col_partitions should be larger than or equal to 1"
        self._num_row_partitions = num_row_partitions
        self._num_col_partitions = num_col_partitions
        self._target = None
        self._ctx = None
        self._register()
        # 2D graph partitioning
        if self._num_row_partitions > 1 or self._num_col_partitions > 1:
            edge_id_list, adj_row_indices, adj_col_indices = self._preprocess_adj(
                adj_scipy_coo, self._num_row_partitions, self._num_col_partitions)
            self._edge_mapping = np.argsort(edge_id_list)
        else:
            adj_row_indices = np.ascontiguousarray(adj_scipy_coo.row, dtype=np.int32)
            adj_col_indices = np.ascontiguousarray(adj_scipy_coo.col, dtype=np.int32)
            self._edge_mapping = None
        nnz = adj_row_indices.shape[0]
        if nnz:
            if adj_row_indices.min() < 0 or adj_row_indices.max() >= self._num_rows or \
                    adj_col_indices.min() < 0 or adj_col_indices.max() >= self._num_cols:
                raise ValueError("edge endpoints outside the %d x %d matrix" % (self._num_rows, self._num_cols))
        self._adj_row_indices = adj_row_indices
        self._adj_col_indices = adj_col_indices
        # (the stored row / col arrays go to the device when something first needs them -- see _adj_row_indices_dev
        # below -- so a module that only ever runs the tiled traversal holds the partitioned copy only)
        self._share_from = None
        # Stored order with non-decreasing row ids is CSR order: row pieces from the SpMM plan
        # then replace the per-edge row array and dst rows are fetched once per piece.
        self._plan = ctypes.c_void_p()
        self._adj_indptr_dev = None
        self._row_sorted = bool(nnz == 0 or (np.diff(adj_row_indices) >= 0).all())
        if self._row_sorted:
            counts = np.bincount(adj_row_indices, minlength=self._num_rows) if nnz else np.zeros(self._num_rows, np.int64)
            indptr = np.zeros(self._num_rows + 1, dtype=np.int32)
            np.cumsum(counts, out=indptr[1:])
            self._adj_indptr = indptr
            self._adj_indptr_dev = common.to_device_i32(indptr, self._ctx)
            with torch.cuda.device(self._ctx):
                _lib.check(_lib.lib().fg_spmm_plan_create(_lib.host_ptr(indptr), self._num_rows, self._num_cols,
                                                          1, _lib.plan_opts_ptr(), ctypes.byref(self._plan)))
        # source-column-partitioned copies of the edge list for the tiled traversal, by P
        self._dds = {}
        # To be updated in self.build
        self._func = None
        self._placeholders = None
        self._tiled = None
        self._heads = 1
        self._head_len = None
        self._use_csr = False
        self._notes = []
        self.out_tvm = None

    # The stored edge list's device arrays (uploaded on first use).
    @property
    def _adj_row_indices_dev(self):
        if '_row_dev' not in self.__dict__:
            self.__dict__['_row_dev'] = common.to_device_i32(self._adj_row_indices, self._ctx)
        return self.__dict__['_row_dev']

    @property
    def _adj_col_indices_dev(self):
        if '_col_dev' not in self.__dict__:
            self.__dict__['_col_dev'] = common.to_device_i32(self._adj_col_indices, self._ctx)
        return self.__dict__['_col_dev']

    def _upload_edge_list(self):
        return self._adj_row_indices_dev, self._adj_col_indices_dev

    def share_layouts(self, spmm_module):
        """Lets the tiled traversal use the partitioned copies of an SpMM module built on the same adjacency -- the
        position and column arrays, the 16-bit ids, the plan and its scratch -- instead of making its own (at the
        benchmark size: 0.7 GB of arrays and up to 3.7 GB of scratch less per shared layout).  Needs stored edges in CSR
        order with exactly that module's structure.  The two modules then share one scratch: their run() calls must
        follow each other on one stream, as two calls on one module must.  Keeps `spmm_module` alive."""
        ok = self._row_sorted and (self._num_rows, self._num_cols) == (spmm_module._num_rows, spmm_module._num_cols) \
            and np.array_equal(self._adj_col_indices, spmm_module._adj_indices) \
            and np.array_equal(getattr(self, '_adj_indptr', None), spmm_module._adj_indptr)
        if not ok:
            raise ValueError("share_layouts needs stored edges in CSR order with the same structure as the SpMM module's adjacency")
        self._share_from = spmm_module

    @staticmethod
    def _destroy_plan(plan):
        if plan is not None and plan.value:
            try:
                _lib.lib().fg_spmm_plan_destroy(plan)
            except Exception:
                pass
            plan.value = None

    def _drop_dds(self, P):
        d = self._dds.pop(P)
        if d.get('shared_with') is not None:
            d['shared_with']['users'] = d['shared_with'].get('users', 1) - 1
        else:
            self._destroy_plan(d['plan'])

    def device_bytes(self):
        """Device memory this module holds: {'graph': the stored edge list and the partitioned copies it made itself,
        'plans': work items, scratch, tile-by-tile copy and 16-bit ids of its own plans (fg_spmm_plan_bytes),
        'buffers': output and padding}; what it shares with an SpMM module is counted there."""
        tensors = [self.__dict__.get('_row_dev'), self.__dict__.get('_col_dev'), self._adj_indptr_dev]
        plans = int(_lib.lib().fg_spmm_plan_bytes(self._plan)) if self._plan.value else 0
        for d in self._dds.values():
            tensors.append(d['edge_pos'])
            if d.get('shared_with') is None:
                tensors += [d['pos'], d['idx']]
                plans += int(_lib.lib().fg_spmm_plan_bytes(d['plan']))
        size = lambda ts: sum(t.numel() * t.element_size() for t in ts if isinstance(t, torch.Tensor))
        return {'graph': size(tensors), 'plans': plans,
                'buffers': size([self.out_tvm, getattr(self, '_src_pad', None), getattr(self, '_dst_pad', None)])}

    def __del__(self):
        self._destroy_plan(getattr(self, "_plan", None))
        for P in list(getattr(self, "_dds", {})):
            self._drop_dds(P)

    def _dds_layout(self, P):
        """DDS copy of the stored edges (P source-column partitions, CSR inside each) with, per
        traversed edge, its position in the stored order; device arrays + plan, built once per P."""
        if P in self._dds:
            return self._dds[P]
        import scipy.sparse
        nnz = self._adj_row_indices.shape[0]
        if self._share_from is not None and P > 1:
            src = self._share_from._layout(P)
            src['users'] = src.get('users', 0) + 1
            # stored order is CSR order: a traversed edge's stored position is its position in the DDS copy's own CSR
            # numbering, which the conversion of the position numbers 0 .. nnz-1 gives
            csr = scipy.sparse.csr_matrix((np.arange(nnz, dtype=np.int32), self._adj_col_indices, self._adj_indptr),
                                          shape=(self._num_rows, self._num_cols))
            _, _, edge_pos = util_convert_csr_to_dds(csr, P)
            d = {'P': P, 'pos': src['pos'], 'idx': src['idx'], 'edge_pos': common.to_device_i32(edge_pos, self._ctx),
                 'plan': src['plan'], 'shared_with': src}
            self._dds[P] = d
            return d
        if self._row_sorted:
            order = None                        # stored order is already CSR order
            indptr = np.zeros(self._num_rows + 1, dtype=np.int32)
            np.cumsum(np.bincount(self._adj_row_indices, minlength=self._num_rows), out=indptr[1:])
            indices = self._adj_col_indices
            positions = np.arange(nnz, dtype=np.int32)
        else:
            # stable sort by (row, col), i.e. np.lexsort((col, row)), on the device: seconds instead of a minute at 1e8 edges
            key = self._adj_row_indices_dev.long() * self._num_cols + self._adj_col_indices_dev.long()
            order = torch.sort(key, stable=True).indices.to(torch.int32).cpu().numpy()
            del key
            indptr = np.zeros(self._num_rows + 1, dtype=np.int32)
            np.cumsum(np.bincount(self._adj_row_indices, minlength=self._num_rows), out=indptr[1:])
            indices = self._adj_col_indices[order]
            positions = order
        csr = scipy.sparse.csr_matrix((positions, indices, indptr), shape=(self._num_rows, self._num_cols))
        s1_pos, s1_idx, edge_pos = util_convert_csr_to_dds(csr, P)
        d = {'P': P, 'pos': common.to_device_i32(s1_pos, self._ctx), 'idx': common.to_device_i32(s1_idx, self._ctx),
             'edge_pos': common.to_device_i32(edge_pos, self._ctx), 'plan': ctypes.c_void_p()}
        with torch.cuda.device(self._ctx):
            _lib.check(_lib.lib().fg_spmm_plan_create(_lib.host_ptr(s1_pos), self._num_rows, self._num_cols, P, _lib.plan_opts_ptr(),
                                                      ctypes.byref(d['plan'])))
        common.narrow_indices(d['plan'], d['idx'], self._num_cols, P, self._ctx)
        self._dds[P] = d
        return d

    def _preprocess_adj(self, adj_scipy_coo, num_row_partitions=1, num_col_partitions=1):
        return util_partition_adj_coo_2d(adj_scipy_coo, num_row_partitions, num_col_partitions)

    def _register(self):
        raise NotImplementedError("Please register target and ctx.")

    def _feature_shape(self, src_ph, dst_ph):
        """(H, D) from the two placeholders; vanilla SDDMM takes 2-D inputs."""
        if len(src_ph.shape) != 2 or len(dst_ph.shape) != 2:
            raise ValueError("SrcFeat / DstFeat must be 2-D, got %s and %s" % (src_ph.shape, dst_ph.shape))
        return 1, src_ph.shape[1]

    def _resolve(self, input_placeholders, compute_args, schedule_args):
        compute_args = common.take_args(compute_args, self._compute_keys, "compute_func")
        schedule_args = common.take_args(schedule_args, self._schedule_keys, "schedule_func")
        if len(input_placeholders) != 2:
            raise ValueError("SDDMM takes two dense inputs (SrcFeat, DstFeat), got %d" % len(input_placeholders))
        src_ph, dst_ph = input_placeholders
        assert src_ph.shape[1:] == dst_ph.shape[1:], "dimension mismatch"
        if src_ph.shape[0] != self._num_cols or dst_ph.shape[0] != self._num_rows:
            raise ValueError("SrcFeat must have num_cols=%d rows and DstFeat num_rows=%d rows, got %s and %s"
                             % (self._num_cols, self._num_rows, src_ph.shape, dst_ph.shape))
        H, D = self._feature_shape(src_ph, dst_ph)
        notes = []
        T = compute_args.get('num_feat_partitions', 1) or 1
        Ts = schedule_args.get('num_feat_partitions', T) or 1
        for t in (T, Ts):
            if t < 1 or (H * D) % t != 0:
                raise ValueError("feat_len %d is not divisible by num_feat_partitions %d" % (H * D, t))
        # The reference's knob (python/featgraph/op/vanilla_sddmm.py:48-60) asks for T feature tiles; it
        # becomes the tiled traversal's tile count when F / T is a tile width the kernel takes.
        knob = T if T != 1 else Ts
        knob_tiles = None
        if knob != 1:
            tile_w = (H * D) // knob
            legal = tile_w % 4 == 0 and 16 <= tile_w <= 256 and (tile_w & (tile_w - 1)) == 0 and \
                (H == 1 or tile_w % D == 0 or D == tile_w)
            if legal:
                knob_tiles = knob
            else:
                notes.append("num_feat_partitions=%d gives tiles of %d floats; the kernel takes power-of-two tiles of "
                             "16..256 floats, so the default tiling is used" % (knob, tile_w))
        blocks = schedule_args.get('num_cuda_blocks')
        if blocks is not None:
            # same bound as schedule_vanilla_sddmm_cuda_tree_reduce (vanilla_sddmm.py:82-83)
            assert blocks <= self._adj_row_indices.shape[0], \
                "num_cuda_blocks must be smaller than num_edges, which is {}.".format(self._adj_row_indices.shape[0])
            notes.append("num_cuda_blocks has no counterpart: the grid follows the edge count")
        order = schedule_args.get('order', 'auto')
        if order not in ('auto', 'csr', 'coo', 'tiled'):
            raise ValueError("order must be 'auto', 'csr', 'coo' or 'tiled'")
        if order == 'csr' and not self._row_sorted:
            raise ValueError("order='csr' needs stored edges with non-decreasing row ids")
        # 'auto' takes the stored edges as they are (the COO kernel): on five graphs it is level with the CSR-order kernel
        # at F <= 128 and 4-15 % ahead at F = 512 or on low-degree graphs; order='csr' asks for the CSR-order kernel
        use_csr = self._row_sorted and order == 'csr'
        # Tiled traversal for feature matrices beyond the L2: (source partitions, feature tiles)
        tiled = None
        nnz = self._adj_row_indices.shape[0]
        if order in ('auto', 'tiled') and nnz > 0:
            tiled = tuning.choose_sddmm(self._num_rows, self._num_cols, nnz, H, D, self._graph_stats() if H == 1 else None)
            p_arg, t_arg = schedule_args.get('num_src_partitions'), schedule_args.get('num_feat_tiles')
            if t_arg is None and knob_tiles is not None and order != 'coo' and order != 'csr':
                t_arg = knob_tiles
            if order == 'tiled' or p_arg is not None or t_arg is not None:
                base = tiled or (1, 1)
                tiled = (int(p_arg) if p_arg is not None else base[0], int(t_arg) if t_arg is not None else base[1])
            if tiled is not None:
                notes.append("tiled traversal: %d source-column partitions x %d feature tiles; results are "
                             "written back in the stored edge order" % tiled)
        return [src_ph, dst_ph], H, D, use_csr, tiled, notes

    def _graph_stats(self):
        """Column reference counts and row degrees of the adjacency, as the tuning model reads them (once per object)."""
        if getattr(self, '_stats', None) is None:
            counts = np.bincount(self._adj_col_indices, minlength=self._num_cols) if len(self._adj_col_indices) else np.zeros(self._num_cols, np.int64)
            degs = np.bincount(self._adj_row_indices, minlength=self._num_rows) if len(self._adj_row_indices) else np.zeros(self._num_rows, np.int64)
            cv, cm = np.unique(counts, return_counts=True)
            dv, dm = np.unique(degs, return_counts=True)
            self._stats = tuning.GraphStats(self._num_rows, self._num_cols, len(self._adj_col_indices), cv, cm, dv, dm)
        return self._stats

    def _tune(self, phs, compute_args, schedule_args, how_many):
        """Times the stored-order kernel(s) and the cost model's `how_many` most promising tiled traversals on
        this graph (zero features: the kernels' time does not depend on the values); returns the fastest's schedule arguments."""
        H, D = self._feature_shape(*phs)
        cands = [{'order': 'coo'}] + ([{'order': 'csr'}] if self._row_sorted else [])
        if H == 1:
            for p, t in tuning.rank_sddmm(self._graph_stats(), D)[:max(1, how_many)]:
                tile = D // t
                if (p, t) != (1, 1) and tile <= 256 and tile >= 16 and (tile & (tile - 1)) == 0:
                    cands.append({'order': 'tiled', 'num_src_partitions': p, 'num_feat_tiles': t})
        else:
            cands.append({})
        src = torch.zeros(phs[0].shape, dtype=torch.float32, device=self._ctx)
        dst = torch.zeros(phs[1].shape, dtype=torch.float32, device=self._ctx)
        timed = []
        self._tuning = True             # candidates' layouts are kept until the choice is built
        try:
            for extra in cands:
                sa = {k: v for k, v in schedule_args.items() if k != 'tune'}
                sa.update(extra)
                try:
                    self.build(phs, compute_args, sa)
                except ValueError:
                    continue
                timed.append((self.measure_average_time([src, dst], 3), sa))
        finally:
            self._tuning = False
        timed.sort(key=lambda e: e[0])
        self._tuned = [(round(s * 1e3, 4), sa) for s, sa in timed]
        return timed[0][1]

    def build(self, input_placeholders, compute_args, schedule_args):
        """Fix the feature shape and kernel variant, allocate the output once.

        Parameters
        ----------
        input_placeholders : list of placeholder
            [SrcFeat (num_cols, feat_len), DstFeat (num_rows, feat_len)]

        compute_args : dict
            {'num_feat_partitions': T}: T feature tiles handled by different workgroups (the tiled
            traversal), when feat_len / T is a power of two between 16 and 256; otherwise a note is
            recorded (see lower_to_ir) and the default tiling applies

        schedule_args : dict
            'num_feat_partitions', 'num_cuda_blocks' (reference keys); 'order' in
            {'auto', 'csr', 'coo', 'tiled'}: which kernel walks the edges ('auto' picks the tiled
            traversal when the feature matrices exceed the L2); 'num_src_partitions' /
            'num_feat_tiles': override the tiled traversal's shape; 'tune': k -- time the stored-order
            kernels and the cost model's k most promising tiled traversals on this graph and keep the
            fastest (True: 6), in the manner of the reference's own sweeps
            (benchmark/bench_vanilla_sddmm.py:41-46); only when no order / shape was given
        """
        tune = schedule_args.get('tune')
        if tune and len(input_placeholders) == 2 and not any(k in schedule_args for k in ('order', 'num_src_partitions', 'num_feat_tiles')) \
                and (compute_args.get('num_feat_partitions', 1) or 1) == 1 and self._adj_row_indices.shape[0] > 0:
            schedule_args = self._tune(list(input_placeholders), dict(compute_args), dict(schedule_args), 6 if tune is True else int(tune))
        schedule_args = {k: v for k, v in schedule_args.items() if k != 'tune'}
        # Single-head rows of an awkward length run at the next friendly one, on zero-padded copies of both operands
        # (tuning.padded_feature_len): the extra columns add zeros to every dot product.
        self._pad_from = None
        given = list(input_placeholders)
        if len(given) == 2 and len(given[0].shape) == 2 and len(given[1].shape) == 2 and given[0].shape[1] == given[1].shape[1] \
                and schedule_args.get('pad_features', True) and not compute_args.get('num_feat_partitions') \
                and not any(schedule_args.get(k) for k in ('num_feat_partitions', 'num_feat_tiles')):
            D0 = given[0].shape[1]
            want = tuning.padded_feature_len(D0)
            if want != D0 and self._adj_row_indices.shape[0] * D0 >= tuning.PAD_MIN_GATHERED:
                self._pad_from = D0
                input_placeholders = [common.placeholder((given[0].shape[0], want)), common.placeholder((given[1].shape[0], want))]
        elif len(given) == 2 and len(given[0].shape) == 3 and tuple(given[0].shape[1:]) == tuple(given[1].shape[1:]) \
                and schedule_args.get('pad_features', True) and not compute_args.get('num_feat_partitions') \
                and not any(schedule_args.get(k) for k in ('num_feat_partitions', 'num_feat_tiles')):
            # several heads: every head padded to a length that fills whole lane groups (tuning.padded_head_len)
            H0, D0 = given[0].shape[1], given[0].shape[2]
            want = tuning.padded_head_len(D0)
            if want != D0 and self._adj_row_indices.shape[0] * H0 * D0 >= tuning.PAD_MIN_GATHERED:
                self._pad_from = D0
                input_placeholders = [common.placeholder((given[0].shape[0], H0, want)), common.placeholder((given[1].shape[0], H0, want))]
        schedule_args = {k: v for k, v in schedule_args.items() if k != 'pad_features'}
        phs, H, D, use_csr, tiled, notes = self._resolve(input_placeholders, compute_args, schedule_args)
        self._src_pad = self._dst_pad = None
        if self._pad_from is not None:
            notes.append("rows of %d floats run as rows of %d on zero-padded copies" % (self._pad_from, D))
            phs = given
            tail = (D,) if len(given[0].shape) == 2 else (H, D)
            self._src_pad = torch.zeros((self._num_cols,) + tail, dtype=torch.float32, device=self._ctx)
            self._dst_pad = torch.zeros((self._num_rows,) + tail, dtype=torch.float32, device=self._ctx)
        self._placeholders = phs
        self._heads, self._head_len, self._use_csr, self._notes = H, D, use_csr, notes
        self._tiled = None
        if tiled is not None:
            self._tiled = (self._dds_layout(tiled[0]), tiled[1])
            if not getattr(self, '_tuning', False):
                for P in [P for P in self._dds if P != tiled[0]]:
                    self._drop_dds(P)          # partitioned copies the built configuration does not use
            common.reserve(self._tiled[0]['plan'], common.OP_SDDMM_DDS, H, D, tiled[1], self._ctx)
        self._func = _lib.lib().fg_sddmm_csr_f32 if use_csr else _lib.lib().fg_sddmm_coo_f32
        if self._tiled is None:
            self._upload_edge_list()           # the stored-order kernels read it; run() itself must not upload anything
        nnz = self._adj_row_indices.shape[0]
        oshape = (nnz,) if self._out_1d else (nnz, H)
        self.out_tvm = torch.zeros(oshape, dtype=torch.float32, device=self._ctx)

    def lower_to_ir(self, input_placeholders, compute_args, schedule_args):
        """Return a text description of the launch. This can be useful for debug."""
        _, H, D, use_csr, tiled, notes = self._resolve(input_placeholders, compute_args, schedule_args)
        nnz = self._adj_row_indices.shape[0]
        text = "featgraph-hip SDDMM (gfx950)\n"
        text += "  adjacency        : %d x %d, %d stored edges, %d x %d partition blocks\n" % (
            self._num_rows, self._num_cols, nnz, self._num_row_partitions, self._num_col_partitions)
        text += "  features         : %d head(s) x %d floats\n" % (H, D)
        text += "  kernel           : %s\n" % ("sddmm_tiled_kernel over a source-column-partitioned edge list" if tiled
                                               else "sddmm_csr_kernel over row pieces (dst row held in registers)"
                                               if use_csr else "sddmm_coo_kernel, 256 stored edges per wavefront")
        if tiled:
            P, T = tiled
            conc = min(8 // T, P) if (T < 8 and 8 % T == 0) else 1
            text += "  traversal        : %d source-column partition(s) x %d feature tile(s) of %d floats; %d partition(s) per launch, %d launch(es)\n" % (
                P, T, H * D // T, conc, (P + conc - 1) // conc)
        for n in notes:
            text += "  note             : %s\n" % n
        return text

    def _launch(self, src_feat, dst_feat):
        s = common.stream_ptr()
        if getattr(self, '_pad_from', None) is not None:
            self._src_pad[..., :self._pad_from].copy_(src_feat)     # the padding columns stay zero
            self._dst_pad[..., :self._pad_from].copy_(dst_feat)
            src_feat, dst_feat = self._src_pad, self._dst_pad
        if self._tiled is not None:
            d, T = self._tiled
            _lib.check(_lib.lib().fg_sddmm_dds_f32(d['plan'], _lib.dev_ptr(d['pos']), _lib.dev_ptr(d['idx']),
                                                   _lib.dev_ptr(d['edge_pos']), _lib.dev_ptr(src_feat),
                                                   _lib.dev_ptr(dst_feat), _lib.dev_ptr(self.out_tvm),
                                                   self._heads, self._head_len, T, s))
        elif self._use_csr:
            _lib.check(self._func(self._plan, _lib.dev_ptr(self._adj_indptr_dev), _lib.dev_ptr(self._adj_col_indices_dev),
                                  _lib.dev_ptr(src_feat), _lib.dev_ptr(dst_feat), _lib.dev_ptr(self.out_tvm),
                                  self._heads, self._head_len, s))
        else:
            _lib.check(self._func(_lib.dev_ptr(self._adj_row_indices_dev), _lib.dev_ptr(self._adj_col_indices_dev),
                                  self._adj_row_indices.shape[0], _lib.dev_ptr(src_feat), _lib.dev_ptr(dst_feat),
                                  _lib.dev_ptr(self.out_tvm), self._heads, self._head_len, s))

    def run(self, input_tvm_ndarrays):
        """Run the built func with the given inputs [SrcFeat, DstFeat] (float32 torch tensors on
        the module's device).  Returns self.out_tvm, one value per stored edge (and head), in the
        stored (possibly partitioned) edge order; enqueued on torch's current stream."""
        if self._func is None:
            raise RuntimeError("call build() before run()")
        common.ensure_output(self)
        common.check_inputs(input_tvm_ndarrays, self._placeholders, self._ctx)
        self._launch(input_tvm_ndarrays[0], input_tvm_ndarrays[1])
        return self.out_tvm

    def measure_average_time(self, input_tvm_ndarrays, num_runs):
        """Average run time in seconds over `num_runs` back-to-back launches."""
        if self._func is None:
            raise RuntimeError("call build() before measure_average_time()")
        common.ensure_output(self)
        common.check_inputs(input_tvm_ndarrays, self._placeholders, self._ctx)
        s, d = input_tvm_ndarrays
        return common.timed_mean_seconds(lambda: self._launch(s, d), num_runs)

    @property
    def edge_mapping(self):
        assert self._target != 'cuda', "no graph partitioning on cuda, no edge_mapping"
        assert self._num_row_partitions > 1 or self._num_col_partitions > 1, \
            "no graph partitioning, no edge_mapping"
        return self._edge_mapping

    @property
    def ctx(self):
        return self._ctx

    @property
    def target(self):
        return self._target


class VanillaSDDMMhip(SDDMMbase):
    """Edge-wise dot product on gfx950, optionally over a 2-D partitioned edge order."""
    _compute_keys = ('num_feat_partitions',)
    _schedule_keys = ('num_feat_partitions', 'num_cuda_blocks', 'order', 'num_src_partitions', 'num_feat_tiles', 'tune', 'pad_features')
    _out_1d = True

    def __init__(self, adj_scipy, num_row_partitions=1, num_col_partitions=1):
        super(VanillaSDDMMhip, self).__init__(adj_scipy, num_row_partitions, num_col_partitions)

    def _register(self):
        self._target = 'rocm'
        self._ctx = common.device()


class VanillaSDDMMx86(VanillaSDDMMhip):
    """Constructor and knobs of the reference's VanillaSDDMMx86
    (python/featgraph/module/sddmm.py:168-176); the partitioned traversal runs on the GPU."""
    _schedule_keys = ('num_feat_partitions', 'order', 'num_src_partitions', 'num_feat_tiles', 'tune', 'pad_features')


class VanillaSDDMMcuda(VanillaSDDMMhip):
    """Constructor and knobs of the reference's VanillaSDDMMcuda
    (python/featgraph/module/sddmm.py:179-187): no partitioning, hence no edge_mapping."""
    _schedule_keys = ('num_feat_partitions', 'num_cuda_blocks', 'order', 'num_src_partitions', 'num_feat_tiles', 'tune', 'pad_features')

    def __init__(self, adj_scipy):
        super(VanillaSDDMMcuda, self).__init__(adj_scipy, num_row_partitions=1, num_col_partitions=1)

    @property
    def edge_mapping(self):
        raise AssertionError("no graph partitioning on cuda, no edge_mapping")


class MultiHeadSDDMMhip(VanillaSDDMMhip):
    """Per-edge, per-head dot products: SrcFeat (num_cols, H, D), DstFeat (num_rows, H, D),
    output (num_edges, H).  Not present in the reference; H == 1 equals VanillaSDDMM."""
    _out_1d = False

    def _feature_shape(self, src_ph, dst_ph):
        if len(src_ph.shape) != 3 or len(dst_ph.shape) != 3:
            raise ValueError("multi-head SrcFeat / DstFeat must be 3-D [n, H, D], got %s and %s"
                             % (src_ph.shape, dst_ph.shape))
        return src_ph.shape[1], src_ph.shape[2]


class GSDDMMhip(VanillaSDDMMhip):
    """Generalised SDDMM.  compute_args:
      'op'         : 'dot' | 'add' | 'sub' | 'mul' | 'div' | 'copy_lhs' | 'copy_rhs'   (default 'dot')
      'lhs_target' : 'u' | 'v' | 'e'   (default 'u': the first input is indexed by the edge's column)
      'rhs_target' : 'u' | 'v' | 'e'   (default 'v': the second input is indexed by the edge's row)
    'dot' with the default targets and equal shapes is VanillaSDDMMhip (2-D inputs) or MultiHeadSDDMMhip (3-D
    inputs, one result per head) and the element-wise
    'add' / 'sub' / 'mul' with the default targets and equal 2-D shapes give out[e, :] = SrcFeat[col[e], :]
    op DstFeat[row[e], :].  Everything else goes to the library's broadcasting kernel: an operand on 'u' has
    num_cols rows, on 'v' num_rows rows, on 'e' one row per stored edge, in the stored edge order (what
    edge_mapping refers to); the feature shapes broadcast against each other the numpy way; 'dot' contracts
    the last axis.  out is (num_edges,) + the broadcast
    shape, in the stored edge order.
    Not present in the reference (README.md:9-11 names it)."""
    _compute_keys = ('num_feat_partitions', 'op', 'lhs_target', 'rhs_target')
    _EDGE_OPS = {'add': 0, 'sub': 1, 'mul': 2}

    def _feature_shape(self, src_ph, dst_ph):
        if len(src_ph.shape) == 3 and len(dst_ph.shape) == 3:
            return src_ph.shape[1], src_ph.shape[2]
        return super(GSDDMMhip, self)._feature_shape(src_ph, dst_ph)

    def build(self, input_placeholders, compute_args, schedule_args):
        compute_args = dict(compute_args)
        self._op = compute_args.pop('op', 'dot')
        lt = compute_args.pop('lhs_target', 'u')
        rt = compute_args.pop('rhs_target', 'v')
        self._bop = None
        if self._op not in general.BINARY:
            raise ValueError("op must be one of %s" % sorted(general.BINARY))
        self._swap_inputs = False
        if self._op == 'dot' and (lt, rt) == ('v', 'u') and len(input_placeholders) == 2:
            # a dot product does not care which operand comes first: (DstFeat, SrcFeat) is the dot-product kernels' pair
            lt, rt, input_placeholders = 'u', 'v', [input_placeholders[1], input_placeholders[0]]
            self._swap_inputs = True
        same = (lt, rt) == ('u', 'v') and len(input_placeholders) == 2 and \
            input_placeholders[0].shape[1:] == input_placeholders[1].shape[1:]
        plain = same and len(input_placeholders[0].shape) == 2
        self._out_1d = True
        if self._op == 'dot' and same and len(input_placeholders[0].shape) in (2, 3):
            # the dot-product kernels proper: single head (2-D inputs) or one result per head (3-D inputs)
            self._out_1d = len(input_placeholders[0].shape) == 2
            return super(GSDDMMhip, self).build(input_placeholders, compute_args, schedule_args)
        if plain and self._op in self._EDGE_OPS:
            phs, H, D, _, _, notes = self._resolve(input_placeholders, compute_args, dict(schedule_args, order='coo'))
            self._placeholders, self._heads, self._head_len, self._notes = phs, H, D, notes
            self._tiled, self._use_csr = None, False
            self._upload_edge_list()
            self._func = _lib.lib().fg_gsddmm_elementwise_f32
            self.out_tvm = torch.zeros((self._adj_row_indices.shape[0], H * D), dtype=torch.float32, device=self._ctx)
            return
        common.take_args(compute_args, self._compute_keys, "compute_func")
        common.take_args(schedule_args, self._schedule_keys, "schedule_func")
        single = self._op in ('copy_lhs', 'copy_rhs')
        if len(input_placeholders) != (1 if single else 2):
            raise ValueError("op %r takes %d input(s), got %d" % (self._op, 1 if single else 2, len(input_placeholders)))
        nnz = self._adj_row_indices.shape[0]
        if single:
            # one operand: it is the left one of the library call
            target = lt if self._op == 'copy_lhs' else rt
            bop = general.BroadcastOp('copy_lhs', target, None, input_placeholders[0], None,
                                      self._num_rows, self._num_cols, nnz, self._ctx, allow_v=True)
        else:
            bop = general.BroadcastOp(self._op, lt, rt, input_placeholders[0], input_placeholders[1],
                                      self._num_rows, self._num_cols, nnz, self._ctx, allow_v=True)
        self._bop = bop
        self._placeholders = list(input_placeholders)
        self._heads, self._head_len = 1, bop.out_len
        self._notes = [bop.describe()]
        self._tiled, self._use_csr = None, False
        self._upload_edge_list()
        self._func = _lib.lib().fg_gsddmm_bcast_f32
        self.out_tvm = torch.zeros((nnz,) + tuple(bop.out_shape), dtype=torch.float32, device=self._ctx)

    def _launch(self, src_feat, dst_feat):
        if getattr(self, '_op', 'dot') == 'dot' and self._bop is None:
            return super(GSDDMMhip, self)._launch(src_feat, dst_feat)
        if self._bop is not None:
            self._bop.run_sddmm(self._adj_row_indices_dev, self._adj_col_indices_dev, self._adj_row_indices.shape[0],
                                src_feat, dst_feat, self.out_tvm)
            return
        _lib.check(self._func(_lib.dev_ptr(self._adj_row_indices_dev), _lib.dev_ptr(self._adj_col_indices_dev),
                              self._adj_row_indices.shape[0], _lib.dev_ptr(src_feat), _lib.dev_ptr(dst_feat),
                              _lib.dev_ptr(self.out_tvm), self._heads * self._head_len,
                              self._EDGE_OPS[self._op], common.stream_ptr()))

    def run(self, input_tvm_ndarrays):
        if self._func is None:
            raise RuntimeError("call build() before run()")
        if getattr(self, '_swap_inputs', False):
            input_tvm_ndarrays = list(input_tvm_ndarrays)[::-1]
        if self._bop is None:
            return super(GSDDMMhip, self).run(input_tvm_ndarrays)
        common.ensure_output(self)
        common.check_inputs(input_tvm_ndarrays, self._placeholders, self._ctx)
        self._launch(input_tvm_ndarrays[0], input_tvm_ndarrays[1] if len(input_tvm_ndarrays) > 1 else None)
        return self.out_tvm

    def measure_average_time(self, input_tvm_ndarrays, num_runs):
        if self._func is None:
            raise RuntimeError("call build() before measure_average_time()")
        if getattr(self, '_swap_inputs', False):
            input_tvm_ndarrays = list(input_tvm_ndarrays)[::-1]
        if self._bop is None:
            return super(GSDDMMhip, self).measure_average_time(input_tvm_ndarrays, num_runs)
        common.ensure_output(self)
        common.check_inputs(input_tvm_ndarrays, self._placeholders, self._ctx)
        a = input_tvm_ndarrays[0]
        b = input_tvm_ndarrays[1] if len(input_tvm_ndarrays) > 1 else None
        return common.timed_mean_seconds(lambda: self._launch(a, b), num_runs)
