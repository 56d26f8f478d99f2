"""Host-side graph partitioning, executed by the C++ routines of libfeatgraph_hip.so.

Same names, arguments and return values as the reference's
python/featgraph/util/adj_partitioning.py (:7-57 and :60-128).
"""
import numpy as np

from .. import _lib


def util_convert_csr_to_dds(adj_scipy_csr, num_col_partitions):
    """Src-vertex (column) partitioning: CSR -> DDS (dense-dense-sparse).

    Returns
    -------
    s1_pos : int32 [num_col_partitions * (num_rows + 1)]
    s1_idx : int32 [nnz], partition-local column ids
    vals   : [nnz], dtype of ``adj_scipy_csr.data`` (any dtype, as in the reference; values that are
             not 32 bits wide are permuted on the host through the positions the library returns)
    """
    assert num_col_partitions >= 1, "num_col_partitions should be larger than or equal to 1"
    num_rows, num_cols = adj_scipy_csr.shape
    indptr = np.ascontiguousarray(adj_scipy_csr.indptr, dtype=np.int32)
    indices = np.ascontiguousarray(adj_scipy_csr.indices, dtype=np.int32)
    data = np.ascontiguousarray(adj_scipy_csr.data)
    moved = None
    if data.dtype.itemsize != 4:
        if indices.shape[0] >= 2 ** 31:
            raise ValueError("too many stored elements for int32 positions")
        moved, data = data, np.arange(indices.shape[0], dtype=np.int32)      # the library moves 32-bit words
    s1_pos = np.zeros(num_col_partitions * (num_rows + 1), dtype=np.int32)
    s1_idx = np.zeros(indices.shape, dtype=np.int32)
    vals = np.zeros(data.shape, dtype=data.dtype)
    _lib.check(_lib.lib().fg_csr_to_dds(num_rows, num_cols, _lib.host_ptr(indptr), _lib.host_ptr(indices),
                                        _lib.host_ptr(data), num_col_partitions, _lib.host_ptr(s1_pos),
                                        _lib.host_ptr(s1_idx), _lib.host_ptr(vals)))
    assert len(s1_idx) == s1_pos[-1] and len(vals) == s1_pos[-1]
    if moved is not None:
        vals = moved[vals]
    return s1_pos, s1_idx, vals


def util_partition_adj_coo_2d(adj_scipy_coo, num_row_partitions, num_col_partitions):
    """2-D partitioning of a COO matrix.

    Returns the 1-based edge ids in traversal order (blocks in row-major block order,
    row-major / column-ascending inside a block) and the global row / col ids of the
    traversed edges, all int32 [nnz].  Unlike the reference (adj_partitioning.py:92) the
    caller's matrix is left untouched; duplicate (row, col) pairs raise ValueError.
    """
    assert num_row_partitions >= 1, "num_row_partitions should be larger than or equal to 1"
    assert num_col_partitions >= 1, "num_col_partitions should be larger than or equal to 1"
    num_rows, num_cols = adj_scipy_coo.shape
    row = np.ascontiguousarray(adj_scipy_coo.row, dtype=np.int32)
    col = np.ascontiguousarray(adj_scipy_coo.col, dtype=np.int32)
    nnz = row.shape[0]
    assert col.shape[0] == nnz, "length of adj_row_indices and that of adj_col_indices do not match"
    edge_id = np.zeros(nnz, dtype=np.int32)
    out_row = np.zeros(nnz, dtype=np.int32)
    out_col = np.zeros(nnz, dtype=np.int32)
    _lib.check(_lib.lib().fg_partition_coo_2d(num_rows, num_cols, nnz, _lib.host_ptr(row), _lib.host_ptr(col),
                                              num_row_partitions, num_col_partitions,
                                              _lib.host_ptr(edge_id), _lib.host_ptr(out_row),
                                              _lib.host_ptr(out_col)))
    return edge_id, out_row, out_col
