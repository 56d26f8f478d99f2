"""The reference benchmarks' dataset path: scipy .npz adjacency files in the format written by
benchmark/download_reddit_dataset.py:11-17 (save_npz of a float32 csr_matrix / coo_matrix), loaded
as at benchmark/bench_vanilla_spmm.py:78-79 and bench_vanilla_sddmm.py:84-85, and run through the
sweep functions.  Every sweep point's output is compared with the CPU oracle."""
import argparse

import numpy as np
import pytest
import scipy.sparse as sp

from helpers import RTOL, ATOL, assert_sum_close, spmm_mass, sddmm_mass


def _graph(seed=31, n_rows=700, n_cols=900, density=0.02):
    rng = np.random.default_rng(seed)
    a = sp.random(n_rows, n_cols, density=density, format="csr", random_state=rng,
                  data_rvs=lambda k: rng.random(k)).astype("float32")
    a.sort_indices()
    return a


@pytest.mark.gpu
def test_spmm_sweep_from_csr_npz(tmp_path, oracle):
    import torch
    from featgraph_amd.benchmark.common import load_adjacency
    from featgraph_amd.benchmark.bench_vanilla_spmm import bench_vanilla_spmm
    adj = _graph()
    path = str(tmp_path / "toy_csr_float32.npz")
    sp.save_npz(path, adj)
    loaded = load_adjacency(argparse.Namespace(dataset=path, workload=None), 'csr')
    assert loaded.format == 'csr' and loaded.dtype == np.float32
    assert np.array_equal(loaded.indptr, adj.indptr) and np.array_equal(loaded.indices, adj.indices)
    assert np.array_equal(loaded.data, adj.data)
    feat_len = 64
    x = np.random.default_rng(32).random((adj.shape[1], feat_len)).astype("float32")
    results = []
    bench_vanilla_spmm(loaded, feat_len, max_col_partitions=4, num_runs=2, src_feat=torch.from_numpy(x).cuda(),
                       collect=results)
    assert len(results) == 1 + 3 * 3            # auto + {1,2,4} partitions x {1,2,4} feature tiles
    ref = oracle.spmm_f64(adj, x)
    mass = spmm_mass(adj, x)
    ref32 = oracle.spmm_csr_x86(adj.indptr, adj.indices, adj.data, x)
    for knobs, seconds, out in results:
        assert 0 < seconds < 1.0, knobs
        assert_sum_close(out, ref, mass, str(knobs))
        np.testing.assert_allclose(out, ref32, rtol=RTOL, atol=ATOL, err_msg=str(knobs))
    # a float64 file (scipy's default dtype) is accepted and computed in fp32
    path64 = str(tmp_path / "toy_csr_float64.npz")
    sp.save_npz(path64, adj.astype(np.float64))
    again = load_adjacency(argparse.Namespace(dataset=path64, workload=None), 'csr')
    assert again.dtype == np.float32 and np.array_equal(again.data, adj.data)


@pytest.mark.gpu
def test_sddmm_sweep_from_coo_npz(tmp_path, oracle):
    import torch
    from featgraph_amd.benchmark.common import load_adjacency
    from featgraph_amd.benchmark.bench_vanilla_sddmm import bench_vanilla_sddmm
    coo = _graph(seed=33).tocoo()
    path = str(tmp_path / "toy_coo_float32.npz")
    sp.save_npz(path, coo)
    loaded = load_adjacency(argparse.Namespace(dataset=path, workload=None), 'coo')
    assert loaded.format == 'coo'
    assert np.array_equal(loaded.row, coo.row) and np.array_equal(loaded.col, coo.col)
    feat_len = 32
    rng = np.random.default_rng(34)
    src = rng.random((coo.shape[1], feat_len)).astype("float32")
    dst = rng.random((coo.shape[0], feat_len)).astype("float32")
    results = []
    bench_vanilla_sddmm(loaded, feat_len, max_partitions=2, num_runs=2, src_feat=torch.from_numpy(src).cuda(),
                        dst_feat=torch.from_numpy(dst).cuda(), collect=results)
    assert len(results) >= 5
    ref = oracle.sddmm_f64(coo.row, coo.col, src, dst)
    mass = sddmm_mass(coo.row, coo.col, src, dst)
    ref32 = oracle.sddmm_x86(coo.row, coo.col, src, dst)
    seen = set()
    for knobs, seconds, out in results:
        assert 0 < seconds < 1.0, knobs
        assert_sum_close(out, ref, mass, str(knobs))
        np.testing.assert_allclose(out, ref32, rtol=RTOL, atol=ATOL, err_msg=str(knobs))
        seen.add(knobs.get("order"))
    assert {"auto", "coo", "csr", "tiled"} <= seen


def test_wrong_format_is_refused(tmp_path):
    """bench_vanilla_spmm.py:79 / bench_vanilla_sddmm.py:85 assert the stored format."""
    from featgraph_amd.benchmark.common import load_adjacency
    adj = _graph()
    p_csr, p_coo = str(tmp_path / "a_csr.npz"), str(tmp_path / "a_coo.npz")
    sp.save_npz(p_csr, adj)
    sp.save_npz(p_coo, adj.tocoo())
    with pytest.raises(AssertionError):
        load_adjacency(argparse.Namespace(dataset=p_csr, workload=None), 'coo')
    with pytest.raises(AssertionError):
        load_adjacency(argparse.Namespace(dataset=p_coo, workload=None), 'csr')
