"""SpMM over several source partitions: every pass either adds to `out` in place or writes a buffer of its
own that a last kernel adds up, all passes in one launch (plan option `pass_buffers`: 1 = always, 2 = never;
default: buffers unless they would take more than 8 GiB).  The
sums and their order are the same, so the two must agree bit for bit -- on graphs with empty rows, rows
whose elements all lie in one partition, partitions without any element, and rows split over wavefronts."""
import numpy as np
import pytest
import scipy.sparse as sp

from helpers import assert_sum_close, spmm_mass

pytestmark = pytest.mark.gpu


def _graph(rng, n_rows=400, n_cols=3000, long_len=2600, empty_partition=False):
    a = sp.random(n_rows, n_cols, density=0.01, format="csr", random_state=rng,
                  data_rvs=lambda k: rng.standard_normal(k)).astype("float32").tolil()
    a[[0, 1, 2, n_rows // 2, n_rows - 1], :] = 0                        # empty rows, a run of them at the start
    a[7, rng.choice(n_cols, size=long_len, replace=False)] = 1.5       # longer than the split threshold
    a[100:180, n_cols // 2:] = 0                                       # 80 rows with elements in the first partitions only
    if empty_partition:
        a[:, n_cols // 4: n_cols // 2] = 0                             # a column range nobody references
    a = a.tocsr().astype("float32"); a.eliminate_zeros(); a.sort_indices()
    return a


def _run(adj, x, P, T, mode, w=None):
    import torch
    from featgraph_amd import _lib
    from featgraph_amd.module import VanillaSpMMhip, GSpMMhip, placeholder
    _lib.plan_opts = _lib.FgPlanOpts(pass_buffers=mode)
    try:
        if w is None:
            m = VanillaSpMMhip(adj, P)
            m.build([placeholder(x.shape)], {'num_feat_partitions': T}, {'num_src_partitions': None})
            text = m.lower_to_ir([placeholder(x.shape)], {'num_feat_partitions': T}, {'num_src_partitions': None})
            m.out_tvm.fill_(float("nan"))
            return m.run([torch.from_numpy(x).cuda()]).cpu().numpy().copy(), text
        m = GSpMMhip(adj, P)
        m.build([placeholder(x.shape), placeholder(w.shape)], {}, {'num_src_partitions': None})
        m.out_tvm.fill_(float("nan"))
        return m.run([torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()]).cpu().numpy().copy(), ""
    finally:
        _lib.plan_opts = None


@pytest.mark.parametrize("feat_len,P,T", [(128, 2, 2), (128, 5, 1), (64, 8, 0), (512, 4, 8), (96, 3, 3), (32, 16, 1)])
@pytest.mark.parametrize("empty_partition", [False, True])
def test_buffers_equal_in_place(oracle, feat_len, P, T, empty_partition):
    rng = np.random.default_rng(feat_len + P)
    adj = _graph(rng, empty_partition=empty_partition)
    x = rng.standard_normal((adj.shape[1], feat_len)).astype("float32")
    in_place, text = _run(adj, x, P, T, 2)
    assert "add to out in place" in text
    buffered, text = _run(adj, x, P, T, 1)
    assert "buffer of its own" in text
    assert np.isfinite(buffered).all()
    assert np.array_equal(in_place, buffered)
    assert (buffered[[0, 1, 2, adj.shape[0] // 2, adj.shape[0] - 1]] == 0).all()
    assert_sum_close(buffered, oracle.spmm_f64(adj, x), spmm_mass(adj, x), "F=%d P=%d T=%d" % (feat_len, P, T))


def test_per_head_weights_and_odd_lengths():
    """Per-head weights take the buffers too; scalar-lane shapes (feature length not a multiple of 4) never do."""
    rng = np.random.default_rng(3)
    adj = _graph(rng)
    H, D = 4, 32
    x = rng.standard_normal((adj.shape[1], H, D)).astype("float32")
    w = rng.random((adj.nnz, H)).astype("float32")
    a, _ = _run(adj, x, 3, 0, 2, w)
    b, _ = _run(adj, x, 3, 0, 1, w)
    assert np.array_equal(a, b)
    x7 = rng.standard_normal((adj.shape[1], 7)).astype("float32")
    a, _ = _run(adj, x7, 3, 1, 2)
    b, text = _run(adj, x7, 3, 1, 1)
    assert np.array_equal(a, b)
    ref = adj.astype(np.float64).dot(x7.astype(np.float64))
    np.testing.assert_allclose(b, ref, rtol=1e-4, atol=1e-4)
