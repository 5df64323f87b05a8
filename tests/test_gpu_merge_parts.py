"""knn_merge_parts on the GPU against a numpy restatement: per row the k smallest of n_parts * k
candidates, ascending, ids shifted by the part's translation
(cpp/src/neighbors/detail/knn_merge_parts.cuh:23-110).  The reference leaves the order of equal
keys to its block select; here it is fixed (lower part, then lower column) and the check uses it."""
import numpy as np
import pytest
import torch

import gpu_helpers as G
import datasets as testing
from cuvs_amd import ivf_pq, knn_merge_parts

pytestmark = pytest.mark.gpu


def _expect(keys, ids, translations, n_parts):
    n, k = keys.shape[0] // n_parts, keys.shape[1]
    kk = keys.reshape(n_parts, n, k).transpose(1, 0, 2).reshape(n, n_parts * k)
    ii = (ids.reshape(n_parts, n, k) + translations[:, None, None]).transpose(1, 0, 2).reshape(n, n_parts * k)
    order = np.argsort(kk, axis=1, kind="stable")[:, :k]
    return np.take_along_axis(kk, order, 1), np.take_along_axis(ii, order, 1)


@pytest.mark.parametrize("n_parts,n,k", [(1, 7, 5), (2, 100, 10), (8, 333, 32), (3, 50, 100), (8, 20, 1024),
                                         (5, 1, 1)])
def test_merge_parts_matches_numpy(n_parts, n, k):
    rng = np.random.default_rng(n_parts * 1000 + k)
    keys = np.sort(rng.random((n_parts * n, k), dtype=np.float32), axis=1)
    # ties across parts and within a part
    keys[rng.random(keys.shape) < 0.2] = 0.5
    keys = np.sort(keys, axis=1)
    ids = rng.integers(0, 1 << 40, size=keys.shape, dtype=np.int64)
    tr = (np.arange(n_parts, dtype=np.int64) * (1 << 41))
    ok, oi = knn_merge_parts(G.to_dev(keys), G.to_dev(ids), G.to_dev(tr))
    want_k, want_i = _expect(keys, ids, tr, n_parts)
    assert np.array_equal(ok.cpu().numpy(), want_k)
    assert np.array_equal(oi.cpu().numpy(), want_i)


def test_merge_parts_special_values_and_validation():
    keys = np.array([[np.inf, -1.0, np.nan], [0.0, -0.0, 3.0]], dtype=np.float32)  # 2 parts, 1 row, k = 3
    ids = np.array([[1, 2, 3], [4, 5, 6]], dtype=np.int64)
    tr = np.array([0, 10], dtype=np.int64)
    ok, oi = knn_merge_parts(G.to_dev(keys), G.to_dev(ids), G.to_dev(tr))
    assert oi.cpu().numpy().tolist() == [[2, 14, 15]]
    assert ok.cpu().numpy().tolist() == [[-1.0, 0.0, -0.0]]
    with pytest.raises(Exception, match="8192"):
        big = torch.zeros((9 * 2, 1024), dtype=torch.float32, device="cuda")
        knn_merge_parts(big, torch.zeros((18, 1024), dtype=torch.int64, device="cuda"),
                        torch.zeros(9, dtype=torch.int64, device="cuda"))


def test_row_sharded_search_equals_one_index(orc):
    """Two indexes over the halves of a dataset, same model: searching both and merging with the
    second half's id offset gives what one index over all rows gives (with every list probed, so
    the shards' own list contents do not matter)."""
    import helpers as H
    x = testing.gaussian_mixture(4000, 32, 20, 0.3, seed=3).numpy()
    q = x[:64] + 0.01
    model = H.train(x, 16, 16, 8, iters=5)
    whole = G.build_gpu_index(model, x, 16, 8)
    parts = [G.build_gpu_index(model, x[:2000], 16, 8), G.build_gpu_index(model, x[2000:], 16, 8)]
    sp = ivf_pq.SearchParams(n_probes=16)
    d, nb = ivf_pq.search(sp, whole, G.to_dev(q), 10)
    ds, ns = zip(*[ivf_pq.search(sp, p, G.to_dev(q), 10) for p in parts])
    ok, oi = knn_merge_parts(torch.cat(ds), torch.cat(ns), G.to_dev(np.array([0, 2000], dtype=np.int64)))
    assert torch.equal(ok, d)
    same = (oi == nb) | (ok == torch.roll(ok, 1, 1)) | (ok == torch.roll(ok, -1, 1))
    assert bool(same.all())
