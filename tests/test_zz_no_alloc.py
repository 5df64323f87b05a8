"""cuvsAmdIvfPqSearchNoAlloc runs the search on a fixed workspace inside the library and makes no
device allocation.  Its results must equal cuvsIvfPqSearch's bit for bit, also on a second call
with a smaller input (the workspace keeps the first call's contents), and a search that does not
fit the workspace must be refused with a message."""
import numpy as np
import pytest
import torch

import gpu_helpers as G
import helpers as H
from cuvs_amd import ivf_pq
from cuvs_amd._lib import CuvsError
from cuvs_amd.resources import Resources

pytestmark = pytest.mark.gpu


def _index(n=60000, dim=64, n_lists=256, pq_dim=32, dtype=np.float32, seed=3):
    data = H.make_data(n, dim, dtype, seed, n_components=64)
    model = H.train(data, n_lists, pq_dim, 8, iters=4)
    return G.build_gpu_index(model, data, pq_dim, 8), dim


def _both(index, sp, queries, k, res):
    n = queries.shape[0]
    nb = torch.full((n, k), -7, dtype=torch.int64, device="cuda")
    d = torch.full((n, k), -7.0, dtype=torch.float32, device="cuda")
    ivf_pq.search_no_alloc(sp, index, queries, nb, d, resources=res)
    res.sync()
    want_d, want_nb = ivf_pq.search(sp, index, queries, k, resources=res)
    res.sync()
    return nb, d, want_nb, want_d


@pytest.mark.parametrize("lut,internal,n_probes,k", [
    (np.float16, np.float32, 20, 10),   # early-stop path: counters, survivor lists, alive flags
    (np.float32, np.float32, 8, 32),
    (np.uint8, np.float16, 16, 100),
])
def test_two_calls_in_a_row_equal_the_allocating_search(lut, internal, n_probes, k):
    index, dim = _index()
    res = Resources()
    sp = ivf_pq.SearchParams(n_probes=n_probes, lut_dtype=lut, internal_distance_dtype=internal)
    for n_queries, seed in [(500, 11), (37, 12)]:  # the second call is smaller
        queries = G.to_dev(H.make_data(n_queries, dim, np.float32, seed, n_components=64))
        nb, d, want_nb, want_d = _both(index, sp, queries, k, res)
        assert torch.equal(nb, want_nb), (n_queries, "neighbors")
        assert torch.equal(d, want_d), (n_queries, "distances")


def test_no_device_allocation_is_made():
    index, dim = _index()
    res = Resources()
    sp = ivf_pq.SearchParams(n_probes=20, lut_dtype=np.float16)
    queries = G.to_dev(H.make_data(200, dim, np.float32, 5, n_components=64))
    nb = torch.empty((200, 10), dtype=torch.int64, device="cuda")
    d = torch.empty((200, 10), dtype=torch.float32, device="cuda")
    ivf_pq.search_no_alloc(sp, index, queries, nb, d, resources=res)  # first call: symbol lookup
    res.sync()
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        ivf_pq.search_no_alloc(sp, index, queries, nb, d, resources=res)
    res.sync()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before


def test_a_search_beyond_the_workspace_is_refused():
    index, dim = _index()
    res = Resources()
    n_queries = 20000  # x 256 lists x 4 bytes of coarse scores alone is 20 MB; with k = 100 far beyond 32 MiB
    sp = ivf_pq.SearchParams(n_probes=64, lut_dtype=np.float16, max_internal_batch_size=n_queries)
    queries = G.to_dev(H.make_data(n_queries, dim, np.float32, 6, n_components=64))
    nb = torch.full((n_queries, 100), -7, dtype=torch.int64, device="cuda")
    d = torch.empty((n_queries, 100), dtype=torch.float32, device="cuda")
    with pytest.raises(CuvsError, match="bytes of workspace"):
        ivf_pq.search_no_alloc(sp, index, queries, nb, d, resources=res)
    assert int((nb != -7).sum()) == 0  # nothing ran
    # the same search in internal batches that fit is served
    sp_small = ivf_pq.SearchParams(n_probes=64, lut_dtype=np.float16, max_internal_batch_size=100)
    ivf_pq.search_no_alloc(sp_small, index, queries[:1000], nb[:1000], d[:1000], resources=res)
    res.sync()
    want_d, want_nb = ivf_pq.search(sp_small, index, queries[:1000], 100, resources=res)
    res.sync()
    assert torch.equal(nb[:1000], want_nb) and torch.equal(d[:1000], want_d)
