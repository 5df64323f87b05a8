"""cuvsAmdIvfPqSearchNoAlloc runs the search on a fixed workspace inside the library and makes no
device allocation.  Its results must equal cuvsIvfPqSearch's bit for bit, also on a second call
with a smaller input (the workspace keeps the first call's contents); a search that does not fit
the workspace runs in internal batches that do, calls on two streams take turns on it, and the call
can be captured into a HIP graph."""
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


def test_a_search_beyond_the_workspace_runs_in_batches_that_fit():
    index, dim = _index()
    res = Resources()
    n_queries = 20000  # x 256 lists x 4 bytes of coarse scores alone is 20 MB; with k = 100 far beyond 32 MiB
    sp = ivf_pq.SearchParams(n_probes=64, lut_dtype=np.float16, max_internal_batch_size=n_queries)
    queries = G.to_dev(H.make_data(n_queries, dim, np.float32, 6, n_components=64))
    nb = torch.full((n_queries, 100), -7, dtype=torch.int64, device="cuda")
    d = torch.empty((n_queries, 100), dtype=torch.float32, device="cuda")
    ivf_pq.search_no_alloc(sp, index, queries, nb, d, resources=res)
    res.sync()
    want_d, want_nb = ivf_pq.search(sp, index, queries, 100, resources=res)
    res.sync()
    assert torch.equal(nb, want_nb) and torch.equal(d, want_d)


def test_calls_on_two_streams_take_turns():
    """Two handles on two streams share the one workspace: the second call waits for the first."""
    index, dim = _index()
    sp = ivf_pq.SearchParams(n_probes=20, lut_dtype=np.float16)
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    handles, outs, qs = [], [], []
    for i, st in enumerate(streams):
        with torch.cuda.stream(st):
            res = Resources()
            res.use_torch_current_stream()
            handles.append(res)
        qs.append(G.to_dev(H.make_data(300, dim, np.float32, 20 + i, n_components=64)))
        outs.append((torch.empty((300, 10), dtype=torch.int64, device="cuda"),
                     torch.empty((300, 10), dtype=torch.float32, device="cuda")))
    torch.cuda.synchronize()
    for rep in range(5):
        for i in range(2):
            ivf_pq.search_no_alloc(sp, index, qs[i], outs[i][0], outs[i][1], resources=handles[i])
    torch.cuda.synchronize()
    ref = Resources()
    for i in range(2):
        want_d, want_nb = ivf_pq.search(sp, index, qs[i], 10, resources=ref)
        ref.sync()
        assert torch.equal(outs[i][0], want_nb) and torch.equal(outs[i][1], want_d)


def test_captured_call_replays_like_eager():
    """The entry point under HIP graph capture (what it is for): replays on new query contents equal
    eager searches, with eager work and synchronisations between the replays."""
    index, dim = _index()
    n_queries = 200
    pool = G.to_dev(H.make_data(4 * n_queries, dim, np.float32, 31, n_components=64))
    sp = ivf_pq.SearchParams(n_probes=20, lut_dtype=np.float16)
    res = Resources()
    queries = pool[:n_queries].clone()
    nb = torch.empty((n_queries, 10), dtype=torch.int64, device="cuda")
    d = torch.empty((n_queries, 10), dtype=torch.float32, device="cuda")
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        res.use_torch_current_stream()
        for _ in range(2):
            ivf_pq.search_no_alloc(sp, index, queries, nb, d, resources=res)
        res.sync()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        res.use_torch_current_stream()
        ivf_pq.search_no_alloc(sp, index, queries, nb, d, resources=res)
    for rep in range(4):
        fresh = pool[rep * n_queries:(rep + 1) * n_queries].contiguous()
        queries.copy_(fresh)
        graph.replay()
        torch.cuda.synchronize()
        got_nb, got_d = nb.clone(), d.clone()
        res.use_torch_current_stream()
        want_d, want_nb = ivf_pq.search(sp, index, fresh, 10, resources=res)
        res.sync()
        torch.cuda.synchronize()
        assert torch.equal(got_nb, want_nb) and torch.equal(got_d, want_d), rep
