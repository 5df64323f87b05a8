"""A search in its steady state (workspace allocated, kernel attributes set by a first call) is a
sequence of kernel launches on the resource's stream: it can be captured into a HIP graph and
replayed on new query contents.  Replays are compared with eager searches, with eager work and
synchronisations in between, several times over."""
import numpy as np
import pytest
import torch

import datasets as testing

from cuvs_amd import ivf_pq
from cuvs_amd.resources import Resources

pytestmark = pytest.mark.gpu


# (the last case: three internal batches, which an eager call runs side by side on streams of the
# handle's own and a captured call one after the other on the capturing stream)
@pytest.mark.parametrize("n_queries,n_probes,batch", [(1, 20, 4096), (100, 20, 4096), (2000, 8, 4096), (2000, 8, 700)])
def test_captured_search_replays_like_eager(n_queries, n_probes, batch):
    n, dim = 100000, 64
    allrows = testing.gaussian_mixture(n + 4 * n_queries, dim, 100, 0.2, seed=5, device="cuda")
    data, pool = allrows[:n], allrows[n:]
    index = ivf_pq.build(ivf_pq.IndexParams(n_lists=256, pq_dim=32, kmeans_trainset_fraction=0.3), data)
    res = Resources()
    sp = ivf_pq.SearchParams(n_probes=n_probes, lut_dtype=np.float16, max_internal_batch_size=batch)
    queries = pool[:n_queries].clone()
    nb = torch.empty((n_queries, 10), dtype=torch.int64, device="cuda")
    d = torch.empty((n_queries, 10), dtype=torch.float32, device="cuda")
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        res.use_torch_current_stream()
        for _ in range(2):
            ivf_pq.search(sp, index, queries, 10, neighbors=nb, distances=d, resources=res)
        res.sync()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        res.use_torch_current_stream()
        ivf_pq.search(sp, index, queries, 10, neighbors=nb, distances=d, resources=res)
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
