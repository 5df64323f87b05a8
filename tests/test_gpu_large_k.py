"""k and candidate counts beyond what the selection kernels hold in LDS: the reference's search has
no limit on k other than the index size (its non-fused path selects over every probed row,
cpp/src/neighbors/ivf_pq/ivf_pq_search.cuh:637-655), nor has its refinement on the number of
candidates.  Here the selection's output then lives in a global scratch buffer.  The same holds for
the number of probes (the reference takes any n_probes up to n_lists, ivf_pq_search.cuh:932): the
probe selection keeps up to 8192 probes in LDS and writes to the workspace beyond."""
import numpy as np
import pytest
import torch

import gpu_helpers as G
import helpers as H
from cuvs_amd import ivf_pq, refine

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("k", [8192, 8193, 20000])
def test_search_with_k_beyond_the_merge_kernels_lds(orc, k):
    n, dim, n_lists, pq_dim = 30000, 16, 6, 8
    data = H.make_data(n, dim, np.float32, 3)
    model = H.train(data, n_lists, pq_dim, 8, iters=3)
    queries = H.make_data(5, dim, np.float32, 103)
    index = G.build_gpu_index(model, data, pq_dim, 8)
    ix, _ = G.read_back(orc, index, model, dim, pq_dim, 8)
    for n_probes in (6, 3):
        sp = ivf_pq.SearchParams(n_probes=n_probes)
        d, nb = ivf_pq.search(sp, index, G.to_dev(queries), k)
        torch.cuda.synchronize()
        want_nb, want_d = orc.search(ix, queries, k, n_probes)
        H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 1e-5, exact=True)


def test_refine_of_more_candidates_than_lds_holds(orc):
    rng = np.random.default_rng(7)
    n, dim, nq, n_cand, k = 40000, 24, 6, 30000, 9000
    data = rng.standard_normal((n, dim)).astype(np.float32)
    queries = rng.standard_normal((nq, dim)).astype(np.float32)
    cand = np.stack([rng.permutation(n)[:n_cand] for _ in range(nq)]).astype(np.int64)
    cand[0, :50] = -1  # unfilled slots are skipped
    d, nb = refine(G.to_dev(data), G.to_dev(queries), G.to_dev(cand), k)
    torch.cuda.synchronize()
    want_nb, want_d = orc.refine(data, queries, cand, k)
    got_nb, got_d = nb.cpu().numpy(), d.cpu().numpy()
    assert np.allclose(got_d, want_d, rtol=1e-5, atol=1e-6)
    # ids may swap only where distances tie within the tolerance
    differ = got_nb != want_nb
    assert differ.mean() < 1e-2
    for q, r in zip(*np.nonzero(differ)):
        assert abs(want_d[q, r] - got_d[q, r]) <= 1e-5 * max(1.0, abs(want_d[q, r]))


@pytest.mark.parametrize("n_probes", [8192, 8193, 9000])
def test_search_with_more_probes_than_the_selection_kernels_lds(orc, n_probes):
    rng = np.random.default_rng(17)
    n, dim, n_lists, pq_dim = 60000, 32, 9000, 16
    data = rng.standard_normal((n, dim)).astype(np.float32)
    queries = rng.standard_normal((7, dim)).astype(np.float32)
    model = H.train(data, n_lists, pq_dim, 8, iters=2)
    index = G.build_gpu_index(model, data, pq_dim, 8)
    ix, _ = G.read_back(orc, index, model, dim, pq_dim, 8)
    for k in (10, 300):
        sp = ivf_pq.SearchParams(n_probes=n_probes, lut_dtype=np.float16)
        d, nb = ivf_pq.search(sp, index, G.to_dev(queries), k)
        torch.cuda.synchronize()
        want_nb, want_d = orc.search(ix, queries, k, n_probes, lut_dtype=2)
        H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 2e-3, exact=True)
