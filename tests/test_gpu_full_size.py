"""The benchmark configurations at their real shapes, through the C ABI.

A CPU run of the whole batch would take minutes, so these tests rely on what does not depend on
the size: results are well formed (ids in range, no repeats, distances in order), they do not
depend on how the batch is split, a larger probe count can only improve every rank, the first k
of a longer result list are the shorter list, exact re-ranking restores exact neighbours, and
recall against a brute-force search stays where the small cases put it.  Where the host copy of
the index is cheap (8-bit codes), the CPU oracle also answers a sample of the queries on the same
index and must agree bit for bit.
"""
import numpy as np
import pytest
import torch

import gpu_helpers as G
import helpers as H
import datasets as testing
from cuvs_amd import ivf_pq, refine

pytestmark = pytest.mark.gpu

R_32F, R_16F, R_8U = 0, 2, 8
ORC_DT = {R_32F: 0, R_16F: 2, R_8U: 8}


def _model_of(index):
    return {"centers": index.centers_padded.cpu().numpy(),
            "centers_rot": index.centers_rot.cpu().numpy(),
            "rotation_matrix": index.rotation_matrix.cpu().numpy(),
            "pq_centers": index.pq_centers.cpu().numpy()}


def _search(index, queries, k, n_probes, lut=R_16F, internal=R_32F, batch=None):
    sp = ivf_pq.SearchParams(n_probes=n_probes, lut_dtype=lut, internal_distance_dtype=internal,
                             max_internal_batch_size=batch or queries.shape[0])
    d, nb = ivf_pq.search(sp, index, queries, k)
    torch.cuda.synchronize()
    return d, nb


def _well_formed(d, nb, n_rows, descending=False):
    ids = nb.cpu().numpy()
    dist = d.cpu().numpy()
    assert ((ids >= 0) & (ids < n_rows)).all()
    srt = np.sort(ids, axis=1)
    assert (srt[:, 1:] != srt[:, :-1]).all(), "a row was returned twice"
    step = np.diff(dist, axis=1)
    assert (step <= 0).all() if descending else (step >= 0).all()
    assert np.isfinite(dist).all()


def _rankwise_no_worse(d_more, d_fewer, descending=False):
    """Probing more lists adds candidates and removes none: every rank's distance can only improve."""
    a, b = d_more.cpu().numpy(), d_fewer.cpu().numpy()
    assert (a >= b).all() if descending else (a <= b).all()


def _prefix_of(d_short, nb_short, d_long, nb_long):
    k = d_short.shape[1]
    ds, dl = d_short.cpu().numpy(), d_long.cpu().numpy()[:, :k]
    assert np.array_equal(ds, dl)
    ns, nl = nb_short.cpu().numpy(), nb_long.cpu().numpy()[:, :k]
    # ids may differ only where a distance repeats (ties are ordered by position, and the k-th
    # place of the shorter list can take either of two equal candidates)
    differ = ns != nl
    if differ.any():
        full = d_long.cpu().numpy()
        for q, r in zip(*np.nonzero(differ)):
            assert (full[q] == ds[q, r]).sum() > 1


# ------------------------------------------------------------------------------------------------
# 10M x 128 uint8, 16384 lists, pq_dim 64, 8 bits: the configuration the benchmark is quoted on
# ------------------------------------------------------------------------------------------------

@pytest.fixture(scope="module")
def sift10m():
    n, nq = 10_000_000, 10_000
    allrows = testing.sift_like_u8(n + nq, 128, 4096, seed=1234, device="cuda")
    data, queries = allrows[:n], allrows[n:].contiguous()
    params = ivf_pq.IndexParams(n_lists=16384, pq_bits=8, pq_dim=64, kmeans_trainset_fraction=524288 / n)
    index = ivf_pq.build(params, data)
    truth = testing.exact_knn(data, queries, 10).cpu().numpy()
    yield data, queries, index, truth
    del index, data, allrows
    torch.cuda.empty_cache()


def test_10m_u8_results_and_recall(sift10m):
    data, queries, index, truth = sift10m
    n = data.shape[0]
    assert len(index) == n
    found = {}
    for lut in (R_16F, R_8U):
        d, nb = _search(index, queries, 10, 64, lut=lut)
        _well_formed(d, nb, n)
        found[lut] = testing.recall(nb.cpu().numpy(), truth)
    print(f"recall@10: fp16 table {found[R_16F]:.4f}, fp8 table {found[R_8U]:.4f}", flush=True)
    assert found[R_16F] >= 0.80 and found[R_8U] >= found[R_16F] - 0.03


def test_10m_u8_batch_split_probe_count_and_k(sift10m):
    data, queries, index, _ = sift10m
    d64, nb64 = _search(index, queries, 10, 64)
    d_split, nb_split = _search(index, queries, 10, 64, batch=3000)
    assert torch.equal(nb64, nb_split) and torch.equal(d64, d_split)
    d32, _ = _search(index, queries, 10, 32)
    d128, nb128 = _search(index, queries, 10, 128)
    _rankwise_no_worse(d64, d32)
    _rankwise_no_worse(d128, d64)
    d100, nb100 = _search(index, queries, 100, 64)
    _well_formed(d100, nb100, data.shape[0])
    _prefix_of(d64, nb64, d100, nb100)


def test_10m_u8_oracle_on_a_sample(orc, sift10m):
    data, queries, index, _ = sift10m
    ix = G.read_back_bulk(orc, index, _model_of(index), 128, 64, 8)
    q = queries[:256].cpu().numpy()
    for lut, k, n_probes in ((R_16F, 10, 64), (R_8U, 10, 32), (R_16F, 100, 128)):
        d, nb = _search(index, queries[:256].contiguous(), k, n_probes, lut=lut)
        want_nb, want_d = orc.search(ix, q, k, n_probes, lut_dtype=ORC_DT[lut])
        H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 2e-3, exact=True)


def test_10m_u8_refine_restores_exact_neighbours(sift10m):
    data, queries, index, truth = sift10m
    _, cand = _search(index, queries, 40, 64)
    d, nb = refine(data, queries, cand, 10)
    torch.cuda.synchronize()
    _well_formed(d, nb, data.shape[0])
    assert testing.recall(nb.cpu().numpy(), truth) >= 0.99
    # the refined distances are the exact squared distances to the rows returned
    rows = data[nb.reshape(-1)].reshape(nb.shape[0], nb.shape[1], -1).float()
    exact = ((rows - queries[:, None, :].float()) ** 2).sum(-1)
    assert torch.equal(exact, d)


# ------------------------------------------------------------------------------------------------
# 1M x 96 fp32 unit vectors, 1024 lists, pq_dim 48
# ------------------------------------------------------------------------------------------------

def test_1m_f32_normalised(orc):
    n, nq, dim = 1_000_000, 10_000, 96
    allrows = testing.gaussian_mixture(n + nq, dim, 1000, 0.2, seed=11, device="cuda",
                                       normalize_centers=True, normalize_rows=True)
    data, queries = allrows[:n], allrows[n:].contiguous()
    index = ivf_pq.build(ivf_pq.IndexParams(n_lists=1024, pq_bits=8, pq_dim=48,
                                            kmeans_trainset_fraction=0.2), data)
    truth = testing.exact_knn(data, queries[:2000], 10).cpu().numpy()
    ix = G.read_back_bulk(orc, index, _model_of(index), dim, 48, 8)
    prev, recalls = None, []
    for n_probes in (16, 32, 64):
        d, nb = _search(index, queries, 10, n_probes)
        _well_formed(d, nb, n)
        if prev is not None:
            _rankwise_no_worse(d, prev)
        prev = d
        recalls.append(testing.recall(nb[:2000].cpu().numpy(), truth))
        want_nb, want_d = orc.search(ix, queries[:200].cpu().numpy(), 10, n_probes, lut_dtype=ORC_DT[R_16F])
        H.compare_results(nb[:200].cpu().numpy(), d[:200].cpu().numpy(), want_nb, want_d, 2e-3, exact=True)
    print("recall@10 at 16 / 32 / 64 probes:", recalls, flush=True)
    # this mixture is nearly isotropic after normalisation: product quantisation of 96 dimensions
    # into 48 bytes ranks its near neighbours only roughly (the oracle finds the same)
    assert recalls[0] <= recalls[1] + 0.01 <= recalls[2] + 0.02 and recalls[2] >= 0.6


# ------------------------------------------------------------------------------------------------
# 10M x 768 fp32 unit vectors, inner product, 16384 lists, pq_dim 384, 4 bits, fp8 table, fp16 sums
# ------------------------------------------------------------------------------------------------

def test_10m_f32_inner_product_four_bit():
    n, nq, dim = 10_000_000, 10_000, 768
    allrows = testing.gaussian_mixture(n + nq, dim, 8192, 0.3, seed=13, device="cuda", dim_decay=0.9,
                                       normalize_rows=True)
    data, queries = allrows[:n], allrows[n:].contiguous()
    params = ivf_pq.IndexParams(n_lists=16384, metric="inner_product", pq_bits=4, pq_dim=384,
                                kmeans_trainset_fraction=524288 / n)
    index = ivf_pq.build(params, data)
    assert len(index) == n
    d64, nb64 = _search(index, queries, 10, 64, lut=R_8U, internal=R_16F)
    _well_formed(d64, nb64, n, descending=True)
    d_split, nb_split = _search(index, queries, 10, 64, lut=R_8U, internal=R_16F, batch=4096)
    assert torch.equal(nb64, nb_split) and torch.equal(d64, d_split)
    d16, _ = _search(index, queries, 10, 16, lut=R_8U, internal=R_16F)
    _rankwise_no_worse(d64, d16, descending=True)
    d40, nb40 = _search(index, queries, 40, 64, lut=R_8U, internal=R_16F)
    _prefix_of(d64, nb64, d40, nb40)
    # 4-bit codes rank the rows of a list only roughly; re-ranking the 40 candidates by exact inner
    # products must find most of the true neighbours the probed lists hold
    truth = testing.exact_knn(data, queries[:1000], 10, metric="inner_product").cpu().numpy()
    d_ref, nb_ref = refine(data, queries[:1000].contiguous(), nb40[:1000].contiguous(), 10,
                           metric="inner_product")
    torch.cuda.synchronize()
    coarse = testing.recall(nb64[:1000].cpu().numpy(), truth)
    refined = testing.recall(nb_ref.cpu().numpy(), truth)
    print(f"recall@10: codes only {coarse:.4f}, 40 candidates re-ranked {refined:.4f}", flush=True)
    assert refined > coarse
    del index, data, allrows
    torch.cuda.empty_cache()


# ------------------------------------------------------------------------------------------------
# fp16 rows, per-cluster codebooks, 200 probes, lists of 2000 rows: the 100M-row configuration at a
# fifth of its rows and lists (the build of the whole set takes a minute; the search path per
# (query, list) pair is the same)
# ------------------------------------------------------------------------------------------------

def test_20m_f16_per_cluster(orc):
    n, nq, dim, n_lists = 20_000_000, 10_000, 96, 10_000
    allrows = testing.gaussian_mixture(n + nq, dim, n_lists, 0.25, seed=17, device="cuda", dtype=torch.float16)
    data, queries = allrows[:n], allrows[n:].contiguous()
    params = ivf_pq.IndexParams(n_lists=n_lists, pq_bits=8, pq_dim=48, codebook_kind="cluster",
                                kmeans_trainset_fraction=800_000 / n)
    index = ivf_pq.build(params, data)
    assert len(index) == n
    truth = testing.exact_knn(data, queries[:1000], 10).cpu().numpy()
    results = {}
    for batch in (1, 100, 10_000):
        q = queries[:batch].contiguous()
        d, nb = _search(index, q, 10, 200)
        _well_formed(d, nb, n)
        results[batch] = (d, nb)
    # a query's answer does not depend on the batch it arrives in
    for small in (1, 100):
        assert torch.equal(results[small][0], results[10_000][0][:small])
        assert torch.equal(results[small][1], results[10_000][1][:small])
    rec = testing.recall(results[10_000][1][:1000].cpu().numpy(), truth)
    print(f"recall@10 at 200 probes: {rec:.4f}", flush=True)
    assert rec >= 0.75
    d100, _ = _search(index, queries[:2000].contiguous(), 10, 100)
    _rankwise_no_worse(results[10_000][0][:2000], d100)
    ix = G.read_back_bulk(orc, index, _model_of(index), dim, 48, 8, codebook_kind="cluster")
    want_nb, want_d = orc.search(ix, queries[:64].cpu().numpy(), 10, 200, lut_dtype=ORC_DT[R_16F])
    H.compare_results(results[10_000][1][:64].cpu().numpy(), results[10_000][0][:64].cpu().numpy(),
                      want_nb, want_d, 2e-3, exact=True)
    del index, data, allrows
    torch.cuda.empty_cache()


# ------------------------------------------------------------------------------------------------
# The 100M-row configuration itself: 100M x 96 fp16, 50,000 lists, per-cluster codebooks, pq_dim 48,
# 200 probes (4.8 GB of codes + 0.8 GB of ids on the GPU).  Properties only: a host copy of this index
# for the oracle would take longer than everything else here (the case above has the oracle sample).
# ------------------------------------------------------------------------------------------------

def test_100m_f16_per_cluster():
    n, nq, dim, n_lists = 100_000_000, 10_000, 96, 50_000
    allrows = testing.gaussian_mixture(n + nq, dim, n_lists, 0.25, seed=1234, device="cuda", dtype=torch.float16)
    data, queries = allrows[:n], allrows[n:].contiguous()
    params = ivf_pq.IndexParams(n_lists=n_lists, pq_bits=8, pq_dim=48, codebook_kind="cluster",
                                kmeans_trainset_fraction=1_600_000 / n)
    index = ivf_pq.build(params, data)
    assert len(index) == n
    sizes = index.list_sizes.cpu().numpy()
    assert int(sizes.sum()) == n and sizes.max() < 20 * sizes.mean()
    results = {}
    for batch in (1, 100, 10_000):
        q = queries[:batch].contiguous()
        d, nb = _search(index, q, 10, 200)
        _well_formed(d, nb, n)
        results[batch] = (d, nb)
    # a query's answer depends neither on the batch it arrives in nor on how the batch is split
    for small in (1, 100):
        assert torch.equal(results[small][0], results[10_000][0][:small])
        assert torch.equal(results[small][1], results[10_000][1][:small])
    d_split, nb_split = _search(index, queries, 10, 200, batch=3000)
    assert torch.equal(nb_split, results[10_000][1]) and torch.equal(d_split, results[10_000][0])
    # more probes can only improve every rank; the first k of a longer list are the shorter list
    d100, _ = _search(index, queries[:2000].contiguous(), 10, 100)
    _rankwise_no_worse(results[10_000][0][:2000], d100)
    d40, nb40 = _search(index, queries[:2000].contiguous(), 40, 200)
    _prefix_of(results[10_000][0][:2000], results[10_000][1][:2000], d40, nb40)
    # recall against exact search, and exact re-ranking of 40 candidates
    truth = testing.exact_knn(data, queries[:500], 10).cpu().numpy()
    rec = testing.recall(results[10_000][1][:500].cpu().numpy(), truth)
    d_ref, nb_ref = refine(data, queries[:500].contiguous(), nb40[:500].contiguous(), 10)
    torch.cuda.synchronize()
    refined = testing.recall(nb_ref.cpu().numpy(), truth)
    print(f"recall@10 at 200 probes: {rec:.4f}; 40 candidates re-ranked: {refined:.4f}", flush=True)
    assert rec >= 0.75 and refined >= rec
    del index, data, allrows
    torch.cuda.empty_cache()
