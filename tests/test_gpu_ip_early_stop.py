"""Early stop of inner-product and cosine searches: a (query, list) pair is dropped when a proven
lower bound of what its rows can still reach lies above the query's k-th best score so far (the
entries of these metrics have either sign, so the bound comes from the least entry each remaining
subspace can add).  The results must be the full scan's and the oracle's, bit for bit, whatever is
dropped; on clustered data something must be dropped.
"""
import numpy as np
import pytest
import torch

import datasets as testing
import gpu_helpers as G
import helpers as H
from cuvs_amd import ivf_pq
from cuvs_amd.resources import Resources

pytestmark = pytest.mark.gpu

R_32F, R_16F, R_8U = np.float32, np.float16, np.uint8
ORC_DT = {np.float32: 0, np.float16: 2, np.int8: 3, np.uint8: 8}


def _rows(n, dim, dtype, seed, normalize, decay=None):
    x = testing.gaussian_mixture(n, dim, 64, 0.12, seed=seed, normalize_rows=normalize,
                                 **({"dim_decay": decay} if decay else {})).numpy()
    if dtype == np.uint8:
        x = np.clip(np.round((x - x.min()) / (x.max() - x.min()) * 255), 0, 255).astype(np.uint8)
    return x.astype(dtype)


def _case(orc, dim, pq_dim, pq_bits, metric, dtype=np.float32, n=24000, n_lists=160, normalize=True, decay=None):
    print(f"case dim={dim} pq_dim={pq_dim} bits={pq_bits} metric={metric} dtype={np.dtype(dtype).name}", flush=True)
    allrows = _rows(n + 150, dim, dtype, 91, normalize, decay)
    x, q = allrows[:n], allrows[n:]
    model = H.train(x, n_lists, pq_dim, pq_bits, metric=metric, iters=4)
    index = G.build_gpu_index(model, x, pq_dim, pq_bits, metric)
    ix, _ = G.read_back(orc, index, model, dim, pq_dim, pq_bits, metric)
    return x, q, index, ix


def _both_ways(orc, index, ix, q, k, n_probes, lut, internal, expect_drops=True):
    res = Resources()
    res.enable_profiling(True)
    res.set_search_tuning(early_stop="on")
    sp = ivf_pq.SearchParams(n_probes=n_probes, lut_dtype=lut, internal_distance_dtype=internal)
    d, nb = ivf_pq.search(sp, index, G.to_dev(q), k, resources=res)
    res.sync()
    prof = ivf_pq.get_search_profile(res)
    assert prof["n_screened_pairs"] == q.shape[0] * (n_probes - 1), "the early stop did not run"
    print(f"  k={k} lut={np.dtype(lut).name} internal={np.dtype(internal).name}: {prof['n_surviving_pairs']} of "
          f"{prof['n_screened_pairs']} screened pairs kept", flush=True)
    if expect_drops:
        assert prof["n_surviving_pairs"] < prof["n_screened_pairs"]
    want_nb, want_d = orc.search(ix, q, k, n_probes, lut_dtype=ORC_DT[lut], internal_distance_dtype=ORC_DT[internal])
    H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 2e-3, exact=True)
    res.set_search_tuning(early_stop="off")
    d2, nb2 = ivf_pq.search(sp, index, G.to_dev(q), k, resources=res)
    res.sync()
    assert ivf_pq.get_search_profile(res)["n_screened_pairs"] == 0
    assert torch.equal(nb, nb2) and torch.equal(d, d2)
    return prof


TABLES = [(R_32F, R_32F), (R_16F, R_32F), (R_8U, R_32F), (R_16F, R_16F), (R_8U, R_16F)]


@pytest.mark.parametrize("metric", ["inner_product", "cosine"])
@pytest.mark.parametrize("dim,pq_dim", [(128, 64), (96, 48), (128, 32), (256, 128), (64, 64), (72, 36)])
def test_inner_product_early_stop_byte_codes(orc, metric, dim, pq_dim):
    x, q, index, ix = _case(orc, dim, pq_dim, 8, metric)
    for lut, internal in TABLES:
        for k in (1, 10, 100):
            _both_ways(orc, index, ix, q, k, 40, lut, internal, expect_drops=(internal == R_32F and k <= 10))


@pytest.mark.parametrize("metric", ["inner_product", "cosine"])
@pytest.mark.parametrize("dim,pq_dim", [(256, 128), (128, 128), (768, 384)])
def test_inner_product_early_stop_nibble_codes(orc, metric, dim, pq_dim):
    """4-bit codes (the 768 x 384 shape of the benchmark's inner-product configuration): 16 subspaces
    in a row's eight leading bytes."""
    x, q, index, ix = _case(orc, dim, pq_dim, 4, metric, decay=0.97 if dim == 768 else None)
    for lut, internal in [(R_16F, R_32F), (R_8U, R_32F), (R_16F, R_16F), (R_8U, R_16F)]:
        for k in (10, 64):
            _both_ways(orc, index, ix, q, k, 40, lut, internal, expect_drops=False)


@pytest.mark.parametrize("dtype", [np.uint8, np.float16])
def test_inner_product_early_stop_element_types(orc, dtype):
    x, q, index, ix = _case(orc, 128, 64, 8, "inner_product", dtype=dtype, normalize=False)
    for lut, internal in [(R_16F, R_32F), (R_8U, R_16F)]:
        _both_ways(orc, index, ix, q, 10, 40, lut, internal, expect_drops=False)


def test_inner_product_early_stop_with_a_filter(orc):
    """A filter can leave the leading list with fewer than k rows: no bound, nothing dropped."""
    x, q, index, ix = _case(orc, 128, 64, 8, "inner_product")
    n = x.shape[0]
    rng = np.random.default_rng(5)
    keep = rng.random(n) < 0.1
    bits = np.packbits(keep, bitorder="little")
    bits = np.concatenate([bits, np.zeros((-bits.size) % 4, dtype=np.uint8)]).view(np.uint32)
    res = Resources()
    res.set_search_tuning(early_stop="on")
    sp = ivf_pq.SearchParams(n_probes=40, lut_dtype=R_16F)
    d, nb = ivf_pq.search(sp, index, G.to_dev(q), 20, filter_bitset=G.to_dev(bits.view(np.int32)), filter_nbits=n,
                          resources=res)
    res.sync()
    want_nb, want_d = orc.search(ix, q, 20, 40, lut_dtype=ORC_DT[R_16F], filter_bitset=bits, filter_nbits=n)
    H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 2e-3, exact=True)
