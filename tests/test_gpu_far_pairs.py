"""L2 searches drop (query, list) pairs whose lists lie provably past the query's bound without reading
a row: a row's score is at least (|rotated query - rotated centre| - |decoded residual|)^2, the
index keeps the largest decoded residual of every list, and the probe selection's own score gives
the first length.  Whatever is dropped, the results must be the oracle's bit for bit: with every
table and sum type, with a random rotation (padded dimensions included), per-cluster codebooks and
4-bit codes, and with model tensors that do not belong together (rotated centres that are not the
rotation of the centres, a rotation that is not orthonormal), where the bound has to notice.
On well separated clusters most pairs must go that way.

Inner-product and cosine searches drop pairs on the same two numbers (a row's score is at least the
probe selection's score minus |query| times the list's radius; cosine divides the score by the
length of the rotated query first); the tests run all three metrics.
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

ORC_DT = {np.float32: 0, np.float16: 2, np.uint8: 8}


def _rows(n, dim, dtype, seed, sigma=0.05):
    x = testing.gaussian_mixture(n, dim, 48, sigma, seed=seed).numpy()
    if dtype == np.uint8:
        x = np.clip(np.round((x - x.min()) / (x.max() - x.min()) * 255), 0, 255)
    return x.astype(dtype)


def _search_all_ways(orc, index, ix, q, k, n_probes, lut, internal, expect_far, some_far=False):
    want_nb, want_d = orc.search(ix, q, k, n_probes, lut_dtype=ORC_DT[lut], internal_distance_dtype=ORC_DT[internal])
    res = Resources()
    res.enable_profiling(True)
    sp = ivf_pq.SearchParams(n_probes=n_probes, lut_dtype=lut, internal_distance_dtype=internal)
    far = {}
    for mode in ("on", "auto", "auto", "off"):
        res.set_search_tuning(early_stop=mode)
        d, nb = ivf_pq.search(sp, index, G.to_dev(q), k, resources=res)
        res.sync()
        prof = ivf_pq.get_search_profile(res)
        far[mode] = prof["n_far_pairs"]
        H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 1e-5 if lut == np.float32 else 2e-3,
                          exact=True)
    assert far["off"] == 0
    if expect_far:
        assert far["on"] > 0.5 * q.shape[0] * (n_probes - 1), f"only {far['on']} pairs dropped on their lists' distance"
    if some_far:
        assert far["on"] > 0
    return far


@pytest.mark.parametrize("lut,internal", [(np.float32, np.float32), (np.float16, np.float32), (np.uint8, np.float32),
                                          (np.float16, np.float16), (np.uint8, np.float16)])
@pytest.mark.parametrize("dtype", [np.float32, np.uint8])
@pytest.mark.parametrize("metric", ["sqeuclidean", "inner_product", "cosine"])
def test_far_pairs_are_dropped_and_results_stay_exact(orc, lut, internal, dtype, metric):
    n, dim, n_lists, pq_dim = 40000, 64, 192, 32
    allrows = _rows(n + 300, dim, dtype, 7)
    x, q = allrows[:n], allrows[n:]
    model = H.train(x, n_lists, pq_dim, 8, metric=metric, iters=4)
    index = G.build_gpu_index(model, x, pq_dim, 8, metric)
    ix, _ = G.read_back(orc, index, model, dim, pq_dim, 8, metric)
    l2 = metric == "sqeuclidean"
    # (inner product with an 8-bit table or binary16 sums: the allowance for their rounding eats most of the bound)
    far = _search_all_ways(orc, index, ix, q, 10, 32, lut, internal, expect_far=l2,
                           some_far=not l2 and lut != np.uint8 and internal == np.float32)
    print(f"{metric} {np.dtype(dtype).name} {np.dtype(lut).name} {np.dtype(internal).name}: {far} of {q.shape[0] * 31}",
          flush=True)


@pytest.mark.parametrize("dim,pq_dim,pq_bits,kind,rotate", [
    (64, 32, 8, "subspace", True),     # random rotation
    (61, 32, 8, "subspace", False),    # padded rotated dimension: a rotation that is no square matrix
    (64, 32, 8, "cluster", False),     # per-cluster codebooks
    (64, 64, 4, "subspace", False),    # nibble codes
    (96, 48, 6, "subspace", True),     # 6-bit codes on their byte-wide copy
    (320, 160, 8, "subspace", False),  # a residual of more than 256 dimensions
])
def test_far_pairs_with_other_index_shapes(orc, dim, pq_dim, pq_bits, kind, rotate):
    n, n_lists = 30000, 128
    allrows = _rows(n + 200, dim, np.float32, 11)
    x, q = allrows[:n], allrows[n:]
    model = H.train(x, n_lists, pq_dim, pq_bits, codebook_kind=kind, iters=3, force_random_rotation=rotate)
    index = G.build_gpu_index(model, x, pq_dim, pq_bits, "sqeuclidean", kind)
    ix, _ = G.read_back(orc, index, model, dim, pq_dim, pq_bits, "sqeuclidean", kind)
    _search_all_ways(orc, index, ix, q, 10, 24, np.float16, np.float32, expect_far=True)
    _search_all_ways(orc, index, ix, q, 100, 24, np.float16, np.float32, expect_far=False)


@pytest.mark.parametrize("tamper", ["centers_rot_shifted", "centers_rot_unrelated", "rotation_scaled",
                                    "rotation_long_rows", "norm_column_wrong"])
@pytest.mark.parametrize("metric", ["sqeuclidean", "inner_product", "cosine"])
def test_model_tensors_that_do_not_belong_together(orc, tamper, metric):
    """`build(res, params, dim, pq_centers, centers, centers_rot, rotation_matrix)` takes the four
    tensors as they come.  The probe selection uses `centers`, the scan `centers_rot` and the rotated
    query: a bound that took one for the other would drop rows the scan keeps."""
    n, dim, n_lists, pq_dim = 30000, 64, 128, 32
    rng = np.random.default_rng(5)
    allrows = _rows(n + 200, dim, np.float32, 13)
    x, q = allrows[:n], allrows[n:]
    model = H.train(x, n_lists, pq_dim, 8, metric=metric, iters=3, force_random_rotation=True)
    model = {name: np.array(v, copy=True) for name, v in model.items()}
    if tamper == "centers_rot_shifted":
        model["centers_rot"] += 0.3 * rng.standard_normal(model["centers_rot"].shape).astype(np.float32)
    elif tamper == "centers_rot_unrelated":
        model["centers_rot"] = model["centers_rot"][rng.permutation(n_lists)].copy()
    elif tamper == "rotation_scaled":
        model["rotation_matrix"] *= np.float32(1.4)
    elif tamper == "rotation_long_rows":
        model["rotation_matrix"] *= np.float32(3.0)
    elif tamper == "norm_column_wrong":
        model["centers"][:, dim] *= np.float32(0.5)
    index = G.build_gpu_index(model, x, pq_dim, 8, metric)
    ix, _ = G.read_back(orc, index, model, dim, pq_dim, 8, metric)
    far = _search_all_ways(orc, index, ix, q, 10, 32, np.float16, np.float32, expect_far=False)
    print(f"{metric} {tamper}: pairs dropped on their lists' distance {far} of {q.shape[0] * 31} screened", flush=True)


def test_far_pairs_follow_an_edit_of_a_list(orc):
    """The radius of a list is made from its rows: rows added later may lie further out."""
    n, dim, n_lists, pq_dim = 20000, 64, 96, 32
    allrows = _rows(n + 200, dim, np.float32, 17)
    x, q = allrows[:n], allrows[n:]
    model = H.train(x, n_lists, pq_dim, 8, iters=3)
    index = G.build_gpu_index(model, x[: n // 2], pq_dim, 8)
    # the second half arrives with outliers that their lists' first rows do not announce
    late = x[n // 2:].copy()
    late[::7] += np.float32(0.8) * np.random.default_rng(3).standard_normal((late[::7].shape[0], dim)).astype(np.float32)
    ivf_pq.extend(index, G.to_dev(late), None)
    ix, _ = G.read_back(orc, index, model, dim, pq_dim, 8)
    _search_all_ways(orc, index, ix, np.concatenate([q, late[::7][:100]]), 10, 24, np.float16, np.float32,
                     expect_far=False)
