"""The oracle's refinement against textbook brute force in float64 / exact integers."""
import numpy as np
import pytest


def _brute(dataset, queries, candidates, k, metric):
    nq = queries.shape[0]
    ids = np.full((nq, k), -1, dtype=np.int64)
    dist = np.full((nq, k), np.finfo(np.float32).max, dtype=np.float64)
    integer = dataset.dtype.kind in "iu"
    for q in range(nq):
        rows = []
        for slot, c in enumerate(candidates[q]):
            if c < 0 or c >= dataset.shape[0]:
                continue
            if integer:
                a, b = queries[q].astype(np.int64), dataset[c].astype(np.int64)
            else:
                a, b = queries[q].astype(np.float64), dataset[c].astype(np.float64)
            d = float(np.dot(a, b)) if metric == 6 else float(np.dot(a - b, a - b))
            rows.append((-d if metric == 6 else d, slot, c, d))
        rows.sort()
        for r, (_, _, c, d) in enumerate(rows[:k]):
            ids[q, r] = c
            dist[q, r] = np.sqrt(d) if metric == 1 else d
    return ids, dist


@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.int8, np.uint8])
@pytest.mark.parametrize("metric", [0, 1, 6])
def test_refine_matches_brute_force(orc, dtype, metric):
    rng = np.random.default_rng(11)
    n, dim, nq, nc, k = 500, 37, 23, 40, 7
    if np.dtype(dtype).kind == "f":
        data = rng.standard_normal((n, dim)).astype(dtype)
        q = rng.standard_normal((nq, dim)).astype(dtype)
    else:
        lo, hi = (-128, 128) if dtype == np.int8 else (0, 256)
        data = rng.integers(lo, hi, (n, dim)).astype(dtype)
        q = rng.integers(lo, hi, (nq, dim)).astype(dtype)
    cand = rng.integers(0, n, (nq, nc)).astype(np.int64)
    cand[0, :5] = [-1, n, n + 7, -9, 2 ** 40]       # out of range: skipped
    cand[1, :] = -1                                  # nothing valid: unfilled outputs
    cand[2, : nc - 3] = n                            # fewer valid candidates than k
    ids, dist = orc.refine(data, q, cand, k, metric)
    want_ids, want_dist = _brute(data, q, cand, k, metric)
    assert np.array_equal(ids[1], np.full(k, -1)) and np.all(dist[1] == np.finfo(np.float32).max)
    assert (ids[2, 3:] == -1).all()
    if np.dtype(dtype).kind in "iu":
        assert np.array_equal(ids, want_ids)
        assert np.array_equal(dist.astype(np.float64), want_dist.astype(np.float32).astype(np.float64))
    else:
        np.testing.assert_allclose(dist, want_dist, rtol=2e-5, atol=1e-6)
        same = ids == want_ids
        # a swap is only acceptable between (near-)equal distances
        assert np.all(same | np.isclose(dist, want_dist, rtol=2e-5, atol=1e-6))


def test_refine_rejects_bad_arguments(orc):
    data = np.zeros((4, 3), dtype=np.float32)
    cand = np.zeros((2, 2), dtype=np.int64)
    with pytest.raises(RuntimeError):
        orc.refine(data, data[:2], cand, 3, 0)      # k > n_candidates
    with pytest.raises(RuntimeError):
        orc.refine(data, data[:2], cand, 1, 2)      # cosine: not supported
