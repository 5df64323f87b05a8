"""Pins the oracle's search against textbook formulas computed independently with numpy (no GPU).

What is checked, and against what:
  * lookup table + scan  ==  || (q - centre) - decode(codes) ||^2  by brute-force reconstruction
    in float64 (L2), q . decode (inner product), 1 - q^ . decode (cosine);
  * reduced-precision tables: numpy's own float16 rounding / the closed-form fp8 truncation of the
    fp32 table, then a sequential float32 / float16 sum done with numpy scalars;
  * coarse selection vs. textbook squared distances; chunk indices vs. cumsum; id translation vs.
    searchsorted; distance post-processing closed forms; invariance to threading;
  * recall against exact search on the distribution the reference's own tests use.
"""
import os

import numpy as np
import pytest

import helpers as H

GOLD = os.path.join(os.path.dirname(__file__), "golden")

R_32F, R_16F, R_8U = 0, 2, 8


def _setup(orc, n=1500, dim=24, n_lists=12, pq_dim=12, pq_bits=8, dtype=np.float32,
           metric="sqeuclidean", kind="subspace", force_rot=False, seed=5):
    data = H.make_data(n, dim, dtype, seed)
    model = H.train(data, n_lists, pq_dim, pq_bits, metric=metric, codebook_kind=kind,
                    force_random_rotation=force_rot, iters=4)
    ix, labels, codes = H.oracle_index_with_data(orc, model, data, pq_dim, pq_bits, metric, kind)
    queries = H.make_data(40, dim, dtype, seed + 100)
    return data, model, ix, labels, codes, queries


def _all_pairs(orc, ix, queries, **kw):
    """Distances of every query to every stored row, as a dense [n_queries, n] array by id."""
    n = ix.size
    nb, d = orc.search(ix, queries, n, ix.n_lists, **kw)
    dense = np.full((queries.shape[0], n), np.nan, dtype=np.float32)
    for q in range(queries.shape[0]):
        dense[q, nb[q]] = d[q]
    assert not np.isnan(dense).any()
    return dense


@pytest.mark.parametrize("dtype,pq_bits,kind,force_rot", [
    (np.float32, 8, "subspace", False), (np.float32, 5, "subspace", True),
    (np.float16, 6, "cluster", False), (np.uint8, 8, "subspace", False),
    (np.int8, 4, "cluster", True), (np.float32, 7, "subspace", False)])
def test_l2_scores_equal_reconstruction_distance(orc, dtype, pq_bits, kind, force_rot):
    dim = 24 if not force_rot else 22   # 22 is not a multiple of pq_dim: rot_dim = 24 > dim
    pq_dim = 12 if pq_bits != 5 and pq_bits != 7 else 8
    data, model, ix, labels, codes, queries = _setup(orc, dim=dim, pq_dim=pq_dim, pq_bits=pq_bits,
                                                     dtype=dtype, kind=kind, force_rot=force_rot)
    got = _all_pairs(orc, ix, queries)
    rec = H.decode_rows(model, labels, codes, pq_bits, kind)                    # [n, rot_dim] f64
    rq = H.to_float(queries).astype(np.float64) @ model["rotation_matrix"].astype(np.float64).T
    want = ((rq[:, None, :] - rec[None, :, :]) ** 2).sum(-1)
    s = {np.uint8: 256.0, np.int8: 128.0}.get(dtype, 1.0)
    want = want * s * s
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=1e-6 * want.max())


def test_l2sqrt_is_the_root_of_l2(orc):
    data, model, ix, labels, codes, queries = _setup(orc, dtype=np.uint8)
    l2 = _all_pairs(orc, ix, queries)
    ix2 = H.oracle_index(orc, model, data.shape[1], 12, 8, "euclidean")
    ix2.fill(labels, codes)
    root = _all_pairs(orc, ix2, queries)
    # sqrt(d) * 256 versus d * 65536
    np.testing.assert_allclose(root, np.sqrt(l2.astype(np.float64)), rtol=1e-6)


@pytest.mark.parametrize("kind", ["subspace", "cluster"])
def test_inner_product_scores_equal_dot_with_reconstruction(orc, kind):
    data, model, ix, labels, codes, queries = _setup(orc, metric="inner_product", kind=kind,
                                                     dtype=np.int8)
    got = _all_pairs(orc, ix, queries)
    rec = H.decode_rows(model, labels, codes, 8, kind)
    rq = H.to_float(queries).astype(np.float64) @ model["rotation_matrix"].astype(np.float64).T
    want = (rq @ rec.T) * 128.0 * 128.0      # returned "distance" is the positive similarity
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=2e-5 * np.abs(want).max())


def test_cosine_scores_equal_one_minus_cos(orc):
    data, model, ix, labels, codes, queries = _setup(orc, metric="cosine", force_rot=True, dim=22)
    got = _all_pairs(orc, ix, queries)
    rec = H.decode_rows(model, labels, codes, 8)
    rq = H.to_float(queries).astype(np.float64) @ model["rotation_matrix"].astype(np.float64).T
    rq /= np.linalg.norm(rq, axis=1, keepdims=True)
    want = 1.0 - rq @ rec.T
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=2e-6)


def _fp8_encode_np(v, signed):
    """Closed form of fp_8bit<5, S>::float2fp_8bit on a float32 array."""
    a = np.abs(v) if signed else v
    bits = a.astype(np.float32).view(np.uint32).astype(np.int64)
    u = ((bits + (15 << 23) - 0x3f800000) >> 20).astype(np.int64)
    u = np.where(a < 2.0 ** -15, 0, u)
    u = np.where(a >= 122880.0, 0xFF, u) & 0xFF
    if signed:
        u = (u & 0xFE) | (v < 0)
    return u.astype(np.uint8)


def _fp8_decode_np(u, signed, half):
    mag = (u & 0xFE) if signed else u
    if half:
        bits = (0x0040 + (mag.astype(np.uint32) << 7)).astype(np.uint16)
        out = bits.view(np.float16)
    else:
        bits = (0x38080000 + (mag.astype(np.uint32) << 20)).astype(np.uint32)
        out = bits.view(np.float32)
    if signed:
        out = np.where(u & 1, -out, out)
    return out


@pytest.mark.parametrize("metric,lut,internal", [
    ("sqeuclidean", R_16F, R_32F), ("sqeuclidean", R_8U, R_32F), ("sqeuclidean", R_16F, R_16F),
    ("sqeuclidean", R_8U, R_16F), ("inner_product", R_8U, R_32F), ("inner_product", R_8U, R_16F),
    ("inner_product", R_16F, R_16F)])
def test_reduced_precision_tables_and_sums(orc, metric, lut, internal):
    data, model, ix, labels, codes, queries = _setup(orc, n=600, n_lists=5, metric=metric, seed=9)
    queries = queries[:6]
    signed = metric != "sqeuclidean"
    n = ix.size
    nb, d = orc.search(ix, queries, n, ix.n_lists, lut_dtype=lut, internal_distance_dtype=internal)
    for q in range(queries.shape[0]):
        dense = np.empty(n, dtype=np.float32)
        dense[nb[q]] = d[q]
        for l in range(ix.n_lists):
            rows = np.nonzero(labels == l)[0]
            if rows.size == 0:
                continue
            lut32 = orc.make_lut(ix, queries[q], l, R_32F)
            got_lut = orc.make_lut(ix, queries[q], l, lut)
            if lut == R_16F:
                with np.errstate(over="ignore"):
                    want_lut = lut32.astype(np.float16)
                assert np.array_equal(got_lut, want_lut.view(np.uint16))
                table = want_lut if internal == R_16F else want_lut.astype(np.float32)
            else:
                want_u = _fp8_encode_np(lut32, signed)
                assert np.array_equal(got_lut, want_u)
                table = _fp8_decode_np(want_u, signed, internal == R_16F)
            acc_t = np.float16 if internal == R_16F else np.float32
            acc = np.zeros(rows.size, dtype=acc_t)
            with np.errstate(over="ignore", invalid="ignore"):
                for j in range(ix.pq_dim):
                    acc = (acc + table[j, codes[rows, j]].astype(acc_t)).astype(acc_t)
            want = acc.astype(np.float32)
            if signed:
                want = want * np.float32(-1.0)
            keep = ~np.isnan(want)
            assert np.array_equal(dense[rows][keep], want[keep])


def test_lut_fp32_matches_numpy(orc):
    data, model, ix, labels, codes, queries = _setup(orc, pq_bits=6, kind="cluster")
    q = H.to_float(queries[3]).astype(np.float64)
    for l in (0, 3, 7):
        got = orc.make_lut(ix, queries[3], l, R_32F)
        diff = q - model["centers_rot"][l].astype(np.float64)
        book = model["pq_centers"][l].astype(np.float64)          # [pq_len, B]
        want = ((diff.reshape(ix.pq_dim, ix.pq_len, 1) - book[None]) ** 2).sum(1)
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("metric", ["sqeuclidean", "inner_product"])
def test_coarse_selection_matches_textbook(orc, metric):
    data, model, ix, labels, codes, queries = _setup(orc, n_lists=40, metric=metric, n=800)
    P = 7
    probes, scores = orc.select_clusters(ix, queries, P)
    c = model["centers"][:, :data.shape[1]].astype(np.float64)
    qf = H.to_float(queries).astype(np.float64)
    if metric == "sqeuclidean":
        dist = ((qf[:, None, :] - c[None]) ** 2).sum(-1)
        # the reference ranks by ||c||^2 - 2 q.c, i.e. the distance minus ||q||^2
        ref_score = dist - (qf ** 2).sum(1, keepdims=True)
    else:
        dist = -(qf @ c.T)
        ref_score = dist
    order = np.argsort(dist, axis=1, kind="stable")[:, :P]
    for q in range(queries.shape[0]):
        assert set(probes[q].tolist()) == set(order[q].tolist())
        assert list(probes[q]) == sorted(probes[q], key=lambda l: (scores[q][list(probes[q]).index(l)], l))
        np.testing.assert_allclose(scores[q], ref_score[q, probes[q]], rtol=1e-4, atol=1e-4)
    # column `dim` of the centres holds the squared norm (ivf_pq_build.cuh:277-283)
    np.testing.assert_allclose(model["centers"][:, data.shape[1]], (c ** 2).sum(1), rtol=1e-5)


def test_sample_numbering_and_id_translation(orc):
    """neighbours come back as source ids: cumsum of probed sizes + searchsorted(side='right')."""
    data, model, ix0, labels, codes, queries = _setup(orc, n=500, n_lists=9)
    ids = (np.arange(500, dtype=np.int64) * 7 + 1000)[::-1].copy()
    ix = H.oracle_index(orc, model, data.shape[1], 12, 8)
    ix.fill(labels, codes, ids)
    P, k = 3, 6
    nb, d, probes = orc.search(ix, queries, k, P, return_probes=True)
    for q in range(queries.shape[0]):
        rows = np.concatenate([np.nonzero(labels == l)[0] for l in probes[q]])
        chunk = np.cumsum([int(ix.list_sizes[l]) for l in probes[q]])
        assert rows.size == chunk[-1]
        # every returned id belongs to a probed list
        assert set(nb[q].tolist()) <= set(ids[rows].tolist())
        # the distance of a returned id equals its distance in an exhaustive search
    full_nb, full_d = orc.search(ix, queries, ix.size, ix.n_lists)
    for q in range(queries.shape[0]):
        lookup = dict(zip(full_nb[q].tolist(), full_d[q].tolist()))
        for r in range(k):
            assert lookup[int(nb[q, r])] == d[q, r]
        assert np.all(np.diff(d[q]) >= 0)
        # nothing closer was skipped inside the probed lists
        rows = np.concatenate([np.nonzero(labels == l)[0] for l in probes[q]])
        best = sorted(lookup[int(i)] for i in ids[rows])[:k]
        assert np.array_equal(np.array(best, dtype=np.float32), d[q])


def test_unfilled_slots(orc):
    data, model, ix, labels, codes, queries = _setup(orc, n=300, n_lists=30)
    sizes = ix.list_sizes.astype(np.int64)
    k = int(sizes.max()) + 5
    nb, d, probes = orc.search(ix, queries, k, 1, return_probes=True)
    for q in range(queries.shape[0]):
        have = int(sizes[probes[q, 0]])
        assert np.all(nb[q, :have] != np.iinfo(np.int64).max)
        assert np.all(nb[q, have:] == np.iinfo(np.int64).max)      # kOutOfBoundsRecord
        assert np.all(d[q, have:] == np.finfo(np.float32).max)


def test_threading_and_query_order_do_not_change_results(orc):
    data, model, ix, labels, codes, queries = _setup(orc)
    a = orc.search(ix, queries, 10, 4, n_threads=1)
    b = orc.search(ix, queries, 10, 4, n_threads=5)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    perm = np.random.default_rng(0).permutation(queries.shape[0])
    c = orc.search(ix, queries[perm], 10, 4)
    assert np.array_equal(a[0][perm], c[0]) and np.array_equal(a[1][perm], c[1])


def test_bitset_filter(orc):
    data, model, ix, labels, codes, queries = _setup(orc, n=700)
    n = data.shape[0]
    keep = np.ones(n, dtype=bool)
    keep[:300] = False                      # the reference's filter test removes ids [0, 300)
    bits = np.packbits(keep, bitorder="little")
    bits = np.concatenate([bits, np.zeros((-bits.size) % 4, dtype=np.uint8)]).view(np.uint32)
    nb, d = orc.search(ix, queries, 8, ix.n_lists, filter_bitset=bits, filter_nbits=n)
    assert nb.min() >= 300
    # same as searching an index that only holds the kept rows
    ix2 = H.oracle_index(orc, model, data.shape[1], 12, 8)
    ix2.fill(labels[keep], codes[keep], np.nonzero(keep)[0].astype(np.int64))
    nb2, d2 = orc.search(ix2, queries, 8, ix.n_lists)
    assert np.array_equal(d, d2)
    assert np.array_equal(nb, nb2)


def test_parameter_validation(orc):
    data, model, ix, labels, codes, queries = _setup(orc, n=200, n_lists=4)
    with pytest.raises(ValueError, match="must be positive"):
        orc.search(ix, queries, 0, 2)
    with pytest.raises(ValueError, match="total size"):
        orc.search(ix, queries, 201, 2)
    with pytest.raises(ValueError, match="n_probes"):
        orc.search(ix, queries, 5, 0)
    with pytest.raises(ValueError, match="combination"):
        orc.search(ix, queries, 5, 2, lut_dtype=R_32F, internal_distance_dtype=R_16F)
    with pytest.raises(ValueError, match="lut_dtype"):
        orc.search(ix, queries, 5, 2, lut_dtype=3)
    # n_probes larger than n_lists is clamped
    a = orc.search(ix, queries, 5, 4)
    b = orc.search(ix, queries, 5, 400)
    assert np.array_equal(a[0], b[0])


@pytest.mark.parametrize("pq_bits,lut,floor", [(8, R_32F, 0.86), (8, R_8U, 0.84), (6, R_16F, 0.84),
                                                (4, R_32F, 0.79)])
def test_recall_on_the_reference_test_distribution(orc, pq_bits, lut, floor):
    """Recall floors the reference's own suite enforces on uniform [0.1, 2) data, 4096 x 64,
    k = 32, 32 lists, 20 probes (cpp/tests/neighbors/ann_ivf_pq.cuh:27-43,979-1122).  The 4-bit floor
    there is for per-cluster codebooks."""
    data = H.uniform_data(4096, 64, 1234)
    queries = H.uniform_data(256, 64, 4321)
    kind = "cluster" if pq_bits == 4 else "subspace"
    model = H.train(data, 32, 64, pq_bits, codebook_kind=kind, iters=10)
    ix, _, _ = H.oracle_index_with_data(orc, model, data, 64, pq_bits, codebook_kind=kind)
    nb, _ = orc.search(ix, queries, 32, 20, lut_dtype=lut)
    d = ((queries[:, None, :].astype(np.float64) - data[None].astype(np.float64)) ** 2).sum(-1)
    truth = np.argsort(d, axis=1)[:, :32]
    hits = sum(len(set(a.tolist()) & set(b.tolist())) for a, b in zip(nb, truth))
    assert hits / truth.size >= floor


def test_committed_toy_index(orc):
    g = np.load(os.path.join(GOLD, "toy_index.npz"))
    dim, pq_dim, pq_bits = 8, 4, 8
    ix = orc.Index(0, 0, dim, pq_dim, pq_bits, g["centers"], g["centers"][:, :dim].copy(),
                   np.eye(dim, dtype=np.float32), g["pq_centers"])
    labels, codes = orc.encode(ix, g["data"], n_threads=1)
    assert np.array_equal(labels, g["labels"]) and np.array_equal(codes, g["codes"])
    ix.fill(labels, codes)
    nb, d, probes = orc.search(ix, g["queries"], 3, 2, return_probes=True, n_threads=1)
    assert np.array_equal(nb, g["neighbors"])
    assert np.array_equal(d, g["distances"])
    assert np.array_equal(probes, g["probes"])
    # hand check: labels are the nearest centres, codes the nearest codebook entries
    c = g["centers"][:, :dim].astype(np.float64)
    x = g["data"].astype(np.float64)
    assert np.array_equal(labels, ((x[:, None] - c[None]) ** 2).sum(-1).argmin(1))
    res = (x - c[labels]).reshape(-1, pq_dim, dim // pq_dim)
    book = g["pq_centers"].astype(np.float64)                      # [pq_dim, pq_len, B]
    dist = ((res[:, :, :, None] - book[None]) ** 2).sum(2)          # [n, pq_dim, B]
    assert np.array_equal(codes, dist.argmin(2))


@pytest.mark.parametrize("metric", ["sqeuclidean", "inner_product", "cosine"])
def test_encode_labels_follow_the_coarse_clustering_metric(orc, metric):
    """Rows join the nearest centre by L2 for L2 and inner-product indexes, and the centre of
    largest inner product with the normalised row for cosine (coarse_clustering_metric,
    cpp/src/neighbors/ivf_pq/ivf_pq_build.cuh:70-76, :1141)."""
    rng = np.random.default_rng(11)
    dim, n_lists = 16, 24
    data = rng.standard_normal((600, dim)).astype(np.float32)
    # centres of very different norms, so that L2 and inner product disagree on most rows
    centers = (rng.standard_normal((n_lists, dim)) * rng.uniform(0.2, 3.0, (n_lists, 1))).astype(np.float32)
    model = H.train(data, n_lists, 8, 8, metric=metric, iters=2)
    ext = model["centers"].copy()
    ext[:, :dim] = centers
    ext[:, dim] = (centers.astype(np.float64) ** 2).sum(1).astype(np.float32)
    model["centers"] = ext
    model["centers_rot"] = (centers @ model["rotation_matrix"].T).astype(np.float32)
    ix = H.oracle_index(orc, model, dim, 8, 8, metric=metric)
    labels, _ = orc.encode(ix, data)
    x, c = data.astype(np.float64), centers.astype(np.float64)
    by_l2 = ((x[:, None] - c[None]) ** 2).sum(-1).argmin(1)
    by_ip = ((x / np.linalg.norm(x, axis=1, keepdims=True)) @ c.T).argmax(1)
    want = by_ip if metric == "cosine" else by_l2
    assert (by_l2 != by_ip).mean() > 0.3
    assert np.array_equal(labels, want)


# --- coarse search in reduced precision (ivf_pq_search.cuh:170-340) ---

R_8I = 3


def _f32_fma_chain(a, b):
    """sum_d a[..., d] * b[..., d] as one fp32 fused-multiply-add chain over ascending d, with numpy
    scalars only.  The operands used below (binary16 values) have 11-bit significands, so a product
    is exact in float64 and `product + acc` in float64 is the exact sum unless the exponents are
    more than 29 binades apart, where the smaller term is far below half an fp32 ulp anyway: one
    rounding to float32 per step is the fused multiply-add."""
    acc = np.zeros(np.broadcast_shapes(a.shape, b.shape)[:-1], dtype=np.float32)
    for d in range(a.shape[-1]):
        acc = (a[..., d].astype(np.float64) * b[..., d].astype(np.float64)
               + acc.astype(np.float64)).astype(np.float32)
    return acc


def _half_scores_numpy(model, dim, qf, ip):
    """The binary16 coarse score of every (query, list) from numpy's own float16: centres (norm
    column included) and queries rounded to binary16, products accumulated in fp32 over ascending
    columns, the norm column times -0.5 (L2) last, times alpha, rounded to binary16."""
    ch = model["centers"].astype(np.float16).astype(np.float32)
    qh = qf.astype(np.float16).astype(np.float32)
    acc = _f32_fma_chain(ch[None, :, :dim], qh[:, None, :])
    if not ip:
        acc = (ch[None, :, dim].astype(np.float64) * -0.5 + acc.astype(np.float64)).astype(np.float32)
    alpha = np.float32(-1.0 if ip else -2.0)
    return (alpha * acc).astype(np.float16).astype(np.float32)


@pytest.mark.parametrize("metric,dtype", [("sqeuclidean", np.float32), ("inner_product", np.float32),
                                          ("sqeuclidean", np.uint8), ("cosine", np.float16)])
def test_half_coarse_scores_equal_numpy_float16(orc, metric, dtype):
    dim = 24
    data, model, ix, labels, codes, queries = _setup(orc, n_lists=40, metric=metric, n=800, dtype=dtype)
    ip = metric != "sqeuclidean"
    # centres whose norms (8 .. 40 here after scaling) and elements need rounding to binary16
    assert np.any(model["centers"].astype(np.float16).astype(np.float32) != model["centers"])
    want = _half_scores_numpy(model, dim, H.to_float(queries), ip)
    P = ix.n_lists  # all lists: every score is compared
    probes, scores = orc.select_clusters(ix, queries, P, coarse_search_dtype=R_16F)
    for q in range(queries.shape[0]):
        assert sorted(probes[q].tolist()) == list(range(P))
        np.testing.assert_array_equal(scores[q], want[q, probes[q]])
        # ascending (score, list)
        key = list(zip(scores[q].tolist(), probes[q].tolist()))
        assert key == sorted(key)
    # the half scores differ from the fp32 ones (the test would not notice a path that ignores the dtype)
    _, s32 = orc.select_clusters(ix, queries, P, coarse_search_dtype=R_32F)
    assert np.any(np.sort(s32, axis=1) != np.sort(scores, axis=1))


def test_half_coarse_scores_on_exact_integers(orc):
    """Integer-valued centres and queries: every product and partial sum is exact, so the score has
    a closed form, and the norm column (2049 -> 2048 in binary16) shows whether it was rounded."""
    dim, pq_dim = 8, 4
    rng = np.random.default_rng(3)
    c = rng.integers(-20, 21, (6, dim)).astype(np.float32)
    c[0] = [32, 32, 1, 0, 0, 0, 0, 0]          # squared norm 2049: not a binary16 number
    de = orc.dim_ext(dim)
    centers = np.zeros((6, de), dtype=np.float32)
    centers[:, :dim] = c
    centers[:, dim] = (c.astype(np.float64) ** 2).sum(1)
    assert centers[0, dim] == 2049
    model = {"centers": centers, "centers_rot": c.copy(), "rotation_matrix": np.eye(dim, dtype=np.float32),
             "pq_centers": np.zeros((pq_dim, 2, 256), dtype=np.float32)}
    ix = H.oracle_index(orc, model, dim, pq_dim, 8)
    q = rng.integers(-9, 10, (5, dim)).astype(np.float32)
    probes, scores = orc.select_clusters(ix, q, 6, coarse_search_dtype=R_16F)
    n16 = centers[:, dim].astype(np.float16).astype(np.float64)
    assert n16[0] == 2048
    want = (n16[None, :] - 2.0 * (q.astype(np.float64) @ c.astype(np.float64).T))
    want = want.astype(np.float16).astype(np.float32)
    for i in range(5):
        np.testing.assert_array_equal(scores[i], want[i, probes[i]])


def _int8_rows_numpy(model, dim, qf, ip):
    """Quantised centre and query rows of the 8-bit coarse search from the formulas in
    ivf_pq_index.cu:661-738 and ivf_pq_search.cuh:199-210, in numpy."""
    de8 = (dim + 2 + 15) // 16 * 16
    m = de8 - dim
    c = model["centers"]
    n = c.shape[0]
    c8 = np.zeros((n, de8), dtype=np.int64)
    c8[:, :dim] = np.trunc(np.clip(c[:, :dim] * np.float32(128), -128, 127))
    x = c[:, dim]
    y = np.clip(x * (np.float32(64) / np.float32(m - 1)), -128, 127).astype(np.float32)
    ry = np.where(y >= 0, np.floor(y + np.float32(0.5)), np.ceil(y - np.float32(0.5)))  # roundf: half away from zero
    z = np.clip((y - ry.astype(np.float32)) * np.float32(128), -128, 127)
    c8[:, dim] = np.trunc(z)
    c8[:, dim + 1:] = ry[:, None]
    q8 = np.zeros((qf.shape[0], de8), dtype=np.int64)
    q8[:, :dim] = np.trunc(np.clip(qf * np.float32(128), -128, 127))
    q8[:, dim] = 1 - m
    q8[:, dim + 1:] = 0 if ip else -128
    return c8, q8


@pytest.mark.parametrize("metric,dtype,dim", [("sqeuclidean", np.float32, 24), ("inner_product", np.float32, 24),
                                              ("sqeuclidean", np.uint8, 24), ("sqeuclidean", np.int8, 12)])
def test_int8_coarse_scores_equal_the_formulas(orc, metric, dtype, dim):
    pq_dim = dim // 2
    data = H.make_data(800, dim, dtype, 5)
    if dtype == np.float32:
        data = (data * 0.25).astype(np.float32)  # keep 128 x within int8 for most elements
    model = H.train(data, 40, pq_dim, 8, metric=metric, iters=4)
    ix, labels, codes = H.oracle_index_with_data(orc, model, data, pq_dim, 8, metric)
    queries = H.make_data(40, dim, dtype, 105)
    if dtype == np.float32:
        queries = (queries * 0.25).astype(np.float32)
    ip = metric != "sqeuclidean"
    qf = H.to_float(queries)
    c8, q8 = _int8_rows_numpy(model, dim, qf, ip)
    if dtype == np.uint8:   # mapping<int8_t>(uint8_t x) = x >> 1
        np.testing.assert_array_equal(q8[:, :dim], queries.astype(np.int64) >> 1)
    if dtype == np.int8:
        np.testing.assert_array_equal(q8[:, :dim], queries.astype(np.int64))
    want = (-1 if ip else -2) * (q8 @ c8.T)
    P = ix.n_lists
    probes, scores = orc.select_clusters(ix, queries, P, coarse_search_dtype=R_8I)
    for q in range(queries.shape[0]):
        np.testing.assert_array_equal(scores[q].astype(np.int64), want[q, probes[q]])
        key = list(zip(scores[q].tolist(), probes[q].tolist()))
        assert key == sorted(key)
    if not ip:
        # what the split norm is for: the integer score tracks 128^2 (||c||^2 - 2 q.c) to within the
        # quantisation of the elements, so the nearest list by the fp32 score is among the first few
        p32, _ = orc.select_clusters(ix, queries, 1, coarse_search_dtype=R_32F)
        hits = sum(int(p32[q, 0]) in probes[q, :4].tolist() for q in range(queries.shape[0]))
        assert hits >= 0.9 * queries.shape[0]


def test_int8_split_norm_identity():
    """dot of the padding columns = -(m - 1) (128 round(y) + z) ~ -128^2 * ||c||^2 / 2."""
    dim = 24
    model = {"centers": np.zeros((3, 32), dtype=np.float32)}
    model["centers"][:, dim] = [0.3, 1.0, 2.5]
    c8, q8 = _int8_rows_numpy(model, dim, np.zeros((1, dim), dtype=np.float32), False)
    pad = (q8[:, dim:] @ c8[:, dim:].T)[0]
    np.testing.assert_allclose(pad, -8192.0 * model["centers"][:, dim], atol=8)  # z is truncated: up to m - 1 = 7 off


@pytest.mark.parametrize("coarse", [R_16F, R_8I])
@pytest.mark.parametrize("force_rot", [False, True])
def test_rotation_takes_the_coarse_search_operands(orc, coarse, force_rot):
    """With a 16-bit or 8-bit coarse search the rotation GEMM multiplies the rounded query rows by
    the rotation matrix in the same type (ivf_pq_search.cuh:996-1019): seen through the fp32 lookup
    table, whose entries are (rot_q - centre - codebook entry)^2."""
    dim = 22 if force_rot else 24
    data, model, ix, labels, codes, queries = _setup(orc, dim=dim, force_rot=force_rot, n=600)
    queries = (queries * 0.3).astype(np.float32)
    qf = H.to_float(queries)
    R = model["rotation_matrix"]
    if coarse == R_16F:
        rq = qf.astype(np.float16).astype(np.float64) @ R.astype(np.float16).astype(np.float64).T
    else:
        q8 = np.trunc(np.clip(qf * np.float32(128), -128, 127)).astype(np.float64)
        r8 = np.trunc(np.clip(R * np.float32(128), -128, 127)).astype(np.float64)
        rq = (q8 @ r8.T) / 16384.0
    rq32 = qf.astype(np.float64) @ R.astype(np.float64).T
    assert np.abs(rq - rq32).max() > 1e-4   # the rounded operands are visible
    for qi in (0, 7):
        for l in (1, 5):
            got = orc.make_lut(ix, queries[qi], l, R_32F, coarse_search_dtype=coarse)
            diff = rq[qi] - model["centers_rot"][l].astype(np.float64)
            book = model["pq_centers"].astype(np.float64)      # [pq_dim, pq_len, B]
            want = ((diff.reshape(ix.pq_dim, ix.pq_len, 1) - book) ** 2).sum(1)
            np.testing.assert_allclose(got, want, rtol=2e-5, atol=1e-7)
