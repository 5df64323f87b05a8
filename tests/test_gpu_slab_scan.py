"""GPU parity of the CU-wide scan with the lookup table in slabs of 64 subspaces (scan_slab_kernel):
8-bit codes whose pq_dim is a multiple of 32 and not one of the whole-table kernel's shapes - the
reference's default pq_dim for 256- to 1536-dimensional rows (dim / 2: 128 ... 768 subspaces of
length 2, cpp/src/neighbors/ivf_pq_index.cu:612-622) and subspace lengths 1, 3, 4, 8.

Every case goes through the C ABI and is compared with the CPU oracle bit for bit (ids and
distances); the search profile says which kernel scanned the pairs.
"""
import numpy as np
import pytest
import torch

import gpu_helpers as G
import helpers as H
from cuvs_amd import ivf_pq
from cuvs_amd.resources import Resources

pytestmark = pytest.mark.gpu

R_32F, R_16F, R_8U = np.float32, np.float16, np.uint8
ORC_DT = {np.float32: 0, np.float16: 2, np.int8: 3, np.uint8: 8}
SLAB, GENERIC = 6, 0
TABLES = [(R_32F, R_32F), (R_16F, R_32F), (R_8U, R_32F), (R_16F, R_16F), (R_8U, R_16F)]


def _build(orc, n, dim, n_lists, pq_dim, pq_bits=8, dtype=np.float32, metric="sqeuclidean", kind="subspace",
           seed=3, n_queries=40, rows=None, labels=None):
    print(f"case n={n} dim={dim} lists={n_lists} pq_dim={pq_dim} bits={pq_bits} dtype={np.dtype(dtype).name} "
          f"metric={metric} kind={kind}", flush=True)
    data = H.make_data(n, dim, dtype, seed) if rows is None else rows
    model = H.train(data, n_lists, pq_dim, pq_bits, metric=metric, codebook_kind=kind, iters=3)
    queries = H.make_data(n_queries, dim, dtype, seed + 100)
    index = G.build_gpu_index(model, data, pq_dim, pq_bits, metric, kind, labels=labels)
    ix, _ = G.read_back(orc, index, model, dim, pq_dim, pq_bits, metric, kind)
    return data, queries, index, ix


def _check(orc, res, index, ix, queries, k, n_probes, lut, internal, kernel=SLAB, exact=True, **kw):
    sp = ivf_pq.SearchParams(n_probes=n_probes, lut_dtype=lut, internal_distance_dtype=internal)
    d, nb = ivf_pq.search(sp, index, G.to_dev(queries), k, resources=res, **kw)
    res.sync()
    prof = ivf_pq.get_search_profile(res)
    assert prof["scan_kernel"] == kernel, f"scanned by kernel {prof['scan_kernel']}, expected {kernel}"
    okw = {}
    if "filter_bitset" in kw:
        okw = dict(filter_bitset=kw["filter_bitset"].cpu().numpy().view(np.uint32), filter_nbits=kw["filter_nbits"])
    want_nb, want_d = orc.search(ix, queries, k, n_probes, lut_dtype=ORC_DT[lut],
                                 internal_distance_dtype=ORC_DT[internal], **okw)
    H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 2e-3, exact=exact)
    return nb, d, prof


def _profiling_resources(early_stop="auto"):
    res = Resources()
    res.enable_profiling(True)
    res.set_search_tuning(early_stop=early_stop)
    return res


# (dim, pq_dim): two slabs; six slabs; seven and a half; pq_len 1 in one slab; pq_len 3, 4, 8;
# a half slab behind a whole one with pq_len 3; two and a half slabs of pq_len 1; one half slab of pq_len 8
SHAPES = [(256, 128), (768, 384), (960, 480), (64, 64), (192, 64), (256, 64), (512, 64), (288, 96), (160, 160),
          (256, 32)]


@pytest.mark.parametrize("metric,kind", [("sqeuclidean", "subspace"), ("inner_product", "subspace"),
                                         ("sqeuclidean", "cluster"), ("cosine", "cluster")])
@pytest.mark.parametrize("dim,pq_dim", SHAPES)
def test_slab_scan_shapes(orc, dim, pq_dim, metric, kind):
    """Every table / sum type on each shape, both codebook kinds, L2 and inner-product metrics; one
    launch over all pairs (the early stop has its own tests below)."""
    data, queries, index, ix = _build(orc, 6000, dim, 12, pq_dim, metric=metric, kind=kind)
    res = _profiling_resources("off")
    for lut, internal in TABLES:
        _check(orc, res, index, ix, queries, 10, 5, lut, internal)


@pytest.mark.parametrize("dtype", [np.float16, np.int8, np.uint8])
def test_slab_scan_element_types(orc, dtype):
    data, queries, index, ix = _build(orc, 5000, 256, 10, 128, dtype=dtype, metric="euclidean")
    res = _profiling_resources("off")
    _check(orc, res, index, ix, queries, 10, 4, R_16F, R_32F, exact=False)
    data, queries, index, ix = _build(orc, 5000, 256, 10, 128, dtype=dtype)
    _check(orc, res, index, ix, queries, 10, 4, R_8U, R_16F)


@pytest.mark.parametrize("k", [1, 10, 64, 65, 128])
def test_slab_scan_k(orc, k):
    """k up to the kernel's limit: above 64 a wave buffers three tiles' worth of candidates."""
    data, queries, index, ix = _build(orc, 20000, 256, 6, 128, dtype=np.uint8, n_queries=24)
    res = _profiling_resources("off")
    for lut, internal in [(R_16F, R_32F), (R_8U, R_16F)]:
        _check(orc, res, index, ix, queries, k, 3, lut, internal)


def test_slab_scan_beyond_its_k_takes_the_generic_kernel(orc):
    data, queries, index, ix = _build(orc, 8000, 256, 6, 128, n_queries=16)
    res = _profiling_resources("off")
    _check(orc, res, index, ix, queries, 129, 3, R_16F, R_32F, kernel=GENERIC)
    _check(orc, res, index, ix, queries, 128, 3, R_16F, R_32F, kernel=SLAB)


@pytest.mark.parametrize("metric", ["sqeuclidean", "inner_product"])
def test_slab_scan_lists_longer_than_a_row_block(orc, metric):
    """Lists of more than 8192 rows: their sums do not fit the area that carries them from slab to
    slab, so they are scanned in row blocks, each with its tables built again.  Two lists of very
    different lengths share a block iteration (3 lists, pairs in list order)."""
    rng = np.random.default_rng(11)
    dim = 256
    cent = rng.standard_normal((3, dim)).astype(np.float32) * 2
    sizes = [21000, 700, 9000]
    rows = np.concatenate([cent[i] + 0.3 * rng.standard_normal((n, dim)).astype(np.float32)
                           for i, n in enumerate(sizes)])
    labels = np.repeat(np.arange(3), sizes)  # the lists are given, whatever the trained centres say
    order = rng.permutation(rows.shape[0])
    rows, labels = rows[order], labels[order]
    data, queries, index, ix = _build(orc, rows.shape[0], dim, 3, 128, metric=metric, rows=rows, n_queries=37,
                                      labels=labels)
    assert ix.list_sizes.max() > 2 * 8192 and ix.list_sizes.min() < 4096
    res = _profiling_resources("off")
    for lut, internal in [(R_32F, R_32F), (R_16F, R_32F), (R_8U, R_16F)]:
        for k in (10, 100):
            _check(orc, res, index, ix, queries, k, 3, lut, internal)
            _check(orc, res, index, ix, queries, k, 2, lut, internal)


def test_slab_scan_filter_and_empty_lists(orc):
    data, queries, index, ix = _build(orc, 300, 256, 40, 128, n_queries=16)
    n = data.shape[0]
    keep = np.ones(n, dtype=bool)
    keep[::3] = False
    bits = np.packbits(keep, bitorder="little")
    bits = np.concatenate([bits, np.zeros((-bits.size) % 4, dtype=np.uint8)]).view(np.uint32)
    res = _profiling_resources("off")
    for lut, internal in [(R_32F, R_32F), (R_16F, R_32F), (R_8U, R_16F)]:
        _check(orc, res, index, ix, queries, 20, 6, lut, internal,
               filter_bitset=G.to_dev(bits.view(np.int32)), filter_nbits=n)
        _check(orc, res, index, ix, queries, 30, 2, lut, internal)
    # a filter that leaves whole tiles without a row in play, on lists of a few thousand rows
    data, queries, index, ix = _build(orc, 12000, 256, 4, 128, n_queries=16)
    n = data.shape[0]
    keep = np.zeros(n, dtype=bool)
    keep[::97] = True
    bits = np.packbits(keep, bitorder="little")
    bits = np.concatenate([bits, np.zeros((-bits.size) % 4, dtype=np.uint8)]).view(np.uint32)
    _check(orc, res, index, ix, queries, 10, 3, R_16F, R_32F, filter_bitset=G.to_dev(bits.view(np.int32)),
           filter_nbits=n)


@pytest.mark.parametrize("pq_bits,metric", [(5, "sqeuclidean"), (6, "inner_product"), (7, "sqeuclidean")])
def test_slab_scan_of_the_byte_wide_copy_of_narrow_codes(orc, pq_bits, metric):
    """5 - 7 bit codes at 128 subspaces run on the index's byte-per-code copy of the lists."""
    data, queries, index, ix = _build(orc, 6000, 256, 8, 128, pq_bits=pq_bits, metric=metric)
    res = _profiling_resources("off")
    for lut, internal in [(R_16F, R_32F), (R_8U, R_16F)]:
        _check(orc, res, index, ix, queries, 10, 4, lut, internal)


@pytest.mark.parametrize("dim,pq_dim,kind", [(256, 128, "subspace"), (64, 64, "subspace"), (192, 64, "subspace"),
                                             (512, 64, "subspace"), (768, 384, "subspace"), (384, 96, "cluster")])
def test_slab_scan_under_the_early_stop(orc, dim, pq_dim, kind):
    """The three launches of the L2 early stop with this kernel scanning the leading and the
    surviving pairs: the oracle's results, and those of the single launch."""
    import datasets as testing
    allrows = testing.gaussian_mixture(16200, dim, 48, 0.15, seed=82).numpy()
    x, q = allrows[:16000], allrows[16000:]
    model = H.train(x, 80, pq_dim, 8, codebook_kind=kind, iters=3)
    index = G.build_gpu_index(model, x, pq_dim, 8, "sqeuclidean", kind)
    ix, _ = G.read_back(orc, index, model, dim, pq_dim, 8, "sqeuclidean", kind)
    res = _profiling_resources("on")
    for lut, internal in [(R_32F, R_32F), (R_16F, R_32F), (R_8U, R_16F)]:
        for k in (10, 100):
            nb, d, prof = _check(orc, res, index, ix, q, k, 24, lut, internal)
            assert prof["n_screened_pairs"] == q.shape[0] * 23
            assert 0 < prof["n_surviving_pairs"] <= prof["n_screened_pairs"]
            res.set_search_tuning(early_stop="off")
            nb2, d2, prof2 = _check(orc, res, index, ix, q, k, 24, lut, internal)
            assert prof2["n_screened_pairs"] == 0
            res.set_search_tuning(early_stop="on")
            assert torch.equal(nb, nb2) and torch.equal(d, d2)
