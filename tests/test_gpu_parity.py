"""GPU parity: the HIP path through the C ABI against the CPU oracle on the same index and queries.

Bar: probe lists and stored codes bit-exact; neighbour ids equal except at distance ties; distances
within 1e-5 relative for an fp32 lookup table and 2e-3 for fp16 / 8-bit tables.  Because the
kernels use the same operation order as the oracle, most cases are in fact checked for exact
equality (`exact=True`).
"""
import numpy as np
import pytest
import torch

import gpu_helpers as G
import helpers as H
from cuvs_amd import ivf_pq
from cuvs_amd._lib import CuvsError
from cuvs_amd.resources import Resources

pytestmark = pytest.mark.gpu

R_32F, R_16F, R_8U = np.float32, np.float16, np.uint8
ORC_DT = {np.float32: 0, np.float16: 2, np.int8: 3, np.uint8: 8}


def _case(orc, n, dim, n_lists, pq_dim, pq_bits, dtype=np.float32, metric="sqeuclidean",
          kind="subspace", force_rot=False, seed=3, n_queries=64, batches=1):
    print(f"case n={n} dim={dim} lists={n_lists} pq_dim={pq_dim} bits={pq_bits} "
          f"dtype={np.dtype(dtype).name} metric={metric} kind={kind} rot={force_rot}", flush=True)
    data = H.make_data(n, dim, dtype, seed)
    model = H.train(data, n_lists, pq_dim, pq_bits, metric=metric, codebook_kind=kind,
                    force_random_rotation=force_rot, iters=4)
    queries = H.make_data(n_queries, dim, dtype, seed + 100)
    index = G.build_gpu_index(model, data, pq_dim, pq_bits, metric, kind, batches=batches)
    ix, gpu_codes = G.read_back(orc, index, model, dim, pq_dim, pq_bits, metric, kind)
    return data, model, queries, index, ix, gpu_codes


def _search_both(orc, index, ix, queries, k, n_probes, lut=R_32F, internal=R_32F, coarse=R_32F,
                 **kw):
    sp = ivf_pq.SearchParams(n_probes=n_probes, lut_dtype=lut, internal_distance_dtype=internal,
                             coarse_search_dtype=coarse, **kw)
    d, nb = ivf_pq.search(sp, index, G.to_dev(queries), k)
    torch.cuda.synchronize()
    want_nb, want_d = orc.search(ix, queries, k, n_probes, lut_dtype=ORC_DT[lut],
                                 internal_distance_dtype=ORC_DT[internal],
                                 coarse_search_dtype=ORC_DT[coarse])
    return nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d


def test_config1_tiny_l2_fp32(orc):
    """BASELINE configs[0]: 10,000 x 128 fp32 from a 64-component mixture, 64 lists, pq_dim 32,
    8-bit, 100 queries, k = 10, 8 probes, fp32 table and distances."""
    import datasets as testing
    x = testing.gaussian_mixture(10000, 128, 64, 0.3, seed=1234).numpy()
    q = testing.gaussian_mixture(10100, 128, 64, 0.3, seed=1234).numpy()[10000:]
    model = H.train(x, 64, 32, 8, iters=10)
    index = G.build_gpu_index(model, x, 32, 8)
    ix, gpu_codes = G.read_back(orc, index, model, 128, 32, 8)
    # stored codes and list membership equal the oracle's encoding of the same rows
    labels, codes = orc.encode(ix, x)
    sizes = np.bincount(labels, minlength=64)
    assert np.array_equal(sizes, ix.list_sizes)
    for l in range(64):
        order = np.argsort(ix.list_inds[l])
        assert np.array_equal(ix.list_inds[l][order], np.nonzero(labels == l)[0])
        assert np.array_equal(gpu_codes[l][order], codes[labels == l])
    # probes bit-exact
    sp = ivf_pq.SearchParams(n_probes=8)
    probes = ivf_pq.select_clusters(sp, index, G.to_dev(q)).cpu().numpy().view(np.uint32)
    want_probes, _ = orc.select_clusters(ix, q, 8)
    assert np.array_equal(probes, want_probes)
    nb, d, want_nb, want_d = _search_both(orc, index, ix, q, 10, 8)
    H.compare_results(nb, d, want_nb, want_d, 1e-5, exact=True)
    truth = testing.exact_knn(torch.from_numpy(x), torch.from_numpy(q), 10).numpy()
    assert abs(testing.recall(nb, truth) - testing.recall(want_nb, truth)) <= 0.005
    assert testing.recall(nb, truth) > 0.5  # pq_len = 4 and 8 of 64 lists: recall is modest


@pytest.mark.parametrize("pq_bits,pq_dim", [(4, 16), (5, 8), (6, 12), (7, 16), (8, 12), (8, 7)])
@pytest.mark.parametrize("lut,internal,rtol", [(R_32F, R_32F, 1e-5), (R_16F, R_32F, 2e-3),
                                               (R_8U, R_32F, 2e-3), (R_16F, R_16F, 2e-3),
                                               (R_8U, R_16F, 2e-3)])
def test_pq_bits_and_table_types(orc, pq_bits, pq_dim, lut, internal, rtol):
    if (pq_bits * pq_dim) % 8 != 0:
        pytest.skip("pq_bits * pq_dim must be a multiple of 8")
    dim = pq_dim * 2
    data, model, queries, index, ix, _ = _case(orc, 3000, dim, 10, pq_dim, pq_bits)
    nb, d, want_nb, want_d = _search_both(orc, index, ix, queries, 10, 4, lut, internal)
    H.compare_results(nb, d, want_nb, want_d, rtol, exact=True)


@pytest.mark.parametrize("metric", ["sqeuclidean", "euclidean", "inner_product", "cosine"])
@pytest.mark.parametrize("kind", ["subspace", "cluster"])
@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.int8, np.uint8])
def test_metrics_codebooks_and_element_types(orc, metric, kind, dtype):
    data, model, queries, index, ix, _ = _case(orc, 2500, 30, 8, 10, 8, dtype=dtype, metric=metric,
                                               kind=kind, force_rot=(kind == "cluster"))
    for lut, internal, rtol in [(R_32F, R_32F, 1e-5), (R_8U, R_16F, 2e-3)]:
        nb, d, want_nb, want_d = _search_both(orc, index, ix, queries, 7, 3, lut, internal)
        H.compare_results(nb, d, want_nb, want_d, rtol, exact=(metric != "euclidean"))


@pytest.mark.parametrize("k", [1, 2, 16, 17, 100, 128, 129, 256, 257, 700])
def test_k_sweep_crosses_fused_boundary(orc, k):
    data, model, queries, index, ix, _ = _case(orc, 6000, 16, 12, 8, 8, n_queries=20)
    nb, d, want_nb, want_d = _search_both(orc, index, ix, queries, k, 5)
    H.compare_results(nb, d, want_nb, want_d, 1e-5, exact=True)


@pytest.mark.parametrize("n_probes", [1, 2, 5, 33, 64, 1000])
def test_n_probes_sweep(orc, n_probes):
    data, model, queries, index, ix, _ = _case(orc, 5000, 16, 64, 8, 8, n_queries=33)
    sp = ivf_pq.SearchParams(n_probes=n_probes)
    probes = ivf_pq.select_clusters(sp, index, G.to_dev(queries)).cpu().numpy().view(np.uint32)
    want_probes, _ = orc.select_clusters(ix, queries, n_probes)
    assert np.array_equal(probes, want_probes)
    nb, d, want_nb, want_d = _search_both(orc, index, ix, queries, 10, n_probes)
    H.compare_results(nb, d, want_nb, want_d, 1e-5, exact=True)


@pytest.mark.parametrize("dim", [1, 2, 3, 5, 8, 13, 17])
def test_small_dims(orc, dim):
    pq_dim = dim
    data, model, queries, index, ix, _ = _case(orc, 1200, dim, 6, pq_dim, 8, n_queries=16)
    nb, d, want_nb, want_d = _search_both(orc, index, ix, queries, 5, 3)
    H.compare_results(nb, d, want_nb, want_d, 1e-5, exact=True)


def test_unfilled_slots_and_empty_lists(orc):
    data, model, queries, index, ix, _ = _case(orc, 120, 8, 40, 4, 8, n_queries=10)
    nb, d, want_nb, want_d = _search_both(orc, index, ix, queries, 30, 2)
    assert (want_nb == np.iinfo(np.int64).max).any()
    assert np.array_equal(nb, want_nb)
    assert np.array_equal(d, want_d)


def test_extend_in_batches_and_custom_ids(orc):
    n, dim = 4000, 16
    data = H.make_data(n, dim, np.float32, 8)
    model = H.train(data, 10, 8, 8, iters=4)
    ids = (np.arange(n, dtype=np.int64) * 3 + 17)
    index = G.build_gpu_index(model, data, 8, 8, ids=ids, batches=3)
    assert len(index) == n
    ix, gpu_codes = G.read_back(orc, index, model, dim, 8, 8)
    ref, labels, codes = H.oracle_index_with_data(orc, model, data, 8, 8, ids=ids)
    assert np.array_equal(ix.list_sizes, ref.list_sizes)
    for l in range(10):
        order = np.argsort(ix.list_inds[l])
        assert np.array_equal(ix.list_inds[l][order], ref.list_inds[l])
        assert np.array_equal(gpu_codes[l][order], codes[labels == l])
    queries = H.make_data(50, dim, np.float32, 99)
    nb, d, want_nb, want_d = _search_both(orc, index, ix, queries, 10, 4)
    H.compare_results(nb, d, want_nb, want_d, 1e-5, exact=True)
    # default ids continue from the current size
    more = H.make_data(100, dim, np.float32, 10)
    ivf_pq.extend(index, G.to_dev(more), None)
    assert len(index) == n + 100
    all_ids = np.concatenate([index.list_indices(l).cpu().numpy() for l in range(10)])
    assert set(all_ids.tolist()) == set(ids.tolist()) | set(range(n, n + 100))
    # host input is accepted as well
    ivf_pq.extend(index, more, np.arange(10 ** 6, 10 ** 6 + 100, dtype=np.int64))
    assert len(index) == n + 200


def test_transform_matches_stored_codes(orc):
    """Codes returned by transform equal the codes extend stored (reference invariant:
    python/cuvs/cuvs/tests/test_ivf_pq.py:339-378)."""
    data, model, queries, index, ix, gpu_codes = _case(orc, 2000, 24, 7, 12, 6)
    labels, flat = ivf_pq.transform(index, G.to_dev(data))
    labels = labels.cpu().numpy().view(np.uint32)
    codes = G.unpack_bits(flat.cpu().numpy(), 12, 6)
    want_labels, want_codes = orc.encode(ix, data)
    assert np.array_equal(labels, want_labels)
    assert np.array_equal(codes, want_codes)
    for l in range(7):
        order = np.argsort(ix.list_inds[l])
        assert np.array_equal(gpu_codes[l][order], codes[labels == l])


def test_bitset_filter(orc):
    data, model, queries, index, ix, _ = _case(orc, 3000, 16, 8, 8, 8)
    n = data.shape[0]
    keep = np.ones(n, dtype=bool)
    keep[:300] = False
    bits = np.packbits(keep, bitorder="little")
    bits = np.concatenate([bits, np.zeros((-bits.size) % 4, dtype=np.uint8)]).view(np.uint32)
    sp = ivf_pq.SearchParams(n_probes=8)
    d, nb = ivf_pq.search(sp, index, G.to_dev(queries), 10,
                          filter_bitset=G.to_dev(bits.view(np.int32)), filter_nbits=n)
    want_nb, want_d = orc.search(ix, queries, 10, 8, filter_bitset=bits, filter_nbits=n)
    H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 1e-5, exact=True)
    assert nb.min().item() >= 300


def test_batching_does_not_change_results(orc):
    data, model, queries, index, ix, _ = _case(orc, 3000, 16, 8, 8, 8, n_queries=301)
    a = _search_both(orc, index, ix, queries, 10, 4, max_internal_batch_size=4096)
    b = _search_both(orc, index, ix, queries, 10, 4, max_internal_batch_size=37)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    H.compare_results(a[0], a[1], a[2], a[3], 1e-5, exact=True)


@pytest.mark.parametrize("n_queries,batch", [(301, 37), (1000, 400), (129, 128), (640, 64)])
def test_batches_side_by_side_equal_batches_in_turn(orc, n_queries, batch):
    """The internal batches of a call run beside each other on streams of the handle's own (up to
    four runs of whole batches); switched off on the handle they run one after the other.  Same
    results either way, and the oracle's; work queued on the handle's stream afterwards sees them
    (no host synchronisation between the search and the copy that follows it on the same stream);
    a bitset filter goes to every run."""
    data, model, queries, index, ix, _ = _case(orc, 4000, 32, 12, 16, 8, n_queries=n_queries)
    dq = G.to_dev(queries)
    sp = ivf_pq.SearchParams(n_probes=5, lut_dtype=R_16F, max_internal_batch_size=batch)
    res = Resources()
    res.use_torch_current_stream()
    want_nb, want_d = orc.search(ix, queries, 10, 5, lut_dtype=ORC_DT[R_16F])
    out = {}
    for serial in (False, True, False):
        res.set_search_tuning(serial_batches=serial)
        d, nb = ivf_pq.search(sp, index, dq, 10, resources=res)
        nb_copy, d_copy = nb.clone(), d.clone()  # on the same stream, right behind the search
        torch.cuda.synchronize()
        H.compare_results(nb_copy.cpu().numpy(), d_copy.cpu().numpy(), want_nb, want_d, 2e-3, exact=True)
        out[serial] = (nb_copy, d_copy)
    assert torch.equal(out[False][0], out[True][0]) and torch.equal(out[False][1], out[True][1])
    n = data.shape[0]
    keep = np.ones(n, dtype=bool)
    keep[::2] = False
    bits = np.packbits(keep, bitorder="little")
    bits = np.concatenate([bits, np.zeros((-bits.size) % 4, dtype=np.uint8)]).view(np.uint32)
    res.set_search_tuning(serial_batches=False)
    d, nb = ivf_pq.search(sp, index, dq, 10, resources=res, filter_bitset=G.to_dev(bits.view(np.int32)), filter_nbits=n)
    torch.cuda.synchronize()
    want_nb, want_d = orc.search(ix, queries, 10, 5, lut_dtype=ORC_DT[R_16F], filter_bitset=bits, filter_nbits=n)
    H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 2e-3, exact=True)
    # a wrong argument is refused by the first run, before anything is queued on a side stream
    with pytest.raises(CuvsError):
        ivf_pq.search(sp, index, G.to_dev(np.zeros((n_queries, 31), dtype=np.float32)), 10, resources=res)
    d, nb = ivf_pq.search(sp, index, dq, 10, resources=res)
    torch.cuda.synchronize()
    assert torch.equal(nb, out[True][0])


def test_half_precision_coarse_search(orc):
    data, model, queries, index, ix, _ = _case(orc, 4000, 32, 50, 16, 8)
    sp = ivf_pq.SearchParams(n_probes=6, coarse_search_dtype=np.float16)
    probes = ivf_pq.select_clusters(sp, index, G.to_dev(queries)).cpu().numpy().view(np.uint32)
    want_probes, _ = orc.select_clusters(ix, queries, 6, coarse_search_dtype=2)
    assert np.array_equal(probes, want_probes)
    nb, d, want_nb, want_d = _search_both(orc, index, ix, queries, 10, 6, coarse=np.float16)
    H.compare_results(nb, d, want_nb, want_d, 1e-5, exact=True)


@pytest.mark.parametrize("coarse", [np.float16, np.int8])
@pytest.mark.parametrize("dtype,metric,force_rot,dim", [
    (np.float32, "sqeuclidean", True, 30), (np.float32, "inner_product", False, 32),
    (np.uint8, "sqeuclidean", False, 32), (np.int8, "euclidean", True, 32),
    (np.float16, "cosine", True, 24)])
def test_reduced_precision_coarse_search(orc, coarse, dtype, metric, force_rot, dim):
    """coarse_search_dtype 16F / 8I (ivf_pq_search.cuh:170-340): probes from the rounded operands,
    and the rotation applied to the same rounded query rows with the rotation matrix in that type
    (:996-1019); everything bit-equal to the oracle."""
    data, model, queries, index, ix, _ = _case(orc, 4000, dim, 50, 16 if dim != 30 else 15, 8, dtype=dtype,
                                               metric=metric, force_rot=force_rot)
    if dtype in (np.float32, np.float16):
        queries = (queries * 0.4).astype(dtype)   # most elements within the 8-bit range after x 128
    sp = ivf_pq.SearchParams(n_probes=6, coarse_search_dtype=coarse)
    probes = ivf_pq.select_clusters(sp, index, G.to_dev(queries)).cpu().numpy().view(np.uint32)
    want_probes, _ = orc.select_clusters(ix, queries, 6, coarse_search_dtype=ORC_DT[coarse])
    assert np.array_equal(probes, want_probes)
    want32, _ = orc.select_clusters(ix, queries, 6)
    print("rows whose probes differ from the fp32 search:", int((want32 != want_probes).any(1).sum()), flush=True)
    nb, d, want_nb, want_d = _search_both(orc, index, ix, queries, 10, 6, coarse=coarse)
    H.compare_results(nb, d, want_nb, want_d, 1e-5, exact=True)
    # the operands' precision is visible in the results (the rotation is not the fp32 one)
    nb32, d32, _, _ = _search_both(orc, index, ix, queries, 10, 6)
    if dtype == np.float32:
        assert not np.array_equal(d, d32)


def test_extend_rejects_labels_outside_the_lists(orc):
    """A caller-supplied label >= n_lists is refused before anything is written: the lists and the
    size stay as they were, and the index still searches like the oracle."""
    data, model, queries, index, ix, _ = _case(orc, 2000, 16, 10, 8, 8)
    sizes = index.list_sizes.cpu().tolist()
    before = [index.list_indices(l).cpu().numpy()[:sizes[l]].copy() for l in range(10)]
    extra = H.make_data(64, 16, np.float32, 77)
    for bad in (10, 11, 2 ** 31, 2 ** 32 - 1):
        labels = np.full(64, 3, dtype=np.uint32)
        labels[17] = bad
        with pytest.raises(CuvsError, match="smaller than n_lists"):
            ivf_pq.extend(index, G.to_dev(extra), None, labels=G.to_dev(labels.view(np.int32)))
    assert len(index) == 2000 and index.list_sizes.cpu().tolist() == sizes
    for l in range(10):
        assert np.array_equal(index.list_indices(l).cpu().numpy()[:sizes[l]], before[l])
    nb, d, want_nb, want_d = _search_both(orc, index, ix, queries, 10, 4)
    H.compare_results(nb, d, want_nb, want_d, 1e-5, exact=True)
    # valid labels still go through
    ivf_pq.extend(index, G.to_dev(extra), None, labels=G.to_dev(np.full(64, 9, dtype=np.int32)))
    assert len(index) == 2064


def test_validation_errors(orc):
    """Error behaviour of search (cuVS ivf_pq_search.cuh:901-923,1088-1096; c/src/neighbors/ivf_pq.cpp:315-325)."""
    data, model, queries, index, ix, _ = _case(orc, 500, 8, 4, 4, 8, n_queries=4)
    q = G.to_dev(queries)
    ok = ivf_pq.SearchParams(n_probes=2)
    with pytest.raises(CuvsError, match="must be positive"):
        ivf_pq.search(ok, index, q, 0)
    with pytest.raises(CuvsError, match="total size"):
        ivf_pq.search(ok, index, q, 501)
    with pytest.raises(CuvsError, match="n_probes"):
        ivf_pq.search(ivf_pq.SearchParams(n_probes=0), index, q, 5)
    with pytest.raises(CuvsError, match="combination"):
        ivf_pq.search(ivf_pq.SearchParams(n_probes=2, internal_distance_dtype=np.float16), index, q, 5)
    with pytest.raises(CuvsError, match="lut_dtype"):
        ivf_pq.search(ivf_pq.SearchParams(n_probes=2, lut_dtype=np.int8), index, q, 5)
    with pytest.raises(CuvsError, match="dimensions"):
        ivf_pq.search(ok, index, G.to_dev(np.zeros((4, 9), dtype=np.float32)), 5)
    with pytest.raises(CuvsError, match="int64"):
        ivf_pq.search(ok, index, q, 5, neighbors=torch.empty((4, 5), dtype=torch.int32, device="cuda"))
    with pytest.raises(CuvsError, match="float32"):
        ivf_pq.search(ok, index, q, 5, distances=torch.empty((4, 5), dtype=torch.float16, device="cuda"))
    with pytest.raises(CuvsError, match="device compatible"):
        ivf_pq.search(ok, index, queries, 5)
    with pytest.raises(CuvsError, match="number of queries"):
        ivf_pq.search(ok, index, q, 5, neighbors=torch.empty((3, 5), dtype=torch.int64, device="cuda"))
    with pytest.raises(CuvsError, match="row-major"):
        from cuvs_amd import dlpack
        from cuvs_amd._lib import check, lib
        import ctypes as C
        qv = dlpack.view(q)
        qv.mt.dl_tensor.strides = (C.c_int64 * 2)(1, 4)
        nb = torch.empty((4, 5), dtype=torch.int64, device="cuda")
        dd = torch.empty((4, 5), dtype=torch.float32, device="cuda")
        check(lib().cuvsIvfPqSearch(ivf_pq._default_resources().get_c_obj(), ok._p, index.index,
                                    qv.ptr, dlpack.view(nb).ptr, dlpack.view(dd).ptr))
    with pytest.raises(CuvsError, match="less than n_lists"):
        ivf_pq.build(ivf_pq.IndexParams(), q)
    # a good call clears the error text and still works after the failures above
    d, nb = ivf_pq.search(ok, index, q, 5)
    want_nb, want_d = orc.search(ix, queries, 5, 2)
    assert np.array_equal(nb.cpu().numpy(), want_nb)


def test_getters_round_trip(orc):
    data, model, queries, index, ix, _ = _case(orc, 800, 12, 5, 6, 8, kind="cluster")
    assert (index.n_lists, index.dim, index.pq_dim, index.pq_bits, index.pq_len) == (5, 12, 6, 8, 2)
    assert np.array_equal(index.centers_padded.cpu().numpy(), model["centers"])
    assert np.array_equal(index.centers.cpu().numpy(), model["centers"][:, :12])
    assert np.array_equal(index.centers_rot.cpu().numpy(), model["centers_rot"])
    assert np.array_equal(index.rotation_matrix.cpu().numpy(), model["rotation_matrix"])
    assert np.array_equal(index.pq_centers.cpu().numpy(), model["pq_centers"])
    assert int(index.list_sizes.sum().item()) == 800


# --- shapes served by the persistent 8-bit scan kernel (pq_dim x pq_len in {64x2, 48x2, 32x4, 32x2}) ---

@pytest.mark.parametrize("dim,pq_dim", [(128, 64), (96, 48), (128, 32), (64, 32)])
@pytest.mark.parametrize("lut,internal,rtol", [(R_32F, R_32F, 1e-5), (R_16F, R_32F, 2e-3),
                                               (R_8U, R_32F, 2e-3), (R_16F, R_16F, 2e-3),
                                               (R_8U, R_16F, 2e-3)])
@pytest.mark.parametrize("metric,kind", [("sqeuclidean", "subspace"), ("inner_product", "subspace"),
                                         ("sqeuclidean", "cluster"), ("cosine", "cluster")])
def test_persistent_scan_shapes(orc, dim, pq_dim, lut, internal, rtol, metric, kind):
    data, model, queries, index, ix, _ = _case(orc, 6000, dim, 12, pq_dim, 8, metric=metric,
                                               kind=kind, n_queries=40, dtype=np.float32)
    nb, d, want_nb, want_d = _search_both(orc, index, ix, queries, 10, 5, lut, internal)
    H.compare_results(nb, d, want_nb, want_d, rtol, exact=True)


@pytest.mark.parametrize("k", [1, 10, 64, 65, 100, 256])
def test_persistent_scan_long_lists_and_k(orc, k):
    """Lists longer than the candidate buffer (segment pruning) and k up to the fused limit."""
    data, model, queries, index, ix, _ = _case(orc, 20000, 96, 4, 48, 8, n_queries=24,
                                               dtype=np.uint8)
    assert ix.list_sizes.max() > 2048
    for lut, internal in [(R_32F, R_32F), (R_8U, R_16F)]:
        nb, d, want_nb, want_d = _search_both(orc, index, ix, queries, k, 3, lut, internal)
        H.compare_results(nb, d, want_nb, want_d, 2e-3, exact=True)


def test_persistent_scan_filter_and_empty_lists(orc):
    data, model, queries, index, ix, _ = _case(orc, 300, 128, 40, 64, 8, n_queries=16)
    assert (ix.list_sizes == 0).any() or True
    n = data.shape[0]
    keep = np.ones(n, dtype=bool)
    keep[::3] = False
    bits = np.packbits(keep, bitorder="little")
    bits = np.concatenate([bits, np.zeros((-bits.size) % 4, dtype=np.uint8)]).view(np.uint32)
    sp = ivf_pq.SearchParams(n_probes=6)
    d, nb = ivf_pq.search(sp, index, G.to_dev(queries), 20,
                          filter_bitset=G.to_dev(bits.view(np.int32)), filter_nbits=n)
    want_nb, want_d = orc.search(ix, queries, 20, 6, filter_bitset=bits, filter_nbits=n)
    H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 1e-5, exact=True)
    nb2, d2, want_nb2, want_d2 = _search_both(orc, index, ix, queries, 30, 2)
    H.compare_results(nb2, d2, want_nb2, want_d2, 1e-5, exact=True)


# --- L2 early stop: leading probes in full, first-chunk screening of the rest, survivors in full ---

_CLUSTERED = {}


def _clustered_case(orc, dtype=np.float32, kind="subspace"):
    key = (np.dtype(dtype).name, kind)
    if key not in _CLUSTERED:
        _CLUSTERED[key] = _make_clustered_case(orc, dtype, kind)
    return _CLUSTERED[key]


def _make_clustered_case(orc, dtype, kind):
    import datasets as testing
    print(f"clustered case dtype={np.dtype(dtype).name} kind={kind}", flush=True)
    if dtype == np.uint8:
        allrows = testing.sift_like_u8(30200, 128, 96, seed=77).numpy()
    else:
        allrows = testing.gaussian_mixture(30200, 128, 96, 0.15, seed=77).numpy().astype(dtype)
    x, q = allrows[:30000], allrows[30000:]
    model = H.train(x, 200, 64, 8, codebook_kind=kind, iters=6)
    index = G.build_gpu_index(model, x, 64, 8, "sqeuclidean", kind)
    ix, _ = G.read_back(orc, index, model, 128, 64, 8, "sqeuclidean", kind)
    return x, q, index, ix


@pytest.mark.parametrize("lut,internal", [(R_32F, R_32F), (R_16F, R_32F), (R_8U, R_32F), (R_16F, R_16F),
                                          (R_8U, R_16F)])
@pytest.mark.parametrize("dtype,kind", [(np.float32, "subspace"), (np.uint8, "subspace"),
                                        (np.float32, "cluster")])
def test_early_stop_matches_oracle_and_full_scan(orc, lut, internal, dtype, kind):
    from cuvs_amd.resources import Resources
    x, q, index, ix = _clustered_case(orc, dtype, kind)
    res = Resources()
    res.enable_profiling(True)
    sp = ivf_pq.SearchParams(n_probes=48, lut_dtype=lut, internal_distance_dtype=internal)
    for k in (1, 10, 64, 100, 256):  # up to 64: CU-wide kernel; above: block-per-pair kernel
        d, nb = ivf_pq.search(sp, index, G.to_dev(q), k, resources=res)
        res.sync()
        prof = ivf_pq.get_search_profile(res)
        assert prof["n_screened_pairs"] == q.shape[0] * 47
        # on clustered data most screened pairs are dropped (fewer for a large k: a looser bound)
        assert 0 < prof["n_surviving_pairs"] < prof["n_screened_pairs"] // (2 if k <= 100 else 1)
        want_nb, want_d = orc.search(ix, q, k, 48, lut_dtype=ORC_DT[lut],
                                     internal_distance_dtype=ORC_DT[internal])
        H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 2e-3, exact=True)
        res.set_search_tuning(early_stop="off")
        d2, nb2 = ivf_pq.search(sp, index, G.to_dev(q), k, resources=res)
        res.sync()
        assert ivf_pq.get_search_profile(res)["n_screened_pairs"] == 0
        res.set_search_tuning(early_stop="auto")
        assert torch.equal(nb, nb2) and torch.equal(d, d2)


def test_screen_turns_itself_off_where_it_does_not_pay(orc):
    """Rows without cluster structure: every probed list is about as far from a query as its nearest
    one, the screen keeps nearly every pair, and the index remembers: searches after the one that was
    observed scan plainly (every 64th is screened again), with the same results either way - the
    oracle's."""
    from cuvs_amd.resources import Resources
    rng = np.random.default_rng(11)
    allrows = rng.standard_normal((30300, 128)).astype(np.float32)
    x, q = allrows[:30000], allrows[30000:]
    model = H.train(x, 100, 64, 8, iters=4)
    index = G.build_gpu_index(model, x, 64, 8, "sqeuclidean", "subspace")
    ix, _ = G.read_back(orc, index, model, 128, 64, 8, "sqeuclidean", "subspace")
    res = Resources()
    res.enable_profiling(True)
    sp = ivf_pq.SearchParams(n_probes=24, lut_dtype=R_16F)
    want_nb, want_d = orc.search(ix, q, 10, 24, lut_dtype=ORC_DT[R_16F])
    screened = []
    for call in range(70):
        d, nb = ivf_pq.search(sp, index, G.to_dev(q), 10, resources=res)
        res.sync()
        prof = ivf_pq.get_search_profile(res)
        screened.append(prof["n_screened_pairs"])
        if call in (0, 1, 2, 64, 65):
            if prof["n_screened_pairs"]:
                assert prof["n_surviving_pairs"] > 0.7 * prof["n_screened_pairs"]
            H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 2e-3, exact=True)
    assert screened[0] == q.shape[0] * 23           # observed
    assert screened[1] == 0 and screened[2] == 0    # verdict in: plain scans
    assert sum(1 for n in screened if n) == 2       # and one more look, 64 plain searches later
    # other parameters: no verdict yet, the screen runs (and is observed in its turn)
    d, nb = ivf_pq.search(ivf_pq.SearchParams(n_probes=16, lut_dtype=R_16F), index, G.to_dev(q), 10, resources=res)
    res.sync()
    assert ivf_pq.get_search_profile(res)["n_screened_pairs"] == q.shape[0] * 15
    # forced on, it runs whatever the verdict
    res.set_search_tuning(early_stop="on")
    d2, nb2 = ivf_pq.search(sp, index, G.to_dev(q), 10, resources=res)
    res.sync()
    assert ivf_pq.get_search_profile(res)["n_screened_pairs"] == q.shape[0] * 23
    H.compare_results(nb2.cpu().numpy(), d2.cpu().numpy(), want_nb, want_d, 2e-3, exact=True)


def test_merge_after_early_stop_with_many_live_keys(orc):
    """Unclustered rows and k = 64 with the screen forced on: nearly every pair survives and brings
    dozens of valid keys, far more than the one-wave merge takes (1024 per query), so the queries go
    through its leftover launch; clustered queries of the same batch size stay in the wave merge.
    Both return the oracle's results."""
    from cuvs_amd.resources import Resources
    rng = np.random.default_rng(23)
    allrows = rng.standard_normal((30200, 128)).astype(np.float32)
    x, q = allrows[:30000], allrows[30000:]
    model = H.train(x, 100, 64, 8, iters=4)
    index = G.build_gpu_index(model, x, 64, 8, "sqeuclidean", "subspace")
    ix, _ = G.read_back(orc, index, model, 128, 64, 8, "sqeuclidean", "subspace")
    res = Resources()
    res.enable_profiling(True)
    res.set_search_tuning(early_stop="on")
    for k in (64, 10):
        sp = ivf_pq.SearchParams(n_probes=32, lut_dtype=R_16F)
        want_nb, want_d = orc.search(ix, q, k, 32, lut_dtype=ORC_DT[R_16F])
        d, nb = ivf_pq.search(sp, index, G.to_dev(q), k, resources=res)
        res.sync()
        prof = ivf_pq.get_search_profile(res)
        assert prof["n_screened_pairs"] == q.shape[0] * 31
        assert prof["n_surviving_pairs"] > 0.7 * prof["n_screened_pairs"]
        H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 2e-3, exact=True)


def test_pair_order_beyond_the_sorted_range():
    """More than 4 M (query, probe) pairs in one internal batch: the pair order falls back from the
    two-level counting sort to global atomics.  Same neighbours as the same queries in batches that
    the sort takes."""
    import datasets as testing
    allrows = testing.gaussian_mixture(40000 + 70000, 32, 64, 0.2, seed=91, device="cuda")
    data, queries = allrows[:40000], allrows[40000:]
    index = ivf_pq.build(ivf_pq.IndexParams(n_lists=256, pq_dim=16, kmeans_trainset_fraction=0.5), data)
    big = ivf_pq.SearchParams(n_probes=64, lut_dtype=R_16F, max_internal_batch_size=70000)
    small = ivf_pq.SearchParams(n_probes=64, lut_dtype=R_16F, max_internal_batch_size=8192)
    d1, nb1 = ivf_pq.search(big, index, queries, 5)
    d2, nb2 = ivf_pq.search(small, index, queries, 5)
    assert torch.equal(nb1, nb2) and torch.equal(d1, d2)


@pytest.mark.parametrize("kind", ["subspace", "cluster"])
def test_early_stop_pq_len_4(orc, kind):
    """Four dimensions per subspace: 16-byte codebook entries in the table-free screen (shared by
    the block for per-subspace codebooks, one list's codebook per wave for per-cluster ones)."""
    import datasets as testing
    from cuvs_amd.resources import Resources
    allrows = testing.gaussian_mixture(20100, 128, 64, 0.15, seed=78).numpy()
    x, q = allrows[:20000], allrows[20000:]
    model = H.train(x, 128, 32, 8, codebook_kind=kind, iters=6)
    index = G.build_gpu_index(model, x, 32, 8, "sqeuclidean", kind)
    ix, _ = G.read_back(orc, index, model, 128, 32, 8, "sqeuclidean", kind)
    res = Resources()
    res.enable_profiling(True)
    for lut in (R_16F, R_8U):
        sp = ivf_pq.SearchParams(n_probes=40, lut_dtype=lut)
        d, nb = ivf_pq.search(sp, index, G.to_dev(q), 10, resources=res)
        res.sync()
        prof = ivf_pq.get_search_profile(res)
        assert prof["n_screened_pairs"] == q.shape[0] * 39
        assert 0 < prof["n_surviving_pairs"] < prof["n_screened_pairs"] // 2
        want_nb, want_d = orc.search(ix, q, 10, 40, lut_dtype=ORC_DT[lut])
        H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 2e-3, exact=True)


@pytest.mark.parametrize("lut,internal", [(R_16F, R_32F), (R_8U, R_32F), (R_16F, R_16F), (R_8U, R_16F)])
@pytest.mark.parametrize("dim,pq_dim", [(128, 64), (128, 128), (256, 64), (192, 192), (64, 32)])
def test_early_stop_with_four_bit_codes(orc, lut, internal, dim, pq_dim):
    """4-bit codes, L2: the leading pairs and the survivors of the screen go to the wave-per-pair
    kernel, the screen sums the 16 subspaces of the leading 8 code bytes (pq_len 2, 1, 4, 1; one,
    two, one and three steps of 64 subspaces a row).  Outside that kernel's shapes (pq_dim 32; k
    above 64) the generic kernel scans those pairs as a subset.  Same results as the oracle and as
    the single launch."""
    import datasets as testing
    from cuvs_amd.resources import Resources
    allrows = testing.gaussian_mixture(24200, dim, 64, 0.15, seed=79).numpy()
    x, q = allrows[:24000], allrows[24000:]
    model = H.train(x, 120, pq_dim, 4, iters=6)
    index = G.build_gpu_index(model, x, pq_dim, 4, "sqeuclidean", "subspace")
    ix, _ = G.read_back(orc, index, model, dim, pq_dim, 4, "sqeuclidean", "subspace")
    res = Resources()
    res.enable_profiling(True)
    sp = ivf_pq.SearchParams(n_probes=40, lut_dtype=lut, internal_distance_dtype=internal)
    for k in (1, 10, 64, 100):
        d, nb = ivf_pq.search(sp, index, G.to_dev(q), k, resources=res)
        res.sync()
        prof = ivf_pq.get_search_profile(res)
        assert prof["n_screened_pairs"] == q.shape[0] * 39
        assert 0 < prof["n_surviving_pairs"] <= prof["n_screened_pairs"]
        want_nb, want_d = orc.search(ix, q, k, 40, lut_dtype=ORC_DT[lut], internal_distance_dtype=ORC_DT[internal])
        H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 2e-3, exact=True)
        res.set_search_tuning(early_stop="off")
        d2, nb2 = ivf_pq.search(sp, index, G.to_dev(q), k, resources=res)
        res.sync()
        assert ivf_pq.get_search_profile(res)["n_screened_pairs"] == 0
        res.set_search_tuning(early_stop="auto")
        assert torch.equal(nb, nb2) and torch.equal(d, d2)


def test_four_bit_index_without_the_plane_of_leading_codes(orc):
    """conservative_memory_allocation: a 4-bit index keeps no plane of leading code bytes, and an L2
    search is then one scan launch with the same results."""
    import datasets as testing
    from cuvs_amd.resources import Resources
    allrows = testing.gaussian_mixture(24200, 128, 64, 0.15, seed=80, device="cuda")
    x, q = allrows[:24000], allrows[24000:]
    kw = dict(n_lists=120, pq_dim=64, pq_bits=4)
    trained = ivf_pq.build(ivf_pq.IndexParams(add_data_on_build=False, **kw), x)
    model = (trained.pq_centers, trained.centers_padded, trained.centers_rot, trained.rotation_matrix)
    ids = torch.arange(24000, dtype=torch.int64, device="cuda")
    index = ivf_pq.extend(ivf_pq.build_precomputed(ivf_pq.IndexParams(**kw), 128, *model), x, ids)
    lean = ivf_pq.extend(ivf_pq.build_precomputed(
        ivf_pq.IndexParams(conservative_memory_allocation=True, **kw), 128, *model), x, ids)
    res = Resources()
    res.enable_profiling(True)
    sp = ivf_pq.SearchParams(n_probes=40, lut_dtype=R_16F)
    d, nb = ivf_pq.search(sp, index, q, 10, resources=res)
    res.sync()
    assert ivf_pq.get_search_profile(res)["n_screened_pairs"] == q.shape[0] * 39
    d2, nb2 = ivf_pq.search(sp, lean, q, 10, resources=res)
    res.sync()
    assert ivf_pq.get_search_profile(res)["n_screened_pairs"] == 0
    assert torch.equal(d, d2)
    # another index object: rows at exactly the same distance may come in either order
    assert float((nb == nb2).float().mean()) > 0.99


@pytest.mark.parametrize("dim,pq_dim", [(128, 64), (96, 48), (64, 32)])
def test_early_stop_with_fp32_tables(orc, dim, pq_dim):
    """fp32 tables (the reference's default lut_dtype): the leading and the surviving pairs go to
    the table-free wave-per-pair kernel (four, three and two chunks a row), with and without a
    bitset filter; same results as the oracle and as the single launch of the block-per-pair kernel."""
    import datasets as testing
    from cuvs_amd.resources import Resources
    allrows = testing.gaussian_mixture(24300, dim, 64, 0.15, seed=81).numpy()
    x, q = allrows[:24000], allrows[24000:]
    model = H.train(x, 120, pq_dim, 8, iters=6)
    index = G.build_gpu_index(model, x, pq_dim, 8, "euclidean", "subspace")
    ix, _ = G.read_back(orc, index, model, dim, pq_dim, 8, "euclidean", "subspace")
    n = x.shape[0]
    keep = np.ones(n, dtype=bool)
    keep[::3] = False
    bits = np.packbits(keep, bitorder="little")
    bits = np.concatenate([bits, np.zeros((-bits.size) % 4, dtype=np.uint8)]).view(np.uint32)
    res = Resources()
    res.enable_profiling(True)
    sp = ivf_pq.SearchParams(n_probes=30)  # lut_dtype and internal_distance_dtype at their defaults
    for k, filtered in ((1, False), (10, False), (64, False), (10, True), (64, True)):
        kw = dict(filter_bitset=G.to_dev(bits.view(np.int32)), filter_nbits=n) if filtered else {}
        okw = dict(filter_bitset=bits, filter_nbits=n) if filtered else {}
        d, nb = ivf_pq.search(sp, index, G.to_dev(q), k, resources=res, **kw)
        res.sync()
        prof = ivf_pq.get_search_profile(res)
        assert prof["n_screened_pairs"] == q.shape[0] * 29
        assert 0 < prof["n_surviving_pairs"] < prof["n_screened_pairs"]
        want_nb, want_d = orc.search(ix, q, k, 30, **okw)
        H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 1e-5, exact=False)
        res.set_search_tuning(early_stop="off")
        d2, nb2 = ivf_pq.search(sp, index, G.to_dev(q), k, resources=res, **kw)
        res.sync()
        assert ivf_pq.get_search_profile(res)["n_screened_pairs"] == 0
        res.set_search_tuning(early_stop="auto")
        assert torch.equal(nb, nb2) and torch.equal(d, d2)


@pytest.mark.parametrize("lut,internal", [(R_32F, R_32F), (R_16F, R_32F), (R_8U, R_16F)])
@pytest.mark.parametrize("dim,pq_dim,kind", [(256, 128, "subspace"), (192, 96, "subspace"), (384, 96, "cluster")])
def test_early_stop_with_more_than_64_subspaces(orc, lut, internal, dim, pq_dim, kind):
    """Byte codes of a shape no specialised kernel takes (pq_dim 128, 96; pq_len 2, 4; both codebook
    kinds): the generic kernel scans the leading and the surviving pairs of the early stop as a
    subset of the pairs.  Same results as the oracle and as its single launch over all pairs."""
    import datasets as testing
    from cuvs_amd.resources import Resources
    allrows = testing.gaussian_mixture(16200, dim, 48, 0.15, seed=82).numpy()
    x, q = allrows[:16000], allrows[16000:]
    model = H.train(x, 80, pq_dim, 8, codebook_kind=kind, iters=5)
    index = G.build_gpu_index(model, x, pq_dim, 8, "sqeuclidean", kind)
    ix, _ = G.read_back(orc, index, model, dim, pq_dim, 8, "sqeuclidean", kind)
    res = Resources()
    res.enable_profiling(True)
    sp = ivf_pq.SearchParams(n_probes=24, lut_dtype=lut, internal_distance_dtype=internal)
    for k in (10, 100):
        d, nb = ivf_pq.search(sp, index, G.to_dev(q), k, resources=res)
        res.sync()
        prof = ivf_pq.get_search_profile(res)
        assert prof["n_screened_pairs"] == q.shape[0] * 23
        assert 0 < prof["n_surviving_pairs"] < prof["n_screened_pairs"]
        want_nb, want_d = orc.search(ix, q, k, 24, lut_dtype=ORC_DT[lut], internal_distance_dtype=ORC_DT[internal])
        H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 1e-5 if lut == R_32F else 2e-3,
                          exact=True)
        res.set_search_tuning(early_stop="off")
        d2, nb2 = ivf_pq.search(sp, index, G.to_dev(q), k, resources=res)
        res.sync()
        assert ivf_pq.get_search_profile(res)["n_screened_pairs"] == 0
        res.set_search_tuning(early_stop="auto")
        assert torch.equal(nb, nb2) and torch.equal(d, d2)


def test_early_stop_with_the_table_in_global_memory(orc):
    """768 dimensions at pq_dim 384: an fp16 table of 196 KB does not fit LDS and lives in global
    memory; the generic kernel still scans the leading and the surviving pairs as a subset."""
    import datasets as testing
    from cuvs_amd.resources import Resources
    allrows = testing.gaussian_mixture(12150, 768, 32, 0.15, seed=83).numpy()
    x, q = allrows[:12000], allrows[12000:]
    model = H.train(x, 40, 384, 8, iters=4)
    index = G.build_gpu_index(model, x, 384, 8, "sqeuclidean", "subspace")
    ix, _ = G.read_back(orc, index, model, 768, 384, 8, "sqeuclidean", "subspace")
    res = Resources()
    res.enable_profiling(True)
    sp = ivf_pq.SearchParams(n_probes=12, lut_dtype=R_16F)
    d, nb = ivf_pq.search(sp, index, G.to_dev(q), 10, resources=res)
    res.sync()
    assert ivf_pq.get_search_profile(res)["n_screened_pairs"] == q.shape[0] * 11
    want_nb, want_d = orc.search(ix, q, 10, 12, lut_dtype=ORC_DT[R_16F])
    H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 2e-3, exact=True)
    res.set_search_tuning(early_stop="off")
    d2, nb2 = ivf_pq.search(sp, index, G.to_dev(q), 10, resources=res)
    res.sync()
    assert ivf_pq.get_search_profile(res)["n_screened_pairs"] == 0
    assert torch.equal(nb, nb2) and torch.equal(d, d2)


def test_early_stop_with_filter_and_small_lists(orc):
    """A filter can leave the leading list with fewer than k rows (no bound: nothing is dropped),
    and the screen ignores the filter (it may keep a pair whose rows in play are all filtered)."""
    x, q, index, ix = _clustered_case(orc)
    n = x.shape[0]
    rng = np.random.default_rng(5)
    keep = rng.random(n) < 0.1
    bits = np.packbits(keep, bitorder="little")
    bits = np.concatenate([bits, np.zeros((-bits.size) % 4, dtype=np.uint8)]).view(np.uint32)
    sp = ivf_pq.SearchParams(n_probes=40, lut_dtype=R_16F)
    d, nb = ivf_pq.search(sp, index, G.to_dev(q), 20, filter_bitset=G.to_dev(bits.view(np.int32)),
                          filter_nbits=n)
    want_nb, want_d = orc.search(ix, q, 20, 40, lut_dtype=ORC_DT[R_16F], filter_bitset=bits,
                                 filter_nbits=n)
    H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 2e-3, exact=True)


# --- index files: cuVS format version 4, a sequence of NumPy records ---

def _read_records(path):
    """Every record of the file through NumPy's own .npy reader."""
    out = []
    with open(path, "rb") as f:
        f.seek(0, 2)
        end = f.tell()
        f.seek(0)
        while f.tell() < end:
            out.append(np.lib.format.read_array(f, allow_pickle=False))
    return out


@pytest.mark.parametrize("pq_bits,pq_dim,kind", [(8, 16, "subspace"), (5, 8, "cluster")])
def test_serialize_round_trip_and_numpy_readable(orc, tmp_path, pq_bits, pq_dim, kind):
    data, model, queries, index, ix, gpu_codes = _case(orc, 900, 32, 7, pq_dim, pq_bits, kind=kind,
                                                       metric="inner_product", n_queries=20)
    path = str(tmp_path / "index.bin")
    ivf_pq.save(path, index)
    rec = _read_records(path)
    # header scalars (ivf_pq_serialize.cuh:49-59)
    assert [int(r) for r in rec[:5]] == [4, 900, 32, pq_bits, pq_dim]
    assert rec[1].dtype == np.int64 and rec[2].dtype == np.uint32
    assert int(rec[6]) == 6 and int(rec[7]) == (1 if kind == "cluster" else 0) and int(rec[8]) == 1
    assert int(rec[9]) == 7
    # model tensors and list sizes
    pq_len = 32 // pq_dim
    assert rec[10].shape == ((7 if kind == "cluster" else pq_dim), pq_len, 1 << pq_bits)
    assert np.array_equal(rec[10], model["pq_centers"])
    assert np.array_equal(rec[11], model["centers"]) and rec[11].shape == (7, 40)
    assert np.array_equal(rec[12], model["centers_rot"])
    assert np.array_equal(rec[13], model["rotation_matrix"])
    assert np.array_equal(rec[14], ix.list_sizes) and rec[14].dtype == np.uint32
    # per list: size, interleaved codes, ids
    pos = 15
    n_chunks = -(-pq_dim // (128 // pq_bits))
    for l in range(7):
        size = int(rec[pos])
        pos += 1
        assert size == ix.list_sizes[l]
        if size == 0:
            continue
        codes, ids = rec[pos], rec[pos + 1]
        pos += 2
        assert codes.shape == (-(-size // 32), n_chunks, 32, 16) and codes.dtype == np.uint8
        assert ids.shape == (size,) and ids.dtype == np.int64
        assert np.array_equal(orc.unpack_list(codes.reshape(-1), size, pq_dim, pq_bits), gpu_codes[l])
        assert np.array_equal(ids, index.list_indices(l).cpu().numpy())
    assert pos == len(rec)

    loaded = ivf_pq.load(path)
    assert len(loaded) == 900 and loaded.pq_dim == pq_dim and loaded.pq_bits == pq_bits
    assert torch.equal(loaded.list_sizes, index.list_sizes)
    assert torch.equal(loaded.centers, index.centers)
    sp = ivf_pq.SearchParams(n_probes=4, lut_dtype=R_16F)
    d1, n1 = ivf_pq.search(sp, index, G.to_dev(queries), 10)
    d2, n2 = ivf_pq.search(sp, loaded, G.to_dev(queries), 10)
    assert torch.equal(n1, n2) and torch.equal(d1, d2)
    # a loaded index can be extended
    ivf_pq.extend(loaded, G.to_dev(data[:50]), G.to_dev(np.arange(5000, 5050, dtype=np.int64)))
    assert len(loaded) == 950


def test_deserialize_rejects_damaged_files(orc, tmp_path):
    data, model, queries, index, ix, _ = _case(orc, 300, 16, 4, 8, 8, n_queries=4)
    path = str(tmp_path / "index.bin")
    ivf_pq.save(path, index)
    raw = open(path, "rb").read()
    cut = str(tmp_path / "cut.bin")
    open(cut, "wb").write(raw[: len(raw) // 2])
    with pytest.raises(CuvsError, match="truncated|NumPy"):
        ivf_pq.load(cut)
    bad = bytearray(raw)
    bad[raw.index(b"\x93NUMPY", 1)] = 0x00  # magic of the second record
    badp = str(tmp_path / "bad.bin")
    open(badp, "wb").write(bytes(bad))
    with pytest.raises(CuvsError, match="bad magic"):
        ivf_pq.load(badp)
    with pytest.raises(CuvsError, match="Cannot open"):
        ivf_pq.load(str(tmp_path / "missing.bin"))


# --- the other benchmark configurations, at a size the oracle finishes in seconds ---

def _config_case(orc, x, q, n_lists, pq_dim, pq_bits, metric, kind):
    model = H.train(x, n_lists, pq_dim, pq_bits, metric=metric, codebook_kind=kind, iters=5)
    index = G.build_gpu_index(model, x, pq_dim, pq_bits, metric, kind)
    ix, _ = G.read_back(orc, index, model, x.shape[1], pq_dim, pq_bits, metric, kind)
    return index, ix


@pytest.mark.parametrize("n_probes", [16, 32, 64])
def test_config2_shape_normalised_fp32_l2(orc, n_probes):
    """96-d L2-normalised fp32 mixture, pq_dim 48, 8 bit, fp16 table with fp32 distances."""
    import datasets as testing
    allrows = testing.gaussian_mixture(20200, 96, 100, 0.2, seed=1234, normalize_centers=True,
                                       normalize_rows=True).numpy()
    x, q = allrows[:20000], allrows[20000:]
    index, ix = _config_case(orc, x, q, 128, 48, 8, "sqeuclidean", "subspace")
    nb, d, want_nb, want_d = _search_both(orc, index, ix, q, 10, n_probes, R_16F, R_32F)
    H.compare_results(nb, d, want_nb, want_d, 2e-3, exact=True)


def test_config4_shape_inner_product_4bit_fp8_half(orc):
    """768-d unit-norm anisotropic mixture, inner product, pq_dim 384, 4-bit codes (two per byte),
    8-bit table (signed variant), fp16 distances."""
    import datasets as testing
    allrows = testing.gaussian_mixture(3064, 768, 40, 0.05, seed=1234, dim_decay=0.9,
                                       normalize_rows=True).numpy()
    x, q = allrows[:3000], allrows[3000:]
    index, ix = _config_case(orc, x, q, 24, 384, 4, "inner_product", "subspace")
    nb, d, want_nb, want_d = _search_both(orc, index, ix, q, 10, 8, R_8U, R_16F)
    H.compare_results(nb, d, want_nb, want_d, 2e-3, exact=True)


@pytest.mark.parametrize("batch", [1, 100])
def test_config5_shape_half_rows_per_cluster(orc, batch):
    """96-d fp16 rows, per-cluster codebooks, pq_dim 48, 8 bit, fp16 table, many probes; batch sizes
    1 and 100."""
    import datasets as testing
    allrows = testing.gaussian_mixture(12100, 96, 300, 0.25, seed=1234).numpy().astype(np.float16)
    x, q = allrows[:12000], allrows[12000:12000 + batch]
    index, ix = _config_case(orc, x, q, 150, 48, 8, "sqeuclidean", "cluster")
    nb, d, want_nb, want_d = _search_both(orc, index, ix, q, 10, 100, R_16F, R_32F)
    H.compare_results(nb, d, want_nb, want_d, 2e-3, exact=True)


@pytest.mark.parametrize("k", [10, 300])
def test_lookup_table_larger_than_lds_goes_to_global_memory(orc, k):
    """pq_dim 192 x 256 entries x 4 bytes = 192 KB: more than the 160 KB of LDS."""
    data, model, queries, index, ix, _ = _case(orc, 3000, 192, 8, 192, 8, n_queries=24)
    for metric_lut in [(R_32F, R_32F)]:
        nb, d, want_nb, want_d = _search_both(orc, index, ix, queries, k, 4, *metric_lut)
        H.compare_results(nb, d, want_nb, want_d, 1e-5, exact=True)
    # the fp16 table of the same index (96 KB) stays in LDS and agrees with its own oracle run
    nb, d, want_nb, want_d = _search_both(orc, index, ix, queries, k, 4, R_16F, R_32F)
    H.compare_results(nb, d, want_nb, want_d, 2e-3, exact=True)


# --- refinement: exact re-ranking of the candidates an approximate search returned ---

@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.int8, np.uint8])
@pytest.mark.parametrize("metric", ["sqeuclidean", "euclidean", "inner_product"])
def test_refine_matches_oracle(orc, dtype, metric):
    from cuvs_amd import refine
    rng = np.random.default_rng(5)
    n, dim, nq, nc, k = 3000, 100, 70, 64, 10
    data = H.make_data(n, dim, dtype, 21)
    q = H.make_data(nq, dim, dtype, 22)
    cand = rng.integers(0, n, (nq, nc)).astype(np.int64)
    cand[0, :6] = [-1, n, -5, n + 1, 2 ** 40, -2 ** 40]
    cand[1, :] = n
    d, ids = refine(G.to_dev(data), G.to_dev(q), G.to_dev(cand), k, metric=metric)
    code = {"sqeuclidean": 0, "euclidean": 1, "inner_product": 6}[metric]
    want_ids, want_d = orc.refine(data, q, cand, k, code)
    ids, d = ids.cpu().numpy(), d.cpu().numpy()
    if np.dtype(dtype).kind in "iu":
        # integer rows: exact arithmetic on both sides (the reduction order cannot matter)
        assert np.array_equal(d, want_d)
        # equal distances may come out in another candidate order only if the ids tie exactly
        assert np.all((ids == want_ids) | (d == np.roll(d, 1, axis=1)) | (d == np.roll(d, -1, axis=1)))
    else:
        np.testing.assert_allclose(d, want_d, rtol=1e-5, atol=1e-6)
        assert np.all((ids == want_ids) | np.isclose(d, want_d, rtol=1e-5, atol=1e-6))
    assert (ids[1] == -1).all()


def test_refine_after_search_raises_recall(orc):
    """The use the reference documents: search 4k candidates, refine to k."""
    import datasets as testing
    from cuvs_amd import refine
    x, q, index, ix = _clustered_case(orc)
    sp = ivf_pq.SearchParams(n_probes=20, lut_dtype=R_16F)
    k = 10
    _, cand = ivf_pq.search(sp, index, G.to_dev(q), 4 * k)
    _, plain = ivf_pq.search(sp, index, G.to_dev(q), k)
    d, ids = refine(G.to_dev(x), G.to_dev(q), cand, k)
    truth = testing.exact_knn(torch.from_numpy(x), torch.from_numpy(q), k).numpy()
    r_plain = testing.recall(plain.cpu().numpy(), truth)
    r_ref = testing.recall(ids.cpu().numpy(), truth)
    assert r_ref > r_plain and r_ref > 0.9
    want_ids, want_d = orc.refine(x, q, cand.cpu().numpy(), k, 0)
    np.testing.assert_allclose(d.cpu().numpy(), want_d, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.int8, np.uint8])
@pytest.mark.parametrize("metric", ["sqeuclidean", "euclidean", "inner_product"])
def test_refine_of_host_matrices_is_the_device_result(orc, dtype, metric):
    """Matrices in plain host memory (the reference refines those on the CPU): staged through the
    device, same rows and distances as the device overload, and the oracle's."""
    from cuvs_amd import refine
    rng = np.random.default_rng(15)
    n, dim, nq, nc, k = 3000, 100, 70, 64, 10
    data = H.make_data(n, dim, dtype, 31)
    q = H.make_data(nq, dim, dtype, 32)
    cand = rng.integers(0, n, (nq, nc)).astype(np.int64)
    cand[0, :6] = [-1, n, -5, n + 1, 2 ** 40, -2 ** 40]
    cand[1, :] = n
    cand[2, 1:] = cand[2, 0]  # one row sixty-four times: ties go by position in both overloads
    d_dev, ids_dev = refine(G.to_dev(data), G.to_dev(q), G.to_dev(cand), k, metric=metric)
    d, ids = refine(data, q, cand, k, metric=metric)
    assert isinstance(d, np.ndarray) and isinstance(ids, np.ndarray)
    assert np.array_equal(ids, ids_dev.cpu().numpy())
    assert np.array_equal(d.view(np.uint32), d_dev.cpu().numpy().view(np.uint32))
    # CPU tensors take the same way, into outputs the caller made
    out_i = torch.full((nq, k), -7, dtype=torch.int64)
    out_d = torch.zeros((nq, k), dtype=torch.float32)
    refine(torch.from_numpy(data), torch.from_numpy(q), torch.from_numpy(cand), metric=metric,
           indices=out_i, distances=out_d)
    assert np.array_equal(out_i.numpy(), ids) and np.array_equal(out_d.numpy(), d)
    code = {"sqeuclidean": 0, "euclidean": 1, "inner_product": 6}[metric]
    want_ids, want_d = orc.refine(data, q, cand, k, code)
    np.testing.assert_allclose(d, want_d, rtol=1e-5, atol=1e-6)
    assert (ids[1] == -1).all()


def test_refine_of_host_matrices_in_several_batches(orc):
    """More candidate rows than one staging batch holds (256 MiB): the batches join up."""
    from cuvs_amd import refine
    rng = np.random.default_rng(16)
    n, dim, nq, nc, k = 5000, 1024, 2500, 40, 5   # 2500 x 40 x 4 KiB = 390 MiB of candidate rows
    data = rng.standard_normal((n, dim), dtype=np.float32)
    q = rng.standard_normal((nq, dim), dtype=np.float32)
    cand = rng.integers(0, n, (nq, nc)).astype(np.int64)
    d, ids = refine(data, q, cand, k)
    d_dev, ids_dev = refine(G.to_dev(data), G.to_dev(q), G.to_dev(cand), k)
    assert np.array_equal(ids, ids_dev.cpu().numpy())
    assert np.array_equal(d.view(np.uint32), d_dev.cpu().numpy().view(np.uint32))


def test_refine_refuses_a_mix_of_host_and_device_matrices(orc):
    from cuvs_amd import refine
    data = np.zeros((10, 4), dtype=np.float32)
    q = np.zeros((3, 4), dtype=np.float32)
    cand = np.zeros((3, 5), dtype=np.int64)
    with pytest.raises(CuvsError, match="either all be on device memory, or all on host memory"):
        refine(G.to_dev(data), q, cand, 2, indices=np.zeros((3, 2), np.int64),
               distances=np.zeros((3, 2), np.float32))
    with pytest.raises(CuvsError, match="either all be on device memory, or all on host memory"):
        refine(data, q, G.to_dev(cand), 2)


def test_refine_validation(orc):
    from cuvs_amd import refine
    data = G.to_dev(np.zeros((10, 4), dtype=np.float32))
    q = G.to_dev(np.zeros((3, 4), dtype=np.float32))
    cand = G.to_dev(np.zeros((3, 5), dtype=np.int64))
    with pytest.raises(CuvsError, match="candidates must not be smaller than k"):
        refine(data, q, cand, 6)
    with pytest.raises(CuvsError, match="Number of columns must be equal"):
        refine(data, G.to_dev(np.zeros((3, 5), dtype=np.float32)), cand, 2)
    with pytest.raises(CuvsError, match="type mismatch"):
        refine(data, G.to_dev(np.zeros((3, 4), dtype=np.float16)), cand, 2)
    with pytest.raises(ValueError):
        refine(data, q, cand, 2, metric="cosine")


# --- probe selection in two precisions (fp16 matrix cores + exact rescoring of the candidates) ---

def _coarse_model(n_lists, dim, pq_dim, seed, scale=1.0, cluster=True):
    """A model with many lists and no training: centres drawn around a few hundred hubs (so that
    scores near the n_probes-th best are close together), identity rotation, random codebooks."""
    rng = np.random.default_rng(seed)
    if cluster:
        hubs = rng.standard_normal((max(n_lists // 16, 1), dim)).astype(np.float32)
        centers = hubs[rng.integers(0, hubs.shape[0], n_lists)] + 0.05 * rng.standard_normal((n_lists, dim)).astype(np.float32)
    else:
        centers = rng.standard_normal((n_lists, dim)).astype(np.float32)
    centers = (centers * scale).astype(np.float32)
    ext = np.zeros((n_lists, ((dim + 1 + 7) // 8) * 8), dtype=np.float32)
    ext[:, :dim] = centers
    ext[:, dim] = (centers.astype(np.float64) ** 2).sum(1).astype(np.float32)
    return {"centers": ext, "centers_rot": centers.copy(),
            "rotation_matrix": np.eye(dim, dtype=np.float32),
            "pq_centers": rng.standard_normal((pq_dim, dim // pq_dim, 256)).astype(np.float32)}


@pytest.mark.parametrize("metric", ["sqeuclidean", "inner_product", "cosine"])
# (dimensions from 129 on run the GEMM shapes of one list tile or one query tile a wave: padded to
# 256, 384, 512, 768 and 1024)
@pytest.mark.parametrize("dtype,dim", [(np.float32, 96), (np.float16, 128), (np.int8, 64), (np.uint8, 40),
                                       (np.float32, 256), (np.float16, 200), (np.float32, 384), (np.int8, 512),
                                       (np.uint8, 768), (np.float32, 1024), (np.float16, 1000), (np.float32, 640)])
def test_two_precision_probe_selection_equals_the_fp32_path(orc, metric, dtype, dim):
    n_lists, pq_dim = 4096, dim // 4
    model = _coarse_model(n_lists, dim, pq_dim, 3, scale=(0.5 if dtype in (np.int8, np.uint8) else 1.0))
    params = ivf_pq.IndexParams(n_lists=n_lists, metric=metric, pq_dim=pq_dim, pq_bits=8)
    dev = {k: G.to_dev(v) for k, v in model.items()}
    index = ivf_pq.build_precomputed(params, dim, dev["pq_centers"], dev["centers"], dev["centers_rot"],
                                     dev["rotation_matrix"])
    ix = H.oracle_index(orc, model, dim, pq_dim, 8, metric=metric)
    rng = np.random.default_rng(8)
    if dtype == np.uint8:
        q = rng.integers(0, 256, (300, dim)).astype(np.uint8)
    elif dtype == np.int8:
        q = rng.integers(-128, 128, (300, dim)).astype(np.int8)
    else:
        # some queries sit on a centre, some between two
        c = model["centers"][:, :dim]
        q = np.concatenate([c[:100], 0.5 * (c[100:200] + c[200:300]),
                            rng.standard_normal((100, dim)).astype(np.float32)]).astype(dtype)
    for n_probes in (1, 20, 64, 128):
        sp = ivf_pq.SearchParams(n_probes=n_probes)
        got = ivf_pq.select_clusters(sp, index, G.to_dev(q)).cpu().numpy().view(np.uint32)
        want, _ = orc.select_clusters(ix, q, n_probes)
        assert np.array_equal(got, want), (metric, dtype, n_probes)


@pytest.mark.parametrize("metric,dtype", [("sqeuclidean", np.float16), ("inner_product", np.float32)])
def test_two_precision_probe_selection_many_lists_and_probes(orc, metric, dtype):
    """50,000 lists (more group minima than a wave holds in 16 registers a lane) and up to 256
    probes (candidate lists of up to 512)."""
    n_lists, dim, pq_dim = 50_000, 96, 48
    model = _coarse_model(n_lists, dim, pq_dim, 11)
    params = ivf_pq.IndexParams(n_lists=n_lists, metric=metric, pq_dim=pq_dim, pq_bits=8)
    dev = {k: G.to_dev(v) for k, v in model.items()}
    index = ivf_pq.build_precomputed(params, dim, dev["pq_centers"], dev["centers"], dev["centers_rot"],
                                     dev["rotation_matrix"])
    ix = H.oracle_index(orc, model, dim, pq_dim, 8, metric=metric)
    rng = np.random.default_rng(12)
    c = model["centers"][:, :dim]
    q = np.concatenate([c[:40], 0.5 * (c[100:140] + c[200:240]),
                        rng.standard_normal((40, dim)).astype(np.float32)]).astype(dtype)
    for n_probes in (1, 100, 200, 256):
        sp = ivf_pq.SearchParams(n_probes=n_probes)
        got = ivf_pq.select_clusters(sp, index, G.to_dev(q)).cpu().numpy().view(np.uint32)
        want, _ = orc.select_clusters(ix, q, n_probes)
        assert np.array_equal(got, want), (metric, n_probes)


def test_two_precision_probe_selection_falls_back(orc):
    """Identical centres put hundreds of lists inside the error margin (more candidates than the
    fast path holds), and a query with a NaN has no usable bound: both take the plain fp32 path and
    still equal the oracle.  Centres beyond binary16's range switch the fast path off."""
    dim, n_lists = 32, 2048
    model = _coarse_model(n_lists, dim, 8, 4)
    model["centers"][:600] = model["centers"][0]           # 600 identical centres
    model["centers_rot"][:600] = model["centers_rot"][0]
    params = ivf_pq.IndexParams(n_lists=n_lists, pq_dim=8, pq_bits=8)
    dev = {k: G.to_dev(v) for k, v in model.items()}
    index = ivf_pq.build_precomputed(params, dim, dev["pq_centers"], dev["centers"], dev["centers_rot"],
                                     dev["rotation_matrix"])
    ix = H.oracle_index(orc, model, dim, 8, 8)
    rng = np.random.default_rng(9)
    q = rng.standard_normal((64, dim)).astype(np.float32)
    q[:8] = model["centers"][0, :dim] + 0.001 * rng.standard_normal((8, dim)).astype(np.float32)
    got = ivf_pq.select_clusters(ivf_pq.SearchParams(n_probes=32), index, G.to_dev(q)).cpu().numpy().view(np.uint32)
    want, _ = orc.select_clusters(ix, q, 32)
    assert np.array_equal(got, want)
    # huge centres: the fp16 copy would overflow, the index says so and the plain path runs
    big = _coarse_model(n_lists, dim, 8, 5, scale=1e5)
    devb = {k: G.to_dev(v) for k, v in big.items()}
    index_b = ivf_pq.build_precomputed(params, dim, devb["pq_centers"], devb["centers"], devb["centers_rot"],
                                       devb["rotation_matrix"])
    ixb = H.oracle_index(orc, big, dim, 8, 8)
    qb = (1e5 * rng.standard_normal((32, dim))).astype(np.float32)
    got = ivf_pq.select_clusters(ivf_pq.SearchParams(n_probes=16), index_b, G.to_dev(qb)).cpu().numpy().view(np.uint32)
    want, _ = orc.select_clusters(ixb, qb, 16)
    assert np.array_equal(got, want)


# --- 4-bit codes: the block kernel with tables held in the accumulator's type ---

_NIBBLE = {}


def _nibble_case(orc, dim, pq_dim, metric, kind):
    key = (dim, pq_dim, metric, kind)
    if key not in _NIBBLE:
        _NIBBLE[key] = _case(orc, 6000, dim, 24, pq_dim, 4, metric=metric, kind=kind, n_queries=48)
    return _NIBBLE[key]


@pytest.mark.parametrize("lut,internal", [(R_32F, R_32F), (R_16F, R_32F), (R_8U, R_32F), (R_16F, R_16F),
                                          (R_8U, R_16F)])
@pytest.mark.parametrize("dim,pq_dim,metric,kind", [
    (128, 64, "sqeuclidean", "subspace"),    # two chunks (half a step), pq_len 2
    (96, 96, "inner_product", "subspace"),   # three chunks: a partial step, pq_len 1
    (128, 32, "cosine", "cluster"),          # one chunk, pq_len 4, per-cluster codebooks
    (320, 160, "euclidean", "subspace"),     # five chunks: a full step and a partial one
])
def test_four_bit_block_kernel_matches_oracle(orc, lut, internal, dim, pq_dim, metric, kind):
    data, model, queries, index, ix, _ = _nibble_case(orc, dim, pq_dim, metric, kind)
    for k, n_probes in ((1, 3), (10, 8), (100, 24), (200, 24)):
        nb, d, want_nb, want_d = _search_both(orc, index, ix, queries, k, n_probes, lut=lut,
                                              internal=internal)
        H.compare_results(nb, d, want_nb, want_d, 1e-5 if lut == R_32F else 2e-3,
                          exact=(metric != "euclidean"))


@pytest.mark.parametrize("lut", [R_16F, R_8U])
@pytest.mark.parametrize("internal", [R_16F, R_32F])
@pytest.mark.parametrize("dim,pq_dim,metric,kind", [
    (256, 128, "sqeuclidean", "subspace"),   # two steps, pq_len 2, early stop inside a tile
    (128, 128, "inner_product", "subspace"), # pq_len 1
    (512, 128, "cosine", "cluster"),         # pq_len 4, per-cluster codebooks
    (512, 256, "euclidean", "subspace"),     # four steps
    (128, 64, "sqeuclidean", "subspace"),    # a single step (L2 takes any number of them)
    (192, 192, "euclidean", "cluster"),      # three steps, pq_len 1, per-cluster codebooks
])
def test_four_bit_two_rows_per_lane_kernel_matches_oracle(orc, lut, internal, dim, pq_dim, metric, kind):
    """pq_dim a multiple of 128, k <= 64, binary16 tables (sums of either type): the kernel that
    scores two rows per lane, one wave per pair, with the bound looked at inside a step."""
    data, model, queries, index, ix, _ = _nibble_case(orc, dim, pq_dim, metric, kind)
    for k, n_probes in ((1, 3), (10, 8), (64, 24)):
        nb, d, want_nb, want_d = _search_both(orc, index, ix, queries, k, n_probes, lut=lut, internal=internal)
        H.compare_results(nb, d, want_nb, want_d, 2e-3, exact=(metric != "euclidean"))


def test_four_bit_two_rows_per_lane_kernel_filter_and_long_lists(orc):
    """Lists of several thousand rows (many tiles of 128 rows per wave, the candidate buffer is
    reduced several times) and a bitset filter."""
    data, model, queries, index, ix, _ = _case(orc, 40000, 128, 6, 128, 4, n_queries=24)
    n = data.shape[0]
    keep = np.ones(n, dtype=bool)
    keep[::4] = False
    bits = np.packbits(keep, bitorder="little")
    bits = np.concatenate([bits, np.zeros((-bits.size) % 4, dtype=np.uint8)]).view(np.uint32)
    for lut in (R_16F, R_8U):
        sp = ivf_pq.SearchParams(n_probes=4, lut_dtype=lut, internal_distance_dtype=R_16F)
        d, nb = ivf_pq.search(sp, index, G.to_dev(queries), 50,
                              filter_bitset=G.to_dev(bits.view(np.int32)), filter_nbits=n)
        want_nb, want_d = orc.search(ix, queries, 50, 4, lut_dtype=ORC_DT[lut], internal_distance_dtype=ORC_DT[R_16F],
                                     filter_bitset=bits, filter_nbits=n)
        H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 2e-3, exact=True)
        nb2, d2, want_nb2, want_d2 = _search_both(orc, index, ix, queries, 64, 6, lut=lut, internal=R_16F)
        H.compare_results(nb2, d2, want_nb2, want_d2, 2e-3, exact=True)


_BITS = {}


def _bits_case(orc, dim, pq_dim, pq_bits, metric, kind):
    key = (dim, pq_dim, pq_bits, metric, kind)
    if key not in _BITS:
        _BITS[key] = _case(orc, 6000, dim, 24, pq_dim, pq_bits, metric=metric, kind=kind, n_queries=48)
    return _BITS[key]


@pytest.mark.parametrize("lut,internal", [(R_16F, R_32F), (R_8U, R_32F), (R_16F, R_16F), (R_8U, R_16F)])
@pytest.mark.parametrize("dim,pq_dim,pq_bits,metric,kind", [
    (128, 64, 5, "sqeuclidean", "subspace"),    # 25 codes a chunk: three chunks, the last one 14 codes
    (128, 64, 6, "inner_product", "subspace"),  # 21 codes a chunk: four chunks, the last one a single code
    (128, 64, 7, "sqeuclidean", "cluster"),     # 18 codes a chunk, per-cluster codebooks
    (96, 96, 6, "cosine", "subspace"),          # pq_len 1, five chunks
    (128, 32, 7, "euclidean", "subspace"),      # pq_len 4, two chunks
])
def test_five_to_seven_bit_codes_match_oracle(orc, lut, internal, dim, pq_dim, pq_bits, metric, kind):
    """Codes of 5, 6 and 7 bits (bit-packed, some straddling two words of a chunk, the last chunk
    partly filled) at the benchmark's subspace counts."""
    data, model, queries, index, ix, _ = _bits_case(orc, dim, pq_dim, pq_bits, metric, kind)
    for k, n_probes in ((1, 3), (10, 8), (64, 24)):
        nb, d, want_nb, want_d = _search_both(orc, index, ix, queries, k, n_probes, lut=lut, internal=internal)
        H.compare_results(nb, d, want_nb, want_d, 2e-3, exact=(metric != "euclidean"))


def test_five_to_seven_bit_codes_filter_and_long_lists(orc):
    """Lists of several thousand rows and a bitset filter, 6-bit codes."""
    data, model, queries, index, ix, _ = _case(orc, 40000, 64, 6, 32, 6, n_queries=24)
    n = data.shape[0]
    keep = np.ones(n, dtype=bool)
    keep[::4] = False
    bits = np.packbits(keep, bitorder="little")
    bits = np.concatenate([bits, np.zeros((-bits.size) % 4, dtype=np.uint8)]).view(np.uint32)
    for lut in (R_16F, R_8U):
        sp = ivf_pq.SearchParams(n_probes=4, lut_dtype=lut)
        d, nb = ivf_pq.search(sp, index, G.to_dev(queries), 50,
                              filter_bitset=G.to_dev(bits.view(np.int32)), filter_nbits=n)
        want_nb, want_d = orc.search(ix, queries, 50, 4, lut_dtype=ORC_DT[lut], filter_bitset=bits, filter_nbits=n)
        H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 2e-3, exact=True)
        nb2, d2, want_nb2, want_d2 = _search_both(orc, index, ix, queries, 64, 6, lut=lut)
        H.compare_results(nb2, d2, want_nb2, want_d2, 2e-3, exact=True)


def test_byte_wide_copy_of_narrow_codes_follows_the_lists():
    """5 - 7 bit codes are searched on a byte-per-code copy of the lists.  The copy is an
    acceleration only: the generic kernel on the packed lists (search tuning), an index built with
    conservative_memory_allocation (no copy) and the default path return the same neighbours and
    distances, before and after the lists grow, and the early stop runs on these widths too."""
    import datasets as testing
    from cuvs_amd.resources import Resources
    allrows = testing.gaussian_mixture(60000 + 2000, 128, 96, 0.15, seed=123, device="cuda")
    data, queries = allrows[:60000], allrows[60000:]
    first, second = data[:40000], data[40000:]
    ids2 = torch.arange(40000, 60000, dtype=torch.int64, device="cuda")
    for bits in (5, 6, 7):
        kw = dict(n_lists=128, pq_dim=64, pq_bits=bits)
        ids1 = torch.arange(40000, dtype=torch.int64, device="cuda")
        trained = ivf_pq.build(ivf_pq.IndexParams(kmeans_trainset_fraction=0.5, add_data_on_build=False, **kw), first)
        model = (trained.pq_centers, trained.centers_padded, trained.centers_rot, trained.rotation_matrix)
        index = ivf_pq.extend(ivf_pq.build_precomputed(ivf_pq.IndexParams(**kw), 128, *model), first, ids1)
        lean = ivf_pq.extend(ivf_pq.build_precomputed(
            ivf_pq.IndexParams(conservative_memory_allocation=True, **kw), 128, *model), first, ids1)
        plain, tuned = Resources(), Resources()
        plain.enable_profiling(True)
        tuned.set_search_tuning(generic_scan=True)
        sp = ivf_pq.SearchParams(n_probes=20, lut_dtype=R_16F)
        for step in range(2):
            d, nb = ivf_pq.search(sp, index, queries, 10, resources=plain)
            plain.sync()
            assert ivf_pq.get_search_profile(plain)["n_screened_pairs"] == queries.shape[0] * 19, bits
            d2, nb2 = ivf_pq.search(sp, index, queries, 10, resources=tuned)
            d3, nb3 = ivf_pq.search(sp, lean, queries, 10)
            assert torch.equal(nb, nb2) and torch.equal(d, d2), (bits, step, "generic kernel")
            # another index object: rows take their places inside a list in the order the encoding
            # blocks finish, so of two rows at exactly the same distance (equal codes in one list)
            # either may come first, or alone if the tie is at rank k: the distances say it all
            assert torch.equal(d, d3), (bits, step, "no copy")
            assert float((nb == nb3).float().mean()) > 0.99, (bits, step, "no copy")
            if step == 0:
                index = ivf_pq.extend(index, second, ids2)
                lean = ivf_pq.extend(lean, second, ids2)
        assert int(nb.max()) >= 40000  # the rows added later are found


@pytest.mark.parametrize("lut", [R_32F, R_16F])
def test_block_per_pair_kernel_prunes_long_lists(orc, lut):
    """Lists of 5,000 rows scanned by the block-per-pair kernel (fp32 tables; k above the CU-wide
    kernel's limit): its candidate buffer fills to 1,280 and more keys several times a list and is
    pruned by the waves' radix selection, in one piece up to 1,024 keys and in two halves beyond."""
    data, model, queries, index, ix, _ = _case(orc, 20000, 128, 4, 64, 8, n_queries=32)
    for k, n_probes in ((256, 3), (100, 4), (10, 2)):
        nb, d, want_nb, want_d = _search_both(orc, index, ix, queries, k, n_probes, lut=lut)
        H.compare_results(nb, d, want_nb, want_d, 1e-5 if lut == R_32F else 2e-3, exact=True)


def test_four_bit_block_kernel_filter_and_long_lists(orc):
    """Lists of several thousand rows (more than one pruning segment of the candidate buffer) and a
    bitset filter."""
    data, model, queries, index, ix, _ = _case(orc, 40000, 64, 6, 32, 4, n_queries=24)
    n = data.shape[0]
    keep = np.ones(n, dtype=bool)
    keep[::4] = False
    bits = np.packbits(keep, bitorder="little")
    bits = np.concatenate([bits, np.zeros((-bits.size) % 4, dtype=np.uint8)]).view(np.uint32)
    for lut in (R_32F, R_16F, R_8U):
        sp = ivf_pq.SearchParams(n_probes=4, lut_dtype=lut)
        d, nb = ivf_pq.search(sp, index, G.to_dev(queries), 50,
                              filter_bitset=G.to_dev(bits.view(np.int32)), filter_nbits=n)
        want_nb, want_d = orc.search(ix, queries, 50, 4, lut_dtype=ORC_DT[lut], filter_bitset=bits,
                                     filter_nbits=n)
        H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d,
                          1e-5 if lut == R_32F else 2e-3, exact=True)
        nb2, d2, want_nb2, want_d2 = _search_both(orc, index, ix, queries, 128, 6, lut=lut)
        H.compare_results(nb2, d2, want_nb2, want_d2, 1e-5 if lut == R_32F else 2e-3, exact=True)
