"""Index training on the GPU (cuvsIvfPqBuild): coarse k-means, rotation, codebooks.

Training is randomised in the reference (its own RNG, atomics in the centre updates), so nothing
fixes a bit pattern for the trained model: **parity unpinned** for the model tensors.  What the
reference's tests hold a build to is recall (cpp/tests/neighbors/ann_ivf_pq.cuh), and that is what
these tests check, together with the structural facts that do not depend on the random draw: the
model has the reference's shapes and invariants, the stored lists are exactly the oracle's encoding
of the dataset under the trained model, and searching the trained index equals the oracle bit for
bit.
"""
import numpy as np
import pytest
import torch

import gpu_helpers as G
import helpers as H
import datasets as testing
from cuvs_amd import ivf_pq

pytestmark = pytest.mark.gpu

R_32F, R_16F, R_8U = 0, 2, 8


def _model_of(index):
    return {"centers": index.centers_padded.cpu().numpy(),
            "centers_rot": index.centers_rot.cpu().numpy(),
            "rotation_matrix": index.rotation_matrix.cpu().numpy(),
            "pq_centers": index.pq_centers.cpu().numpy()}


def _recall(nb, truth):
    return testing.recall(nb, truth)


def _data(dtype, n, dim, seed):
    if dtype == np.uint8:
        return testing.sift_like_u8(n, dim, 50, seed=seed).numpy()
    if dtype == np.int8:
        return (testing.sift_like_u8(n, dim, 50, seed=seed).numpy().astype(np.int16) - 128).astype(np.int8)
    return testing.gaussian_mixture(n, dim, 50, 0.25, seed=seed).numpy().astype(dtype)


@pytest.mark.parametrize("metric,kind,dtype,pq_bits", [
    ("sqeuclidean", "subspace", np.float32, 8),
    ("sqeuclidean", "cluster", np.float32, 8),
    ("inner_product", "subspace", np.float32, 8),
    ("cosine", "subspace", np.float16, 8),
    ("euclidean", "subspace", np.uint8, 8),
    ("sqeuclidean", "subspace", np.int8, 5),
    ("sqeuclidean", "cluster", np.float32, 4),
])
def test_build_model_lists_and_search(orc, metric, kind, dtype, pq_bits):
    n, dim, n_lists, pq_dim = 12000, 32, 48, 16
    allrows = _data(dtype, n + 100, dim, 21)
    x, q = allrows[:n], allrows[n:]
    params = ivf_pq.IndexParams(n_lists=n_lists, metric=metric, pq_dim=pq_dim, pq_bits=pq_bits,
                                codebook_kind=kind, kmeans_n_iters=10, kmeans_trainset_fraction=0.5)
    index = ivf_pq.build(params, G.to_dev(x))
    assert len(index) == n and index.n_lists == n_lists and index.pq_dim == pq_dim
    model = _model_of(index)
    book = 1 << pq_bits
    # shapes and invariants of the model (ivf_pq.hpp: centers carry their squared norm in column dim)
    c = model["centers"]
    assert c.shape == (n_lists, 40) and model["centers_rot"].shape == (n_lists, dim)
    assert model["pq_centers"].shape == ((n_lists if kind == "cluster" else pq_dim), dim // pq_dim, book)
    assert np.all(np.isfinite(c)) and np.all(np.isfinite(model["pq_centers"]))
    np.testing.assert_allclose(c[:, dim], (c[:, :dim].astype(np.float64) ** 2).sum(1), rtol=1e-5)
    assert np.array_equal(c[:, dim + 1:], np.zeros((n_lists, 40 - dim - 1), np.float32))
    assert np.array_equal(model["rotation_matrix"], np.eye(dim, dtype=np.float32))
    np.testing.assert_allclose(model["centers_rot"], c[:, :dim], rtol=0, atol=0)
    if metric == "cosine":
        np.testing.assert_allclose(np.linalg.norm(c[:, :dim], axis=1), 1.0, rtol=1e-5)
    # balanced lists: nothing empty, nothing above four times the average
    sizes = index.list_sizes.cpu().numpy()
    assert sizes.sum() == n and sizes.min() > 0 and sizes.max() <= 4 * n / n_lists
    # the stored lists are the oracle's encoding of the dataset under this model
    ix, gpu_codes = G.read_back(orc, index, model, dim, pq_dim, pq_bits, metric, kind)
    labels, codes = orc.encode(ix, x)
    assert np.array_equal(np.bincount(labels, minlength=n_lists), sizes)
    for l in range(0, n_lists, 5):
        order = np.argsort(ix.list_inds[l])
        assert np.array_equal(ix.list_inds[l][order], np.nonzero(labels == l)[0])
        assert np.array_equal(gpu_codes[l][order], codes[labels == l])
    # search on the trained index equals the oracle on the same index
    sp = ivf_pq.SearchParams(n_probes=12)
    d, nb = ivf_pq.search(sp, index, G.to_dev(q), 10)
    want_nb, want_d = orc.search(ix, q, 10, 12)
    H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 1e-5, exact=(metric != "euclidean"))
    # and it finds neighbours about as well as a model trained by plain Lloyd iterations on the CPU
    xm = x.astype(np.float32)
    qm = q.astype(np.float32)
    if metric == "inner_product":
        truth = np.argsort(-(qm @ xm.T), axis=1)[:, :10]
    elif metric == "cosine":
        xn = xm / np.linalg.norm(xm, axis=1, keepdims=True)
        truth = np.argsort(-((qm / np.linalg.norm(qm, axis=1, keepdims=True)) @ xn.T), axis=1)[:, :10]
    else:
        truth = testing.exact_knn(torch.from_numpy(xm), torch.from_numpy(qm), 10).numpy()
    got = _recall(nb.cpu().numpy(), truth)
    ref_model = H.train(x, n_lists, pq_dim, pq_bits, metric=metric, codebook_kind=kind, iters=10)
    ref_index = G.build_gpu_index(ref_model, x, pq_dim, pq_bits, metric, kind)
    _, ref_nb = ivf_pq.search(sp, ref_index, G.to_dev(q), 10)
    ref = _recall(ref_nb.cpu().numpy(), truth)
    print(f"recall: built {got:.3f}, CPU-trained model {ref:.3f}", flush=True)
    assert got >= ref - 0.05


@pytest.mark.parametrize("pq_bits,lut,floor", [(8, R_32F, 0.86), (8, R_8U, 0.84), (6, R_16F, 0.84),
                                                (4, R_32F, 0.79)])
def test_build_meets_the_reference_recall_floors(pq_bits, lut, floor):
    """Recall floors of the reference's own suite on uniform [0.1, 2) data, 4096 x 64, k = 32,
    32 lists, 20 probes (cpp/tests/neighbors/ann_ivf_pq.cuh:27-43,979-1122); the 4-bit floor there is
    for per-cluster codebooks."""
    data = H.uniform_data(4096, 64, 1234)
    queries = H.uniform_data(256, 64, 4321)
    kind = "cluster" if pq_bits == 4 else "subspace"
    params = ivf_pq.IndexParams(n_lists=32, pq_dim=64, pq_bits=pq_bits, codebook_kind=kind,
                                kmeans_trainset_fraction=1.0)
    index = ivf_pq.build(params, G.to_dev(data))
    sp = ivf_pq.SearchParams(n_probes=20, lut_dtype=lut)
    _, nb = ivf_pq.search(sp, index, G.to_dev(queries), 32)
    d = ((queries[:, None, :].astype(np.float64) - data[None].astype(np.float64)) ** 2).sum(-1)
    truth = np.argsort(d, axis=1)[:, :32]
    assert _recall(nb.cpu().numpy(), truth) >= floor


def test_build_random_rotation_padded_dim_and_host_dataset(orc):
    """dim 30 with pq_dim 8: rot_dim 32 > dim forces a random rotation with orthonormal columns;
    the dataset comes from host memory; add_data_on_build=False leaves the index empty."""
    n, dim, pq_dim = 6000, 30, 8
    x = testing.gaussian_mixture(n, dim, 30, 0.25, seed=5).numpy()
    params = ivf_pq.IndexParams(n_lists=24, pq_dim=pq_dim, kmeans_n_iters=8, add_data_on_build=False)
    index = ivf_pq.build(params, torch.from_numpy(x))
    assert len(index) == 0
    rot = index.rotation_matrix.cpu().numpy()
    assert rot.shape == (32, 30)
    np.testing.assert_allclose(rot.T @ rot, np.eye(30), atol=1e-5)
    np.testing.assert_allclose(index.centers_rot.cpu().numpy(),
                               index.centers.cpu().numpy() @ rot.T, atol=1e-4)
    ivf_pq.extend(index, G.to_dev(x), None)
    assert len(index) == n
    model = _model_of(index)
    ix, _ = G.read_back(orc, index, model, dim, pq_dim, 8)
    q = x[:50] + 0.01
    d, nb = ivf_pq.search(ivf_pq.SearchParams(n_probes=6), index, G.to_dev(q), 5)
    want_nb, want_d = orc.search(ix, q, 5, 6)
    H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 1e-5, exact=True)
    assert (nb.cpu().numpy()[:, 0] == np.arange(50)).mean() > 0.9


def test_build_kmeans_quality_against_lloyd():
    """The coarse centres' mean squared distance to the training rows is within 5 % of what plain
    Lloyd iterations from a k-means++-free random start reach on the CPU (same data, same count)."""
    n, dim, n_lists = 20000, 24, 64
    x = testing.gaussian_mixture(n, dim, 80, 0.3, seed=9).numpy()
    params = ivf_pq.IndexParams(n_lists=n_lists, pq_dim=12, kmeans_trainset_fraction=1.0,
                                add_data_on_build=False)
    index = ivf_pq.build(params, G.to_dev(x))
    c = index.centers.cpu().numpy().astype(np.float64)
    xd = x.astype(np.float64)

    def inertia(centers):
        d = (xd ** 2).sum(1)[:, None] - 2 * xd @ centers.T + (centers ** 2).sum(1)[None]
        return d.min(1).mean(), d.argmin(1)

    got, _ = inertia(c)
    rng = np.random.default_rng(0)
    ref = xd[rng.choice(n, n_lists, replace=False)].copy()
    for _ in range(25):
        _, lab = inertia(ref)
        for l in range(n_lists):
            if (lab == l).any():
                ref[l] = xd[lab == l].mean(0)
    want, _ = inertia(ref)
    print(f"inertia: built {got:.4f}, Lloyd {want:.4f}", flush=True)
    assert got <= 1.05 * want


def test_build_validation():
    x = G.to_dev(testing.gaussian_mixture(100, 16, 4, 0.3, seed=1).numpy())
    with pytest.raises(Exception, match="less than n_lists"):
        ivf_pq.build(ivf_pq.IndexParams(n_lists=200, pq_dim=8), x)
    with pytest.raises(Exception, match="kmeans_trainset_fraction"):
        ivf_pq.build(ivf_pq.IndexParams(n_lists=4, pq_dim=8, kmeans_trainset_fraction=0.0), x)


@pytest.mark.parametrize("codebook_kind", ["subspace", "cluster"])
@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.int8, np.uint8])
@pytest.mark.parametrize("n_rows,pq_bits", [(500, 6), (100000, 8)])
def test_transform_matches_the_stored_lists(codebook_kind, dtype, n_rows, pq_bits):
    """The reference's own transform test (python/cuvs/cuvs/tests/test_ivf_pq.py:337-378):
    transforming the dataset an index was built from gives the labels and codes the index stores."""
    n_cols, n_lists, pq_dim = 32, 50, 8
    dataset = _data(dtype, n_rows, n_cols, 33)
    params = ivf_pq.IndexParams(n_lists=n_lists, pq_bits=pq_bits, pq_dim=pq_dim, codebook_kind=codebook_kind)
    index = ivf_pq.build(params, G.to_dev(dataset))
    labels_exp = np.zeros(n_rows, dtype=np.uint32)
    transformed_exp = np.zeros((n_rows, int(np.ceil(index.pq_dim * index.pq_bits / 8))), dtype=np.uint8)
    total = 0
    for cluster_id, (ids, codes) in enumerate(index.lists()):
        ids = ids.cpu().numpy()
        labels_exp[ids] = cluster_id
        transformed_exp[ids] = codes.cpu().numpy()
        total += ids.size
    assert total == n_rows == len(index)
    labels, transformed = ivf_pq.transform(index, G.to_dev(dataset))
    np.testing.assert_array_equal(labels.cpu().numpy().view(np.uint32), labels_exp)
    np.testing.assert_array_equal(transformed.cpu().numpy(), transformed_exp)


def test_python_mirror_of_the_reference_workflow(tmp_path):
    """build on a host array, extend in two halves with explicit indices (device, then host
    arrays), save / load, search with preallocated outputs, model getters: the calls of the
    reference's run_ivf_pq_build_search_test (python/cuvs/cuvs/tests/test_ivf_pq.py:21-125)."""
    n_rows, n_cols, n_queries, k = 10000, 10, 100, 10
    rng = np.random.default_rng(3)
    dataset = rng.random((n_rows, n_cols), dtype=np.float32)
    queries = rng.random((n_queries, n_cols), dtype=np.float32)
    params = ivf_pq.IndexParams(n_lists=100, metric="sqeuclidean", kmeans_n_iters=20, pq_bits=8, pq_dim=0,
                                add_data_on_build=False)
    assert params.n_lists == 100 and params.pq_bits == 8 and params.add_data_on_build is False
    index = ivf_pq.build(params, torch.from_numpy(dataset))
    assert index.trained and len(index) == 0 and "IvfPq" in repr(index)
    half = n_rows // 2
    ids = np.arange(n_rows, dtype=np.int64)
    index = ivf_pq.extend(index, G.to_dev(dataset[:half]), G.to_dev(ids[:half]))
    index = ivf_pq.extend(index, torch.from_numpy(dataset[half:]), torch.from_numpy(ids[half:]))
    assert len(index) == n_rows
    path = tmp_path / "index.bin"
    ivf_pq.save(str(path), index)
    index = ivf_pq.load(str(path))
    out_idx = torch.zeros((n_queries, k), dtype=torch.int64, device="cuda")
    out_dist = torch.zeros((n_queries, k), dtype=torch.float32, device="cuda")
    sp = ivf_pq.SearchParams(n_probes=100, lut_dtype=np.float32, internal_distance_dtype=np.float32)
    ret = ivf_pq.search(sp, index, G.to_dev(queries), k, neighbors=out_idx, distances=out_dist)
    torch.cuda.synchronize()
    assert ret[0].data_ptr() == out_dist.data_ptr() and ret[1].data_ptr() == out_idx.data_ptr()
    d = ((queries[:, None, :] - dataset[None]) ** 2).sum(-1)
    truth = np.argsort(d, axis=1)[:, :k]
    assert _recall(out_idx.cpu().numpy(), truth) > 0.7  # the reference's own bar for this test
    assert index.centers.shape == (100, n_cols) and index.pq_centers.shape[2] == 256
    assert sum(i.shape[0] for i, _ in index.lists()) == n_rows
