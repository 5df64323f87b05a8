"""Shared helpers of the test-suite: small models and result comparison."""
import numpy as np
import torch

import datasets as testing

METRIC_CODES = {"sqeuclidean": 0, "euclidean": 1, "cosine": 2, "inner_product": 6}
KIND_CODES = {"subspace": 0, "cluster": 1}


def make_data(n, dim, dtype, seed, n_components=16):
    """Clustered data in the element type under test."""
    rng = np.random.default_rng(seed)
    cent = rng.standard_normal((n_components, dim)).astype(np.float32)
    x = cent[rng.integers(0, n_components, n)] + 0.3 * rng.standard_normal((n, dim)).astype(np.float32)
    if dtype == np.uint8:
        return np.clip(np.round(x * 30 + 100), 0, 255).astype(np.uint8)
    if dtype == np.int8:
        return np.clip(np.round(x * 30), -128, 127).astype(np.int8)
    return x.astype(dtype)


def uniform_data(n, dim, seed):
    """The distribution the reference's own tests use: uniform [0.1, 2.0)
    (cpp/tests/neighbors/ann_ivf_pq.cuh:150-168)."""
    rng = np.random.default_rng(seed)
    return rng.uniform(0.1, 2.0, (n, dim)).astype(np.float32)


def train(data, n_lists, pq_dim, pq_bits, metric="sqeuclidean", codebook_kind="subspace",
          force_random_rotation=False, seed=137, iters=8):
    """Model tensors as numpy arrays (trained on the CPU)."""
    x = torch.from_numpy(np.ascontiguousarray(data))
    m = testing.train_model(x, n_lists, pq_dim, pq_bits, metric=metric, codebook_kind=codebook_kind,
                            kmeans_iters=iters, pq_iters=iters, seed=seed,
                            force_random_rotation=force_random_rotation)
    return {k: v.numpy() for k, v in m.items()}


def oracle_index(orc, model, dim, pq_dim, pq_bits, metric="sqeuclidean", codebook_kind="subspace"):
    return orc.Index(METRIC_CODES[metric], KIND_CODES[codebook_kind], dim, pq_dim, pq_bits,
                     model["centers"], model["centers_rot"], model["rotation_matrix"],
                     model["pq_centers"])


def oracle_index_with_data(orc, model, data, pq_dim, pq_bits, metric="sqeuclidean",
                           codebook_kind="subspace", ids=None):
    ix = oracle_index(orc, model, data.shape[1], pq_dim, pq_bits, metric, codebook_kind)
    labels, codes = orc.encode(ix, data)
    ix.fill(labels, codes, ids)
    return ix, labels, codes


def to_float(x):
    if x.dtype == np.uint8:
        return x.astype(np.float32) / np.float32(256)
    if x.dtype == np.int8:
        return x.astype(np.float32) / np.float32(128)
    return x.astype(np.float32)


def decode_rows(model, labels, codes, pq_bits, codebook_kind="subspace"):
    """Reconstruct rotated-space vectors: centre_rot[label] + codebook entries
    (cuVS reconstruct: cpp/src/neighbors/ivf_pq/ivf_pq_build.cuh:555-570)."""
    pqc = model["pq_centers"].astype(np.float64)
    n, pq_dim = codes.shape
    pq_len = pqc.shape[1]
    out = model["centers_rot"][labels].astype(np.float64).copy()
    for j in range(pq_dim):
        book = pqc[labels] if codebook_kind == "cluster" else pqc[j][None].repeat(n, 0)
        out[:, j * pq_len:(j + 1) * pq_len] += book[np.arange(n), :, codes[:, j]]
    return out


def compare_results(got_ids, got_d, want_ids, want_d, rtol, exact=False):
    """ids equal except at (near-)ties of the expected distances; distances within rtol."""
    got_ids, want_ids = np.asarray(got_ids), np.asarray(want_ids)
    got_d, want_d = np.asarray(got_d, dtype=np.float64), np.asarray(want_d, dtype=np.float64)
    assert got_ids.shape == want_ids.shape and got_d.shape == want_d.shape
    if exact:
        assert np.array_equal(got_ids, want_ids), "neighbour ids differ"
        assert np.array_equal(got_d.astype(np.float32), want_d.astype(np.float32)), "distances differ"
        return 0
    finite = np.isfinite(want_d) & np.isfinite(got_d)
    assert np.array_equal(np.isfinite(want_d), np.isfinite(got_d))
    scale = np.maximum(np.abs(want_d), 1e-30)
    err = np.abs(got_d - want_d) / scale
    assert np.all(err[finite] <= rtol), f"max relative distance error {err[finite].max():.3e} > {rtol}"
    mism = got_ids != want_ids
    n_mism = int(mism.sum())
    if n_mism:
        # a differing id is acceptable only where the expected distances tie within rtol:
        # the row must still hold the same multiset of distances (checked above) and every id
        # that moved must have a neighbour at (nearly) the same distance
        for q, r in zip(*np.nonzero(mism)):
            row = want_d[q]
            others = np.delete(row, r)
            gap = np.min(np.abs(others - row[r])) / max(abs(row[r]), 1e-30) if others.size else 0.0
            boundary = r == row.shape[0] - 1
            assert gap <= max(rtol, 1e-5) or boundary, (
                f"query {q} rank {r}: id {got_ids[q, r]} != {want_ids[q, r]} without a distance tie")
    return n_mism
