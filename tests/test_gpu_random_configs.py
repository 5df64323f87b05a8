"""Seeded random configurations of the search path against the CPU oracle on the same index.

Each case draws code width, subspace shape (with and without a padded rotated dimension), metric,
codebook kind, element type, sizes, table / accumulator types, k, probe count, an optional bitset
filter and the number of extend calls, builds the index through the C ABI, and compares with the
oracle: the stored lists and `transform` against the oracle's encoding of the same rows (labels
and codes), ids and distances of a search bit for bit (except for the square-root metric, whose
ids may swap at equal distances), and a saved and reloaded index against the original.  The fixed
cases of test_gpu_parity.py aim at particular kernels and edges; these cover the combinations
nobody thought of.

A second family draws larger cases on clustered rows (30,000 to 160,000 rows, up to 900 lists and
1,200 queries, the subspace shapes of the CU-wide and slab kernels among them) with the early stop
forced on, left to the library or switched off, internal batches of 100 to 4096 queries, and checks
the oracle's answer bit for bit and that the answer does not depend on the early stop.
"""
import os
import tempfile

import numpy as np
import pytest
import torch

import datasets as testing
import gpu_helpers as G
import helpers as H
from cuvs_amd import ivf_pq
from cuvs_amd.resources import Resources

pytestmark = pytest.mark.gpu

R_32F, R_16F, R_8U = 0, 2, 8
ORC_DT = {R_32F: 0, R_16F: 2, R_8U: 8}


def _run(orc, seed):
    rng = np.random.default_rng(seed)
    pq_bits = int(rng.choice([4, 5, 6, 7, 8], p=[0.3, 0.1, 0.1, 0.1, 0.4]))
    pq_len = int(rng.choice([1, 2, 4, 3]))
    while True:
        pq_dim = int(rng.choice([8, 16, 24, 32, 40, 48, 64, 96, 128, 160]))
        if (pq_dim * pq_bits) % 8 == 0:
            break
    exact_dim = rng.random() < 0.7
    dim = pq_dim * pq_len if exact_dim else max(2, pq_dim * pq_len - int(rng.integers(1, pq_len + 1)))
    if dim > 512:
        dim, pq_len = pq_dim, 1
    metric = str(rng.choice(["sqeuclidean", "euclidean", "inner_product", "cosine"]))
    kind = str(rng.choice(["subspace", "cluster"]))
    dtype = [np.float32, np.float16, np.int8, np.uint8][int(rng.integers(0, 4))]
    n = int(rng.choice([1500, 6000, 20000, 50000]))
    n_lists = int(rng.choice([3, 10, 40, 150, 400]))
    nq = int(rng.choice([1, 7, 40, 130, 300]))
    lut, internal = [(R_32F, R_32F), (R_16F, R_32F), (R_8U, R_32F), (R_16F, R_16F), (R_8U, R_16F)][int(rng.integers(0, 5))]
    k = int(rng.choice([1, 5, 10, 33, 64, 100, 128, 200, 300]))
    n_probes = int(min(n_lists, rng.choice([1, 2, 5, 20, 60, 150])))
    use_filter = rng.random() < 0.25
    batches = int(rng.choice([1, 1, 3]))
    desc = dict(seed=seed, bits=pq_bits, pq_dim=pq_dim, dim=dim, metric=metric, kind=kind, dtype=np.dtype(dtype).name,
                n=n, lists=n_lists, nq=nq, lut=lut, internal=internal, k=k, probes=n_probes, filt=use_filter,
                batches=batches)
    print(desc, flush=True)
    data = H.make_data(n, dim, dtype, seed)
    queries = H.make_data(nq, dim, dtype, seed + 1)
    model = H.train(data, n_lists, pq_dim, pq_bits, metric=metric, codebook_kind=kind, iters=3,
                    force_random_rotation=bool(rng.random() < 0.2))
    index = G.build_gpu_index(model, data, pq_dim, pq_bits, metric, kind, batches=batches)
    ix, gpu_codes = G.read_back(orc, index, model, dim, pq_dim, pq_bits, metric, kind)
    # the stored lists are the oracle's encoding of the rows
    labels, codes = orc.encode(ix, data)
    sizes = index.list_sizes.cpu().numpy()
    assert np.array_equal(np.bincount(labels, minlength=n_lists), sizes), "list sizes differ from the oracle's labels"
    for l in range(0, n_lists, max(1, n_lists // 7)):
        order = np.argsort(ix.list_inds[l])
        assert np.array_equal(ix.list_inds[l][order], np.nonzero(labels == l)[0]), f"list {l}: members differ"
        assert np.array_equal(gpu_codes[l][order], codes[labels == l]), f"list {l}: codes differ"
    # transform gives the same labels and codes, bit-contiguous
    tl, tc = ivf_pq.transform(index, G.to_dev(data[:500]))
    assert np.array_equal(tl.cpu().numpy().view(np.uint32), labels[:500].astype(np.uint32)), "transform labels"
    assert np.array_equal(G.unpack_bits(tc.cpu().numpy(), pq_dim, pq_bits), codes[:500]), "transform codes"
    # a saved and reloaded index answers identically
    path = os.path.join(tempfile.gettempdir(), f"fuzz_{seed}.bin")
    ivf_pq.save(path, index)
    reloaded = ivf_pq.load(path)
    os.remove(path)
    kk = min(k, n)
    sp = ivf_pq.SearchParams(n_probes=n_probes, lut_dtype=lut, internal_distance_dtype=internal)
    kw, okw = {}, {}
    if use_filter:
        keep = rng.random(n) < 0.6
        bits = np.packbits(keep, bitorder="little")
        bits = np.concatenate([bits, np.zeros((-bits.size) % 4, dtype=np.uint8)]).view(np.uint32)
        kw = dict(filter_bitset=G.to_dev(bits.view(np.int32)), filter_nbits=n)
        okw = dict(filter_bitset=bits, filter_nbits=n)
    d, nb = ivf_pq.search(sp, index, G.to_dev(queries), kk, **kw)
    torch.cuda.synchronize()
    want_nb, want_d = orc.search(ix, queries, kk, n_probes, lut_dtype=ORC_DT[lut],
                                 internal_distance_dtype=ORC_DT[internal], **okw)
    H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 1e-5 if lut == R_32F else 2e-3,
                      exact=(metric != "euclidean"))
    d2, nb2 = ivf_pq.search(sp, reloaded, G.to_dev(queries), kk, **kw)
    torch.cuda.synchronize()
    assert torch.equal(d, d2) and torch.equal(nb, nb2), "reloaded index answers differently"


# 9126 and 9188: cosine indexes where a row's nearest centre differs between the normalised row and
# the row as it is by an fp32 rounding (labels must be those of the normalised row)
@pytest.mark.parametrize("seed", list(range(7000, 7032)) + [9126, 9188])
def test_random_configuration_matches_oracle(orc, seed):
    _run(orc, seed)


_SHAPES = [(64, 2), (48, 2), (32, 4), (32, 2), (128, 2), (96, 1), (64, 1), (192, 2), (384, 2), (16, 4), (40, 2),
           (128, 1), (64, 4), (24, 8), (96, 2), (256, 1), (64, 3), (72, 2), (512, 2), (256, 2)]
_NP_DT = {R_32F: np.float32, R_16F: np.float16, R_8U: np.uint8}


def _run_larger(orc, seed):
    rng = np.random.default_rng(seed)
    pq_bits = int(rng.choice([8, 4, 5, 6, 7], p=[0.55, 0.25, 0.07, 0.07, 0.06]))
    while True:
        pq_dim, pq_len = _SHAPES[int(rng.integers(0, len(_SHAPES)))]
        if (pq_dim * pq_bits) % 8 == 0:
            break
    dim = pq_dim * pq_len - (int(rng.integers(1, pq_len + 1)) if (pq_len > 1 and rng.random() < 0.2) else 0)
    metric = str(rng.choice(["sqeuclidean", "euclidean", "inner_product", "cosine"], p=[0.45, 0.1, 0.3, 0.15]))
    kind = str(rng.choice(["subspace", "cluster"], p=[0.75, 0.25]))
    dtype = [np.float32, np.float16, np.int8, np.uint8][int(rng.integers(0, 4))]
    n = int(rng.choice([30000, 80000, 160000]))
    if dim >= 512:
        n = min(n, 80000)
    n_lists = int(rng.choice([64, 160, 400, 900]))
    nq = int(rng.choice([50, 300, 1200]))
    lut, internal = [(R_32F, R_32F), (R_16F, R_32F), (R_8U, R_32F), (R_16F, R_16F), (R_8U, R_16F)][int(rng.integers(0, 5))]
    k = int(rng.choice([1, 10, 10, 40, 64, 100, 128, 130, 256]))
    n_probes = min(int(rng.choice([3, 8, 16, 32, 64, 100])), n_lists)
    early_stop = str(rng.choice(["on", "auto", "off"], p=[0.6, 0.3, 0.1]))
    batch = int(rng.choice([4096, 4096, 256, 100]))
    use_filter = rng.random() < 0.2
    sigma = float(rng.choice([0.05, 0.12, 0.3]))
    normalize = metric in ("inner_product", "cosine") and rng.random() < 0.7
    print(dict(seed=seed, bits=pq_bits, pq_dim=pq_dim, pq_len=pq_len, dim=dim, metric=metric, kind=kind,
               dtype=np.dtype(dtype).name, n=n, lists=n_lists, nq=nq, lut=lut, internal=internal, k=k, probes=n_probes,
               early_stop=early_stop, batch=batch, filt=use_filter, sigma=sigma, norm=normalize), flush=True)
    x = testing.gaussian_mixture(n + nq, dim, 64, sigma, seed=seed, normalize_rows=normalize).numpy()
    if dtype in (np.uint8, np.int8):
        lo, hi = x.min(), x.max()
        x = (np.clip(np.round((x - lo) / (hi - lo) * 255), 0, 255) if dtype == np.uint8
             else np.clip(np.round((x - lo) / (hi - lo) * 254 - 127), -127, 127))
    x = x.astype(dtype)
    data, q = x[:n], x[n:]
    model = H.train(data, n_lists, pq_dim, pq_bits, metric=metric, codebook_kind=kind, iters=3,
                    force_random_rotation=bool(rng.random() < 0.15))
    index = G.build_gpu_index(model, data, pq_dim, pq_bits, metric, kind)
    ix, _ = G.read_back(orc, index, model, dim, pq_dim, pq_bits, metric, kind)
    res = Resources()
    res.set_search_tuning(early_stop=early_stop)
    sp = ivf_pq.SearchParams(n_probes=n_probes, lut_dtype=_NP_DT[lut], internal_distance_dtype=_NP_DT[internal],
                             max_internal_batch_size=batch)
    kw, okw = {}, {}
    if use_filter:
        keep = rng.random(n) < 0.6
        bits = np.packbits(keep, bitorder="little")
        bits = np.concatenate([bits, np.zeros((-bits.size) % 4, dtype=np.uint8)]).view(np.uint32)
        kw = dict(filter_bitset=G.to_dev(bits.view(np.int32)), filter_nbits=n)
        okw = dict(filter_bitset=bits, filter_nbits=n)
    kk = min(k, n)
    d, nb = ivf_pq.search(sp, index, G.to_dev(q), kk, resources=res, **kw)
    res.sync()
    want_nb, want_d = orc.search(ix, q, kk, n_probes, lut_dtype=ORC_DT[lut], internal_distance_dtype=ORC_DT[internal],
                                 **okw)
    H.compare_results(nb.cpu().numpy(), d.cpu().numpy(), want_nb, want_d, 1e-5 if lut == R_32F else 2e-3,
                      exact=(metric != "euclidean"))
    res.set_search_tuning(early_stop="off" if early_stop != "off" else "on")
    d2, nb2 = ivf_pq.search(sp, index, G.to_dev(q), kk, resources=res, **kw)
    res.sync()
    if metric != "euclidean":
        assert torch.equal(nb, nb2) and torch.equal(d, d2), "the answer depends on the early stop"


# (30002, 30006, 30011, 30020 and 30021 pass as well and take 9 - 15 s each: left out to keep the suite short)
@pytest.mark.parametrize("seed", [s for s in range(30000, 30024) if s not in (30002, 30006, 30011, 30020, 30021)])
def test_random_larger_configuration_matches_oracle(orc, seed):
    _run_larger(orc, seed)
