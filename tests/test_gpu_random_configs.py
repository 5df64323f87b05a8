"""Seeded random configurations of the search path against the CPU oracle on the same index.

Each case draws code width, subspace shape (with and without a padded rotated dimension), metric,
codebook kind, element type, sizes, table / accumulator types, k, probe count, an optional bitset
filter and the number of extend calls, builds the index through the C ABI, and compares with the
oracle: the stored lists and `transform` against the oracle's encoding of the same rows (labels
and codes), ids and distances of a search bit for bit (except for the square-root metric, whose
ids may swap at equal distances), and a saved and reloaded index against the original.  The fixed
cases of test_gpu_parity.py aim at particular kernels and edges; these cover the combinations
nobody thought of.
"""
import os
import tempfile

import numpy as np
import pytest
import torch

import gpu_helpers as G
import helpers as H
from cuvs_amd import ivf_pq

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
