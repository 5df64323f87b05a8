"""Concurrent searches: one resources handle (stream + workspace) per thread against one shared index,
the threading contract of the reference (a handle is not thread-safe, a built index is read-only)."""
import threading

import numpy as np
import pytest
import torch

from cuvs_amd import ivf_pq, testing
from cuvs_amd.resources import Resources

pytestmark = pytest.mark.gpu


def test_four_threads_share_an_index():
    n, dim, nq = 200000, 64, 3000
    allrows = testing.gaussian_mixture(n + nq, dim, 100, 0.2, seed=9, device="cuda")
    data, queries = allrows[:n], allrows[n:].contiguous()
    index = ivf_pq.build(ivf_pq.IndexParams(n_lists=512, pq_dim=32, kmeans_trainset_fraction=0.3), data)
    variants = [dict(n_probes=16, lut_dtype=np.float16), dict(n_probes=32, lut_dtype=np.uint8),
                dict(n_probes=8, lut_dtype=np.float32), dict(n_probes=64, lut_dtype=np.float16)]
    want = []
    for v in variants:
        d, nb = ivf_pq.search(ivf_pq.SearchParams(**v), index, queries, 10)
        torch.cuda.synchronize()
        want.append((d.clone(), nb.clone()))
    errors = []

    def worker(i):
        try:
            stream = torch.cuda.Stream()
            res = Resources()
            res.set_stream(stream.cuda_stream)
            sp = ivf_pq.SearchParams(**variants[i])
            with torch.cuda.stream(stream):
                for _ in range(20):
                    d, nb = ivf_pq.search(sp, index, queries, 10, resources=res)
                    res.sync()
                    if not (torch.equal(d, want[i][0]) and torch.equal(nb, want[i][1])):
                        errors.append(f"thread {i}: results differ")
                        return
        except Exception as e:  # noqa: BLE001
            errors.append(f"thread {i}: {e!r}")

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
