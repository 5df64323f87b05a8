"""Concurrent searches: one resources handle (stream + workspace) per thread against one shared index,
the threading contract of the reference (a handle is not thread-safe, a built index is read-only)."""
import threading

import numpy as np
import pytest
import torch

import datasets as testing

from cuvs_amd import ivf_pq
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


def test_threads_make_the_first_call_of_their_variant():
    """Per-kernel launch state (LDS limits, occupancy) is set up by whichever thread comes first:
    four threads start together, each with a kernel variant this process has not launched yet
    (inner product, 48 subspaces: other tests search such an index with L2 only), and their results
    must equal what the main thread computes afterwards."""
    n, dim, nq = 100000, 96, 2000
    allrows = testing.gaussian_mixture(n + nq, dim, 100, 0.2, seed=19, device="cuda")
    data, queries = allrows[:n], allrows[n:].contiguous()
    index = ivf_pq.build(ivf_pq.IndexParams(n_lists=256, pq_dim=48, metric="inner_product",
                                            kmeans_trainset_fraction=0.3), data)
    torch.cuda.synchronize()
    variants = [dict(n_probes=16, lut_dtype=np.float16), dict(n_probes=16, lut_dtype=np.uint8),
                dict(n_probes=16, lut_dtype=np.float16, internal_distance_dtype=np.float16),
                dict(n_probes=16, lut_dtype=np.uint8, internal_distance_dtype=np.float16)]
    got, errors = [None] * 4, []
    gate = threading.Barrier(4)

    def worker(i):
        try:
            stream = torch.cuda.Stream()
            res = Resources()
            res.set_stream(stream.cuda_stream)
            sp = ivf_pq.SearchParams(**variants[i])
            with torch.cuda.stream(stream):
                gate.wait(timeout=60)
                d, nb = ivf_pq.search(sp, index, queries, 10, resources=res)
                res.sync()
            got[i] = (d, nb)
        except Exception as e:  # noqa: BLE001
            errors.append(f"thread {i}: {e!r}")

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i, v in enumerate(variants):
        d, nb = ivf_pq.search(ivf_pq.SearchParams(**v), index, queries, 10)
        torch.cuda.synchronize()
        assert torch.equal(d, got[i][0]) and torch.equal(nb, got[i][1]), i


def test_switching_streams_keeps_calls_on_one_handle_ordered():
    """Two searches on one handle share its workspace.  The second is queued on another stream
    right after the first, without a synchronisation in between: the handle makes the new stream
    wait for the work still queued on the previous one, so both give the sequential results."""
    n, dim, nq = 200000, 64, 8000
    allrows = testing.gaussian_mixture(n + 2 * nq, dim, 100, 0.2, seed=29, device="cuda")
    data, qa, qb = allrows[:n], allrows[n:n + nq].contiguous(), allrows[n + nq:].contiguous()
    index = ivf_pq.build(ivf_pq.IndexParams(n_lists=512, pq_dim=32, kmeans_trainset_fraction=0.3), data)
    res = Resources()
    sp = ivf_pq.SearchParams(n_probes=64, lut_dtype=np.float16, max_internal_batch_size=nq)
    want_a = ivf_pq.search(sp, index, qa, 10, resources=res)
    want_b = ivf_pq.search(sp, index, qb, 10, resources=res)
    res.sync()
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    out = [(torch.empty((nq, 10), dtype=torch.float32, device="cuda"),
            torch.empty((nq, 10), dtype=torch.int64, device="cuda")) for _ in range(2)]
    for rep in range(5):
        for o in out:
            o[0].zero_(), o[1].zero_()
        torch.cuda.synchronize()
        res.set_stream(s1.cuda_stream)
        ivf_pq.search(sp, index, qa, 10, neighbors=out[0][1], distances=out[0][0], resources=res)
        res.set_stream(s2.cuda_stream)
        ivf_pq.search(sp, index, qb, 10, neighbors=out[1][1], distances=out[1][0], resources=res)
        torch.cuda.synchronize()
        assert torch.equal(out[0][0], want_a[0]) and torch.equal(out[0][1], want_a[1]), rep
        assert torch.equal(out[1][0], want_b[0]) and torch.equal(out[1][1], want_b[1]), rep
    res.set_stream(torch.cuda.current_stream().cuda_stream)
