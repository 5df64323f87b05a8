"""The library's device memory sources under real use: an index filled, searched and destroyed while
the process draws from a pool (or the stream-ordered allocator) holds the lists and gives the answers
it gives on plain allocations, memory taken from a pool survives the switch back, the trainer runs on
pooled memory, and a handle's own pool serves its search workspace."""
import numpy as np
import pytest
import torch

import gpu_helpers as G
import helpers as H
import datasets as testing
from cuvs_amd import ivf_pq, resources
from cuvs_amd.resources import Resources

pytestmark = pytest.mark.gpu

N, DIM, NQ, LISTS, PQ_DIM = 40000, 64, 500, 100, 32


@pytest.fixture(scope="module")
def workload():
    data = H.make_data(N, DIM, np.float32, 31)
    queries = H.make_data(NQ, DIM, np.float32, 32)
    model = H.train(data, LISTS, PQ_DIM, 8, iters=3)
    return data, G.to_dev(queries), model


def _fill_and_search(data, queries, model, n_probes=16):
    """Deterministic given the model: lists filled in three batches, then one search."""
    index = G.build_gpu_index(model, data, PQ_DIM, 8, batches=3)
    d, nb = ivf_pq.search(ivf_pq.SearchParams(n_probes=n_probes), index, queries, 10)
    torch.cuda.synchronize()
    return index, d.clone(), nb.clone()


def _lists(index):
    """Members and codes of every list, in the order of the source indices (the order inside a list is
    the order in which the rows of a batch claimed their slots)."""
    out = []
    for ids, codes in index.lists():
        ids, codes = ids.cpu().numpy(), codes.cpu().numpy()
        order = np.argsort(ids, kind="stable")
        out.append((ids[order], codes[order]))
    return out


def _same_lists(a, b):
    return len(a) == len(b) and all(np.array_equal(x[0], y[0]) and np.array_equal(x[1], y[1])
                                    for x, y in zip(a, b))


def test_index_life_cycle_on_a_process_wide_pool(workload):
    data, queries, model = workload
    plain, want_d, want_nb = _fill_and_search(data, queries, model)
    want_lists = _lists(plain)
    del plain
    resources.pool_memory_resource_enable(2, 60)
    try:
        # twice: the second index lives in ranges the first one gave back, not in fresh memory
        for _ in range(2):
            index, d, nb = _fill_and_search(data, queries, model)
            assert torch.equal(nb, want_nb) and torch.equal(d, want_d)
            assert _same_lists(_lists(index), want_lists)
        # the library's own trainer on pooled memory
        rows = G.to_dev(data)
        trained = ivf_pq.build(ivf_pq.IndexParams(n_lists=LISTS, pq_dim=PQ_DIM, kmeans_trainset_fraction=0.5), rows)
        _, nb_t = ivf_pq.search(ivf_pq.SearchParams(n_probes=LISTS), trained, queries, 10)
        exact = torch.cdist(queries, rows).topk(10, largest=False).indices
        hits = sum(len(set(a.tolist()) & set(b.tolist())) for a, b in zip(nb_t.cpu(), exact.cpu()))
        assert hits / (NQ * 10) > 0.7
        del trained
    finally:
        resources.memory_resource_reset()
    # the index still lives in the retired pool: it answers, grows and goes away cleanly
    d, nb = ivf_pq.search(ivf_pq.SearchParams(n_probes=16), index, queries, 10)
    torch.cuda.synchronize()
    assert torch.equal(nb, want_nb) and torch.equal(d, want_d)
    extra = torch.arange(N, N + 1000, dtype=torch.int64, device="cuda")
    ivf_pq.extend(index, G.to_dev(data[:1000]), extra)
    assert len(index) == N + 1000
    del index
    _, d, nb = _fill_and_search(data, queries, model)
    assert torch.equal(nb, want_nb) and torch.equal(d, want_d)


def test_index_life_cycle_on_the_stream_ordered_allocator(workload):
    data, queries, model = workload
    _, want_d, want_nb = _fill_and_search(data, queries, model)
    resources.async_memory_resource_enable()
    try:
        index, d, nb = _fill_and_search(data, queries, model)
    finally:
        resources.memory_resource_reset()
    assert torch.equal(nb, want_nb) and torch.equal(d, want_d)
    del index


def test_search_workspace_out_of_the_handles_own_pool(workload):
    data, queries, model = workload
    index, want_d, want_nb = _fill_and_search(data, queries, model)
    res = Resources()
    res.use_torch_current_stream()
    res.set_workspace_pool(512 << 20)
    wants = {}
    for n_probes in (16, 64):
        wants[n_probes] = ivf_pq.search(ivf_pq.SearchParams(n_probes=n_probes), index, queries, 10)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for n_probes, want in wants.items():
        got = ivf_pq.search(ivf_pq.SearchParams(n_probes=n_probes), index, queries, 10, resources=res)
        res.sync()
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
    # the workspaces of both searches fit the reservation: the device gave nothing more to the handle
    assert free_before - torch.cuda.mem_get_info()[0] < (64 << 20)
    # a second reservation replaces the first
    res.set_workspace_pool(64 << 20)
    got = ivf_pq.search(ivf_pq.SearchParams(n_probes=16), index, queries, 10, resources=res)
    res.sync()
    assert torch.equal(got[0], want_d) and torch.equal(got[1], want_nb)


def test_memory_tracking_writes_csv(tmp_path, workload):
    """The reference's own test of the tracking handle (python/cuvs/cuvs/tests/test_memory_tracking.py:
    the file exists, is not empty and starts with a header), plus what the rows must say."""
    import time
    data, queries, model = workload
    csv = tmp_path / "alloc.csv"
    res = Resources(memory_tracking_csv_path=str(csv), memory_tracking_sample_interval_ms=2)
    assert csv.read_text().startswith("elapsed_ms,device_current_bytes,device_peak_bytes")  # flushed at once
    from cuvs_amd._lib import CuvsError
    with pytest.raises(CuvsError, match="already active"):
        Resources(memory_tracking_csv_path=str(tmp_path / "second.csv"))
    try:
        index, d, nb = _fill_and_search(data, queries, model)
        time.sleep(0.05)
        arena_bytes = sum(((s + 31) // 32) * 32 for s in index.list_sizes.cpu().tolist()) * (PQ_DIM + 8)
        del index
        time.sleep(0.05)
    finally:
        del res
    rows = [line.split(",") for line in csv.read_text().splitlines()]
    assert rows[0][0] == "elapsed_ms" and len(rows) >= 3
    body = [[float(v) for v in r] for r in rows[1:]]
    assert all(len(r) == 7 for r in body)
    times = [r[0] for r in body]
    assert times == sorted(times)
    assert all(b - a >= 1.9 for a, b in zip(times[:-2], times[1:-1]))  # at least the interval apart
    peak = max(r[2] for r in body)
    assert peak >= arena_bytes  # the codes and ids of the lists were live at some point
    last = body[-1]
    assert last[5] >= last[6] > 0 and last[2] == peak
    # what the index held is gone; the default handle's workspace may still be there
    assert last[1] < peak
