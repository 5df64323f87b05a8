"""Mirror of ``cuvs.neighbors.refine`` (python/cuvs/cuvs/neighbors/refine.pyx:34-160)."""
from . import dlpack
from ._lib import check, lib
from .ivf_pq import _prep, _torch

# cuvsDistanceType values (c/include/cuvs/distance/distance.h:15-60)
REFINE_METRICS = {"sqeuclidean": 0, "euclidean": 1, "inner_product": 6}


def refine(dataset, queries, candidates, k=None, metric="sqeuclidean", indices=None,
           distances=None, resources=None):
    """Exact distances between every query and its candidates; the ``k`` nearest are returned as
    ``(distances, indices)``.  ``k`` may be left out when ``indices`` or ``distances`` is given."""
    torch = _torch()
    res, own = _prep(resources)
    if k is None:
        if indices is not None:
            k = indices.shape[1]
        elif distances is not None:
            k = distances.shape[1]
        else:
            raise ValueError("Argument k must be specified if both indices and distances arg is None")
    if metric not in REFINE_METRICS:
        raise ValueError("metric %s is not supported" % metric)
    n_queries = queries.shape[0]
    if indices is None:
        indices = torch.empty((n_queries, k), dtype=torch.int64, device="cuda")
    if distances is None:
        distances = torch.empty((n_queries, k), dtype=torch.float32, device="cuda")
    dv, qv, cv = dlpack.view(dataset), dlpack.view(queries), dlpack.view(candidates)
    iv, ov = dlpack.view(indices), dlpack.view(distances)
    check(lib().cuvsRefine(res.get_c_obj(), dv.ptr, qv.ptr, cv.ptr, REFINE_METRICS[metric], iv.ptr,
                           ov.ptr))
    if own:
        res.sync()
    return distances, indices
