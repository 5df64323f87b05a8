"""Mirror of ``cuvs.neighbors.refine`` (python/cuvs/cuvs/neighbors/refine.pyx:34-160)."""
import numpy as np

from . import dlpack
from ._lib import check, lib
from .ivf_pq import _prep, _torch

# cuvsDistanceType values (c/include/cuvs/distance/distance.h:15-60)
REFINE_METRICS = {"sqeuclidean": 0, "euclidean": 1, "inner_product": 6}


def refine(dataset, queries, candidates, k=None, metric="sqeuclidean", indices=None,
           distances=None, resources=None):
    """Exact distances between every query and its candidates; the ``k`` nearest are returned as
    ``(distances, indices)``.  ``k`` may be left out when ``indices`` or ``distances`` is given.
    The matrices are either all on the device or all in host memory (the reference takes both)."""
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
    # outputs live where the dataset does: matrices in host memory (numpy arrays, CPU tensors) are
    # staged through the device by the library and come back in host memory
    if isinstance(dataset, np.ndarray):
        if indices is None:
            indices = np.empty((n_queries, k), dtype=np.int64)
        if distances is None:
            distances = np.empty((n_queries, k), dtype=np.float32)
    else:
        where = "cuda" if dataset.is_cuda else "cpu"
        if indices is None:
            indices = torch.empty((n_queries, k), dtype=torch.int64, device=where)
        if distances is None:
            distances = torch.empty((n_queries, k), dtype=torch.float32, device=where)
    dv, qv, cv = dlpack.view(dataset), dlpack.view(queries), dlpack.view(candidates)
    iv, ov = dlpack.view(indices), dlpack.view(distances)
    check(lib().cuvsRefine(res.get_c_obj(), dv.ptr, qv.ptr, cv.ptr, REFINE_METRICS[metric], iv.ptr,
                           ov.ptr))
    if own:
        res.sync()
    return distances, indices
