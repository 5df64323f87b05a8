"""Merge of per-shard search results (cuvs::neighbors::knn_merge_parts,
cpp/include/cuvs/neighbors/knn_merge_parts.hpp:36-100; no Python binding in the reference)."""
from . import dlpack
from ._lib import check, lib
from .ivf_pq import _prep, _torch


def knn_merge_parts(in_keys, in_ids, translations, k=None, out_keys=None, out_ids=None, resources=None):
    """``in_keys`` float32 / ``in_ids`` int64 of shape [n_parts * n_samples, k] (part-major),
    ``translations`` int64 [n_parts]: returns ``(out_keys, out_ids)`` of shape [n_samples, k] with the
    k smallest keys of every row over all parts, ids shifted by their part's translation."""
    torch = _torch()
    res, own = _prep(resources)
    n_parts = translations.shape[0]
    n_samples = in_keys.shape[0] // n_parts
    k = in_keys.shape[1] if k is None else k
    if out_keys is None:
        out_keys = torch.empty((n_samples, k), dtype=torch.float32, device="cuda")
    if out_ids is None:
        out_ids = torch.empty((n_samples, k), dtype=torch.int64, device="cuda")
    views = [dlpack.view(t) for t in (in_keys, in_ids, translations, out_keys, out_ids)]
    check(lib().cuvsAmdKnnMergeParts(res.get_c_obj(), *[v.ptr for v in views]))
    if own:
        res.sync()
    return out_keys, out_ids
