"""Mirror of ``cuvs.neighbors.ivf_pq`` (python/cuvs/cuvs/neighbors/ivf_pq/ivf_pq.pyx) over the C ABI.

Same class and function names, keyword arguments and defaults: IndexParams (:134-147),
SearchParams (:704-707), build_precomputed (:543), extend (:913), search (:745-840, returns
``(distances, neighbors)``), transform (:987).  Inputs are torch tensors on the GPU (or numpy
arrays where the C API accepts host memory); outputs are torch tensors.
"""
import ctypes as C

import numpy as np

from . import dlpack
from ._lib import (IndexParamsStruct, IndexStruct, SearchParamsStruct, SearchProfileStruct,
                   check, lib)
from .resources import Resources

DISTANCE_TYPES = {"sqeuclidean": 0, "euclidean": 1, "cosine": 2, "inner_product": 6}
CUDA_R_32F, CUDA_R_16F, CUDA_R_8I, CUDA_R_8U = 0, 2, 3, 8


def _map_dtype_np_to_cuda(dt):
    """python/cuvs/cuvs/neighbors/ivf_pq/ivf_pq.pyx: _map_dtype_np_to_cuda"""
    if isinstance(dt, int):
        return dt
    dt = np.dtype(dt)
    table = {np.dtype(np.float32): CUDA_R_32F, np.dtype(np.float16): CUDA_R_16F,
             np.dtype(np.int8): CUDA_R_8I, np.dtype(np.uint8): CUDA_R_8U}
    if dt not in table:
        raise TypeError("Type %s is not supported" % str(dt))
    return table[dt]


class IndexParams:
    def __init__(self, *, n_lists=1024, metric="sqeuclidean", metric_arg=2.0, kmeans_n_iters=20,
                 kmeans_trainset_fraction=0.5, pq_bits=8, pq_dim=0, codebook_kind="subspace",
                 force_random_rotation=False, add_data_on_build=True,
                 conservative_memory_allocation=False, max_train_points_per_pq_code=256,
                 codes_layout="interleaved"):
        self._p = C.POINTER(IndexParamsStruct)()
        check(lib().cuvsIvfPqIndexParamsCreate(C.byref(self._p)))
        p = self._p.contents
        p.n_lists = n_lists
        p.metric = DISTANCE_TYPES[metric]
        p.metric_arg = metric_arg
        p.kmeans_n_iters = kmeans_n_iters
        p.kmeans_trainset_fraction = kmeans_trainset_fraction
        p.pq_bits = pq_bits
        p.pq_dim = pq_dim
        if codebook_kind == "subspace":
            p.codebook_kind = 0
        elif codebook_kind == "cluster":
            p.codebook_kind = 1
        else:
            raise ValueError("Incorrect codebook kind %s" % codebook_kind)
        p.force_random_rotation = force_random_rotation
        p.add_data_on_build = add_data_on_build
        p.conservative_memory_allocation = conservative_memory_allocation
        p.max_train_points_per_pq_code = max_train_points_per_pq_code
        if codes_layout == "flat":
            p.codes_layout = 0
        elif codes_layout == "interleaved":
            p.codes_layout = 1
        else:
            raise ValueError("Incorrect codes layout %s" % codes_layout)
        self.metric = metric

    n_lists = property(lambda self: self._p.contents.n_lists)
    metric_arg = property(lambda self: self._p.contents.metric_arg)
    kmeans_n_iters = property(lambda self: self._p.contents.kmeans_n_iters)
    kmeans_trainset_fraction = property(lambda self: self._p.contents.kmeans_trainset_fraction)
    pq_bits = property(lambda self: self._p.contents.pq_bits)
    pq_dim = property(lambda self: self._p.contents.pq_dim)
    force_random_rotation = property(lambda self: bool(self._p.contents.force_random_rotation))
    add_data_on_build = property(lambda self: bool(self._p.contents.add_data_on_build))
    conservative_memory_allocation = property(lambda self: bool(self._p.contents.conservative_memory_allocation))
    max_train_points_per_pq_code = property(lambda self: self._p.contents.max_train_points_per_pq_code)
    codebook_kind = property(lambda self: self._p.contents.codebook_kind)
    codes_layout = property(lambda self: "flat" if self._p.contents.codes_layout == 0 else "interleaved")

    @property
    def params(self):
        return self._p.contents

    def get_handle(self):
        """Address of the C parameter struct (ivf_pq.pyx:236)."""
        return C.cast(self._p, C.c_void_p).value

    def __del__(self):
        try:
            if self._p:
                lib().cuvsIvfPqIndexParamsDestroy(self._p)
                self._p = None
        except Exception:
            pass


class SearchParams:
    def __init__(self, *, n_probes=20, lut_dtype=np.float32, internal_distance_dtype=np.float32,
                 coarse_search_dtype=np.float32, max_internal_batch_size=4096):
        self._p = C.POINTER(SearchParamsStruct)()
        check(lib().cuvsIvfPqSearchParamsCreate(C.byref(self._p)))
        p = self._p.contents
        p.n_probes = n_probes
        p.lut_dtype = _map_dtype_np_to_cuda(lut_dtype)
        p.internal_distance_dtype = _map_dtype_np_to_cuda(internal_distance_dtype)
        p.coarse_search_dtype = _map_dtype_np_to_cuda(coarse_search_dtype)
        p.max_internal_batch_size = max_internal_batch_size

    @property
    def params(self):
        return self._p.contents

    n_probes = property(lambda self: self.params.n_probes)
    lut_dtype = property(lambda self: self.params.lut_dtype)
    internal_distance_dtype = property(lambda self: self.params.internal_distance_dtype)
    coarse_search_dtype = property(lambda self: self.params.coarse_search_dtype)
    max_internal_batch_size = property(lambda self: self.params.max_internal_batch_size)

    def get_handle(self):
        """Address of the C parameter struct (ivf_pq.pyx:739)."""
        return C.cast(self._p, C.c_void_p).value

    def __del__(self):
        try:
            if self._p:
                lib().cuvsIvfPqSearchParamsDestroy(self._p)
                self._p = None
        except Exception:
            pass


def _torch():
    import torch
    return torch


class _BorrowedView:
    """A DLManagedTensor filled by a getter; frees the library-side shape arrays on release."""

    def __init__(self):
        from ._lib import DLManagedTensor
        self.mt = DLManagedTensor()

    def release(self):
        if self.mt.deleter:
            self.mt.deleter(C.byref(self.mt))


class Index:
    """Mirror of cuvs.neighbors.ivf_pq.Index (ivf_pq.pyx:239-474)."""

    def __init__(self):
        self._i = C.POINTER(IndexStruct)()
        check(lib().cuvsIvfPqIndexCreate(C.byref(self._i)))
        self.trained = False
        self._keepalive = []

    @property
    def index(self):
        return self._i

    def _scalar(self, fn):
        v = C.c_int64(0)
        check(fn(self._i, C.byref(v)))
        return v.value

    n_lists = property(lambda self: self._scalar(lib().cuvsIvfPqIndexGetNLists))
    dim = property(lambda self: self._scalar(lib().cuvsIvfPqIndexGetDim))
    pq_dim = property(lambda self: self._scalar(lib().cuvsIvfPqIndexGetPqDim))
    pq_len = property(lambda self: self._scalar(lib().cuvsIvfPqIndexGetPqLen))
    pq_bits = property(lambda self: self._scalar(lib().cuvsIvfPqIndexGetPqBits))

    def __len__(self):
        return self._scalar(lib().cuvsIvfPqIndexGetSize)

    def _device_copy(self, getter, dtype, *args):
        """Copy a getter's device view into a fresh torch tensor."""
        torch = _torch()
        v = _BorrowedView()
        check(getter(self._i, *args, C.byref(v.mt)))
        t = v.mt.dl_tensor
        shape = [t.shape[i] for i in range(t.ndim)]
        strides = [t.strides[i] for i in range(t.ndim)] if t.strides else None
        n = int(np.prod(shape)) if shape else 1
        out = torch.empty(shape, dtype=dtype, device="cuda")
        if n > 0:
            itemsize = out.element_size()
            if strides is None or len(shape) < 2 or strides[0] == shape[1]:
                _memcpy_d2d(out.data_ptr(), t.data, n * itemsize)
            else:
                _memcpy_2d(out.data_ptr(), shape[1] * itemsize, t.data, strides[0] * itemsize,
                           shape[1] * itemsize, shape[0])
        v.release()
        return out

    @property
    def centers(self):
        return self._device_copy(lib().cuvsIvfPqIndexGetCenters, _torch().float32)

    @property
    def centers_padded(self):
        return self._device_copy(lib().cuvsIvfPqIndexGetCentersPadded, _torch().float32)

    @property
    def pq_centers(self):
        return self._device_copy(lib().cuvsIvfPqIndexGetPqCenters, _torch().float32)

    @property
    def centers_rot(self):
        return self._device_copy(lib().cuvsIvfPqIndexGetCentersRot, _torch().float32)

    @property
    def rotation_matrix(self):
        return self._device_copy(lib().cuvsIvfPqIndexGetRotationMatrix, _torch().float32)

    @property
    def list_sizes(self):
        return self._device_copy(lib().cuvsIvfPqIndexGetListSizes, _torch().int32)

    def __repr__(self):
        attrs = ", ".join(f"{name}={getattr(self, name)}" for name in ("n_lists", "dim", "pq_dim", "pq_len", "pq_bits"))
        return f"Index(type=IvfPq, {attrs})"

    def lists(self, resources=None):
        """Iterates over the lists: (source indices, bit-contiguous codes) of each (ivf_pq.pyx:392-408)."""
        for label, size in enumerate(self.list_sizes.cpu().tolist()):
            yield self.list_indices(label, n_rows=size), self.list_data(label, n_rows=size, resources=resources)

    def list_indices(self, label, n_rows=0):
        """Source indices of one list; the first `n_rows` of them when given (ivf_pq.pyx:451-474)."""
        v = _BorrowedView()
        check(lib().cuvsIvfPqIndexGetListIndices(self._i, int(label), C.byref(v.mt)))
        n = v.mt.dl_tensor.shape[0]
        if n_rows:
            n = min(n, int(n_rows))
        torch = _torch()
        out = torch.empty(n, dtype=torch.int64, device="cuda")
        if n > 0:
            _memcpy_d2d(out.data_ptr(), v.mt.dl_tensor.data, n * 8)
        v.release()
        return out

    def list_data(self, label, n_rows=None, offset=0, resources=None):
        """Bit-contiguous codes of one list (cuvsIvfPqIndexUnpackContiguousListData)."""
        torch = _torch()
        res = resources or _default_resources()
        if n_rows is None:
            n_rows = int(self.list_sizes[label].item()) - offset
        row_bytes = (self.pq_dim * self.pq_bits + 7) // 8
        out = torch.empty((n_rows, row_bytes), dtype=torch.uint8, device="cuda")
        if n_rows > 0:
            res.use_torch_current_stream()
            check(lib().cuvsIvfPqIndexUnpackContiguousListData(
                res.get_c_obj(), self._i, dlpack.view(out).ptr, int(label), int(offset)))
            res.sync()
        return out

    def __del__(self):
        try:
            if self._i:
                lib().cuvsIvfPqIndexDestroy(self._i)
                self._i = None
        except Exception:
            pass


def _hip():
    import ctypes.util
    global _hip_lib
    try:
        return _hip_lib
    except NameError:
        pass
    for name in ("libamdhip64.so", "libamdhip64.so.7", "libamdhip64.so.6"):
        try:
            _hip_lib = C.CDLL(name)
            break
        except OSError:
            continue
    else:
        _hip_lib = C.CDLL(ctypes.util.find_library("amdhip64"))
    _hip_lib.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    _hip_lib.hipMemcpy.restype = C.c_int
    _hip_lib.hipMemcpy2D.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t,
                                     C.c_size_t, C.c_int]
    _hip_lib.hipMemcpy2D.restype = C.c_int
    return _hip_lib


def _memcpy_d2d(dst, src, nbytes):
    rc = _hip().hipMemcpy(C.c_void_p(dst), C.c_void_p(src), nbytes, 3)
    if rc != 0:
        raise RuntimeError("hipMemcpy failed with %d" % rc)


def _memcpy_2d(dst, dpitch, src, spitch, width, height):
    rc = _hip().hipMemcpy2D(C.c_void_p(dst), dpitch, C.c_void_p(src), spitch, width, height, 3)
    if rc != 0:
        raise RuntimeError("hipMemcpy2D failed with %d" % rc)


_default = None


def _default_resources():
    global _default
    if _default is None:
        _default = Resources()
    return _default


def _prep(res):
    """Role of the auto_sync_resources decorator: default handle on torch's current stream."""
    own = res is None
    res = res or _default_resources()
    if own:
        res.use_torch_current_stream()
    return res, own


def build(index_params, dataset, resources=None):
    """ivf_pq.pyx:477 -- train an index on `dataset` and (add_data_on_build) add the rows."""
    res, own = _prep(resources)
    index = Index()
    check(lib().cuvsIvfPqBuild(res.get_c_obj(), index_params._p, dlpack.view(dataset).ptr,
                               index.index))
    if own:
        res.sync()
    index.trained = True
    return index


def build_precomputed(index_params, dim, pq_centers, centers, centers_rot, rotation_matrix,
                      resources=None):
    """ivf_pq.pyx:543 -- index from a trained model held in device tensors."""
    res, own = _prep(resources)
    index = Index()
    check(lib().cuvsIvfPqBuildPrecomputed(
        res.get_c_obj(), index_params._p, int(dim), dlpack.view(pq_centers).ptr,
        dlpack.view(centers).ptr, dlpack.view(centers_rot).ptr, dlpack.view(rotation_matrix).ptr,
        index.index))
    if own:
        res.sync()
    index.trained = True
    return index


def extend(index, new_vectors, new_indices, resources=None, labels=None):
    """ivf_pq.pyx:913.  `labels` (int32/uint32 tensor) routes through cuvsAmdIvfPqExtendLabeled."""
    res, own = _prep(resources)
    vv = dlpack.view(new_vectors)
    iv = dlpack.view(new_indices) if new_indices is not None else None
    if labels is None:
        check(lib().cuvsIvfPqExtend(res.get_c_obj(), vv.ptr, iv.ptr if iv else None, index.index))
    else:
        lv = dlpack.view(labels, as_dtype=dlpack.UINT32)
        check(lib().cuvsAmdIvfPqExtendLabeled(res.get_c_obj(), vv.ptr, iv.ptr if iv else None,
                                              lv.ptr, index.index))
    if own:
        res.sync()
    return index


def search(search_params, index, queries, k, neighbors=None, distances=None, resources=None,
           filter_bitset=None, filter_nbits=None):
    """ivf_pq.pyx:745-840.  Returns (distances, neighbors)."""
    torch = _torch()
    res, own = _prep(resources)
    n_queries = queries.shape[0]
    if neighbors is None:
        neighbors = torch.empty((n_queries, k), dtype=torch.int64, device="cuda")
    if distances is None:
        distances = torch.empty((n_queries, k), dtype=torch.float32, device="cuda")
    qv, nv, dv = dlpack.view(queries), dlpack.view(neighbors), dlpack.view(distances)
    if filter_bitset is None:
        check(lib().cuvsIvfPqSearch(res.get_c_obj(), search_params._p, index.index, qv.ptr,
                                    nv.ptr, dv.ptr))
    else:
        bv = dlpack.view(filter_bitset, as_dtype=dlpack.UINT32)
        nbits = filter_nbits if filter_nbits is not None else filter_bitset.numel() * 32
        check(lib().cuvsAmdIvfPqSearchWithBitset(res.get_c_obj(), search_params._p, index.index,
                                                 qv.ptr, nv.ptr, dv.ptr, bv.ptr, int(nbits)))
    if own:
        res.sync()
    return distances, neighbors


NO_ALLOC_WORKSPACE_BYTES = 32 << 20


def search_no_alloc(search_params, index, queries, neighbors, distances, resources=None):
    """cuvsAmdIvfPqSearchNoAlloc: `search` into outputs the caller made, on a fixed workspace that
    is part of the library (at most NO_ALLOC_WORKSPACE_BYTES per internal batch; larger searches
    raise CuvsError), without allocating device memory.  Returns (distances, neighbors)."""
    res, own = _prep(resources)
    qv, nv, dv = dlpack.view(queries), dlpack.view(neighbors), dlpack.view(distances)
    check(lib().cuvsAmdIvfPqSearchNoAlloc(res.get_c_obj(), search_params._p, index.index, qv.ptr,
                                          nv.ptr, dv.ptr))
    if own:
        res.sync()
    return distances, neighbors


def select_clusters(search_params, index, queries, resources=None):
    """Probe lists [n_queries, min(n_probes, n_lists)] as an int32 tensor holding uint32 values."""
    torch = _torch()
    res, own = _prep(resources)
    P = min(search_params.n_probes, index.n_lists)
    probes = torch.empty((queries.shape[0], P), dtype=torch.int32, device="cuda")
    check(lib().cuvsAmdIvfPqSelectClusters(res.get_c_obj(), search_params._p, index.index,
                                           dlpack.view(queries).ptr,
                                           dlpack.view(probes, as_dtype=dlpack.UINT32).ptr))
    if own:
        res.sync()
    return probes


def transform(index, input_dataset, output_labels=None, output_dataset=None, resources=None):
    """ivf_pq.pyx:987.  Returns (labels as int32 tensor holding uint32 values, codes uint8)."""
    torch = _torch()
    res, own = _prep(resources)
    n = input_dataset.shape[0]
    row_bytes = (index.pq_dim * index.pq_bits + 7) // 8
    if output_labels is None:
        output_labels = torch.empty(n, dtype=torch.int32, device="cuda")
    if output_dataset is None:
        output_dataset = torch.empty((n, row_bytes), dtype=torch.uint8, device="cuda")
    check(lib().cuvsIvfPqTransform(res.get_c_obj(), index.index, dlpack.view(input_dataset).ptr,
                                   dlpack.view(output_labels, as_dtype=dlpack.UINT32).ptr,
                                   dlpack.view(output_dataset).ptr))
    if own:
        res.sync()
    return output_labels, output_dataset


def save(filename, index, include_dataset=True, resources=None):
    res, _ = _prep(resources)
    check(lib().cuvsIvfPqSerialize(res.get_c_obj(), str(filename).encode(), index.index))


def load(filename, resources=None):
    res, _ = _prep(resources)
    index = Index()
    check(lib().cuvsIvfPqDeserialize(res.get_c_obj(), str(filename).encode(), index.index))
    index.trained = True
    return index


def get_search_profile(resources=None):
    """Stage times (ms) and scanned bytes of the last search made with profiling enabled."""
    res = resources or _default_resources()
    p = SearchProfileStruct()
    check(lib().cuvsAmdIvfPqGetSearchProfile(res.get_c_obj(), C.byref(p)))
    return {f: getattr(p, f) for f, _ in SearchProfileStruct._fields_}
