"""Loader and ctypes prototypes of ``libcuvs_c.so``.

The library must have been built (``python -c "import __graft_entry__ as g; g.build()"`` or
``make -C cuvs_amd/csrc``); there is no fallback path.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("CUVS_AMD_LIB", os.path.join(_HERE, "libcuvs_c.so"))

CUVS_ERROR, CUVS_SUCCESS = 0, 1


class CuvsError(RuntimeError):
    """Raised when a C entry point returns CUVS_ERROR; carries cuvsGetLastErrorText()."""


class DLDevice(C.Structure):
    _fields_ = [("device_type", C.c_int32), ("device_id", C.c_int32)]


class DLDataType(C.Structure):
    _fields_ = [("code", C.c_uint8), ("bits", C.c_uint8), ("lanes", C.c_uint16)]


class DLTensor(C.Structure):
    _fields_ = [("data", C.c_void_p), ("device", DLDevice), ("ndim", C.c_int32),
                ("dtype", DLDataType), ("shape", C.POINTER(C.c_int64)),
                ("strides", C.POINTER(C.c_int64)), ("byte_offset", C.c_uint64)]


class DLManagedTensor(C.Structure):
    pass


_DELETER = C.CFUNCTYPE(None, C.POINTER(DLManagedTensor))
DLManagedTensor._fields_ = [("dl_tensor", DLTensor), ("manager_ctx", C.c_void_p),
                            ("deleter", _DELETER)]


class IndexParamsStruct(C.Structure):
    # include/cuvs/neighbors/ivf_pq.h: struct cuvsIvfPqIndexParams
    _fields_ = [("metric", C.c_int), ("metric_arg", C.c_float), ("add_data_on_build", C.c_bool),
                ("n_lists", C.c_uint32), ("kmeans_n_iters", C.c_uint32),
                ("kmeans_trainset_fraction", C.c_double), ("pq_bits", C.c_uint32),
                ("pq_dim", C.c_uint32), ("codebook_kind", C.c_int),
                ("force_random_rotation", C.c_bool),
                ("conservative_memory_allocation", C.c_bool),
                ("max_train_points_per_pq_code", C.c_uint32), ("codes_layout", C.c_int)]


class SearchParamsStruct(C.Structure):
    # include/cuvs/neighbors/ivf_pq.h: struct cuvsIvfPqSearchParams
    _fields_ = [("n_probes", C.c_uint32), ("lut_dtype", C.c_int),
                ("internal_distance_dtype", C.c_int), ("coarse_search_dtype", C.c_int),
                ("max_internal_batch_size", C.c_uint32), ("preferred_shmem_carveout", C.c_double)]


class IndexStruct(C.Structure):
    _fields_ = [("addr", C.c_void_p), ("dtype", DLDataType)]


class SearchTuningStruct(C.Structure):
    _fields_ = [("early_stop", C.c_int32), ("generic_scan", C.c_int32), ("plain_coarse", C.c_int32),
                ("serial_batches", C.c_int32), ("reserved_", C.c_int32 * 4)]


class SearchProfileStruct(C.Structure):
    _fields_ = [("n_queries", C.c_uint32), ("n_probes", C.c_uint32), ("k", C.c_uint32),
                ("n_scan_launches", C.c_uint32), ("coarse_ms", C.c_float),
                ("rotate_ms", C.c_float), ("scan_ms", C.c_float), ("merge_ms", C.c_float),
                ("total_ms", C.c_float), ("scan_bytes", C.c_uint64), ("scan_rows", C.c_uint64),
                ("lead_scan_ms", C.c_float), ("screen_ms", C.c_float),
                ("survivor_scan_ms", C.c_float), ("scan_kernel", C.c_uint32),
                ("lead_bytes", C.c_uint64), ("screen_bytes", C.c_uint64),
                ("survivor_bytes", C.c_uint64), ("n_screened_pairs", C.c_uint64),
                ("n_surviving_pairs", C.c_uint64), ("n_far_pairs", C.c_uint64)]


# every symbol include/cuvs/core/c_api.h and include/cuvs/neighbors/ivf_pq.h declare
EXPORTED_SYMBOLS = [
    "cuvsGetLastErrorText", "cuvsSetLastErrorText", "cuvsGetLogLevel", "cuvsSetLogLevel",
    "cuvsResourcesCreate", "cuvsResourcesDestroy", "cuvsStreamSet", "cuvsStreamGet",
    "cuvsStreamSync", "cuvsDeviceIdGet", "cuvsResourcesSetWorkspacePool", "cuvsRMMAlloc",
    "cuvsRMMFree", "cuvsVersionGet", "cuvsRMMPoolMemoryResourceEnable",
    "cuvsRMMAsyncMemoryResourceEnable", "cuvsRMMMemoryResourceReset", "cuvsRMMHostAlloc",
    "cuvsRMMHostFree", "cuvsMatrixCopy", "cuvsMatrixSliceRows", "cuvsResourcesCreateWithMemoryTracking",
    "cuvsMultiGpuResourcesCreate", "cuvsMultiGpuResourcesCreateWithDeviceIds",
    "cuvsMultiGpuResourcesDestroy", "cuvsMultiGpuResourcesSetMemoryPool",
    "cuvsIvfPqIndexParamsCreate", "cuvsIvfPqIndexParamsDestroy", "cuvsIvfPqSearchParamsCreate",
    "cuvsIvfPqSearchParamsDestroy", "cuvsIvfPqIndexCreate", "cuvsIvfPqIndexDestroy",
    "cuvsIvfPqIndexGetNLists", "cuvsIvfPqIndexGetDim", "cuvsIvfPqIndexGetSize",
    "cuvsIvfPqIndexGetPqDim", "cuvsIvfPqIndexGetPqBits", "cuvsIvfPqIndexGetPqLen",
    "cuvsIvfPqIndexGetCenters", "cuvsIvfPqIndexGetCentersPadded", "cuvsIvfPqIndexGetPqCenters",
    "cuvsIvfPqIndexGetCentersRot", "cuvsIvfPqIndexGetRotationMatrix",
    "cuvsIvfPqIndexGetListSizes", "cuvsIvfPqIndexUnpackContiguousListData",
    "cuvsIvfPqIndexGetListIndices", "cuvsIvfPqBuild", "cuvsIvfPqBuildPrecomputed",
    "cuvsIvfPqSearch", "cuvsIvfPqSerialize", "cuvsIvfPqDeserialize", "cuvsIvfPqExtend",
    "cuvsIvfPqTransform", "cuvsAmdIvfPqSelectClusters", "cuvsAmdIvfPqSearchWithBitset",
    "cuvsAmdIvfPqSearchNoAlloc", "cuvsAmdIvfPqSetSearchTuning",
    "cuvsAmdIvfPqExtendLabeled", "cuvsAmdIvfPqProfilingEnable", "cuvsAmdIvfPqGetSearchProfile",
    "cuvsRefine",
    "cuvsAmdKnnMergeParts",
]

_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C cuvs_amd/csrc` (needs hipcc); "
            "this package has no fallback implementation")
    L = C.CDLL(LIB_PATH)
    P = C.POINTER
    T = P(DLManagedTensor)
    res_t = C.c_size_t
    L.cuvsGetLastErrorText.restype = C.c_char_p
    L.cuvsGetLastErrorText.argtypes = []
    L.cuvsSetLastErrorText.restype = None
    L.cuvsSetLastErrorText.argtypes = [C.c_char_p]
    L.cuvsGetLogLevel.restype = C.c_int
    L.cuvsSetLogLevel.restype = None
    L.cuvsSetLogLevel.argtypes = [C.c_int]

    def proto(name, *args):
        f = getattr(L, name)
        f.restype = C.c_int
        f.argtypes = list(args)

    proto("cuvsResourcesCreate", P(res_t))
    proto("cuvsResourcesCreateWithMemoryTracking", P(res_t), C.c_char_p, C.c_int64)
    proto("cuvsMultiGpuResourcesCreate", P(res_t))
    proto("cuvsMultiGpuResourcesCreateWithDeviceIds", P(res_t), T)
    proto("cuvsMultiGpuResourcesDestroy", res_t)
    proto("cuvsMultiGpuResourcesSetMemoryPool", res_t, C.c_int)
    proto("cuvsResourcesDestroy", res_t)
    proto("cuvsStreamSet", res_t, C.c_void_p)
    proto("cuvsStreamGet", res_t, P(C.c_void_p))
    proto("cuvsStreamSync", res_t)
    proto("cuvsDeviceIdGet", res_t, P(C.c_int))
    proto("cuvsResourcesSetWorkspacePool", res_t, C.c_size_t)
    proto("cuvsRMMPoolMemoryResourceEnable", C.c_int, C.c_int, C.c_bool)
    proto("cuvsRMMAsyncMemoryResourceEnable")
    proto("cuvsRMMMemoryResourceReset")
    proto("cuvsRMMHostAlloc", P(C.c_void_p), C.c_size_t)
    proto("cuvsRMMHostFree", C.c_void_p, C.c_size_t)
    proto("cuvsMatrixCopy", res_t, T, T)
    proto("cuvsMatrixSliceRows", res_t, T, C.c_int64, C.c_int64, T)
    proto("cuvsRMMAlloc", res_t, P(C.c_void_p), C.c_size_t)
    proto("cuvsRMMFree", res_t, C.c_void_p, C.c_size_t)
    proto("cuvsVersionGet", P(C.c_uint16), P(C.c_uint16), P(C.c_uint16))
    proto("cuvsIvfPqIndexParamsCreate", P(P(IndexParamsStruct)))
    proto("cuvsIvfPqIndexParamsDestroy", P(IndexParamsStruct))
    proto("cuvsIvfPqSearchParamsCreate", P(P(SearchParamsStruct)))
    proto("cuvsIvfPqSearchParamsDestroy", P(SearchParamsStruct))
    proto("cuvsIvfPqIndexCreate", P(P(IndexStruct)))
    proto("cuvsIvfPqIndexDestroy", P(IndexStruct))
    for n in ("NLists", "Dim", "Size", "PqDim", "PqBits", "PqLen"):
        proto("cuvsIvfPqIndexGet" + n, P(IndexStruct), P(C.c_int64))
    for n in ("Centers", "CentersPadded", "PqCenters", "CentersRot", "RotationMatrix",
              "ListSizes"):
        proto("cuvsIvfPqIndexGet" + n, P(IndexStruct), T)
    proto("cuvsIvfPqIndexUnpackContiguousListData", res_t, P(IndexStruct), T, C.c_uint32,
          C.c_uint32)
    proto("cuvsIvfPqIndexGetListIndices", P(IndexStruct), C.c_uint32, T)
    proto("cuvsIvfPqBuild", res_t, P(IndexParamsStruct), T, P(IndexStruct))
    proto("cuvsIvfPqBuildPrecomputed", res_t, P(IndexParamsStruct), C.c_uint32, T, T, T, T,
          P(IndexStruct))
    proto("cuvsIvfPqSearch", res_t, P(SearchParamsStruct), P(IndexStruct), T, T, T)
    proto("cuvsRefine", res_t, T, T, T, C.c_int, T, T)
    proto("cuvsAmdKnnMergeParts", res_t, T, T, T, T, T)
    proto("cuvsIvfPqSerialize", res_t, C.c_char_p, P(IndexStruct))
    proto("cuvsIvfPqDeserialize", res_t, C.c_char_p, P(IndexStruct))
    proto("cuvsIvfPqExtend", res_t, T, T, P(IndexStruct))
    proto("cuvsIvfPqTransform", res_t, P(IndexStruct), T, T, T)
    proto("cuvsAmdIvfPqSelectClusters", res_t, P(SearchParamsStruct), P(IndexStruct), T, T)
    proto("cuvsAmdIvfPqSearchWithBitset", res_t, P(SearchParamsStruct), P(IndexStruct), T, T, T,
          T, C.c_int64)
    proto("cuvsAmdIvfPqSearchNoAlloc", res_t, P(SearchParamsStruct), P(IndexStruct), T, T, T)
    proto("cuvsAmdIvfPqExtendLabeled", res_t, T, T, T, P(IndexStruct))
    proto("cuvsAmdIvfPqSetSearchTuning", res_t, P(SearchTuningStruct))
    proto("cuvsAmdIvfPqProfilingEnable", res_t, C.c_bool)
    proto("cuvsAmdIvfPqGetSearchProfile", res_t, P(SearchProfileStruct))
    _lib = L
    return L


def check(status):
    """Role of cuvs.common.exceptions.check_cuvs."""
    if status != CUVS_SUCCESS:
        msg = lib().cuvsGetLastErrorText()
        raise CuvsError(msg.decode() if msg else "unknown cuVS error")
