"""The C-ABI library loads without a GPU and exports exactly what include/*.h declares."""
import ctypes as C
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = set()
    for rel in ("include/cuvs/core/c_api.h", "include/cuvs/neighbors/ivf_pq.h",
                "include/cuvs/neighbors/refine.h",
                "include/cuvs/neighbors/knn_merge_parts.h"):
        with open(os.path.join(ROOT, rel)) as f:
            text = f.read()
        names |= set(re.findall(r"CUVS_EXPORT\s+[\w\s\*]+?\b(cuvs\w+)\s*\(", text))
    return names


def test_library_exports_every_declared_symbol():
    from cuvs_amd import _lib
    L = _lib.lib()
    declared = declared_symbols()
    assert len(declared) >= 40
    for name in sorted(declared):
        assert hasattr(L, name), f"{name} is declared in include/ but not exported"
    assert declared == set(_lib.EXPORTED_SYMBOLS)


def test_params_defaults_and_error_text():
    """Calls that touch no device: parameter objects, defaults, error text plumbing."""
    from cuvs_amd import _lib
    L = _lib.lib()
    sp = C.POINTER(_lib.SearchParamsStruct)()
    assert L.cuvsIvfPqSearchParamsCreate(C.byref(sp)) == _lib.CUVS_SUCCESS
    s = sp.contents
    # defaults of c/src/neighbors/ivf_pq.cpp:372-382
    assert (s.n_probes, s.lut_dtype, s.internal_distance_dtype, s.coarse_search_dtype,
            s.max_internal_batch_size, s.preferred_shmem_carveout) == (20, 0, 0, 0, 4096, 1.0)
    assert L.cuvsIvfPqSearchParamsDestroy(sp) == _lib.CUVS_SUCCESS
    ip = C.POINTER(_lib.IndexParamsStruct)()
    assert L.cuvsIvfPqIndexParamsCreate(C.byref(ip)) == _lib.CUVS_SUCCESS
    p = ip.contents
    # defaults of c/src/neighbors/ivf_pq.cpp:348-365
    assert (p.metric, p.metric_arg, p.add_data_on_build, p.n_lists, p.kmeans_n_iters,
            p.kmeans_trainset_fraction, p.pq_bits, p.pq_dim, p.codebook_kind,
            p.force_random_rotation, p.conservative_memory_allocation,
            p.max_train_points_per_pq_code, p.codes_layout) == (
                0, 2.0, True, 1024, 20, 0.5, 8, 0, 0, False, False, 256, 1)
    assert L.cuvsIvfPqIndexParamsDestroy(ip) == _lib.CUVS_SUCCESS

    # an unbuilt index reports an error and the text is retrievable, then cleared by a success
    idx = C.POINTER(_lib.IndexStruct)()
    assert L.cuvsIvfPqIndexCreate(C.byref(idx)) == _lib.CUVS_SUCCESS
    assert L.cuvsGetLastErrorText() is None
    out = C.c_int64(0)
    assert L.cuvsIvfPqIndexGetDim(idx, C.byref(out)) == _lib.CUVS_ERROR
    assert b"not been built" in L.cuvsGetLastErrorText()
    assert L.cuvsIvfPqIndexDestroy(idx) == _lib.CUVS_SUCCESS
    assert L.cuvsGetLastErrorText() is None
    L.cuvsSetLastErrorText(b"custom")
    assert L.cuvsGetLastErrorText() == b"custom"
    L.cuvsSetLastErrorText(None)
    assert L.cuvsGetLastErrorText() is None

    major, minor, patch = C.c_uint16(), C.c_uint16(), C.c_uint16()
    assert L.cuvsVersionGet(C.byref(major), C.byref(minor), C.byref(patch)) == _lib.CUVS_SUCCESS
    assert (major.value, minor.value) == (26, 10)


def test_python_mirror_keeps_reference_defaults():
    from cuvs_amd import ivf_pq
    sp = ivf_pq.SearchParams()
    assert (sp.n_probes, sp.lut_dtype, sp.internal_distance_dtype, sp.coarse_search_dtype,
            sp.max_internal_batch_size) == (20, 0, 0, 0, 4096)
    import numpy as np
    sp = ivf_pq.SearchParams(n_probes=7, lut_dtype=np.uint8, internal_distance_dtype=np.float16)
    assert (sp.n_probes, sp.lut_dtype, sp.internal_distance_dtype) == (7, 8, 2)
    ip = ivf_pq.IndexParams(n_lists=10, metric="inner_product", codebook_kind="cluster", pq_bits=5)
    assert (ip.params.n_lists, ip.params.metric, ip.params.codebook_kind, ip.params.pq_bits) == (
        10, 6, 1, 5)
    import pytest
    with pytest.raises(ValueError):
        ivf_pq.IndexParams(codebook_kind="nope")
    # the read-only views of the reference's parameter objects (ivf_pq.pyx:174-236, 716-739)
    assert (ip.n_lists, ip.pq_bits, ip.codebook_kind, ip.codes_layout, ip.add_data_on_build) == (
        10, 5, 1, "interleaved", True)
    assert ivf_pq.IndexParams(codes_layout="flat").codes_layout == "flat"
    import ctypes
    from cuvs_amd._lib import IndexParamsStruct, SearchParamsStruct
    assert ctypes.cast(ip.get_handle(), ctypes.POINTER(IndexParamsStruct)).contents.n_lists == 10
    assert ctypes.cast(sp.get_handle(), ctypes.POINTER(SearchParamsStruct)).contents.n_probes == 7


def test_memory_entry_points_reject_bad_arguments_without_a_gpu():
    """Argument checks that come before any device call."""
    from cuvs_amd import _lib
    L = _lib.lib()
    res = C.c_size_t(0)
    assert L.cuvsResourcesCreateWithMemoryTracking(C.byref(res), b"", 10) == _lib.CUVS_ERROR
    assert b"csv_path" in L.cuvsGetLastErrorText()
    assert L.cuvsResourcesCreateWithMemoryTracking(C.byref(res), None, 10) == _lib.CUVS_ERROR
    assert L.cuvsRMMHostFree(None, 0) == _lib.CUVS_SUCCESS
    # one GPU per process: the multi-GPU handles exist to link against and say so when called
    assert L.cuvsMultiGpuResourcesCreate(C.byref(res)) == _lib.CUVS_ERROR
    assert b"one GPU" in L.cuvsGetLastErrorText()
    assert L.cuvsMultiGpuResourcesSetMemoryPool(res, 50) == _lib.CUVS_ERROR
