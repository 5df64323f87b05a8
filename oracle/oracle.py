"""ctypes driver for the CPU oracle (test infrastructure only).

Only tests, the smoke check and the benchmark's CPU-baseline leg import this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

L2Expanded, L2SqrtExpanded, CosineExpanded, InnerProduct = 0, 1, 2, 6
R_32F, R_16F, R_8I, R_8U = 0, 2, 3, 8
PER_SUBSPACE, PER_CLUSTER = 0, 1
T_F32, T_F16, T_I8, T_U8 = 0, 1, 2, 3

_NP_TO_T = {np.dtype(np.float32): T_F32, np.dtype(np.float16): T_F16,
            np.dtype(np.int8): T_I8, np.dtype(np.uint8): T_U8}


def build():
    """Compile liboracle.so from the sources next to this file."""
    subprocess.check_call(["make", "-B", "-C", _HERE, "liboracle.so"])


class _Index(C.Structure):
    _fields_ = [("metric", C.c_int32), ("codebook_kind", C.c_int32), ("n_lists", C.c_uint32),
                ("dim", C.c_uint32), ("pq_dim", C.c_uint32), ("pq_bits", C.c_uint32),
                ("centers", C.c_void_p), ("centers_rot", C.c_void_p),
                ("rotation_matrix", C.c_void_p), ("pq_centers", C.c_void_p),
                ("list_sizes", C.c_void_p), ("list_data", C.c_void_p), ("list_inds", C.c_void_p)]


class _Params(C.Structure):
    _fields_ = [("n_probes", C.c_uint32), ("lut_dtype", C.c_int32),
                ("internal_distance_dtype", C.c_int32), ("coarse_search_dtype", C.c_int32)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        L.orc_last_error.restype = C.c_char_p
        L.orc_dim_ext.restype = C.c_uint32
        L.orc_pq_len.restype = C.c_uint32
        L.orc_rot_dim.restype = C.c_uint32
        for f in (L.orc_dim_ext,):
            f.argtypes = [C.c_uint32]
        for f in (L.orc_pq_len, L.orc_rot_dim):
            f.argtypes = [C.c_uint32, C.c_uint32]
        L.orc_float_to_half.restype = C.c_uint16
        L.orc_float_to_half.argtypes = [C.c_float]
        L.orc_half_to_float.restype = C.c_float
        L.orc_half_to_float.argtypes = [C.c_uint16]
        L.orc_half_add.restype = C.c_uint16
        L.orc_half_add.argtypes = [C.c_uint16, C.c_uint16]
        L.orc_fp8_encode.restype = C.c_uint8
        L.orc_fp8_encode.argtypes = [C.c_float, C.c_int]
        L.orc_fp8_decode.restype = C.c_float
        L.orc_fp8_decode.argtypes = [C.c_uint8, C.c_int]
        L.orc_fp8_decode_half.restype = C.c_uint16
        L.orc_fp8_decode_half.argtypes = [C.c_uint8, C.c_int]
        L.orc_list_bytes.restype = C.c_uint64
        L.orc_list_bytes.argtypes = [C.c_uint32] * 3
        L.orc_pack_list.restype = None
        L.orc_pack_list.argtypes = [C.c_void_p] + [C.c_uint32] * 4 + [C.c_void_p]
        L.orc_unpack_list.restype = None
        L.orc_unpack_list.argtypes = [C.c_void_p] + [C.c_uint32] * 4 + [C.c_void_p]
        L.orc_unpack_list_contiguous.restype = None
        L.orc_unpack_list_contiguous.argtypes = [C.c_void_p] + [C.c_uint32] * 4 + [C.c_void_p]
        L.orc_select_clusters.restype = C.c_int
        L.orc_select_clusters.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_uint32,
                                          C.c_void_p, C.c_void_p, C.c_int]
        L.orc_make_lut.restype = C.c_int
        L.orc_make_lut.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_uint32,
                                   C.c_void_p]
        L.orc_search.restype = C.c_int
        L.orc_search.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_uint32,
                                 C.c_uint32, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p,
                                 C.c_void_p, C.c_int]
        L.orc_encode.restype = C.c_int
        L.orc_encode.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_uint64, C.c_void_p,
                                 C.c_void_p, C.c_int]
        L.orc_refine.restype = C.c_int
        L.orc_refine.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int64, C.c_uint32, C.c_uint32,
                                 C.c_void_p, C.c_uint32, C.c_uint32, C.c_int, C.c_void_p, C.c_void_p]
        _lib = L
    return _lib


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def default_threads():
    return max(1, min(os.cpu_count() or 1, 64))


def dim_ext(dim):
    return int(lib().orc_dim_ext(dim))


def pq_len(dim, pq_dim):
    return int(lib().orc_pq_len(dim, pq_dim))


def rot_dim(dim, pq_dim):
    return int(lib().orc_rot_dim(dim, pq_dim))


def list_bytes(n_rows, pq_dim, pq_bits):
    return int(lib().orc_list_bytes(n_rows, pq_dim, pq_bits))


def pack_list(codes, pq_bits, out=None, row_offset=0):
    """codes: uint8 [n_rows, pq_dim], one code per byte -> interleaved list bytes."""
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    n_rows, pq_dim = codes.shape
    if out is None:
        out = np.zeros(list_bytes(row_offset + n_rows, pq_dim, pq_bits), dtype=np.uint8)
    lib().orc_pack_list(_ptr(codes), n_rows, pq_dim, pq_bits, row_offset, _ptr(out))
    return out


def unpack_list(list_data, n_rows, pq_dim, pq_bits, row_offset=0):
    list_data = np.ascontiguousarray(list_data, dtype=np.uint8)
    out = np.empty((n_rows, pq_dim), dtype=np.uint8)
    lib().orc_unpack_list(_ptr(list_data), n_rows, pq_dim, pq_bits, row_offset, _ptr(out))
    return out


def unpack_list_contiguous(list_data, n_rows, pq_dim, pq_bits, row_offset=0):
    list_data = np.ascontiguousarray(list_data, dtype=np.uint8)
    out = np.empty((n_rows, (pq_dim * pq_bits + 7) // 8), dtype=np.uint8)
    lib().orc_unpack_list_contiguous(_ptr(list_data), n_rows, pq_dim, pq_bits, row_offset,
                                     _ptr(out))
    return out


class Index:
    """Host-side index contents in the layout cuVS search reads."""

    def __init__(self, metric, codebook_kind, dim, pq_dim, pq_bits, centers, centers_rot,
                 rotation_matrix, pq_centers, list_sizes=None, list_data=None, list_inds=None):
        self.metric, self.codebook_kind = int(metric), int(codebook_kind)
        self.dim, self.pq_dim, self.pq_bits = int(dim), int(pq_dim), int(pq_bits)
        self.centers = np.ascontiguousarray(centers, dtype=np.float32)
        self.n_lists = self.centers.shape[0]
        self.centers_rot = np.ascontiguousarray(centers_rot, dtype=np.float32)
        self.rotation_matrix = np.ascontiguousarray(rotation_matrix, dtype=np.float32)
        self.pq_centers = np.ascontiguousarray(pq_centers, dtype=np.float32)
        self.dim_ext = dim_ext(self.dim)
        self.pq_len = pq_len(self.dim, self.pq_dim)
        self.rot_dim = self.pq_len * self.pq_dim
        assert self.centers.shape == (self.n_lists, self.dim_ext)
        assert self.centers_rot.shape == (self.n_lists, self.rot_dim)
        assert self.rotation_matrix.shape == (self.rot_dim, self.dim)
        n_books = self.pq_dim if self.codebook_kind == PER_SUBSPACE else self.n_lists
        assert self.pq_centers.shape == (n_books, self.pq_len, 1 << self.pq_bits)
        if list_sizes is None:
            list_sizes = np.zeros(self.n_lists, dtype=np.uint32)
            list_data = [np.zeros(0, dtype=np.uint8) for _ in range(self.n_lists)]
            list_inds = [np.zeros(0, dtype=np.int64) for _ in range(self.n_lists)]
        self.set_lists(list_sizes, list_data, list_inds)

    def set_lists(self, list_sizes, list_data, list_inds):
        self.list_sizes = np.ascontiguousarray(list_sizes, dtype=np.uint32)
        self.list_data = [np.ascontiguousarray(d, dtype=np.uint8) for d in list_data]
        self.list_inds = [np.ascontiguousarray(i, dtype=np.int64) for i in list_inds]
        for l in range(self.n_lists):
            assert self.list_data[l].size >= list_bytes(int(self.list_sizes[l]), self.pq_dim,
                                                        self.pq_bits)
            assert self.list_inds[l].size >= int(self.list_sizes[l])
        self._data_ptrs = (C.c_void_p * self.n_lists)(*[d.ctypes.data for d in self.list_data])
        self._inds_ptrs = (C.c_void_p * self.n_lists)(*[i.ctypes.data for i in self.list_inds])
        self._c = _Index(self.metric, self.codebook_kind, self.n_lists, self.dim, self.pq_dim,
                         self.pq_bits, self.centers.ctypes.data, self.centers_rot.ctypes.data,
                         self.rotation_matrix.ctypes.data, self.pq_centers.ctypes.data,
                         self.list_sizes.ctypes.data,
                         C.cast(self._data_ptrs, C.c_void_p).value,
                         C.cast(self._inds_ptrs, C.c_void_p).value)

    @property
    def size(self):
        return int(self.list_sizes.sum())

    def fill(self, labels, codes, ids=None):
        """Populate lists from per-row labels and codes (row order preserved within a list)."""
        labels = np.asarray(labels)
        n = labels.shape[0]
        ids = np.arange(n, dtype=np.int64) if ids is None else np.asarray(ids, dtype=np.int64)
        order = np.argsort(labels, kind="stable")
        sizes = np.bincount(labels, minlength=self.n_lists).astype(np.uint32)
        starts = np.concatenate([[0], np.cumsum(sizes.astype(np.int64))]).astype(np.int64)
        data, inds = [], []
        for l in range(self.n_lists):
            rows = order[starts[l]:starts[l + 1]]
            data.append(pack_list(codes[rows].reshape(-1, self.pq_dim), self.pq_bits))
            inds.append(ids[rows].copy())
        self.set_lists(sizes, data, inds)

    def c_ptr(self):
        return C.addressof(self._c)


def _check(rc):
    if rc != 0:
        raise ValueError(lib().orc_last_error().decode())


def _params(n_probes, lut_dtype, internal_distance_dtype, coarse_search_dtype):
    return _Params(int(n_probes), int(lut_dtype), int(internal_distance_dtype),
                   int(coarse_search_dtype))


def _rows(a):
    a = np.ascontiguousarray(a)
    return a, _NP_TO_T[a.dtype]


def select_clusters(index, queries, n_probes, coarse_search_dtype=R_32F, n_threads=None):
    q, t = _rows(queries)
    P = min(int(n_probes), index.n_lists)
    probes = np.empty((q.shape[0], P), dtype=np.uint32)
    scores = np.empty((q.shape[0], P), dtype=np.float32)
    p = _params(n_probes, R_32F, R_32F, coarse_search_dtype)
    _check(lib().orc_select_clusters(index.c_ptr(), C.addressof(p), _ptr(q), t, q.shape[0],
                                     _ptr(probes), _ptr(scores), n_threads or default_threads()))
    return probes, scores


def make_lut(index, query, label, lut_dtype=R_32F, coarse_search_dtype=R_32F):
    q, t = _rows(np.asarray(query).reshape(1, -1))
    n = index.pq_dim << index.pq_bits
    out = np.empty(n, dtype={R_32F: np.float32, R_16F: np.uint16, R_8U: np.uint8}[lut_dtype])
    p = _params(1, lut_dtype, R_32F, coarse_search_dtype)
    _check(lib().orc_make_lut(index.c_ptr(), C.addressof(p), _ptr(q), t, int(label), _ptr(out)))
    return out.reshape(index.pq_dim, 1 << index.pq_bits)


def search(index, queries, k, n_probes, lut_dtype=R_32F, internal_distance_dtype=R_32F,
           coarse_search_dtype=R_32F, filter_bitset=None, filter_nbits=0, n_threads=None,
           return_probes=False):
    q, t = _rows(queries)
    nq = q.shape[0]
    neighbors = np.empty((nq, k), dtype=np.int64)
    distances = np.empty((nq, k), dtype=np.float32)
    P = min(int(n_probes), index.n_lists)
    probes = np.empty((nq, P), dtype=np.uint32) if return_probes else None
    p = _params(n_probes, lut_dtype, internal_distance_dtype, coarse_search_dtype)
    fb = None
    if filter_bitset is not None:
        fb = np.ascontiguousarray(filter_bitset, dtype=np.uint32)
    _check(lib().orc_search(index.c_ptr(), C.addressof(p), _ptr(q), t, nq, int(k),
                            _ptr(fb) if fb is not None else None, int(filter_nbits),
                            _ptr(neighbors), _ptr(distances),
                            _ptr(probes) if probes is not None else None,
                            n_threads or default_threads()))
    if return_probes:
        return neighbors, distances, probes
    return neighbors, distances


def encode(index, rows, n_threads=None):
    x, t = _rows(rows)
    labels = np.empty(x.shape[0], dtype=np.uint32)
    codes = np.empty((x.shape[0], index.pq_dim), dtype=np.uint8)
    _check(lib().orc_encode(index.c_ptr(), _ptr(x), t, x.shape[0], _ptr(labels), _ptr(codes),
                            n_threads or default_threads()))
    return labels, codes


def refine(dataset, queries, candidates, k, metric=0):
    """Exact re-ranking of candidates (orc_refine): returns (indices, distances)."""
    dataset = np.ascontiguousarray(dataset)
    queries = np.ascontiguousarray(queries, dtype=dataset.dtype)
    candidates = np.ascontiguousarray(candidates, dtype=np.int64)
    row_type = {np.dtype(np.float32): 0, np.dtype(np.float16): 1, np.dtype(np.int8): 2,
                np.dtype(np.uint8): 3}[dataset.dtype]
    nq, nc = candidates.shape
    indices = np.empty((nq, k), dtype=np.int64)
    distances = np.empty((nq, k), dtype=np.float32)
    rc = lib().orc_refine(_ptr(dataset), _ptr(queries), row_type, dataset.shape[0], nq,
                          dataset.shape[1], _ptr(candidates), nc, k, metric, _ptr(indices),
                          _ptr(distances))
    if rc != 0:
        raise RuntimeError(lib().orc_last_error().decode())
    return indices, distances
