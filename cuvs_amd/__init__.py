"""MI355X-native IVF-PQ search engine behind the cuVS C / Python API surface.

The Python layer is a thin ctypes binding over ``libcuvs_c.so`` (HIP kernels for gfx950 behind the
cuVS C ABI); it mirrors ``cuvs.neighbors.ivf_pq`` of the reference Python package.
"""
from . import ivf_pq  # noqa: F401
from .refine import refine  # noqa: F401
from .knn_merge_parts import knn_merge_parts  # noqa: F401
from .resources import Resources  # noqa: F401

__all__ = ["ivf_pq", "refine", "knn_merge_parts", "Resources"]
