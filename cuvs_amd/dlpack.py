"""DLManagedTensor views over torch tensors and numpy arrays for the C ABI (borrowed, no copy)."""
import ctypes as C

import numpy as np

from ._lib import DLDataType, DLDevice, DLManagedTensor, DLTensor

kDLCPU, kDLCUDA, kDLCUDAHost, kDLROCM, kDLROCMHost = 1, 2, 3, 10, 11
kDLInt, kDLUInt, kDLFloat = 0, 1, 2

_NP_CODES = {"i": kDLInt, "u": kDLUInt, "f": kDLFloat}


def _torch_dtype_info(dtype):
    import torch
    table = {torch.float32: (kDLFloat, 32), torch.float16: (kDLFloat, 16),
             torch.int8: (kDLInt, 8), torch.uint8: (kDLUInt, 8), torch.int32: (kDLInt, 32),
             torch.int64: (kDLInt, 64)}
    if hasattr(torch, "uint32"):
        table[torch.uint32] = (kDLUInt, 32)
    return table[dtype]


class TensorView:
    """Keeps the ctypes struct, its shape array and the viewed object alive together."""

    def __init__(self, obj, as_dtype=None):
        self.obj = obj
        if isinstance(obj, np.ndarray):
            if not obj.flags["C_CONTIGUOUS"]:
                raise ValueError("array must be C-contiguous")
            data, shape = obj.ctypes.data, obj.shape
            code, bits = _NP_CODES[obj.dtype.kind], obj.dtype.itemsize * 8
            device = DLDevice(kDLCPU, 0)
        else:
            if not obj.is_contiguous():
                raise ValueError("tensor must be contiguous")
            data, shape = obj.data_ptr(), tuple(obj.shape)
            code, bits = _torch_dtype_info(obj.dtype)
            if obj.is_cuda:
                device = DLDevice(kDLROCM, obj.device.index or 0)
            else:
                device = DLDevice(kDLCPU, 0)
        if as_dtype is not None:
            code, bits = as_dtype
        self.shape = (C.c_int64 * max(len(shape), 1))(*shape)
        self.mt = DLManagedTensor()
        self.mt.dl_tensor = DLTensor(C.c_void_p(data), device, len(shape),
                                     DLDataType(code, bits, 1), self.shape, None, 0)
        self.mt.manager_ctx = None

    @property
    def ptr(self):
        return C.byref(self.mt)


def view(obj, as_dtype=None):
    return TensorView(obj, as_dtype)


UINT32 = (kDLUInt, 32)
