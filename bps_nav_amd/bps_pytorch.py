"""Counterpart of the reference's `bps_pytorch` torch extension (simulator/pytorch.cpp:13-75):
tensors that alias device memory owned by the simulator, without a copy and without a
deleter.  The reference wraps renderer images; here the same entry points wrap any HIP
device pointer (torch-ROCm addresses the GPU as device type "cuda").
"""
import ctypes

import numpy as np
import torch

_PyCapsule_New = ctypes.pythonapi.PyCapsule_New
_PyCapsule_New.restype = ctypes.py_object
_PyCapsule_New.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_void_p]
_PyCapsule_GetPointer = ctypes.pythonapi.PyCapsule_GetPointer
_PyCapsule_GetPointer.restype = ctypes.c_void_p
_PyCapsule_GetPointer.argtypes = [ctypes.py_object, ctypes.c_char_p]

_TYPESTR = {torch.float32: "<f4", torch.uint8: "|u1", torch.float16: "<f2", torch.int64: "<i8",
            torch.int32: "<i4"}


class _DeviceArray:
    """Minimal __cuda_array_interface__ producer; `owner` is kept alive by the tensor."""

    def __init__(self, ptr, shape, dtype, owner):
        self.owner = owner
        self.__cuda_array_interface__ = {
            "shape": tuple(int(s) for s in shape), "typestr": _TYPESTR[dtype], "data": (int(ptr), False),
            "version": 2, "strides": None}


def tensor_from_pointer(ptr, shape, dtype, dev_id, owner=None):
    """Tensor of `shape`/`dtype` aliasing device memory at `ptr` on GPU `dev_id` (no copy)."""
    if not ptr:
        raise ValueError("null device pointer")
    if int(np.prod(shape)) == 0:
        return torch.empty(tuple(shape), dtype=dtype, device=f"cuda:{dev_id}")
    return torch.as_tensor(_DeviceArray(ptr, shape, dtype, owner), device=f"cuda:{dev_id}")


def _pointer(capsule_or_ptr):
    if isinstance(capsule_or_ptr, int):
        return capsule_or_ptr
    return _PyCapsule_GetPointer(capsule_or_ptr, None)


def make_color_tensor(ptr_capsule, dev_id, batch_size, resolution):
    """u8[batch, H, W, 4] over a device pointer (pytorch.cpp:15-29)."""
    return tensor_from_pointer(_pointer(ptr_capsule), (batch_size, resolution[0], resolution[1], 4), torch.uint8, dev_id)


def make_depth_tensor(ptr_capsule, dev_id, batch_size, resolution):
    """f32[batch, H, W] over a device pointer (pytorch.cpp:33-47)."""
    return tensor_from_pointer(_pointer(ptr_capsule), (batch_size, resolution[0], resolution[1]), torch.float32, dev_id)


def make_fcout_tensor(ptr_capsule, dev_id, batch_size, num_features):
    """f16[batch, features] over a device pointer (pytorch.cpp:50-64)."""
    return tensor_from_pointer(_pointer(ptr_capsule), (batch_size, num_features), torch.float16, dev_id)


def tensor_to_capsule(tensor):
    """Capsule holding tensor.data_ptr() (pytorch.cpp:66-69)."""
    return _PyCapsule_New(tensor.data_ptr(), None, None)
