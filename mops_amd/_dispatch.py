"""Array-library dispatch for the Python front-end.

The reference front-end accepts numpy arrays (host) and cupy arrays (device)
(``python/mops/src/mops/_dispatch.py:5-94`` of lab-cosmo/mops). Here the device
arrays are PyTorch tensors on a ROCm GPU; numpy arrays and CPU tensors are
routed to the host entry points, which validate and then report that this
build has no host arithmetic.
"""
import numpy as np

try:
    import torch
except ImportError:  # pragma: no cover - torch is a hard requirement of the device path
    torch = None


def is_torch(array):
    return torch is not None and isinstance(array, torch.Tensor)


def is_array(array):
    return isinstance(array, np.ndarray) or is_torch(array)


def is_scalar(value):
    return isinstance(value, (int, float, np.integer, np.floating))


def on_device(array):
    return is_torch(array) and array.is_cuda


def is_floating(array):
    if is_torch(array):
        return array.dtype.is_floating_point
    return np.issubdtype(array.dtype, np.floating)


def is_integer(array):
    if is_torch(array):
        return not array.dtype.is_floating_point and not array.dtype.is_complex and array.dtype != torch.bool
    return np.issubdtype(array.dtype, np.integer)


def dtype_name(array):
    return str(array.dtype).replace("torch.", "")


def contiguous(array):
    if is_torch(array):
        return array.contiguous()
    return np.ascontiguousarray(array)


def as_int32(array):
    if is_torch(array):
        return array.to(torch.int32).contiguous()
    return np.ascontiguousarray(array.astype(np.int32))


def empty(shape, like):
    """Uninitialised array of ``shape`` with the dtype and device of ``like``."""
    if is_torch(like):
        return torch.empty(tuple(shape), dtype=like.dtype, device=like.device)
    return np.empty(tuple(shape), dtype=like.dtype)
