"""Locate and load the device library.

The library is built in-tree by ``make -C mops_amd/csrc`` (or
``__graft_entry__.build()``) into ``mops_amd/lib/libmops.so``. There is no
fallback: without it nothing in this package can compute, and loading fails
with an error that says how to build it.
"""
import ctypes
import os

from ._c_api import Library

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.path.join(_HERE, "lib", "libmops.so")

_device = None
_host = None


def _require_built():
    if not os.path.exists(LIBRARY_PATH):
        raise ImportError(
            f"{LIBRARY_PATH} is missing: build the HIP library first with "
            "`make -C mops_amd/csrc` (needs hipcc); there is no other implementation to fall back to"
        )


def device_library():
    """The ``mops_cuda_*`` entry points (HIP, device memory)."""
    global _device
    if _device is None:
        _require_built()
        # PyTorch ships its own copy of the HIP runtime under the same soname;
        # importing torch first makes this library bind to that one copy, so
        # that tensors allocated by torch and kernels launched here share one
        # runtime, one context and one set of streams.
        import torch  # noqa: F401

        _device = Library(LIBRARY_PATH, "mops_cuda_", "mops_get_last_error_message")
        cdll = _device.cdll
        cdll.mops_amd_set_stream.argtypes = [ctypes.c_void_p]
        cdll.mops_amd_set_stream.restype = ctypes.c_int
        cdll.mops_amd_get_stream.argtypes = []
        cdll.mops_amd_get_stream.restype = ctypes.c_void_p
        cdll.mops_amd_set_synchronous.argtypes = [ctypes.c_int]
        cdll.mops_amd_set_synchronous.restype = ctypes.c_int
        cdll.mops_amd_first_occurrences.argtypes = [
            ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p,
        ]  # fmt: skip
        cdll.mops_amd_first_occurrences.restype = ctypes.c_int
        cdll.mops_amd_accept_unsorted_indices.argtypes = [ctypes.c_int]
        cdll.mops_amd_accept_unsorted_indices.restype = ctypes.c_int
        cdll.mops_amd_kernel_timing.argtypes = [ctypes.c_int]
        cdll.mops_amd_kernel_timing.restype = ctypes.c_int
        cdll.mops_amd_kernel_time.argtypes = [
            ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_int64),
        ]  # fmt: skip
        cdll.mops_amd_kernel_time.restype = ctypes.c_int
    return _device


def host_library():
    """The ``mops_*`` entry points for host memory (validation only)."""
    global _host
    if _host is None:
        _require_built()
        import torch  # noqa: F401  (see device_library)

        _host = Library(LIBRARY_PATH, "mops_", "mops_get_last_error_message")
    return _host
