"""ctypes description of the mops C ABI and a generic caller.

The tensor views are passed BY VALUE (``include/mops/tensor.h``): a data
pointer followed by ``ndim`` int64 extents. The argument lists below restate
``include/mops/detail/signatures.h`` (which in turn keeps the orders of
``mops/include/mops/*.h`` of lab-cosmo/mops); ``tests/test_abi.py`` checks the
two against each other.

:py:class:`Library` binds any shared object that exports this ABI under some
symbol prefix: the device library (``mops_cuda_`` / ``mops_``) and, in the
test-suite, the CPU oracle (``mops_oracle_``).
"""
import ctypes

import numpy as np

from .status import MopsError

_ELEMENT = {"f32": ctypes.c_float, "f64": ctypes.c_double, "i32": ctypes.c_int32}


def _make_struct(name, element, ndim):
    return type(
        name,
        (ctypes.Structure,),
        {"_fields_": [("data", ctypes.POINTER(element)), ("shape", ctypes.c_int64 * ndim)]},
    )


#: ``STRUCTS[(ndim, "f32"|"f64"|"i32")]`` is the ctypes structure type
STRUCTS = {
    (ndim, tag): _make_struct(f"mops_tensor_{ndim}d_{tag}_t", _ELEMENT[tag], ndim)
    for ndim, tag in [
        (1, "f32"), (2, "f32"), (3, "f32"),
        (1, "f64"), (2, "f64"), (3, "f64"),
        (1, "i32"), (2, "i32"),
    ]
}  # fmt: skip

# kind -> (number of dimensions of the C struct, is an index tensor)
_KINDS = {
    "R1": (1, False), "R2": (2, False), "R3": (3, False),
    "I1": (1, True), "I2": (2, True),
    # three-dimensional tensor that the C header declares with the 2-D struct
    "Q3": (2, False),
}  # fmt: skip

_HPE = [("R2", "A"), ("R1", "C"), ("I2", "indices_A")]
_SAP = [
    ("R2", "A"), ("R2", "B"), ("R1", "C"),
    ("I1", "indices_A"), ("I1", "indices_B"), ("I1", "indices_output"),
]  # fmt: skip
_OPSA = [("R2", "A"), ("R2", "B"), ("I1", "indices_output")]
_OPSAW = [("R2", "A"), ("R2", "B"), ("R2", "W"), ("I1", "indices_W"), ("I1", "indices_output")]
_SASAW = [
    ("R2", "A"), ("R2", "B"), ("R1", "C"), ("R3", "W"),
    ("I1", "indices_A"), ("I1", "indices_W_1"), ("I1", "indices_W_2"),
    ("I1", "indices_output_1"), ("I1", "indices_output_2"),
]  # fmt: skip

#: function name -> ordered (kind, parameter name) pairs
SIGNATURES = {
    "homogeneous_polynomial_evaluation": [("R1", "output")] + _HPE,
    "homogeneous_polynomial_evaluation_vjp": [("R2", "grad_A"), ("R1", "grad_output")] + _HPE,
    "homogeneous_polynomial_evaluation_vjp_vjp": [
        ("R1", "grad_grad_output"), ("R2", "grad_A_2"), ("R2", "grad_grad_A"), ("R1", "grad_output"),
    ] + _HPE,
    "sparse_accumulation_of_products": [("R2", "output")] + _SAP,
    "sparse_accumulation_of_products_vjp": [
        ("R2", "grad_A"), ("R2", "grad_B"), ("R2", "grad_output"),
    ] + _SAP,
    "sparse_accumulation_of_products_vjp_vjp": [
        ("R2", "grad_grad_output"), ("R2", "grad_A_2"), ("R2", "grad_B_2"),
        ("R2", "grad_grad_A"), ("R2", "grad_grad_B"), ("R2", "grad_output"),
    ] + _SAP,
    "outer_product_scatter_add": [("R3", "output")] + _OPSA,
    "outer_product_scatter_add_vjp": [
        ("R2", "grad_A"), ("R2", "grad_B"), ("R3", "grad_output"),
    ] + _OPSA,
    "outer_product_scatter_add_vjp_vjp": [
        ("R3", "grad_grad_output"), ("R2", "grad_A_2"), ("R2", "grad_B_2"),
        ("R2", "grad_grad_A"), ("R2", "grad_grad_B"), ("R3", "grad_output"),
    ] + _OPSA,
    "outer_product_scatter_add_with_weights": [("R3", "output")] + _OPSAW,
    "outer_product_scatter_add_with_weights_vjp": [
        ("R2", "grad_A"), ("R2", "grad_B"), ("R2", "grad_W"), ("R3", "grad_output"),
    ] + _OPSAW,
    "outer_product_scatter_add_with_weights_vjp_vjp": [
        ("R3", "grad_grad_output"), ("R2", "grad_A_2"), ("R2", "grad_B_2"), ("R2", "grad_W_2"),
        ("R2", "grad_grad_A"), ("R2", "grad_grad_B"), ("R2", "grad_grad_W"), ("R3", "grad_output"),
    ] + _OPSAW,
    "sparse_accumulation_scatter_add_with_weights": [("R3", "output")] + _SASAW,
    "sparse_accumulation_scatter_add_with_weights_vjp": [
        ("R2", "grad_A"), ("R2", "grad_B"), ("R3", "grad_W"), ("R3", "grad_output"),
    ] + _SASAW,
    "sparse_accumulation_scatter_add_with_weights_vjp_vjp": [
        ("R3", "grad_grad_output"), ("R2", "grad_A_2"), ("R2", "grad_B_2"), ("R3", "grad_W_2"),
        ("R2", "grad_grad_A"), ("R2", "grad_grad_B"), ("Q3", "grad_grad_W"), ("R3", "grad_output"),
    ] + _SASAW,
}  # fmt: skip

_DTYPE_TAG = {"float32": "f32", "float64": "f64"}


def _describe(array):
    """(address, shape, dtype name) of a numpy array or a torch tensor."""
    if isinstance(array, np.ndarray):
        if not array.flags["C_CONTIGUOUS"]:
            raise ValueError("arrays passed to the C ABI must be C-contiguous")
        return array.ctypes.data, array.shape, array.dtype.name
    # torch tensor (duck-typed so that numpy-only users need no torch import)
    if not array.is_contiguous():
        raise ValueError("tensors passed to the C ABI must be contiguous")
    return array.data_ptr(), tuple(array.shape), str(array.dtype).replace("torch.", "")


def view(array, kind, tag):
    """Build the by-value struct for ``array`` (``None`` gives a null view)."""
    ndim, is_index = _KINDS[kind]
    struct_type = STRUCTS[(ndim, "i32" if is_index else tag)]
    struct = struct_type()
    if array is None:
        return struct  # data = NULL, extents = 0
    address, shape, dtype = _describe(array)
    expected = "int32" if is_index else {"f32": "float32", "f64": "float64"}[tag]
    if dtype != expected:
        raise TypeError(f"expected an array of {expected}, got {dtype}")
    if kind == "Q3":
        shape = shape[:2]
    if len(shape) != ndim:
        raise ValueError(f"expected {ndim} dimensions, got {len(shape)}")
    element = _ELEMENT["i32" if is_index else tag]
    struct.data = ctypes.cast(ctypes.c_void_p(address), ctypes.POINTER(element))
    for d, extent in enumerate(shape):
        struct.shape[d] = extent
    return struct


class Library:
    """A shared object exporting the mops C ABI under ``prefix``."""

    def __init__(self, path, prefix, error_symbol):
        self.path = str(path)
        self.prefix = prefix
        self.cdll = ctypes.CDLL(self.path)
        self._last_error = getattr(self.cdll, error_symbol)
        self._last_error.restype = ctypes.c_char_p
        self._last_error.argtypes = []
        self._functions = {}

    def has(self, name, tag):
        return hasattr(self.cdll, f"{self.prefix}{name}_{tag}")

    def function(self, name, tag):
        key = (name, tag)
        if key not in self._functions:
            symbol = getattr(self.cdll, f"{self.prefix}{name}_{tag}")
            symbol.restype = ctypes.c_int
            symbol.argtypes = [
                STRUCTS[(_KINDS[kind][0], "i32" if _KINDS[kind][1] else tag)]
                for kind, _ in SIGNATURES[name]
            ]
            self._functions[key] = symbol
        return self._functions[key]

    def last_error(self):
        message = self._last_error()
        return message.decode("utf8") if message else ""

    def call(self, name, *arrays):
        """Call ``<prefix><name>_<dtype>`` with arrays in ABI order.

        The floating-point type is taken from the first non-``None``
        floating-point argument. Raises :py:class:`MopsError` on failure.
        """
        signature = SIGNATURES[name]
        if len(arrays) != len(signature):
            raise TypeError(f"{name} takes {len(signature)} tensors, got {len(arrays)}")
        tag = None
        for (kind, _), array in zip(signature, arrays):
            if array is not None and not _KINDS[kind][1]:
                tag = _DTYPE_TAG.get(_describe(array)[2])
                if tag is None:
                    raise TypeError(f"unsupported dtype {_describe(array)[2]} in {name}")
                break
        if tag is None:
            raise TypeError(f"{name}: no floating-point argument to take the dtype from")
        structs = [view(array, kind, tag) for (kind, _), array in zip(signature, arrays)]
        status = self.function(name, tag)(*structs)
        if status != 0:
            raise MopsError(self.last_error(), status)
