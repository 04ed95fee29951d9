"""Python-side argument checks: array-ness, number of dimensions and dtype.

Sizes are checked by the library itself. Messages follow
``python/mops/src/mops/checks.py:9-34`` of lab-cosmo/mops; which parameter has
how many dimensions comes from the ABI table instead of being repeated per
operation.
"""
from . import _dispatch
from ._c_api import _KINDS, SIGNATURES


def check_array(array, ndim, operation, name):
    if not _dispatch.is_array(array):
        raise TypeError(f"`{name}` must be an array in {operation}, got {type(array)}")
    if len(array.shape) != ndim:
        raise ValueError(
            f"`{name}` must be a {ndim}D array in {operation}, "
            f"got a {len(array.shape)}D array instead"
        )


def check_scalar(value, operation, name):
    if not _dispatch.is_scalar(value):
        raise TypeError(f"`{name}` must be a scalar in {operation}, got {type(value)}")
    if not isinstance(value, (int, _dispatch.np.integer)):
        raise TypeError(f"Wrong dtype for {name} in {operation}: got {type(value)}")


def check_dtype(array, want_index, operation, name):
    ok = _dispatch.is_integer(array) if want_index else _dispatch.is_floating(array)
    if not ok:
        raise TypeError(f"Wrong dtype for {name} in {operation}: got {_dispatch.dtype_name(array)}")


def check_arguments(function, arguments):
    """Check the user-supplied tensors of ``function``.

    ``arguments`` maps parameter names of the C signature to arrays (``None``
    for an optional tensor that was not given). First all dimension counts,
    then all dtypes, in signature order.
    """
    kinds = {name: kind for kind, name in SIGNATURES[function]}
    for name, array in arguments.items():
        if array is None:
            continue
        kind = kinds[name]
        ndim = 3 if kind == "Q3" else _KINDS[kind][0]
        check_array(array, ndim, function, name)
    for name, array in arguments.items():
        if array is None:
            continue
        check_dtype(array, _KINDS[kinds[name]][1], function, name)
