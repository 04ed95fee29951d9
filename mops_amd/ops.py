"""The fifteen mops functions on PyTorch-ROCm tensors, over the C ABI.

Names, argument orders, defaults and return values follow the reference's
numpy/cupy front-end (``python/mops/src/mops/{hpe,sap,opsa,opsaw,sasaw}.py`` of
lab-cosmo/mops). Inputs are made contiguous, index tensors are converted to
int32, outputs are allocated here (uninitialised; the library overwrites them
completely) and a skipped gradient is passed as a null view and returned as
``None``.

Device tensors go to the ``mops_cuda_*`` entry points, which run on the
current PyTorch stream of the tensors' device without blocking the host.
"""
from . import _dispatch
from ._c_api import SIGNATURES
from ._c_lib import device_library, host_library
from .checks import check_arguments, check_scalar


def _call(function, reference, tensors):
    """Invoke ``function`` with ``tensors`` in ABI order on the right device."""
    names = [name for _, name in SIGNATURES[function]]
    if _dispatch.on_device(reference):
        import torch

        # A host pointer handed to a device kernel is a memory fault, not an
        # exception: refuse anything that does not live where `reference` does.
        for name, tensor in zip(names, tensors):
            if tensor is None:
                continue
            if not _dispatch.is_torch(tensor):
                raise TypeError(
                    f"`{name}` must be a torch tensor on {reference.device} in {function} "
                    f"(the first tensor is there), got {type(tensor)}"
                )
            if tensor.device != reference.device:
                raise ValueError(
                    f"`{name}` is on {tensor.device} but the first tensor is on "
                    f"{reference.device} in {function}: all tensors must be on the same device"
                )
        library = device_library()
        with torch.cuda.device(reference.device):
            stream = torch.cuda.current_stream(reference.device)
            library.cdll.mops_amd_set_stream(stream.cuda_stream)
            library.cdll.mops_amd_set_synchronous(0)
            library.call(function, *tensors)
    else:
        for name, tensor in zip(names, tensors):
            if tensor is not None and _dispatch.on_device(tensor):
                raise ValueError(
                    f"`{name}` is on {tensor.device} but the first tensor is in host memory "
                    f"in {function}: all tensors must be on the same device"
                )
        host_library().call(function, *tensors)


def _floats(*arrays):
    return [None if a is None else _dispatch.contiguous(a) for a in arrays]


def _indices(*arrays):
    return [_dispatch.as_int32(a) for a in arrays]


def _optional(requested, like):
    return _dispatch.empty(like.shape, like) if requested else None


# ------------------------------------------------------------------- HPE ----
def homogeneous_polynomial_evaluation(A, C, indices_A):
    function = "homogeneous_polynomial_evaluation"
    check_arguments(function, {"A": A, "C": C, "indices_A": indices_A})
    A, C = _floats(A, C)
    (indices_A,) = _indices(indices_A)
    output = _dispatch.empty((A.shape[0],), A)
    _call(function, A, [output, A, C, indices_A])
    return output


def homogeneous_polynomial_evaluation_vjp(grad_output, A, C, indices_A, compute_grad_A=True):
    function = "homogeneous_polynomial_evaluation_vjp"
    check_arguments(
        function, {"grad_output": grad_output, "A": A, "C": C, "indices_A": indices_A}
    )
    grad_output, A, C = _floats(grad_output, A, C)
    (indices_A,) = _indices(indices_A)
    grad_A = _optional(compute_grad_A, A)
    _call(function, A, [grad_A, grad_output, A, C, indices_A])
    return grad_A


def homogeneous_polynomial_evaluation_vjp_vjp(
    grad_grad_A,
    grad_output,
    A,
    C,
    indices_A,
    compute_grad_grad_output=True,
    compute_grad_A_2=True,
):
    function = "homogeneous_polynomial_evaluation_vjp_vjp"
    check_arguments(
        function,
        {"grad_grad_A": grad_grad_A, "grad_output": grad_output, "A": A, "C": C, "indices_A": indices_A},
    )
    grad_grad_A, grad_output, A, C = _floats(grad_grad_A, grad_output, A, C)
    (indices_A,) = _indices(indices_A)
    grad_grad_output = _optional(compute_grad_grad_output, grad_output)
    grad_A_2 = _optional(compute_grad_A_2, A)
    _call(function, A, [grad_grad_output, grad_A_2, grad_grad_A, grad_output, A, C, indices_A])
    return grad_grad_output, grad_A_2


# ------------------------------------------------------------------- SAP ----
def sparse_accumulation_of_products(A, B, C, indices_A, indices_B, indices_output, output_size):
    function = "sparse_accumulation_of_products"
    check_arguments(
        function,
        {"A": A, "B": B, "C": C, "indices_A": indices_A, "indices_B": indices_B,
         "indices_output": indices_output},
    )  # fmt: skip
    check_scalar(output_size, function, "output_size")
    A, B, C = _floats(A, B, C)
    indices_A, indices_B, indices_output = _indices(indices_A, indices_B, indices_output)
    output = _dispatch.empty((A.shape[0], output_size), A)
    _call(function, A, [output, A, B, C, indices_A, indices_B, indices_output])
    return output


def sparse_accumulation_of_products_vjp(
    grad_output,
    A,
    B,
    C,
    indices_A,
    indices_B,
    indices_output,
    compute_grad_A=True,
    compute_grad_B=True,
):
    function = "sparse_accumulation_of_products_vjp"
    check_arguments(
        function,
        {"grad_output": grad_output, "A": A, "B": B, "C": C, "indices_A": indices_A,
         "indices_B": indices_B, "indices_output": indices_output},
    )  # fmt: skip
    grad_output, A, B, C = _floats(grad_output, A, B, C)
    indices_A, indices_B, indices_output = _indices(indices_A, indices_B, indices_output)
    grad_A = _optional(compute_grad_A, A)
    grad_B = _optional(compute_grad_B, B)
    _call(function, A, [grad_A, grad_B, grad_output, A, B, C, indices_A, indices_B, indices_output])
    return grad_A, grad_B


def sparse_accumulation_of_products_vjp_vjp(
    grad_grad_A,
    grad_grad_B,
    grad_output,
    A,
    B,
    C,
    indices_A,
    indices_B,
    indices_output,
    compute_grad_grad_output=True,
    compute_grad_A_2=True,
    compute_grad_B_2=True,
):
    function = "sparse_accumulation_of_products_vjp_vjp"
    check_arguments(
        function,
        {"grad_grad_A": grad_grad_A, "grad_grad_B": grad_grad_B, "grad_output": grad_output,
         "A": A, "B": B, "C": C, "indices_A": indices_A, "indices_B": indices_B,
         "indices_output": indices_output},
    )  # fmt: skip
    grad_grad_A, grad_grad_B, grad_output, A, B, C = _floats(
        grad_grad_A, grad_grad_B, grad_output, A, B, C
    )
    indices_A, indices_B, indices_output = _indices(indices_A, indices_B, indices_output)
    grad_grad_output = _optional(compute_grad_grad_output, grad_output)
    grad_A_2 = _optional(compute_grad_A_2, A)
    grad_B_2 = _optional(compute_grad_B_2, B)
    _call(
        function,
        A,
        [grad_grad_output, grad_A_2, grad_B_2, grad_grad_A, grad_grad_B, grad_output, A, B, C,
         indices_A, indices_B, indices_output],
    )  # fmt: skip
    return grad_grad_output, grad_A_2, grad_B_2


# ------------------------------------------------------------------ OPSA ----
def outer_product_scatter_add(A, B, indices_output, output_size):
    function = "outer_product_scatter_add"
    check_arguments(function, {"A": A, "B": B, "indices_output": indices_output})
    check_scalar(output_size, function, "output_size")
    A, B = _floats(A, B)
    (indices_output,) = _indices(indices_output)
    output = _dispatch.empty((output_size, A.shape[1], B.shape[1]), A)
    _call(function, A, [output, A, B, indices_output])
    return output


def outer_product_scatter_add_vjp(
    grad_output, A, B, indices_output, compute_grad_A=True, compute_grad_B=True
):
    function = "outer_product_scatter_add_vjp"
    check_arguments(
        function, {"grad_output": grad_output, "A": A, "B": B, "indices_output": indices_output}
    )
    grad_output, A, B = _floats(grad_output, A, B)
    (indices_output,) = _indices(indices_output)
    grad_A = _optional(compute_grad_A, A)
    grad_B = _optional(compute_grad_B, B)
    _call(function, A, [grad_A, grad_B, grad_output, A, B, indices_output])
    return grad_A, grad_B


def outer_product_scatter_add_vjp_vjp(
    grad_grad_A,
    grad_grad_B,
    grad_output,
    A,
    B,
    indices_output,
    compute_grad_grad_output=True,
    compute_grad_A_2=True,
    compute_grad_B_2=True,
):
    function = "outer_product_scatter_add_vjp_vjp"
    check_arguments(
        function,
        {"grad_grad_A": grad_grad_A, "grad_grad_B": grad_grad_B, "grad_output": grad_output,
         "A": A, "B": B, "indices_output": indices_output},
    )  # fmt: skip
    grad_grad_A, grad_grad_B, grad_output, A, B = _floats(grad_grad_A, grad_grad_B, grad_output, A, B)
    (indices_output,) = _indices(indices_output)
    grad_grad_output = _optional(compute_grad_grad_output, grad_output)
    grad_A_2 = _optional(compute_grad_A_2, A)
    grad_B_2 = _optional(compute_grad_B_2, B)
    _call(
        function,
        A,
        [grad_grad_output, grad_A_2, grad_B_2, grad_grad_A, grad_grad_B, grad_output, A, B, indices_output],
    )
    return grad_grad_output, grad_A_2, grad_B_2


# ----------------------------------------------------------------- OPSAW ----
def outer_product_scatter_add_with_weights(A, B, W, indices_W, indices_output):
    function = "outer_product_scatter_add_with_weights"
    check_arguments(
        function, {"A": A, "B": B, "W": W, "indices_W": indices_W, "indices_output": indices_output}
    )
    A, B, W = _floats(A, B, W)
    indices_W, indices_output = _indices(indices_W, indices_output)
    output = _dispatch.empty((W.shape[0], A.shape[1], B.shape[1]), A)
    _call(function, A, [output, A, B, W, indices_W, indices_output])
    return output


def outer_product_scatter_add_with_weights_vjp(
    grad_output,
    A,
    B,
    W,
    indices_W,
    indices_output,
    compute_grad_A=True,
    compute_grad_B=True,
    compute_grad_W=True,
):
    function = "outer_product_scatter_add_with_weights_vjp"
    check_arguments(
        function,
        {"grad_output": grad_output, "A": A, "B": B, "W": W, "indices_W": indices_W,
         "indices_output": indices_output},
    )  # fmt: skip
    grad_output, A, B, W = _floats(grad_output, A, B, W)
    indices_W, indices_output = _indices(indices_W, indices_output)
    grad_A = _optional(compute_grad_A, A)
    grad_B = _optional(compute_grad_B, B)
    grad_W = _optional(compute_grad_W, W)
    _call(function, A, [grad_A, grad_B, grad_W, grad_output, A, B, W, indices_W, indices_output])
    return grad_A, grad_B, grad_W


def outer_product_scatter_add_with_weights_vjp_vjp(
    grad_grad_A,
    grad_grad_B,
    grad_grad_W,
    grad_output,
    A,
    B,
    W,
    indices_W,
    indices_output,
    compute_grad_grad_output=True,
    compute_grad_A_2=True,
    compute_grad_B_2=True,
    compute_grad_W_2=True,
):
    function = "outer_product_scatter_add_with_weights_vjp_vjp"
    check_arguments(
        function,
        {"grad_grad_A": grad_grad_A, "grad_grad_B": grad_grad_B, "grad_grad_W": grad_grad_W,
         "grad_output": grad_output, "A": A, "B": B, "W": W, "indices_W": indices_W,
         "indices_output": indices_output},
    )  # fmt: skip
    grad_grad_A, grad_grad_B, grad_grad_W, grad_output, A, B, W = _floats(
        grad_grad_A, grad_grad_B, grad_grad_W, grad_output, A, B, W
    )
    indices_W, indices_output = _indices(indices_W, indices_output)
    grad_grad_output = _optional(compute_grad_grad_output, grad_output)
    grad_A_2 = _optional(compute_grad_A_2, A)
    grad_B_2 = _optional(compute_grad_B_2, B)
    grad_W_2 = _optional(compute_grad_W_2, W)
    _call(
        function,
        A,
        [grad_grad_output, grad_A_2, grad_B_2, grad_W_2, grad_grad_A, grad_grad_B, grad_grad_W,
         grad_output, A, B, W, indices_W, indices_output],
    )  # fmt: skip
    return grad_grad_output, grad_A_2, grad_B_2, grad_W_2


# ----------------------------------------------------------------- SASAW ----
def sparse_accumulation_scatter_add_with_weights(
    A,
    B,
    C,
    W,
    indices_A,
    indices_W_1,
    indices_W_2,
    indices_output_1,
    indices_output_2,
    output_size,
):
    function = "sparse_accumulation_scatter_add_with_weights"
    check_arguments(
        function,
        {"A": A, "B": B, "C": C, "W": W, "indices_A": indices_A, "indices_W_1": indices_W_1,
         "indices_W_2": indices_W_2, "indices_output_1": indices_output_1,
         "indices_output_2": indices_output_2},
    )  # fmt: skip
    check_scalar(output_size, function, "output_size")
    A, B, C, W = _floats(A, B, C, W)
    indices_A, indices_W_1, indices_W_2, indices_output_1, indices_output_2 = _indices(
        indices_A, indices_W_1, indices_W_2, indices_output_1, indices_output_2
    )
    output = _dispatch.empty((W.shape[0], output_size, B.shape[1]), A)
    _call(
        function,
        A,
        [output, A, B, C, W, indices_A, indices_W_1, indices_W_2, indices_output_1, indices_output_2],
    )
    return output


def sparse_accumulation_scatter_add_with_weights_vjp(
    grad_output,
    A,
    B,
    C,
    W,
    indices_A,
    indices_W_1,
    indices_W_2,
    indices_output_1,
    indices_output_2,
    compute_grad_A=True,
    compute_grad_B=True,
    compute_grad_C=True,
    compute_grad_W=True,
):
    # compute_grad_C is accepted for signature compatibility and ignored, as
    # in the reference: there is no gradient with respect to C.
    function = "sparse_accumulation_scatter_add_with_weights_vjp"
    check_arguments(
        function,
        {"grad_output": grad_output, "A": A, "B": B, "C": C, "W": W, "indices_A": indices_A,
         "indices_W_1": indices_W_1, "indices_W_2": indices_W_2,
         "indices_output_1": indices_output_1, "indices_output_2": indices_output_2},
    )  # fmt: skip
    grad_output, A, B, C, W = _floats(grad_output, A, B, C, W)
    indices_A, indices_W_1, indices_W_2, indices_output_1, indices_output_2 = _indices(
        indices_A, indices_W_1, indices_W_2, indices_output_1, indices_output_2
    )
    grad_A = _optional(compute_grad_A, A)
    grad_B = _optional(compute_grad_B, B)
    grad_W = _optional(compute_grad_W, W)
    _call(
        function,
        A,
        [grad_A, grad_B, grad_W, grad_output, A, B, C, W, indices_A, indices_W_1, indices_W_2,
         indices_output_1, indices_output_2],
    )  # fmt: skip
    return grad_A, grad_B, grad_W


def sparse_accumulation_scatter_add_with_weights_vjp_vjp(
    grad_grad_A,
    grad_grad_B,
    grad_grad_W,
    grad_output,
    A,
    B,
    C,
    W,
    indices_A,
    indices_W_1,
    indices_W_2,
    indices_output_1,
    indices_output_2,
    compute_grad_grad_output=True,
    compute_grad_A_2=True,
    compute_grad_B_2=True,
    compute_grad_W_2=True,
):
    function = "sparse_accumulation_scatter_add_with_weights_vjp_vjp"
    check_arguments(
        function,
        {"grad_grad_A": grad_grad_A, "grad_grad_B": grad_grad_B, "grad_grad_W": grad_grad_W,
         "grad_output": grad_output, "A": A, "B": B, "C": C, "W": W, "indices_A": indices_A,
         "indices_W_1": indices_W_1, "indices_W_2": indices_W_2,
         "indices_output_1": indices_output_1, "indices_output_2": indices_output_2},
    )  # fmt: skip
    grad_grad_A, grad_grad_B, grad_grad_W, grad_output, A, B, C, W = _floats(
        grad_grad_A, grad_grad_B, grad_grad_W, grad_output, A, B, C, W
    )
    indices_A, indices_W_1, indices_W_2, indices_output_1, indices_output_2 = _indices(
        indices_A, indices_W_1, indices_W_2, indices_output_1, indices_output_2
    )
    grad_grad_output = _optional(compute_grad_grad_output, grad_output)
    grad_A_2 = _optional(compute_grad_A_2, A)
    grad_B_2 = _optional(compute_grad_B_2, B)
    grad_W_2 = _optional(compute_grad_W_2, W)
    _call(
        function,
        A,
        [grad_grad_output, grad_A_2, grad_B_2, grad_W_2, grad_grad_A, grad_grad_B, grad_grad_W,
         grad_output, A, B, C, W, indices_A, indices_W_1, indices_W_2, indices_output_1,
         indices_output_2],
    )  # fmt: skip
    return grad_grad_output, grad_A_2, grad_B_2, grad_W_2


def first_occurrences(sorted_indices, output_size):
    """Segment boundaries of a sorted int32 device tensor.

    Returns an int32 tensor of shape ``[2, output_size]``: row 0 holds the
    position of the first element equal to ``v``, row 1 one past the last, and
    both are -1 where ``v`` does not occur.
    """
    import torch

    if not _dispatch.on_device(sorted_indices):
        raise TypeError("first_occurrences needs an int32 tensor on a ROCm device")
    sorted_indices = _dispatch.as_int32(sorted_indices)
    result = torch.empty((2, output_size), dtype=torch.int32, device=sorted_indices.device)
    library = device_library()
    with torch.cuda.device(sorted_indices.device):
        stream = torch.cuda.current_stream(sorted_indices.device)
        library.cdll.mops_amd_set_stream(stream.cuda_stream)
        library.cdll.mops_amd_set_synchronous(0)
        status = library.cdll.mops_amd_first_occurrences(
            sorted_indices.data_ptr(), sorted_indices.shape[0], output_size, result.data_ptr()
        )
    if status != 0:
        from .status import MopsError

        raise MopsError(library.last_error(), status)
    return result


# ----------------------------------------------------- unsorted indices ----
def accept_unsorted_indices(accept=True):
    """Let the scatter operations take a scatter index in any order (this thread).

    The device kernels need ``indices_output`` / ``indices_output_1`` sorted,
    like the reference's device path; with this switch on, every call tests
    the index on the device and re-orders the edges by a stable sort when it
    has to, which gives the results of the reference's host path
    (``mops/src/opsa/cpu.tpp:29``). Costs one wait for the device per call.
    Returns the previous setting.
    """
    return bool(device_library().cdll.mops_amd_accept_unsorted_indices(1 if accept else 0))
