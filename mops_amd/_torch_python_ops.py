"""Registration of ``torch.ops.mops.*`` from Python, over the C ABI.

Used by ``mops_amd.torch`` when the C++ operators (``mops_amd/csrc/torch_ops.cpp``) have not been
built, or when ``MOPS_AMD_TORCH_PYTHON_OPS=1`` asks for it. Same operators, schemas, gradients and
second derivatives; every call goes through the interpreter (and the backward passes through
``torch.library``'s Python autograd), which costs some hundred microseconds per forward + backward.
"""
import torch

from . import ops as _ops


_library = torch.library.Library("mops", "DEF")
_library.define("homogeneous_polynomial_evaluation(Tensor A, Tensor C, Tensor indices_A) -> Tensor")
_library.define(
    "outer_product_scatter_add(Tensor A, Tensor B, Tensor indices_output, int output_size) -> Tensor"
)
_library.define(
    "sparse_accumulation_of_products(Tensor A, Tensor B, Tensor C, Tensor indices_A, Tensor indices_B, "
    "Tensor indices_output, int output_size) -> Tensor"
)
_library.define(
    "outer_product_scatter_add_with_weights(Tensor A, Tensor B, Tensor W, Tensor indices_W, "
    "Tensor indices_output) -> Tensor"
)
_library.define(
    "sparse_accumulation_scatter_add_with_weights(Tensor A, Tensor B, Tensor C, Tensor W, Tensor indices_A, "
    "Tensor indices_W_1, Tensor indices_W_2, Tensor indices_output_1, Tensor indices_output_2, "
    "int output_size) -> Tensor"
)
# the vector-Jacobian products, as operators of their own so that the
# backward pass is a dispatcher call as well (bool[] mask: which gradients)
_library.define(
    "homogeneous_polynomial_evaluation_vjp(Tensor grad_output, Tensor A, Tensor C, Tensor indices_A) -> Tensor"
)
_library.define(
    "outer_product_scatter_add_vjp(Tensor grad_output, Tensor A, Tensor B, Tensor indices_output, "
    "bool[2] wanted) -> (Tensor, Tensor)"
)
_library.define(
    "sparse_accumulation_of_products_vjp(Tensor grad_output, Tensor A, Tensor B, Tensor C, Tensor indices_A, "
    "Tensor indices_B, Tensor indices_output, bool[2] wanted) -> (Tensor, Tensor)"
)
_library.define(
    "outer_product_scatter_add_with_weights_vjp(Tensor grad_output, Tensor A, Tensor B, Tensor W, "
    "Tensor indices_W, Tensor indices_output, bool[3] wanted) -> (Tensor, Tensor, Tensor)"
)
_library.define(
    "sparse_accumulation_scatter_add_with_weights_vjp(Tensor grad_output, Tensor A, Tensor B, Tensor C, "
    "Tensor W, Tensor indices_A, Tensor indices_W_1, Tensor indices_W_2, Tensor indices_output_1, "
    "Tensor indices_output_2, bool[3] wanted) -> (Tensor, Tensor, Tensor)"
)
# second order: cotangents of the vjp's outputs in, cotangents of its inputs out;
# `have`: which cotangents are given (the others are empty tensors), `wanted`:
# which of (grad_grad_output, grad_A_2[, grad_B_2]) are computed
_library.define(
    "homogeneous_polynomial_evaluation_vjp_vjp(Tensor grad_grad_A, Tensor grad_output, Tensor A, Tensor C, "
    "Tensor indices_A, bool[2] wanted) -> (Tensor, Tensor)"
)
_library.define(
    "outer_product_scatter_add_vjp_vjp(Tensor grad_grad_A, Tensor grad_grad_B, Tensor grad_output, Tensor A, "
    "Tensor B, Tensor indices_output, bool[2] have, bool[3] wanted) -> (Tensor, Tensor, Tensor)"
)
_library.define(
    "sparse_accumulation_of_products_vjp_vjp(Tensor grad_grad_A, Tensor grad_grad_B, Tensor grad_output, "
    "Tensor A, Tensor B, Tensor C, Tensor indices_A, Tensor indices_B, Tensor indices_output, bool[2] have, "
    "bool[3] wanted) -> (Tensor, Tensor, Tensor)"
)


def _or_empty(gradient, like):
    """Operators cannot return None: a gradient that was not asked for is an empty tensor."""
    return gradient if gradient is not None else like.new_empty((0,))


# ----------------------------------------------------------------- kernels --
def _hpe(A, C, indices_A):
    return _ops.homogeneous_polynomial_evaluation(A, C, indices_A)


def _hpe_vjp(grad_output, A, C, indices_A):
    return _ops.homogeneous_polynomial_evaluation_vjp(grad_output, A, C, indices_A)


def _hpe_vjp_vjp(grad_grad_A, grad_output, A, C, indices_A, wanted):
    grad_grad_output, grad_A_2 = _ops.homogeneous_polynomial_evaluation_vjp_vjp(
        grad_grad_A, grad_output, A, C, indices_A,
        compute_grad_grad_output=wanted[0], compute_grad_A_2=wanted[1],
    )  # fmt: skip
    return _or_empty(grad_grad_output, A), _or_empty(grad_A_2, A)


def _opsa_vjp_vjp(grad_grad_A, grad_grad_B, grad_output, A, B, indices_output, have, wanted):
    grad_grad_output, grad_A_2, grad_B_2 = _ops.outer_product_scatter_add_vjp_vjp(
        grad_grad_A if have[0] else None, grad_grad_B if have[1] else None, grad_output, A, B, indices_output,
        compute_grad_grad_output=wanted[0], compute_grad_A_2=wanted[1], compute_grad_B_2=wanted[2],
    )  # fmt: skip
    return _or_empty(grad_grad_output, A), _or_empty(grad_A_2, A), _or_empty(grad_B_2, B)


def _sap_vjp_vjp(
    grad_grad_A, grad_grad_B, grad_output, A, B, C, indices_A, indices_B, indices_output, have, wanted
):
    grad_grad_output, grad_A_2, grad_B_2 = _ops.sparse_accumulation_of_products_vjp_vjp(
        grad_grad_A if have[0] else None, grad_grad_B if have[1] else None, grad_output, A, B, C,
        indices_A, indices_B, indices_output,
        compute_grad_grad_output=wanted[0], compute_grad_A_2=wanted[1], compute_grad_B_2=wanted[2],
    )  # fmt: skip
    return _or_empty(grad_grad_output, A), _or_empty(grad_A_2, A), _or_empty(grad_B_2, B)


def _opsa(A, B, indices_output, output_size):
    return _ops.outer_product_scatter_add(A, B, indices_output, output_size)


def _opsa_vjp(grad_output, A, B, indices_output, wanted):
    grad_A, grad_B = _ops.outer_product_scatter_add_vjp(
        grad_output, A, B, indices_output, compute_grad_A=wanted[0], compute_grad_B=wanted[1]
    )
    return _or_empty(grad_A, A), _or_empty(grad_B, B)


def _sap(A, B, C, indices_A, indices_B, indices_output, output_size):
    return _ops.sparse_accumulation_of_products(A, B, C, indices_A, indices_B, indices_output, output_size)


def _sap_vjp(grad_output, A, B, C, indices_A, indices_B, indices_output, wanted):
    grad_A, grad_B = _ops.sparse_accumulation_of_products_vjp(
        grad_output, A, B, C, indices_A, indices_B, indices_output,
        compute_grad_A=wanted[0], compute_grad_B=wanted[1],
    )  # fmt: skip
    return _or_empty(grad_A, A), _or_empty(grad_B, B)


def _opsaw(A, B, W, indices_W, indices_output):
    return _ops.outer_product_scatter_add_with_weights(A, B, W, indices_W, indices_output)


def _opsaw_vjp(grad_output, A, B, W, indices_W, indices_output, wanted):
    grad_A, grad_B, grad_W = _ops.outer_product_scatter_add_with_weights_vjp(
        grad_output, A, B, W, indices_W, indices_output,
        compute_grad_A=wanted[0], compute_grad_B=wanted[1], compute_grad_W=wanted[2],
    )  # fmt: skip
    return _or_empty(grad_A, A), _or_empty(grad_B, B), _or_empty(grad_W, W)


def _sasaw(A, B, C, W, indices_A, indices_W_1, indices_W_2, indices_output_1, indices_output_2, output_size):
    return _ops.sparse_accumulation_scatter_add_with_weights(
        A, B, C, W, indices_A, indices_W_1, indices_W_2, indices_output_1, indices_output_2, output_size
    )


def _sasaw_vjp(
    grad_output, A, B, C, W, indices_A, indices_W_1, indices_W_2, indices_output_1, indices_output_2, wanted
):
    grad_A, grad_B, grad_W = _ops.sparse_accumulation_scatter_add_with_weights_vjp(
        grad_output, A, B, C, W, indices_A, indices_W_1, indices_W_2, indices_output_1, indices_output_2,
        compute_grad_A=wanted[0], compute_grad_B=wanted[1], compute_grad_W=wanted[2],
    )  # fmt: skip
    return _or_empty(grad_A, A), _or_empty(grad_B, B), _or_empty(grad_W, W)


for _name, _kernel in [
    ("homogeneous_polynomial_evaluation", _hpe),
    ("homogeneous_polynomial_evaluation_vjp", _hpe_vjp),
    ("outer_product_scatter_add", _opsa),
    ("outer_product_scatter_add_vjp", _opsa_vjp),
    ("sparse_accumulation_of_products", _sap),
    ("sparse_accumulation_of_products_vjp", _sap_vjp),
    ("outer_product_scatter_add_with_weights", _opsaw),
    ("outer_product_scatter_add_with_weights_vjp", _opsaw_vjp),
    ("sparse_accumulation_scatter_add_with_weights", _sasaw),
    ("sparse_accumulation_scatter_add_with_weights_vjp", _sasaw_vjp),
    ("homogeneous_polynomial_evaluation_vjp_vjp", _hpe_vjp_vjp),
    ("outer_product_scatter_add_vjp_vjp", _opsa_vjp_vjp),
    ("sparse_accumulation_of_products_vjp_vjp", _sap_vjp_vjp),
]:
    # ROCm tensors carry the CUDA dispatch key
    _library.impl(_name, _kernel, "CUDA")


def _refuse_host(name):
    def kernel(*args):
        raise RuntimeError(
            f"mops::{name}: tensors must be on a ROCm device; this library implements the device path only"
        )

    return kernel


for _name in [
    "homogeneous_polynomial_evaluation",
    "outer_product_scatter_add",
    "sparse_accumulation_of_products",
    "outer_product_scatter_add_with_weights",
    "sparse_accumulation_scatter_add_with_weights",
]:
    _library.impl(_name, _refuse_host(_name), "CPU")
    _library.impl(_name + "_vjp", _refuse_host(_name + "_vjp"), "CPU")
for _name in [
    "homogeneous_polynomial_evaluation_vjp_vjp",
    "outer_product_scatter_add_vjp_vjp",
    "sparse_accumulation_of_products_vjp_vjp",
]:
    _library.impl(_name, _refuse_host(_name), "CPU")


# ------------------------------------------------------------------ shapes --
# (FakeTensor / torch.compile support: output shapes without running anything)
def _register_fake(name, function):
    torch.library.register_fake(f"mops::{name}", function, lib=_library)


_register_fake("homogeneous_polynomial_evaluation", lambda A, C, indices_A: A.new_empty((A.shape[0],)))
_register_fake(
    "outer_product_scatter_add",
    lambda A, B, indices_output, output_size: A.new_empty((output_size, A.shape[1], B.shape[1])),
)
_register_fake(
    "sparse_accumulation_of_products",
    lambda A, B, C, indices_A, indices_B, indices_output, output_size: A.new_empty((A.shape[0], output_size)),
)
_register_fake(
    "outer_product_scatter_add_with_weights",
    lambda A, B, W, indices_W, indices_output: A.new_empty((W.shape[0], A.shape[1], B.shape[1])),
)
_register_fake(
    "sparse_accumulation_scatter_add_with_weights",
    lambda A, B, C, W, indices_A, indices_W_1, indices_W_2, indices_output_1, indices_output_2, output_size: (
        A.new_empty((W.shape[0], output_size, B.shape[1]))
    ),
)


# ---------------------------------------------------------------- autograd --
def _hpe_setup(ctx, inputs, output):
    ctx.save_for_backward(*inputs)


def _hpe_backward(ctx, grad_output):
    A, C, indices_A = ctx.saved_tensors
    grad_A = None
    if ctx.needs_input_grad[0]:
        grad_A = torch.ops.mops.homogeneous_polynomial_evaluation_vjp(
            grad_output.contiguous(), A, C, indices_A
        )
    if ctx.needs_input_grad[1]:
        raise RuntimeError("gradients with respect to C are not supported")
    return grad_A, None, None


def _opsa_setup(ctx, inputs, output):
    A, B, indices_output, _ = inputs
    ctx.save_for_backward(A, B, indices_output)


def _opsa_backward(ctx, grad_output):
    A, B, indices_output = ctx.saved_tensors
    wanted = [ctx.needs_input_grad[0], ctx.needs_input_grad[1]]
    grad_A, grad_B = torch.ops.mops.outer_product_scatter_add_vjp(
        grad_output.contiguous(), A, B, indices_output, wanted
    )
    return grad_A if wanted[0] else None, grad_B if wanted[1] else None, None, None


def _sap_setup(ctx, inputs, output):
    ctx.save_for_backward(*inputs[:6])


def _sap_backward(ctx, grad_output):
    A, B, C, indices_A, indices_B, indices_output = ctx.saved_tensors
    if ctx.needs_input_grad[2]:
        raise RuntimeError("gradients with respect to C are not supported")
    wanted = [ctx.needs_input_grad[0], ctx.needs_input_grad[1]]
    grad_A, grad_B = torch.ops.mops.sparse_accumulation_of_products_vjp(
        grad_output.contiguous(), A, B, C, indices_A, indices_B, indices_output, wanted
    )
    return (grad_A if wanted[0] else None, grad_B if wanted[1] else None, None, None, None, None, None)


def _opsaw_setup(ctx, inputs, output):
    ctx.save_for_backward(*inputs)


def _opsaw_backward(ctx, grad_output):
    A, B, W, indices_W, indices_output = ctx.saved_tensors
    wanted = [ctx.needs_input_grad[0], ctx.needs_input_grad[1], ctx.needs_input_grad[2]]
    grad_A, grad_B, grad_W = torch.ops.mops.outer_product_scatter_add_with_weights_vjp(
        grad_output.contiguous(), A, B, W, indices_W, indices_output, wanted
    )
    return (
        grad_A if wanted[0] else None, grad_B if wanted[1] else None, grad_W if wanted[2] else None,
        None, None,
    )  # fmt: skip


def _sasaw_setup(ctx, inputs, output):
    ctx.save_for_backward(*inputs[:9])


def _sasaw_backward(ctx, grad_output):
    A, B, C, W, indices_A, indices_W_1, indices_W_2, indices_output_1, indices_output_2 = ctx.saved_tensors
    if ctx.needs_input_grad[2]:
        raise RuntimeError("gradients with respect to C are not supported")
    wanted = [ctx.needs_input_grad[0], ctx.needs_input_grad[1], ctx.needs_input_grad[3]]
    grad_A, grad_B, grad_W = torch.ops.mops.sparse_accumulation_scatter_add_with_weights_vjp(
        grad_output.contiguous(), A, B, C, W, indices_A, indices_W_1, indices_W_2, indices_output_1,
        indices_output_2, wanted,
    )  # fmt: skip
    return (
        grad_A if wanted[0] else None, grad_B if wanted[1] else None, None, grad_W if wanted[2] else None,
        None, None, None, None, None, None,
    )  # fmt: skip


# ---- second order: backward of the *_vjp operators of HPE, OPSA and SAP ----
def _given(cotangent, wanted):
    """A cotangent counts when its output was computed and autograd passes one."""
    return bool(wanted) and cotangent is not None


def _hpe_vjp_setup(ctx, inputs, output):
    ctx.save_for_backward(*inputs)


def _hpe_vjp_backward(ctx, grad_grad_A):
    grad_output, A, C, indices_A = ctx.saved_tensors
    if ctx.needs_input_grad[2]:
        raise RuntimeError("gradients with respect to C are not supported")
    wanted = [ctx.needs_input_grad[0], ctx.needs_input_grad[1]]
    grad_grad_output, grad_A_2 = torch.ops.mops.homogeneous_polynomial_evaluation_vjp_vjp(
        grad_grad_A.contiguous(), grad_output, A, C, indices_A, wanted
    )
    return grad_grad_output if wanted[0] else None, grad_A_2 if wanted[1] else None, None, None


def _opsa_vjp_setup(ctx, inputs, output):
    grad_output, A, B, indices_output, wanted = inputs
    ctx.save_for_backward(grad_output, A, B, indices_output)
    ctx.computed = list(wanted)


def _opsa_vjp_backward(ctx, grad_grad_A, grad_grad_B):
    grad_output, A, B, indices_output = ctx.saved_tensors
    have = [_given(grad_grad_A, ctx.computed[0]), _given(grad_grad_B, ctx.computed[1])]
    wanted = [ctx.needs_input_grad[0], ctx.needs_input_grad[1], ctx.needs_input_grad[2]]
    grad_grad_output, grad_A_2, grad_B_2 = torch.ops.mops.outer_product_scatter_add_vjp_vjp(
        grad_grad_A.contiguous() if have[0] else A.new_empty((0,)),
        grad_grad_B.contiguous() if have[1] else B.new_empty((0,)),
        grad_output, A, B, indices_output, have, wanted,
    )  # fmt: skip
    return (
        grad_grad_output if wanted[0] else None, grad_A_2 if wanted[1] else None,
        grad_B_2 if wanted[2] else None, None, None,
    )  # fmt: skip


def _sap_vjp_setup(ctx, inputs, output):
    ctx.save_for_backward(*inputs[:7])
    ctx.computed = list(inputs[7])


def _sap_vjp_backward(ctx, grad_grad_A, grad_grad_B):
    grad_output, A, B, C, indices_A, indices_B, indices_output = ctx.saved_tensors
    if ctx.needs_input_grad[3]:
        raise RuntimeError("gradients with respect to C are not supported")
    have = [_given(grad_grad_A, ctx.computed[0]), _given(grad_grad_B, ctx.computed[1])]
    wanted = [ctx.needs_input_grad[0], ctx.needs_input_grad[1], ctx.needs_input_grad[2]]
    grad_grad_output, grad_A_2, grad_B_2 = torch.ops.mops.sparse_accumulation_of_products_vjp_vjp(
        grad_grad_A.contiguous() if have[0] else A.new_empty((0,)),
        grad_grad_B.contiguous() if have[1] else B.new_empty((0,)),
        grad_output, A, B, C, indices_A, indices_B, indices_output, have, wanted,
    )  # fmt: skip
    return (
        grad_grad_output if wanted[0] else None, grad_A_2 if wanted[1] else None,
        grad_B_2 if wanted[2] else None, None, None, None, None, None,
    )  # fmt: skip


for _name, _backward, _setup in [
    ("homogeneous_polynomial_evaluation_vjp", _hpe_vjp_backward, _hpe_vjp_setup),
    ("outer_product_scatter_add_vjp", _opsa_vjp_backward, _opsa_vjp_setup),
    ("sparse_accumulation_of_products_vjp", _sap_vjp_backward, _sap_vjp_setup),
    ("homogeneous_polynomial_evaluation", _hpe_backward, _hpe_setup),
    ("outer_product_scatter_add", _opsa_backward, _opsa_setup),
    ("sparse_accumulation_of_products", _sap_backward, _sap_setup),
    ("outer_product_scatter_add_with_weights", _opsaw_backward, _opsaw_setup),
    ("sparse_accumulation_scatter_add_with_weights", _sasaw_backward, _sasaw_setup),
]:
    torch.library.register_autograd(f"mops::{_name}", _backward, setup_context=_setup, lib=_library)


