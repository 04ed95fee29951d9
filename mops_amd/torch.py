"""``torch.ops.mops.*``: the five operations as PyTorch operators with autograd.

Same operator names and schemas as the reference's TorchScript extension
(``mops-torch/src/register.cpp:5-38`` of lab-cosmo/mops), so models written
against ``mops.torch`` call these without change::

    import mops_amd.torch            # registers the operators
    O = torch.ops.mops.outer_product_scatter_add(A, B, indices_output, output_size)

The operators come from the C++ library ``mops_amd/lib/libmops_amd_torch.so``
(``mops_amd/csrc/torch_ops.cpp``, built by ``mops_amd/csrc/build_torch_ops.py``)
when it has been built, and are otherwise registered from Python through
``torch.library`` (``mops_amd/_torch_python_ops.py``; ``MOPS_AMD_TORCH_PYTHON_OPS=1``
forces that). Either way ROCm tensors (which PyTorch reports as ``cuda``) go to
the HIP library on the current PyTorch stream. The backward of each operator is the
library's ``*_vjp`` function; only the gradients autograd asks for are
computed. As in the reference, tensors are made contiguous and there is no
gradient with respect to ``C`` or the index tensors. Second derivatives: the
``*_vjp`` operators of HPE, SAP and OPSA have a backward of their own, the
library's ``*_vjp_vjp`` functions (the operations for which the reference
has one, ``mops-torch/src/{hpe,sap,opsa}.cpp``); the two weighted operations
have none, as in the reference.

Host tensors are refused: this library is the device path only.
"""
import os

import torch

from ._c_lib import LIBRARY_PATH

__all__ = [
    "homogeneous_polynomial_evaluation",
    "sparse_accumulation_of_products",
    "outer_product_scatter_add",
    "outer_product_scatter_add_with_weights",
    "sparse_accumulation_scatter_add_with_weights",
    "OPERATORS_FROM",
]

CPP_OPERATORS_PATH = os.path.join(os.path.dirname(LIBRARY_PATH), "libmops_amd_torch.so")

if os.path.exists(CPP_OPERATORS_PATH) and os.environ.get("MOPS_AMD_TORCH_PYTHON_OPS", "0") in ("", "0"):
    torch.ops.load_library(CPP_OPERATORS_PATH)
    OPERATORS_FROM = "c++"
else:
    from . import _torch_python_ops  # noqa: F401  (registers the operators)

    OPERATORS_FROM = "python"

homogeneous_polynomial_evaluation = torch.ops.mops.homogeneous_polynomial_evaluation
sparse_accumulation_of_products = torch.ops.mops.sparse_accumulation_of_products
outer_product_scatter_add = torch.ops.mops.outer_product_scatter_add
outer_product_scatter_add_with_weights = torch.ops.mops.outer_product_scatter_add_with_weights
sparse_accumulation_scatter_add_with_weights = torch.ops.mops.sparse_accumulation_scatter_add_with_weights
