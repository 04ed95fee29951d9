"""mops on AMD Instinct MI355X: the five sparse tensor operations of
lab-cosmo/mops and their vector-Jacobian products, as hand-written HIP kernels
for gfx950 behind mops' own C ABI, called here on PyTorch-ROCm tensors.

The public names are those of the reference's Python package
(``python/mops/src/mops/__init__.py`` of lab-cosmo/mops).
"""
from .ops import (  # noqa: F401
    accept_unsorted_indices,
    first_occurrences,
    homogeneous_polynomial_evaluation,
    homogeneous_polynomial_evaluation_vjp,
    homogeneous_polynomial_evaluation_vjp_vjp,
    outer_product_scatter_add,
    outer_product_scatter_add_vjp,
    outer_product_scatter_add_vjp_vjp,
    outer_product_scatter_add_with_weights,
    outer_product_scatter_add_with_weights_vjp,
    outer_product_scatter_add_with_weights_vjp_vjp,
    sparse_accumulation_of_products,
    sparse_accumulation_of_products_vjp,
    sparse_accumulation_of_products_vjp_vjp,
    sparse_accumulation_scatter_add_with_weights,
    sparse_accumulation_scatter_add_with_weights_vjp,
    sparse_accumulation_scatter_add_with_weights_vjp_vjp,
)
from .status import MopsError  # noqa: F401

__all__ = [name for name in dir() if not name.startswith("_")]
