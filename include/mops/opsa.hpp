// C++ API of outer_product_scatter_add (OPSA).
//
//   O[indices_output[j], :, :] += A[j, :, None] * B[j, None, :]
//
// Declares, in namespace mops (host memory) and again in namespace
// mops::cuda (device memory, HIP implementation for gfx950):
//
//   template <typename scalar_t> void outer_product_scatter_add(...);
//   template <typename scalar_t> void outer_product_scatter_add_vjp(...);
//   template <typename scalar_t> void outer_product_scatter_add_vjp_vjp(...);
//
// with float and double precompiled in the library. Tensors are passed by
// value as mops::Tensor views, outputs first; a gradient whose data pointer
// is null is skipped. Replaces mops/include/mops/opsa.hpp:32-245 of lab-cosmo/mops
// with identical template names, namespaces and argument orders (the orders
// are spelled once in mops/detail/signatures.h).
#ifndef MOPS_OPSA_HPP
#define MOPS_OPSA_HPP

#include <cstdint>

#include "mops/exports.h"
#include "mops/tensor.hpp"
#include "mops/detail/signatures.h"

#define MOPS_OPSA_DECLARE_API()                                                                     \
    MOPS_CXX_DECLARE(outer_product_scatter_add, MOPS_OPSA_PARAMS)                                                      \
    MOPS_CXX_DECLARE(outer_product_scatter_add_vjp, MOPS_OPSA_VJP_PARAMS)                                              \
    MOPS_CXX_DECLARE(outer_product_scatter_add_vjp_vjp, MOPS_OPSA_VJP_VJP_PARAMS)

namespace mops {
MOPS_OPSA_DECLARE_API()
namespace cuda {
MOPS_OPSA_DECLARE_API()
} // namespace cuda
} // namespace mops

#undef MOPS_OPSA_DECLARE_API

#endif
