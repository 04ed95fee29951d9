// C++ API of outer_product_scatter_add_with_weights (OPSAW).
//
//   O[indices_output[e], :, :] += A[e, :, None] * B[e, None, :] * W[indices_W[e], None, :]
//
// Declares, in namespace mops (host memory) and again in namespace
// mops::cuda (device memory, HIP implementation for gfx950):
//
//   template <typename scalar_t> void outer_product_scatter_add_with_weights(...);
//   template <typename scalar_t> void outer_product_scatter_add_with_weights_vjp(...);
//   template <typename scalar_t> void outer_product_scatter_add_with_weights_vjp_vjp(...);
//
// with float and double precompiled in the library. Tensors are passed by
// value as mops::Tensor views, outputs first; a gradient whose data pointer
// is null is skipped. Replaces mops/include/mops/opsaw.hpp:31-290 of lab-cosmo/mops
// with identical template names, namespaces and argument orders (the orders
// are spelled once in mops/detail/signatures.h).
#ifndef MOPS_OPSAW_HPP
#define MOPS_OPSAW_HPP

#include <cstdint>

#include "mops/exports.h"
#include "mops/tensor.hpp"
#include "mops/detail/signatures.h"

#define MOPS_OPSAW_DECLARE_API()                                                                     \
    MOPS_CXX_DECLARE(outer_product_scatter_add_with_weights, MOPS_OPSAW_PARAMS)                                                      \
    MOPS_CXX_DECLARE(outer_product_scatter_add_with_weights_vjp, MOPS_OPSAW_VJP_PARAMS)                                              \
    MOPS_CXX_DECLARE(outer_product_scatter_add_with_weights_vjp_vjp, MOPS_OPSAW_VJP_VJP_PARAMS)

namespace mops {
MOPS_OPSAW_DECLARE_API()
namespace cuda {
MOPS_OPSAW_DECLARE_API()
} // namespace cuda
} // namespace mops

#undef MOPS_OPSAW_DECLARE_API

#endif
