// C++ API of sparse_accumulation_scatter_add_with_weights (SASAW).
//
//   O[indices_output_1[e], indices_output_2[n], :] += A[e, indices_A[n]] * B[e, :] * C[n] * W[indices_W_1[e], indices_W_2[n], :]
//
// Declares, in namespace mops (host memory) and again in namespace
// mops::cuda (device memory, HIP implementation for gfx950):
//
//   template <typename scalar_t> void sparse_accumulation_scatter_add_with_weights(...);
//   template <typename scalar_t> void sparse_accumulation_scatter_add_with_weights_vjp(...);
//   template <typename scalar_t> void sparse_accumulation_scatter_add_with_weights_vjp_vjp(...);
//
// with float and double precompiled in the library. Tensors are passed by
// value as mops::Tensor views, outputs first; a gradient whose data pointer
// is null is skipped. Replaces mops/include/mops/sasaw.hpp:40-372 of lab-cosmo/mops
// with identical template names, namespaces and argument orders (the orders
// are spelled once in mops/detail/signatures.h).
#ifndef MOPS_SASAW_HPP
#define MOPS_SASAW_HPP

#include <cstdint>

#include "mops/exports.h"
#include "mops/tensor.hpp"
#include "mops/detail/signatures.h"

#define MOPS_SASAW_DECLARE_API()                                                                     \
    MOPS_CXX_DECLARE(sparse_accumulation_scatter_add_with_weights, MOPS_SASAW_PARAMS)                                                      \
    MOPS_CXX_DECLARE(sparse_accumulation_scatter_add_with_weights_vjp, MOPS_SASAW_VJP_PARAMS)                                              \
    MOPS_CXX_DECLARE(sparse_accumulation_scatter_add_with_weights_vjp_vjp, MOPS_SASAW_VJP_VJP_PARAMS)

namespace mops {
MOPS_SASAW_DECLARE_API()
namespace cuda {
MOPS_SASAW_DECLARE_API()
} // namespace cuda
} // namespace mops

#undef MOPS_SASAW_DECLARE_API

#endif
