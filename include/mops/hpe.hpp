// C++ API of homogeneous_polynomial_evaluation (HPE).
//
//   O[i] = sum_j C[j] * prod_k A[i, indices_A[j, k]]
//
// Declares, in namespace mops (host memory) and again in namespace
// mops::cuda (device memory, HIP implementation for gfx950):
//
//   template <typename scalar_t> void homogeneous_polynomial_evaluation(...);
//   template <typename scalar_t> void homogeneous_polynomial_evaluation_vjp(...);
//   template <typename scalar_t> void homogeneous_polynomial_evaluation_vjp_vjp(...);
//
// with float and double precompiled in the library. Tensors are passed by
// value as mops::Tensor views, outputs first; a gradient whose data pointer
// is null is skipped. Replaces mops/include/mops/hpe.hpp:24-172 of lab-cosmo/mops
// with identical template names, namespaces and argument orders (the orders
// are spelled once in mops/detail/signatures.h).
#ifndef MOPS_HPE_HPP
#define MOPS_HPE_HPP

#include <cstdint>

#include "mops/exports.h"
#include "mops/tensor.hpp"
#include "mops/detail/signatures.h"

#define MOPS_HPE_DECLARE_API()                                                                     \
    MOPS_CXX_DECLARE(homogeneous_polynomial_evaluation, MOPS_HPE_PARAMS)                                                      \
    MOPS_CXX_DECLARE(homogeneous_polynomial_evaluation_vjp, MOPS_HPE_VJP_PARAMS)                                              \
    MOPS_CXX_DECLARE(homogeneous_polynomial_evaluation_vjp_vjp, MOPS_HPE_VJP_VJP_PARAMS)

namespace mops {
MOPS_HPE_DECLARE_API()
namespace cuda {
MOPS_HPE_DECLARE_API()
} // namespace cuda
} // namespace mops

#undef MOPS_HPE_DECLARE_API

#endif
