// C++ API of sparse_accumulation_of_products (SAP).
//
//   O[i, indices_output[k]] += C[k] * A[i, indices_A[k]] * B[i, indices_B[k]]
//
// Declares, in namespace mops (host memory) and again in namespace
// mops::cuda (device memory, HIP implementation for gfx950):
//
//   template <typename scalar_t> void sparse_accumulation_of_products(...);
//   template <typename scalar_t> void sparse_accumulation_of_products_vjp(...);
//   template <typename scalar_t> void sparse_accumulation_of_products_vjp_vjp(...);
//
// with float and double precompiled in the library. Tensors are passed by
// value as mops::Tensor views, outputs first; a gradient whose data pointer
// is null is skipped. Replaces mops/include/mops/sap.hpp:32-262 of lab-cosmo/mops
// with identical template names, namespaces and argument orders (the orders
// are spelled once in mops/detail/signatures.h).
#ifndef MOPS_SAP_HPP
#define MOPS_SAP_HPP

#include <cstdint>

#include "mops/exports.h"
#include "mops/tensor.hpp"
#include "mops/detail/signatures.h"

#define MOPS_SAP_DECLARE_API()                                                                     \
    MOPS_CXX_DECLARE(sparse_accumulation_of_products, MOPS_SAP_PARAMS)                                                      \
    MOPS_CXX_DECLARE(sparse_accumulation_of_products_vjp, MOPS_SAP_VJP_PARAMS)                                              \
    MOPS_CXX_DECLARE(sparse_accumulation_of_products_vjp_vjp, MOPS_SAP_VJP_VJP_PARAMS)

namespace mops {
MOPS_SAP_DECLARE_API()
namespace cuda {
MOPS_SAP_DECLARE_API()
} // namespace cuda
} // namespace mops

#undef MOPS_SAP_DECLARE_API

#endif
