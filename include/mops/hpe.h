/* C ABI of homogeneous_polynomial_evaluation (HPE).
 *
 *   O[i] = sum_j C[j] * prod_k A[i, indices_A[j, k]]
 *
 * Tensors (row-major, caller-owned, outputs are fully overwritten):
 *   output [n_batch]
 *   A [n_batch, n_factors]
 *   C [n_monomials]
 *   indices_A int32 [n_monomials, degree]
 *
 * This header declares twelve functions, replacing mops/include/mops/hpe.h:12-139
 * of lab-cosmo/mops one for one:
 *
 *   mops_homogeneous_polynomial_evaluation[_vjp[_vjp]]_{f32,f64}        host memory
 *   mops_cuda_homogeneous_polynomial_evaluation[_vjp[_vjp]]_{f32,f64}   device memory
 *
 * The "cuda" in the device entry points is the reference's spelling and is
 * kept so that existing callers (which build the symbol name as
 * "mops_" + "cuda_" + op + "_" + dtype, python/mops/src/mops/dispatch_operation.py:24-28)
 * resolve without change; behind it is the HIP implementation for gfx950.
 *
 * Return value: 0 on success, 1 when a C++ exception was caught (text via
 * mops_get_last_error_message()), 2 for an unknown error. A gradient whose
 * `data` is NULL is skipped. The argument orders live in
 * mops/detail/signatures.h.
 */
#ifndef MOPS_HPE_H
#define MOPS_HPE_H

#include "mops/exports.h"
#include "mops/tensor.h"
#include "mops/detail/signatures.h"

#ifdef __cplusplus
extern "C" {
#endif

MOPS_C_DECLARE_ALL(homogeneous_polynomial_evaluation, MOPS_HPE_PARAMS)
MOPS_C_DECLARE_ALL(homogeneous_polynomial_evaluation_vjp, MOPS_HPE_VJP_PARAMS)
MOPS_C_DECLARE_ALL(homogeneous_polynomial_evaluation_vjp_vjp, MOPS_HPE_VJP_VJP_PARAMS)

#ifdef __cplusplus
}
#endif

#endif
