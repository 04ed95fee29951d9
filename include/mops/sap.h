/* C ABI of sparse_accumulation_of_products (SAP).
 *
 *   O[i, indices_output[k]] += C[k] * A[i, indices_A[k]] * B[i, indices_B[k]]
 *
 * Tensors (row-major, caller-owned, outputs are fully overwritten):
 *   output [n_batch, output_size]
 *   A [n_batch, size_A]
 *   B [n_batch, size_B]
 *   C [n_products]
 *   indices_A, indices_B, indices_output int32 [n_products]
 *
 * This header declares twelve functions, replacing mops/include/mops/sap.h:12-195
 * of lab-cosmo/mops one for one:
 *
 *   mops_sparse_accumulation_of_products[_vjp[_vjp]]_{f32,f64}        host memory
 *   mops_cuda_sparse_accumulation_of_products[_vjp[_vjp]]_{f32,f64}   device memory
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
#ifndef MOPS_SAP_H
#define MOPS_SAP_H

#include "mops/exports.h"
#include "mops/tensor.h"
#include "mops/detail/signatures.h"

#ifdef __cplusplus
extern "C" {
#endif

MOPS_C_DECLARE_ALL(sparse_accumulation_of_products, MOPS_SAP_PARAMS)
MOPS_C_DECLARE_ALL(sparse_accumulation_of_products_vjp, MOPS_SAP_VJP_PARAMS)
MOPS_C_DECLARE_ALL(sparse_accumulation_of_products_vjp_vjp, MOPS_SAP_VJP_VJP_PARAMS)

#ifdef __cplusplus
}
#endif

#endif
