/* C ABI of outer_product_scatter_add (OPSA).
 *
 *   O[indices_output[j], :, :] += A[j, :, None] * B[j, None, :]
 *
 * Tensors (row-major, caller-owned, outputs are fully overwritten):
 *   output [output_size, size_A, size_B]
 *   A [n_batch, size_A]
 *   B [n_batch, size_B]
 *   indices_output int32 [n_batch]
 *
 * This header declares twelve functions, replacing mops/include/mops/opsa.h:12-139
 * of lab-cosmo/mops one for one:
 *
 *   mops_outer_product_scatter_add[_vjp[_vjp]]_{f32,f64}        host memory
 *   mops_cuda_outer_product_scatter_add[_vjp[_vjp]]_{f32,f64}   device memory
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
#ifndef MOPS_OPSA_H
#define MOPS_OPSA_H

#include "mops/exports.h"
#include "mops/tensor.h"
#include "mops/detail/signatures.h"

#ifdef __cplusplus
extern "C" {
#endif

MOPS_C_DECLARE_ALL(outer_product_scatter_add, MOPS_OPSA_PARAMS)
MOPS_C_DECLARE_ALL(outer_product_scatter_add_vjp, MOPS_OPSA_VJP_PARAMS)
MOPS_C_DECLARE_ALL(outer_product_scatter_add_vjp_vjp, MOPS_OPSA_VJP_VJP_PARAMS)

#ifdef __cplusplus
}
#endif

#endif
