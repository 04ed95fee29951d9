/* C ABI of sparse_accumulation_scatter_add_with_weights (SASAW).
 *
 *   O[indices_output_1[e], indices_output_2[n], :] += A[e, indices_A[n]] * B[e, :] * C[n] * W[indices_W_1[e], indices_W_2[n], :]
 *
 * Tensors (row-major, caller-owned, outputs are fully overwritten):
 *   output [n_nodes, output_size, size_B]
 *   A [n_edges, size_A]
 *   B [n_edges, size_B]
 *   C [n_products]
 *   W [n_nodes, size_W, size_B]
 *   indices_A, indices_W_2, indices_output_2 int32 [n_products]
 *   indices_W_1, indices_output_1 int32 [n_edges]
 *
 * This header declares twelve functions, replacing mops/include/mops/sasaw.h:12-237
 * of lab-cosmo/mops one for one:
 *
 *   mops_sparse_accumulation_scatter_add_with_weights[_vjp[_vjp]]_{f32,f64}        host memory
 *   mops_cuda_sparse_accumulation_scatter_add_with_weights[_vjp[_vjp]]_{f32,f64}   device memory
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
#ifndef MOPS_SASAW_H
#define MOPS_SASAW_H

#include "mops/exports.h"
#include "mops/tensor.h"
#include "mops/detail/signatures.h"

#ifdef __cplusplus
extern "C" {
#endif

MOPS_C_DECLARE_ALL(sparse_accumulation_scatter_add_with_weights, MOPS_SASAW_PARAMS)
MOPS_C_DECLARE_ALL(sparse_accumulation_scatter_add_with_weights_vjp, MOPS_SASAW_VJP_PARAMS)
MOPS_C_DECLARE_ALL(sparse_accumulation_scatter_add_with_weights_vjp_vjp, MOPS_SASAW_VJP_VJP_PARAMS)

#ifdef __cplusplus
}
#endif

#endif
