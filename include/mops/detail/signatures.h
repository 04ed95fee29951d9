/* Parameter lists of the fifteen mops functions, written once.
 *
 * Every list is an X-macro over (KIND, NAME) pairs: FIRST is applied to the
 * first parameter and NEXT to each following one, so an expansion can put
 * the separating commas where it needs them. KIND is one of
 *
 *   R1 R2 R3   floating-point tensor with 1, 2 or 3 dimensions
 *   I1 I2      int32 index tensor with 1 or 2 dimensions
 *   Q3         floating-point tensor that is 3-D in the C++ API but declared
 *              with the 2-D struct in the C ABI (the reference's C header
 *              does this for grad_grad_W of the SASAW double backward,
 *              mops/include/mops/sasaw.h:84,106,192,214, and binary
 *              compatibility requires keeping it)
 *
 * The C declarations (mops/<op>.h), the C++ declarations (mops/<op>.hpp) and
 * the C-ABI wrappers are all generated from these lists, so the three can
 * never disagree on an argument order. The orders themselves are those of
 * lab-cosmo/mops: outputs first, then grad_output, then the forward inputs
 * (mops/include/mops/hpe.h:12-83, sap.h:12-101, opsa.h:12-74,
 * opsaw.h:12-92, sasaw.h:12-118).
 */
#ifndef MOPS_DETAIL_SIGNATURES_H
#define MOPS_DETAIL_SIGNATURES_H

/* ---- homogeneous_polynomial_evaluation (HPE) --------------------------- */
#define MOPS_HPE_INPUTS(NEXT) NEXT(R2, A) NEXT(R1, C) NEXT(I2, indices_A)

#define MOPS_HPE_PARAMS(FIRST, NEXT) FIRST(R1, output) MOPS_HPE_INPUTS(NEXT)

#define MOPS_HPE_VJP_PARAMS(FIRST, NEXT)                                                           \
    FIRST(R2, grad_A) NEXT(R1, grad_output) MOPS_HPE_INPUTS(NEXT)

#define MOPS_HPE_VJP_VJP_PARAMS(FIRST, NEXT)                                                       \
    FIRST(R1, grad_grad_output)                                                                    \
    NEXT(R2, grad_A_2) NEXT(R2, grad_grad_A) NEXT(R1, grad_output) MOPS_HPE_INPUTS(NEXT)

/* ---- sparse_accumulation_of_products (SAP) ----------------------------- */
#define MOPS_SAP_INPUTS(NEXT)                                                                      \
    NEXT(R2, A)                                                                                    \
    NEXT(R2, B) NEXT(R1, C) NEXT(I1, indices_A) NEXT(I1, indices_B) NEXT(I1, indices_output)

#define MOPS_SAP_PARAMS(FIRST, NEXT) FIRST(R2, output) MOPS_SAP_INPUTS(NEXT)

#define MOPS_SAP_VJP_PARAMS(FIRST, NEXT)                                                           \
    FIRST(R2, grad_A) NEXT(R2, grad_B) NEXT(R2, grad_output) MOPS_SAP_INPUTS(NEXT)

#define MOPS_SAP_VJP_VJP_PARAMS(FIRST, NEXT)                                                       \
    FIRST(R2, grad_grad_output)                                                                    \
    NEXT(R2, grad_A_2)                                                                             \
    NEXT(R2, grad_B_2)                                                                             \
    NEXT(R2, grad_grad_A) NEXT(R2, grad_grad_B) NEXT(R2, grad_output) MOPS_SAP_INPUTS(NEXT)

/* ---- outer_product_scatter_add (OPSA) ---------------------------------- */
#define MOPS_OPSA_INPUTS(NEXT) NEXT(R2, A) NEXT(R2, B) NEXT(I1, indices_output)

#define MOPS_OPSA_PARAMS(FIRST, NEXT) FIRST(R3, output) MOPS_OPSA_INPUTS(NEXT)

#define MOPS_OPSA_VJP_PARAMS(FIRST, NEXT)                                                          \
    FIRST(R2, grad_A) NEXT(R2, grad_B) NEXT(R3, grad_output) MOPS_OPSA_INPUTS(NEXT)

#define MOPS_OPSA_VJP_VJP_PARAMS(FIRST, NEXT)                                                      \
    FIRST(R3, grad_grad_output)                                                                    \
    NEXT(R2, grad_A_2)                                                                             \
    NEXT(R2, grad_B_2)                                                                             \
    NEXT(R2, grad_grad_A) NEXT(R2, grad_grad_B) NEXT(R3, grad_output) MOPS_OPSA_INPUTS(NEXT)

/* ---- outer_product_scatter_add_with_weights (OPSAW) -------------------- */
#define MOPS_OPSAW_INPUTS(NEXT)                                                                    \
    NEXT(R2, A) NEXT(R2, B) NEXT(R2, W) NEXT(I1, indices_W) NEXT(I1, indices_output)

#define MOPS_OPSAW_PARAMS(FIRST, NEXT) FIRST(R3, output) MOPS_OPSAW_INPUTS(NEXT)

#define MOPS_OPSAW_VJP_PARAMS(FIRST, NEXT)                                                         \
    FIRST(R2, grad_A)                                                                              \
    NEXT(R2, grad_B) NEXT(R2, grad_W) NEXT(R3, grad_output) MOPS_OPSAW_INPUTS(NEXT)

#define MOPS_OPSAW_VJP_VJP_PARAMS(FIRST, NEXT)                                                     \
    FIRST(R3, grad_grad_output)                                                                    \
    NEXT(R2, grad_A_2)                                                                             \
    NEXT(R2, grad_B_2)                                                                             \
    NEXT(R2, grad_W_2)                                                                             \
    NEXT(R2, grad_grad_A)                                                                          \
    NEXT(R2, grad_grad_B) NEXT(R2, grad_grad_W) NEXT(R3, grad_output) MOPS_OPSAW_INPUTS(NEXT)

/* ---- sparse_accumulation_scatter_add_with_weights (SASAW) -------------- */
#define MOPS_SASAW_INPUTS(NEXT)                                                                    \
    NEXT(R2, A)                                                                                    \
    NEXT(R2, B)                                                                                    \
    NEXT(R1, C)                                                                                    \
    NEXT(R3, W)                                                                                    \
    NEXT(I1, indices_A)                                                                            \
    NEXT(I1, indices_W_1)                                                                          \
    NEXT(I1, indices_W_2) NEXT(I1, indices_output_1) NEXT(I1, indices_output_2)

#define MOPS_SASAW_PARAMS(FIRST, NEXT) FIRST(R3, output) MOPS_SASAW_INPUTS(NEXT)

#define MOPS_SASAW_VJP_PARAMS(FIRST, NEXT)                                                         \
    FIRST(R2, grad_A)                                                                              \
    NEXT(R2, grad_B) NEXT(R3, grad_W) NEXT(R3, grad_output) MOPS_SASAW_INPUTS(NEXT)

#define MOPS_SASAW_VJP_VJP_PARAMS(FIRST, NEXT)                                                     \
    FIRST(R3, grad_grad_output)                                                                    \
    NEXT(R2, grad_A_2)                                                                             \
    NEXT(R2, grad_B_2)                                                                             \
    NEXT(R3, grad_W_2)                                                                             \
    NEXT(R2, grad_grad_A)                                                                          \
    NEXT(R2, grad_grad_B) NEXT(Q3, grad_grad_W) NEXT(R3, grad_output) MOPS_SASAW_INPUTS(NEXT)

/* ---- the table of all functions ---------------------------------------- *
 * APPLY(name, PARAMS) is expanded once per function; `name` is the part of
 * the symbol between the "mops_" / "mops_cuda_" prefix and the "_f32" /
 * "_f64" suffix, which is also the name of the C++ template. */
#define MOPS_FOR_EACH_FUNCTION(APPLY)                                                              \
    APPLY(homogeneous_polynomial_evaluation, MOPS_HPE_PARAMS)                                      \
    APPLY(homogeneous_polynomial_evaluation_vjp, MOPS_HPE_VJP_PARAMS)                              \
    APPLY(homogeneous_polynomial_evaluation_vjp_vjp, MOPS_HPE_VJP_VJP_PARAMS)                      \
    APPLY(sparse_accumulation_of_products, MOPS_SAP_PARAMS)                                        \
    APPLY(sparse_accumulation_of_products_vjp, MOPS_SAP_VJP_PARAMS)                                \
    APPLY(sparse_accumulation_of_products_vjp_vjp, MOPS_SAP_VJP_VJP_PARAMS)                        \
    APPLY(outer_product_scatter_add, MOPS_OPSA_PARAMS)                                             \
    APPLY(outer_product_scatter_add_vjp, MOPS_OPSA_VJP_PARAMS)                                     \
    APPLY(outer_product_scatter_add_vjp_vjp, MOPS_OPSA_VJP_VJP_PARAMS)                             \
    APPLY(outer_product_scatter_add_with_weights, MOPS_OPSAW_PARAMS)                               \
    APPLY(outer_product_scatter_add_with_weights_vjp, MOPS_OPSAW_VJP_PARAMS)                       \
    APPLY(outer_product_scatter_add_with_weights_vjp_vjp, MOPS_OPSAW_VJP_VJP_PARAMS)               \
    APPLY(sparse_accumulation_scatter_add_with_weights, MOPS_SASAW_PARAMS)                         \
    APPLY(sparse_accumulation_scatter_add_with_weights_vjp, MOPS_SASAW_VJP_PARAMS)                 \
    APPLY(sparse_accumulation_scatter_add_with_weights_vjp_vjp, MOPS_SASAW_VJP_VJP_PARAMS)

/* C parameter spelling: MOPS_C_PARAM(f32, R2) -> mops_tensor_2d_f32_t */
#define MOPS_C_KIND_R1(S) mops_tensor_1d_##S##_t
#define MOPS_C_KIND_R2(S) mops_tensor_2d_##S##_t
#define MOPS_C_KIND_R3(S) mops_tensor_3d_##S##_t
#define MOPS_C_KIND_Q3(S) mops_tensor_2d_##S##_t
#define MOPS_C_KIND_I1(S) mops_tensor_1d_i32_t
#define MOPS_C_KIND_I2(S) mops_tensor_2d_i32_t

#define MOPS_C_FIRST_f32(KIND, NAME) MOPS_C_KIND_##KIND(f32) NAME
#define MOPS_C_NEXT_f32(KIND, NAME) , MOPS_C_KIND_##KIND(f32) NAME
#define MOPS_C_FIRST_f64(KIND, NAME) MOPS_C_KIND_##KIND(f64) NAME
#define MOPS_C_NEXT_f64(KIND, NAME) , MOPS_C_KIND_##KIND(f64) NAME

/* One C prototype: MOPS_C_PROTOTYPE(cuda_, name, f32, PARAMS) */
#define MOPS_C_PROTOTYPE(DEVICE, NAME, S, PARAMS)                                                  \
    int MOPS_EXPORT mops_##DEVICE##NAME##_##S(PARAMS(MOPS_C_FIRST_##S, MOPS_C_NEXT_##S))

/* The four C prototypes of one function: host and device, f32 and f64. */
#define MOPS_C_DECLARE_ALL(NAME, PARAMS)                                                           \
    MOPS_C_PROTOTYPE(, NAME, f32, PARAMS);                                                         \
    MOPS_C_PROTOTYPE(, NAME, f64, PARAMS);                                                         \
    MOPS_C_PROTOTYPE(cuda_, NAME, f32, PARAMS);                                                    \
    MOPS_C_PROTOTYPE(cuda_, NAME, f64, PARAMS);

#ifdef __cplusplus
/* C++ parameter spelling, valid inside a template over scalar_t. */
#define MOPS_CXX_KIND_R1 ::mops::Tensor<scalar_t, 1>
#define MOPS_CXX_KIND_R2 ::mops::Tensor<scalar_t, 2>
#define MOPS_CXX_KIND_R3 ::mops::Tensor<scalar_t, 3>
#define MOPS_CXX_KIND_Q3 ::mops::Tensor<scalar_t, 3>
#define MOPS_CXX_KIND_I1 ::mops::Tensor<int32_t, 1>
#define MOPS_CXX_KIND_I2 ::mops::Tensor<int32_t, 2>

#define MOPS_CXX_FIRST(KIND, NAME) MOPS_CXX_KIND_##KIND NAME
#define MOPS_CXX_NEXT(KIND, NAME) , MOPS_CXX_KIND_##KIND NAME

/* Same, with the element type spelled out (explicit instantiations). */
#define MOPS_CXX_FIRST_AS(T, KIND, NAME) MOPS_CXX_TYPED_##KIND(T) NAME
#define MOPS_CXX_TYPED_R1(T) ::mops::Tensor<T, 1>
#define MOPS_CXX_TYPED_R2(T) ::mops::Tensor<T, 2>
#define MOPS_CXX_TYPED_R3(T) ::mops::Tensor<T, 3>
#define MOPS_CXX_TYPED_Q3(T) ::mops::Tensor<T, 3>
#define MOPS_CXX_TYPED_I1(T) ::mops::Tensor<int32_t, 1>
#define MOPS_CXX_TYPED_I2(T) ::mops::Tensor<int32_t, 2>
#define MOPS_CXX_FIRST_float(KIND, NAME) MOPS_CXX_TYPED_##KIND(float) NAME
#define MOPS_CXX_NEXT_float(KIND, NAME) , MOPS_CXX_TYPED_##KIND(float) NAME
#define MOPS_CXX_FIRST_double(KIND, NAME) MOPS_CXX_TYPED_##KIND(double) NAME
#define MOPS_CXX_NEXT_double(KIND, NAME) , MOPS_CXX_TYPED_##KIND(double) NAME

/* Declaration of one function template plus the two `extern template`
 * lines that say "float and double are precompiled in the library".
 * Expanded inside namespace mops and again inside namespace mops::cuda. */
#define MOPS_CXX_DECLARE(NAME, PARAMS)                                                             \
    template <typename scalar_t> void MOPS_EXPORT NAME(PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT));     \
    extern template void NAME<float>(PARAMS(MOPS_CXX_FIRST_float, MOPS_CXX_NEXT_float));           \
    extern template void NAME<double>(PARAMS(MOPS_CXX_FIRST_double, MOPS_CXX_NEXT_double));

/* Explicit instantiation of both element types (library side). */
#define MOPS_CXX_INSTANTIATE(QUALIFIED_NAME, PARAMS)                                               \
    template void QUALIFIED_NAME<float>(PARAMS(MOPS_CXX_FIRST_float, MOPS_CXX_NEXT_float));        \
    template void QUALIFIED_NAME<double>(PARAMS(MOPS_CXX_FIRST_double, MOPS_CXX_NEXT_double));
#endif

#endif
