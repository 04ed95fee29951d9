// The host-memory side of the C++ API (namespace mops, symbols mops_*_f32/f64
// without "cuda_").
//
// This library is the device implementation only. The host entry points are
// exported so that it can stand in for the reference's libmops at link and
// load time, and they validate their arguments exactly like the reference's
// CPU functions do (same tests, same order, same text; see checks.hpp), but
// they do not compute: after a successful validation they raise an error
// that says so. Nothing in the device path ever falls back to the host.
#include <stdexcept>
#include <string>

#include "mops.hpp"

#include "checks.hpp"

namespace {

[[noreturn]] void host_path_unavailable(const char* operation) {
    throw std::runtime_error(
        std::string("mops (AMD build): ") + operation +
        " on host memory is not part of this library, which implements the device path only; "
        "pass device tensors to the mops::cuda:: / mops_cuda_* entry point of the same name"
    );
}

template <typename... Tensors> bool all_null(const Tensors&... tensors) {
    return ((tensors.data == nullptr) && ...);
}

} // namespace

#define MOPS_NAME_FIRST(KIND, NAME) NAME
#define MOPS_NAME_NEXT(KIND, NAME) , NAME

// Validate like the reference's CPU function `NAME` (operation name
// "cpu_<NAME>"), then refuse to compute.
#define MOPS_HOST_ENTRY(NAME, PARAMS, CHECK)                                                       \
    template <typename scalar_t> void mops::NAME(PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {          \
        mops::checks::Validator validator("cpu_" #NAME);                                           \
        mops::checks::CHECK(validator, PARAMS(MOPS_NAME_FIRST, MOPS_NAME_NEXT));                   \
        host_path_unavailable(#NAME);                                                              \
    }                                                                                              \
    MOPS_CXX_INSTANTIATE(mops::NAME, PARAMS)

// A vjp whose gradients are all skipped is a no-op in the reference
// (e.g. mops/src/opsa/cpu.tpp:66-69): keep that, it needs no arithmetic.
#define MOPS_HOST_ENTRY_VJP(NAME, PARAMS, CHECK, ...)                                              \
    template <typename scalar_t> void mops::NAME(PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {          \
        mops::checks::Validator validator("cpu_" #NAME);                                           \
        mops::checks::CHECK(validator, PARAMS(MOPS_NAME_FIRST, MOPS_NAME_NEXT));                   \
        if (all_null(__VA_ARGS__)) {                                                               \
            return;                                                                                \
        }                                                                                          \
        host_path_unavailable(#NAME);                                                              \
    }                                                                                              \
    MOPS_CXX_INSTANTIATE(mops::NAME, PARAMS)

// The reference has no double backward for these on any device and raises
// this text without looking at the arguments (mops/src/opsaw/cpu.tpp:133-150,
// mops/src/sasaw/cpu.tpp:173-194).
#define MOPS_HOST_NOT_IMPLEMENTED(NAME, PARAMS)                                                    \
    template <typename scalar_t> void mops::NAME(PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {          \
        throw std::runtime_error("Not implemented");                                               \
    }                                                                                              \
    MOPS_CXX_INSTANTIATE(mops::NAME, PARAMS)

MOPS_HOST_ENTRY(homogeneous_polynomial_evaluation, MOPS_HPE_PARAMS, hpe)
MOPS_HOST_ENTRY_VJP(homogeneous_polynomial_evaluation_vjp, MOPS_HPE_VJP_PARAMS, hpe_vjp, grad_A)
MOPS_HOST_ENTRY(homogeneous_polynomial_evaluation_vjp_vjp, MOPS_HPE_VJP_VJP_PARAMS, hpe_vjp_vjp)

MOPS_HOST_ENTRY(sparse_accumulation_of_products, MOPS_SAP_PARAMS, sap)
MOPS_HOST_ENTRY_VJP(sparse_accumulation_of_products_vjp, MOPS_SAP_VJP_PARAMS, sap_vjp, grad_A, grad_B)
MOPS_HOST_ENTRY(sparse_accumulation_of_products_vjp_vjp, MOPS_SAP_VJP_VJP_PARAMS, sap_vjp_vjp)

MOPS_HOST_ENTRY(outer_product_scatter_add, MOPS_OPSA_PARAMS, opsa)
MOPS_HOST_ENTRY_VJP(outer_product_scatter_add_vjp, MOPS_OPSA_VJP_PARAMS, opsa_vjp, grad_A, grad_B)
MOPS_HOST_ENTRY(outer_product_scatter_add_vjp_vjp, MOPS_OPSA_VJP_VJP_PARAMS, opsa_vjp_vjp)

MOPS_HOST_ENTRY(outer_product_scatter_add_with_weights, MOPS_OPSAW_PARAMS, opsaw)
MOPS_HOST_ENTRY_VJP(
    outer_product_scatter_add_with_weights_vjp, MOPS_OPSAW_VJP_PARAMS, opsaw_vjp, grad_A, grad_B, grad_W
)
MOPS_HOST_NOT_IMPLEMENTED(outer_product_scatter_add_with_weights_vjp_vjp, MOPS_OPSAW_VJP_VJP_PARAMS)

MOPS_HOST_ENTRY(sparse_accumulation_scatter_add_with_weights, MOPS_SASAW_PARAMS, sasaw)
MOPS_HOST_ENTRY_VJP(
    sparse_accumulation_scatter_add_with_weights_vjp, MOPS_SASAW_VJP_PARAMS, sasaw_vjp, grad_A, grad_B, grad_W
)
MOPS_HOST_NOT_IMPLEMENTED(
    sparse_accumulation_scatter_add_with_weights_vjp_vjp, MOPS_SASAW_VJP_VJP_PARAMS
)
