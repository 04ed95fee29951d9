// The C ABI: 60 operation entry points, the error-text accessor and the
// AMD-specific additions. Every operation wrapper does the same three
// things as mops/src/<op>/capi.cpp of lab-cosmo/mops: convert each int64
// extent to size_t (rejecting negative values), call the C++ template, and
// translate exceptions into a status code plus a per-thread message.
// The wrappers are generated from the parameter lists in
// mops/detail/signatures.h.
#include <cstdint>
#include <stdexcept>
#include <string>

#include "mops.h"
#include "mops.hpp"

#include "first_occurrences.hpp"
#include "no_alloc.hpp"
#include "edge_order.hpp"
#include "runtime.hpp"

namespace {

thread_local std::string LAST_ERROR;

size_t extent(int64_t value) {
    if (value < 0 || static_cast<uint64_t>(value) > static_cast<uint64_t>(SIZE_MAX)) {
        throw std::runtime_error(
            "integer value '" + std::to_string(value) + "' does not fit in size_t"
        );
    }
    return static_cast<size_t>(value);
}

// C view -> C++ view, one overload per struct type
#define MOPS_DEFINE_VIEW(STRUCT, ELEMENT)                                                          \
    [[maybe_unused]] mops::Tensor<ELEMENT, sizeof(STRUCT::shape) / sizeof(int64_t)> view(STRUCT t) {                \
        constexpr size_t N = sizeof(STRUCT::shape) / sizeof(int64_t);                              \
        mops::Tensor<ELEMENT, N> result;                                                           \
        result.data = t.data;                                                                      \
        for (size_t d = 0; d < N; d++) {                                                           \
            result.shape[d] = extent(t.shape[d]);                                                  \
        }                                                                                          \
        return result;                                                                             \
    }

MOPS_DEFINE_VIEW(mops_tensor_1d_f32_t, float)
MOPS_DEFINE_VIEW(mops_tensor_2d_f32_t, float)
MOPS_DEFINE_VIEW(mops_tensor_3d_f32_t, float)
MOPS_DEFINE_VIEW(mops_tensor_1d_f64_t, double)
MOPS_DEFINE_VIEW(mops_tensor_2d_f64_t, double)
MOPS_DEFINE_VIEW(mops_tensor_3d_f64_t, double)
MOPS_DEFINE_VIEW(mops_tensor_1d_i32_t, int32_t)
MOPS_DEFINE_VIEW(mops_tensor_2d_i32_t, int32_t)

// A tensor that the C ABI declares with the 2-D struct although it has three
// dimensions: the missing last extent is taken from `last`.
template <typename Element, typename Struct2D>
mops::Tensor<Element, 3> view_with_last_extent(Struct2D t, int64_t last) {
    mops::Tensor<Element, 3> result;
    result.data = t.data;
    result.shape[0] = extent(t.shape[0]);
    result.shape[1] = extent(t.shape[1]);
    result.shape[2] = extent(last);
    return result;
}

[[maybe_unused]] mops::Tensor<float, 3> view_3d(mops_tensor_2d_f32_t t, int64_t last) {
    return view_with_last_extent<float>(t, last);
}

[[maybe_unused]] mops::Tensor<double, 3> view_3d(mops_tensor_2d_f64_t t, int64_t last) {
    return view_with_last_extent<double>(t, last);
}

} // namespace

void mops::store_error_message(std::string message) { LAST_ERROR = std::move(message); }

const std::string& mops::get_last_error_message() { return LAST_ERROR; }

extern "C" const char* mops_get_last_error_message(void) { return LAST_ERROR.c_str(); }

#define MOPS_FORWARD_R1(NAME) view(NAME)
#define MOPS_FORWARD_R2(NAME) view(NAME)
#define MOPS_FORWARD_R3(NAME) view(NAME)
#define MOPS_FORWARD_I1(NAME) view(NAME)
#define MOPS_FORWARD_I2(NAME) view(NAME)
#define MOPS_FORWARD_Q3(NAME) view_3d(NAME, W.shape[2])
#define MOPS_FORWARD_FIRST(KIND, NAME) MOPS_FORWARD_##KIND(NAME)
#define MOPS_FORWARD_NEXT(KIND, NAME) , MOPS_FORWARD_##KIND(NAME)

#define MOPS_C_DEFINE(DEVICE, NAMESPACE, NAME, S, T, PARAMS)                                       \
    extern "C" MOPS_C_PROTOTYPE(DEVICE, NAME, S, PARAMS) {                                         \
        MOPS_CATCH_EXCEPTIONS_BEGIN                                                                \
        NAMESPACE NAME<T>(PARAMS(MOPS_FORWARD_FIRST, MOPS_FORWARD_NEXT));                          \
        MOPS_CATCH_EXCEPTIONS_END                                                                  \
    }

#define MOPS_C_DEFINE_ALL(NAME, PARAMS)                                                            \
    MOPS_C_DEFINE(, ::mops::, NAME, f32, float, PARAMS)                                            \
    MOPS_C_DEFINE(, ::mops::, NAME, f64, double, PARAMS)                                           \
    MOPS_C_DEFINE(cuda_, ::mops::cuda::, NAME, f32, float, PARAMS)                                 \
    MOPS_C_DEFINE(cuda_, ::mops::cuda::, NAME, f64, double, PARAMS)

MOPS_FOR_EACH_FUNCTION(MOPS_C_DEFINE_ALL)

// ---- AMD-specific additions (mops/amd.h) ---------------------------------

extern "C" int mops_amd_set_stream(void* hip_stream) {
    mops::amd::set_current_stream(static_cast<hipStream_t>(hip_stream));
    return 0;
}

extern "C" void* mops_amd_get_stream(void) { return mops::amd::current_stream(); }

extern "C" int mops_amd_set_synchronous(int synchronous) {
    return mops::amd::set_synchronous(synchronous != 0) ? 1 : 0;
}

extern "C" int mops_amd_first_occurrences(
    const int32_t* sorted_indices, int64_t n_input, int64_t n_output, int32_t* first_occurrences
) {
    MOPS_CATCH_EXCEPTIONS_BEGIN
    mops::amd::first_occurrences(
        sorted_indices,
        mops::amd::narrow_i32(extent(n_input), "n_input"),
        mops::amd::narrow_i32(extent(n_output), "n_output"),
        first_occurrences,
        mops::amd::current_stream()
    );
    mops::amd::finish_call("first_occurrences");
    MOPS_CATCH_EXCEPTIONS_END
}

extern "C" int mops_amd_accept_unsorted_indices(int accept) {
    return mops::amd::set_accept_unsorted(accept != 0) ? 1 : 0;
}

extern "C" int mops_amd_kernel_timing(int enable) {
    return mops::amd::set_kernel_timing(enable != 0) ? 1 : 0;
}

extern "C" int mops_amd_kernel_time(double* total_milliseconds, int64_t* launches) {
    MOPS_CATCH_EXCEPTIONS_BEGIN
    if (total_milliseconds == nullptr || launches == nullptr) {
        throw std::runtime_error("mops_amd_kernel_time: both result pointers must be given");
    }
    mops::amd::collect_kernel_time(total_milliseconds, launches);
    MOPS_CATCH_EXCEPTIONS_END
}

extern "C" int mops_amd_reserve_scratch(int64_t bytes) {
    MOPS_CATCH_EXCEPTIONS_BEGIN
    (void)mops::amd::scratch(extent(bytes));
    mops::amd::finish_call("reserve_scratch");
    MOPS_CATCH_EXCEPTIONS_END
}

extern "C" int64_t mops_amd_scratch_capacity(void) {
    return static_cast<int64_t>(mops::amd::scratch_capacity());
}

extern "C" int mops_amd_sparse_accumulation_scatter_add_with_weights_vjp_no_alloc_f32(
    MOPS_SASAW_VJP_PARAMS(MOPS_C_FIRST_f32, MOPS_C_NEXT_f32)
) {
    MOPS_CATCH_EXCEPTIONS_BEGIN
    mops::amd::sasaw_vjp_no_alloc(MOPS_SASAW_VJP_PARAMS(MOPS_FORWARD_FIRST, MOPS_FORWARD_NEXT));
    MOPS_CATCH_EXCEPTIONS_END
}
