/* C views of dense row-major tensors, passed BY VALUE across the C ABI.
 *
 * Layout contract (replaces mops/include/mops/tensor.h:11-49 of
 * lab-cosmo/mops): one data pointer followed by `ndim` int64 extents. The
 * memory is caller-owned, contiguous and row-major. A view whose `data` is
 * NULL means "this optional gradient is not requested".
 *
 * For the mops_cuda_* entry points every pointer (index tensors included)
 * is a device pointer. */
#ifndef MOPS_TENSOR_H
#define MOPS_TENSOR_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MOPS_DEFINE_TENSOR_VIEW(NAME, ELEMENT, NDIM)                                               \
    typedef struct NAME {                                                                          \
        ELEMENT* __restrict__ data;                                                                \
        int64_t shape[NDIM];                                                                       \
    } NAME;

MOPS_DEFINE_TENSOR_VIEW(mops_tensor_1d_f32_t, float, 1)
MOPS_DEFINE_TENSOR_VIEW(mops_tensor_2d_f32_t, float, 2)
MOPS_DEFINE_TENSOR_VIEW(mops_tensor_3d_f32_t, float, 3)
MOPS_DEFINE_TENSOR_VIEW(mops_tensor_1d_f64_t, double, 1)
MOPS_DEFINE_TENSOR_VIEW(mops_tensor_2d_f64_t, double, 2)
MOPS_DEFINE_TENSOR_VIEW(mops_tensor_3d_f64_t, double, 3)
MOPS_DEFINE_TENSOR_VIEW(mops_tensor_1d_i32_t, int32_t, 1)
MOPS_DEFINE_TENSOR_VIEW(mops_tensor_2d_i32_t, int32_t, 2)

#undef MOPS_DEFINE_TENSOR_VIEW

#ifdef __cplusplus
}
#endif

#endif
