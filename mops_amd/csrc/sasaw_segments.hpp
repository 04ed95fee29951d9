// SASAW for coupling tables whose component indices have at most 16 values
// each (equivariant message passing), any number of feature channels, as
// per-node sums of rank-one updates on the matrix cores. sasaw.hip calls these
// when `supports()` says so and keeps its general kernels for everything else.
#ifndef MOPS_AMD_SASAW_SEGMENTS_HPP
#define MOPS_AMD_SASAW_SEGMENTS_HPP

#include <cstddef>
#include <cstdint>

#include <hip/hip_runtime.h>

#include "sasaw_mfma.hpp"

namespace mops::amd::sasaw_segments {

using sasaw_mfma::Indices;
using sasaw_mfma::Shape;

/// Whether these kernels cover the shape for elements of `element_size` bytes
/// with one launch (at most 16 values of each component index).
bool supports(const Shape& shape, size_t element_size);
/// Whether forward() covers the shape: also more values of a component index,
/// in several launches that take the index ranges in parts of 16.
bool supports_forward(const Shape& shape, size_t element_size);

template <typename T>
void forward(
    T* output, const T* A, const T* B, const T* C, const T* W, const Indices& indices,
    const Shape& shape, hipStream_t stream
);

/// Whether vjp() serves the shape (grad_W needs a sparse graph: at most 48
/// edges per node on average), the device scratch it needs and the number of
/// 32-bit counters (see SenderArrivals in sender_buckets.hpp). vjp() makes no
/// allocation and uses no second stream.
bool vjp_supported(const Shape& shape, size_t element_size, bool want_grad_W);
size_t vjp_workspace_bytes(const Shape& shape, bool want_grad_W);
size_t vjp_counters(const Shape& shape, bool want_grad_W);

/// Any of grad_A, grad_B, grad_W may be null (not all). `counters`: the
/// vjp_counters() counters; they are zero again when the kernels have run.
/// `counters_are_zero`: whether they are zero now (otherwise a launch in front
/// clears them).
template <typename T>
void vjp(
    T* grad_A, T* grad_B, T* grad_W, const T* grad_output, const T* A, const T* B, const T* C,
    const T* W, const Indices& indices, const Shape& shape, void* workspace, int32_t* counters,
    bool counters_are_zero, hipStream_t stream
);

} // namespace mops::amd::sasaw_segments

#endif
