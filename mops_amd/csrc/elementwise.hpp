// Small element-wise helpers for the second-order entry points, which are
// compositions of the first-order kernels: clear a tensor, add one tensor to
// another, and a temporary tensor that lives on the stream.
#ifndef MOPS_AMD_ELEMENTWISE_HPP
#define MOPS_AMD_ELEMENTWISE_HPP

#include <cstddef>

#include <hip/hip_runtime.h>

namespace mops::amd {

/// data[i] = 0 for i < count (a kernel, not hipMemsetAsync, so that a caller
/// may capture the call into a graph).
template <typename T> void fill_zero(T* data, size_t count, hipStream_t stream);

/// target[i] += addend[i] for i < count.
template <typename T> void add_in_place(T* target, const T* addend, size_t count, hipStream_t stream);

/// Device memory allocated and released in stream order.
template <typename T> class StreamTemporary {
public:
    StreamTemporary(size_t count, hipStream_t stream);
    ~StreamTemporary();
    StreamTemporary(const StreamTemporary&) = delete;
    StreamTemporary& operator=(const StreamTemporary&) = delete;
    T* data() const { return data_; }

private:
    T* data_ = nullptr;
    hipStream_t stream_;
};

} // namespace mops::amd

#endif
