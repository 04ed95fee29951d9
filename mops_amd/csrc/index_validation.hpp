// Optional validation of device-resident index tensors.
//
// The reference checks index ranges only on its CPU path and says so
// ("TODO: check CUDA index tensors", mops/src/internal/checks/hpe.hpp:19);
// its device kernels assume a sorted scatter index without looking
// (mops/src/internal/checks/opsa.hpp:20-22). That is the default here too,
// because looking costs a device-to-host copy and a stall. Setting
// MOPS_AMD_CHECK_INDICES=1 in the environment turns the copy on: ranges are
// then checked with the same messages as on the host path, and the scatter
// index additionally for being non-decreasing.
#ifndef MOPS_AMD_INDEX_VALIDATION_HPP
#define MOPS_AMD_INDEX_VALIDATION_HPP

#include <stdexcept>
#include <string>
#include <vector>

#include "mops/tensor.hpp"

#include "checks.hpp"
#include "runtime.hpp"

namespace mops::amd {

template <size_t N>
std::vector<int32_t> copy_indices_to_host(const Tensor<int32_t, N>& indices) {
    size_t count = 1;
    for (size_t d = 0; d < N; d++) {
        count *= indices.shape[d];
    }
    std::vector<int32_t> host(count);
    if (count > 0) {
        hipStream_t stream = current_stream();
        MOPS_HIP_CHECK(hipMemcpyAsync(
            host.data(), indices.data, count * sizeof(int32_t), hipMemcpyDeviceToHost, stream
        ));
        MOPS_HIP_CHECK(hipStreamSynchronize(stream));
    }
    return host;
}

/// Range check of an index tensor that is used to gather.
template <size_t N>
void validate_gather_index(
    const Tensor<int32_t, N>& indices, size_t bound, const char* name, const char* operation
) {
    if (!validate_device_indices()) {
        return;
    }
    std::vector<int32_t> host = copy_indices_to_host(indices);
    Tensor<int32_t, N> host_view = indices;
    host_view.data = host.data();
    checks::Validator(operation).index_range(host_view, name, bound);
}

/// Range and order check of the index that rows are scattered by.
inline void validate_scatter_index(
    const Tensor<int32_t, 1>& indices, size_t bound, const char* name, const char* operation
) {
    if (!validate_device_indices()) {
        return;
    }
    std::vector<int32_t> host = copy_indices_to_host(indices);
    Tensor<int32_t, 1> host_view = indices;
    host_view.data = host.data();
    checks::Validator(operation).index_range(host_view, name, bound);
    for (size_t i = 1; i < host.size(); i++) {
        if (host[i] < host[i - 1]) {
            throw std::runtime_error(
                std::string("Index array ") + name + " in operation " + operation +
                " is not sorted: element " + std::to_string(i) + " is " + std::to_string(host[i]) +
                " after " + std::to_string(host[i - 1]) +
                "; the device implementation needs a non-decreasing scatter index"
            );
        }
    }
}

} // namespace mops::amd

#endif
