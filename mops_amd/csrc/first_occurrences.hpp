// Segment boundaries of a sorted index vector (device).
#ifndef MOPS_AMD_FIRST_OCCURRENCES_HPP
#define MOPS_AMD_FIRST_OCCURRENCES_HPP

#include <cstdint>

#include <hip/hip_runtime.h>

namespace mops::amd {

/// Enqueue on `stream` the kernel that fills `result[0 .. 2*n_output)`:
/// result[v] = first position j with sorted_indices[j] == v,
/// result[n_output + v] = one past the last such position, both -1 when v
/// does not occur. Every element of `result` is written exactly once, so the
/// buffer needs no initialisation. All pointers are device pointers.
void first_occurrences(
    const int32_t* sorted_indices,
    int32_t n_input,
    int32_t n_output,
    int32_t* result,
    hipStream_t stream
);

} // namespace mops::amd

#endif
