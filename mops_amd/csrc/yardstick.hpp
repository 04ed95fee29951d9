// A plain copy kernel that benchmarks use as the yardstick for the time it
// takes to move an operation's algorithmic bytes (mops/amd.h: mops_amd_copy_yardstick).
#ifndef MOPS_AMD_YARDSTICK_HPP
#define MOPS_AMD_YARDSTICK_HPP

#include <cstdint>

#include <hip/hip_runtime.h>

namespace mops::amd {

constexpr int YARDSTICK_MAX_SPANS = 16;

struct YardstickSpan {
    const void* data;
    int64_t bytes;
};

/// One launch on `stream` that reads every span of `reads` once and writes
/// every span of `writes` once.
void copy_yardstick(
    const YardstickSpan* reads, int n_reads, const YardstickSpan* writes, int n_writes, hipStream_t stream
);

} // namespace mops::amd

#endif
