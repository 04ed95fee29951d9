// Small device-side helpers shared by the kernels.
#ifndef MOPS_AMD_DEVICE_COMMON_HPP
#define MOPS_AMD_DEVICE_COMMON_HPP

#include <cstdint>

#include <hip/hip_runtime.h>

namespace mops::amd {

constexpr int WAVE = 64; // wavefront width of CDNA

/// 0 <= value < bound, in one unsigned comparison.
__device__ __forceinline__ bool in_bounds(int32_t value, int32_t bound) {
    return static_cast<uint32_t>(value) < static_cast<uint32_t>(bound);
}

/// Next extent >= n that is odd, used as LDS row stride so that lanes that
/// walk down a column (stride = row length) fall into different banks.
__host__ __device__ __forceinline__ int odd_stride(int n) { return n | 1; }

/// Round up to a multiple of the wavefront width.
__host__ __device__ __forceinline__ int round_up_wave(int n) {
    return (n + WAVE - 1) / WAVE * WAVE;
}

} // namespace mops::amd

#endif
