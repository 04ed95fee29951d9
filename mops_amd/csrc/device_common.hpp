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

/// Division of small non-negative integers by a run-time constant without a
/// divide: the host computes `magic = ceil(2^32 / divisor)` once, the device
/// takes the high half of a 32x32 multiplication. Exact for all
/// 0 <= n with n * divisor < 2^32 (checked by the host before it picks a
/// kernel that uses this). An integer division by a run-time value costs
/// some thirty instructions on this hardware; index arithmetic of that kind
/// in front of every element dominated the instruction count of the staging
/// loops before.
struct FastDivisor {
    uint32_t divisor;
    uint32_t magic;

    __host__ static FastDivisor make(uint32_t divisor) {
        FastDivisor d;
        d.divisor = divisor;
        d.magic = divisor <= 1
                      ? 0u
                      : static_cast<uint32_t>(((uint64_t(1) << 32) + divisor - 1) / divisor);
        return d;
    }

    __device__ __forceinline__ uint32_t divide(uint32_t n) const {
        return divisor <= 1 ? n : __umulhi(n, magic);
    }
};

/// `pointer[index]` when `ok`, else 0, WITHOUT a branch: the load is always
/// issued (from element 0 when not ok, which must exist) and the value is
/// selected afterwards. A conditional load would be compiled to a branch
/// that waits for its own load, which serialises a batch of loads that are
/// meant to be in flight together.
template <typename T>
__device__ __forceinline__ T load_or_zero(const T* __restrict__ pointer, size_t index, bool ok) {
    const T value = pointer[ok ? index : 0];
    return ok ? value : T(0);
}

} // namespace mops::amd

#endif
