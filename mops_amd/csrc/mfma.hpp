// The one matrix instruction shape used by the kernels: D[16x16] += A[16x4] * B[4x16]
// on one wavefront, in float (v_mfma_f32_16x16x4_f32) and double
// (v_mfma_f64_16x16x4_f64).
//
// Operand layout (checked on the hardware with one-hot operands):
//   A[i][k]  lives in lane i + 16 * k            (i = lane & 15, k = lane >> 4)
//   B[k][j]  lives in lane j + 16 * k            (j = lane & 15, k = lane >> 4)
//   D[i][j]  lives in lane j + 16 * g, element r of the 4-vector, where
//            float :  i = 4 * g + r
//            double:  i = 4 * r + g
#ifndef MOPS_AMD_MFMA_HPP
#define MOPS_AMD_MFMA_HPP

#include <hip/hip_runtime.h>

namespace mops::amd {

template <typename T> struct Mfma;

template <> struct Mfma<float> {
    typedef float Acc __attribute__((ext_vector_type(4)));
    static __device__ __forceinline__ Acc zero() { return Acc{0.f, 0.f, 0.f, 0.f}; }
    static __device__ __forceinline__ Acc mma(float a, float b, Acc c) {
        return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
    }
    /// row i of D held in element r of `lane`
    static __device__ __forceinline__ int row(int lane, int r) { return 4 * (lane >> 4) + r; }
};

template <> struct Mfma<double> {
    typedef double Acc __attribute__((ext_vector_type(4)));
    static __device__ __forceinline__ Acc zero() { return Acc{0., 0., 0., 0.}; }
    static __device__ __forceinline__ Acc mma(double a, double b, Acc c) {
        return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ int row(int lane, int r) { return 4 * r + (lane >> 4); }
};

} // namespace mops::amd

#endif
