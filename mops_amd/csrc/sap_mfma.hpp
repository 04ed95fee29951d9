// Matrix-core path of SAP for small dense index ranges (the Clebsch-Gordan
// tables of equivariant models: a dozen values per index). sap.hip calls it
// when `supports()` says so and keeps its table-driven kernels otherwise.
#ifndef MOPS_AMD_SAP_MFMA_HPP
#define MOPS_AMD_SAP_MFMA_HPP

#include <cstddef>
#include <cstdint>

#include <hip/hip_runtime.h>

namespace mops::amd::sap_mfma {

struct Shape {
    int32_t n_rows;
    int32_t nA; // A.shape[1]
    int32_t nB; // B.shape[1]
    int32_t nO; // output.shape[1]
    int32_t K;  // entries of the table
};

struct Table {
    const void* C; // [K] coefficients
    const int32_t* indices_A;
    const int32_t* indices_B;
    const int32_t* indices_output;
};

bool supports_forward(const Shape& shape, size_t element_size);
bool supports_vjp(const Shape& shape, size_t element_size);

template <typename T>
void forward(T* output, const T* A, const T* B, const Table& table, const Shape& shape, hipStream_t stream);

/// output = sap(A, B) + sap(A2, B2) in one launch (what the second-order
/// function needs: the sum of the forward with grad_grad_A for A and of the
/// forward with grad_grad_B for B). Shapes of `supports_forward` whose launch
/// has a workgroup for every 128 rows.
bool supports_forward_of_two_pairs(const Shape& shape, size_t element_size);
template <typename T>
void forward_of_two_pairs(
    T* output, const T* A, const T* B, const T* A2, const T* B2, const Table& table, const Shape& shape,
    hipStream_t stream
);

/// grad_A or grad_B may be null.
template <typename T>
void vjp(
    T* grad_A, T* grad_B, const T* grad_output, const T* A, const T* B, const Table& table,
    const Shape& shape, hipStream_t stream
);

} // namespace mops::amd::sap_mfma

#endif
