// The one entry point of the library that allocates nothing (mops/amd.h:
// mops_amd_sparse_accumulation_scatter_add_with_weights_vjp_no_alloc_f32).
#ifndef MOPS_AMD_NO_ALLOC_HPP
#define MOPS_AMD_NO_ALLOC_HPP

#include <cstddef>
#include <cstdint>

#include "mops/tensor.hpp"

namespace mops::amd {

/// Bytes of the file-scope device array that stands in for the scratch block.
constexpr size_t NO_ALLOC_SCRATCH_BYTES = size_t(4) << 20;

/// mops::cuda::sparse_accumulation_scatter_add_with_weights_vjp<float> with
/// its temporaries in that array; throws for shapes whose temporaries do not
/// fit or whose kernels need more than the array (see mops/amd.h).
void sasaw_vjp_no_alloc(
    Tensor<float, 2> grad_A,
    Tensor<float, 2> grad_B,
    Tensor<float, 3> grad_W,
    Tensor<float, 3> grad_output,
    Tensor<float, 2> A,
    Tensor<float, 2> B,
    Tensor<float, 1> C,
    Tensor<float, 3> W,
    Tensor<int32_t, 1> indices_A,
    Tensor<int32_t, 1> indices_W_1,
    Tensor<int32_t, 1> indices_W_2,
    Tensor<int32_t, 1> indices_output_1,
    Tensor<int32_t, 1> indices_output_2
);

} // namespace mops::amd

#endif
