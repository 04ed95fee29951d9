// Non-owning tensor view used by the C++ API: a pointer plus N extents.
// Same contract as mops/include/mops/tensor.hpp:7-13 of lab-cosmo/mops:
// contiguous row-major data, passed by value, `data == nullptr` marks an
// optional gradient that is not requested.
#ifndef MOPS_TENSOR_HPP
#define MOPS_TENSOR_HPP

#include <cstddef>
#include <cstdint>

namespace mops {

template <typename scalar_t, size_t N_DIMS> struct Tensor {
    scalar_t* __restrict__ data;
    size_t shape[N_DIMS];
};

} // namespace mops

#endif
