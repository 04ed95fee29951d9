#include "elementwise.hpp"

#include <algorithm>
#include <cstdint>

#include "runtime.hpp"

namespace mops::amd {
namespace {

constexpr int THREADS = 256;

template <typename T> __global__ __launch_bounds__(THREADS) void fill_zero_kernel(T* __restrict__ data, size_t count) {
    for (size_t i = blockIdx.x * static_cast<size_t>(THREADS) + threadIdx.x; i < count;
         i += static_cast<size_t>(gridDim.x) * THREADS) {
        data[i] = T(0);
    }
}

template <typename T>
__global__ __launch_bounds__(THREADS) void add_in_place_kernel(
    T* __restrict__ target, const T* __restrict__ addend, size_t count
) {
    for (size_t i = blockIdx.x * static_cast<size_t>(THREADS) + threadIdx.x; i < count;
         i += static_cast<size_t>(gridDim.x) * THREADS) {
        target[i] += addend[i];
    }
}

unsigned blocks_for(size_t count) {
    return static_cast<unsigned>(std::min<size_t>(ceil_div(count, THREADS), 8192));
}

} // namespace

template <typename T> void fill_zero(T* data, size_t count, hipStream_t stream) {
    if (count == 0) {
        return;
    }
    fill_zero_kernel<T><<<blocks_for(count), THREADS, 0, stream>>>(data, count);
    MOPS_HIP_CHECK(hipGetLastError());
}

template <typename T> void add_in_place(T* target, const T* addend, size_t count, hipStream_t stream) {
    if (count == 0) {
        return;
    }
    add_in_place_kernel<T><<<blocks_for(count), THREADS, 0, stream>>>(target, addend, count);
    MOPS_HIP_CHECK(hipGetLastError());
}

template <typename T> StreamTemporary<T>::StreamTemporary(size_t count, hipStream_t stream) : stream_(stream) {
    if (count > 0) {
        void* block = nullptr;
        MOPS_HIP_CHECK(hipMallocAsync(&block, count * sizeof(T), stream));
        data_ = static_cast<T*>(block);
    }
}

template <typename T> StreamTemporary<T>::~StreamTemporary() {
    if (data_ != nullptr) {
        (void)hipFreeAsync(data_, stream_);
    }
}

template void fill_zero<float>(float*, size_t, hipStream_t);
template void fill_zero<double>(double*, size_t, hipStream_t);
template void add_in_place<float>(float*, const float*, size_t, hipStream_t);
template void add_in_place<double>(double*, const double*, size_t, hipStream_t);
template class StreamTemporary<float>;
template class StreamTemporary<double>;
template class StreamTemporary<int32_t>;
template class StreamTemporary<unsigned char>;

} // namespace mops::amd
