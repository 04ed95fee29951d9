#include "edge_order.hpp"

#include <algorithm>
#include <cstdlib>
#include <cstring>

#include <rocprim/rocprim.hpp>

#include "runtime.hpp"

namespace mops::amd {
namespace {

constexpr int THREADS = 256;

struct Switch {
    bool value;
    Switch() {
        const char* text = std::getenv("MOPS_AMD_ACCEPT_UNSORTED");
        value = text != nullptr && std::strcmp(text, "0") != 0 && text[0] != '\0';
    }
};

Switch& the_switch() {
    static thread_local Switch instance;
    return instance;
}

__global__ __launch_bounds__(THREADS) void find_descent_kernel(
    const int32_t* __restrict__ index, int32_t n, int32_t* __restrict__ descents
) {
    bool found = false;
    for (size_t i = blockIdx.x * static_cast<size_t>(THREADS) + threadIdx.x; i + 1 < static_cast<size_t>(n);
         i += static_cast<size_t>(gridDim.x) * THREADS) {
        found |= index[i] > index[i + 1];
    }
    if (found) {
        *descents = 1; // every writer stores the same value
    }
}

__global__ void clear_flag_kernel(int32_t* flag) { *flag = 0; }

template <typename T, bool GATHER>
__global__ __launch_bounds__(THREADS) void move_rows_kernel(
    T* __restrict__ out, const T* __restrict__ in, const int32_t* __restrict__ permutation, size_t count,
    int32_t width
) {
    for (size_t i = blockIdx.x * static_cast<size_t>(THREADS) + threadIdx.x; i < count;
         i += static_cast<size_t>(gridDim.x) * THREADS) {
        const size_t p = i / width;
        const size_t column = i - p * width;
        const size_t other = static_cast<size_t>(permutation[p]) * width + column;
        if (GATHER) {
            out[i] = in[other];
        } else {
            out[other] = in[i];
        }
    }
}

unsigned blocks_for(size_t count) {
    return static_cast<unsigned>(std::min<size_t>(ceil_div(std::max<size_t>(count, 1), THREADS), 8192));
}

} // namespace

bool accept_unsorted() { return the_switch().value; }

bool set_accept_unsorted(bool value) {
    const bool previous = the_switch().value;
    the_switch().value = value;
    return previous;
}

bool is_sorted_on_device(const int32_t* index, int32_t n, hipStream_t stream) {
    if (n < 2) {
        return true;
    }
    StreamTemporary<int32_t> flag(1, stream);
    clear_flag_kernel<<<1, 1, 0, stream>>>(flag.data());
    find_descent_kernel<<<blocks_for(static_cast<size_t>(n)), THREADS, 0, stream>>>(index, n, flag.data());
    MOPS_HIP_CHECK(hipGetLastError());
    int32_t descents = 0;
    MOPS_HIP_CHECK(hipMemcpyAsync(&descents, flag.data(), sizeof(int32_t), hipMemcpyDeviceToHost, stream));
    MOPS_HIP_CHECK(hipStreamSynchronize(stream));
    return descents == 0;
}

EdgeOrder::EdgeOrder(const int32_t* index, int32_t n_edges, hipStream_t stream)
    : n_edges_(n_edges), stream_(stream), sorted_(static_cast<size_t>(n_edges), stream),
      permutation_(static_cast<size_t>(n_edges), stream) {
    if (n_edges == 0) {
        return;
    }
    // radix sort of (index value, edge number) pairs by the value: stable, so
    // equal values keep ascending edge numbers
    rocprim::counting_iterator<int32_t> edge_numbers(0);
    size_t temporary_bytes = 0;
    MOPS_HIP_CHECK(rocprim::radix_sort_pairs(
        nullptr, temporary_bytes, index, sorted_.data(), edge_numbers, permutation_.data(),
        static_cast<size_t>(n_edges), 0, 32, stream
    ));
    StreamTemporary<unsigned char> temporary(temporary_bytes, stream);
    MOPS_HIP_CHECK(rocprim::radix_sort_pairs(
        temporary.data(), temporary_bytes, index, sorted_.data(), edge_numbers, permutation_.data(),
        static_cast<size_t>(n_edges), 0, 32, stream
    ));
}

template <typename T> void EdgeOrder::gather_rows(T* out, const T* in, int32_t width) const {
    const size_t count = static_cast<size_t>(n_edges_) * width;
    if (count == 0) {
        return;
    }
    move_rows_kernel<T, true><<<blocks_for(count), THREADS, 0, stream_>>>(out, in, permutation_.data(), count, width);
    MOPS_HIP_CHECK(hipGetLastError());
}

template <typename T> void EdgeOrder::scatter_rows(T* out, const T* in, int32_t width) const {
    const size_t count = static_cast<size_t>(n_edges_) * width;
    if (count == 0) {
        return;
    }
    move_rows_kernel<T, false><<<blocks_for(count), THREADS, 0, stream_>>>(out, in, permutation_.data(), count, width);
    MOPS_HIP_CHECK(hipGetLastError());
}

template void EdgeOrder::gather_rows<float>(float*, const float*, int32_t) const;
template void EdgeOrder::gather_rows<double>(double*, const double*, int32_t) const;
template void EdgeOrder::gather_rows<int32_t>(int32_t*, const int32_t*, int32_t) const;
template void EdgeOrder::scatter_rows<float>(float*, const float*, int32_t) const;
template void EdgeOrder::scatter_rows<double>(double*, const double*, int32_t) const;

} // namespace mops::amd
