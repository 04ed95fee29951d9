// first_occurrences: for a sorted index vector, the [first, one-past-last)
// range of positions of every value. Integer work, bit-exact.
//
// What it replaces: mops/src/internal/cuda_first_occurences.cu:14-117 of
// lab-cosmo/mops, which clears the result to -1 with a memset and then lets
// threads that see a change of value write the two boundaries. Here one
// kernel writes EVERY element of the result exactly once, so there is no
// separate clear: the thread that sees the value change from `previous` to
// `current` also writes -1/-1 for the values strictly between them, the
// thread of element 0 for the values below the first one, and the thread of
// the last element for the values above the last one. An empty input fills
// the whole result with -1 (the reference reads element 0 unguarded).
#include "first_occurrences.hpp"

#include "runtime.hpp"

namespace mops::amd {

namespace {

constexpr int THREADS = 256;

__global__ __launch_bounds__(THREADS) void first_occurrences_kernel(
    const int32_t* __restrict__ sorted_indices,
    int32_t n_input,
    int32_t n_output,
    int32_t* __restrict__ first,
    int32_t* __restrict__ last
) {
    const int32_t position = blockIdx.x * THREADS + threadIdx.x;

    if (n_input == 0) {
        for (int32_t v = position; v < n_output; v += gridDim.x * THREADS) {
            first[v] = -1;
            last[v] = -1;
        }
        return;
    }
    if (position >= n_input) {
        return;
    }

    const int32_t current = sorted_indices[position];
    const bool is_first = position == 0;
    const bool is_last = position == n_input - 1;
    const int32_t previous = is_first ? -1 : sorted_indices[position - 1];
    const bool in_range = current >= 0 && current < n_output;

    if (is_first || current != previous) {
        if (in_range) {
            first[current] = position;
        }
        // values skipped between the previous segment and this one
        int32_t absent_end = current < n_output ? current : n_output;
        for (int32_t v = previous + 1 > 0 ? previous + 1 : 0; v < absent_end; v++) {
            first[v] = -1;
            last[v] = -1;
        }
    }
    if (is_last || current != sorted_indices[position + 1]) {
        if (in_range) {
            last[current] = position + 1;
        }
    }
    if (is_last) {
        for (int32_t v = current + 1 > 0 ? current + 1 : 0; v < n_output; v++) {
            first[v] = -1;
            last[v] = -1;
        }
    }
}

} // namespace

void first_occurrences(
    const int32_t* sorted_indices,
    int32_t n_input,
    int32_t n_output,
    int32_t* result,
    hipStream_t stream
) {
    if (n_output == 0) {
        return;
    }
    int32_t work = n_input > 0 ? n_input : n_output;
    unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<size_t>(work), THREADS));
    if (n_input == 0 && blocks > 1024) {
        blocks = 1024;
    }
    first_occurrences_kernel<<<blocks, THREADS, 0, stream>>>(
        sorted_indices, n_input, n_output, result, result + n_output
    );
    MOPS_HIP_CHECK(hipGetLastError());
}

} // namespace mops::amd
