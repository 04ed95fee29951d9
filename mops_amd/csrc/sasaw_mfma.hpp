// Matrix-core path of SASAW for the table shapes of equivariant message
// passing (at most 16 values of every component index; any number of feature
// channels, taken 64 at a time). sasaw.hip calls it when `supports()` says so
// and keeps its general kernels for everything else.
#ifndef MOPS_AMD_SASAW_MFMA_HPP
#define MOPS_AMD_SASAW_MFMA_HPP

#include <cstddef>
#include <cstdint>

#include <hip/hip_runtime.h>

namespace mops::amd::sasaw_mfma {

struct Shape {
    int32_t n_nodes; // rows of the output / of W
    int32_t n_edges;
    int32_t nA;      // A.shape[1]
    int32_t L;       // B.shape[1]
    int32_t N;       // entries of the coupling table
    int32_t n2;      // W.shape[1]
    int32_t n3;      // output.shape[1]
};

struct Indices {
    const int32_t* A;        // [N]
    const int32_t* W_1;      // [n_edges]  sender
    const int32_t* W_2;      // [N]
    const int32_t* output_1; // [n_edges]  receiver, sorted
    const int32_t* output_2; // [N]
};

/// Whether these kernels cover the shape for elements of `element_size` bytes.
bool supports(const Shape& shape, size_t element_size);

/// Device scratch the calls below need.
size_t workspace_bytes(const Shape& shape, size_t element_size);

template <typename T>
void forward(
    T* output, const T* A, const T* B, const T* C, const T* W, const Indices& indices,
    const Shape& shape, void* workspace, hipStream_t stream
);

/// Whether grad_W of this shape first puts the edges in the order of their
/// senders by a counting sort (large graphs whose senders' edges overflow the
/// slots).
bool orders_edges_by_sender(const Shape& shape, size_t element_size);

/// Whether vjp() for this shape and these wanted gradients only launches
/// kernels on `stream` with `workspace` as their temporary memory: no second
/// stream, no events, no allocation.
bool vjp_allocates_nothing(const Shape& shape, size_t element_size, bool want_edge_gradients, bool want_grad_W);

/// Any of grad_A, grad_B, grad_W may be null.
template <typename T>
void vjp(
    T* grad_A, T* grad_B, T* grad_W, const T* grad_output, const T* A, const T* B, const T* C,
    const T* W, const Indices& indices, const Shape& shape, void* workspace, hipStream_t stream
);

} // namespace mops::amd::sasaw_mfma

#endif
