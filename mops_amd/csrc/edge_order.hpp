// Scatter indices that are not sorted, on the device path.
//
// The scatter kernels (OPSA, OPSAW, SASAW) reduce over runs of equal values of
// the scatter index and therefore need it non-decreasing, like the device
// path of the reference (python/mops/tests/opsa.py:96 of lab-cosmo/mops); the
// reference's HOST path accepts any order (get_write_list,
// mops/src/internal/utils.cpp:7-14, mops/src/opsa/cpu.tpp:29). A calling
// thread that turns `accept_unsorted` on gets the host semantics on the
// device: every call first looks whether the index is sorted (one small
// kernel and a 4-byte copy back: the call then blocks once, so it cannot be
// captured into a graph) and, if it is not, sorts the edges by it with a
// STABLE sort, runs the kernels on the re-ordered rows and puts per-edge
// results back. Stable means that edges with the same destination keep their
// order, which is the order in which the host loops add them.
#ifndef MOPS_AMD_EDGE_ORDER_HPP
#define MOPS_AMD_EDGE_ORDER_HPP

#include <cstddef>
#include <cstdint>

#include <hip/hip_runtime.h>

#include "elementwise.hpp"

namespace mops::amd {

/// Per-thread switch (default: off, or on when the environment has
/// MOPS_AMD_ACCEPT_UNSORTED=1). Returns the previous setting.
bool accept_unsorted();
bool set_accept_unsorted(bool value);

/// Whether `index` (device memory, n values) is non-decreasing. Waits for the
/// stream.
bool is_sorted_on_device(const int32_t* index, int32_t n, hipStream_t stream);

/// The edges in the order of a stable sort by `index`.
class EdgeOrder {
public:
    EdgeOrder(const int32_t* index, int32_t n_edges, hipStream_t stream);

    /// index[permutation[p]], non-decreasing
    const int32_t* sorted_index() const { return sorted_.data(); }
    /// position p of the sorted order holds edge permutation[p]
    const int32_t* permutation() const { return permutation_.data(); }

    /// out[p, :] = in[permutation[p], :]
    template <typename T> void gather_rows(T* out, const T* in, int32_t width) const;
    /// out[permutation[p], :] = in[p, :]
    template <typename T> void scatter_rows(T* out, const T* in, int32_t width) const;

private:
    int32_t n_edges_;
    hipStream_t stream_;
    StreamTemporary<int32_t> sorted_;
    StreamTemporary<int32_t> permutation_;
};

} // namespace mops::amd

#endif
