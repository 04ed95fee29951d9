// Edges grouped by an UNSORTED index (the "sender" of a message-passing
// graph): a counting sort that yields, for every node, the list of edges that
// name it. Needed by the weight gradients of OPSAW and SASAW, which scatter by
// the sender index; grouping first turns that scatter into a gather, so no
// floating-point atomics are needed and the sums are reproducible.
//
// The reference's CPU code does the same bucketing on the host
// (get_write_list on indices_W, mops/src/opsaw/cpu.tpp:102,
// mops/src/sasaw/cpu.tpp:136, mops/src/internal/utils.cpp:7-14); the
// reference has no device version.
#ifndef MOPS_AMD_SENDER_BUCKETS_HPP
#define MOPS_AMD_SENDER_BUCKETS_HPP

#include <cstddef>
#include <cstdint>

#include <hip/hip_runtime.h>

#include "device_common.hpp"

namespace mops::amd {

struct SenderBuckets {
    /// [n_nodes + 1] start of every node's list in `order`
    const int32_t* offsets;
    /// [n_edges] edge numbers grouped by node; inside one node's list the
    /// order is arbitrary (it is made ascending by whoever consumes it)
    const int32_t* order;
    /// [n_edges] spare room for consumers that have to sort a list that does
    /// not fit in LDS
    int32_t* order_sorted;
};

/// Bytes of scratch memory build_sender_buckets needs.
size_t sender_buckets_bytes(int32_t n_nodes, int32_t n_edges);

/// Enqueue the kernels that group edges 0..n_edges by senders[e] (values
/// outside [0, n_nodes) are dropped). `workspace` must hold
/// sender_buckets_bytes() bytes of device memory.
SenderBuckets build_sender_buckets(
    const int32_t* senders, int32_t n_edges, int32_t n_nodes, void* workspace, hipStream_t stream
);

/// The edges in the order of their senders, edges of one sender in ascending
/// edge number: what a kernel needs that walks a SORTED index
/// (segment_walk.hpp) over the senders.
struct EdgesBySender {
    /// [n_edges] sender of position p, non-decreasing; positions after the
    /// last listed edge (edges whose sender is out of range are not listed)
    /// hold n_nodes
    const int32_t* sender;
    /// [n_edges] edge number of position p (0 after the last listed edge)
    const int32_t* edge;
    /// [n_nodes + 1] first position of every sender's edges
    const int32_t* offsets;
};

/// Bytes of scratch memory order_edges_by_sender needs.
size_t edges_by_sender_bytes(int32_t n_nodes, int32_t n_edges);

/// Enqueue the kernels that order the edges by senders[e]. `workspace` must
/// hold edges_by_sender_bytes() bytes of device memory.
EdgesBySender order_edges_by_sender(
    const int32_t* senders, int32_t n_edges, int32_t n_nodes, void* workspace, hipStream_t stream
);

/// Capacity (in edges) of the LDS array passed to sorted_bucket.
constexpr int BUCKET_LDS_CAPACITY = 1024;

/// A node's edge list in ascending edge order.
struct SortedBucket {
    const int32_t* edges; // LDS or global
    int32_t count;
};

/// Called by ALL threads of a workgroup: returns node `node`'s edges sorted
/// ascending, which makes every consumer sum in one fixed order (the order of
/// the reference's CPU loops). Lists of up to BUCKET_LDS_CAPACITY edges are
/// sorted in `lds` (a bitonic network); longer ones by counting ranks through
/// the global spare buffer.
/// `capacity`: entries `lds` has room for (BUCKET_LDS_CAPACITY unless the caller has more).
__device__ inline SortedBucket sorted_bucket(
    const SenderBuckets& buckets, int32_t node, int32_t* lds, int32_t capacity = BUCKET_LDS_CAPACITY
) {
    const int32_t begin = buckets.offsets[node];
    const int32_t count = buckets.offsets[node + 1] - begin;
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;

    if (count <= capacity) {
        int padded = 1;
        while (padded < count) {
            padded <<= 1;
        }
        for (int i = tid; i < padded; i += nthreads) {
            lds[i] = i < count ? buckets.order[begin + i] : INT32_MAX;
        }
        __syncthreads();
        for (int span = 2; span <= padded; span <<= 1) {
            for (int step = span >> 1; step > 0; step >>= 1) {
                for (int i = tid; i < padded; i += nthreads) {
                    int partner = i ^ step;
                    if (partner > i) {
                        int32_t low = lds[i];
                        int32_t high = lds[partner];
                        bool ascending = (i & span) == 0;
                        if ((low > high) == ascending) {
                            lds[i] = high;
                            lds[partner] = low;
                        }
                    }
                }
                __syncthreads();
            }
        }
        return SortedBucket{lds, count};
    }

    // Long list: every edge number is unique, so its rank is the number of
    // smaller entries.
    const int32_t* unsorted = buckets.order + begin;
    int32_t* sorted = buckets.order_sorted + begin;
    for (int i = tid; i < count; i += nthreads) {
        int32_t mine = unsorted[i];
        int32_t rank = 0;
        for (int j = 0; j < count; j++) {
            rank += unsorted[j] < mine ? 1 : 0;
        }
        sorted[rank] = mine;
    }
    __threadfence();
    __syncthreads();
    return SortedBucket{sorted, count};
}

} // namespace mops::amd

#endif
