#include "sender_buckets.hpp"

#include "runtime.hpp"

namespace mops::amd {

namespace {

constexpr int THREADS = 256;
constexpr int SCAN_THREADS = 1024;

__global__ __launch_bounds__(THREADS) void clear_kernel(int32_t* __restrict__ data, int32_t count) {
    int32_t i = blockIdx.x * THREADS + threadIdx.x;
    if (i < count) {
        data[i] = 0;
    }
}

// integer atomics: the final counts do not depend on the order of arrival
__global__ __launch_bounds__(THREADS) void count_kernel(
    const int32_t* __restrict__ senders, int32_t n_edges, int32_t n_nodes, int32_t* __restrict__ counts
) {
    int32_t e = blockIdx.x * THREADS + threadIdx.x;
    if (e < n_edges) {
        int32_t node = senders[e];
        if (in_bounds(node, n_nodes)) {
            atomicAdd(&counts[node], 1);
        }
    }
}

// one workgroup: exclusive prefix sum of counts -> offsets (and a copy of the
// offsets in `cursor`, the running insertion point of each list)
__global__ __launch_bounds__(SCAN_THREADS) void scan_kernel(
    const int32_t* __restrict__ counts,
    int32_t n_nodes,
    int32_t* __restrict__ offsets,
    int32_t* __restrict__ cursor
) {
    __shared__ int32_t tile[SCAN_THREADS];
    __shared__ int32_t carry;
    const int tid = threadIdx.x;
    if (tid == 0) {
        carry = 0;
    }
    __syncthreads();
    for (int32_t base = 0; base < n_nodes; base += SCAN_THREADS) {
        int32_t i = base + tid;
        int32_t value = i < n_nodes ? counts[i] : 0;
        tile[tid] = value;
        __syncthreads();
        for (int distance = 1; distance < SCAN_THREADS; distance <<= 1) {
            int32_t add = tid >= distance ? tile[tid - distance] : 0;
            __syncthreads();
            tile[tid] += add;
            __syncthreads();
        }
        int32_t exclusive = carry + tile[tid] - value;
        if (i < n_nodes) {
            offsets[i] = exclusive;
            cursor[i] = exclusive;
        }
        __syncthreads();
        if (tid == SCAN_THREADS - 1) {
            carry += tile[tid];
        }
        __syncthreads();
    }
    if (tid == 0) {
        offsets[n_nodes] = carry;
    }
}

// the position inside a list depends on the order of arrival; consumers sort
// each list, so the arrival order never reaches a floating-point sum
__global__ __launch_bounds__(THREADS) void fill_kernel(
    const int32_t* __restrict__ senders,
    int32_t n_edges,
    int32_t n_nodes,
    int32_t* __restrict__ cursor,
    int32_t* __restrict__ order
) {
    int32_t e = blockIdx.x * THREADS + threadIdx.x;
    if (e < n_edges) {
        int32_t node = senders[e];
        if (in_bounds(node, n_nodes)) {
            int32_t slot = atomicAdd(&cursor[node], 1);
            order[slot] = e;
        }
    }
}

// workgroup `node` writes its list, sorted, and its own number next to every
// entry; workgroup n_nodes fills what is left after the last list
// (threads, entries sorted in LDS; longer lists take the slow way through global memory):
// small workgroups for the short lists of a graph, large ones where lists are long on average
constexpr int SHORT_LIST_THREADS = 64;
constexpr int SHORT_LIST_CAPACITY = BUCKET_LDS_CAPACITY;
constexpr int LONG_LIST_THREADS = 256;
constexpr int LONG_LIST_CAPACITY = 8192;

template <int LIST_THREADS, int LIST_LDS_CAPACITY>
__global__ __launch_bounds__(LIST_THREADS) void write_lists_kernel(
    SenderBuckets buckets, int32_t n_nodes, int32_t n_edges, int32_t* __restrict__ sender_of_position,
    int32_t* __restrict__ edge_of_position
) {
    __shared__ int32_t list[LIST_LDS_CAPACITY];
    const int32_t node = blockIdx.x;
    if (node == n_nodes) {
        for (int32_t at = buckets.offsets[n_nodes] + threadIdx.x; at < n_edges; at += LIST_THREADS) {
            sender_of_position[at] = n_nodes;
            edge_of_position[at] = 0;
        }
        return;
    }
    const int32_t begin = buckets.offsets[node];
    const SortedBucket sorted = sorted_bucket(buckets, node, list, LIST_LDS_CAPACITY);
    for (int32_t at = threadIdx.x; at < sorted.count; at += LIST_THREADS) {
        sender_of_position[begin + at] = node;
        edge_of_position[begin + at] = sorted.edges[at];
    }
}

} // namespace

size_t edges_by_sender_bytes(int32_t n_nodes, int32_t n_edges) {
    return sender_buckets_bytes(n_nodes, n_edges) + 2 * align256(static_cast<size_t>(n_edges) * 4);
}

EdgesBySender order_edges_by_sender(
    const int32_t* senders, int32_t n_edges, int32_t n_nodes, void* workspace, hipStream_t stream
) {
    const SenderBuckets buckets = build_sender_buckets(senders, n_edges, n_nodes, workspace, stream);
    char* base = static_cast<char*>(workspace) + sender_buckets_bytes(n_nodes, n_edges);
    int32_t* sender_of_position = reinterpret_cast<int32_t*>(base);
    int32_t* edge_of_position = reinterpret_cast<int32_t*>(base + align256(static_cast<size_t>(n_edges) * 4));
    if (static_cast<size_t>(n_edges) <= static_cast<size_t>(n_nodes) * 256) {
        write_lists_kernel<SHORT_LIST_THREADS, SHORT_LIST_CAPACITY>
            <<<static_cast<unsigned>(n_nodes) + 1, SHORT_LIST_THREADS, 0, stream>>>(
                buckets, n_nodes, n_edges, sender_of_position, edge_of_position
            );
    } else {
        write_lists_kernel<LONG_LIST_THREADS, LONG_LIST_CAPACITY>
            <<<static_cast<unsigned>(n_nodes) + 1, LONG_LIST_THREADS, 0, stream>>>(
                buckets, n_nodes, n_edges, sender_of_position, edge_of_position
            );
    }
    MOPS_HIP_CHECK(hipGetLastError());
    return EdgesBySender{sender_of_position, edge_of_position, buckets.offsets};
}

size_t sender_buckets_bytes(int32_t n_nodes, int32_t n_edges) {
    size_t nodes = static_cast<size_t>(n_nodes);
    size_t edges = static_cast<size_t>(n_edges);
    return align256(nodes * 4) + align256((nodes + 1) * 4) + align256(nodes * 4) +
           2 * align256(edges * 4);
}

SenderBuckets build_sender_buckets(
    const int32_t* senders, int32_t n_edges, int32_t n_nodes, void* workspace, hipStream_t stream
) {
    char* base = static_cast<char*>(workspace);
    size_t nodes = static_cast<size_t>(n_nodes);
    size_t edges = static_cast<size_t>(n_edges);
    int32_t* counts = reinterpret_cast<int32_t*>(base);
    base += align256(nodes * 4);
    int32_t* offsets = reinterpret_cast<int32_t*>(base);
    base += align256((nodes + 1) * 4);
    int32_t* cursor = reinterpret_cast<int32_t*>(base);
    base += align256(nodes * 4);
    int32_t* order = reinterpret_cast<int32_t*>(base);
    base += align256(edges * 4);
    int32_t* order_sorted = reinterpret_cast<int32_t*>(base);

    unsigned node_blocks = static_cast<unsigned>(ceil_div(nodes, THREADS));
    unsigned edge_blocks = static_cast<unsigned>(ceil_div(edges, THREADS));

    if (node_blocks > 0) {
        clear_kernel<<<node_blocks, THREADS, 0, stream>>>(counts, n_nodes);
    }
    if (edge_blocks > 0) {
        count_kernel<<<edge_blocks, THREADS, 0, stream>>>(senders, n_edges, n_nodes, counts);
    }
    scan_kernel<<<1, SCAN_THREADS, 0, stream>>>(counts, n_nodes, offsets, cursor);
    if (edge_blocks > 0) {
        fill_kernel<<<edge_blocks, THREADS, 0, stream>>>(senders, n_edges, n_nodes, cursor, order);
    }
    MOPS_HIP_CHECK(hipGetLastError());
    return SenderBuckets{offsets, order, order_sorted};
}

} // namespace mops::amd
