#include "sender_buckets.hpp"

#include <algorithm>

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

// Small problems (a table of some thousands of entries over a few hundred values:
// the monomial table of HPE turned round) in ONE workgroup, without atomics on
// shared counters and without a sort afterwards: wavefront w looks after a
// contiguous share of the edges; counts per (wavefront, value) in LDS, a scan
// over them, and then every edge takes the next free place of its value, edges
// of one group of 64 with the same value in lane order (ranks from ballots
// over the bits of the value). The places are handed out in ascending edge
// order, so every list comes out sorted.
constexpr int SMALL_WAVES = 16;
constexpr int SMALL_THREADS = SMALL_WAVES * WAVE;
constexpr int32_t SMALL_MAX_NODES = 896; // (SMALL_WAVES + 1) counters per value in 64 KB of LDS
constexpr int32_t SMALL_MAX_EDGES = 131072;

/// LDS: counts[SMALL_WAVES][n_nodes] totals[n_nodes] (ints).
__global__ __launch_bounds__(SMALL_THREADS) void order_small_kernel(
    const int32_t* __restrict__ senders, int32_t n_edges, int32_t n_nodes, int32_t value_bits,
    int32_t* __restrict__ offsets, int32_t* __restrict__ sender_of_position, int32_t* __restrict__ edge_of_position
) {
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    int32_t* counts = reinterpret_cast<int32_t*>(lds_bytes);
    int32_t* totals = counts + SMALL_WAVES * n_nodes;
    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = tid >> 6;
    const int32_t share = (n_edges + SMALL_THREADS - 1) / SMALL_THREADS * WAVE;
    const int32_t my_begin = min(wave * share, n_edges);
    const int32_t my_end = min(my_begin + share, n_edges);
    // the value of edge e for this lane: negative if there is no such edge or the value is out of range
    auto value_of = [&](int32_t e) {
        const int32_t loaded = load_or_zero(senders, static_cast<size_t>(e), e < my_end);
        return e < my_end && in_bounds(loaded, n_nodes) ? loaded : -1;
    };

    for (int32_t i = tid; i < SMALL_WAVES * n_nodes; i += SMALL_THREADS) {
        counts[i] = 0;
    }
    __syncthreads();
    constexpr int AHEAD = 8; // loads in flight
    for (int32_t e0 = my_begin; e0 < my_end; e0 += AHEAD * WAVE) {
        int32_t value[AHEAD];
#pragma unroll
        for (int c = 0; c < AHEAD; c++) {
            value[c] = value_of(e0 + c * WAVE + lane);
        }
#pragma unroll
        for (int c = 0; c < AHEAD; c++) {
            if (value[c] >= 0) {
                atomicAdd(&counts[wave * n_nodes + value[c]], 1); // integer counts in LDS: no order involved
            }
        }
    }
    __syncthreads();
    // counts[w][v] := edges of value v in the shares before w; totals[v] := all of them
    if (tid < n_nodes) {
        int32_t running = 0;
        for (int w = 0; w < SMALL_WAVES; w++) {
            const int32_t here = counts[w * n_nodes + tid];
            counts[w * n_nodes + tid] = running;
            running += here;
        }
        totals[tid] = running;
    }
    __syncthreads();
    // inclusive scan of totals over the values (at most one per thread)
    for (int32_t step = 1; step < n_nodes; step <<= 1) {
        const int32_t mine = tid < n_nodes ? totals[tid] : 0;
        const int32_t left = tid < n_nodes && tid >= step ? totals[tid - step] : 0;
        __syncthreads();
        if (tid < n_nodes) {
            totals[tid] = mine + left;
        }
        __syncthreads();
    }
    const int32_t listed = totals[n_nodes - 1];
    if (tid < n_nodes) {
        const int32_t before = tid > 0 ? totals[tid - 1] : 0;
        offsets[tid] = before;
        if (tid == n_nodes - 1) {
            offsets[n_nodes] = totals[tid];
        }
        for (int w = 0; w < SMALL_WAVES; w++) {
            counts[w * n_nodes + tid] += before;
        }
    }
    __syncthreads();
    for (int32_t e0 = my_begin; e0 < my_end; e0 += AHEAD * WAVE) {
        int32_t value[AHEAD];
#pragma unroll
        for (int c = 0; c < AHEAD; c++) {
            value[c] = value_of(e0 + c * WAVE + lane);
        }
#pragma unroll
        for (int c = 0; c < AHEAD; c++) {
            if (e0 + c * WAVE < my_end) { // uniform
                const bool valid = value[c] >= 0;
                // the lanes with my value: agreement on every bit of it
                unsigned long long match = __ballot(valid);
                for (int32_t bit = 0; bit < value_bits; bit++) {
                    const bool set = ((value[c] >> bit) & 1) != 0;
                    const unsigned long long with_bit = __ballot(valid && set);
                    match &= set ? with_bit : ~with_bit;
                }
                const int32_t rank = __popcll(match & ((1ull << lane) - 1ull));
                const int32_t same = __popcll(match);
                int32_t place = -1;
                if (valid) {
                    place = counts[wave * n_nodes + value[c]] + rank;
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                if (valid && rank == same - 1) {
                    counts[wave * n_nodes + value[c]] += same; // one lane per value of the group
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                if (place >= 0) {
                    sender_of_position[place] = value[c];
                    edge_of_position[place] = e0 + c * WAVE + lane;
                }
            }
        }
    }
    for (int32_t at = listed + tid; at < n_edges; at += SMALL_THREADS) {
        sender_of_position[at] = n_nodes;
        edge_of_position[at] = 0;
    }
}

// Sparse graphs: one launch of list_in_slots_block (sender_buckets.hpp), four
// wavefronts per workgroup.
constexpr int SLOT_THREADS = 4 * WAVE;

__global__ __launch_bounds__(SLOT_THREADS) void list_in_slots_kernel(
    int32_t* __restrict__ slots, int32_t* __restrict__ counts, const int32_t* __restrict__ senders,
    int32_t n_edges, int32_t n_nodes, bool aligned
) {
    __shared__ SlotLists lists;
    list_in_slots_block<SLOT_THREADS>(lists, slots, counts, senders, n_edges, n_nodes, aligned, blockIdx.x);
}

// Sparse graphs, by arrival: one thread per edge.
constexpr int ARRIVAL_THREADS = 4 * WAVE;

__global__ __launch_bounds__(ARRIVAL_THREADS) void list_by_arrival_kernel(
    const SenderArrivals lists, const int32_t* __restrict__ senders, int32_t n_edges, int32_t n_nodes
) {
    const int32_t edge = static_cast<int32_t>(blockIdx.x) * ARRIVAL_THREADS + static_cast<int32_t>(threadIdx.x);
    if (edge < n_edges) {
        list_arrival(lists, n_nodes, senders[edge], edge);
    }
}

__global__ __launch_bounds__(ARRIVAL_THREADS) void clear_counters_kernel(int32_t* __restrict__ counters, size_t count) {
    const size_t at = static_cast<size_t>(blockIdx.x) * ARRIVAL_THREADS + threadIdx.x;
    if (at < count) {
        counters[at] = 0;
    }
}

} // namespace

size_t sender_slots_bytes(int32_t n_nodes) {
    return align256(static_cast<size_t>(n_nodes) * SLOT_CAPACITY * 4) +
           align256(static_cast<size_t>(n_nodes) * SLOT_PARTS * 4);
}

SenderSlots sender_slots_in(void* workspace, int32_t n_nodes) {
    int32_t* slots = static_cast<int32_t*>(workspace);
    int32_t* counts = reinterpret_cast<int32_t*>(
        static_cast<char*>(workspace) + align256(static_cast<size_t>(n_nodes) * SLOT_CAPACITY * 4)
    );
    return SenderSlots{slots, counts};
}

unsigned sender_slots_blocks(int32_t n_nodes) {
    return static_cast<unsigned>(ceil_div(static_cast<size_t>(std::max(n_nodes, 0)), SLOT_SENDERS)) * SLOT_PARTS;
}

SenderSlots list_edges_in_slots(
    const int32_t* senders, int32_t n_edges, int32_t n_nodes, void* workspace, hipStream_t stream
) {
    const SenderSlots slots = sender_slots_in(workspace, n_nodes);
    if (n_nodes > 0) {
        const bool aligned = reinterpret_cast<uintptr_t>(senders) % 16 == 0;
        list_in_slots_kernel<<<sender_slots_blocks(n_nodes), SLOT_THREADS, 0, stream>>>(
            const_cast<int32_t*>(slots.edges), const_cast<int32_t*>(slots.counts), senders, n_edges, n_nodes, aligned
        );
        MOPS_HIP_CHECK(hipGetLastError());
    }
    return slots;
}

SenderArrivals list_edges_by_arrival(
    const int32_t* senders, int32_t n_edges, int32_t n_nodes, int32_t copies, void* workspace, int32_t* counts,
    hipStream_t stream
) {
    const SenderArrivals lists{static_cast<int32_t*>(workspace), counts, copies};
    if (n_nodes > 0 && n_edges > 0) {
        const unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<size_t>(n_edges), ARRIVAL_THREADS));
        list_by_arrival_kernel<<<blocks, ARRIVAL_THREADS, 0, stream>>>(lists, senders, n_edges, n_nodes);
        MOPS_HIP_CHECK(hipGetLastError());
    }
    return lists;
}

void clear_counters(int32_t* counters, size_t count, hipStream_t stream) {
    if (count > 0) {
        const unsigned blocks = static_cast<unsigned>(ceil_div(count, ARRIVAL_THREADS));
        clear_counters_kernel<<<blocks, ARRIVAL_THREADS, 0, stream>>>(counters, count);
        MOPS_HIP_CHECK(hipGetLastError());
    }
}

size_t edges_by_sender_bytes(int32_t n_nodes, int32_t n_edges) {
    return sender_buckets_bytes(n_nodes, n_edges) + 2 * align256(static_cast<size_t>(n_edges) * 4);
}

EdgesBySender order_edges_by_sender(
    const int32_t* senders, int32_t n_edges, int32_t n_nodes, void* workspace, hipStream_t stream
) {
    if (n_nodes >= 1 && n_nodes <= SMALL_MAX_NODES && n_edges >= 1 && n_edges <= SMALL_MAX_EDGES) {
        // same places in the workspace as below
        char* at = static_cast<char*>(workspace);
        int32_t* offsets = reinterpret_cast<int32_t*>(at + align256(static_cast<size_t>(n_nodes) * 4));
        at += sender_buckets_bytes(n_nodes, n_edges);
        int32_t* sender_of_position = reinterpret_cast<int32_t*>(at);
        int32_t* edge_of_position = reinterpret_cast<int32_t*>(at + align256(static_cast<size_t>(n_edges) * 4));
        int32_t value_bits = 0;
        while ((1 << value_bits) < n_nodes) {
            value_bits++;
        }
        const size_t lds = static_cast<size_t>(SMALL_WAVES + 1) * n_nodes * sizeof(int32_t);
        order_small_kernel<<<1, SMALL_THREADS, lds, stream>>>(
            senders, n_edges, n_nodes, value_bits, offsets, sender_of_position, edge_of_position
        );
        MOPS_HIP_CHECK(hipGetLastError());
        return EdgesBySender{sender_of_position, edge_of_position, offsets};
    }
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
