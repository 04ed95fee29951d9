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

#include <climits>
#include <cstddef>
#include <cstdint>

#include <hip/hip_runtime.h>

#include "device_common.hpp"
#include "runtime.hpp"

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

/// Sparse graphs (a few dozen edges per sender): every sender owns
/// SLOT_CAPACITY places, so no offsets have to be known before the lists are
/// written and ONE launch does it, without counters shared between workgroups
/// and without anything to clear first. The index is cut into SLOT_PARTS parts
/// of consecutive edges, each looked at by workgroups of its own, and so are a
/// sender's places: its edges in part p go to places [32 p, 32 p + 32). The
/// parts one after the other are the sender's edges in ascending order.
constexpr int SLOT_PARTS = 4;
constexpr int SLOT_PART_CAPACITY = 32;
constexpr int SLOT_CAPACITY = SLOT_PARTS * SLOT_PART_CAPACITY;
struct SenderSlots {
    /// [n_nodes][SLOT_PARTS][SLOT_PART_CAPACITY] the edges that name the node in
    /// each part of the index, ascending, in the first counts[node][part] places
    /// (nothing in a part whose count exceeds SLOT_PART_CAPACITY)
    const int32_t* edges;
    /// [n_nodes][SLOT_PARTS] number of edges of the part that name the node (may
    /// exceed SLOT_PART_CAPACITY: the consumer then has to find the node's edges
    /// itself)
    const int32_t* counts;
};

/// Bytes of scratch memory list_edges_in_slots needs.
size_t sender_slots_bytes(int32_t n_nodes);

/// Where the two arrays lie in a workspace of sender_slots_bytes() bytes (for a
/// kernel that does the listing among other work: list_in_slots_block).
SenderSlots sender_slots_in(void* workspace, int32_t n_nodes);

/// Workgroups the listing takes: SLOT_PARTS for every 16 senders.
unsigned sender_slots_blocks(int32_t n_nodes);

/// Enqueue the kernel that lists the edges of every sender in its slots
/// (values outside [0, n_nodes) are dropped). A workgroup serves 16 senders and
/// reads a quarter of the index: meant for graphs where n_edges * n_nodes / 16
/// is small.
SenderSlots list_edges_in_slots(
    const int32_t* senders, int32_t n_edges, int32_t n_nodes, void* workspace, hipStream_t stream
);

/// Senders per workgroup of the listing.
constexpr int SLOT_SENDERS = 16;
/// LDS of one workgroup of the listing.
struct SlotLists {
    int32_t edges[SLOT_SENDERS][SLOT_PART_CAPACITY];
    int32_t found[SLOT_SENDERS];
};

/// The listing itself, called by ALL threads of a workgroup of THREADS threads
/// (a multiple of 64): workgroup `block` lists the edges of senders
/// [16 g, 16 g + 16), g = block / SLOT_PARTS, in part block % SLOT_PARTS of the
/// index. Every thread looks at its share of the part, sixteen loads in flight
/// (128-bit loads when `aligned`: `senders` on a 16-byte boundary); an edge that
/// names one of the sixteen takes the next place of that sender's list in LDS
/// (integer LDS atomic: the places depend on the order of arrival, the set of
/// edges does not); a wavefront then puts a list in ascending order (the rank of
/// an edge is the number of smaller ones: edge numbers are distinct) and writes
/// it to the sender's slots. A device function so that a kernel with other work
/// can give some of its workgroups to it: no launch of its own then.
template <int THREADS>
__device__ __forceinline__ void list_in_slots_block(
    SlotLists& lds, int32_t* __restrict__ slots, int32_t* __restrict__ counts,
    const int32_t* __restrict__ senders, int32_t n_edges, int32_t n_nodes, bool aligned, int32_t block
) {
    constexpr int WAVES = THREADS / WAVE;
    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = tid >> 6;
    const int32_t part = block % SLOT_PARTS;
    const int32_t node0 = block / SLOT_PARTS * SLOT_SENDERS;
    const int32_t served = min(SLOT_SENDERS, n_nodes - node0);
    if (tid < SLOT_SENDERS) {
        lds.found[tid] = 0;
    }
    __syncthreads();
    auto look = [&](int32_t value, int32_t edge) {
        const int32_t which = value - node0;
        if (in_bounds(which, served)) {
            const int32_t place = atomicAdd(&lds.found[which], 1);
            if (place < SLOT_PART_CAPACITY) {
                lds.edges[which][place] = edge;
            }
        }
    };
    // four positions at once: the four places are asked for together, so that a
    // thread waits for the LDS once and not four times
    auto look4 = [&](const int4& values, int32_t edge) {
        const int32_t which[4] = {values.x - node0, values.y - node0, values.z - node0, values.w - node0};
        int32_t place[4];
#pragma unroll
        for (int c = 0; c < 4; c++) {
            place[c] = SLOT_PART_CAPACITY;
            if (in_bounds(which[c], served)) {
                place[c] = atomicAdd(&lds.found[which[c]], 1);
            }
        }
#pragma unroll
        for (int c = 0; c < 4; c++) {
            if (place[c] < SLOT_PART_CAPACITY) {
                lds.edges[which[c]][place[c]] = edge + c;
            }
        }
    };
    constexpr int AHEAD = 16;
    if (aligned) {
        // parts of whole groups of four; the last part also takes the n_edges % 4 edges after them
        const int32_t groups = n_edges >> 2;
        const int32_t per_part = (groups + SLOT_PARTS - 1) / SLOT_PARTS;
        const int32_t begin = min(part * per_part, groups);
        const int32_t end = min(begin + per_part, groups);
        for (int32_t g0 = begin; g0 < end; g0 += AHEAD * THREADS) {
            int4 values[AHEAD];
#pragma unroll
            for (int u = 0; u < AHEAD; u++) {
                // beyond the end: a group that exists, and values that name nobody
                // (a conditional load would make every load wait for the one before)
                const int32_t g = g0 + u * THREADS + tid;
                const bool ok = g < end;
                const int4 loaded = reinterpret_cast<const int4*>(senders)[ok ? g : 0];
                values[u].x = ok ? loaded.x : -1;
                values[u].y = ok ? loaded.y : -1;
                values[u].z = ok ? loaded.z : -1;
                values[u].w = ok ? loaded.w : -1;
            }
#pragma unroll
            for (int u = 0; u < AHEAD; u++) {
                look4(values[u], (g0 + u * THREADS + tid) << 2);
            }
        }
        const int32_t e = (n_edges & ~3) + tid;
        if (part == SLOT_PARTS - 1 && tid < 4 && e < n_edges) {
            look(senders[e], e);
        }
    } else {
        const int32_t per_part = (n_edges + SLOT_PARTS - 1) / SLOT_PARTS;
        const int32_t begin = min(part * per_part, n_edges);
        const int32_t end = min(begin + per_part, n_edges);
        for (int32_t e0 = begin; e0 < end; e0 += AHEAD * THREADS) {
            int32_t values[AHEAD];
#pragma unroll
            for (int u = 0; u < AHEAD; u++) {
                const int32_t e = e0 + u * THREADS + tid;
                const int32_t loaded = load_or_zero(senders, static_cast<size_t>(e), e < end);
                values[u] = e < end ? loaded : -1;
            }
#pragma unroll
            for (int u = 0; u < AHEAD; u++) {
                look(values[u], e0 + u * THREADS + tid);
            }
        }
    }
    __syncthreads();
    for (int32_t which = wave; which < served; which += WAVES) {
        const int32_t n = lds.found[which];
        if (lane < n && n <= SLOT_PART_CAPACITY) {
            const int32_t edge = lds.edges[which][lane];
            int32_t rank = 0;
            for (int32_t other = 0; other < n; other++) {
                rank += lds.edges[which][other] < edge ? 1 : 0; // the same address for all lanes
            }
            slots[(static_cast<size_t>(node0 + which) * SLOT_PARTS + part) * SLOT_PART_CAPACITY + rank] = edge;
        }
        if (lane == 0) {
            counts[static_cast<size_t>(node0 + which) * SLOT_PARTS + part] = n;
        }
    }
}

/// Sparse graphs, with ONE look at every edge: a sender owns SLOT_CAPACITY
/// places and a counter in global memory, and an edge takes the next place of
/// its sender (an integer atomic that returns the count before it). The places
/// of a sender then hold its edges in the order of arrival, which whoever uses
/// them puts right first (arrivals_in_order). No workgroup reads more of the
/// index than its own share: 4 bytes per edge instead of 4 bytes per edge and
/// 16 senders.
///
/// The counters have to be zero before the listing. Every counter is read by
/// exactly one wavefront of the consuming launch, which sets it back to zero:
/// nothing has to be cleared between calls (or between replays of a graph).
/// A consuming launch in which `copies` wavefronts want the list of the same
/// sender gets `copies` counters per sender, all of which count every edge.
struct SenderArrivals {
    /// [n_nodes][SLOT_CAPACITY] edges that name the node, in the order of arrival
    int32_t* edges;
    /// [copies][n_nodes] number of edges that name the node (may exceed
    /// SLOT_CAPACITY: the consumer then has to find the node's edges itself)
    int32_t* counts;
    int32_t copies;
};

/// Bytes of scratch memory the places take (the counters are elsewhere).
inline size_t sender_arrivals_bytes(int32_t n_nodes) {
    return align256(static_cast<size_t>(n_nodes) * SLOT_CAPACITY * 4);
}

/// Edge `edge` names `sender`: called by one thread per edge.
__device__ __forceinline__ void list_arrival(
    const SenderArrivals& lists, int32_t n_nodes, int32_t sender, int32_t edge
) {
    if (in_bounds(sender, n_nodes)) {
        const int32_t place = atomicAdd(&lists.counts[sender], 1);
        for (int32_t c = 1; c < lists.copies; c++) {
            atomicAdd(&lists.counts[static_cast<size_t>(c) * n_nodes + sender], 1);
        }
        if (place < SLOT_CAPACITY) {
            lists.edges[static_cast<size_t>(sender) * SLOT_CAPACITY + place] = edge;
        }
    }
}

/// Enqueue the kernel that lists the edges of every sender by arrival (values
/// outside [0, n_nodes) are dropped). `counts`: copies x n_nodes counters, zero.
SenderArrivals list_edges_by_arrival(
    const int32_t* senders, int32_t n_edges, int32_t n_nodes, int32_t copies, void* workspace, int32_t* counts,
    hipStream_t stream
);

/// Enqueue a kernel that sets `count` counters to zero (for counters whose
/// earlier contents are not known).
void clear_counters(int32_t* counters, size_t count, hipStream_t stream);

/// A sender's `count` <= SLOT_CAPACITY places (lane k holds places k and
/// k + 64 in `first_half`, `second_half`) in ascending order: lane k gets
/// entries k and k + 64 of the sorted list. Edge numbers are distinct, so the
/// rank of one is the number of smaller ones. `area`: SLOT_CAPACITY integers in
/// LDS for this wavefront alone (used for lists of more than 64 edges).
__device__ __forceinline__ void arrivals_in_order(
    int32_t& first_half, int32_t& second_half, int32_t count, int32_t* area, int lane
) {
    const int32_t mine0 = lane < count ? first_half : INT32_MAX;
    const int32_t mine1 = lane + WAVE < count ? second_half : INT32_MAX;
    int32_t rank0 = 0, rank1 = 0;
    if (count <= WAVE) {
        for (int32_t k = 0; k < count; k++) {
            rank0 += __builtin_amdgcn_readlane(mine0, k) < mine0 ? 1 : 0;
        }
        // (lanes without an edge send to themselves)
        first_half = __builtin_amdgcn_ds_permute((lane < count ? rank0 : lane) << 2, mine0);
        second_half = mine1;
        return;
    }
    for (int32_t k = 0; k < WAVE; k++) {
        const int32_t other = __builtin_amdgcn_readlane(mine0, k);
        rank0 += other < mine0 ? 1 : 0;
        rank1 += other < mine1 ? 1 : 0;
    }
    for (int32_t k = 0; k < count - WAVE; k++) {
        const int32_t other = __builtin_amdgcn_readlane(mine1, k);
        rank0 += other < mine0 ? 1 : 0;
        rank1 += other < mine1 ? 1 : 0;
    }
    area[rank0] = mine0;
    area[lane + WAVE < count ? rank1 : lane + WAVE] = mine1;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    first_half = area[lane];
    second_half = area[lane + WAVE];
    // (the next list of this wavefront is written after these reads)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

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
