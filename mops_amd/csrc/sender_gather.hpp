// Edges grouped by an UNSORTED index (the "sender" of a message-passing
// graph) inside the kernel that consumes them, without any list in global
// memory.
//
// A workgroup of NW wavefronts serves the NW consecutive nodes
// [node0, node0 + NW). All its wavefronts first read the whole sender index
// (wavefront v the v-th slice of it, 128-bit loads, the index stays in L2 for
// the other workgroups) and keep the few edges that name one of these nodes,
// in edge order, in a list in LDS; then wavefront s picks the edges of node
// node0 + s out of the lists and hands them on, 16 at a time.
//
// Lists are bounded (CAPACITY matches per slice); a wavefront whose list is
// full stops scanning, everything found so far is consumed, and the scan
// resumes where it stopped ("rounds"). With one round, the usual case, every
// node sees its edges in ascending order, which is the order of the
// reference's CPU loops over get_write_list (mops/src/internal/utils.cpp:7-14,
// used at mops/src/opsaw/cpu.tpp:102 and mops/src/sasaw/cpu.tpp:136); with
// more rounds (nodes named by thousands of edges) the order is a fixed
// interleaving of slices, still the same on every run.
//
// Compared with a counting sort in global memory (clear, count, scan, fill:
// four launches and two rounds of global atomics) this costs one pass over
// the index per workgroup, a few microseconds, and no launch.
#ifndef MOPS_AMD_SENDER_GATHER_HPP
#define MOPS_AMD_SENDER_GATHER_HPP

#include <cstdint>

#include <hip/hip_runtime.h>

#include "device_common.hpp"

namespace mops::amd {

/// Orders LDS traffic between the lanes of one wavefront.
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int NW> struct SenderGather {
    static constexpr int CAPACITY = 256; // >= 64 * 4: one load of a wavefront always fits
    static constexpr int RING = 128; // a power of two
    static constexpr int STAGE = 16;

    struct Storage {
        int32_t edges[NW][CAPACITY];
        int32_t ring[NW][RING];
        int32_t counts[NW];
        int32_t resume[NW];
        uint8_t which[NW][CAPACITY];
    };

    /// Called by all threads of the workgroup (blockDim.x == NW * 64).
    /// `on_stage(my_edge, n)` is called by wavefront s, all lanes, for every
    /// batch of n <= 16 edges of node node0 + s; lane k (and k + 16, k + 32,
    /// k + 48) holds edge k of the batch in `my_edge`, -1 beyond n.
    /// VEC = 4 needs `senders` aligned to 16 bytes.
    /// `keep_waiting`: batches are handed on while more edges than this wait
    /// (at most RING - 64, so that the matches of one more look fit): STAGE - 1
    /// hands every full batch on at once, RING - 64 collects as many edges as
    /// possible first, for consumers that only start loads per batch.
    template <int VEC, typename StageFn>
    static __device__ __forceinline__ void run(
        Storage& lds,
        const int32_t* __restrict__ senders,
        int32_t n_edges,
        int32_t node0,
        int32_t n_nodes,
        StageFn&& on_stage,
        int32_t keep_waiting = STAGE - 1
    ) {
        const int lane = threadIdx.x & (WAVE - 1);
        const int wave = threadIdx.x >> 6;
        const int32_t served = min(NW, n_nodes - node0);
        constexpr int UNIT = WAVE * VEC; // positions per load of a wavefront
        const int32_t total_units = (n_edges + UNIT - 1) / UNIT;
        const int32_t units_per_wave = (total_units + NW - 1) / NW;
        const int32_t unit_end = min((wave + 1) * units_per_wave, total_units);
        int32_t unit = min(wave * units_per_wave, total_units);
        const unsigned long long below = (1ull << lane) - 1ull;

        // the waiting edges of my node: a circular buffer of RING positions
        int32_t ring_head = 0;
        int32_t ring_count = 0;
        auto drain = [&](int32_t keep_below) {
            // hands on batches while more than `keep_below` edges wait
            while (ring_count > keep_below) {
                const int32_t n = min(STAGE, ring_count);
                const int k = lane & (STAGE - 1);
                const int32_t my_edge = k < n ? lds.ring[wave][(ring_head + k) & (RING - 1)] : -1;
                on_stage(my_edge, n);
                ring_head = (ring_head + n) & (RING - 1);
                ring_count -= n;
            }
        };

        // the wavefront of the last slice also looks after the last n_edges % 4 positions
        bool tail_done = VEC != 4 || wave != NW - 1;
        bool more = true;
        while (more) {
            // ---- scan my slice until it ends or my list is full
            int32_t count = 0;
            bool full = false;
            constexpr int BATCH = 8;
            while (unit < unit_end && !full) {
                int32_t values[BATCH][VEC];
#pragma unroll
                for (int u = 0; u < BATCH; u++) {
                    const int32_t position = (unit + u) * UNIT + lane * VEC;
                    if constexpr (VEC == 4) {
                        const bool whole = unit + u < unit_end && position + 3 < n_edges;
                        const int4 loaded =
                            *reinterpret_cast<const int4*>(senders + (whole ? position : 0));
                        values[u][0] = whole ? loaded.x : -1;
                        values[u][1] = whole ? loaded.y : -1;
                        values[u][2] = whole ? loaded.z : -1;
                        values[u][3] = whole ? loaded.w : -1;
                        // (the last n_edges % 4 positions are looked at below:
                        // a conditional load here would make every load of the
                        // batch wait for the one before)
                    } else {
                        const bool ok = unit + u < unit_end && position < n_edges;
                        values[u][0] = load_or_zero(senders, position, ok);
                        values[u][0] = ok ? values[u][0] : -1;
                    }
                }
                // The matches of one load go to the list together: every lane
                // counts its own, the lanes before it give its place (sums of
                // ballots over the bits of the counts: no loop over matches, no
                // scalar branches), and it writes them itself. Lane order, then
                // component order, is ascending edge order.
                int consumed = 0;
#pragma unroll
                for (int u = 0; u < BATCH; u++) {
                    if (full || unit + u >= unit_end) {
                        continue;
                    }
                    uint32_t found = 0; // bit c: component c names one of our nodes
#pragma unroll
                    for (int c = 0; c < VEC; c++) {
                        found |= in_bounds(values[u][c] - node0, served) ? (1u << c) : 0u;
                    }
                    if (__ballot(found != 0) != 0) {
                        const uint32_t mine = __popc(found); // 0..VEC, VEC <= 4
                        const unsigned long long ones = __ballot((mine & 1u) != 0);
                        const unsigned long long twos = __ballot((mine & 2u) != 0);
                        const unsigned long long fours = __ballot((mine & 4u) != 0);
                        const int32_t total = __popcll(ones) + 2 * __popcll(twos) + 4 * __popcll(fours);
                        if (count + total > CAPACITY) {
                            full = true;
                            continue;
                        }
                        const int32_t before =
                            __popcll(ones & below) + 2 * __popcll(twos & below) + 4 * __popcll(fours & below);
#pragma unroll
                        for (int c = 0; c < VEC; c++) {
                            if (found & (1u << c)) {
                                const int32_t slot = count + before + __popc(found & ((1u << c) - 1u));
                                lds.edges[wave][slot] = (unit + u) * UNIT + lane * VEC + c;
                                lds.which[wave][slot] = static_cast<uint8_t>(values[u][c] - node0);
                            }
                        }
                        count += total;
                    }
                    consumed = u + 1;
                }
                unit += consumed;
            }
            if (VEC == 4 && !tail_done && unit >= unit_end && !full) {
                // the positions after the last whole group of four
                if (count + 3 <= CAPACITY) {
                    for (int32_t position = n_edges & ~3; position < n_edges; position++) {
                        const int32_t value = senders[position];
                        if (in_bounds(value - node0, served)) {
                            lds.edges[wave][count] = position;
                            lds.which[wave][count] = static_cast<uint8_t>(value - node0);
                            count++;
                        }
                    }
                    tail_done = true;
                }
            }
            if (lane == 0) {
                lds.counts[wave] = count;
                lds.resume[wave] = (unit < unit_end || !tail_done) ? 1 : 0;
            }
            __syncthreads();

            // ---- pick my node's edges out of all lists
            more = false;
            for (int v = 0; v < NW; v++) {
                more |= lds.resume[v] != 0;
                const int32_t listed = lds.counts[v];
                for (int32_t base = 0; base < listed; base += WAVE) {
                    const int32_t at = base + lane;
                    const bool mine = at < listed && lds.which[v][at] == wave;
                    const unsigned long long mask = __ballot(mine);
                    if (mask != 0) {
                        if (mine) {
                            lds.ring[wave][(ring_head + ring_count + __popcll(mask & below)) & (RING - 1)] =
                                lds.edges[v][at];
                        }
                        ring_count += __popcll(mask);
                        wave_sync();
                        drain(keep_waiting);
                    }
                }
            }
            __syncthreads(); // the lists may be overwritten
        }
        wave_sync();
        drain(0);
    }
};

} // namespace mops::amd

#endif
