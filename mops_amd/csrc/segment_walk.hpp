// Ownership of output rows by wavefronts, for reductions over a SORTED index.
//
// The positions 0..n_input of the sorted index are cut into chunks of CHUNK
// consecutive positions, one wavefront per chunk. A wavefront owns every
// segment (maximal run of equal values) that STARTS inside its chunk, and
// follows such a segment beyond the end of the chunk if it continues there.
// So every segment has exactly one owner, found from a single look at CHUNK
// index values: no separate pass over the index, no table of boundaries in
// memory, no atomics. The boundaries are those first_occurrences would give:
// [first, last) of each value.
//
// The owner of a segment also learns which output rows just before it receive
// nothing (the values skipped between the previous segment and this one); the
// owner of position 0 learns the rows before the first value and the owner of
// the last position the rows after the last value. Calling `on_empty_rows`
// for these ranges lets a kernel write every output row exactly once.
#ifndef MOPS_AMD_SEGMENT_WALK_HPP
#define MOPS_AMD_SEGMENT_WALK_HPP

#include <cstdint>

#include <hip/hip_runtime.h>

#include "device_common.hpp"

namespace mops::amd {

/// Called by all lanes of a wavefront. `wave_index` is the global number of
/// the wavefront (uniform). CHUNK <= 64.
///   on_segment(row, first, last)  all lanes, uniform arguments, 0 <= row < n_rows
///   on_empty_rows(begin, end)     all lanes, rows in [begin, end) receive nothing
template <int CHUNK, typename SegmentFn, typename EmptyRowsFn>
__device__ __forceinline__ void walk_owned_segments(
    const int32_t* __restrict__ sorted_index,
    int32_t n_input,
    int32_t n_rows,
    int32_t wave_index,
    SegmentFn&& on_segment,
    EmptyRowsFn&& on_empty_rows
) {
    static_assert(CHUNK >= 1 && CHUNK <= WAVE, "one index value per lane");
    const int lane = threadIdx.x & (WAVE - 1);
    const int32_t chunk_begin = wave_index * CHUNK;
    if (chunk_begin >= n_input) {
        return;
    }
    const int32_t position = chunk_begin + lane;
    const bool inside = lane < CHUNK && position < n_input;
    const int32_t mine = inside ? sorted_index[position] : 0;
    const int32_t before = (inside && position > 0) ? sorted_index[position - 1] : -1;
    // the 64 positions after the chunk, asked for now: the last segment of the
    // chunk almost always ends there, and its end is then known without
    // another round trip to memory
    const int32_t ahead_position = chunk_begin + CHUNK + lane;
    const int32_t ahead = load_or_zero(sorted_index, static_cast<size_t>(ahead_position), ahead_position < n_input);
    const bool starts_here = inside && (position == 0 || mine != before);

    unsigned long long starts = __ballot(starts_here);
    while (starts != 0) {
        const int start_lane = __ffsll(static_cast<long long>(starts)) - 1;
        starts &= starts - 1;
        const int32_t first = chunk_begin + start_lane;
        const int32_t row = __shfl(mine, start_lane);
        const int32_t previous_row = __shfl(before, start_lane); // -1 at position 0

        int32_t last;
        if (starts != 0) {
            last = chunk_begin + __ffsll(static_cast<long long>(starts)) - 1;
        } else {
            // the run reaches the end of the chunk: follow it
            last = n_input;
            for (int32_t probe = chunk_begin + CHUNK; probe < n_input; probe += WAVE) {
                const int32_t at = probe + lane;
                const bool first_look = probe == chunk_begin + CHUNK; // uniform
                const int32_t value = first_look ? ahead : load_or_zero(sorted_index, static_cast<size_t>(at), at < n_input);
                const bool differs = at >= n_input || value != row;
                const unsigned long long mask = __ballot(differs);
                if (mask != 0) {
                    last = min(probe + __ffsll(static_cast<long long>(mask)) - 1, n_input);
                    break;
                }
            }
        }

        const int32_t empty_begin = max(previous_row + 1, 0);
        const int32_t empty_end = min(row, n_rows);
        if (empty_begin < empty_end) {
            on_empty_rows(empty_begin, empty_end);
        }
        if (in_bounds(row, n_rows)) {
            on_segment(row, first, last);
        }
    }

    // rows after the last value
    if (n_input - 1 >= chunk_begin && n_input - 1 < chunk_begin + CHUNK) {
        const int32_t tail_begin = max(sorted_index[n_input - 1] + 1, 0);
        if (tail_begin < n_rows) {
            on_empty_rows(tail_begin, n_rows);
        }
    }
}

} // namespace mops::amd

#endif
