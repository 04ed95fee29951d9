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
//
// SPLIT > 0 (walk_split_segments): segments are additionally cut at every
// multiple of SPLIT positions, so that no piece is longer than SPLIT and a
// long segment is shared by many wavefronts. A piece is reported with whether
// it begins where its segment begins and ends where its segment ends; whoever
// calls this has to add up the pieces of a cut segment afterwards.
#ifndef MOPS_AMD_SEGMENT_WALK_HPP
#define MOPS_AMD_SEGMENT_WALK_HPP

#include <cstdint>

#include <hip/hip_runtime.h>

#include "device_common.hpp"

namespace mops::amd {

/// What a wavefront looks at of the sorted index: asked for as early as a
/// kernel likes (the loads do not depend on anything), used by walk_pieces.
struct ChunkIndex {
    int32_t mine;   // value at the lane's position of the chunk
    int32_t before; // value at the position before it (-1 in front of position 0)
    int32_t ahead;  // value at the lane's position of the 64 positions after the chunk
};

/// `chunk`: positions per wavefront, 1..64 (uniform).
__device__ __forceinline__ ChunkIndex load_chunk_index_of(
    const int32_t* __restrict__ sorted_index, int32_t n_input, int32_t wave_index, const int32_t chunk
) {
    const int lane = threadIdx.x & (WAVE - 1);
    const int32_t chunk_begin = wave_index * chunk;
    const int32_t position = chunk_begin + lane;
    const bool inside = lane < chunk && position < n_input;
    ChunkIndex index;
    index.mine = load_or_zero(sorted_index, static_cast<size_t>(position), inside);
    index.before = (inside && position > 0) ? sorted_index[position - 1] : -1;
    // the 64 positions after the chunk, asked for now: the last segment of the
    // chunk almost always ends there, and its end is then known without
    // another round trip to memory
    const int32_t ahead_position = chunk_begin + chunk + lane;
    index.ahead = load_or_zero(sorted_index, static_cast<size_t>(ahead_position), ahead_position < n_input);
    return index;
}

template <int CHUNK>
__device__ __forceinline__ ChunkIndex load_chunk_index(
    const int32_t* __restrict__ sorted_index, int32_t n_input, int32_t wave_index
) {
    static_assert(CHUNK >= 1 && CHUNK <= WAVE, "one index value per lane");
    return load_chunk_index_of(sorted_index, n_input, wave_index, CHUNK);
}

/// Called by all lanes of a wavefront. `wave_index` is the global number of
/// the wavefront (uniform). CHUNK <= 64 (a template argument of the wrappers
/// below, or a uniform run-time value of walk_pieces_of). `index`:
/// load_chunk_index of the same arguments.
///   on_segment(row, first, last)  all lanes, uniform arguments, 0 <= row < n_rows
///   on_empty_rows(begin, end)     all lanes, rows in [begin, end) receive nothing
///   on_piece(row, first, last, from_start, to_end)   (walk_split_segments)
template <int SPLIT, typename PieceFn, typename EmptyRowsFn>
__device__ __forceinline__ void walk_pieces_of(
    const int32_t* __restrict__ sorted_index,
    int32_t n_input,
    int32_t n_rows,
    int32_t wave_index,
    const int32_t chunk,
    const ChunkIndex& index,
    PieceFn&& on_piece,
    EmptyRowsFn&& on_empty_rows
) {
    const int lane = threadIdx.x & (WAVE - 1);
    const int32_t chunk_begin = wave_index * chunk;
    if (chunk_begin >= n_input) {
        return;
    }
    const int32_t position = chunk_begin + lane;
    const bool inside = lane < chunk && position < n_input;
    const int32_t mine = index.mine;
    const int32_t before = index.before;
    const int32_t ahead = index.ahead;
    const bool segment_starts_here = inside && (position == 0 || mine != before);
    const bool starts_here = segment_starts_here || (SPLIT > 0 && inside && position % (SPLIT > 0 ? SPLIT : 1) == 0);

    unsigned long long starts = __ballot(starts_here);
    const unsigned long long segment_starts = __ballot(segment_starts_here);
    while (starts != 0) {
        const int start_lane = __ffsll(static_cast<long long>(starts)) - 1;
        starts &= starts - 1;
        const int32_t first = chunk_begin + start_lane;
        const int32_t row = __shfl(mine, start_lane);
        const int32_t previous_row = __shfl(before, start_lane); // -1 at position 0

        const bool from_start = ((segment_starts >> start_lane) & 1) != 0;
        bool to_end = true;
        int32_t last;
        if (starts != 0) {
            const int next_lane = __ffsll(static_cast<long long>(starts)) - 1;
            last = chunk_begin + next_lane;
            to_end = ((segment_starts >> next_lane) & 1) != 0;
        } else {
            // the run reaches the end of the chunk: follow it (to the next cut at most)
            int32_t limit = n_input;
            if constexpr (SPLIT > 0) {
                limit = min(n_input, (first / SPLIT + 1) * SPLIT);
            }
            last = limit;
            bool found_end = false;
            for (int32_t probe = chunk_begin + chunk; probe < limit; probe += WAVE) {
                const int32_t at = probe + lane;
                const bool first_look = probe == chunk_begin + chunk; // uniform
                const int32_t value = first_look ? ahead : load_or_zero(sorted_index, static_cast<size_t>(at), at < n_input);
                const bool differs = at >= n_input || value != row;
                const unsigned long long mask = __ballot(differs);
                if (mask != 0) {
                    const int32_t end = min(probe + __ffsll(static_cast<long long>(mask)) - 1, n_input);
                    if (end <= limit) {
                        last = end;
                        found_end = true;
                    }
                    break;
                }
            }
            if constexpr (SPLIT > 0) {
                if (!found_end && last < n_input) {
                    to_end = sorted_index[last] != row; // the piece stops at a cut: does the segment?
                }
            }
        }

        const int32_t empty_begin = max(previous_row + 1, 0);
        const int32_t empty_end = min(row, n_rows);
        if (from_start && empty_begin < empty_end) {
            on_empty_rows(empty_begin, empty_end);
        }
        if (in_bounds(row, n_rows)) {
            on_piece(row, first, last, from_start, to_end);
        }
    }

    // rows after the last value
    if (n_input - 1 >= chunk_begin && n_input - 1 < chunk_begin + chunk) {
        const int32_t tail_begin = max(sorted_index[n_input - 1] + 1, 0);
        if (tail_begin < n_rows) {
            on_empty_rows(tail_begin, n_rows);
        }
    }
}

template <int CHUNK, int SPLIT, typename PieceFn, typename EmptyRowsFn>
__device__ __forceinline__ void walk_pieces(
    const int32_t* __restrict__ sorted_index,
    int32_t n_input,
    int32_t n_rows,
    int32_t wave_index,
    const ChunkIndex& index,
    PieceFn&& on_piece,
    EmptyRowsFn&& on_empty_rows
) {
    static_assert(CHUNK >= 1 && CHUNK <= WAVE, "one index value per lane");
    static_assert(SPLIT == 0 || SPLIT % CHUNK == 0, "cuts fall on chunk boundaries");
    walk_pieces_of<SPLIT>(sorted_index, n_input, n_rows, wave_index, CHUNK, index, on_piece, on_empty_rows);
}

template <int CHUNK, typename SegmentFn, typename EmptyRowsFn>
__device__ __forceinline__ void walk_owned_segments(
    const int32_t* __restrict__ sorted_index,
    int32_t n_input,
    int32_t n_rows,
    int32_t wave_index,
    SegmentFn&& on_segment,
    EmptyRowsFn&& on_empty_rows
) {
    if (wave_index * CHUNK >= n_input) {
        return;
    }
    const ChunkIndex index = load_chunk_index<CHUNK>(sorted_index, n_input, wave_index);
    walk_pieces<CHUNK, 0>(
        sorted_index, n_input, n_rows, wave_index, index,
        [&](int32_t row, int32_t first, int32_t last, bool, bool) { on_segment(row, first, last); }, on_empty_rows
    );
}

/// The same with the index values asked for beforehand (load_chunk_index).
template <int CHUNK, typename SegmentFn, typename EmptyRowsFn>
__device__ __forceinline__ void walk_owned_segments(
    const int32_t* __restrict__ sorted_index,
    int32_t n_input,
    int32_t n_rows,
    int32_t wave_index,
    const ChunkIndex& index,
    SegmentFn&& on_segment,
    EmptyRowsFn&& on_empty_rows
) {
    walk_pieces<CHUNK, 0>(
        sorted_index, n_input, n_rows, wave_index, index,
        [&](int32_t row, int32_t first, int32_t last, bool, bool) { on_segment(row, first, last); }, on_empty_rows
    );
}

template <int CHUNK, int SPLIT, typename PieceFn, typename EmptyRowsFn>
__device__ __forceinline__ void walk_split_segments(
    const int32_t* __restrict__ sorted_index,
    int32_t n_input,
    int32_t n_rows,
    int32_t wave_index,
    PieceFn&& on_piece,
    EmptyRowsFn&& on_empty_rows
) {
    static_assert(SPLIT > 0, "distance between cuts");
    if (wave_index * CHUNK >= n_input) {
        return;
    }
    const ChunkIndex index = load_chunk_index<CHUNK>(sorted_index, n_input, wave_index);
    walk_pieces<CHUNK, SPLIT>(sorted_index, n_input, n_rows, wave_index, index, on_piece, on_empty_rows);
}

} // namespace mops::amd

#endif
