// A plain copy kernel as a yardstick for the operations' kernels: it reads a
// list of spans of device memory once and writes another list once, 16 bytes
// per lane, and does nothing else. A benchmark points it at the very tensors
// an operation reads and writes; the time it takes is what moving the
// operation's algorithmic bytes costs on this device at this size.
#include "yardstick.hpp"

#include <algorithm>
#include <stdexcept>

#include "runtime.hpp"

namespace mops::amd {
namespace {

constexpr int THREADS = 256;

struct Spans {
    const uint32_t* data[YARDSTICK_MAX_SPANS];
    uint64_t first_piece[YARDSTICK_MAX_SPANS + 1]; // prefix sums of the pieces (16 bytes; the last may be short)
    uint32_t words[YARDSTICK_MAX_SPANS];           // 4-byte words of the span
    int32_t count;
};

/// The span that holds `piece`, and the piece's number inside it.
__device__ __forceinline__ int locate(const Spans& spans, uint64_t piece, uint64_t& within) {
    int span = 0;
#pragma unroll
    for (int s = 1; s < YARDSTICK_MAX_SPANS; s++) {
        span += (s < spans.count && piece >= spans.first_piece[s]) ? 1 : 0;
    }
    within = piece - spans.first_piece[span];
    return span;
}

constexpr int IN_FLIGHT = 4; // pieces a thread asks for before it looks at any of them

__device__ __forceinline__ uint4 read_piece(const Spans& reads, uint64_t piece, bool inside) {
    uint64_t within;
    const int span = locate(reads, inside ? piece : 0, within);
    const uint32_t* from = reads.data[span] + 4 * within;
    const uint32_t left = reads.words[span] - static_cast<uint32_t>(4 * within);
    uint4 value = make_uint4(0u, 0u, 0u, 0u);
    if (inside && left >= 4) {
        value = *reinterpret_cast<const uint4*>(from);
    } else if (inside) {
        for (uint32_t w = 0; w < left; w++) {
            value.x ^= from[w];
        }
    }
    return value;
}

__global__ __launch_bounds__(THREADS) void copy_yardstick_kernel(const Spans reads, const Spans writes) {
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * THREADS;
    const uint64_t start = static_cast<uint64_t>(blockIdx.x) * THREADS + threadIdx.x;
    uint4 seen = make_uint4(0u, 0u, 0u, 0u);
    const uint64_t read_pieces = reads.first_piece[reads.count];
    for (uint64_t piece = start; piece < read_pieces; piece += IN_FLIGHT * stride) {
        uint4 value[IN_FLIGHT];
#pragma unroll
        for (int u = 0; u < IN_FLIGHT; u++) {
            value[u] = read_piece(reads, piece + u * stride, piece + u * stride < read_pieces);
        }
#pragma unroll
        for (int u = 0; u < IN_FLIGHT; u++) {
            seen.x ^= value[u].x;
            seen.y ^= value[u].y;
            seen.z ^= value[u].z;
            seen.w ^= value[u].w;
        }
    }
    const uint64_t write_pieces = writes.first_piece[writes.count];
    for (uint64_t piece = start; piece < write_pieces; piece += stride) {
        uint64_t within;
        const int span = locate(writes, piece, within);
        uint32_t* to = const_cast<uint32_t*>(writes.data[span]) + 4 * within;
        const uint32_t left = writes.words[span] - static_cast<uint32_t>(4 * within);
        if (left >= 4) {
            *reinterpret_cast<uint4*>(to) = seen;
        } else {
            for (uint32_t w = 0; w < left; w++) {
                to[w] = seen.x;
            }
        }
    }
}

Spans pack(const YardstickSpan* spans, int count, const char* what) {
    if (count < 0 || count > YARDSTICK_MAX_SPANS) {
        throw std::runtime_error(std::string("copy yardstick: at most 16 spans to ") + what);
    }
    Spans packed{};
    packed.count = count;
    uint64_t pieces = 0;
    for (int s = 0; s < count; s++) {
        if (spans[s].bytes < 0 || spans[s].bytes % 4 != 0 || reinterpret_cast<uintptr_t>(spans[s].data) % 16 != 0 ||
            spans[s].bytes / 4 > 0xffffffffll) {
            throw std::runtime_error(
                std::string("copy yardstick: every span to ") + what +
                " must start at a multiple of 16 bytes and hold a multiple of 4 bytes (fewer than 16 GiB)"
            );
        }
        packed.data[s] = static_cast<const uint32_t*>(spans[s].data);
        packed.words[s] = static_cast<uint32_t>(spans[s].bytes / 4);
        packed.first_piece[s] = pieces;
        pieces += static_cast<uint64_t>((spans[s].bytes + 15) / 16);
    }
    for (int s = count; s <= YARDSTICK_MAX_SPANS; s++) {
        packed.first_piece[s] = pieces;
    }
    return packed;
}

} // namespace

void copy_yardstick(
    const YardstickSpan* reads, int n_reads, const YardstickSpan* writes, int n_writes, hipStream_t stream
) {
    const Spans from = pack(reads, n_reads, "read");
    const Spans to = pack(writes, n_writes, "write");
    const uint64_t pieces = std::max(from.first_piece[from.count], to.first_piece[to.count]);
    if (pieces == 0) {
        return;
    }
    // a few pieces per thread, all of a thread's loads in flight together, and no more than
    // eight workgroups per compute unit
    const unsigned blocks =
        static_cast<unsigned>(std::min<uint64_t>(ceil_div(pieces, THREADS * IN_FLIGHT), 256 * 8));
    copy_yardstick_kernel<<<blocks, THREADS, 0, stream>>>(from, to);
    MOPS_HIP_CHECK(hipGetLastError());
}

} // namespace mops::amd
