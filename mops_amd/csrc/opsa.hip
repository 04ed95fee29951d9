// Outer-product scatter-add, without (OPSA) and with (OPSAW) per-sender
// weights, forward and vector-Jacobian product, for gfx950.
//
//   OPSA   O[P[j], k, l]  += A[j, k] * B[j, l]
//   OPSAW  O[PO[e], k, l] += A[e, k] * B[e, l] * W[PW[e], l]
//
// Reference semantics restated here: mops/src/opsa/cpu.tpp:9-112 and
// mops/src/opsaw/cpu.tpp:9-131 of lab-cosmo/mops (formulas, optional
// gradients, rows without edges are zero). The reference's CUDA OPSA kernels
// (mops/src/opsa/opsa.cu:14-284) run first_occurrences as a separate launch
// and then one block per output row that reads A and B from global memory
// once per output element; OPSAW has no reference device code at all
// (mops/src/opsaw/opsaw.cu:1).
//
// Here the scatter index is sorted, so the edges of one output row are one
// contiguous segment, and per segment the operation is a small dense
// contraction over the edges:
//
//   forward   O[i]      = A_seg^T  (K x n) * B_seg (n x L)        (B_seg scaled by W rows for OPSAW)
//   vjp       grad_B_seg = A_seg   (n x K) * G[i]  (K x L)
//             grad_A_seg = B_seg   (n x L) * G[i]^T (L x K)
//
// Each segment is owned by one wavefront (segment_walk.hpp: found from the
// index itself inside the same kernel, no boundary table, no second launch),
// which runs the contraction on the matrix cores with 16x16x4 MFMA tiles in
// the element type of the data (mfma.hpp) and writes its rows once. Operands
// are loaded from global memory directly in the register layout the
// instruction wants: for A_seg^T that is 4 consecutive rows of A per load,
// i.e. one contiguous stretch of memory. No LDS, no atomics; the summation
// order is fixed (ascending edge number in steps of four), so results are
// bit-reproducible.
#include <algorithm>
#include <optional>
#include <cstdlib>
#include <memory>

#include "mops/opsa.hpp"
#include "mops/opsaw.hpp"

#include "checks.hpp"
#include "device_common.hpp"
#include "dispatch_thresholds.hpp"
#include "first_occurrences.hpp"
#include "index_validation.hpp"
#include "mfma.hpp"
#include "edge_order.hpp"
#include "elementwise.hpp"
#include "runtime.hpp"
#include "segment_walk.hpp"
#include "sender_buckets.hpp"
#include "sender_gather.hpp"

namespace mops::amd {
namespace opsa { // a name of its own for this file's kernels: profilers print it
namespace {

constexpr int CHUNK = 32;            // index positions per wavefront
constexpr int WAVES_PER_BLOCK = 4;   // independent wavefronts share a workgroup
constexpr int BLOCK = WAVES_PER_BLOCK * WAVE;

// ---------------------------------------------------------------------------
// forward, one segment: O_row[K, L] = sum_e A[e, :]^T (B[e, :] (* W[PW[e], :]))
// NT = number of 16-column tiles of L accumulated at once.
// MFMA roles: D rows = k, D columns = l, reduction = edges (4 per instruction)
// ---------------------------------------------------------------------------
// (byte offsets beyond 32 bits: addresses of 64 bits, a choice of address and of result per load)
template <typename T, int NT, bool WEIGHTED>
__device__ __forceinline__ void forward_segment_wide(
    T* __restrict__ out_row,
    const T* __restrict__ A,
    const T* __restrict__ B,
    const T* __restrict__ W,
    const int32_t* __restrict__ indices_W,
    int32_t n_weights,
    int32_t first,
    int32_t last,
    int32_t K,
    int32_t L
) {
    using M = Mfma<T>;
    constexpr int UNROLL = 8; // 32 edges in flight per iteration
    const int lane = threadIdx.x & (WAVE - 1);
    const int sub = lane & 15;
    const int quarter = lane >> 4;

    for (int32_t k0 = 0; k0 < K; k0 += 16) {
        const int32_t k = k0 + sub;
        const bool k_ok = k < K;
        for (int32_t l0 = 0; l0 < L; l0 += 16 * NT) {
            typename M::Acc acc[NT];
#pragma unroll
            for (int t = 0; t < NT; t++) {
                acc[t] = M::zero();
            }
            for (int32_t e0 = first; e0 < last; e0 += 4 * UNROLL) {
                T a[UNROLL];
                T b[UNROLL][NT];
                T w[WEIGHTED ? UNROLL : 1][NT];
                int32_t w_row[UNROLL];
                if (WEIGHTED) {
#pragma unroll
                    for (int u = 0; u < UNROLL; u++) {
                        const int32_t e = e0 + 4 * u + quarter;
                        const int32_t loaded = indices_W[e < last ? e : first];
                        w_row[u] = e < last ? loaded : -1;
                    }
                }
#pragma unroll
                for (int u = 0; u < UNROLL; u++) {
                    const int32_t e = e0 + 4 * u + quarter;
                    const bool e_ok = e < last;
                    a[u] = load_or_zero(A, static_cast<size_t>(e) * K + k, e_ok && k_ok);
#pragma unroll
                    for (int t = 0; t < NT; t++) {
                        const int32_t col = l0 + 16 * t + sub;
                        b[u][t] = load_or_zero(B, static_cast<size_t>(e) * L + col, e_ok && col < L);
                    }
                }
                if (WEIGHTED) {
#pragma unroll
                    for (int u = 0; u < UNROLL; u++) {
#pragma unroll
                        for (int t = 0; t < NT; t++) {
                            const int32_t col = l0 + 16 * t + sub;
                            w[u][t] = load_or_zero(
                                W,
                                static_cast<size_t>(w_row[u]) * L + col,
                                in_bounds(w_row[u], n_weights) && col < L
                            );
                        }
                    }
                    // every load is asked for before the first product needs one:
                    // left to itself the compiler chains them in the widest variant,
                    // each waiting for the one before (its own order is kept for the
                    // narrower ones, where it measured a little faster)
                    if (NT >= 4) {
                        __builtin_amdgcn_sched_barrier(0);
                    }
#pragma unroll
                    for (int u = 0; u < UNROLL; u++) {
#pragma unroll
                        for (int t = 0; t < NT; t++) {
                            b[u][t] *= w[u][t];
                        }
                    }
                }
                // keep every load above ahead of the first matrix instruction:
                // the loads of all 32 edges are meant to be in flight together
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < UNROLL; u++) {
#pragma unroll
                    for (int t = 0; t < NT; t++) {
                        acc[t] = M::mma(a[u], b[u][t], acc[t]);
                    }
                }
            }
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const int32_t col = l0 + 16 * t + sub;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int32_t row_k = k0 + M::row(lane, r);
                    if (row_k < K && col < L) {
                        out_row[static_cast<size_t>(row_k) * L + col] = acc[t][r];
                    }
                }
            }
        }
    }
}

/// A tensor as a buffer: a load is a uniform descriptor, a 32-bit byte offset
/// per lane and a uniform byte offset (the hardware adds the three), and an
/// offset beyond the tensor reads as zero without touching memory: a lane
/// that has nothing to load gets all ones OR-ed into its offset, which costs
/// one instruction where a choice of address and of result costs three.
template <typename T> struct RowBuffer {
    __amdgpu_buffer_rsrc_t descriptor;
    __device__ __forceinline__ explicit RowBuffer(const T* base) {
        descriptor = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<T*>(base), 0, static_cast<int>(0xfffffff0u), 0x00020000
        );
    }
    __device__ __forceinline__ T load(uint32_t lane_bytes, uint32_t uniform_bytes) const {
        if constexpr (sizeof(T) == 4) {
            return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b32(descriptor, lane_bytes, uniform_bytes, 0));
        } else {
            return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b64(descriptor, lane_bytes, uniform_bytes, 0));
        }
    }
    /// N consecutive elements (N = 2 or 4) by loads of 8 or 16 bytes.
    template <int N> __device__ __forceinline__ void load_vector(T (&to)[N], uint32_t lane_bytes, uint32_t uniform_bytes) const {
        static_assert(N == 2 || N == 4, "two or four elements");
        typedef uint32_t Two __attribute__((ext_vector_type(2)));
        if constexpr (sizeof(T) == 4 && N == 2) {
            const auto raw = __builtin_amdgcn_raw_buffer_load_b64(descriptor, lane_bytes, uniform_bytes, 0);
            to[0] = __builtin_bit_cast(T, static_cast<uint32_t>(raw[0]));
            to[1] = __builtin_bit_cast(T, static_cast<uint32_t>(raw[1]));
        } else if constexpr (sizeof(T) == 4) {
            const auto raw = __builtin_amdgcn_raw_buffer_load_b128(descriptor, lane_bytes, uniform_bytes, 0);
#pragma unroll
            for (int v = 0; v < 4; v++) {
                to[v] = __builtin_bit_cast(T, static_cast<uint32_t>(raw[v]));
            }
        } else {
#pragma unroll
            for (int half = 0; half < N / 2; half++) {
                // (the second half through the uniform offset: the lane's may be all ones)
                const auto raw = __builtin_amdgcn_raw_buffer_load_b128(descriptor, lane_bytes, uniform_bytes + 16 * half, 0);
                to[2 * half] = __builtin_bit_cast(T, Two{raw[0], raw[1]});
                to[2 * half + 1] = __builtin_bit_cast(T, Two{raw[2], raw[3]});
            }
        }
    }
};
/// N consecutive elements to memory by stores of 8 or 16 bytes (`to` aligned to them).
template <typename T, int N> __device__ __forceinline__ void store_vector(T* to, const T (&from)[N]) {
    static_assert(N == 2 || N == 4, "two or four elements");
    if constexpr (sizeof(T) == 4 && N == 2) {
        typedef T Pair __attribute__((ext_vector_type(2)));
        *reinterpret_cast<Pair*>(to) = Pair{from[0], from[1]};
    } else if constexpr (sizeof(T) == 4) {
        typedef T Four __attribute__((ext_vector_type(4)));
        *reinterpret_cast<Four*>(to) = Four{from[0], from[1], from[2], from[3]};
    } else {
        typedef T Pair __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int half = 0; half < N / 2; half++) {
            reinterpret_cast<Pair*>(to)[half] = Pair{from[2 * half], from[2 * half + 1]};
        }
    }
}
/// All ones unless `wanted`.
__device__ __forceinline__ uint32_t unless(bool wanted) { return static_cast<uint32_t>(wanted) - 1u; }

/// PAIRS = 2: the sum over the edges of A (x) B and of A2 (x) B2 in the same accumulators
/// (NARROW only).
/// PACKED (NARROW, NT = 2 or 4, L a multiple of NT, B, W and the output aligned to NT elements):
/// a lane holds NT CONSECUTIVE columns of a block of 16 NT (tile t of lane `sub` is column
/// NT sub + t, not 16 t + sub), so that a row of B or W is one load of NT elements per lane and
/// a row of the output one store, not NT of each: the kernel is bound by the number of its
/// load instructions (half of them were loads of B), and which column a tile's lane stands
/// for is free.
template <typename T, int NT, bool WEIGHTED, bool NARROW, int PAIRS = 1, bool PACKED = false>
__device__ __forceinline__ void forward_segment(
    T* __restrict__ out_row,
    const T* __restrict__ A,
    const T* __restrict__ B,
    const T* __restrict__ W,
    const int32_t* __restrict__ indices_W,
    int32_t n_weights,
    int32_t first,
    int32_t last,
    int32_t K,
    int32_t L,
    const T* __restrict__ A2 = nullptr,
    const T* __restrict__ B2 = nullptr
) {
    static_assert(PAIRS == 1 || NARROW, "two pairs: offsets of 32 bits only");
    static_assert(!PACKED || (NARROW && NT > 1), "packed columns: offsets of 32 bits, more than one tile");
    if constexpr (!NARROW) {
        forward_segment_wide<T, NT, WEIGHTED>(out_row, A, B, W, indices_W, n_weights, first, last, K, L);
        return;
    }
    using M = Mfma<T>;
    constexpr int UNROLL = 8; // 32 edges in flight per iteration
    constexpr uint32_t ES = sizeof(T);
    const int lane = threadIdx.x & (WAVE - 1);
    const int sub = lane & 15;
    const int quarter = lane >> 4;
    const RowBuffer<T> rows_W(W);
    const RowBuffer<T> pair_A[2] = {RowBuffer<T>(A), RowBuffer<T>(PAIRS > 1 ? A2 : A)};
    const RowBuffer<T> pair_B[2] = {RowBuffer<T>(B), RowBuffer<T>(PAIRS > 1 ? B2 : B)};
    const RowBuffer<int32_t> rows_of_W(indices_W);
    const uint32_t a_row_bytes = static_cast<uint32_t>(K) * ES;
    const uint32_t b_row_bytes = static_cast<uint32_t>(L) * ES;

    for (int32_t k0 = 0; k0 < K; k0 += 16) {
        const int32_t k = k0 + sub;
        const uint32_t a_lane = (static_cast<uint32_t>(quarter) * a_row_bytes + static_cast<uint32_t>(k) * ES) | unless(k < K);
        for (int32_t l0 = 0; l0 < L; l0 += 16 * NT) {
            uint32_t b_lane[NT], w_column[NT], no_column[NT];
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const int32_t col = PACKED ? l0 + NT * sub + t : l0 + 16 * t + sub;
                no_column[t] = unless(col < L);
                w_column[t] = static_cast<uint32_t>(col) * ES;
                b_lane[t] = (static_cast<uint32_t>(quarter) * b_row_bytes + w_column[t]) | no_column[t];
            }
            // (PACKED: the lane's NT columns are all inside a row or all outside: index 0 stands for them)
            typename M::Acc acc[NT];
#pragma unroll
            for (int t = 0; t < NT; t++) {
                acc[t] = M::zero();
            }
#pragma unroll
            for (int pair = 0; pair < PAIRS; pair++) {
            const RowBuffer<T>& rows_A = pair_A[pair];
            const RowBuffer<T>& rows_B = pair_B[pair];
            for (int32_t e0 = first; e0 < last; e0 += 4 * UNROLL) {
                T a[UNROLL];
                T b[UNROLL][NT];
                T w[WEIGHTED ? UNROLL : 1][NT];
                uint32_t beyond[UNROLL]; // all ones for a lane whose edge is not of this segment
                int32_t w_row[UNROLL];
#pragma unroll
                for (int u = 0; u < UNROLL; u++) {
                    beyond[u] = unless(e0 + 4 * u + quarter < last);
                    if (WEIGHTED) {
                        w_row[u] = rows_of_W.load(static_cast<uint32_t>(quarter) * 4u | beyond[u], static_cast<uint32_t>(e0 + 4 * u) * 4u);
                    }
                }
#pragma unroll
                for (int u = 0; u < UNROLL; u++) {
                    const uint32_t row = static_cast<uint32_t>(e0 + 4 * u); // (uniform)
                    a[u] = rows_A.load(a_lane | beyond[u], row * a_row_bytes);
                    if constexpr (PACKED) {
                        rows_B.template load_vector<NT>(b[u], b_lane[0] | beyond[u], row * b_row_bytes);
                    } else {
#pragma unroll
                        for (int t = 0; t < NT; t++) {
                            b[u][t] = rows_B.load(b_lane[t] | beyond[u], row * b_row_bytes);
                        }
                    }
                }
                if (WEIGHTED) {
#pragma unroll
                    for (int u = 0; u < UNROLL; u++) {
                        const uint32_t from = static_cast<uint32_t>(w_row[u]) * b_row_bytes;
                        const uint32_t nothing = unless(in_bounds(w_row[u], n_weights)) | beyond[u];
                        if constexpr (PACKED) {
                            rows_W.template load_vector<NT>(w[u], (from + w_column[0]) | nothing | no_column[0], 0);
                        } else {
#pragma unroll
                            for (int t = 0; t < NT; t++) {
                                w[u][t] = rows_W.load((from + w_column[t]) | nothing | no_column[t], 0);
                            }
                        }
                    }
                    if (NT >= 4) {
                        __builtin_amdgcn_sched_barrier(0);
                    }
#pragma unroll
                    for (int u = 0; u < UNROLL; u++) {
#pragma unroll
                        for (int t = 0; t < NT; t++) {
                            b[u][t] *= w[u][t];
                        }
                    }
                }
                // keep every load above ahead of the first matrix instruction:
                // the loads of all 32 edges are meant to be in flight together
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < UNROLL; u++) {
#pragma unroll
                    for (int t = 0; t < NT; t++) {
                        acc[t] = M::mma(a[u], b[u][t], acc[t]);
                    }
                }
            }
            }
            if constexpr (PACKED) {
                const int32_t col = l0 + NT * sub;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int32_t row_k = k0 + M::row(lane, r);
                    if (row_k < K && col < L) {
                        T values[NT];
#pragma unroll
                        for (int t = 0; t < NT; t++) {
                            values[t] = acc[t][r];
                        }
                        store_vector<T, NT>(out_row + static_cast<size_t>(row_k) * L + col, values);
                    }
                }
            } else {
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    const int32_t col = l0 + 16 * t + sub;
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const int32_t row_k = k0 + M::row(lane, r);
                        if (row_k < K && col < L) {
                            out_row[static_cast<size_t>(row_k) * L + col] = acc[t][r];
                        }
                    }
                }
            }
        }
    }
}

/// NARROW: every tensor is smaller than 4 GB, byte offsets of 32 bits (see RowBuffer).
template <typename T, int NT, bool WEIGHTED, bool NARROW, bool PACKED = false>
__global__ __launch_bounds__(BLOCK) void forward_kernel(
    T* __restrict__ output,
    const T* __restrict__ A,
    const T* __restrict__ B,
    const T* __restrict__ W,
    const int32_t* __restrict__ indices_W,
    const int32_t* __restrict__ indices_output,
    int32_t n_edges,
    int32_t n_output,
    int32_t K,
    int32_t L
) {
    const int32_t wave_index =
        __builtin_amdgcn_readfirstlane(blockIdx.x * WAVES_PER_BLOCK + (threadIdx.x >> 6));
    const int lane = threadIdx.x & (WAVE - 1);
    const size_t row_elements = static_cast<size_t>(K) * L;
    walk_owned_segments<CHUNK>(
        indices_output,
        n_edges,
        n_output,
        wave_index,
        [&](int32_t row, int32_t first, int32_t last) {
            forward_segment<T, NT, WEIGHTED, NARROW, 1, PACKED>(
                output + row * row_elements, A, B, W, indices_W, n_output, first, last, K, L
            );
        },
        [&](int32_t begin, int32_t end) {
            T* base = output + begin * row_elements;
            const size_t count = (end - begin) * row_elements;
            for (size_t i = lane; i < count; i += WAVE) {
                base[i] = T(0);
            }
        }
    );
}

/// output = opsa(A, B) + opsa(A2, B2) in one launch: what the second-order function needs
/// (the forward with grad_grad_A for A plus the forward with grad_grad_B for B).
template <typename T, int NT>
__global__ __launch_bounds__(BLOCK) void forward_two_pairs_kernel(
    T* __restrict__ output,
    const T* __restrict__ A,
    const T* __restrict__ B,
    const T* __restrict__ A2,
    const T* __restrict__ B2,
    const int32_t* __restrict__ indices_output,
    int32_t n_edges,
    int32_t n_output,
    int32_t K,
    int32_t L
) {
    const int32_t wave_index =
        __builtin_amdgcn_readfirstlane(blockIdx.x * WAVES_PER_BLOCK + (threadIdx.x >> 6));
    const int lane = threadIdx.x & (WAVE - 1);
    const size_t row_elements = static_cast<size_t>(K) * L;
    walk_owned_segments<CHUNK>(
        indices_output,
        n_edges,
        n_output,
        wave_index,
        [&](int32_t row, int32_t first, int32_t last) {
            forward_segment<T, NT, false, true, 2>(
                output + row * row_elements, A, B, nullptr, nullptr, n_output, first, last, K, L, A2, B2
            );
        },
        [&](int32_t begin, int32_t end) {
            T* base = output + begin * row_elements;
            const size_t count = (end - begin) * row_elements;
            for (size_t i = lane; i < count; i += WAVE) {
                base[i] = T(0);
            }
        }
    );
}

// ---------------------------------------------------------------------------
// forward for LONG segments (pooling over whole structures: a few output rows,
// thousands of edges each). One wavefront per segment would leave the device
// idle, so segments are cut every SPLIT positions (segment_walk.hpp); a piece
// that is a whole segment goes to its output row as above, the others to
//   tail[b]  the piece that begins its segment inside block b and leaves it
//   head[b]  the piece that entered block b from the block before
// (at most one of each per block of SPLIT positions), and
// combine_pieces_kernel adds tail[b] + head[b + 1] + head[b + 2] + ... in that
// order for every cut segment: no atomics, one fixed order.
// ---------------------------------------------------------------------------
constexpr int SPLIT = thresholds::OPSA_SPLIT_POSITIONS;

template <typename T, int NT, bool WEIGHTED, bool NARROW>
__global__ __launch_bounds__(BLOCK) void forward_split_kernel(
    T* __restrict__ output,
    T* __restrict__ tails,
    T* __restrict__ heads,
    const T* __restrict__ A,
    const T* __restrict__ B,
    const T* __restrict__ W,
    const int32_t* __restrict__ indices_W,
    const int32_t* __restrict__ indices_output,
    int32_t n_edges,
    int32_t n_output,
    int32_t K,
    int32_t L
) {
    const int32_t wave_index =
        __builtin_amdgcn_readfirstlane(blockIdx.x * WAVES_PER_BLOCK + (threadIdx.x >> 6));
    const int lane = threadIdx.x & (WAVE - 1);
    const size_t row_elements = static_cast<size_t>(K) * L;
    walk_split_segments<CHUNK, SPLIT>(
        indices_output,
        n_edges,
        n_output,
        wave_index,
        [&](int32_t row, int32_t first, int32_t last, bool from_start, bool to_end) {
            const int32_t block = first / SPLIT;
            T* target = from_start && to_end ? output + row * row_elements
                        : from_start         ? tails + block * row_elements
                                             : heads + block * row_elements;
            forward_segment<T, NT, WEIGHTED, NARROW>(target, A, B, W, indices_W, n_output, first, last, K, L);
        },
        [&](int32_t begin, int32_t end) {
            T* base = output + begin * row_elements;
            const size_t count = (end - begin) * row_elements;
            for (size_t i = lane; i < count; i += WAVE) {
                base[i] = T(0);
            }
        }
    );
}

constexpr int COMBINE_THREADS = 256;

/// Workgroup b: if a segment begins in block b of SPLIT positions and goes on
/// into block b + 1, its output row = tail[b] + head[b + 1] + ... (all its pieces).
template <typename T>
__global__ __launch_bounds__(COMBINE_THREADS) void combine_pieces_kernel(
    T* __restrict__ output,
    const T* __restrict__ tails,
    const T* __restrict__ heads,
    const int32_t* __restrict__ indices_output,
    int32_t n_edges,
    int32_t n_output,
    int32_t row_elements
) {
    const int32_t block = blockIdx.x;
    const int32_t cut = (block + 1) * SPLIT; // first position of the next block
    if (cut >= n_edges) {
        return;
    }
    const int32_t row = indices_output[cut];
    if (indices_output[cut - 1] != row || !in_bounds(row, n_output)) {
        return; // nothing crosses this cut
    }
    if (block > 0 && indices_output[block * SPLIT - 1] == row) {
        return; // the segment began before this block: another workgroup adds it up
    }
    // blocks block + 1 .. last_block hold head pieces of this row
    int32_t last_block = block + 1;
    while ((last_block + 1) * SPLIT < n_edges && indices_output[(last_block + 1) * SPLIT] == row) {
        last_block++;
    }
    constexpr int AHEAD = 8;
    for (int32_t element = threadIdx.x; element < row_elements; element += COMBINE_THREADS) {
        T sum = tails[static_cast<size_t>(block) * row_elements + element];
        for (int32_t b0 = block + 1; b0 <= last_block; b0 += AHEAD) {
            T piece[AHEAD];
#pragma unroll
            for (int u = 0; u < AHEAD; u++) {
                const int32_t b = min(b0 + u, last_block);
                piece[u] = heads[static_cast<size_t>(b) * row_elements + element];
            }
#pragma unroll
            for (int u = 0; u < AHEAD; u++) {
                if (b0 + u <= last_block) {
                    sum += piece[u];
                }
            }
        }
        output[static_cast<size_t>(row) * row_elements + element] = sum;
    }
}

// every element of `data` := 0 (used when there is no edge at all)
template <typename T>
__global__ __launch_bounds__(256) void zero_kernel(T* __restrict__ data, size_t count) {
    for (size_t i = blockIdx.x * static_cast<size_t>(256) + threadIdx.x; i < count;
         i += static_cast<size_t>(gridDim.x) * 256) {
        data[i] = T(0);
    }
}

// ---------------------------------------------------------------------------
// vjp. One wavefront per workgroup; per segment, in stages of up to 32 edges:
//
//   S      = A_stage (n x K) * G (K x L)      -> grad_B = S (* W rows), edge_W = S * B
//   grad_A = BW_stage (n x L) * G^T (L x K)   with BW = B (* W rows)
//
// MFMA roles: D rows = edges (16 per tile), D columns = l (or k), reduction =
// k (or l). G (the segment's grad_output row) and the stage's rows of A, B
// (and the gathered W rows) are first copied to LDS with row-contiguous loads
// that are all in flight together, then fed to the matrix cores from LDS.
// LDS rows have an odd stride so that the column walks of the operand reads
// (stride = one row) spread over the banks. `shift_K` / `shift_L` are
// log2 of the row widths rounded up to a power of two: a wavefront copies
// 64 >> shift rows per load instruction, lane = (row, column) without any
// integer division.
// ---------------------------------------------------------------------------
constexpr int STAGE_EDGES = 32;

// A batch of up to U row-passes held in registers between the global loads
// and the LDS stores, so that the loads of several batches (G, A and B) are
// all issued before the first one is waited for.
template <typename T, int U> struct RowBatch {
    T value[U];
    int32_t lds_offset[U]; // -1: nothing to store

    /// Issue the loads of passes [pass0, pass0 + U) of a [n_rows, width] block.
    __device__ __forceinline__ void load(
        const T* __restrict__ source,
        int32_t stage_stride,
        int32_t n_rows,
        int32_t width,
        int32_t shift,
        int32_t pass0
    ) {
        const int lane = threadIdx.x & (WAVE - 1);
        const int32_t column = lane & ((1 << shift) - 1);
        const int32_t row_in_pass = lane >> shift;
        const int32_t rows_per_pass = WAVE >> shift;
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int32_t row = (pass0 + u) * rows_per_pass + row_in_pass;
            const bool ok = row < n_rows && column < width;
            value[u] = load_or_zero(source, static_cast<size_t>(row) * width + column, ok);
            lds_offset[u] = ok ? row * stage_stride + column : -1;
        }
    }

    __device__ __forceinline__ void store(T* __restrict__ stage) const {
#pragma unroll
        for (int u = 0; u < U; u++) {
            if (lds_offset[u] >= 0) {
                stage[lds_offset[u]] = value[u];
            }
        }
    }
};

// The same for rows gathered through an index (the weight rows of OPSAW):
// first all index loads, then all row loads, then the LDS stores.
template <typename T, int U> struct GatherBatch {
    T value[U];
    int32_t lds_offset[U];

    __device__ __forceinline__ void load(
        const T* __restrict__ table,
        const int32_t* __restrict__ row_index,
        int32_t table_rows,
        int32_t stage_stride,
        int32_t n_rows,
        int32_t width,
        int32_t shift,
        int32_t pass0
    ) {
        const int lane = threadIdx.x & (WAVE - 1);
        const int32_t column = lane & ((1 << shift) - 1);
        const int32_t row_in_pass = lane >> shift;
        const int32_t rows_per_pass = WAVE >> shift;
        int32_t source_row[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int32_t row = (pass0 + u) * rows_per_pass + row_in_pass;
            const bool ok = row < n_rows && column < width;
            const int32_t loaded = row_index[ok ? row : 0];
            source_row[u] = ok ? loaded : -1;
            lds_offset[u] = ok ? row * stage_stride + column : -1;
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            value[u] = load_or_zero(
                table,
                static_cast<size_t>(source_row[u]) * width + column,
                in_bounds(source_row[u], table_rows)
            );
        }
    }

    __device__ __forceinline__ void store(T* __restrict__ stage) const {
#pragma unroll
        for (int u = 0; u < U; u++) {
            if (lds_offset[u] >= 0) {
                stage[lds_offset[u]] = value[u];
            }
        }
    }
};

// Rows wider than a wavefront (shift > 6): plain loop, one row at a time.
template <typename T>
__device__ __forceinline__ void copy_wide_rows_to_lds(
    T* __restrict__ stage, int32_t stage_stride, const T* __restrict__ source, int32_t n_rows, int32_t width
) {
    const int lane = threadIdx.x & (WAVE - 1);
    for (int32_t row = 0; row < n_rows; row++) {
        for (int32_t c = lane; c < width; c += WAVE) {
            stage[row * stage_stride + c] = source[static_cast<size_t>(row) * width + c];
        }
    }
}

// Passes needed to copy n_rows rows when 64 >> shift rows go per pass.
__device__ __forceinline__ int32_t passes_for(int32_t n_rows, int32_t shift) {
    const int32_t rows_per_pass = WAVE >> shift;
    return (n_rows + rows_per_pass - 1) / rows_per_pass; // shift <= 6 here, no division by zero
}

template <typename T, bool WEIGHTED>
__global__ __launch_bounds__(WAVE) void vjp_kernel(
    T* __restrict__ grad_A,
    T* __restrict__ grad_B,
    T* __restrict__ edge_W,
    const T* __restrict__ grad_output,
    const T* __restrict__ A,
    const T* __restrict__ B,
    const T* __restrict__ W,
    const int32_t* __restrict__ indices_W,
    const int32_t* __restrict__ indices_output,
    int32_t n_edges,
    int32_t n_output,
    int32_t K,
    int32_t L,
    int32_t shift_K,
    int32_t shift_L
) {
    using M = Mfma<T>;
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    const int32_t Ks = odd_stride(K);
    const int32_t Ls = odd_stride(L);
    T* g_stage = reinterpret_cast<T*>(lds_bytes);        // [K][Ls]
    T* a_stage = g_stage + K * Ls;                        // [STAGE_EDGES][Ks]
    T* b_stage = a_stage + STAGE_EDGES * Ks;              // [STAGE_EDGES][Ls]  B
    T* w_stage = b_stage + STAGE_EDGES * Ls;              // [STAGE_EDGES][Ls]  W rows (weighted)

    const int lane = threadIdx.x;
    const int sub = lane & 15;
    const int quarter = lane >> 4;
    const size_t row_elements = static_cast<size_t>(K) * L;
    const bool want_S = grad_B != nullptr || (WEIGHTED && edge_W != nullptr);

    walk_owned_segments<CHUNK>(
        indices_output,
        n_edges,
        n_output,
        static_cast<int32_t>(blockIdx.x),
        [&](int32_t row, int32_t first, int32_t last) {
            constexpr int U = 8;
            const bool narrow = shift_K <= 6 && shift_L <= 6;
            const T* g_source = grad_output + row * row_elements;
            __syncthreads(); // the previous segment's LDS reads are done

            for (int32_t s0 = first; s0 < last; s0 += STAGE_EDGES) {
                const int32_t n = min(STAGE_EDGES, last - s0);
                const T* a_source = A + static_cast<size_t>(s0) * K;
                const T* b_source = B + static_cast<size_t>(s0) * L;
                if (s0 != first) {
                    __syncthreads();
                }
                if (narrow) {
                    // first batches of G, A and B: all loads in flight together
                    RowBatch<T, U> g_batch, a_batch;
                    RowBatch<T, 2 * U> b_batch;
                    const bool with_g = s0 == first;
                    if (with_g) {
                        g_batch.load(g_source, Ls, K, L, shift_L, 0);
                    }
                    a_batch.load(a_source, Ks, n, K, shift_K, 0);
                    b_batch.load(b_source, Ls, n, L, shift_L, 0);
                    if (with_g) {
                        g_batch.store(g_stage);
                    }
                    a_batch.store(a_stage);
                    b_batch.store(b_stage);
                    // whatever does not fit the first batch
                    if (with_g) {
                        for (int32_t pass = U; pass < passes_for(K, shift_L); pass += U) {
                            g_batch.load(g_source, Ls, K, L, shift_L, pass);
                            g_batch.store(g_stage);
                        }
                    }
                    for (int32_t pass = U; pass < passes_for(n, shift_K); pass += U) {
                        a_batch.load(a_source, Ks, n, K, shift_K, pass);
                        a_batch.store(a_stage);
                    }
                    for (int32_t pass = 2 * U; pass < passes_for(n, shift_L); pass += 2 * U) {
                        b_batch.load(b_source, Ls, n, L, shift_L, pass);
                        b_batch.store(b_stage);
                    }
                } else {
                    if (s0 == first) {
                        copy_wide_rows_to_lds(g_stage, Ls, g_source, K, L);
                    }
                    copy_wide_rows_to_lds(a_stage, Ks, a_source, n, K);
                    copy_wide_rows_to_lds(b_stage, Ls, b_source, n, L);
                }
                if (WEIGHTED) {
                    if (narrow) {
                        GatherBatch<T, 2 * U> w_batch;
                        for (int32_t pass = 0; pass < passes_for(n, shift_L); pass += 2 * U) {
                            w_batch.load(W, indices_W + s0, n_output, Ls, n, L, shift_L, pass);
                            w_batch.store(w_stage);
                        }
                    } else {
                        for (int32_t r = 0; r < n; r++) {
                            const int32_t w_row = indices_W[s0 + r];
                            const bool ok = in_bounds(w_row, n_output);
                            for (int32_t c = lane; c < L; c += WAVE) {
                                w_stage[r * Ls + c] =
                                    ok ? W[static_cast<size_t>(w_row) * L + c] : T(0);
                            }
                        }
                    }
                }
                __syncthreads();

                for (int32_t t0 = 0; t0 < n; t0 += 16) {
                    const int32_t local = t0 + sub;       // operand row = edge within the stage
                    const bool edge_ok = local < n;

                    if (want_S) {
                        for (int32_t l0 = 0; l0 < L; l0 += 16) {
                            const int32_t col = l0 + sub;
                            typename M::Acc acc = M::zero();
#pragma unroll 4
                            for (int32_t kk = 0; kk < K; kk += 4) {
                                const int32_t k = kk + quarter;
                                const bool k_ok = k < K;
                                const T a = load_or_zero(a_stage, local * Ks + k, edge_ok && k_ok);
                                const T g = load_or_zero(g_stage, k * Ls + col, k_ok && col < L);
                                acc = M::mma(a, g, acc);
                            }
#pragma unroll
                            for (int r = 0; r < 4; r++) {
                                const int32_t e_local = t0 + M::row(lane, r);
                                if (e_local < n && col < L) {
                                    const size_t at = static_cast<size_t>(s0 + e_local) * L + col;
                                    if (WEIGHTED) {
                                        if (grad_B != nullptr) {
                                            grad_B[at] = acc[r] * w_stage[e_local * Ls + col];
                                        }
                                        if (edge_W != nullptr) {
                                            edge_W[at] = acc[r] * b_stage[e_local * Ls + col];
                                        }
                                    } else {
                                        grad_B[at] = acc[r];
                                    }
                                }
                            }
                        }
                    }

                    if (grad_A != nullptr) {
                        for (int32_t k0 = 0; k0 < K; k0 += 16) {
                            const int32_t kcol = k0 + sub;
                            typename M::Acc acc = M::zero();
#pragma unroll 4
                            for (int32_t ll = 0; ll < L; ll += 4) {
                                const int32_t l = ll + quarter;
                                const bool l_ok = l < L;
                                T b = load_or_zero(b_stage, local * Ls + l, edge_ok && l_ok);
                                if (WEIGHTED) {
                                    b *= load_or_zero(w_stage, local * Ls + l, edge_ok && l_ok);
                                }
                                const T g = load_or_zero(g_stage, kcol * Ls + l, kcol < K && l_ok);
                                acc = M::mma(b, g, acc);
                            }
#pragma unroll
                            for (int r = 0; r < 4; r++) {
                                const int32_t e_local = t0 + M::row(lane, r);
                                if (e_local < n && kcol < K) {
                                    grad_A[static_cast<size_t>(s0 + e_local) * K + kcol] = acc[r];
                                }
                            }
                        }
                    }
                }
            }
        },
        [](int32_t, int32_t) {}
    );
}

// An edge whose scatter index lies outside [0, n_output) belongs to no output
// row: its rows of grad_A / grad_B are then left unwritten (such input is
// invalid; the reference's device path does not define it either). Nothing is
// ever read or written out of bounds because of it.

// ---------------------------------------------------------------------------
// grad_W[w, l] = sum over edges e with PW[e] == w of edge_W[e, l]
// grid: one workgroup per weight row; edges in ascending order.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void gather_weights_kernel(
    T* __restrict__ grad_W, const T* __restrict__ edge_W, SenderBuckets buckets, int32_t L
) {
    __shared__ int32_t bucket_lds[BUCKET_LDS_CAPACITY];
    const int32_t node = blockIdx.x;
    SortedBucket bucket = sorted_bucket(buckets, node, bucket_lds);
    for (int32_t l = threadIdx.x; l < L; l += blockDim.x) {
        T sum = 0;
        for (int32_t i = 0; i < bucket.count; i++) {
            sum += edge_W[static_cast<size_t>(bucket.edges[i]) * L + l];
        }
        grad_W[static_cast<size_t>(node) * L + l] = sum;
    }
}

// ---------------------------------------------------------------------------
// vjp for K <= 32 (any L; beyond 64 columns in passes of 64, see BLOCKS), which
// includes the shapes of the reference's benchmarks: the gradients are per EDGE, so nothing has to follow
// the segments. A wavefront takes 16 consecutive edges, whatever receivers
// they have: it knows which rows of A, B (and W) it needs before it has seen
// any index, all its loads go straight from global memory into matrix
// operands (no LDS), and for every receiver among its edges it multiplies the
// rows of that receiver (the others zeroed) with the receiver's grad_output:
//
//   grad_A[e, k] = sum_l (B * W)[e, l] * gO[node, k, l]     16 x L times L x K
//   grad_B[e, l] = sum_k A[e, k] * gO[node, k, l] (* W)     16 x K times K x L
//
// Rows of the result belong to one edge each, so the products for different
// receivers add up in the same accumulators. Two dependent round trips to
// memory (index, then grad_output), every wavefront the same amount of work.
// ---------------------------------------------------------------------------
//
// VECTORS: the rows of B, W and grad_output are read 16 bytes at a time (L a
// multiple of the vector length, pointers aligned). A lane's vector then holds
// VL consecutive l, so the reduction over l is taken in a different ORDER than
// l = 4 s + q: vector v, component c is step s = VL v + c and stands for
// l = 4 VL v + VL q + c, in the left and in the right operand alike. One
// 16-byte load per lane replaces VL loads that each touch 16 cache lines,
// which is what these kernels otherwise spend their time on (address
// processing, not bandwidth).
//
// LISTS: workgroups are four wavefronts (four groups of 16 edges, independent
// of each other), and the first `list_blocks` workgroups do something else:
// they list the edges of every sender in its slots (sender_buckets.hpp), which
// the sum of the per-edge rows of grad_W needs afterwards. That pass over the
// sender index has no launch of its own then and no time of its own: it runs
// beside the wavefronts that wait for their rows.
constexpr int LISTING_WAVES = 2;

template <typename T, int KT, int NT, bool WEIGHTED, bool VECTORS, bool BLOCKS, bool LISTS>
// (LISTS: at most three wavefronts per SIMD. The workgroups that list run beside the ones that
// work on edges, and more of the latter at a time make the launch longer, not shorter: OPSAW
// vjp, 60 000 edges over 2000 nodes, with 5 / 4 / 3 / 2 wavefronts per SIMD 23.5 / 22.4 / 21.8 /
// 25.7 us. Without the listing workgroups the kernel wants all it can get: 1M edges, 82 us
// uncapped, 102 with four, 120 with three.)
__global__ __launch_bounds__((LISTS ? LISTING_WAVES : 1) * WAVE)
__attribute__((amdgpu_waves_per_eu(1, LISTS ? 3 : 8))) void edge_rows_vjp_kernel(
    T* __restrict__ grad_A,
    T* __restrict__ grad_B,
    T* __restrict__ edge_W,
    const T* __restrict__ grad_output,
    const T* __restrict__ A,
    const T* __restrict__ B,
    const T* __restrict__ W,
    const int32_t* __restrict__ indices_W,
    const int32_t* __restrict__ indices_output,
    int32_t n_edges,
    int32_t n_output,
    int32_t K,
    int32_t L,
    int32_t* __restrict__ slots,
    int32_t* __restrict__ slot_counts,
    int32_t list_blocks,
    bool aligned_senders
) {
    using M = Mfma<T>;
    constexpr int K_STEPS = 4 * KT;
    constexpr int L_STEPS = 4 * NT;
    constexpr int WAVES = LISTS ? LISTING_WAVES : 1;
    if constexpr (LISTS) {
        if (static_cast<int32_t>(blockIdx.x) < list_blocks) {
            __shared__ SlotLists lists;
            list_in_slots_block<WAVES * WAVE>(
                lists, slots, slot_counts, indices_W, n_edges, n_output, aligned_senders, blockIdx.x
            );
            return;
        }
    }
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = LISTS ? threadIdx.x >> 6 : 0;
    const int i = lane & 15;
    const int q = lane >> 4;
    const int32_t first_edge =
        (LISTS ? (static_cast<int32_t>(blockIdx.x) - list_blocks) * WAVES + wave : static_cast<int32_t>(blockIdx.x)) * 16;
    if (LISTS && first_edge >= n_edges) {
        return; // (the wavefronts of a workgroup never wait for each other)
    }
    const int32_t n = min(16, n_edges - first_edge);
    const int32_t my_edge = i < n ? first_edge + i : -1;
    const bool want_A = grad_A != nullptr;
    const bool want_B = grad_B != nullptr;
    const bool want_W = WEIGHTED && edge_W != nullptr;

    const int32_t my_node = my_edge >= 0 ? indices_output[my_edge] : -1;
    int32_t my_sender = 0;
    if constexpr (WEIGHTED) {
        my_sender = my_edge >= 0 ? indices_W[my_edge] : -1;
        if constexpr (!LISTS) {
            // large sparse graphs: every edge takes the next of its sender's places
            // (sender_buckets.hpp: SenderArrivals; `slots` is null when nobody wants the lists)
            if (slots != nullptr && q == 0 && my_edge >= 0) {
                list_arrival(SenderArrivals{slots, slot_counts, 1}, n_output, my_sender, my_edge);
            }
        }
    }
    const bool sender_ok = !WEIGHTED || in_bounds(my_sender, n_output);

    constexpr int VL = 16 / sizeof(T); // elements of a 16-byte vector
    typedef T Wide __attribute__((ext_vector_type(VL)));
    constexpr int L_VECTORS = L_STEPS / VL;
    // VECTORS also decides which columns the accumulators of grad_B stand for: tile t of lane i
    // is column 16 t + i otherwise, and with VECTORS the tiles come in groups of PW whose lanes
    // hold PW CONSECUTIVE columns (group g, lane i: columns 16 PW g + PW i ...), so that the
    // rows of grad_output, W and B that meet these accumulators are read, and grad_B and the
    // per-edge rows of grad_W written, PW columns per instruction: the matrix instruction does
    // not care which column a lane stands for, and the kernel pays per instruction.
    constexpr int PW = VECTORS ? (NT < VL ? NT : VL) : 1;
    // the NT values of a row at this lane's columns (`row_start`: index of the row's column l_base)
    auto load_columns = [&](T (&to)[NT], const T* base, size_t row_start, int32_t l_base, bool row_ok) {
        if constexpr (PW > 1) {
            typedef T Columns __attribute__((ext_vector_type(PW)));
#pragma unroll
            for (int g = 0; g < NT / PW; g++) {
                const int32_t l = 16 * PW * g + PW * i;
                const bool ok = row_ok && l_base + l < L;
                const Columns values = *reinterpret_cast<const Columns*>(base + (ok ? row_start + l : 0));
#pragma unroll
                for (int c = 0; c < PW; c++) {
                    to[PW * g + c] = ok ? values[c] : T(0);
                }
            }
        } else {
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const int32_t l = 16 * t + i;
                to[t] = load_or_zero(base, row_start + l, row_ok && l_base + l < L);
            }
        }
    };
    auto store_columns = [&](T* base, size_t row_start, int32_t l_base, const T (&from)[NT]) {
        if constexpr (PW > 1) {
            typedef T Columns __attribute__((ext_vector_type(PW)));
#pragma unroll
            for (int g = 0; g < NT / PW; g++) {
                const int32_t l = 16 * PW * g + PW * i;
                if (l_base + l < L) {
                    Columns values;
#pragma unroll
                    for (int c = 0; c < PW; c++) {
                        values[c] = from[PW * g + c];
                    }
                    *reinterpret_cast<Columns*>(base + row_start + l) = values;
                }
            }
        } else {
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const int32_t l = 16 * t + i;
                if (l_base + l < L) {
                    base[row_start + l] = from[t];
                }
            }
        }
    };
    auto wide_or_zero = [](const T* pointer, size_t index, bool ok) {
        const Wide value = *reinterpret_cast<const Wide*>(pointer + (ok ? index : 0));
        Wide zero;
#pragma unroll
        for (int c = 0; c < VL; c++) {
            zero[c] = T(0);
        }
        return ok ? value : zero;
    };
    // left operands: lane (row = edge i, reduction index 4 s + q; with VECTORS see above)
    // BLOCKS: L is wider than the 16 NT columns of one pass; the passes follow each
    // other, grad_A collects over all of them, the columns of grad_B are per pass
    T b_left[L_STEPS]; // (B * W)[e, l]
    T a_left[K_STEPS]; // A[e, k]
    auto load_b_left = [&](int32_t l_base) {
    if constexpr (VECTORS) {
#pragma unroll
        for (int v = 0; v < L_VECTORS; v++) {
            const int32_t l = l_base + 4 * VL * v + VL * q;
            const bool ok = my_edge >= 0 && l < L;
            Wide b = wide_or_zero(B, static_cast<size_t>(my_edge) * L + l, ok && want_A);
            if constexpr (WEIGHTED) {
                b *= wide_or_zero(W, static_cast<size_t>(my_sender) * L + l, ok && want_A && sender_ok);
            }
#pragma unroll
            for (int c = 0; c < VL; c++) {
                b_left[VL * v + c] = b[c];
            }
        }
    } else {
#pragma unroll
        for (int s = 0; s < L_STEPS; s++) {
            const int32_t l = l_base + 4 * s + q;
            const bool ok = my_edge >= 0 && l < L;
            b_left[s] = load_or_zero(B, static_cast<size_t>(my_edge) * L + l, ok && want_A);
            if constexpr (WEIGHTED) {
                b_left[s] *= load_or_zero(W, static_cast<size_t>(my_sender) * L + l, ok && want_A && sender_ok);
            }
        }
    }
    };
    load_b_left(0);
    // The 16 rows of A are one contiguous piece of memory: read as such (a few
    // cache lines per load instead of 16) and handed to the operand layout
    // through LDS.
    __shared__ T a_tiles[WAVES][16 * 16 * KT];
    T* a_tile = a_tiles[wave];
    {
        constexpr int LOADS = (16 * 16 * KT + WAVE - 1) / WAVE;
        const int32_t tile_elements = n * K;
        T piece[LOADS];
#pragma unroll
        for (int u = 0; u < LOADS; u++) {
            const int32_t at = u * WAVE + lane;
            piece[u] = load_or_zero(A, static_cast<size_t>(first_edge) * K + at, at < tile_elements && (want_B || want_W));
        }
#pragma unroll
        for (int u = 0; u < LOADS; u++) {
            a_tile[u * WAVE + lane] = piece[u];
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int s = 0; s < K_STEPS; s++) {
        const int32_t k = 4 * s + q;
        const bool ok = my_edge >= 0 && k < K;
        const T value = a_tile[ok ? i * K + k : 0];
        a_left[s] = ok ? value : T(0);
    }

    typename M::Acc acc_A[KT];
#pragma unroll
    for (int t = 0; t < KT; t++) {
        acc_A[t] = M::zero();
    }
    const int32_t k_steps = (K + 3) >> 2;

    for (int32_t next_base = 0;;) {
    const int32_t l_base = BLOCKS ? next_base : 0;
    // factors of the results, per accumulator element (row = edge, column of the tile):
    // asked for now, needed after the matrix products
    T weight_out[4][NT];
    T b_out[4][NT];
    if constexpr (WEIGHTED) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int32_t row = M::row(lane, r);
            const int32_t sender = __shfl(my_sender, row);
            load_columns(
                weight_out[r], W, static_cast<size_t>(sender) * L + l_base, l_base,
                row < n && want_B && in_bounds(sender, n_output)
            );
            load_columns(b_out[r], B, static_cast<size_t>(first_edge + row) * L + l_base, l_base, row < n && want_W);
        }
    }

    typename M::Acc acc_B[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        acc_B[t] = M::zero();
    }

    const int32_t l_steps = (L - l_base + 3) >> 2;
    // the receivers among my edges, in ascending order (the index is sorted)
    int32_t node = __builtin_amdgcn_readfirstlane(my_node);
    while (node >= 0) {
        if (in_bounds(node, n_output)) {
            const bool mine = my_node == node;
            const T* block = grad_output + static_cast<size_t>(node) * K * L;
            if (want_A) {
                // right operand: lane (column k = 16 t + i, reduction index l = 4 s + q,
                // or the order of the vectors)
                T right[L_STEPS][KT];
                if constexpr (VECTORS) {
#pragma unroll
                    for (int v = 0; v < L_VECTORS; v++) {
                        const int32_t l = l_base + 4 * VL * v + VL * q;
#pragma unroll
                        for (int t = 0; t < KT; t++) {
                            const int32_t k = 16 * t + i;
                            const Wide values = wide_or_zero(block, static_cast<size_t>(k) * L + l, k < K && l < L);
#pragma unroll
                            for (int c = 0; c < VL; c++) {
                                right[VL * v + c][t] = values[c];
                            }
                        }
                    }
                } else {
#pragma unroll
                    for (int s = 0; s < L_STEPS; s++) {
                        const int32_t l = l_base + 4 * s + q;
#pragma unroll
                        for (int t = 0; t < KT; t++) {
                            const int32_t k = 16 * t + i;
                            right[s][t] = load_or_zero(block, k * L + l, k < K && l < L);
                        }
                    }
                }
#pragma unroll
                for (int s = 0; s < L_STEPS; s++) {
                    // steps whose l are all beyond L are left out (with VECTORS: whole vectors)
                    if (VECTORS ? l_base + 4 * VL * (s / VL) < L : s < l_steps) {
                        const T left = mine ? b_left[s] : T(0);
#pragma unroll
                        for (int t = 0; t < KT; t++) {
                            acc_A[t] = M::mma(left, right[s][t], acc_A[t]);
                        }
                    }
                }
            }
            if (want_B || want_W) {
                // right operand: lane (column of tile t, reduction index k = 4 s + q)
                T right[K_STEPS][NT];
#pragma unroll
                for (int s = 0; s < K_STEPS; s++) {
                    const int32_t k = 4 * s + q;
                    load_columns(right[s], block, static_cast<size_t>(k) * L + l_base, l_base, k < K);
                }
#pragma unroll
                for (int s = 0; s < K_STEPS; s++) {
                    if (s < k_steps) {
                        const T left = mine ? a_left[s] : T(0);
#pragma unroll
                        for (int t = 0; t < NT; t++) {
                            acc_B[t] = M::mma(left, right[s][t], acc_B[t]);
                        }
                    }
                }
            }
        }
        const unsigned long long later = __ballot(lane < n && my_node > node);
        node = later == 0 ? -1 : __builtin_amdgcn_readlane(my_node, __ffsll(static_cast<long long>(later)) - 1);
    }

    // accumulators: lane (column of tile t, rows = edges M::row(lane, r))
    if (want_B || want_W) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int32_t row = M::row(lane, r);
            if (row < n) {
                const size_t row_start = static_cast<size_t>(first_edge + row) * L + l_base;
                T values[NT];
                if constexpr (WEIGHTED) {
                    if (want_B) {
#pragma unroll
                        for (int t = 0; t < NT; t++) {
                            values[t] = acc_B[t][r] * weight_out[r][t];
                        }
                        store_columns(grad_B, row_start, l_base, values);
                    }
                    if (want_W) {
#pragma unroll
                        for (int t = 0; t < NT; t++) {
                            values[t] = acc_B[t][r] * b_out[r][t];
                        }
                        store_columns(edge_W, row_start, l_base, values);
                    }
                } else {
#pragma unroll
                    for (int t = 0; t < NT; t++) {
                        values[t] = acc_B[t][r];
                    }
                    store_columns(grad_B, row_start, l_base, values);
                }
            }
        }
    }
    if (!BLOCKS) {
        break;
    }
    next_base += 16 * NT;
    if (next_base >= L) {
        break;
    }
    load_b_left(next_base);
    }
    if (want_A) {
#pragma unroll
        for (int t = 0; t < KT; t++) {
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int32_t row = M::row(lane, r);
                const int32_t k = 16 * t + i;
                if (row < n && k < K) {
                    grad_A[static_cast<size_t>(first_edge + row) * K + k] = acc_A[t][r];
                }
            }
        }
    }
}

// The same sum without any list in global memory: the workgroup's eight
// wavefronts find the edges of their eight senders by one pass over the
// sender index (sender_gather.hpp) and add the rows up, sixteen loads in
// flight. Used when a row of W fits one value per lane and register.
constexpr int GATHER_SENDERS = 8;
constexpr int GATHER_COLUMNS = 4; // values of a row per lane
constexpr size_t SENDER_SCAN_LIMIT = thresholds::SENDER_SCAN_LIMIT; // index reads of the in-kernel gather, all workgroups together

template <typename T>
__global__ __launch_bounds__(GATHER_SENDERS* WAVE) void sum_by_sender_kernel(
    T* __restrict__ grad_W, const T* __restrict__ edge_W, const int32_t* __restrict__ senders,
    int32_t n_edges, int32_t n_nodes, int32_t L, bool aligned_senders
) {
    using Gather = SenderGather<GATHER_SENDERS>;
    __shared__ typename Gather::Storage storage;
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x >> 6;
    const int32_t node0 = blockIdx.x * GATHER_SENDERS;
    T sum[GATHER_COLUMNS];
    uint32_t column[GATHER_COLUMNS];
#pragma unroll
    for (int c = 0; c < GATHER_COLUMNS; c++) {
        sum[c] = T(0);
        column[c] = min(lane + c * WAVE, L - 1);
    }
    // rows in flight at a time: what 64 registers per lane hold
    constexpr int ROWS = sizeof(T) == 8 ? Gather::STAGE / 2 : Gather::STAGE;
    auto on_stage = [&](int32_t my_edge, int32_t n) {
#pragma unroll 1 // one group of rows after the other, or the registers run out
        for (int k0 = 0; k0 < Gather::STAGE; k0 += ROWS) {
            T values[ROWS][GATHER_COLUMNS];
#pragma unroll
            for (int k = 0; k < ROWS; k++) {
                // lanes beyond n hold -1: read row 0 and leave it out of the sum
                const int32_t edge = max(__builtin_amdgcn_readlane(my_edge, k0 + k), 0);
                const T* row = edge_W + static_cast<size_t>(edge) * L;
#pragma unroll
                for (int c = 0; c < GATHER_COLUMNS; c++) {
                    if (c * WAVE < L) {
                        values[k][c] = row[column[c]];
                    }
                }
            }
#pragma unroll
            for (int k = 0; k < ROWS; k++) {
                if (k0 + k < n) {
#pragma unroll
                    for (int c = 0; c < GATHER_COLUMNS; c++) {
                        if (c * WAVE < L) {
                            sum[c] += values[k][c];
                        }
                    }
                }
            }
        }
    };
    if (aligned_senders) {
        Gather::template run<4>(storage, senders, n_edges, node0, n_nodes, on_stage);
    } else {
        Gather::template run<1>(storage, senders, n_edges, node0, n_nodes, on_stage);
    }
    const int32_t node = node0 + wave;
    if (node < n_nodes) {
#pragma unroll
        for (int c = 0; c < GATHER_COLUMNS; c++) {
            const int32_t l = lane + c * WAVE;
            if (l < L) {
                grad_W[static_cast<size_t>(node) * L + l] = sum[c];
            }
        }
    }
}

// The pass over the sender index needs none of the per-edge rows, so it can
// run beside the kernel that writes them (sender_buckets.hpp:
// list_edges_in_slots): used while a sender has SLOT_MEAN_LIMIT edges or fewer
// on average.
constexpr int SLOT_MEAN_LIMIT = thresholds::SLOT_MEAN_EDGES;

// The sum over the slots: one wavefront per sender, ascending edge order, as
// many rows in flight as 32 registers hold (COLUMNS values of a row per lane).
// A sender with more edges than places (rare by the choice of SLOT_MEAN_LIMIT)
// is looked after by its wavefront alone, which then reads the whole sender
// index itself.
constexpr int LISTED_WAVES = 4;

/// ARRIVALS: the places hold the sender's edges in the order of arrival, with one
/// count (SenderArrivals), which this kernel sets back to zero.
template <typename T, int COLUMNS, bool ARRIVALS = false>
__global__ __launch_bounds__(LISTED_WAVES* WAVE) void sum_slotted_rows_kernel(
    T* __restrict__ grad_W, const T* __restrict__ edge_W, const int32_t* __restrict__ slots,
    int32_t* __restrict__ counts, const int32_t* __restrict__ senders, int32_t n_edges,
    int32_t n_nodes, int32_t L
) {
    __shared__ int32_t sorting_areas[ARRIVALS ? LISTED_WAVES : 1][ARRIVALS ? SLOT_CAPACITY : 1];
    const int lane = threadIdx.x & (WAVE - 1);
    const int32_t node = __builtin_amdgcn_readfirstlane(blockIdx.x * LISTED_WAVES + (threadIdx.x >> 6));
    if (node >= n_nodes) {
        return;
    }
    const int32_t* mine = slots + static_cast<size_t>(node) * SLOT_CAPACITY;
    // all places asked for before the counts are known
    int32_t first_half = mine[lane];
    int32_t second_half = mine[lane + WAVE];
    static_assert(SLOT_PARTS == 4 && SLOT_CAPACITY == 2 * WAVE, "the four parts of a sender's places in two registers");
    int32_t c0 = 0, c1 = 0, c2 = 0, c3 = 0;
    bool listed;
    int32_t count;
    if constexpr (ARRIVALS) {
        count = max(__builtin_amdgcn_readfirstlane(counts[node]), 0);
        if (lane == 0) {
            counts[node] = 0; // (nobody else reads it: zero again for the next launch)
        }
        listed = count <= SLOT_CAPACITY;
    } else {
        const int4 part_counts = reinterpret_cast<const int4*>(counts)[node];
        c0 = __builtin_amdgcn_readfirstlane(part_counts.x);
        c1 = __builtin_amdgcn_readfirstlane(part_counts.y);
        c2 = __builtin_amdgcn_readfirstlane(part_counts.z);
        c3 = __builtin_amdgcn_readfirstlane(part_counts.w);
        listed = max(max(c0, c1), max(c2, c3)) <= SLOT_PART_CAPACITY;
        count = c0 + c1 + c2 + c3;
    }
    T sum[COLUMNS];
    uint32_t column[COLUMNS];
#pragma unroll
    for (int c = 0; c < COLUMNS; c++) {
        sum[c] = T(0);
        column[c] = min(lane + c * WAVE, L - 1);
    }
    constexpr int ROWS = 32 / (COLUMNS * static_cast<int>(sizeof(T) / 4));
    // adds the rows of the first n <= 64 edges held by the lanes of `my_edge`
    auto add_rows = [&](int32_t my_edge, int32_t n) {
#pragma unroll 1
        for (int32_t k0 = 0; k0 < n; k0 += ROWS) {
            T values[ROWS][COLUMNS];
#pragma unroll
            for (int k = 0; k < ROWS; k++) {
                // beyond n: some row that exists, left out of the sum
                const int32_t edge = __builtin_amdgcn_readlane(my_edge, min(k0 + k, WAVE - 1));
                const T* row = edge_W + static_cast<size_t>(edge) * L;
#pragma unroll
                for (int c = 0; c < COLUMNS; c++) {
                    values[k][c] = row[column[c]];
                }
            }
#pragma unroll
            for (int k = 0; k < ROWS; k++) {
                if (k0 + k < n) {
#pragma unroll
                    for (int c = 0; c < COLUMNS; c++) {
                        sum[c] += values[k][c];
                    }
                }
            }
        }
    };
    if (listed) {
        // the parts moved together: position p of the list is in part `part`, place p - before
        auto edge_at = [&](int32_t position) {
            const int32_t part = (position >= c0 ? 1 : 0) + (position >= c0 + c1 ? 1 : 0) +
                                 (position >= c0 + c1 + c2 ? 1 : 0);
            const int32_t before = part == 0 ? 0 : part == 1 ? c0 : part == 2 ? c0 + c1 : c0 + c1 + c2;
            const int32_t place = part * SLOT_PART_CAPACITY + position - before;
            const int32_t low = __shfl(first_half, place & (WAVE - 1));
            const int32_t high = __shfl(second_half, place & (WAVE - 1));
            return place < WAVE ? low : high;
        };
        const int32_t n_first = min(count, WAVE);
        if constexpr (ARRIVALS) {
            if (count > 0) {
                arrivals_in_order(first_half, second_half, count, sorting_areas[threadIdx.x >> 6], lane);
            }
            // (the counters outlive a call: should a failed launch ever leave a count without its
            // list, what the places hold is kept inside the tensor all the same)
            first_half = min(max(first_half, 0), n_edges - 1);
            second_half = min(max(second_half, 0), n_edges - 1);
        }
        const int32_t first = ARRIVALS ? first_half : edge_at(lane);
        add_rows(lane < n_first ? first : 0, n_first);
        if (count > WAVE) {
            const int32_t n_second = count - WAVE;
            const int32_t second = ARRIVALS ? second_half : edge_at(lane + WAVE);
            add_rows(lane < n_second ? second : 0, n_second);
        }
    } else {
        const unsigned long long below = (1ull << lane) - 1ull;
        for (int32_t base = 0; base < n_edges; base += WAVE) {
            const int32_t e = base + lane;
            const bool named = e < n_edges && senders[min(e, n_edges - 1)] == node;
            const unsigned long long mask = __ballot(named);
            if (mask != 0) {
                // the matches moved to the first lanes, in edge order
                // (a permutation of the lanes: the others follow, in their order)
                const int32_t n = __popcll(mask);
                const int32_t named_below = __popcll(mask & below);
                const int32_t place = named ? named_below : n + lane - named_below;
                const int32_t packed = __builtin_amdgcn_ds_permute(place << 2, e);
                add_rows(lane < n ? packed : 0, n);
            }
        }
    }
#pragma unroll
    for (int c = 0; c < COLUMNS; c++) {
        const int32_t l = lane + c * WAVE;
        if (l < L) {
            grad_W[static_cast<size_t>(node) * L + l] = sum[c];
        }
    }
}

// The same sum over lists that are already there (sender_buckets.hpp: the edges in
// the order of their senders, built beside the per-edge kernel on a side
// stream): one wavefront per sender, sixteen rows in flight.

template <typename T>
__global__ __launch_bounds__(LISTED_WAVES* WAVE) void sum_listed_rows_kernel(
    T* __restrict__ grad_W, const T* __restrict__ edge_W, const int32_t* __restrict__ offsets,
    const int32_t* __restrict__ edge_of_position, int32_t n_nodes, int32_t L
) {
    const int lane = threadIdx.x & (WAVE - 1);
    const int32_t node = __builtin_amdgcn_readfirstlane(blockIdx.x * LISTED_WAVES + (threadIdx.x >> 6));
    if (node >= n_nodes) {
        return;
    }
    const int32_t begin = offsets[node];
    const int32_t end = offsets[node + 1];
    T sum[GATHER_COLUMNS];
    uint32_t column[GATHER_COLUMNS];
#pragma unroll
    for (int c = 0; c < GATHER_COLUMNS; c++) {
        sum[c] = T(0);
        column[c] = min(lane + c * WAVE, L - 1);
    }
    constexpr int ROWS = sizeof(T) == 8 ? 8 : 16;
    for (int32_t p0 = begin; p0 < end; p0 += WAVE) {
        const int32_t n = min(WAVE, end - p0);
        const int32_t my_edge = lane < n ? edge_of_position[p0 + lane] : 0;
#pragma unroll 1
        for (int32_t k0 = 0; k0 < n; k0 += ROWS) {
            T values[ROWS][GATHER_COLUMNS];
#pragma unroll
            for (int k = 0; k < ROWS; k++) {
                // beyond n: some row that exists, left out of the sum
                const int32_t edge = __builtin_amdgcn_readlane(my_edge, min(k0 + k, WAVE - 1));
                const T* row = edge_W + static_cast<size_t>(edge) * L;
#pragma unroll
                for (int c = 0; c < GATHER_COLUMNS; c++) {
                    if (c * WAVE < L) {
                        values[k][c] = row[column[c]];
                    }
                }
            }
#pragma unroll
            for (int k = 0; k < ROWS; k++) {
                if (k0 + k < n) {
#pragma unroll
                    for (int c = 0; c < GATHER_COLUMNS; c++) {
                        if (c * WAVE < L) {
                            sum[c] += values[k][c];
                        }
                    }
                }
            }
        }
    }
#pragma unroll
    for (int c = 0; c < GATHER_COLUMNS; c++) {
        const int32_t l = lane + c * WAVE;
        if (l < L) {
            grad_W[static_cast<size_t>(node) * L + l] = sum[c];
        }
    }
}

// vjp for rows too wide for the LDS tile of vjp_kernel: one wavefront per
// edge, lanes over l in chunks of 64, the receiver's grad_output row read
// from global memory (L2). grad_A[e, k] is a fixed shuffle tree over the
// lanes, accumulated chunk after chunk by one lane; grad_B / the per-edge row
// of grad_W are sums over k inside a lane. Slow (every edge reads K * L
// values) and general.
constexpr int WIDE_WAVES = 4;

template <typename T, bool WEIGHTED>
__global__ __launch_bounds__(WIDE_WAVES* WAVE) void vjp_wide_kernel(
    T* grad_A,
    T* __restrict__ grad_B,
    T* __restrict__ edge_W,
    const T* __restrict__ grad_output,
    const T* __restrict__ A,
    const T* __restrict__ B,
    const T* __restrict__ W,
    const int32_t* __restrict__ indices_W,
    const int32_t* __restrict__ indices_output,
    int32_t n_edges,
    int32_t n_output,
    int32_t K,
    int32_t L
) {
    const int lane = threadIdx.x & (WAVE - 1);
    const int32_t e = blockIdx.x * WIDE_WAVES + (threadIdx.x >> 6);
    if (e >= n_edges) {
        return;
    }
    const int32_t receiver = indices_output[e];
    const bool receiver_ok = in_bounds(receiver, n_output);
    const T* g_row = grad_output + static_cast<size_t>(receiver_ok ? receiver : 0) * K * L;
    const T* a_row = A + static_cast<size_t>(e) * K;
    int32_t w_row = 0;
    bool w_ok = true;
    if constexpr (WEIGHTED) {
        w_row = indices_W[e];
        w_ok = in_bounds(w_row, n_output);
        w_row = w_ok ? w_row : 0;
    }
    for (int32_t l0 = 0; l0 < L; l0 += WAVE) {
        const int32_t l = l0 + lane;
        const bool ok = l < L;
        const T b = load_or_zero(B, static_cast<size_t>(e) * L + l, ok);
        T w = T(1);
        if constexpr (WEIGHTED) {
            w = load_or_zero(W, static_cast<size_t>(w_row) * L + l, ok && w_ok);
        }
        const T bw = b * w;
        T along_k = T(0);
        for (int32_t k = 0; k < K; k++) {
            const T g = load_or_zero(g_row, static_cast<size_t>(k) * L + l, ok && receiver_ok);
            along_k += g * a_row[k];
            T along_l = g * bw;
#pragma unroll
            for (int offset = WAVE / 2; offset > 0; offset >>= 1) {
                along_l += __shfl_xor(along_l, offset);
            }
            if (grad_A != nullptr && lane == 0) {
                T* target = grad_A + static_cast<size_t>(e) * K + k;
                *target = (l0 == 0 ? T(0) : *target) + along_l;
            }
        }
        if (ok) {
            if (grad_B != nullptr) {
                grad_B[static_cast<size_t>(e) * L + l] = along_k * w;
            }
            if (WEIGHTED && edge_W != nullptr) {
                edge_W[static_cast<size_t>(e) * L + l] = along_k * b;
            }
        }
    }
}

/// Whether MOPS_AMD_WIDE_OFFSETS is set: the forward kernels for tensors of 4 GB
/// and more are then used whatever the sizes (what the test of those kernels
/// does; no other use).
bool wide_offsets_forced() {
    const char* value = std::getenv("MOPS_AMD_WIDE_OFFSETS");
    return value != nullptr && value[0] != '\0' && value[0] != '0';
}

unsigned blocks_for(int32_t n_edges) {
    size_t waves = ceil_div(static_cast<size_t>(n_edges), CHUNK);
    return static_cast<unsigned>(ceil_div(waves, WAVES_PER_BLOCK));
}

template <typename T, bool WEIGHTED>
void launch_forward(
    Tensor<T, 3> output,
    Tensor<T, 2> A,
    Tensor<T, 2> B,
    const T* W,
    const int32_t* indices_W,
    Tensor<int32_t, 1> indices_output,
    const char* operation
) {
    const int32_t n_output = narrow_i32(output.shape[0], "output.shape[0]");
    const int32_t n_edges = narrow_i32(A.shape[0], "A.shape[0]");
    const int32_t K = narrow_i32(A.shape[1], "A.shape[1]");
    const int32_t L = narrow_i32(B.shape[1], "B.shape[1]");
    narrow_i32(A.shape[1] * B.shape[1], "size_A * size_B");
    if (n_output == 0 || K == 0 || L == 0) {
        return;
    }
    hipStream_t stream = current_stream();
    if (n_edges == 0) {
        const size_t count = static_cast<size_t>(n_output) * K * L;
        unsigned blocks = static_cast<unsigned>(std::min<size_t>(ceil_div(count, 256), 4096));
        zero_kernel<T><<<blocks, 256, 0, stream>>>(output.data, count);
        finish_call(operation);
        return;
    }
    const unsigned blocks = blocks_for(n_edges);
    // byte offsets of 32 bits into A, B, W and the index of the weight rows (a wavefront asks
    // for up to 36 positions past the end of a segment, with a mask: room for that too)
    const uint64_t widest_row = static_cast<uint64_t>(std::max(K, L)) * sizeof(T);
    const bool narrow = !wide_offsets_forced() &&
                        (static_cast<uint64_t>(n_edges) + 64) * std::max<uint64_t>(widest_row, 4) < (uint64_t(1) << 32) - 64 &&
                        (static_cast<uint64_t>(n_output) + 1) * widest_row < (uint64_t(1) << 32) - 64;
    // few rows with many edges each: cut the segments and add the pieces up
    // (twice SPLIT edges per row on average, or it is not worth a second kernel)
    if (static_cast<size_t>(n_edges) >= static_cast<size_t>(n_output) * 2 * SPLIT && n_edges > SPLIT) {
        const size_t row_elements = static_cast<size_t>(K) * L;
        const size_t n_split_blocks = ceil_div(static_cast<size_t>(n_edges), SPLIT);
        const size_t pieces_bytes = align256(n_split_blocks * row_elements * sizeof(T));
        char* workspace = static_cast<char*>(scratch(2 * pieces_bytes));
        T* tails = reinterpret_cast<T*>(workspace);
        T* heads = reinterpret_cast<T*>(workspace + pieces_bytes);
#define MOPS_LAUNCH_SPLIT(NT)                                                                      \
    if (narrow) {                                                                                  \
        forward_split_kernel<T, NT, WEIGHTED, true><<<blocks, BLOCK, 0, stream>>>(                 \
            output.data, tails, heads, A.data, B.data, W, indices_W, indices_output.data, n_edges, \
            n_output, K, L                                                                         \
        );                                                                                         \
    } else {                                                                                       \
        forward_split_kernel<T, NT, WEIGHTED, false><<<blocks, BLOCK, 0, stream>>>(                \
            output.data, tails, heads, A.data, B.data, W, indices_W, indices_output.data, n_edges, \
            n_output, K, L                                                                         \
        );                                                                                         \
    }
        if (L <= 16) {
            MOPS_LAUNCH_SPLIT(1);
        } else if (L <= 32) {
            MOPS_LAUNCH_SPLIT(2);
        } else {
            MOPS_LAUNCH_SPLIT(4);
        }
#undef MOPS_LAUNCH_SPLIT
        combine_pieces_kernel<T><<<static_cast<unsigned>(n_split_blocks), COMBINE_THREADS, 0, stream>>>(
            output.data, tails, heads, indices_output.data, n_edges, n_output,
            static_cast<int32_t>(row_elements)
        );
        finish_call(operation);
        return;
    }
    {
    MainKernelTimer timer(stream);
    // NT consecutive columns per lane (forward_segment, PACKED) where rows and pointers allow
    const int tiles = L <= 16 ? 1 : L <= 32 ? 2 : 4;
    const size_t vector_bytes = tiles * sizeof(T);
    const bool packed = tiles > 1 && L % tiles == 0 && reinterpret_cast<uintptr_t>(B.data) % vector_bytes == 0 &&
                        reinterpret_cast<uintptr_t>(output.data) % vector_bytes == 0 &&
                        (!WEIGHTED || reinterpret_cast<uintptr_t>(W) % vector_bytes == 0);
#define MOPS_LAUNCH_FORWARD(NT)                                                                    \
    if (narrow && packed) {                                                                        \
        forward_kernel<T, NT, WEIGHTED, true, (NT > 1)><<<blocks, BLOCK, 0, stream>>>(             \
            output.data, A.data, B.data, W, indices_W, indices_output.data, n_edges, n_output, K,  \
            L                                                                                      \
        );                                                                                         \
    } else if (narrow) {                                                                           \
        forward_kernel<T, NT, WEIGHTED, true><<<blocks, BLOCK, 0, stream>>>(                       \
            output.data, A.data, B.data, W, indices_W, indices_output.data, n_edges, n_output, K,  \
            L                                                                                      \
        );                                                                                         \
    } else {                                                                                       \
        forward_kernel<T, NT, WEIGHTED, false><<<blocks, BLOCK, 0, stream>>>(                      \
            output.data, A.data, B.data, W, indices_W, indices_output.data, n_edges, n_output, K,  \
            L                                                                                      \
        );                                                                                         \
    }
    if (L <= 16) {
        MOPS_LAUNCH_FORWARD(1);
    } else if (L <= 32) {
        MOPS_LAUNCH_FORWARD(2);
    } else {
        MOPS_LAUNCH_FORWARD(4);
    }
    }
#undef MOPS_LAUNCH_FORWARD
    finish_call(operation);
}

/// output = opsa(A, B) + opsa(A2, B2); false (and nothing launched) for shapes that
/// launch_forward gives to other kernels than forward_kernel with offsets of 32 bits.
template <typename T>
bool launch_forward_of_two_pairs(
    Tensor<T, 3> output, Tensor<T, 2> A, Tensor<T, 2> B, const T* A2, const T* B2, Tensor<int32_t, 1> indices_output
) {
    const int32_t n_output = narrow_i32(output.shape[0], "output.shape[0]");
    const int32_t n_edges = narrow_i32(A.shape[0], "A.shape[0]");
    const int32_t K = narrow_i32(A.shape[1], "A.shape[1]");
    const int32_t L = narrow_i32(B.shape[1], "B.shape[1]");
    narrow_i32(A.shape[1] * B.shape[1], "size_A * size_B");
    if (n_output == 0 || K == 0 || L == 0 || n_edges == 0) {
        return false;
    }
    const uint64_t widest_row = static_cast<uint64_t>(std::max(K, L)) * sizeof(T);
    const bool narrow = !wide_offsets_forced() &&
                        (static_cast<uint64_t>(n_edges) + 64) * std::max<uint64_t>(widest_row, 4) < (uint64_t(1) << 32) - 64 &&
                        (static_cast<uint64_t>(n_output) + 1) * widest_row < (uint64_t(1) << 32) - 64;
    const bool split = static_cast<size_t>(n_edges) >= static_cast<size_t>(n_output) * 2 * SPLIT && n_edges > SPLIT;
    if (!narrow || split) {
        return false;
    }
    hipStream_t stream = current_stream();
    const unsigned blocks = blocks_for(n_edges);
#define MOPS_LAUNCH_TWO(NT)                                                                        \
    forward_two_pairs_kernel<T, NT><<<blocks, BLOCK, 0, stream>>>(                                 \
        output.data, A.data, B.data, A2, B2, indices_output.data, n_edges, n_output, K, L          \
    )
    if (L <= 16) {
        MOPS_LAUNCH_TWO(1);
    } else if (L <= 32) {
        MOPS_LAUNCH_TWO(2);
    } else {
        MOPS_LAUNCH_TWO(4);
    }
#undef MOPS_LAUNCH_TWO
    return true;
}

template <typename T, bool WEIGHTED>
void launch_vjp(
    Tensor<T, 2> grad_A,
    Tensor<T, 2> grad_B,
    Tensor<T, 2> grad_W,
    Tensor<T, 3> grad_output,
    Tensor<T, 2> A,
    Tensor<T, 2> B,
    const T* W,
    const int32_t* indices_W,
    Tensor<int32_t, 1> indices_output,
    const char* operation
) {
    const bool want_A = grad_A.data != nullptr;
    const bool want_B = grad_B.data != nullptr;
    const bool want_W = WEIGHTED && grad_W.data != nullptr;
    if (!want_A && !want_B && !want_W) {
        return;
    }
    const int32_t n_output = narrow_i32(grad_output.shape[0], "grad_output.shape[0]");
    const int32_t n_edges = narrow_i32(A.shape[0], "A.shape[0]");
    const int32_t K = narrow_i32(A.shape[1], "A.shape[1]");
    const int32_t L = narrow_i32(B.shape[1], "B.shape[1]");
    narrow_i32(A.shape[1] * B.shape[1], "size_A * size_B");
    hipStream_t stream = current_stream();

    // scratch: edge_W | sender buckets   (only when grad_W is wanted)
    const size_t edge_w_bytes =
        want_W ? align256(static_cast<size_t>(n_edges) * L * sizeof(T)) : 0;
    // Every workgroup of the in-kernel gather reads the whole sender index: fine while
    // (edges x workgroups) is small, quadratic in the size of the graph beyond
    const size_t index_reads =
        static_cast<size_t>(n_edges) * ceil_div(static_cast<size_t>(std::max(n_output, 1)), GATHER_SENDERS);
    const bool narrow_rows = L <= GATHER_COLUMNS * WAVE;
    // (at 60 000 edges the lists cost more than the scans: 52 us against 32 for the whole vjp)
    const bool gather_in_kernel = narrow_rows && n_edges > 0 && index_reads <= SENDER_SCAN_LIMIT;
    const bool sparse = n_output > 0 && L > 0 &&
                        static_cast<size_t>(n_edges) <= static_cast<size_t>(n_output) * SLOT_MEAN_LIMIT;
    // large sparse graphs: every edge takes the next of its sender's places in the per-edge
    // kernel itself, an atomic each, and the sum puts the places in order. Whole vjp at 30 edges
    // per sender, L = 32, f32, this way against the slots below (up to 4000 senders) or the
    // counting sort beside the per-edge kernel (beyond): 2000 senders 27.6 / 22.6 us, 3000:
    // 33.4 / 29.6, 4000: 37.6 / 39.3, 6000: 48 / 75, 20 000: 156 / 212
    // (with no edges at all gather_in_kernel is false too: the per-edge kernel that would fill the
    // places is not launched then, so this way needs edges)
    const bool by_arrival = want_W && narrow_rows && sparse && n_edges > 0 && K > 0 && K <= thresholds::OPSA_VJP_ROWS_IN_REGISTERS &&
                            (n_output > thresholds::ARRIVAL_NODES || !gather_in_kernel) &&
                            static_cast<size_t>(n_output) <= SCRATCH_COUNTERS;
    // small sparse graphs: the pass over the sender index is done by workgroups of the
    // per-edge kernel's launch and leaves every sender's edges in places of its own
    // (60 000 edges over 2000 senders, L = 32, f32: 33 -> 22 us for the whole vjp;
    // graphs with more edges per sender keep the gather)
    const bool slotted = want_W && gather_in_kernel && sparse && !by_arrival;
    const size_t slots_bytes = slotted ? sender_slots_bytes(n_output) : by_arrival ? sender_arrivals_bytes(n_output) : 0;
    const size_t buckets_bytes =
        want_W && !gather_in_kernel && !by_arrival ? edges_by_sender_bytes(n_output, n_edges) : slots_bytes;
    char* workspace =
        want_W ? static_cast<char*>(scratch(edge_w_bytes + buckets_bytes)) : nullptr;
    T* edge_W = want_W ? reinterpret_cast<T*>(workspace) : nullptr;

    // the lists of edges per sender do not depend on the kernels below: they are
    // built beside them, on a side stream that joins before the lists are used
    SenderBuckets buckets{};
    EdgesBySender by_sender{};
    SenderSlots slots{};
    std::optional<ScratchCounters> taken; // (until the end of this call, finish_call included)
    if (by_arrival) {
        // (places and counters of SenderArrivals: filled by the per-edge kernel, used by the sum)
        taken.emplace();
        slots = SenderSlots{reinterpret_cast<int32_t*>(workspace + edge_w_bytes), taken->data()};
    }
    const bool use_buckets = want_W && n_output > 0 && L > 0 && !gather_in_kernel && !by_arrival;
    std::unique_ptr<SideStream> beside;
    bool listed = false; // the slots are being filled by a kernel that is already enqueued
    if (use_buckets) {
        beside = std::make_unique<SideStream>(stream);
        if (narrow_rows) {
            by_sender = order_edges_by_sender(indices_W, n_edges, n_output, workspace + edge_w_bytes, beside->get());
        } else {
            buckets = build_sender_buckets(indices_W, n_edges, n_output, workspace + edge_w_bytes, beside->get());
        }
    }

    // degenerate shapes: a gradient that sums over an empty axis is zero
    if (want_A && L == 0 && n_edges > 0 && K > 0) {
        const size_t count = static_cast<size_t>(n_edges) * K;
        zero_kernel<T><<<static_cast<unsigned>(std::min<size_t>(ceil_div(count, 256), 4096)), 256, 0, stream>>>(
            grad_A.data, count
        );
    }
    if (want_B && K == 0 && n_edges > 0 && L > 0) {
        const size_t count = static_cast<size_t>(n_edges) * L;
        zero_kernel<T><<<static_cast<unsigned>(std::min<size_t>(ceil_div(count, 256), 4096)), 256, 0, stream>>>(
            grad_B.data, count
        );
    }
    if (want_W && K == 0 && n_edges > 0 && L > 0) {
        const size_t count = static_cast<size_t>(n_edges) * L;
        zero_kernel<T><<<static_cast<unsigned>(std::min<size_t>(ceil_div(count, 256), 4096)), 256, 0, stream>>>(
            edge_W, count
        );
    }

    if (n_output > 0 && n_edges > 0 && K > 0 && L > 0) {
        const size_t Ks = odd_stride(K), Ls = odd_stride(L);
        const size_t lds =
            (K * Ls + STAGE_EDGES * Ks + (WEIGHTED ? 2 : 1) * STAGE_EDGES * Ls) * sizeof(T);
        auto log2_ceil = [](int32_t n) {
            int32_t shift = 0;
            while ((1 << shift) < n) {
                shift++;
            }
            return shift;
        };
        const unsigned waves = static_cast<unsigned>(ceil_div(static_cast<size_t>(n_edges), CHUNK));
        if (lds > 64 * 1024 && K > thresholds::OPSA_VJP_ROWS_IN_REGISTERS) {
            const unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<size_t>(n_edges), WIDE_WAVES));
            vjp_wide_kernel<T, WEIGHTED><<<blocks, WIDE_WAVES * WAVE, 0, stream>>>(
                grad_A.data, grad_B.data, edge_W, grad_output.data, A.data, B.data, W, indices_W,
                indices_output.data, n_edges, n_output, K, L
            );
        } else if (K <= thresholds::OPSA_VJP_ROWS_IN_REGISTERS) {
            const unsigned groups = static_cast<unsigned>(ceil_div(static_cast<size_t>(n_edges), 16));
            MainKernelTimer timer(stream);
            const bool vectors = L % (16 / static_cast<int32_t>(sizeof(T))) == 0 &&
                                 reinterpret_cast<uintptr_t>(B.data) % 16 == 0 &&
                                 reinterpret_cast<uintptr_t>(grad_output.data) % 16 == 0 &&
                                 reinterpret_cast<uintptr_t>(grad_B.data) % 16 == 0 &&
                                 reinterpret_cast<uintptr_t>(edge_W) % 16 == 0 &&
                                 (!WEIGHTED || reinterpret_cast<uintptr_t>(W) % 16 == 0);
#define MOPS_LAUNCH_ROWS_WITH(KT, NT, VECTORS, BLOCKS, LISTS, GRID, WAVES)                          \
    edge_rows_vjp_kernel<T, KT, NT, WEIGHTED, VECTORS, BLOCKS, LISTS><<<GRID, (WAVES) * WAVE, 0, stream>>>( \
        grad_A.data, grad_B.data, edge_W, grad_output.data, A.data, B.data, W, indices_W,          \
        indices_output.data, n_edges, n_output, K, L, const_cast<int32_t*>(slots.edges),           \
        const_cast<int32_t*>(slots.counts), static_cast<int32_t>(list_blocks), aligned_senders     \
    )
#define MOPS_LAUNCH_ROWS_AS(KT, NT, VECTORS, BLOCKS)                                                \
    if constexpr (WEIGHTED) {                                                                      \
        if (list_blocks > 0) {                                                                     \
            MOPS_LAUNCH_ROWS_WITH(KT, NT, VECTORS, BLOCKS, true, listing_grid, LISTING_WAVES);     \
        } else {                                                                                   \
            MOPS_LAUNCH_ROWS_WITH(KT, NT, VECTORS, BLOCKS, false, groups, 1);                      \
        }                                                                                          \
    } else {                                                                                       \
        MOPS_LAUNCH_ROWS_WITH(KT, NT, VECTORS, BLOCKS, false, groups, 1);                          \
    }
#define MOPS_LAUNCH_ROWS(KT, NT)                                                                   \
    if (vectors) {                                                                                 \
        MOPS_LAUNCH_ROWS_AS(KT, NT, true, false);                                                  \
    } else {                                                                                       \
        MOPS_LAUNCH_ROWS_AS(KT, NT, false, false);                                                 \
    }
#define MOPS_LAUNCH_ROW_PASSES_OF(KT, NT)                                                          \
    if (vectors) {                                                                                 \
        MOPS_LAUNCH_ROWS_AS(KT, NT, true, true);                                                   \
    } else {                                                                                       \
        MOPS_LAUNCH_ROWS_AS(KT, NT, false, true);                                                  \
    }
// More than 32 columns: one pass over 64 (four column tiles), or passes of 64 each beyond that.
// In double the kernel with four column tiles has room for one wavefront per SIMD where the
// rows of W come with it (OPSAW) or A has more than 16 columns; passes of 32 columns (two
// tiles, three wavefronts per SIMD) are then the faster way, although grad_output is read once
// per pass (60 000 edges, f64, 64 / 32 columns per pass: OPSAW K = 13, L = 64: 67.8 / 57.3 us;
// K = 13, L = 128: 139 / 104; K = 25, L = 64: 84.9 / 71.0; OPSA K = 25, L = 64: 54.1 / 45.3;
// K = 25, L = 128: 102 / 89), but not with three or four tiles of columns of A (K = L = 48:
// 61.5 / 78.3; OPSAW K = L = 64: 132 / 158) nor for OPSA with up to 16 columns of A
// (K = 13, L = 64: 27.4 / 29.0).
#define MOPS_LAUNCH_BEYOND_32(KT, SINGLE_PASS)                                                     \
    if constexpr (sizeof(T) == 8 && (WEIGHTED ? KT <= 2 : KT == 2)) {                              \
        MOPS_LAUNCH_ROW_PASSES_OF(KT, 2);                                                          \
    } else if (SINGLE_PASS) {                                                                      \
        MOPS_LAUNCH_ROWS(KT, 4);                                                                   \
    } else {                                                                                       \
        MOPS_LAUNCH_ROW_PASSES_OF(KT, 4);                                                          \
    }
            // the listing of the senders' edges rides along in this launch
            const unsigned list_blocks = slotted ? sender_slots_blocks(n_output) : 0;
            const unsigned listing_grid =
                list_blocks + static_cast<unsigned>(ceil_div(static_cast<size_t>(groups), LISTING_WAVES));
            const bool aligned_senders = reinterpret_cast<uintptr_t>(indices_W) % 16 == 0;
            if (slotted) {
                slots = sender_slots_in(workspace + edge_w_bytes, n_output);
                listed = true;
            }

            if (K <= 16) {
                if (L <= 16) {
                    MOPS_LAUNCH_ROWS(1, 1);
                } else if (L <= 32) {
                    MOPS_LAUNCH_ROWS(1, 2);
                } else {
                    MOPS_LAUNCH_BEYOND_32(1, L <= 64);
                }
            } else if (K <= 32) {
                if (L <= 16) {
                    MOPS_LAUNCH_ROWS(2, 1);
                } else if (L <= 32) {
                    MOPS_LAUNCH_ROWS(2, 2);
                } else {
                    MOPS_LAUNCH_BEYOND_32(2, L <= 64);
                }
            } else if (K <= 48) {
                if (L <= 16) {
                    MOPS_LAUNCH_ROWS(3, 1);
                } else if (L <= 32) {
                    MOPS_LAUNCH_ROWS(3, 2);
                } else {
                    MOPS_LAUNCH_BEYOND_32(3, L <= 64);
                }
            } else {
                if (L <= 16) {
                    MOPS_LAUNCH_ROWS(4, 1);
                } else if (L <= 32) {
                    MOPS_LAUNCH_ROWS(4, 2);
                } else {
                    MOPS_LAUNCH_BEYOND_32(4, L <= 64);
                }
            }
#undef MOPS_LAUNCH_BEYOND_32
#undef MOPS_LAUNCH_ROW_PASSES_OF
#undef MOPS_LAUNCH_ROWS
#undef MOPS_LAUNCH_ROWS_AS
#undef MOPS_LAUNCH_ROWS_WITH
        } else {
            MainKernelTimer timer(stream);
            vjp_kernel<T, WEIGHTED><<<waves, WAVE, lds, stream>>>(
                grad_A.data, grad_B.data, edge_W, grad_output.data, A.data, B.data, W, indices_W,
                indices_output.data, n_edges, n_output, K, L, log2_ceil(K), log2_ceil(L)
            );
        }
    }

    if (by_arrival) {
        test_failure_point("opsaw_vjp_after_listing");
        const unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<size_t>(n_output), LISTED_WAVES));
#define MOPS_LAUNCH_ARRIVED(COLUMNS)                                                               \
    sum_slotted_rows_kernel<T, COLUMNS, true><<<blocks, LISTED_WAVES * WAVE, 0, stream>>>(         \
        grad_W.data, edge_W, slots.edges, const_cast<int32_t*>(slots.counts), indices_W, n_edges, n_output, L \
    )
        if (L <= WAVE) {
            MOPS_LAUNCH_ARRIVED(1);
        } else if (L <= 2 * WAVE) {
            MOPS_LAUNCH_ARRIVED(2);
        } else {
            MOPS_LAUNCH_ARRIVED(4);
        }
#undef MOPS_LAUNCH_ARRIVED
    } else if (slotted) {
        if (!listed) {
            slots = list_edges_in_slots(indices_W, n_edges, n_output, workspace + edge_w_bytes, stream);
        }
        const unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<size_t>(n_output), LISTED_WAVES));
#define MOPS_LAUNCH_SLOTTED(COLUMNS)                                                                \
    sum_slotted_rows_kernel<T, COLUMNS><<<blocks, LISTED_WAVES * WAVE, 0, stream>>>(               \
        grad_W.data, edge_W, slots.edges, const_cast<int32_t*>(slots.counts), indices_W, n_edges, n_output, L \
    )
        if (L <= WAVE) {
            MOPS_LAUNCH_SLOTTED(1);
        } else if (L <= 2 * WAVE) {
            MOPS_LAUNCH_SLOTTED(2);
        } else {
            MOPS_LAUNCH_SLOTTED(4);
        }
#undef MOPS_LAUNCH_SLOTTED
    } else if (want_W && n_output > 0 && L > 0 && gather_in_kernel) {
        const bool aligned = reinterpret_cast<uintptr_t>(indices_W) % 16 == 0;
        const unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<size_t>(n_output), GATHER_SENDERS));
        sum_by_sender_kernel<T><<<blocks, GATHER_SENDERS * WAVE, 0, stream>>>(
            grad_W.data, edge_W, indices_W, n_edges, n_output, L, aligned
        );
    } else if (use_buckets) {
        beside.reset(); // joins
        if (narrow_rows) {
            const unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<size_t>(n_output), LISTED_WAVES));
            sum_listed_rows_kernel<T><<<blocks, LISTED_WAVES * WAVE, 0, stream>>>(
                grad_W.data, edge_W, by_sender.offsets, by_sender.edge, n_output, L
            );
        } else {
            int threads = std::min(256, round_up_wave(L));
            gather_weights_kernel<T><<<n_output, threads, 0, stream>>>(grad_W.data, edge_W, buckets, L);
        }
    }
    finish_call(operation);
}

/// The per-edge tensors of one OPSA / OPSAW call re-ordered by a stable sort
/// of the scatter index, with room for the per-edge gradients in that order.
template <typename T> class SortedEdges {
public:
    SortedEdges(
        Tensor<T, 2> A, Tensor<T, 2> B, const int32_t* second_index, Tensor<int32_t, 1> indices_output,
        bool want_A, bool want_B
    )
        : stream_(current_stream()), n_(A.shape[0]), K_(A.shape[1]), L_(B.shape[1]),
          order_(indices_output.data, narrow_i32(A.shape[0], "A.shape[0]"), stream_), A_(n_ * K_, stream_),
          B_(n_ * L_, stream_), second_(second_index != nullptr ? n_ : 0, stream_),
          grad_A_(want_A ? n_ * K_ : 0, stream_), grad_B_(want_B ? n_ * L_ : 0, stream_), want_A_(want_A),
          want_B_(want_B) {
        order_.gather_rows(A_.data(), A.data, narrow_i32(K_, "A.shape[1]"));
        order_.gather_rows(B_.data(), B.data, narrow_i32(L_, "B.shape[1]"));
        if (second_index != nullptr) {
            order_.gather_rows(second_.data(), second_index, 1);
        }
    }
    Tensor<T, 2> A() const { return {A_.data(), {n_, K_}}; }
    Tensor<T, 2> B() const { return {B_.data(), {n_, L_}}; }
    Tensor<int32_t, 1> index() const { return {const_cast<int32_t*>(order_.sorted_index()), {n_}}; }
    Tensor<int32_t, 1> second_index() const { return {second_.data(), {n_}}; }
    Tensor<T, 2> grad_A() const { return {grad_A_.data(), {want_A_ ? n_ : 0, want_A_ ? K_ : 0}}; }
    Tensor<T, 2> grad_B() const { return {grad_B_.data(), {want_B_ ? n_ : 0, want_B_ ? L_ : 0}}; }
    /// per-edge gradients back to the callers' rows
    void put_back(Tensor<T, 2> grad_A, Tensor<T, 2> grad_B) const {
        if (want_A_) {
            order_.scatter_rows(grad_A.data, grad_A_.data(), static_cast<int32_t>(K_));
        }
        if (want_B_) {
            order_.scatter_rows(grad_B.data, grad_B_.data(), static_cast<int32_t>(L_));
        }
    }

private:
    hipStream_t stream_;
    size_t n_, K_, L_;
    EdgeOrder order_;
    StreamTemporary<T> A_, B_;
    StreamTemporary<int32_t> second_;
    StreamTemporary<T> grad_A_, grad_B_;
    bool want_A_, want_B_;
};

} // namespace
} // namespace opsa
using namespace opsa;
} // namespace mops::amd

// ------------------------------------------------------------ C++ API ----
namespace mops::cuda {

template <typename scalar_t>
void outer_product_scatter_add(MOPS_OPSA_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    const char* operation = "cuda_outer_product_scatter_add";
    checks::Validator validator(operation);
    checks::opsa(validator, output, A, B, indices_output);
    if (amd::accept_unsorted() &&
        !amd::is_sorted_on_device(indices_output.data, amd::narrow_i32(A.shape[0], "A.shape[0]"), amd::current_stream())) {
        // the same call on the edges in the order of a stable sort by destination
        const amd::SortedEdges<scalar_t> sorted(A, B, nullptr, indices_output, false, false);
        ::mops::cuda::outer_product_scatter_add<scalar_t>(output, sorted.A(), sorted.B(), sorted.index());
        return;
    }
    amd::validate_scatter_index(indices_output, output.shape[0], "indices_output", operation);
    amd::launch_forward<scalar_t, false>(output, A, B, nullptr, nullptr, indices_output, operation);
}

template <typename scalar_t>
void outer_product_scatter_add_vjp(MOPS_OPSA_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    const char* operation = "cuda_outer_product_scatter_add_vjp";
    checks::Validator validator(operation);
    checks::opsa_vjp(validator, grad_A, grad_B, grad_output, A, B, indices_output);
    if (amd::accept_unsorted() &&
        !amd::is_sorted_on_device(indices_output.data, amd::narrow_i32(A.shape[0], "A.shape[0]"), amd::current_stream())) {
        const amd::SortedEdges<scalar_t> sorted(
            A, B, nullptr, indices_output, grad_A.data != nullptr, grad_B.data != nullptr
        );
        ::mops::cuda::outer_product_scatter_add_vjp<scalar_t>(
            sorted.grad_A(), sorted.grad_B(), grad_output, sorted.A(), sorted.B(), sorted.index()
        );
        sorted.put_back(grad_A, grad_B);
        amd::finish_call(operation);
        return;
    }
    amd::validate_scatter_index(indices_output, grad_output.shape[0], "indices_output", operation);
    amd::launch_vjp<scalar_t, false>(
        grad_A, grad_B, Tensor<scalar_t, 2>{nullptr, {0, 0}}, grad_output, A, B, nullptr, nullptr,
        indices_output, operation
    );
}

// Second order (semantics of mops/src/opsa/cpu.tpp:114-246; the reference's
// device path has none, mops/src/opsa/opsa.cu:305-318). The operation is
// bilinear, so every output is a first-order call with one operand replaced
// by a cotangent:
//   grad_grad_output = forward(grad_grad_A, B) + forward(A, grad_grad_B)
//   grad_A_2         = vjp's grad_A with B := grad_grad_B
//   grad_B_2         = vjp's grad_B with A := grad_grad_A
// A cotangent that is not given counts as zero.
template <typename scalar_t>
void outer_product_scatter_add_vjp_vjp(MOPS_OPSA_VJP_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using namespace mops::amd;
    const char* operation = "cuda_outer_product_scatter_add_vjp_vjp";
    checks::Validator validator(operation);
    checks::opsa_vjp_vjp(
        validator, grad_grad_output, grad_A_2, grad_B_2, grad_grad_A, grad_grad_B, grad_output, A, B,
        indices_output
    );
    validate_scatter_index(indices_output, grad_output.shape[0], "indices_output", operation);
    const bool have_A = grad_grad_A.data != nullptr, have_B = grad_grad_B.data != nullptr;
    const Tensor<scalar_t, 2> nothing{nullptr, {0, 0}};
    hipStream_t stream = current_stream();
    const size_t output_count = grad_output.shape[0] * grad_output.shape[1] * grad_output.shape[2];

    if (grad_grad_output.data != nullptr) {
        // (callers that may pass unsorted indices: the calls below put the edges in order)
        if (have_A && have_B && !accept_unsorted() &&
            launch_forward_of_two_pairs<scalar_t>(grad_grad_output, grad_grad_A, B, A.data, grad_grad_B.data, indices_output)) {
            // both terms in the sums of one launch
        } else if (have_A && have_B) {
            ::mops::cuda::outer_product_scatter_add<scalar_t>(grad_grad_output, grad_grad_A, B, indices_output);
            StreamTemporary<scalar_t> second(output_count, stream);
            ::mops::cuda::outer_product_scatter_add<scalar_t>(
                Tensor<scalar_t, 3>{second.data(), {grad_output.shape[0], grad_output.shape[1], grad_output.shape[2]}},
                A, grad_grad_B, indices_output
            );
            add_in_place<scalar_t>(grad_grad_output.data, second.data(), output_count, stream);
        } else if (have_B) {
            ::mops::cuda::outer_product_scatter_add<scalar_t>(grad_grad_output, A, grad_grad_B, indices_output);
        } else if (have_A) {
            ::mops::cuda::outer_product_scatter_add<scalar_t>(grad_grad_output, grad_grad_A, B, indices_output);
        } else {
            fill_zero<scalar_t>(grad_grad_output.data, output_count, stream);
        }
    }
    if (grad_A_2.data != nullptr && grad_B_2.data != nullptr && have_A && have_B) {
        // grad_A_2 is the vjp's grad_A with grad_grad_B for B, grad_B_2 its grad_B with
        // grad_grad_A for A, and neither gradient of the vjp reads its own tensor: one call
        ::mops::cuda::outer_product_scatter_add_vjp<scalar_t>(
            grad_A_2, grad_B_2, grad_output, grad_grad_A, grad_grad_B, indices_output
        );
        finish_call(operation);
        return;
    }
    if (grad_A_2.data != nullptr) {
        if (have_B) {
            ::mops::cuda::outer_product_scatter_add_vjp<scalar_t>(grad_A_2, nothing, grad_output, A, grad_grad_B, indices_output);
        } else {
            fill_zero<scalar_t>(grad_A_2.data, A.shape[0] * A.shape[1], stream);
        }
    }
    if (grad_B_2.data != nullptr) {
        if (have_A) {
            ::mops::cuda::outer_product_scatter_add_vjp<scalar_t>(nothing, grad_B_2, grad_output, grad_grad_A, B, indices_output);
        } else {
            fill_zero<scalar_t>(grad_B_2.data, B.shape[0] * B.shape[1], stream);
        }
    }
    finish_call(operation);
}

template <typename scalar_t>
void outer_product_scatter_add_with_weights(MOPS_OPSAW_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    const char* operation = "cuda_outer_product_scatter_add_with_weights";
    checks::Validator validator(operation);
    checks::opsaw(validator, output, A, B, W, indices_W, indices_output);
    if (amd::accept_unsorted() &&
        !amd::is_sorted_on_device(indices_output.data, amd::narrow_i32(A.shape[0], "A.shape[0]"), amd::current_stream())) {
        const amd::SortedEdges<scalar_t> sorted(A, B, indices_W.data, indices_output, false, false);
        ::mops::cuda::outer_product_scatter_add_with_weights<scalar_t>(
            output, sorted.A(), sorted.B(), W, sorted.second_index(), sorted.index()
        );
        return;
    }
    amd::validate_scatter_index(indices_output, output.shape[0], "indices_output", operation);
    amd::validate_gather_index(indices_W, output.shape[0], "indices_W", operation);
    amd::launch_forward<scalar_t, true>(output, A, B, W.data, indices_W.data, indices_output, operation);
}

template <typename scalar_t>
void outer_product_scatter_add_with_weights_vjp(MOPS_OPSAW_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    const char* operation = "cuda_outer_product_scatter_add_with_weights_vjp";
    checks::Validator validator(operation);
    checks::opsaw_vjp(validator, grad_A, grad_B, grad_W, grad_output, A, B, W, indices_W, indices_output);
    if (amd::accept_unsorted() &&
        !amd::is_sorted_on_device(indices_output.data, amd::narrow_i32(A.shape[0], "A.shape[0]"), amd::current_stream())) {
        const amd::SortedEdges<scalar_t> sorted(
            A, B, indices_W.data, indices_output, grad_A.data != nullptr, grad_B.data != nullptr
        );
        ::mops::cuda::outer_product_scatter_add_with_weights_vjp<scalar_t>(
            sorted.grad_A(), sorted.grad_B(), grad_W, grad_output, sorted.A(), sorted.B(), W,
            sorted.second_index(), sorted.index()
        );
        sorted.put_back(grad_A, grad_B);
        amd::finish_call(operation);
        return;
    }
    amd::validate_scatter_index(indices_output, grad_output.shape[0], "indices_output", operation);
    amd::validate_gather_index(indices_W, grad_output.shape[0], "indices_W", operation);
    amd::launch_vjp<scalar_t, true>(
        grad_A, grad_B, grad_W, grad_output, A, B, W.data, indices_W.data, indices_output, operation
    );
}

template <typename scalar_t>
void outer_product_scatter_add_with_weights_vjp_vjp(MOPS_OPSAW_VJP_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    // no double backward exists for this operation on any device
    // (mops/src/opsaw/cpu.tpp:133-150)
    throw std::runtime_error("Not implemented");
}

MOPS_CXX_INSTANTIATE(outer_product_scatter_add, MOPS_OPSA_PARAMS)
MOPS_CXX_INSTANTIATE(outer_product_scatter_add_vjp, MOPS_OPSA_VJP_PARAMS)
MOPS_CXX_INSTANTIATE(outer_product_scatter_add_vjp_vjp, MOPS_OPSA_VJP_VJP_PARAMS)
MOPS_CXX_INSTANTIATE(outer_product_scatter_add_with_weights, MOPS_OPSAW_PARAMS)
MOPS_CXX_INSTANTIATE(outer_product_scatter_add_with_weights_vjp, MOPS_OPSAW_VJP_PARAMS)
MOPS_CXX_INSTANTIATE(outer_product_scatter_add_with_weights_vjp_vjp, MOPS_OPSAW_VJP_VJP_PARAMS)

} // namespace mops::cuda
