// SASAW on the matrix cores of gfx950.
//
//   O[PO1[e], PO2[n], :] += C[n] * A[e, PA[n]] * B[e, :] * W[PW1[e], PW2[n], :]
//
// (semantics: mops/src/sasaw/cpu.tpp:8-171 of lab-cosmo/mops). For the table
// shapes of equivariant message passing every index of the coupling table has
// a handful of values, so the table is first made DENSE,
//
//   D[cell, m1] = sum of C[n] over entries with (PO2[n], PW2[n]) == cell, PA[n] == m1
//   (cell = m3 * n2 + m2),
//
// and everything else becomes small matrix products on v_mfma_*_16x16x4:
//
//   T[cell, e]     = sum_m1 D[cell, m1] * A[e, m1]                  16 edges at a time
//   O[i, m3, l]    = sum_e sum_m2 T[(m3, m2), e] * (B[e, l] * W[PW1[e], m2, l])
//   grad_W[w,m2,l] = sum_e sum_m3 T[(m3, m2), e] * (B[e, l] * G[PO1[e], m3, l])
//   P_e[m3, l]     = sum_m2 T[(m3, m2), e] * W[PW1[e], m2, l];  grad_B[e, l] = sum_m3 G[i, m3, l] * P_e[m3, l]
//   U_e[m3, m2]    = sum_l G[i, m3, l] * (B[e, l] * W[PW1[e], m2, l])
//   grad_A[e, m1]  = sum_cell U_e[cell] * D[cell, m1]              16 edges at a time
//
// The forward pass and grad_W are the same contraction with the roles of m2
// and m3 exchanged, and share their code.
//
// The whole call lasts microseconds and every wavefront sees a few dozen
// edges, so what counts is (a) the number of instructions around every matrix
// instruction and (b) that no wavefront has much more to do than the others:
//  - everything that depends only on the lane is computed once per kernel
//    (byte offsets into blocks, LDS rows); addresses are a uniform base in
//    scalar registers plus one of those offsets plus an immediate;
//  - operand arrays are padded with zeros up to fixed loop bounds instead of
//    being guarded (a matrix instruction on zeros costs what a branch costs);
//  - forward: a workgroup of four wavefronts owns the receiver segments that
//    start in its 64 positions of the sorted index and deals their 16-edge
//    stages out in turn; partial sums meet in LDS in a fixed order;
//  - grad_A / grad_B: one wavefront per 16 consecutive edges, whatever
//    segments they belong to;
//  - grad_W: one wavefront per sender, senders found by sender_gather.hpp.
// Sums never depend on the launch or on timing: no atomics anywhere.
//
// More than 64 feature channels are taken 64 at a time, one launch per block
// of columns (rows keep their distance in memory, `ld`): outputs, grad_B and
// grad_W are per column, and grad_A, a sum over the columns, is added to by
// the launches one after the other on the stream.
#include "sasaw_mfma.hpp"

#include <algorithm>
#include <stdexcept>
#include <type_traits>

#include "device_common.hpp"
#include "dispatch_thresholds.hpp"
#include "mfma.hpp"
#include "runtime.hpp"
#include "segment_walk.hpp"
#include "sender_buckets.hpp"
#include "sender_gather.hpp"

namespace mops::amd::sasaw_mfma {
namespace {

__host__ __device__ constexpr size_t align16(size_t bytes) { return (bytes + 15) & ~static_cast<size_t>(15); }

constexpr int STAGE = 16;      // edges per matrix tile
constexpr int MAX_A_STEPS = 4; // nA <= 16
constexpr int MAX_INDEX = 16;  // n2, n3 <= 16
constexpr int MAX_L = 64;
constexpr int T_ROW = STAGE + 1; // LDS row of one cell: 16 edges, one more to spread the banks
constexpr int TILE_GROUP = 3;    // tiles of 16 cells handled together
constexpr int STEP_GROUP = 8;    // steps of 4 cells handled together
constexpr size_t LDS_BUDGET = 150 * 1024; // of the 160 KB of a compute unit (beyond 64 KB a kernel has to ask)
constexpr size_t WEIGHT_LDS_BUDGET = 96 * 1024; // the weight-gradient kernel asks for more than 64 KB
constexpr size_t SENDER_SCAN_LIMIT = thresholds::SENDER_SCAN_LIMIT; // index reads of the in-kernel gather, all workgroups together

template <typename T>
__device__ __forceinline__ T load_at(const T* __restrict__ base, uint32_t byte_offset) {
    return *reinterpret_cast<const T*>(reinterpret_cast<const char*>(base) + byte_offset);
}

template <typename T>
__device__ __forceinline__ void store_at(T* __restrict__ base, uint32_t byte_offset, T value) {
    *reinterpret_cast<T*>(reinterpret_cast<char*>(base) + byte_offset) = value;
}

// ---------------------------------------------------------------------------
// the dense table, laid out as matrix operands and padded with zeros

struct DenseLayout {
    int32_t n_cells;
    int32_t n_cell_tiles; // tiles of 16 cells, a multiple of TILE_GROUP
    int32_t cell_steps;   // steps of 4 cells, a multiple of STEP_GROUP
    int32_t lds_cells;    // rows of the T area in LDS
    int32_t zero_cell;    // a row of it that stays zero
    int32_t dump_cell;    // a row of it nobody reads

    __host__ __device__ int32_t to_cells_slots() const { return n_cell_tiles * MAX_A_STEPS * WAVE; }
    __host__ __device__ int32_t to_A_slots() const { return cell_steps * WAVE; }
    __host__ __device__ int32_t t_elements() const { return lds_cells * T_ROW; }
};

int32_t round_up(int32_t value, int32_t multiple) { return (value + multiple - 1) / multiple * multiple; }

DenseLayout dense_layout(const Shape& s) {
    DenseLayout d;
    d.n_cells = s.n3 * s.n2;
    d.n_cell_tiles = round_up((d.n_cells + 15) / 16, TILE_GROUP);
    d.cell_steps = round_up((d.n_cells + 3) / 4, STEP_GROUP);
    const int32_t rows = std::max(16 * d.n_cell_tiles, 4 * d.cell_steps);
    d.zero_cell = rows;
    d.dump_cell = rows + 1;
    d.lds_cells = rows + 2;
    return d;
}

constexpr int DENSE_THREADS = 256;
constexpr int TABLE_TILE = 1024;

/// What the workgroups of dense_coupling_kernel from `first_block` on list
/// (nothing: first_block beyond the grid).
struct SlotListing {
    int32_t first_block;
    int32_t* edges;
    int32_t* counts;
    const int32_t* senders;
    int32_t n_edges, n_nodes;
    bool aligned;
};

// Every thread owns one operand slot and adds up, in ascending entry order,
// the coefficients of the entries that fall on it.
//   to_cells[(tile * MAX_A_STEPS + step) * 64 + lane] = D[16 * tile + (lane & 15)][4 * step + (lane >> 4)]
//   to_A[step * 64 + lane]                            = D[4 * step + (lane >> 4)][lane & 15]
template <typename T>
__global__ __launch_bounds__(DENSE_THREADS) void dense_coupling_kernel(
    T* __restrict__ to_cells,
    T* __restrict__ to_A,
    const T* __restrict__ C,
    const int32_t* __restrict__ PA,
    const int32_t* __restrict__ PW2,
    const int32_t* __restrict__ PO2,
    int32_t N,
    int32_t nA,
    int32_t n2,
    int32_t n3,
    DenseLayout layout,
    SlotListing listing
) {
    // Workgroups after the table's own list the edges of every sender in its
    // slots (sender_buckets.hpp) for the weight-gradient kernel of a vjp: the
    // pass over the sender index needs no launch of its own that way, and no
    // time of its own either (this launch is a few microseconds of latency).
    if (static_cast<int32_t>(blockIdx.x) >= listing.first_block) {
        __shared__ SlotLists lists;
        list_in_slots_block<DENSE_THREADS>(
            lists, listing.edges, listing.counts, listing.senders, listing.n_edges, listing.n_nodes,
            listing.aligned, static_cast<int32_t>(blockIdx.x) - listing.first_block
        );
        return;
    }
    __shared__ __align__(16) int32_t keys[TABLE_TILE];
    __shared__ __align__(16) T coefficients[TABLE_TILE];

    const int tid = threadIdx.x;
    const int32_t slot = blockIdx.x * DENSE_THREADS + tid;
    const int32_t n_to_cells = layout.to_cells_slots();
    const int32_t n_slots = n_to_cells + layout.to_A_slots();

    int32_t cell = -1;
    int32_t m1 = -1;
    if (slot < n_to_cells) {
        const int lane = slot & (WAVE - 1);
        const int32_t tile_step = slot >> 6;
        cell = 16 * (tile_step / MAX_A_STEPS) + (lane & 15);
        m1 = 4 * (tile_step % MAX_A_STEPS) + (lane >> 4);
    } else if (slot < n_slots) {
        const int32_t local = slot - n_to_cells;
        const int lane = local & (WAVE - 1);
        cell = 4 * (local >> 6) + (lane >> 4);
        m1 = lane & 15;
    }
    const int32_t key = (cell >= 0 && cell < layout.n_cells && m1 < nA) ? cell * nA + m1 : -2;

    T sum = T(0);
    for (int32_t base = 0; base < N; base += TABLE_TILE) {
        __syncthreads();
        for (int i = tid; i < TABLE_TILE; i += DENSE_THREADS) {
            const int32_t n = base + i;
            int32_t entry_key = -1;
            T coefficient = T(0);
            if (n < N) {
                const int32_t e1 = PA[n];
                const int32_t e2 = PW2[n];
                const int32_t e3 = PO2[n];
                if (in_bounds(e1, nA) && in_bounds(e2, n2) && in_bounds(e3, n3)) {
                    entry_key = (e3 * n2 + e2) * nA + e1;
                    coefficient = C[n];
                }
            }
            keys[i] = entry_key;
            coefficients[i] = coefficient;
        }
        __syncthreads();
        // entries beyond N hold key -1 and match nothing
        const int32_t count = (min(TABLE_TILE, N - base) + 7) & ~7;
        for (int32_t i0 = 0; i0 < count; i0 += 8) {
            // (all lanes read the same addresses: 16 bytes per LDS read)
            int32_t entry_key[8];
            T coefficient[8];
            constexpr int PER_READ = 16 / sizeof(T);
            typedef T Wide __attribute__((ext_vector_type(PER_READ)));
#pragma unroll
            for (int u = 0; u < 8; u += 4) {
                const int4 four = *reinterpret_cast<const int4*>(&keys[i0 + u]);
                entry_key[u] = four.x;
                entry_key[u + 1] = four.y;
                entry_key[u + 2] = four.z;
                entry_key[u + 3] = four.w;
            }
#pragma unroll
            for (int u = 0; u < 8; u += PER_READ) {
                const Wide some = *reinterpret_cast<const Wide*>(&coefficients[i0 + u]);
#pragma unroll
                for (int c = 0; c < PER_READ; c++) {
                    coefficient[u + c] = some[c];
                }
            }
#pragma unroll
            for (int u = 0; u < 8; u++) {
                sum += entry_key[u] == key ? coefficient[u] : T(0);
            }
        }
    }
    if (slot < n_to_cells) {
        to_cells[slot] = sum;
    } else if (slot < n_slots) {
        to_A[slot - n_to_cells] = sum;
    }
}

// ---------------------------------------------------------------------------
// pieces shared by the kernels

/// Row of A of the edge held by this lane's column (lane & 15), as right
/// operand of T = D * A^T; zeros without an edge (`my_edge` -1).
template <typename T>
__device__ __forceinline__ void load_A_rows(
    T (&a_rows)[MAX_A_STEPS], const T* __restrict__ A, int32_t my_edge, int lane, int32_t nA
) {
    const int q = lane >> 4;
#pragma unroll
    for (int s = 0; s < MAX_A_STEPS; s++) {
        const int32_t m1 = 4 * s + q;
        a_rows[s] = load_or_zero(A, static_cast<size_t>(my_edge) * nA + m1, my_edge >= 0 && m1 < nA);
    }
}

/// T[cell, k] = sum_m1 D[cell, m1] * A[edge_k, m1] for the (up to) 16 edges
/// whose rows of A are in `a_rows`, written to t_area[cell * T_ROW + k] for
/// every cell of the padded tiles.
template <typename T>
__device__ __forceinline__ void coupling_times_A(
    T* __restrict__ t_area,
    const T (&a_rows)[MAX_A_STEPS],
    const T* __restrict__ to_cells,
    int lane,
    int32_t n_cell_tiles
) {
    using M = Mfma<T>;
    const int k = lane & 15;
    T* my_rows = t_area + M::row(lane, 0) * T_ROW + k;
    const int row_step = (M::row(0, 1) - M::row(0, 0)) * T_ROW;
    for (int32_t tile0 = 0; tile0 < n_cell_tiles; tile0 += TILE_GROUP) {
        const T* group = to_cells + tile0 * MAX_A_STEPS * WAVE + lane;
        T d[TILE_GROUP][MAX_A_STEPS];
#pragma unroll
        for (int g = 0; g < TILE_GROUP; g++) {
#pragma unroll
            for (int s = 0; s < MAX_A_STEPS; s++) {
                d[g][s] = group[(g * MAX_A_STEPS + s) * WAVE];
            }
        }
        T* rows = my_rows + tile0 * 16 * T_ROW;
#pragma unroll
        for (int g = 0; g < TILE_GROUP; g++) {
            typename M::Acc acc = M::zero();
#pragma unroll
            for (int s = 0; s < MAX_A_STEPS; s++) {
                acc = M::mma(d[g][s], a_rows[s], acc);
            }
#pragma unroll
            for (int r = 0; r < 4; r++) {
                rows[g * 16 * T_ROW + r * row_step] = acc[r];
            }
        }
    }
}

// out[o, l] += sum over the edges k of a batch and over c of
//   T[cell(o, c), k] * B[edge_k, l] * rows[source_k, c, l]
// (forward: o = m3, c = m2, rows = W, source = sender;
//  grad_W:  o = m2, c = m3, rows = grad_output, source = receiver).
template <typename T> struct Contraction {
    const T* A;    // [n_edges][nA]
    const T* B;    // [n_edges][ld], L columns of it
    const T* rows; // [n_blocks][n_red][ld], L columns of it
    const int32_t* gather_index; // block of `rows` of every edge
    const T* to_cells;
    DenseLayout layout;
    int32_t n_blocks, nA, L, n_out, n_red;
    int32_t ld; // distance between rows of B, of `rows` and of the result (>= L: L may be a block of columns)
    int32_t out_cell_stride, red_cell_stride; // cell = o * out_cell_stride + c * red_cell_stride
    bool vector_rows; // NT neighbouring elements of `rows` and of B may be loaded at once
};

/// What one lane needs to know for the whole kernel.
template <typename T, int NT, int RS> struct ContractionLane {
    uint32_t w_offset[RS][NT]; // bytes into a block of `rows`
    uint32_t a_offset[RS];     // bytes into the T area
    uint32_t b_offset[NT];     // bytes into a row of B

    __device__ __forceinline__ void setup(const Contraction<T>& p, int lane) {
        const int i = lane & 15;
        const int q = lane >> 4;
#pragma unroll
        for (int s = 0; s < RS; s++) {
            const int32_t c = 4 * s + q;
            const bool red_ok = c < p.n_red;
            // lanes without a term read zeros from T and some finite value from `rows`
            const int32_t cell =
                red_ok && i < p.n_out ? i * p.out_cell_stride + c * p.red_cell_stride : p.layout.zero_cell;
            a_offset[s] = cell * T_ROW * sizeof(T);
#pragma unroll
            for (int t = 0; t < NT; t++) {
                w_offset[s][t] = ((red_ok ? c : 0) * p.ld + column(p, i, t)) * sizeof(T);
            }
        }
#pragma unroll
        for (int t = 0; t < NT; t++) {
            b_offset[t] = column(p, i, t) * sizeof(T);
        }
    }

    /// Column l of the feature dimension that column i of matrix tile t stands
    /// for: l = NT * i + t, so that one lane's NT columns are neighbours in
    /// memory. Columns beyond L are redirected to existing ones (and never
    /// stored).
    static __device__ __forceinline__ int32_t column(const Contraction<T>& p, int i, int t) {
        if (p.vector_rows) {
            return min(NT * i, p.L - NT) + t;
        }
        return min(NT * i + t, p.L - 1);
    }
};

/// Two independent sets of accumulators, used in turn: consecutive matrix
/// instructions on one accumulator wait for each other.
template <typename T, int NT> struct Accumulators {
    typename Mfma<T>::Acc part[2][NT];

    __device__ __forceinline__ void clear() {
#pragma unroll
        for (int h = 0; h < 2; h++) {
#pragma unroll
            for (int t = 0; t < NT; t++) {
                part[h][t] = Mfma<T>::zero();
            }
        }
    }
    __device__ __forceinline__ T total(int t, int r) const { return part[0][t][r] + part[1][t][r]; }
};

/// One batch of n <= 16 edges (lane k, k + 16, ... hold edge k in `my_edge`
/// and its block of `rows` in `my_source`; both -1 beyond n).
/// The right operands of the matrix instructions come straight from global
/// memory, all edges of the batch in flight together, multiplied by the
/// edge's B row on the way; the left operands are the rows of T in LDS.
template <typename T, int NT, int RS>
__device__ __forceinline__ void contract_batch(
    Accumulators<T, NT>& out, const Contraction<T>& p, const ContractionLane<T, NT, RS>& mine,
    T* __restrict__ t_area, int32_t my_edge, int32_t my_source, int32_t n, int lane
) {
    using M = Mfma<T>;
    typedef T Vec __attribute__((ext_vector_type(NT)));
    // Edges whose operands are in flight together: a round trip to memory
    // costs about as much as the arithmetic of all 16 edges, so as many as
    // the registers hold (RS * NT + NT values per edge).
    constexpr int EB = 4 / (NT >= 4 ? 2 : 1);
    const uint32_t block_elements = static_cast<uint32_t>(p.n_red) * p.ld;
    // Nothing below is conditional: lanes 0..15 without an edge (or with a
    // source out of range) get a zero column of T, and their operand loads are
    // redirected to an edge that exists, so their products vanish.
    const bool usable = my_edge >= 0 && in_bounds(my_source, p.n_blocks);
    const int32_t edge_or_none = usable ? my_edge : -1;
    const int32_t fallback_edge = __builtin_amdgcn_readfirstlane(my_edge);
    const int32_t load_edge = usable ? my_edge : fallback_edge;
    const int32_t load_source = usable ? my_source : 0;

    struct Operands {
        Vec w[EB][RS];
        Vec scale[EB];
    };
    auto load_one = [&](Operands& to, int32_t k0, int u, auto vectors) {
        const int32_t k = min(k0 + u, STAGE - 1);
        const int32_t edge = __builtin_amdgcn_readlane(load_edge, k);
        const int32_t source = __builtin_amdgcn_readlane(load_source, k);
        const T* block = p.rows + static_cast<size_t>(source) * block_elements;
        const T* b_row = p.B + static_cast<size_t>(edge) * p.ld;
        if constexpr (decltype(vectors)::value) {
#pragma unroll
            for (int s = 0; s < RS; s++) {
                to.w[u][s] =
                    *reinterpret_cast<const Vec*>(reinterpret_cast<const char*>(block) + mine.w_offset[s][0]);
            }
            to.scale[u] =
                *reinterpret_cast<const Vec*>(reinterpret_cast<const char*>(b_row) + mine.b_offset[0]);
        } else {
#pragma unroll
            for (int t = 0; t < NT; t++) {
#pragma unroll
                for (int s = 0; s < RS; s++) {
                    to.w[u][s][t] = load_at(block, mine.w_offset[s][t]);
                }
                to.scale[u][t] = load_at(b_row, mine.b_offset[t]);
            }
        }
    };
    auto load = [&](Operands& to, int32_t k0) {
        if (p.vector_rows) {
#pragma unroll
            for (int u = 0; u < EB; u++) {
                load_one(to, k0, u, std::true_type{});
            }
        } else {
#pragma unroll
            for (int u = 0; u < EB; u++) {
                load_one(to, k0, u, std::false_type{});
            }
        }
    };
    auto multiply = [&](const Operands& from, int32_t k0) {
        uint32_t a_base[RS];
#pragma unroll
        for (int s = 0; s < RS; s++) {
            a_base[s] = mine.a_offset[s] + k0 * static_cast<uint32_t>(sizeof(T));
        }
#pragma unroll
        for (int u = 0; u < EB; u++) {
            T a[RS];
#pragma unroll
            for (int s = 0; s < RS; s++) {
                a[s] = load_at(t_area, a_base[s] + u * static_cast<uint32_t>(sizeof(T)));
            }
#pragma unroll
            for (int s = 0; s < RS; s++) {
                const Vec right = from.w[u][s] * from.scale[u];
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    out.part[u & 1][t] = M::mma(a[s], right[t], out.part[u & 1][t]);
                }
            }
        }
    };

    T a_rows[MAX_A_STEPS];
    load_A_rows<T>(a_rows, p.A, edge_or_none, lane, p.nA); // first in the queue: T needs them first
    Operands operands;
    load(operands, 0);
    wave_sync(); // earlier reads of the T area are over
    coupling_times_A<T>(t_area, a_rows, p.to_cells, lane, p.layout.n_cell_tiles);
    wave_sync();
    multiply(operands, 0);
    for (int32_t k0 = EB; k0 < n; k0 += EB) {
        load(operands, k0);
        multiply(operands, k0);
    }
}

/// Writes tile element (row, column i of tile t) to target[row * ld + NT * i + t].
template <typename T, int NT, typename Value>
__device__ __forceinline__ void store_block(
    T* __restrict__ target, Value&& value, int32_t n_out, int32_t L, int32_t ld, int lane
) {
    using M = Mfma<T>;
    const int i = lane & 15;
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int32_t row = M::row(lane, r);
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const int32_t col = NT * i + t;
            if (row < n_out && col < L) {
                target[row * ld + col] = value(t, r);
            }
        }
    }
}

/// The row of the T area that must hold zeros before the first use.
template <typename T>
__device__ __forceinline__ void clear_zero_row(T* __restrict__ t_area, const DenseLayout& layout, int lane) {
    if (lane < T_ROW) {
        t_area[layout.zero_cell * T_ROW + lane] = T(0);
    }
}

// ---------------------------------------------------------------------------
// forward pass

/// Wavefronts per workgroup (their T areas share 64 KB of LDS) ...
template <typename T> constexpr int forward_waves() { return 2; }
/// ... and positions of the sorted index per workgroup, 16 per wavefront.
/// (32 or 64: 64 when 32 would need more workgroups than the device holds at once)
constexpr int SHORT_CHUNK = 32;
constexpr int LONG_CHUNK = 64;
/// Workgroups of the forward kernel that are on the device together: 256 CUs, 3 wavefronts per SIMD.
constexpr int32_t FORWARD_RESIDENT_GROUPS = 256 * 6;

/// Segments whose partial sums wait in LDS before the wavefronts meet.
template <typename T> constexpr int round_segments() { return sizeof(T) == 4 ? 2 : 1; }

/// PERMUTED: position q of the sorted index stands for edge edge_of_position[q]
/// (grad_W of a large graph: the index is the sender of every edge, put in
/// order by sender_buckets.hpp); otherwise for edge q.
template <typename T, int NT, int RS, int FORWARD_CHUNK, bool PERMUTED>
__global__ __launch_bounds__(forward_waves<T>() * WAVE) void forward_kernel(
    T* __restrict__ output, const int32_t* __restrict__ receivers,
    const int32_t* __restrict__ edge_of_position, int32_t n_edges, const Contraction<T> p
) {
    constexpr int FORWARD_WAVES = forward_waves<T>();
    constexpr int ROUND_SEGMENTS = round_segments<T>();
    constexpr int TILE = NT * 4 * WAVE; // elements of one wavefront's partial sums
    extern __shared__ __align__(16) char lds_raw[];
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x >> 6;
    const int i = lane & 15;
    T* t_area = reinterpret_cast<T*>(lds_raw) + wave * p.layout.t_elements();
    // partial sums: [segment of the round][rank][NT][4][64]
    T* meeting = reinterpret_cast<T*>(lds_raw) + FORWARD_WAVES * p.layout.t_elements();
    const size_t row_elements = static_cast<size_t>(p.n_out) * p.ld;

    // the senders of this workgroup's positions, asked for before anything
    // is known about the segments
    const int32_t chunk_begin = blockIdx.x * FORWARD_CHUNK;
    const int32_t chunk_position = chunk_begin + lane;
    const bool chunk_valid = lane < FORWARD_CHUNK && chunk_position < n_edges;
    int32_t chunk_edge = chunk_valid ? chunk_position : -1;
    if constexpr (PERMUTED) {
        chunk_edge = chunk_valid ? edge_of_position[chunk_position] : -1;
    }
    const int32_t chunk_source = chunk_valid ? p.gather_index[chunk_edge] : -1;

    ContractionLane<T, NT, RS> mine;
    mine.setup(p, lane);
    clear_zero_row(t_area, p.layout, lane);

    int32_t stages_before = 0; // 16-edge stages dealt out so far, the same in every wavefront
    int32_t waiting = 0;       // segments of the current round
    int32_t waiting_node[ROUND_SEGMENTS];
    int32_t waiting_participants[ROUND_SEGMENTS];

    // All wavefronts meet; wavefront j adds up, in rank order, the partial
    // sums of the j-th waiting segment and writes its output row.
    auto meet = [&]() {
        __syncthreads();
#pragma unroll
        for (int segment = 0; segment < ROUND_SEGMENTS; segment++) {
            if (segment < waiting && (segment % FORWARD_WAVES) == wave) {
                const T* slots = meeting + segment * FORWARD_WAVES * TILE;
                T sum[NT][4];
#pragma unroll
                for (int t = 0; t < NT; t++) {
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        sum[t][r] = slots[(t * 4 + r) * WAVE + lane];
                    }
                }
                for (int32_t rank = 1; rank < waiting_participants[segment]; rank++) {
#pragma unroll
                    for (int t = 0; t < NT; t++) {
#pragma unroll
                        for (int r = 0; r < 4; r++) {
                            sum[t][r] += slots[rank * TILE + (t * 4 + r) * WAVE + lane];
                        }
                    }
                }
                store_block<T, NT>(
                    output + waiting_node[segment] * row_elements, [&](int t, int r) { return sum[t][r]; },
                    p.n_out, p.L, p.ld, lane
                );
            }
        }
        __syncthreads();
        waiting = 0;
    };

    walk_owned_segments<FORWARD_CHUNK>(
        receivers, n_edges, p.n_blocks, blockIdx.x,
        [&](int32_t node, int32_t first, int32_t last) {
            const int32_t n_stages = (last - first + STAGE - 1) / STAGE;
            Accumulators<T, NT> acc;
            acc.clear();
            // stage number `st` goes to wavefront (stages_before + st) % FORWARD_WAVES
            const int32_t rank = (wave - stages_before) & (FORWARD_WAVES - 1);
            for (int32_t st = rank; st < n_stages; st += FORWARD_WAVES) {
                const int32_t s0 = first + st * STAGE;
                const int32_t n = min(STAGE, last - s0);
                int32_t my_edge = i < n ? s0 + i : -1;
                const int32_t offset = s0 + i - chunk_begin; // >= 0: owned segments start in the chunk
                const bool at_hand = i < n && offset < FORWARD_CHUNK;
                int32_t my_source = __shfl(chunk_source, at_hand ? offset : 0);
                if constexpr (PERMUTED) {
                    const int32_t listed = __shfl(chunk_edge, at_hand ? offset : 0);
                    my_edge = at_hand ? listed : (i < n ? edge_of_position[s0 + i] : -1);
                }
                if (!at_hand) {
                    my_source = i < n ? p.gather_index[my_edge] : -1;
                }
                contract_batch<T, NT, RS>(acc, p, mine, t_area, my_edge, my_source, n, lane);
            }
            const int32_t participants = min(n_stages, FORWARD_WAVES);
            if (participants == 1) {
                if (rank == 0) {
                    store_block<T, NT>(
                        output + node * row_elements, [&](int t, int r) { return acc.total(t, r); }, p.n_out,
                        p.L, p.ld, lane
                    );
                }
            } else {
                if (rank < participants) {
                    T* slot = meeting + (waiting * FORWARD_WAVES + rank) * TILE;
#pragma unroll
                    for (int t = 0; t < NT; t++) {
#pragma unroll
                        for (int r = 0; r < 4; r++) {
                            slot[(t * 4 + r) * WAVE + lane] = acc.total(t, r);
                        }
                    }
                }
#pragma unroll
                for (int segment = 0; segment < ROUND_SEGMENTS; segment++) {
                    if (segment == waiting) {
                        waiting_node[segment] = node;
                        waiting_participants[segment] = participants;
                    }
                }
                waiting++;
                if (waiting == ROUND_SEGMENTS) {
                    meet();
                }
            }
            stages_before += n_stages;
        },
        [&](int32_t begin, int32_t end) {
            T* target = output + begin * row_elements;
            if (p.ld == p.L) {
                const size_t count = (end - begin) * row_elements;
                for (size_t at = threadIdx.x; at < count; at += FORWARD_WAVES * WAVE) {
                    target[at] = T(0);
                }
            } else {
                // a block of columns: row by row
                const int32_t rows = (end - begin) * p.n_out;
                for (int32_t row = 0; row < rows; row++) {
                    for (int32_t col = threadIdx.x; col < p.L; col += FORWARD_WAVES * WAVE) {
                        target[static_cast<size_t>(row) * p.ld + col] = T(0);
                    }
                }
            }
        }
    );
    if (waiting > 0) {
        meet();
    }
}

// ---------------------------------------------------------------------------
// grad_W: one wavefront per sender

/// Wavefronts (= senders) per workgroup.
template <typename T> constexpr int senders_per_group() { return 4; } // (8: 1 % faster at c4, twice the LDS)

/// grad_W of ONE sender by one wavefront, the sender's edges read from its
/// slots (sender_buckets.hpp; listed by workgroups of the launch that made the
/// dense table). `t_area`: this wavefront's T area in LDS.
template <typename T, int NT, int RS>
__device__ __forceinline__ void weight_gradient_of_sender(
    T* __restrict__ grad_W, const int32_t* __restrict__ senders, int32_t n_edges, const Contraction<T>& p,
    const int32_t* __restrict__ slot_edges, const int32_t* __restrict__ slot_counts, int32_t node,
    T* t_area, int lane
) {
    ContractionLane<T, NT, RS> mine_lane;
    mine_lane.setup(p, lane);
    clear_zero_row(t_area, p.layout, lane);
    Accumulators<T, NT> acc;
    acc.clear();
    auto on_stage = [&](int32_t my_edge, int32_t n) {
        const int32_t my_source = my_edge >= 0 ? p.gather_index[my_edge] : -1;
        contract_batch<T, NT, RS>(acc, p, mine_lane, t_area, my_edge, my_source, n, lane);
    };
    const int32_t* mine = slot_edges + static_cast<size_t>(node) * SLOT_CAPACITY;
    const int32_t first_half = mine[lane];
    const int32_t second_half = mine[lane + WAVE];
    static_assert(SLOT_PARTS == 4 && SLOT_CAPACITY == 2 * WAVE, "the four parts of a sender's places in two registers");
    const int4 part_counts = reinterpret_cast<const int4*>(slot_counts)[node];
    const int32_t c0 = __builtin_amdgcn_readfirstlane(part_counts.x);
    const int32_t c1 = __builtin_amdgcn_readfirstlane(part_counts.y);
    const int32_t c2 = __builtin_amdgcn_readfirstlane(part_counts.z);
    const int32_t c3 = __builtin_amdgcn_readfirstlane(part_counts.w);
    const int32_t count = c0 + c1 + c2 + c3;
    // lane p of `edges` holds edge p of n <= 64: handed on 16 at a time
    auto hand_on = [&](int32_t edges, int32_t n) {
        for (int32_t k0 = 0; k0 < n; k0 += STAGE) {
            const int32_t m = min(STAGE, n - k0);
            const int k = lane & (STAGE - 1);
            const int32_t edge = __shfl(edges, k0 + k);
            on_stage(k < m ? edge : -1, m);
        }
    };
    if (max(max(c0, c1), max(c2, c3)) <= SLOT_PART_CAPACITY) {
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
        hand_on(edge_at(lane), min(count, WAVE));
        if (count > WAVE) {
            hand_on(edge_at(lane + WAVE), count - WAVE);
        }
    } else {
        // more edges in a part than places (a hub of a sparse graph): this
        // wavefront reads the whole sender index itself
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
                hand_on(__builtin_amdgcn_ds_permute(place << 2, e), n);
            }
        }
    }
    store_block<T, NT>(
        grad_W + static_cast<size_t>(node) * p.n_out * p.ld, [&](int t, int r) { return acc.total(t, r); },
        p.n_out, p.L, p.ld, lane
    );
}

template <typename T, int NT, int RS>
__global__ __launch_bounds__(senders_per_group<T>() * WAVE) void weight_gradient_kernel(
    T* __restrict__ grad_W, const int32_t* __restrict__ senders, int32_t n_edges, bool aligned_senders,
    const Contraction<T> p, const int32_t* __restrict__ slot_edges, const int32_t* __restrict__ slot_counts
) {
    constexpr int SENDERS_PER_GROUP = senders_per_group<T>();
    using Gather = SenderGather<SENDERS_PER_GROUP>;
    extern __shared__ __align__(16) char lds_raw[];
    typename Gather::Storage& gather = *reinterpret_cast<typename Gather::Storage*>(lds_raw);
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x >> 6;
    T* t_area = reinterpret_cast<T*>(lds_raw + align16(sizeof(typename Gather::Storage))) +
                wave * p.layout.t_elements();
    const int32_t node0 = blockIdx.x * SENDERS_PER_GROUP;
    const int32_t node = node0 + wave;
    if (slot_edges != nullptr) {
        // the edges of every sender are listed already: a wavefront needs nobody else
        if (node < p.n_blocks) {
            weight_gradient_of_sender<T, NT, RS>(grad_W, senders, n_edges, p, slot_edges, slot_counts, node, t_area, lane);
        }
        return;
    }

    ContractionLane<T, NT, RS> mine;
    mine.setup(p, lane);
    clear_zero_row(t_area, p.layout, lane);
    Accumulators<T, NT> acc;
    acc.clear();
    auto on_stage = [&](int32_t my_edge, int32_t n) {
        const int32_t my_source = my_edge >= 0 ? p.gather_index[my_edge] : -1;
        contract_batch<T, NT, RS>(acc, p, mine, t_area, my_edge, my_source, n, lane);
    };
    if (aligned_senders) {
        Gather::template run<4>(gather, senders, n_edges, node0, p.n_blocks, on_stage);
    } else {
        Gather::template run<1>(gather, senders, n_edges, node0, p.n_blocks, on_stage);
    }
    if (node < p.n_blocks) {
        store_block<T, NT>(
            grad_W + static_cast<size_t>(node) * p.n_out * p.ld, [&](int t, int r) { return acc.total(t, r); },
            p.n_out, p.L, p.ld, lane
        );
    }
}

// ---------------------------------------------------------------------------
// grad_A and grad_B: one wavefront per 16 consecutive edges

template <typename T> struct EdgeGradArgs {
    T* grad_A; // may be null
    T* grad_B; // may be null
    const T* G; // grad_output [n_nodes][n3][ld]
    const T* A;
    const T* B;
    const T* W;
    const int32_t* receivers;
    const int32_t* senders;
    const T* to_cells;
    const T* to_A;
    DenseLayout layout;
    int32_t n_edges, n_nodes, nA, L, n2, n3;
    int32_t ld;        // distance between rows of B, W, grad_output, grad_B (>= L: L may be a block of columns)
    bool add_to_A;     // grad_A += (a later block of columns) instead of grad_A =
    int32_t Ls;        // LDS stride of one row of W and of B
    bool vector_loads; // W may be read 128 bits at a time
    FastDivisor by_items, by_lvec, by_L; // n2 * L / vec, L / vec, L
};

constexpr int EDGE_BATCH = 2; // edges whose W blocks are in LDS together (4: more LDS and registers
                              // per wavefront, 98 instead of 89 us for the whole vjp; 1: 112 us)

/// grad_W in the same launch (WITH_WEIGHTS): the workgroups after those of the
/// edges (16 edges each) are one sender each (weight_gradient_of_sender): the
/// short jobs last, where they fill the places the long ones leave as they end
/// (the other order: 74 instead of 70 us in f32, 132 instead of 122 in f64).
/// The two halves of a vjp do not depend on each other and both wait for
/// memory most of the time; as one launch they share the device without a
/// second stream (forking and joining streams costs about 10 us per call,
/// also as nodes of a graph).
template <typename T> struct WeightGradArgs {
    T* grad_W;
    Contraction<T> contraction;
    const int32_t* slot_edges;
    const int32_t* slot_counts;
    int32_t n_senders;
};

template <typename T, int NT, int M2S, bool WITH_WEIGHTS>
__global__ __launch_bounds__(WAVE) void edge_gradients_kernel(const EdgeGradArgs<T> p, const WeightGradArgs<T> w) {
    using M = Mfma<T>;
    constexpr int L_STEPS = 4 * NT;
    constexpr uint32_t ELEMENT = sizeof(T);
    extern __shared__ __align__(16) char lds_raw[];
    T* t_area = reinterpret_cast<T*>(lds_raw);   // T, then U, of the 16 edges
    T* w_lds = t_area + p.layout.t_elements();   // [EDGE_BATCH][n2][Ls]
    T* b_lds = w_lds + EDGE_BATCH * p.n2 * p.Ls; // [EDGE_BATCH][Ls]
    T* partial_lds = b_lds + EDGE_BATCH * p.Ls;  // [EDGE_BATCH][NT][64]
    const int32_t lds_elements = p.layout.t_elements() + EDGE_BATCH * (p.n2 + 1) * p.Ls;

    const int lane = threadIdx.x;
    if constexpr (WITH_WEIGHTS) {
        // (M2S steps of four cover n3 as well as n2 here: the host sees to it)
        const int32_t edge_blocks = (p.n_edges + STAGE - 1) / STAGE;
        if (static_cast<int32_t>(blockIdx.x) >= edge_blocks) {
            weight_gradient_of_sender<T, NT, M2S>(
                w.grad_W, p.senders, p.n_edges, w.contraction, w.slot_edges, w.slot_counts,
                static_cast<int32_t>(blockIdx.x) - edge_blocks, t_area, lane
            );
            return;
        }
    }
    const int i = lane & 15;
    const int q = lane >> 4;
    const bool want_A = p.grad_A != nullptr;
    const bool want_B = p.grad_B != nullptr;

    const int32_t chunk_begin = static_cast<int32_t>(blockIdx.x) * STAGE;
    const int32_t n = min(STAGE, p.n_edges - chunk_begin);
    const int32_t my_edge = i < n ? chunk_begin + i : -1;
    const int32_t my_source = my_edge >= 0 ? p.senders[my_edge] : -1;
    const int32_t my_node = my_edge >= 0 ? p.receivers[my_edge] : -1;

    // padding of the LDS arrays is read (and multiplied by zeros): make it finite
    for (int32_t at = lane; at < lds_elements; at += WAVE) {
        t_area[at] = T(0);
    }

    // ---- what depends on the lane only
    // left operand rows of T for P = T_e * W_e: lane (m3 = i, m2 = 4 s + q)
    uint32_t t_offset[M2S];
    // right operand W_e[m2 = 4 s + q][l = 16 t + i], t as immediate
    uint32_t w_by_column[EDGE_BATCH][M2S];
#pragma unroll
    for (int s = 0; s < M2S; s++) {
        const int32_t m2 = 4 * s + q;
        const bool ok = m2 < p.n2;
        t_offset[s] = (ok && i < p.n3 ? i * p.n2 + m2 : p.layout.zero_cell) * T_ROW * ELEMENT;
#pragma unroll
        for (int kw = 0; kw < EDGE_BATCH; kw++) {
            w_by_column[kw][s] = ((kw * p.n2 + (ok ? m2 : 0)) * p.Ls + i) * ELEMENT;
        }
    }
    // right operand of U = G * Z^T: lane (m2 = i, l = 4 s + q), s as immediate
    uint32_t w_by_row[EDGE_BATCH];
    uint32_t b_by_row[EDGE_BATCH];
#pragma unroll
    for (int kw = 0; kw < EDGE_BATCH; kw++) {
        w_by_row[kw] = ((kw * p.n2 + (i < p.n2 ? i : 0)) * p.Ls + q) * ELEMENT;
        b_by_row[kw] = (kw * p.Ls + q) * ELEMENT;
    }
    // where this lane's elements of U go: U[m3 = D row][m2 = i] of edge k
    uint32_t u_offset[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int32_t m3 = M::row(lane, r);
        u_offset[r] = (m3 < p.n3 && i < p.n2 ? m3 * p.n2 + i : p.layout.dump_cell) * T_ROW * ELEMENT;
    }
    // left operand of grad_A = U * D: lane (edge = i, cell = 4 step + q), step as immediate
    const uint32_t u_by_edge = (q * T_ROW + i) * ELEMENT;

    // W blocks on their way to LDS: 16-byte vectors in registers, asked for one
    // batch ahead so that a batch does not start with a round trip to memory
    typedef T Vec __attribute__((ext_vector_type(4)));
    constexpr int ROUND = 3;
    struct RowsOnTheWay {
        Vec loaded[ROUND];
        uint32_t where[ROUND];
        bool ok[ROUND];
    };
    const uint32_t items_per_edge = p.by_items.divisor;
    const uint32_t lvecs = p.by_lvec.divisor;
    const int32_t block_elements = p.n2 * p.ld;
    auto ask_for_rows = [&](RowsOnTheWay& to, int32_t k0, int32_t n_batch, uint32_t base) {
        const uint32_t total = static_cast<uint32_t>(n_batch) * items_per_edge;
#pragma unroll
        for (int u = 0; u < ROUND; u++) {
            const uint32_t item = base + u * WAVE + lane;
            to.ok[u] = item < total;
            const uint32_t safe = to.ok[u] ? item : 0;
            const uint32_t kw = p.by_items.divide(safe);
            const uint32_t rest = safe - kw * items_per_edge;
            const uint32_t row = p.by_lvec.divide(rest);
            const uint32_t lv = rest - row * lvecs;
            const int32_t source = __shfl(my_source, k0 + static_cast<int>(kw));
            const bool valid = to.ok[u] && in_bounds(source, p.n_nodes);
            const size_t from = valid ? static_cast<size_t>(source) * block_elements + row * p.ld + lv * 4 : 0;
            const Vec value = *reinterpret_cast<const Vec*>(p.W + from);
            to.loaded[u] = valid ? value : Vec(T(0));
            to.where[u] = (kw * p.n2 + row) * p.Ls + lv * 4;
        }
    };
    auto commit_rows = [&](const RowsOnTheWay& from) {
#pragma unroll
        for (int u = 0; u < ROUND; u++) {
            if (from.ok[u]) {
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    w_lds[from.where[u] + v] = from.loaded[u][v];
                }
            }
        }
    };
    RowsOnTheWay ahead;
    if (p.vector_loads) {
        ask_for_rows(ahead, 0, min(EDGE_BATCH, n), 0);
    }

    __syncthreads();
    if (want_B) {
        T a_rows[MAX_A_STEPS];
        load_A_rows<T>(a_rows, p.A, my_edge, lane, p.nA);
        coupling_times_A<T>(t_area, a_rows, p.to_cells, lane, p.layout.n_cell_tiles);
    }

    // G of the receiver of the current edge, as operands
    int32_t current_node = -1;
    T g_rows[NT][4];   // G[m3 = D row of this lane][l = column of this lane]
    T g_left[L_STEPS]; // lane (m3 = i, l = 4 s + q)
#pragma unroll
    for (int t = 0; t < NT; t++) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            g_rows[t][r] = T(0);
        }
    }
#pragma unroll
    for (int s = 0; s < L_STEPS; s++) {
        g_left[s] = T(0);
    }

    for (int32_t k0 = 0; k0 < n; k0 += EDGE_BATCH) {
        const int32_t n_batch = min(EDGE_BATCH, n - k0);
        __syncthreads(); // the previous batch is no longer read
        // ---- W blocks and B rows of the batch into LDS
        if (p.vector_loads) {
            // the first ROUND x 64 vectors of the batch were asked for one batch
            // ago; what a large block has beyond them is read now
            commit_rows(ahead);
            const uint32_t total = static_cast<uint32_t>(n_batch) * items_per_edge;
            for (uint32_t base = ROUND * WAVE; base < total; base += ROUND * WAVE) {
                RowsOnTheWay more;
                ask_for_rows(more, k0, n_batch, base);
                commit_rows(more);
            }
            if (k0 + EDGE_BATCH < n) {
                ask_for_rows(ahead, k0 + EDGE_BATCH, min(EDGE_BATCH, n - k0 - EDGE_BATCH), 0);
            }
        } else {
            const uint32_t total = static_cast<uint32_t>(n_batch) * items_per_edge;
            // all lanes stay in the loop: the shuffle reads lanes that would
            // otherwise have left it
            for (uint32_t base = 0; base < total; base += WAVE) {
                const uint32_t item = base + lane;
                const bool ok = item < total;
                const uint32_t safe = ok ? item : 0;
                const uint32_t kw = p.by_items.divide(safe);
                const uint32_t rest = safe - kw * items_per_edge;
                const uint32_t row = p.by_lvec.divide(rest);
                const uint32_t l = rest - row * lvecs;
                const int32_t source = __shfl(my_source, k0 + static_cast<int>(kw));
                const bool valid = ok && in_bounds(source, p.n_nodes);
                const T value =
                    load_or_zero(p.W, static_cast<size_t>(source) * block_elements + row * p.ld + l, valid);
                if (ok) {
                    w_lds[(kw * p.n2 + row) * p.Ls + l] = value;
                }
            }
        }
        {
            const T* from = p.B + static_cast<size_t>(chunk_begin + k0) * p.ld;
            const uint32_t count = static_cast<uint32_t>(n_batch) * p.L;
            for (uint32_t at = lane; at < count; at += WAVE) {
                const uint32_t kw = p.by_L.divide(at);
                b_lds[kw * p.Ls + (at - kw * p.L)] = from[kw * p.ld + (at - kw * p.L)];
            }
        }
        __syncthreads();

        const uint32_t first_column = k0 * ELEMENT;
#pragma unroll
        for (int kw = 0; kw < EDGE_BATCH; kw++) {
            if (kw >= n_batch) {
                continue;
            }
            const int32_t node = __builtin_amdgcn_readlane(my_node, min(k0 + kw, STAGE - 1));
            if (node != current_node) {
                current_node = node;
                const bool valid = in_bounds(node, p.n_nodes);
                const T* g_block = p.G + static_cast<size_t>(valid ? node : 0) * p.n3 * p.ld;
#pragma unroll
                for (int t = 0; t < NT; t++) {
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const int32_t m3 = M::row(lane, r);
                        const int32_t col = 16 * t + i;
                        g_rows[t][r] = load_or_zero(g_block, m3 * p.ld + col, valid && m3 < p.n3 && col < p.L);
                    }
                }
#pragma unroll
                for (int s = 0; s < L_STEPS; s++) {
                    const int32_t l = 4 * s + q;
                    g_left[s] = load_or_zero(g_block, i * p.ld + l, valid && i < p.n3 && l < p.L);
                }
            }
            const uint32_t column = first_column + kw * ELEMENT;
            if (want_B) {
                // P[m3, l] = sum_m2 T[(m3, m2), k] * W[m2, l]; grad_B[l] = sum_m3 G[m3, l] P[m3, l]
                typename M::Acc product[NT];
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    product[t] = M::zero();
                }
#pragma unroll
                for (int s = 0; s < M2S; s++) {
                    const T left = load_at(t_area, t_offset[s] + column);
#pragma unroll
                    for (int t = 0; t < NT; t++) {
                        const T right = load_at(w_lds, w_by_column[kw][s] + t * 16 * ELEMENT);
                        product[t] = M::mma(left, right, product[t]);
                    }
                }
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    T partial = T(0);
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        partial += product[t][r] * g_rows[t][r];
                    }
                    partial_lds[(kw * NT + t) * WAVE + lane] = partial;
                }
            }
            if (want_A) {
                // U[m3, m2] = sum_l G[m3, l] * B[k, l] * W[m2, l]
                typename M::Acc even = M::zero();
                typename M::Acc odd = M::zero();
#pragma unroll
                for (int s = 0; s < L_STEPS; s += 2) {
                    const T z0 = load_at(w_lds, w_by_row[kw] + s * 4 * ELEMENT) *
                                 load_at(b_lds, b_by_row[kw] + s * 4 * ELEMENT);
                    const T z1 = load_at(w_lds, w_by_row[kw] + (s + 1) * 4 * ELEMENT) *
                                 load_at(b_lds, b_by_row[kw] + (s + 1) * 4 * ELEMENT);
                    even = M::mma(g_left[s], z0, even);
                    odd = M::mma(g_left[s + 1], z1, odd);
                }
                // T of this edge is no longer needed: its column takes U
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    store_at(t_area, u_offset[r] + column, even[r] + odd[r]);
                }
            }
        }
        if (want_B) {
            __syncthreads();
            // the four quarters of the wavefront finish one edge each
#pragma unroll
            for (int t = 0; t < NT; t++) {
                T sum = T(0);
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    sum += partial_lds[(q * NT + t) * WAVE + g * 16 + i];
                }
                const int32_t col = 16 * t + i;
                if (q < n_batch && col < p.L) {
                    p.grad_B[static_cast<size_t>(chunk_begin + k0 + q) * p.ld + col] = sum;
                }
            }
        }
    }

    if (want_A) {
        __syncthreads();
        // grad_A[k, m1] = sum_cell U[k, cell] * D[cell, m1]
        typename M::Acc even = M::zero();
        typename M::Acc odd = M::zero();
        const T* table = p.to_A + lane;
        for (int32_t step0 = 0; step0 < p.layout.cell_steps; step0 += STEP_GROUP) {
            T left[STEP_GROUP];
            T right[STEP_GROUP];
            const uint32_t at = u_by_edge + step0 * 4 * T_ROW * ELEMENT;
#pragma unroll
            for (int u = 0; u < STEP_GROUP; u++) {
                left[u] = load_at(t_area, at + u * 4 * T_ROW * ELEMENT);
                right[u] = table[(step0 + u) * WAVE];
            }
#pragma unroll
            for (int u = 0; u < STEP_GROUP; u += 2) {
                even = M::mma(left[u], right[u], even);
                odd = M::mma(left[u + 1], right[u + 1], odd);
            }
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int32_t k = M::row(lane, r);
            if (k < n && i < p.nA) {
                T* target = p.grad_A + static_cast<size_t>(chunk_begin + k) * p.nA + i;
                const T before = p.add_to_A ? *target : T(0);
                *target = before + (even[r] + odd[r]);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// host side

template <typename T> struct DenseBuffers {
    T* to_cells;
    T* to_A;
};

size_t dense_bytes(const DenseLayout& layout, size_t element_size) {
    return align256(static_cast<size_t>(layout.to_cells_slots()) * element_size) +
           align256(static_cast<size_t>(layout.to_A_slots()) * element_size);
}

template <typename T>
DenseBuffers<T> enqueue_dense(
    void* workspace, const DenseLayout& layout, const T* C, const Indices& indices, const Shape& s,
    hipStream_t stream, const SenderSlots* slots_wanted = nullptr
) {
    DenseBuffers<T> buffers;
    char* base = static_cast<char*>(workspace);
    buffers.to_cells = reinterpret_cast<T*>(base);
    buffers.to_A = reinterpret_cast<T*>(base + align256(static_cast<size_t>(layout.to_cells_slots()) * sizeof(T)));
    const int32_t slots = layout.to_cells_slots() + layout.to_A_slots();
    const int32_t dense_blocks = (slots + DENSE_THREADS - 1) / DENSE_THREADS;
    SlotListing listing{};
    listing.first_block = dense_blocks;
    unsigned listing_blocks = 0;
    if (slots_wanted != nullptr) {
        listing.edges = const_cast<int32_t*>(slots_wanted->edges);
        listing.counts = const_cast<int32_t*>(slots_wanted->counts);
        listing.senders = indices.W_1;
        listing.n_edges = s.n_edges;
        listing.n_nodes = s.n_nodes;
        listing.aligned = reinterpret_cast<uintptr_t>(indices.W_1) % 16 == 0;
        listing_blocks = sender_slots_blocks(s.n_nodes);
    }
    dense_coupling_kernel<T><<<dense_blocks + listing_blocks, DENSE_THREADS, 0, stream>>>(
        buffers.to_cells, buffers.to_A, C, indices.A, indices.W_2, indices.output_2, s.N, s.nA, s.n2, s.n3,
        layout, listing
    );
    MOPS_HIP_CHECK(hipGetLastError());
    return buffers;
}

int tiles_for(int32_t L) { return L <= 32 ? 2 : 4; }

size_t t_area_bytes(const Shape& s, size_t element_size) {
    return static_cast<size_t>(dense_layout(s).t_elements()) * element_size;
}

size_t forward_lds(const Shape& s, size_t element_size) {
    const size_t waves = element_size == 4 ? forward_waves<float>() : forward_waves<double>();
    return waves * t_area_bytes(s, element_size) +
           (element_size == 4 ? round_segments<float>() : round_segments<double>()) * waves * tiles_for(s.L) * 4 *
               WAVE * element_size;
}

size_t weight_gradient_lds(const Shape& s, size_t element_size) {
    return element_size == 4
               ? align16(sizeof(SenderGather<senders_per_group<float>()>::Storage)) +
                     senders_per_group<float>() * t_area_bytes(s, element_size)
               : align16(sizeof(SenderGather<senders_per_group<double>()>::Storage)) +
                     senders_per_group<double>() * t_area_bytes(s, element_size);
}

/// Rows of W in LDS: at least the 16 * NT columns the operands touch, and two
/// more so that lanes walking down a column of 4-byte elements spread over
/// the banks.
int32_t weight_row_stride(const Shape& s) { return 16 * tiles_for(s.L) + 2; }

size_t edge_gradients_lds(const Shape& s, size_t element_size) {
    return t_area_bytes(s, element_size) +
           (static_cast<size_t>(EDGE_BATCH) * (s.n2 + 1) * weight_row_stride(s) +
            static_cast<size_t>(EDGE_BATCH) * tiles_for(s.L) * WAVE) *
               element_size;
}

bool aligned_for_vectors(const void* pointer, size_t element_size) {
    return reinterpret_cast<uintptr_t>(pointer) % (4 * element_size) == 0;
}

template <typename T>
Contraction<T> contraction(
    const T* A, const T* B, const T* rows, const int32_t* gather_index, const T* to_cells,
    const DenseLayout& layout, const Shape& s, int32_t ld, int32_t n_out, int32_t n_red,
    int32_t out_cell_stride, int32_t red_cell_stride
) {
    Contraction<T> c{};
    c.A = A;
    c.B = B;
    c.rows = rows;
    c.gather_index = gather_index;
    c.to_cells = to_cells;
    c.layout = layout;
    c.n_blocks = s.n_nodes;
    c.nA = s.nA;
    c.L = s.L;
    c.ld = ld;
    c.n_out = n_out;
    c.n_red = n_red;
    c.out_cell_stride = out_cell_stride;
    c.red_cell_stride = red_cell_stride;
    const size_t vector_bytes = tiles_for(s.L) * sizeof(T);
    c.vector_rows = s.L % tiles_for(s.L) == 0 && ld % tiles_for(s.L) == 0 &&
                    reinterpret_cast<uintptr_t>(rows) % vector_bytes == 0 &&
                    reinterpret_cast<uintptr_t>(B) % vector_bytes == 0;
    return c;
}

/// A kernel that wants more than 64 KB of dynamic LDS has to say so first.
template <typename Kernel> void allow_lds(Kernel kernel, size_t bytes) {
    if (bytes > 64 * 1024) {
        MOPS_HIP_CHECK(hipFuncSetAttribute(
            reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
            static_cast<int>(bytes)
        ));
    }
}

/// Calls `launch(tiles, steps)` with the two shape parameters the kernels are
/// compiled for as integral constants.
template <typename Launch> void with_shape_constants(int tiles, int steps, Launch&& launch) {
    auto with_steps = [&](auto tiles_constant) {
        switch (steps) {
        case 1:
            launch(tiles_constant, std::integral_constant<int, 1>{});
            break;
        case 2:
            launch(tiles_constant, std::integral_constant<int, 2>{});
            break;
        case 3:
            launch(tiles_constant, std::integral_constant<int, 3>{});
            break;
        default:
            launch(tiles_constant, std::integral_constant<int, 4>{});
            break;
        }
    };
    if (tiles == 2) {
        with_steps(std::integral_constant<int, 2>{});
    } else {
        with_steps(std::integral_constant<int, 4>{});
    }
}

/// Feature channels beyond MAX_L are taken MAX_L at a time: `pass(first_column, shape)`
/// is called with the shape narrowed to one such block of columns.
template <typename Pass> void for_each_column_block(const Shape& s, Pass&& pass) {
    for (int32_t first = 0; first < s.L; first += MAX_L) {
        Shape block = s;
        block.L = std::min<int32_t>(MAX_L, s.L - first);
        pass(first, block);
    }
}

Shape widest_block(const Shape& s) {
    Shape block = s;
    block.L = std::min<int32_t>(MAX_L, s.L);
    return block;
}

} // namespace

bool supports(const Shape& full, size_t element_size) {
    const Shape s = widest_block(full);
    if (s.n_nodes < 1 || s.n_edges < 1 || s.N < 1) {
        return false;
    }
    if (s.nA < 1 || s.nA > 4 * MAX_A_STEPS || s.n2 < 1 || s.n2 > MAX_INDEX || s.n3 < 1 ||
        s.n3 > MAX_INDEX || s.L < 1) {
        return false;
    }
    // (the weight-gradient kernel has the forward kernel to fall back on)
    return forward_lds(s, element_size) <= LDS_BUDGET && edge_gradients_lds(s, element_size) <= LDS_BUDGET;
}

/// grad_W: whether the edges are first put in the order of their senders
/// (sender_buckets.hpp) and walked like the forward pass walks the receivers.
/// Otherwise every workgroup finds the edges of its senders by reading the
/// whole sender index (sender_gather.hpp): no preparation, which is what a
/// small graph wants, but edges x workgroups reads.
bool orders_edges_by_sender(const Shape& s, size_t element_size) {
    const size_t groups = (static_cast<size_t>(s.n_nodes) + senders_per_group<float>() - 1) / senders_per_group<float>();
    return static_cast<size_t>(s.n_edges) * groups > SENDER_SCAN_LIMIT ||
           weight_gradient_lds(widest_block(s), element_size) > WEIGHT_LDS_BUDGET;
}

/// Sparse graphs that take the in-kernel path: the edges of every sender are
/// listed in slots (sender_buckets.hpp) beside the dense table, and the
/// weight-gradient kernel reads the lists instead of the whole index.
constexpr int32_t SLOT_MEAN_LIMIT = thresholds::SLOT_MEAN_EDGES; // edges per sender on average (a part of the index then holds 12 of them, 32 fit)
bool lists_edges_in_slots(const Shape& s) {
    return s.n_nodes > 0 && static_cast<size_t>(s.n_edges) <= static_cast<size_t>(s.n_nodes) * SLOT_MEAN_LIMIT;
}

size_t workspace_bytes(const Shape& s, size_t element_size) {
    return align256(dense_bytes(dense_layout(s), element_size)) +
           (orders_edges_by_sender(s, element_size) ? edges_by_sender_bytes(s.n_nodes, s.n_edges)
            : lists_edges_in_slots(s)               ? sender_slots_bytes(s.n_nodes)
                                                    : 0);
}

bool vjp_allocates_nothing(const Shape& s, size_t element_size, bool want_edge_gradients, bool want_grad_W) {
    if (!want_grad_W) {
        return true; // the edge-gradient launch alone
    }
    if (orders_edges_by_sender(s, element_size)) {
        return false; // the counting sort of a large graph
    }
    if (want_edge_gradients) {
        // one launch for all three gradients; otherwise grad_W runs beside the others on a second stream
        return lists_edges_in_slots(s) && (s.n2 + 3) / 4 == (s.n3 + 3) / 4;
    }
    return true;
}

template <typename T>
void forward(
    T* output, const T* A, const T* B, const T* C, const T* W, const Indices& indices,
    const Shape& s, void* workspace, hipStream_t stream
) {
    const DenseLayout layout = dense_layout(s);
    const DenseBuffers<T> dense = enqueue_dense<T>(workspace, layout, C, indices, s, stream);
    // positions of the sorted index per workgroup: one stage per wavefront while all
    // workgroups still fit on the device together, else two
    const bool short_chunks = (s.n_edges + SHORT_CHUNK - 1) / SHORT_CHUNK <= FORWARD_RESIDENT_GROUPS;
    const int32_t chunk = short_chunks ? SHORT_CHUNK : LONG_CHUNK;
    const int32_t grid = (s.n_edges + chunk - 1) / chunk;
    for_each_column_block(s, [&](int32_t first, const Shape& block) {
        const Contraction<T> c = contraction<T>(
            A, B + first, W + first, indices.W_1, dense.to_cells, layout, block, s.L, s.n3, s.n2, s.n2, 1
        );
        const size_t lds = forward_lds(block, sizeof(T));
        T* target = output + first;
        MainKernelTimer timer(stream);
        with_shape_constants(tiles_for(block.L), (s.n2 + 3) / 4, [&](auto tiles, auto steps) {
            if (short_chunks) {
                auto kernel = forward_kernel<T, decltype(tiles)::value, decltype(steps)::value, SHORT_CHUNK, false>;
                allow_lds(kernel, lds);
                kernel<<<grid, forward_waves<T>() * WAVE, lds, stream>>>(
                    target, indices.output_1, nullptr, s.n_edges, c
                );
            } else {
                auto kernel = forward_kernel<T, decltype(tiles)::value, decltype(steps)::value, LONG_CHUNK, false>;
                allow_lds(kernel, lds);
                kernel<<<grid, forward_waves<T>() * WAVE, lds, stream>>>(
                    target, indices.output_1, nullptr, s.n_edges, c
                );
            }
        });
        MOPS_HIP_CHECK(hipGetLastError());
    });
}

template <typename T>
void vjp(
    T* grad_A, T* grad_B, T* grad_W, const T* grad_output, const T* A, const T* B, const T* C,
    const T* W, const Indices& indices, const Shape& s, void* workspace, hipStream_t stream
) {
    const DenseLayout layout = dense_layout(s);
    const bool want_edges = grad_A != nullptr || grad_B != nullptr;
    const bool by_sender = grad_W != nullptr && orders_edges_by_sender(s, sizeof(T));
    void* order_workspace = static_cast<char*>(workspace) + align256(dense_bytes(layout, sizeof(T)));
    const bool slotted = grad_W != nullptr && !by_sender && lists_edges_in_slots(s);
    const SenderSlots slots = slotted ? sender_slots_in(order_workspace, s.n_nodes) : SenderSlots{nullptr, nullptr};
    const DenseBuffers<T> dense = enqueue_dense<T>(workspace, layout, C, indices, s, stream, slotted ? &slots : nullptr);

    // large graphs: the forward kernel over the edges in the order of their senders
    auto launch_ordered_weights = [&](hipStream_t on, const EdgesBySender& order, int32_t first, const Shape& block) {
        const Contraction<T> c = contraction<T>(
            A, B + first, grad_output + first, indices.output_1, dense.to_cells, layout, block, s.L, s.n2,
            s.n3, 1, s.n2
        );
        const int32_t grid = (s.n_edges + LONG_CHUNK - 1) / LONG_CHUNK;
        const size_t lds = forward_lds(block, sizeof(T));
        with_shape_constants(tiles_for(block.L), (s.n3 + 3) / 4, [&](auto tiles, auto steps) {
            auto kernel = forward_kernel<T, decltype(tiles)::value, decltype(steps)::value, LONG_CHUNK, true>;
            allow_lds(kernel, lds);
            kernel<<<grid, forward_waves<T>() * WAVE, lds, on>>>(
                grad_W + first, order.sender, order.edge, s.n_edges, c
            );
        });
        MOPS_HIP_CHECK(hipGetLastError());
    };

    auto launch_weights = [&](hipStream_t on, int32_t first, const Shape& block) {
        const Contraction<T> c = contraction<T>(
            A, B + first, grad_output + first, indices.output_1, dense.to_cells, layout, block, s.L, s.n2,
            s.n3, 1, s.n2
        );
        constexpr int SENDERS_PER_GROUP = senders_per_group<T>();
        const int32_t grid = (s.n_nodes + SENDERS_PER_GROUP - 1) / SENDERS_PER_GROUP;
        const size_t lds = weight_gradient_lds(block, sizeof(T));
        const bool aligned = aligned_for_vectors(indices.W_1, sizeof(int32_t));
        with_shape_constants(tiles_for(block.L), (s.n3 + 3) / 4, [&](auto tiles_constant, auto steps) {
            auto kernel = weight_gradient_kernel<T, decltype(tiles_constant)::value, decltype(steps)::value>;
            if (lds > 64 * 1024) {
                MOPS_HIP_CHECK(hipFuncSetAttribute(
                    reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                    static_cast<int>(lds)
                ));
            }
            kernel<<<grid, SENDERS_PER_GROUP * WAVE, lds, on>>>(
                grad_W + first, indices.W_1, s.n_edges, aligned, c, slots.edges, slots.counts
            );
        });
        MOPS_HIP_CHECK(hipGetLastError());
    };

    // with_weights: grad_W of this block of columns in the same launch (needs the slots)
    auto launch_edges = [&](int32_t first, const Shape& block, bool with_weights) {
        const bool vectors = block.L % 4 == 0 && s.L % 4 == 0 && aligned_for_vectors(W + first, sizeof(T));
        const int vec = vectors ? 4 : 1;
        EdgeGradArgs<T> args{};
        args.grad_A = grad_A;
        args.add_to_A = first > 0; // the sums over the columns of the blocks follow each other on the stream
        args.grad_B = grad_B != nullptr ? grad_B + first : nullptr;
        args.G = grad_output + first;
        args.A = A;
        args.B = B + first;
        args.W = W + first;
        args.receivers = indices.output_1;
        args.senders = indices.W_1;
        args.to_cells = dense.to_cells;
        args.to_A = dense.to_A;
        args.layout = layout;
        args.n_edges = s.n_edges;
        args.n_nodes = s.n_nodes;
        args.nA = s.nA;
        args.L = block.L;
        args.ld = s.L;
        args.n2 = s.n2;
        args.n3 = s.n3;
        args.Ls = weight_row_stride(block);
        args.vector_loads = vectors;
        args.by_items = FastDivisor::make(s.n2 * block.L / vec);
        args.by_lvec = FastDivisor::make(block.L / vec);
        args.by_L = FastDivisor::make(block.L);
        WeightGradArgs<T> weights{};
        if (with_weights) {
            weights.grad_W = grad_W + first;
            weights.contraction = contraction<T>(
                A, B + first, grad_output + first, indices.output_1, dense.to_cells, layout, block, s.L, s.n2,
                s.n3, 1, s.n2
            );
            weights.slot_edges = slots.edges;
            weights.slot_counts = slots.counts;
            weights.n_senders = s.n_nodes;
        }
        const int32_t grid = (s.n_edges + STAGE - 1) / STAGE + weights.n_senders;
        const size_t lds =
            std::max(edge_gradients_lds(block, sizeof(T)), with_weights ? t_area_bytes(block, sizeof(T)) : 0);
        MainKernelTimer timer(stream);
        with_shape_constants(tiles_for(block.L), (s.n2 + 3) / 4, [&](auto tiles_constant, auto steps) {
            if (with_weights) {
                auto kernel = edge_gradients_kernel<T, decltype(tiles_constant)::value, decltype(steps)::value, true>;
                allow_lds(kernel, lds);
                kernel<<<grid, WAVE, lds, stream>>>(args, weights);
            } else {
                auto kernel = edge_gradients_kernel<T, decltype(tiles_constant)::value, decltype(steps)::value, false>;
                allow_lds(kernel, lds);
                kernel<<<grid, WAVE, lds, stream>>>(args, weights);
            }
        });
        MOPS_HIP_CHECK(hipGetLastError());
    };

    if (want_edges && slotted && (s.n2 + 3) / 4 == (s.n3 + 3) / 4) {
        // sparse graphs: one launch for all three gradients
        for_each_column_block(s, [&](int32_t first, const Shape& block) { launch_edges(first, block, true); });
    } else if (want_edges && grad_W != nullptr) {
        // The two kernels are independent and both wait for memory most of
        // the time: they share the device, the weight kernel on a side stream
        // that forks from `stream` after the dense table and joins it again.
        // (weights first: the other order is slower, 109 instead of 97 us in f32)
        SideStream side(stream);
        EdgesBySender order{};
        if (by_sender) {
            order = order_edges_by_sender(indices.W_1, s.n_edges, s.n_nodes, order_workspace, side.get());
        }
        for_each_column_block(s, [&](int32_t first, const Shape& block) {
            if (by_sender) {
                launch_ordered_weights(side.get(), order, first, block);
            } else {
                launch_weights(side.get(), first, block);
            }
            launch_edges(first, block, false);
        });
    } else if (want_edges) {
        for_each_column_block(s, [&](int32_t first, const Shape& block) { launch_edges(first, block, false); });
    } else if (grad_W != nullptr) {
        EdgesBySender order{};
        if (by_sender) {
            order = order_edges_by_sender(indices.W_1, s.n_edges, s.n_nodes, order_workspace, stream);
        }
        for_each_column_block(s, [&](int32_t first, const Shape& block) {
            if (by_sender) {
                launch_ordered_weights(stream, order, first, block);
            } else {
                launch_weights(stream, first, block);
            }
        });
    }
}

template void forward<float>(
    float*, const float*, const float*, const float*, const float*, const Indices&, const Shape&, void*,
    hipStream_t
);
template void forward<double>(
    double*, const double*, const double*, const double*, const double*, const Indices&, const Shape&,
    void*, hipStream_t
);
template void vjp<float>(
    float*, float*, float*, const float*, const float*, const float*, const float*, const float*,
    const Indices&, const Shape&, void*, hipStream_t
);
template void vjp<double>(
    double*, double*, double*, const double*, const double*, const double*, const double*, const double*,
    const Indices&, const Shape&, void*, hipStream_t
);

} // namespace mops::amd::sasaw_mfma
