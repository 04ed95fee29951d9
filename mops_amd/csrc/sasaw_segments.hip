// SASAW as per-node sums of rank-one updates on the matrix cores of gfx950.
//
//   O[PO1[e], PO2[n], :] += C[n] * A[e, PA[n]] * B[e, :] * W[PW1[e], PW2[n], :]
//
// (semantics: mops/src/sasaw/cpu.tpp:8-171 of lab-cosmo/mops). With the table
// made dense, D[m3, m2, m1] = sum of C[n] over entries (PO2, PW2, PA)[n] ==
// (m3, m2, m1), the output row of node i is
//
//   Z_i[m1, m2, l] = sum over edges e of i of  A[e, m1] * (B[e, l] * W[PW1[e], m2, l])
//   O[i, m3, l]    = sum_{m1, m2} D[m3, m2, m1] * Z_i[m1, m2, l]
//
// The first line is a sum of outer products, one per edge: a matrix product
// whose reduction index is the EDGE, so a segment of the sorted receiver index
// is walked four edges per v_mfma_*_16x16x4 step with nothing to pad in that
// direction and nothing per edge but loads and multiplications; the second
// line is done once per node, on the accumulators as they lie in registers
// (the order of the components m1 in the rows of Z is chosen so that they do).
// No LDS round trip per edge, no dependent chain but index -> rows.
//
// grad_W is the same sum over the edges of a SENDER, with grad_output in the
// place of W and the roles of m2 and m3 exchanged:
//
//   grad_W[w, m2, l] = sum_{m1, m3} D[m3, m2, m1] * sum_{e: PW1[e] = w} A[e, m1] * (B[e, l] * G[PO1[e], m3, l])
//
// grad_A and grad_B: see edge_gradients below.
//
// The dense table is built by every workgroup for itself in LDS, in operand
// layout, entries of one cell added in ascending entry order (no launch of its
// own; it overlaps with the wait for the first rows). No atomics on floating
// point anywhere: two runs give the same bits.
#include "sasaw_segments.hpp"

#include <algorithm>
#include <atomic>
#include <stdexcept>
#include <type_traits>

#include "device_common.hpp"
#include "mfma.hpp"
#include "runtime.hpp"
#include "segment_walk.hpp"
#include "sender_buckets.hpp"

namespace mops::amd::sasaw_segments {
namespace {

constexpr int MAX_INDEX = 16;          // values of a component index
constexpr int ENTRIES_PER_LANE = 4;    // table entries a lane of the building wavefront handles at a time
constexpr int MAX_TABLE = 1 << 16;     // entries (more: the general kernels)

// ---------------------------------------------------------------------------
// the dense table in LDS
//
// For a contraction whose gathered blocks have `n_red` rows (m2 in the forward
// pass) and whose result has `n_out` rows (m3 in the forward pass):
//
//   table[(r * n_red + c) * 64 + 16 * q + o] = D[o, c, m1(q, r)]
//
// i.e. for every register r of an accumulator tile and every block row c, the
// left operand (lane = o + 16 q) of the product with that register. m1(q, r)
// is the component of A that row `Mfma<T>::row(16 q, r)` of the accumulators
// stands for.

/// Component of A in accumulator row `row` (0..15); >= nA: none. Rows whose
/// register number is beyond `registers` = ceil(nA / 4) hold nothing, so that
/// the second product needs `registers` steps per block row and not four.
template <typename T> __host__ __device__ __forceinline__ int32_t component_of_row(int row, int32_t registers) {
    if constexpr (sizeof(T) == 4) {
        const int q = row >> 2, r = row & 3; // row = 4 q + r
        return r < registers ? registers * q + r : 4 * MAX_INDEX;
    } else {
        return row; // row = 4 r + q
    }
}

/// (q, r) of component m1: inverse of the above.
template <typename T> __device__ __forceinline__ void place_of_component(int32_t m1, int32_t registers, int& q, int& r) {
    if constexpr (sizeof(T) == 4) {
        q = m1 / registers;
        r = m1 - q * registers;
    } else {
        r = m1 >> 2;
        q = m1 & 3;
    }
}

struct Table {
    const int32_t* PA;   // [N]
    const int32_t* Pred; // [N] index of the block row that is summed over (forward: PW2)
    const int32_t* Pout; // [N] index of the row of the result (forward: PO2)
    int32_t N, nA, n_red, n_out;
    int32_t registers; // ceil(nA / 4)

    __host__ __device__ int32_t slots() const { return registers * n_red * WAVE; }
};

constexpr int32_t NOBODY = 0x7fffffff;

/// Orders LDS traffic between the lanes of one wavefront.
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

/// Table entries `first` + lane + 64 k (k < ENTRIES_PER_LANE) of one lane, as
/// loaded (asked for at the start of a kernel, looked at when the table is built).
template <typename T> struct MyEntries {
    int32_t m1[ENTRIES_PER_LANE], c[ENTRIES_PER_LANE], o[ENTRIES_PER_LANE];
    T coefficient[ENTRIES_PER_LANE];
};

template <typename T>
__device__ __forceinline__ void load_entries(
    MyEntries<T>& mine, const T* __restrict__ C, const Table& t, int32_t first, int lane
) {
#pragma unroll
    for (int k = 0; k < ENTRIES_PER_LANE; k++) {
        const int32_t n = first + lane + k * WAVE;
        const int32_t safe = n < t.N ? n : 0;
        mine.m1[k] = t.PA[safe];
        mine.c[k] = t.Pred[safe];
        mine.o[k] = t.Pout[safe];
        mine.coefficient[k] = C[safe];
    }
}

/// The dense table, built by ONE wavefront (all 64 lanes call this): nothing
/// in it waits for another wavefront, so the others are free to ask for their
/// first rows meanwhile; they meet the builder at one barrier afterwards.
/// `owner` is an array of slots() integers. `mine`: load_entries(.., first = 0, ..).
template <typename T>
__device__ __forceinline__ void build_table(
    T* __restrict__ table, int32_t* __restrict__ owner, MyEntries<T>& mine, const T* __restrict__ C, const Table& t,
    int lane
) {
    const int32_t n_slots = t.slots();
    for (int32_t s = lane; s < n_slots; s += WAVE) {
        table[s] = T(0);
        owner[s] = NOBODY;
    }
    wave_sync();
    for (int32_t first = 0; first < t.N; first += WAVE * ENTRIES_PER_LANE) {
        if (first > 0) {
            load_entries<T>(mine, C, t, first, lane);
        }
        // where each entry goes (-1: nowhere; an entry outside the tensors is dropped)
        int32_t slot[ENTRIES_PER_LANE];
        uint32_t pending = 0;
#pragma unroll
        for (int k = 0; k < ENTRIES_PER_LANE; k++) {
            const int32_t n = first + lane + k * WAVE;
            const bool inside = n < t.N && in_bounds(mine.m1[k], t.nA) && in_bounds(mine.c[k], t.n_red) &&
                                in_bounds(mine.o[k], t.n_out);
            int q, r;
            place_of_component<T>(inside ? mine.m1[k] : 0, t.registers, q, r);
            slot[k] = inside ? (r * t.n_red + mine.c[k]) * WAVE + 16 * q + mine.o[k] : -1;
            pending |= inside ? 1u << k : 0u;
        }
        // Every round the smallest pending entry of each slot is added to it: the
        // entries of one slot in ascending order. (LDS operations of one
        // wavefront happen in program order.)
        while (__ballot(pending != 0) != 0) {
#pragma unroll
            for (int k = 0; k < ENTRIES_PER_LANE; k++) {
                if ((pending >> k) & 1u) {
                    atomicMin(&owner[slot[k]], first + lane + k * WAVE);
                }
            }
            wave_sync();
            uint32_t winners = 0;
#pragma unroll
            for (int k = 0; k < ENTRIES_PER_LANE; k++) {
                if (((pending >> k) & 1u) && owner[slot[k]] == first + lane + k * WAVE) {
                    winners |= 1u << k;
                    table[slot[k]] += mine.coefficient[k];
                }
            }
            wave_sync();
#pragma unroll
            for (int k = 0; k < ENTRIES_PER_LANE; k++) {
                if ((winners >> k) & 1u) {
                    owner[slot[k]] = NOBODY;
                }
            }
            pending &= ~winners;
            wave_sync();
        }
    }
}

// ---------------------------------------------------------------------------
// the sum over the edges of one node

template <typename T> struct Contraction {
    const T* A;                  // [n_edges][nA]
    const T* B;                  // [n_edges][ld]
    const T* rows;               // [n_blocks][n_red][ld]  (forward: W)
    const int32_t* gather_index; // [n_edges] block of `rows` of every edge (forward: the sender)
    T* result;                   // [n_blocks][n_out][ld]
    int32_t n_edges, n_blocks, nA, L, ld, n_red, n_out;
    int32_t column_tiles; // ceil(L / 16): wavefronts per node
};

/// Edges whose operands a wavefront asks for together: STEPS steps of four.
/// (Two sets of operands are in registers at a time: one being multiplied,
/// one on its way.)
#ifndef MOPS_SEG_STEPS_F32
#define MOPS_SEG_STEPS_F32 1
#endif
#ifndef MOPS_SEG_STEPS_F64
#define MOPS_SEG_STEPS_F64 1
#endif
#ifndef MOPS_SEG_DOUBLE_BUFFER
#define MOPS_SEG_DOUBLE_BUFFER 1
#endif
#ifndef MOPS_SEG_INNER_BARRIER
#define MOPS_SEG_INNER_BARRIER 0
#endif
#ifndef MOPS_SEG_AHEAD
#define MOPS_SEG_AHEAD 2
#endif
template <typename T> constexpr int steps_in_flight() { return sizeof(T) == 4 ? MOPS_SEG_STEPS_F32 : MOPS_SEG_STEPS_F64; }

/// A tensor as a buffer: loads are a uniform descriptor, a 32-bit byte offset
/// per lane and a uniform byte offset (the hardware adds the three), and an
/// offset beyond the tensor reads as zero without touching memory. That is one
/// address register per lane for all the rows of a block, and lanes without an
/// edge need no row that exists: they ask beyond the end.
template <typename T> struct BufferOf {
    __amdgpu_buffer_rsrc_t descriptor;

    __device__ __forceinline__ void set(const T* base, uint32_t bytes) {
        // (word 3: 32-bit data format, as the other libraries of this platform set it for gfx9)
        descriptor = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(base), 0, static_cast<int>(bytes), 0x00020000);
    }
    __device__ __forceinline__ T load(uint32_t lane_bytes, uint32_t uniform_bytes) const {
        if constexpr (sizeof(T) == 4) {
            return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b32(descriptor, lane_bytes, uniform_bytes, 0));
        } else {
            return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b64(descriptor, lane_bytes, uniform_bytes, 0));
        }
    }
};
constexpr uint32_t BEYOND = 0xffffffffu; // a byte offset no tensor reaches (the host sends larger ones elsewhere)

/// What a wavefront keeps for one node. NB = accumulator tiles: the block rows
/// n_red, or (EXACT false) a bucket above them.
template <typename T, int NB, bool EXACT> struct NodeSum {
    using M = Mfma<T>;
    static constexpr int STEPS = steps_in_flight<T>();

    const Contraction<T>& p;
    int lane, i, q;
    int32_t column;       // of the feature axis, this lane's
    bool column_inside;
    uint32_t column_bytes;    // byte offset of a column that exists
    uint32_t component_bytes; // byte offset of this lane's component in a row of A
    uint32_t component_mask;  // all ones when this lane's accumulator row stands for no component
    uint32_t block_bytes, row_bytes, a_row_bytes;
    BufferOf<T> A, B, rows;
    typename M::Acc acc[NB];

    /// What load() asks for, untouched: looking at a loaded value would make
    /// load() wait for it.
    struct Operands {
        T a[STEPS];
        T b[STEPS];
        T w[STEPS][NB];
    };

    __device__ __forceinline__ NodeSum(const Contraction<T>& contraction, int32_t registers) : p(contraction) {
        lane = threadIdx.x & (WAVE - 1);
        i = lane & 15;
        q = lane >> 4;
        set_column_tile(0);
        const int32_t component = component_of_row<T>(i, registers);
        component_bytes = static_cast<uint32_t>(component < p.nA ? component : 0) * sizeof(T);
        component_mask = component < p.nA ? 0u : BEYOND;
        row_bytes = static_cast<uint32_t>(p.ld) * sizeof(T);
        block_bytes = static_cast<uint32_t>(p.n_red) * row_bytes;
        a_row_bytes = static_cast<uint32_t>(p.nA) * sizeof(T);
        A.set(p.A, static_cast<uint32_t>(p.n_edges) * a_row_bytes);
        B.set(p.B, static_cast<uint32_t>(p.n_edges) * row_bytes);
        rows.set(p.rows, static_cast<uint32_t>(p.n_blocks) * block_bytes);
    }

    /// The 16 columns of the feature axis this wavefront works on next.
    __device__ __forceinline__ void set_column_tile(int32_t column_tile) {
        column = 16 * column_tile + i;
        column_inside = column < p.L;
        column_bytes = static_cast<uint32_t>(min(column, p.L - 1)) * sizeof(T);
    }

    __device__ __forceinline__ void clear() {
#pragma unroll
        for (int c = 0; c < NB; c++) {
            acc[c] = M::zero();
        }
    }

    __device__ __forceinline__ bool has_row(int c) const { return EXACT || c < p.n_red; }

    /// Lane k of `edges` / `sources` holds edge k of a list of up to 64 and
    /// its block of `rows` (-1: no edge). Asks for the operands of the edges
    /// first .. first + 4 STEPS of the list. A lane without an edge asks for the
    /// rows of one that exists, and for its element of A beyond the end of A,
    /// which reads as zero. (The offsets are made by arithmetic on a mask, not by
    /// a choice between an offset and a constant: the compiler turns such a
    /// choice in front of a load into two branches with a load each.)
    __device__ __forceinline__ void load(Operands& to, int32_t edges, int32_t sources, int32_t first) const {
        const int32_t some_edge = __builtin_amdgcn_readfirstlane(edges); // the list is not empty
#pragma unroll
        for (int u = 0; u < STEPS; u++) {
            const int place = min(first + 4 * u + q, WAVE - 1);
            const int32_t edge = __shfl(edges, place);
            const int32_t source = __shfl(sources, place);
            const bool usable = first + 4 * u + q < WAVE && edge >= 0 && in_bounds(source, p.n_blocks);
            const uint32_t e = static_cast<uint32_t>(usable ? edge : some_edge);
            const uint32_t block = static_cast<uint32_t>(usable ? source : 0);
            const uint32_t unusable_mask = static_cast<uint32_t>(usable) - 1u; // 0 or all ones
            to.a[u] = A.load((e * a_row_bytes + component_bytes) | unusable_mask | component_mask, 0);
            to.b[u] = B.load(e * row_bytes + column_bytes, 0);
            const uint32_t from = block * block_bytes + column_bytes;
#pragma unroll
            for (int c = 0; c < NB; c++) {
                const uint32_t row = static_cast<uint32_t>(EXACT ? c : min(c, p.n_red - 1));
                to.w[u][c] = rows.load(from, row * row_bytes);
            }
        }
    }

    __device__ __forceinline__ void multiply(const Operands& from) {
#pragma unroll
        for (int u = 0; u < STEPS; u++) {
            // all products first, then the matrix instructions back to back: a
            // matrix instruction right behind the multiplication that feeds it
            // has to idle for the result
            T right[NB];
#pragma unroll
            for (int c = 0; c < NB; c++) {
                right[c] = from.w[u][c] * from.b[u];
            }
#if MOPS_SEG_INNER_BARRIER
            __builtin_amdgcn_sched_barrier(0);
#endif
#pragma unroll
            for (int c = 0; c < NB; c++) {
                if (has_row(c)) { // (uniform)
                    acc[c] = M::mma(from.a[u], right[c], acc[c]);
                }
            }
        }
    }

    /// Adds the n <= 64 edges of a list (lane k: edge k and its block, -1 beyond n).
    /// The operands of the next batch are asked for before the current one is
    /// multiplied, ALWAYS (beyond the end of the list the loads go to rows that
    /// exist and come back as zeros): a load that is issued only under a
    /// condition makes every later wait a wait for all loads.
    __device__ __forceinline__ void add(int32_t edges, int32_t sources, int32_t n) {
        constexpr int BATCH = 4 * STEPS;
#if !MOPS_SEG_DOUBLE_BUFFER
        for (int32_t done = 0; done < n; done += BATCH) {
            Operands operands;
            load(operands, edges, sources, done);
            multiply(operands);
        }
        return;
#endif
        // Unrolled over all batches a list of 64 can have, with an early way out:
        // in straight-line code the compiler counts the loads in flight exactly
        // (around a loop it waits for the oldest ones at the top of every round,
        // before the next batch is even asked for). The scheduling barriers keep
        // it from moving the loads of a later batch down between the matrix
        // instructions of this one. AHEAD batches are on their way while one is
        // multiplied: a round trip to memory lasts several times as long as the
        // matrix instructions of a batch.
        constexpr int AHEAD = MOPS_SEG_AHEAD;
        constexpr int BATCHES = WAVE / BATCH;
        Operands ring[AHEAD + 1];
#pragma unroll
        for (int b = 0; b < AHEAD; b++) {
            load(ring[b], edges, sources, b * BATCH);
        }
#pragma unroll
        for (int b = 0; b < BATCHES; b++) {
            if (b + AHEAD < BATCHES) {
                load(ring[(b + AHEAD) % (AHEAD + 1)], edges, sources, (b + AHEAD) * BATCH);
            }
            __builtin_amdgcn_sched_barrier(0);
            multiply(ring[b % (AHEAD + 1)]);
            __builtin_amdgcn_sched_barrier(0);
            if ((b + 1) * BATCH >= n) {
                break;
            }
        }
    }

    /// result[node] = D * (the sums so far), this wavefront's 16 columns.
    __device__ __forceinline__ void finish(const T* __restrict__ table, int32_t registers, int32_t node) {
        typename M::Acc out[2] = {M::zero(), M::zero()};
#pragma unroll
        for (int r = 0; r < 4; r++) {
            if (r < registers) { // (uniform)
#pragma unroll
                for (int c = 0; c < NB; c++) {
                    if (has_row(c)) {
                        const T d = table[(r * p.n_red + c) * WAVE + lane];
                        out[(r * NB + c) & 1] = M::mma(d, acc[c][r], out[(r * NB + c) & 1]);
                    }
                }
            }
        }
        T* target = p.result + static_cast<size_t>(node) * p.n_out * p.ld + column;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int32_t row = M::row(lane, r);
            if (row < p.n_out && column_inside) {
                target[static_cast<size_t>(row) * p.ld] = out[0][r] + out[1][r];
            }
        }
    }

    /// Rows of the result that no edge names.
    __device__ __forceinline__ void clear_rows(int32_t begin, int32_t end) const {
        if (!column_inside) {
            return;
        }
        const int32_t rows = (end - begin) * p.n_out;
        T* target = p.result + static_cast<size_t>(begin) * p.n_out * p.ld + column;
        for (int32_t row = q; row < rows; row += 4) {
            target[static_cast<size_t>(row) * p.ld] = T(0);
        }
    }
};

#ifdef MOPS_SEG_TRACE
__device__ long long seg_trace[8192 * 8];
#define MOPS_TRACE_SET(k, v) do { if (lane == 0) seg_trace[(group * 16 + wave) * 8 + (k)] = (v); } while (0)
#define MOPS_TRACE_CODE(...) __VA_ARGS__
#else
#define MOPS_TRACE_SET(k, v)
#define MOPS_TRACE_CODE(...)
#endif

/// Where the edges of a node come from.
enum class Source {
    SORTED, // the index that names the node is sorted: segments of consecutive edges
    SLOTS   // the node's edges are listed in its slots (sender_buckets.hpp)
};

template <typename T> struct ContractArgs {
    Contraction<T> contraction;
    Table table;
    const T* C;
    int32_t n_units; // (chunks of positions | nodes) x column tiles
    // SORTED
    const int32_t* sorted_index; // [n_edges] node of every position, non-decreasing
    // SLOTS
    const int32_t* slot_edges;
    const int32_t* slot_counts;
    const int32_t* listed_index; // [n_edges] the index the slots were listed from (for nodes whose slots overflowed)
};

/// Wavefronts per SIMD the registers are limited to, by element type and
/// accumulator tiles; a workgroup is that many wavefronts on each of the four
/// SIMDs of a compute unit, i.e. ONE workgroup per compute unit.
template <typename T, int NB> constexpr int waves_per_simd() {
    return sizeof(T) == 4 ? (NB <= 9 ? 4 : 3) : (NB <= 4 ? 4 : 2);
}
template <typename T, int NB> constexpr int group_threads() { return 4 * waves_per_simd<T, NB>() * WAVE; }

/// What a wavefront asks for ahead of a unit of work: nothing of it depends
/// on anything but the unit's number.
template <Source SOURCE> struct UnitAhead;
template <> struct UnitAhead<Source::SORTED> {
    ChunkIndex index;
    int32_t near_source[2]; // blocks of the 128 positions from the chunk's first
};
template <> struct UnitAhead<Source::SLOTS> {
    int32_t first_half, second_half; // the node's slots
    int4 part_counts;
};

// The kernel is PERSISTENT: one workgroup per compute unit builds the dense
// table once and then works through its share of the units (a chunk of the
// sorted index, or a node, times a tile of 16 columns). Workgroup g of G has
// units g, g + G, g + 2 G, ...; its wavefronts take the next one from a
// counter in LDS as they get free (the first one each without asking), so a
// wavefront that drew long segments does not hold the others up, nothing in
// global memory has to be cleared, and every wavefront leaves when the
// counter has passed the workgroup's last unit. While a wavefront works on a
// unit, the index values of its next unit are on their way.
template <typename T, int NB, bool EXACT, Source SOURCE, int CHUNK>
__global__ __launch_bounds__((group_threads<T, NB>())) void contract_kernel(const ContractArgs<T> args) {
    constexpr int THREADS = group_threads<T, NB>();
    constexpr int GROUP_WAVES = THREADS / WAVE;
    extern __shared__ __align__(16) char lds_raw[];
    T* table = reinterpret_cast<T*>(lds_raw);
    int32_t* owner = reinterpret_cast<int32_t*>(table + args.table.slots());
    int32_t* next_turn = owner + args.table.slots();
    int32_t* table_ready = next_turn + 1;

    const Contraction<T>& p = args.contraction;
    const int32_t registers = args.table.registers;
    const int lane = threadIdx.x & (WAVE - 1);
    const int32_t wave = threadIdx.x >> 6;
    const int32_t group = static_cast<int32_t>(blockIdx.x);
    const int32_t n_groups = static_cast<int32_t>(gridDim.x);
    NodeSum<T, NB, EXACT> sum(p, registers);
    MOPS_TRACE_CODE(long long t_start = clock64(); long long t_add = 0, t_finish = 0, t_turn = 0, t_mark = 0; int n_units_done = 0, n_edges_done = 0;)

    // turn k of this workgroup is unit group + k * n_groups
    auto unit_of_turn = [&](int32_t turn) { return group + turn * n_groups; };
    auto take_turn = [&]() {
        int32_t turn = 0;
        if (lane == 0) {
            turn = atomicAdd(next_turn, 1);
        }
        return __builtin_amdgcn_readfirstlane(turn);
    };
    auto look_ahead = [&](UnitAhead<SOURCE>& ahead, int32_t unit) {
        const bool exists = unit < args.n_units;
        const int32_t item = exists ? unit / p.column_tiles : 0; // chunk or node
        if constexpr (SOURCE == Source::SORTED) {
            ahead.index = load_chunk_index<CHUNK>(args.sorted_index, p.n_edges, item);
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int32_t position = item * CHUNK + h * WAVE + lane;
                const int32_t source =
                    load_or_zero(p.gather_index, static_cast<size_t>(position), position < p.n_edges);
                ahead.near_source[h] = position < p.n_edges ? source : -1;
            }
        } else {
            const int32_t* mine = args.slot_edges + static_cast<size_t>(item) * SLOT_CAPACITY;
            ahead.first_half = mine[lane];
            ahead.second_half = mine[lane + WAVE];
            ahead.part_counts = reinterpret_cast<const int4*>(args.slot_counts)[item];
        }
    };

    // everything that can be asked for without knowing anything is asked for
    // first; the table is built while it is on its way
    int32_t unit = unit_of_turn(wave);
    UnitAhead<SOURCE> current;
    MyEntries<T> entries;
    if (wave == 0) {
        load_entries<T>(entries, args.C, args.table, 0, lane);
    }
    look_ahead(current, unit);
    if (threadIdx.x == 0) {
        *next_turn = GROUP_WAVES;
        *table_ready = 0;
    }
    __syncthreads(); // (everybody is here at once: nothing has been waited for yet)
    // The first wavefront builds the table; the others start on their units,
    // which need the table only when the sums of a node are complete.
    bool table_seen = false;
    if (wave == 0) {
        build_table<T>(table, owner, entries, args.C, args.table, lane);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        if (lane == 0) {
            __hip_atomic_store(table_ready, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
        table_seen = true;
    }
    // (the builder depends on nobody, so the wait ends; a wavefront sleeps
    // between looks and does not take issue slots from the builder)
    auto wait_for_table = [&]() {
        if (!table_seen) {
            while (__hip_atomic_load(table_ready, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) == 0) {
                __builtin_amdgcn_s_sleep(4);
            }
            table_seen = true;
        }
    };
    MOPS_TRACE_CODE(long long t_built = clock64();)

    while (unit < args.n_units) {
        MOPS_TRACE_CODE(n_units_done++; t_mark = clock64();)
        const int32_t next_unit = unit_of_turn(take_turn());
        UnitAhead<SOURCE> next;
        look_ahead(next, next_unit);
        MOPS_TRACE_CODE(t_turn += clock64() - t_mark;)

        const int32_t item = unit / p.column_tiles;
        sum.set_column_tile(unit - item * p.column_tiles);
        if constexpr (SOURCE == Source::SLOTS) {
            const int32_t node = item;
            sum.clear();
            bool any = false;
            // lane k of `edges` holds edge k of n <= 64
            auto hand_on = [&](int32_t edges, int32_t n) {
                const int32_t mine = lane < n ? edges : -1;
                const int32_t sources = load_or_zero(p.gather_index, static_cast<size_t>(max(mine, 0)), mine >= 0);
                sum.add(mine, mine >= 0 ? sources : -1, n);
                any = true;
            };
            static_assert(SLOT_PARTS == 4 && SLOT_CAPACITY == 2 * WAVE, "the four parts of a node's places in two registers");
            const int32_t c0 = __builtin_amdgcn_readfirstlane(current.part_counts.x);
            const int32_t c1 = __builtin_amdgcn_readfirstlane(current.part_counts.y);
            const int32_t c2 = __builtin_amdgcn_readfirstlane(current.part_counts.z);
            const int32_t c3 = __builtin_amdgcn_readfirstlane(current.part_counts.w);
            const int32_t count = c0 + c1 + c2 + c3;
            if (max(max(c0, c1), max(c2, c3)) <= SLOT_PART_CAPACITY) {
                // the parts moved together: position k of the list is in part `part`, place k - before
                auto edge_at = [&](int32_t position) {
                    const int32_t part = (position >= c0 ? 1 : 0) + (position >= c0 + c1 ? 1 : 0) +
                                         (position >= c0 + c1 + c2 ? 1 : 0);
                    const int32_t before = part == 0 ? 0 : part == 1 ? c0 : part == 2 ? c0 + c1 : c0 + c1 + c2;
                    const int32_t place = part * SLOT_PART_CAPACITY + position - before;
                    const int32_t low = __shfl(current.first_half, place & (WAVE - 1));
                    const int32_t high = __shfl(current.second_half, place & (WAVE - 1));
                    return place < WAVE ? low : high;
                };
                if (count > 0) {
                    hand_on(edge_at(lane), min(count, WAVE));
                }
                if (count > WAVE) {
                    hand_on(edge_at(lane + WAVE), count - WAVE);
                }
            } else {
                // more edges in a part than places (a hub of a sparse graph): this
                // wavefront reads the whole index itself
                const unsigned long long below = (1ull << lane) - 1ull;
                for (int32_t base = 0; base < p.n_edges; base += WAVE) {
                    const int32_t e = base + lane;
                    const bool named = e < p.n_edges && args.listed_index[min(e, p.n_edges - 1)] == node;
                    const unsigned long long mask = __ballot(named);
                    if (mask != 0) {
                        // the matches moved to the first lanes, in edge order
                        const int32_t n = __popcll(mask);
                        const int32_t named_below = __popcll(mask & below);
                        const int32_t place = named ? named_below : n + lane - named_below;
                        hand_on(__builtin_amdgcn_ds_permute(place << 2, e), n);
                    }
                }
            }
            if (any) {
                wait_for_table();
                sum.finish(table, registers, node);
            } else {
                sum.clear_rows(node, node + 1);
            }
        } else {
            const int32_t chunk_begin = item * CHUNK;
            walk_owned_segments<CHUNK>(
                args.sorted_index, p.n_edges, p.n_blocks, item, current.index,
                [&](int32_t node, int32_t first, int32_t last) {
                    sum.clear();
                    MOPS_TRACE_CODE(long long t0 = clock64(); n_edges_done += last - first;)
                    for (int32_t base = first; base < last; base += WAVE) {
                        const int32_t n = min(WAVE, last - base);
                        const int32_t offset = base - chunk_begin; // >= 0: owned segments start in the chunk
                        int32_t edges = lane < n ? base + lane : -1;
                        int32_t sources;
                        if (offset + WAVE <= 2 * WAVE) { // (uniform) all 64 positions are at hand
                            const int from = offset + lane;
                            const int32_t s0 = __shfl(current.near_source[0], from & (WAVE - 1));
                            const int32_t s1 = __shfl(current.near_source[1], from & (WAVE - 1));
                            sources = from < WAVE ? s0 : s1;
                        } else {
                            sources = load_or_zero(p.gather_index, static_cast<size_t>(max(edges, 0)), edges >= 0);
                        }
                        sum.add(edges, edges >= 0 ? sources : -1, n);
                    }
                    MOPS_TRACE_CODE(long long t1 = clock64(); t_add += t1 - t0;)
                    wait_for_table();
                    sum.finish(table, registers, node);
                    MOPS_TRACE_CODE(t_finish += clock64() - t1;)
                },
                [&](int32_t begin, int32_t end) { sum.clear_rows(begin, end); }
            );
        }
        unit = next_unit;
        current = next;
    }
    MOPS_TRACE_SET(0, t_start);
    MOPS_TRACE_SET(1, t_built);
    MOPS_TRACE_SET(2, clock64());
    MOPS_TRACE_SET(3, n_units_done);
    MOPS_TRACE_SET(4, t_add);
    MOPS_TRACE_SET(5, t_finish);
    MOPS_TRACE_SET(6, t_turn);
    MOPS_TRACE_SET(7, n_edges_done);
}

// ---------------------------------------------------------------------------
// host side

size_t table_lds(const Table& t, size_t element_size) {
    return static_cast<size_t>(t.slots()) * (element_size + sizeof(int32_t)) + 16;
}

Table table_of(const Shape& s, const int32_t* PA, const int32_t* Pred, const int32_t* Pout, int32_t n_red, int32_t n_out) {
    Table t;
    t.PA = PA;
    t.Pred = Pred;
    t.Pout = Pout;
    t.N = s.N;
    t.nA = s.nA;
    t.n_red = n_red;
    t.n_out = n_out;
    t.registers = (s.nA + 3) / 4;
    return t;
}

/// Accumulator tiles: the block rows themselves when they are 1, 4, 9 or 16 (the
/// numbers of components of spherical harmonics up to some degree), otherwise
/// rounded up to one of those.
template <typename Launch> void with_block_rows(int32_t n_red, Launch&& launch) {
    if (n_red == 1) {
        launch(std::integral_constant<int, 1>{}, std::true_type{});
    } else if (n_red == 4) {
        launch(std::integral_constant<int, 4>{}, std::true_type{});
    } else if (n_red < 4) {
        launch(std::integral_constant<int, 4>{}, std::false_type{});
    } else if (n_red == 9) {
        launch(std::integral_constant<int, 9>{}, std::true_type{});
    } else if (n_red < 9) {
        launch(std::integral_constant<int, 9>{}, std::false_type{});
    } else if (n_red == 16) {
        launch(std::integral_constant<int, 16>{}, std::true_type{});
    } else {
        launch(std::integral_constant<int, 16>{}, std::false_type{});
    }
}

template <typename Kernel> void allow_lds(Kernel kernel, size_t lds) {
    if (lds > 64 * 1024) {
        MOPS_HIP_CHECK(hipFuncSetAttribute(
            reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)
        ));
    }
}

/// Positions of the sorted index per unit of work: the fewest of 16, 32, 64
/// with which every wavefront that is resident on the device has at most one
/// unit (measured at 60 000 edges, 2 column tiles: float, 4096 wavefronts: 30 us
/// with 8, 27 with 16, 25 with 32, 32 with 64; double, 2048 wavefronts: 41, 36,
/// 36, 31).
int32_t chunk_for(int32_t n_edges, int32_t column_tiles, int64_t resident_waves) {
    for (int32_t chunk : {16, 32}) {
        if ((static_cast<int64_t>(n_edges) + chunk - 1) / chunk * column_tiles <= resident_waves) {
            return chunk;
        }
    }
    return 64;
}

/// Compute units of the current device (asked for once per device).
int32_t compute_units() {
    static std::atomic<int> cached[64];
    int device = 0;
    MOPS_HIP_CHECK(hipGetDevice(&device));
    if (device < 0 || device >= 64) {
        return 256;
    }
    int count = cached[device].load(std::memory_order_relaxed);
    if (count == 0) {
        MOPS_HIP_CHECK(hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device));
        count = std::max(count, 1);
        cached[device].store(count, std::memory_order_relaxed);
    }
    return count;
}

template <typename T, Source SOURCE>
void launch_contract(ContractArgs<T> args, hipStream_t stream) {
    const Contraction<T>& p = args.contraction;
    const size_t lds = table_lds(args.table, sizeof(T));
    with_block_rows(p.n_red, [&](auto block_rows, auto exact) {
        constexpr int NB = decltype(block_rows)::value;
        constexpr bool EXACT = decltype(exact)::value;
        auto go = [&](auto chunk_constant) {
            constexpr int CHUNK = decltype(chunk_constant)::value;
            constexpr int GROUP_WAVES = group_threads<T, NB>() / WAVE;
            const int64_t items = SOURCE == Source::SLOTS ? p.n_blocks
                                                          : (static_cast<int64_t>(p.n_edges) + CHUNK - 1) / CHUNK;
            const int64_t units = items * p.column_tiles;
            args.n_units = narrow_i32(static_cast<size_t>(units), "units of work");
            // one workgroup per compute unit, fewer when there is not a unit per wavefront
            const unsigned grid = static_cast<unsigned>(
                std::min<int64_t>(compute_units(), (units + GROUP_WAVES - 1) / GROUP_WAVES)
            );
            auto kernel = contract_kernel<T, NB, EXACT, SOURCE, CHUNK>;
            allow_lds(kernel, lds);
            kernel<<<grid, group_threads<T, NB>(), lds, stream>>>(args);
        };
        if constexpr (SOURCE == Source::SLOTS) {
            go(std::integral_constant<int, 64>{});
        } else {
            constexpr int64_t GROUP_WAVES = group_threads<T, NB>() / WAVE;
            switch (chunk_for(p.n_edges, p.column_tiles, GROUP_WAVES * compute_units())) {
            case 16:
                go(std::integral_constant<int, 16>{});
                break;
            case 32:
                go(std::integral_constant<int, 32>{});
                break;
            default:
                go(std::integral_constant<int, 64>{});
                break;
            }
        }
    });
    MOPS_HIP_CHECK(hipGetLastError());
}

template <typename T>
Contraction<T> contraction_of(
    const Shape& s, const T* A, const T* B, const T* rows, const int32_t* gather_index, T* result, int32_t n_red,
    int32_t n_out
) {
    Contraction<T> c;
    c.A = A;
    c.B = B;
    c.rows = rows;
    c.gather_index = gather_index;
    c.result = result;
    c.n_edges = s.n_edges;
    c.n_blocks = s.n_nodes;
    c.nA = s.nA;
    c.L = s.L;
    c.ld = s.L;
    c.n_red = n_red;
    c.n_out = n_out;
    c.column_tiles = (s.L + 15) / 16;
    return c;
}

} // namespace

#ifdef MOPS_SEG_TRACE
extern "C" __attribute__((visibility("default"))) int mops_seg_trace_read(long long* host, int count) {
    return static_cast<int>(hipMemcpyFromSymbol(host, HIP_SYMBOL(seg_trace), count * sizeof(long long)));
}
extern "C" __attribute__((visibility("default"))) int mops_seg_trace_clear() {
    static long long zeros[8192 * 8];
    return static_cast<int>(hipMemcpyToSymbol(HIP_SYMBOL(seg_trace), zeros, sizeof(zeros)));
}
#endif

bool supports(const Shape& s, size_t element_size) {
    if (s.n_nodes < 1 || s.n_edges < 1 || s.N < 1 || s.N > MAX_TABLE || s.L < 1) {
        return false;
    }
    if (s.nA < 1 || s.nA > MAX_INDEX || s.n2 < 1 || s.n2 > MAX_INDEX || s.n3 < 1 || s.n3 > MAX_INDEX) {
        return false;
    }
    // 32-bit byte offsets into every tensor
    const uint64_t limit = uint64_t(1) << 32;
    const uint64_t widest = static_cast<uint64_t>(std::max(std::max(s.n2, s.n3), 1)) * s.L * element_size;
    return static_cast<uint64_t>(s.n_nodes) * widest < limit &&
           static_cast<uint64_t>(s.n_edges) * std::max(s.nA, s.L) * element_size < limit;
}

template <typename T>
void forward(
    T* output, const T* A, const T* B, const T* C, const T* W, const Indices& indices, const Shape& s,
    hipStream_t stream
) {
    ContractArgs<T> args{};
    args.contraction = contraction_of<T>(s, A, B, W, indices.W_1, output, s.n2, s.n3);
    args.table = table_of(s, indices.A, indices.W_2, indices.output_2, s.n2, s.n3);
    args.C = C;
    args.sorted_index = indices.output_1;
    MainKernelTimer timer(stream);
    launch_contract<T, Source::SORTED>(args, stream);
}

template <typename T>
void grad_W_from_slots(
    T* grad_W, const T* grad_output, const T* A, const T* B, const T* C, const Indices& indices, const Shape& s,
    const SenderSlots& slots, hipStream_t stream
) {
    ContractArgs<T> args{};
    // the blocks that are gathered are rows of grad_output, named by the receiver
    args.contraction = contraction_of<T>(s, A, B, grad_output, indices.output_1, grad_W, s.n3, s.n2);
    args.table = table_of(s, indices.A, indices.output_2, indices.W_2, s.n3, s.n2);
    args.C = C;
    args.slot_edges = slots.edges;
    args.slot_counts = slots.counts;
    args.listed_index = indices.W_1;
    launch_contract<T, Source::SLOTS>(args, stream);
}

template void forward<float>(
    float*, const float*, const float*, const float*, const float*, const Indices&, const Shape&, hipStream_t
);
template void forward<double>(
    double*, const double*, const double*, const double*, const double*, const Indices&, const Shape&, hipStream_t
);
template void grad_W_from_slots<float>(
    float*, const float*, const float*, const float*, const float*, const Indices&, const Shape&, const SenderSlots&,
    hipStream_t
);
template void grad_W_from_slots<double>(
    double*, const double*, const double*, const double*, const double*, const Indices&, const Shape&,
    const SenderSlots&, hipStream_t
);

} // namespace mops::amd::sasaw_segments
