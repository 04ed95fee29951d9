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
// grad_A and grad_B: see "grad_A and grad_B" below (EdgeGradients).
//
// The dense table is built by every workgroup for itself in LDS, in operand
// layout, entries of one cell added in ascending entry order (no launch of its
// own; it overlaps with the wait for the first rows). No atomics on floating
// point anywhere: two runs give the same bits.
#include "sasaw_segments.hpp"

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <stdexcept>
#include <type_traits>

#include "device_common.hpp"
#include "dispatch_thresholds.hpp"
#include "mfma.hpp"
#include "runtime.hpp"
#include "segment_walk.hpp"
#include "sender_buckets.hpp"

namespace mops::amd::sasaw_segments {
namespace {

constexpr int MAX_INDEX = thresholds::SASAW_INDEX_VALUES; // values of a component index
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

/// The layouts the dense table is needed in. All are "what one lane of a
/// wavefront holds as an operand of one matrix instruction, instruction after
/// instruction", so that reading it is one conflict-free LDS access.
enum class Layout : int32_t {
    // result = D * sums (contract_kernel, and grad_W): see above
    RESULT,
    // grad_A: right operand of (grad_output of a node)^T * D[:, m2, :], per
    // block row m2 and step s3 over the rows of the result:
    //   table[((m2 * steps3 + s3) * 64 + 16 * k + m1] = D[4 * s3 + k, m2, m1]
    ALPHA,
    // grad_B: left operand of D' * (grad_output of a node), whose rows are
    // pairs (component of A, block row) in the order the accumulators of the
    // next product want them: pair p = s * bucket + m2 (s = m1 / 4) lies in
    // tile p / 4, register p % 4, of the lanes q = m1 % 4:
    //   table[((p / 4) * steps3 + s3) * 64 + 16 * k + row(q, p % 4)] = D[4 * s3 + k, m2, m1]
    BETA
};

struct Table {
    const int32_t* PA;   // [N]
    const int32_t* Pred; // [N] index of the block row that is summed over (forward: PW2)
    const int32_t* Pout; // [N] index of the row of the result (forward: PO2)
    int32_t N, nA, n_red, n_out;
    int32_t registers; // ceil(nA / 4)
    Layout layout;
    int32_t bucket; // BETA: accumulator tiles of the kernel (>= n_red)
    // The part of the coupling table this launch works with: components m1_begin .. m1_begin + nA
    // of A, block rows red_begin .. red_begin + n_red, rows out_begin .. out_begin + n_out of the
    // result (all zero and the whole ranges for shapes that one launch covers). RESULT only:
    // n_out may exceed 16; the rows of the result then come in blocks of 16.
    int32_t m1_begin, red_begin, out_begin;

    __host__ __device__ int32_t steps3() const { return (n_out + 3) / 4; }
    __host__ __device__ int32_t slots() const {
        switch (layout) {
        case Layout::ALPHA:
            return n_red * steps3() * WAVE;
        case Layout::BETA:
            return (registers * bucket + 3) / 4 * steps3() * WAVE;
        default:
            return out_blocks() * registers * n_red * WAVE;
        }
    }
    __host__ __device__ int32_t out_blocks() const { return (n_out + 15) / 16; }
};

/// Where D[o, c, m1] goes (all three inside their ranges).
template <typename T> __device__ __forceinline__ int32_t slot_in(const Table& t, int32_t m1, int32_t c, int32_t o) {
    switch (t.layout) {
    case Layout::ALPHA:
        return (c * t.steps3() + (o >> 2)) * WAVE + 16 * (o & 3) + m1;
    case Layout::BETA: {
        const int32_t pair = (m1 >> 2) * t.bucket + c;
        const int q = m1 & 3, r = pair & 3;
        const int row = sizeof(T) == 4 ? 4 * q + r : 4 * r + q;
        return ((pair >> 2) * t.steps3() + (o >> 2)) * WAVE + 16 * (o & 3) + row;
    }
    default: {
        int q, r;
        place_of_component<T>(m1, t.registers, q, r);
        return (((o >> 4) * t.registers + r) * t.n_red + c) * WAVE + 16 * q + (o & 15);
    }
    }
}

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
            const int32_t m1 = mine.m1[k] - t.m1_begin, c = mine.c[k] - t.red_begin, o = mine.o[k] - t.out_begin;
            const bool inside = n < t.N && in_bounds(m1, t.nA) && in_bounds(c, t.n_red) && in_bounds(o, t.n_out);
            slot[k] = inside ? slot_in<T>(t, m1, c, o) : -1;
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
    // A launch that works on a part of the tensors (NodeSum<.., GENERAL>): `A`, `rows` and `result`
    // point to the first component / block row / row of the part, nA, n_red and n_out count the
    // part, and these are the full extents the rows are apart by. `accumulate`: the launch adds
    // to what `result` holds (another part of the sums over m1 and the block rows is there already).
    int32_t lda, rows_stride, out_stride;
    bool accumulate;
};

/// Edges whose operands a wavefront asks for together: STEPS steps of four.
/// (Two sets of operands are in registers at a time: one being multiplied,
/// one on its way.)
template <typename T> constexpr int steps_in_flight() { return 1; }

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

/// The value, in a way the compiler cannot see through. What a kernel with
/// several roles derives from the lane number for ONE role would otherwise be
/// computed once in front of the loop over the units of work and kept in
/// registers through all roles: dozens of registers per role, and spills.
__device__ __forceinline__ int opaque(int value) {
    asm volatile("" : "+v"(value));
    return value;
}

/// The (uniform) value, made where it is used. The byte offsets of the rows
/// of a block, c * row_bytes for every c, are the same in every turn of every
/// loop, so the compiler computes them once in front of the loop over the units
/// of work; a kernel with several roles has no scalar registers left for them,
/// keeps them in lanes of a vector register, and every load then costs a
/// `v_readlane` and the five idle cycles between it and the load that uses it.
/// One scalar multiplication per load instead.
__device__ __forceinline__ uint32_t fresh(uint32_t value) {
    // (readfirstlane: where the compiler holds the uniform value in a vector register)
    uint32_t uniform = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(value)));
    asm volatile("" : "+s"(uniform));
    return uniform;
}

/// All ones unless `wanted`: OR-ed into a byte offset it makes the load read
/// zero. (Arithmetic instead of a choice between an offset and a constant: the
/// compiler turns such a choice in front of a load into two branches.)
__device__ __forceinline__ uint32_t unless(bool wanted) { return static_cast<uint32_t>(wanted) - 1u; }

/// Four consecutive elements. VECTORS: as 16-byte loads (the tensor's rows must
/// then be a multiple of four elements long and start on 16-byte boundaries,
/// so that the four are inside or outside a row together); otherwise one by
/// one, each with its own limit `inside` (elements from which on there is nothing).
template <typename T, bool VECTORS>
__device__ __forceinline__ void load_four(
    T (&to)[4], const BufferOf<T>& buffer, uint32_t lane_bytes, uint32_t uniform_bytes, int32_t inside, uint32_t mask
) {
    if constexpr (VECTORS) {
        const uint32_t at = lane_bytes | mask | unless(inside > 0);
        if constexpr (sizeof(T) == 4) {
            const auto raw = __builtin_amdgcn_raw_buffer_load_b128(buffer.descriptor, at, uniform_bytes, 0);
            to[0] = __builtin_bit_cast(T, static_cast<uint32_t>(raw[0]));
            to[1] = __builtin_bit_cast(T, static_cast<uint32_t>(raw[1]));
            to[2] = __builtin_bit_cast(T, static_cast<uint32_t>(raw[2]));
            to[3] = __builtin_bit_cast(T, static_cast<uint32_t>(raw[3]));
        } else {
#pragma unroll
            for (int half = 0; half < 2; half++) {
                const auto raw =
                    __builtin_amdgcn_raw_buffer_load_b128(buffer.descriptor, at, uniform_bytes + 16 * half, 0);
                typedef uint32_t Two __attribute__((ext_vector_type(2)));
                to[2 * half] = __builtin_bit_cast(T, Two{raw[0], raw[1]});
                to[2 * half + 1] = __builtin_bit_cast(T, Two{raw[2], raw[3]});
            }
        }
    } else {
#pragma unroll
        for (int v = 0; v < 4; v++) {
            to[v] = buffer.load((lane_bytes + v * static_cast<uint32_t>(sizeof(T))) | mask | unless(v < inside), uniform_bytes);
        }
    }
}

/// What a wavefront keeps for one node. NB = accumulator tiles: the block rows
/// n_red, or (EXACT false) a bucket above them.
template <typename T, int NB, bool EXACT, bool COMPACT = false, bool GENERAL = false> struct NodeSum {
    using M = Mfma<T>;
    static constexpr int STEPS = steps_in_flight<T>();

    const Contraction<T>& p;
    int32_t registers_of_A; // ceil(nA / 4)
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

    __device__ __forceinline__ NodeSum(const Contraction<T>& contraction, int32_t registers)
        : p(contraction), registers_of_A(registers) {
        set_column_tile(0);
        row_bytes = static_cast<uint32_t>(p.ld) * sizeof(T);
        block_bytes = static_cast<uint32_t>(GENERAL ? p.rows_stride : p.n_red) * row_bytes;
        a_row_bytes = static_cast<uint32_t>(GENERAL ? p.lda : p.nA) * sizeof(T);
        // (GENERAL: the tensors begin up to a row before `A` and `rows`, so these limits lie up to a
        // row behind their ends; no lane that is not masked asks for anything there)
        A.set(p.A, static_cast<uint32_t>(p.n_edges) * a_row_bytes);
        B.set(p.B, static_cast<uint32_t>(p.n_edges) * row_bytes);
        rows.set(p.rows, static_cast<uint32_t>(p.n_blocks) * block_bytes);
    }

    /// The 16 columns of the feature axis this wavefront works on next.
    __device__ __forceinline__ void set_column_tile(int32_t column_tile) {
        lane = opaque(static_cast<int>(threadIdx.x & (WAVE - 1)));
        i = lane & 15;
        q = lane >> 4;
        const int32_t component = component_of_row<T>(i, registers_of_A);
        component_bytes = static_cast<uint32_t>(component < p.nA ? component : 0) * sizeof(T);
        component_mask = component < p.nA ? 0u : BEYOND;
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
                // (COMPACT: the kernel with several roles, where the offsets would not stay in scalar registers)
                to.w[u][c] = rows.load(from, (COMPACT ? fresh(row) : row) * row_bytes);
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
        // Unrolled over all batches a list of 64 can have, with an early way out:
        // in straight-line code the compiler counts the loads in flight exactly
        // (around a loop it waits for the oldest ones at the top of every round,
        // before the next batch is even asked for). The scheduling barriers keep
        // it from moving the loads of a later batch down between the matrix
        // instructions of this one. AHEAD batches are on their way while one is
        // multiplied: a round trip to memory lasts several times as long as the
        // matrix instructions of a batch.
        // (measured at 60 000 edges: the forward kernel with 1 / 2 / 3 batches ahead
        // takes 22.3 / 24.9 / 27.8 us in float, 31.6 / 32.4 / 33.9 in double: operands
        // further ahead cost registers, which are spilled; the kernel with several
        // roles: no difference between 1, 2 and 3)
        constexpr int AHEAD = COMPACT ? 2 : 1;
        constexpr int BATCHES = WAVE / BATCH;
        if constexpr (COMPACT) {
            // (a kernel with other roles beside this one: the same in rounds of
            // four batches, a quarter of the code)
            constexpr int ROUND = 4;
            for (int32_t done = 0; done < n; done += ROUND * BATCH) {
                Operands ring[AHEAD + 1];
#pragma unroll
                for (int b = 0; b < AHEAD; b++) {
                    load(ring[b], edges, sources, done + b * BATCH);
                }
#pragma unroll
                for (int b = 0; b < ROUND; b++) {
                    if (b + AHEAD < ROUND) {
                        load(ring[(b + AHEAD) % (AHEAD + 1)], edges, sources, done + (b + AHEAD) * BATCH);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    multiply(ring[b % (AHEAD + 1)]);
                    __builtin_amdgcn_sched_barrier(0);
                    if (done + (b + 1) * BATCH >= n) {
                        break;
                    }
                }
            }
            return;
        }
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
        if constexpr (GENERAL) {
            // the rows of the result in blocks of 16, each with its own part of the table
            const int32_t blocks = (p.n_out + 15) / 16;
            for (int32_t block = 0; block < blocks; block++) {
                finish_block(table + static_cast<size_t>(block) * registers * p.n_red * WAVE, registers, node, 16 * block);
            }
        } else {
            finish_block(table, registers, node, 0);
        }
    }

    /// Rows first_row .. first_row + 16 of result[node].
    __device__ __forceinline__ void finish_block(
        const T* __restrict__ table, int32_t registers, int32_t node, int32_t first_row
    ) {
        // result = D * sums, one block of NB table operands per register r of the
        // sums; four sums (double: two) take the products in turn, so that
        // consecutive matrix instructions do not wait for each other.
        typename M::Acc out[sizeof(T) == 4 ? 4 : 2];
#pragma unroll
        for (auto& sum : out) {
            sum = M::zero();
        }
        if constexpr (sizeof(T) == 4) {
            // The operands of block r + 1 are read from LDS before the matrix
            // instructions of block r (always: a read under a condition would
            // have to be waited for where it stands).
            T d[2][NB];
            auto read = [&](T (&to)[NB], int r) {
                const int32_t block = min(r, registers - 1);
#pragma unroll
                for (int c = 0; c < NB; c++) {
                    to[c] = table[(block * p.n_red + (EXACT ? c : min(c, p.n_red - 1))) * WAVE + lane];
                }
            };
            read(d[0], 0);
#pragma unroll
            for (int r = 0; r < 4; r++) {
                if (r + 1 < 4) {
                    read(d[(r + 1) & 1], r + 1);
                }
                if (r < registers) { // (uniform)
#pragma unroll
                    for (int c = 0; c < NB; c++) {
                        if (has_row(c)) {
                            out[c & 3] = M::mma(d[r & 1][c], acc[c][r], out[c & 3]);
                        }
                    }
                }
            }
        } else {
            // (double: the registers for operands read ahead are not there)
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
        }
        T* target = p.result + static_cast<size_t>(node) * (GENERAL ? p.out_stride : p.n_out) * p.ld + column;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int32_t row = first_row + M::row(lane, r);
            if (row < p.n_out && column_inside) {
                T value;
                if constexpr (sizeof(T) == 4) {
                    value = (out[0][r] + out[1][r]) + (out[2][r] + out[3][r]);
                } else {
                    value = out[0][r] + out[1][r];
                }
                if constexpr (GENERAL) {
                    if (p.accumulate) { // (uniform)
                        value += target[static_cast<size_t>(row) * p.ld];
                    }
                }
                target[static_cast<size_t>(row) * p.ld] = value;
            }
        }
    }

    /// Rows of the result that no edge names.
    __device__ __forceinline__ void clear_rows(int32_t begin, int32_t end) const {
        if (!column_inside) {
            return;
        }
        if constexpr (GENERAL) {
            if (!p.accumulate) { // (the launch that adds finds the zeros of the one before it)
                for (int32_t node = begin; node < end; node++) {
                    T* target = p.result + static_cast<size_t>(node) * p.out_stride * p.ld + column;
                    for (int32_t row = q; row < p.n_out; row += 4) {
                        target[static_cast<size_t>(row) * p.ld] = T(0);
                    }
                }
            }
            return;
        }
        const int32_t rows = (end - begin) * p.n_out;
        T* target = p.result + static_cast<size_t>(begin) * p.n_out * p.ld + column;
        for (int32_t row = q; row < rows; row += 4) {
            target[static_cast<size_t>(row) * p.ld] = T(0);
        }
    }
};

/// The sums of NODE `node` from its slots (sender_buckets.hpp): `first_half` and
/// `second_half` are the node's 128 places (lane k: places k and k + 64),
/// `part_counts` the numbers of edges in its four parts; `listed_index` the
/// index the slots were listed from, read in full by a node whose slots
/// overflowed. Returns whether the node has edges at all.
template <typename Sum>
__device__ __forceinline__ bool sum_over_slots(
    Sum& sum, int32_t first_half, int32_t second_half, int4 part_counts, const int32_t* __restrict__ listed_index,
    int32_t node, int lane
) {
    const auto& p = sum.p;
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
    const int32_t c0 = __builtin_amdgcn_readfirstlane(part_counts.x);
    const int32_t c1 = __builtin_amdgcn_readfirstlane(part_counts.y);
    const int32_t c2 = __builtin_amdgcn_readfirstlane(part_counts.z);
    const int32_t c3 = __builtin_amdgcn_readfirstlane(part_counts.w);
    const int32_t count = c0 + c1 + c2 + c3;
    if (max(max(c0, c1), max(c2, c3)) <= SLOT_PART_CAPACITY) {
        // the parts moved together: position k of the list is in part `part`, place k - before
        auto edge_at = [&](int32_t position) {
            const int32_t part =
                (position >= c0 ? 1 : 0) + (position >= c0 + c1 ? 1 : 0) + (position >= c0 + c1 + c2 ? 1 : 0);
            const int32_t before = part == 0 ? 0 : part == 1 ? c0 : part == 2 ? c0 + c1 : c0 + c1 + c2;
            const int32_t place = part * SLOT_PART_CAPACITY + position - before;
            const int32_t low = __shfl(first_half, place & (WAVE - 1));
            const int32_t high = __shfl(second_half, place & (WAVE - 1));
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
            const bool named = e < p.n_edges && listed_index[min(e, p.n_edges - 1)] == node;
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
    return any;
}

/// The same from the node's places by arrival (SenderArrivals in
/// sender_buckets.hpp): `count` edges name the node, in no order; `area` is
/// this wavefront's SLOT_CAPACITY integers in LDS.
template <typename Sum>
__device__ __forceinline__ bool sum_over_arrivals(
    Sum& sum, int32_t first_half, int32_t second_half, int32_t count, int32_t* area,
    const int32_t* __restrict__ listed_index, int32_t node, int lane
) {
    if (count > SLOT_CAPACITY) {
        // (more edges than places: the slots' way of saying so makes sum_over_slots read the index)
        return sum_over_slots(sum, 0, 0, make_int4(SLOT_PART_CAPACITY + 1, 0, 0, 0), listed_index, node, lane);
    }
    const auto& p = sum.p;
    sum.clear();
    // (A negative count is no count. The counters outlive a call, so a launch that failed
    // between a listing and its readers can leave counts without lists behind them: what a
    // place holds is used as an edge only if it can be one, so that such a remnant gives wrong
    // sums in the next call but no access outside the tensors.)
    count = max(count, 0);
    auto hand_on = [&](int32_t edges, int32_t n) {
        const int32_t mine = lane < n && in_bounds(edges, p.n_edges) ? edges : -1;
        const int32_t sources = load_or_zero(p.gather_index, static_cast<size_t>(max(mine, 0)), mine >= 0);
        sum.add(mine, mine >= 0 ? sources : -1, n);
    };
    if (count > 0) {
        arrivals_in_order(first_half, second_half, count, area, lane);
        hand_on(first_half, min(count, WAVE));
    }
    if (count > WAVE) {
        hand_on(second_half, count - WAVE);
    }
    return count > 0;
}

template <typename T> struct ContractArgs {
    Contraction<T> contraction;
    Table table;
    const T* C;
    int32_t n_units;             // chunks of positions x column tiles
    const int32_t* sorted_index; // [n_edges] node of every position, non-decreasing
};

/// Wavefronts per SIMD the registers are limited to, by element type and
/// accumulator tiles; a workgroup is that many wavefronts on each of the four
/// SIMDs of a compute unit, i.e. ONE workgroup per compute unit.
template <typename T, int NB> constexpr int waves_per_simd() {
    return sizeof(T) == 4 ? (NB <= 9 ? 4 : 3) : (NB <= 4 ? 4 : 2);
}
template <typename T, int NB> constexpr int group_threads() { return 4 * waves_per_simd<T, NB>() * WAVE; }

constexpr int32_t NO_UNIT = 0x7fffffff; // (a turn beyond the last unit)

/// What a wavefront asks for ahead of a unit of work: nothing of it depends
/// on anything but the unit's number.
struct UnitAhead {
    ChunkIndex index;
    int32_t near_source[2]; // blocks of the 128 positions from the chunk's first
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
template <typename T, int NB, bool EXACT, int CHUNK, bool GENERAL = false>
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
    NodeSum<T, NB, EXACT, false, GENERAL> sum(p, registers);
    // Unit u is column tile u mod column_tiles of chunk u / column_tiles. The
    // column tiles of a chunk are consecutive turns of ONE workgroup (chunks
    // group, group + n_groups, ...): its wavefronts then ask for the same rows at
    // about the same time, and a row comes from memory once instead of once per
    // column tile (half a cache line each, on compute units of different XCDs).
    const int32_t n_chunks = args.n_units / p.column_tiles;
    auto unit_of_turn = [&](int32_t turn) {
        const int32_t round = turn / p.column_tiles;
        const int32_t chunk = group + round * n_groups;
        return chunk < n_chunks ? chunk * p.column_tiles + (turn - round * p.column_tiles) : NO_UNIT;
    };
    auto take_turn = [&]() {
        int32_t turn = 0;
        if (lane == 0) {
            turn = atomicAdd(next_turn, 1);
        }
        return __builtin_amdgcn_readfirstlane(turn);
    };
    auto look_ahead = [&](UnitAhead& ahead, int32_t unit) {
        const bool exists = unit < args.n_units;
        const int32_t item = exists ? unit / p.column_tiles : 0; // chunk
        ahead.index = load_chunk_index<CHUNK>(args.sorted_index, p.n_edges, item);
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int32_t position = item * CHUNK + h * WAVE + lane;
            const int32_t source = load_or_zero(p.gather_index, static_cast<size_t>(position), position < p.n_edges);
            ahead.near_source[h] = position < p.n_edges ? source : -1;
        }
    };

    // everything that can be asked for without knowing anything is asked for
    // first; the table is built while it is on its way
    int32_t unit = unit_of_turn(wave);
    UnitAhead current;
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

    while (unit < args.n_units) {
        const int32_t next_unit = unit_of_turn(take_turn());
        UnitAhead next;
        look_ahead(next, next_unit);
        const int32_t item = unit / p.column_tiles;
        sum.set_column_tile(unit - item * p.column_tiles);
        const int32_t chunk_begin = item * CHUNK;
        walk_owned_segments<CHUNK>(
            args.sorted_index, p.n_edges, p.n_blocks, item, current.index,
            [&](int32_t node, int32_t first, int32_t last) {
                sum.clear();
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
                wait_for_table();
                sum.finish(table, registers, node);
            },
            [&](int32_t begin, int32_t end) { sum.clear_rows(begin, end); }
        );
        unit = next_unit;
        current = next;
    }
}

// ---------------------------------------------------------------------------
// grad_A and grad_B
//
// With G = grad_output, i the receiver of edge e and j its sender:
//
//   Z'_i[m1, m2, l] = sum_m3 D[m3, m2, m1] * G[i, m3, l]          once per node i (segment of the sorted index)
//   grad_A[e, m1]   = sum_{m2, l} Z'_i[m1, m2, l] * (B[e, l] * W[j, m2, l])
//   grad_B[e, l]    = sum_m2 W[j, m2, l] * sum_m1 A[e, m1] * Z'_i[m1, m2, l]
//
// Both are matrix products with 16 edges of the segment as one dimension and
// Z'_i, which all edges of the segment share, as one operand. Z'_i is itself a
// product of the dense table with G[i] and comes out of the matrix cores in
// exactly the register layout the next product wants it in (that is what the
// layouts ALPHA and BETA of the table are for), so nothing goes through LDS.
//   grad_B of a tile of 16 columns l:   Z' as 16 columns x pairs (m1, m2): 27 steps per 16 edges (nA = n2 = 9)
//   grad_A, 16 columns l at a time:     Z' as m1 x (m2, l):                36 steps per 16 edges and 16 columns
// A wavefront does one of these for all segments that start in a chunk of 16
// positions: the roles are units of work of the same kind as in contract_kernel.

template <typename T> struct GradientArgs {
    const T* A;  // [n_edges][nA]
    const T* B;  // [n_edges][L]
    const T* W;  // [n_nodes][n2][L]
    const T* G;  // [n_nodes][n3][L]  grad_output
    const T* C;  // [N]
    T* grad_A;   // null: not wanted
    T* grad_B;
    T* grad_W;
    const int32_t* receivers; // sorted
    const int32_t* senders;
    int32_t n_edges, n_nodes, nA, L, n2, n3, column_tiles;
    Table table_W, table_alpha, table_beta;
    int32_t edge_roles;   // units per chunk: (grad_A ? 1 : 0) + (grad_B ? column_tiles : 0)
    int32_t edge_chunk;   // positions of the sorted index per unit of the per-edge gradients: 16, 32 or 64
    int32_t n_edge_units; // chunks * edge_roles
    int32_t n_W_units;    // n_nodes * column_tiles when grad_W is wanted; these units come last (measured: 6 to 10 us
                          // slower at 60 000 edges when they come first)
    int32_t n_units;      // the sum
    // the senders' edges: in slots (sender_buckets.hpp: SenderSlots), or, `by_arrival`, as SenderArrivals
    // with a counter for every (column tile, node), which the unit that reads it sets back to zero
    const int32_t* slot_edges;
    int32_t* slot_counts;
    bool by_arrival;
    // A launch that works on a part of the index ranges (gradients_kernel<.., GENERAL>): A, W, G,
    // grad_A and grad_W point to the first component / row of the part, nA, n2 and n3 count the
    // part, and these are the full extents; a gradient whose flag is set is added to (another part
    // of its sum is there already).
    int32_t lda, w_stride_rows, g_stride_rows;
    bool add_to_A, add_to_B, add_to_W;
};

template <typename T, int NB, bool EXACT, bool VECTORS, bool GENERAL = false> struct EdgeGradients {
    using M = Mfma<T>;
    static constexpr uint32_t ELEMENT = sizeof(T);

    const GradientArgs<T>& p;
    int lane, i, q;
    int32_t steps1, steps3_of_shape; // ceil(nA / 4), ceil(n3 / 4)
    uint32_t row_bytes, w_block_bytes, g_block_bytes, a_row_bytes;
    BufferOf<T> A, B, W, G;

    __device__ __forceinline__ EdgeGradients(const GradientArgs<T>& args) : p(args) {
        lane = threadIdx.x & (WAVE - 1);
        i = lane & 15;
        q = lane >> 4;
        steps1 = (p.nA + 3) / 4;
        steps3_of_shape = (p.n3 + 3) / 4;
        row_bytes = static_cast<uint32_t>(p.L) * ELEMENT;
        w_block_bytes = static_cast<uint32_t>(GENERAL ? p.w_stride_rows : p.n2) * row_bytes;
        g_block_bytes = static_cast<uint32_t>(GENERAL ? p.g_stride_rows : p.n3) * row_bytes;
        a_row_bytes = static_cast<uint32_t>(GENERAL ? p.lda : p.nA) * ELEMENT;
        // (GENERAL: the limits lie up to a row behind the ends of the tensors, see NodeSum)
        A.set(p.A, static_cast<uint32_t>(p.n_edges) * a_row_bytes);
        B.set(p.B, static_cast<uint32_t>(p.n_edges) * row_bytes);
        W.set(p.W, static_cast<uint32_t>(p.n_nodes) * w_block_bytes);
        G.set(p.G, static_cast<uint32_t>(p.n_nodes) * g_block_bytes);
    }

    __device__ __forceinline__ bool has_row(int c) const { return EXACT || c < p.n2; }
    /// ceil(n3 / 4): known when the kernel is compiled if no row is padding, and
    /// the loops over it then have no branch between a read of the table and
    /// the matrix instruction it feeds (with one, every such pair waits for
    /// the LDS by itself).
    __device__ __forceinline__ int32_t steps3_now() const { return EXACT ? (NB + 3) / 4 : steps3_of_shape; }

    /// grad_B[e, 16 tile .. 16 tile + 16] for the edges first .. last of `node`.
    /// `near_source`: senders of the 128 positions from `near_begin`.
    __device__ __forceinline__ void grad_B_of_segment(
        const T* __restrict__ table, int32_t node, int32_t first, int32_t last, int32_t tile,
        const int32_t (&near_source)[2], int32_t near_begin
    ) const {
        const int lane = opaque(this->lane);
        const int i = lane & 15, q = lane >> 4;
        const int32_t column = 16 * tile + i;
        const bool column_inside = column < p.L;
        const uint32_t column_bytes = static_cast<uint32_t>(min(column, p.L - 1)) * ELEMENT;
        // Z'_i as right operand: lane (column, q) holds, for pair (s, m2), Z'[4 s + q, m2, column]
        T g_rows[4];
#pragma unroll
        for (int s3 = 0; s3 < 4; s3++) {
            const int32_t m3 = 4 * s3 + q;
            g_rows[s3] = G.load(
                (static_cast<uint32_t>(node) * g_block_bytes + static_cast<uint32_t>(min(m3, p.n3 - 1)) * row_bytes +
                 column_bytes) |
                    unless(m3 < p.n3 && column_inside),
                0
            );
        }
        const int32_t pair_tiles = (steps1 * NB + 3) / 4;
        typename M::Acc pairs[NB]; // (4 * NB pairs at most)
#pragma unroll
        for (int t = 0; t < NB; t++) {
            pairs[t] = M::zero();
        }
        // (step by step over all tiles: consecutive matrix instructions belong to
        // different tiles and do not wait for each other)
#pragma unroll
        for (int s3 = 0; s3 < 4; s3++) {
            if (s3 < steps3_now()) {
#pragma unroll
                for (int t = 0; t < NB; t++) {
                    if (t < pair_tiles) { // (uniform)
                        pairs[t] = M::mma(table[(t * steps3_now() + s3) * WAVE + lane], g_rows[s3], pairs[t]);
                    }
                }
            }
        }
        for (int32_t base = first; base < last; base += 16) {
            const int32_t n = min(16, last - base);
            // the edge of row `row` of the tile, and its sender
            auto edge_of_row = [&](int row, int32_t& edge, int32_t& sender) {
                const int32_t position = base + row;
                edge = row < n ? position : -1;
                const int32_t offset = position - near_begin;
                if (base + 15 - near_begin < 2 * WAVE) { // (uniform: the whole tile is at hand)
                    const int32_t s0 = __shfl(near_source[0], offset & (WAVE - 1));
                    const int32_t s1 = __shfl(near_source[1], offset & (WAVE - 1));
                    sender = offset < WAVE ? s0 : s1;
                } else {
                    sender = load_or_zero(p.senders, static_cast<size_t>(max(edge, 0)), edge >= 0);
                }
            };
            // left operand: lane (edge i, q) holds A[edge, 4 s + q]
            int32_t my_edge, my_sender;
            edge_of_row(i, my_edge, my_sender);
            T a_rows[4];
#pragma unroll
            for (int s = 0; s < 4; s++) {
                const int32_t m1 = 4 * s + q;
                a_rows[s] = A.load(
                    (static_cast<uint32_t>(max(my_edge, 0)) * a_row_bytes + static_cast<uint32_t>(min(m1, p.nA - 1)) * ELEMENT) |
                        unless(my_edge >= 0 && m1 < p.nA),
                    0
                );
            }
            // the rows of W of the four edges this lane holds results for
            int32_t row_edge[4];
            T w[4][NB];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                int32_t sender;
                edge_of_row(M::row(lane, r), row_edge[r], sender);
                const bool usable = row_edge[r] >= 0 && in_bounds(sender, p.n_nodes) && column_inside;
                const uint32_t from =
                    (static_cast<uint32_t>(usable ? sender : 0) * w_block_bytes + column_bytes) | unless(usable);
#pragma unroll
                for (int c = 0; c < NB; c++) {
                    w[r][c] = W.load(from, fresh(static_cast<uint32_t>(EXACT ? c : min(c, p.n2 - 1))) * row_bytes);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            // Y'[edge, m2, column] = sum_m1 A[edge, m1] Z'[m1, m2, column]
            T result[4] = {T(0), T(0), T(0), T(0)};
#pragma unroll
            for (int c = 0; c < NB; c++) {
                if (has_row(c)) {
                    typename M::Acc y = M::zero();
#pragma unroll
                    for (int s = 0; s < 4; s++) {
                        if (s < steps1) {
                            y = M::mma(a_rows[s], pairs[(s * NB + c) >> 2][(s * NB + c) & 3], y);
                        }
                    }
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        result[r] += y[r] * w[r][c];
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < 4; r++) {
                if (row_edge[r] >= 0 && column_inside) {
                    T* target = p.grad_B + static_cast<size_t>(row_edge[r]) * p.L + column;
                    if constexpr (GENERAL) {
                        if (p.add_to_B) { // (uniform)
                            result[r] += *target;
                        }
                    }
                    *target = result[r];
                }
            }
        }
    }

    /// grad_A[e, :] for the edges first .. last of `node`.
    __device__ __forceinline__ void grad_A_of_segment(
        const T* __restrict__ table, int32_t node, int32_t first, int32_t last, const int32_t (&near_source)[2],
        int32_t near_begin
    ) const {
        // tiles of 16 edges whose sums over the columns are in registers together (Z' of a
        // column tile serves them all; measured at 60 000 edges with 1 / 2 / 4: float
        // 62.7 / 59.9 / 62.9 us, double 111.7 / 106.2 / 121.6)
        constexpr int TILES = 2;
        const int lane = opaque(this->lane);
        const int i = lane & 15, q = lane >> 4;
        // row `row` of a tile of Z' stands for column 4 q + r of the 16 (the lane
        // that holds it, and the register): consecutive columns in one lane
        const int local_column = sizeof(T) == 4 ? i : 4 * (i & 3) + (i >> 2);
        for (int32_t base = first; base < last; base += 16 * TILES) {
            const int32_t n = min(16 * TILES, last - base);
            const int32_t n_tiles = (n + 15) / 16;
            // the edge of this lane's column of tile t, and its sender
            int32_t my_edge[TILES], my_sender[TILES];
#pragma unroll
            for (int t = 0; t < TILES; t++) {
                const int32_t position = base + 16 * t + i;
                my_edge[t] = 16 * t + i < n ? position : -1;
                const int32_t offset = position - near_begin;
                if (base + 16 * t + 15 - near_begin < 2 * WAVE) { // (uniform: the whole tile is at hand)
                    const int32_t s0 = __shfl(near_source[0], offset & (WAVE - 1));
                    const int32_t s1 = __shfl(near_source[1], offset & (WAVE - 1));
                    my_sender[t] = offset < WAVE ? s0 : s1;
                } else {
                    my_sender[t] = load_or_zero(p.senders, static_cast<size_t>(max(my_edge[t], 0)), my_edge[t] >= 0);
                }
            }
            typename M::Acc sums[TILES];
#pragma unroll
            for (int t = 0; t < TILES; t++) {
                sums[t] = M::zero();
            }
            for (int32_t tile = 0; tile < p.column_tiles; tile++) {
                // Z'_i of these 16 columns as left operand: lane (m1, q), register r of
                // tile m2: Z'[m1, m2, 16 tile + 4 q + r]
                T g_columns[4];
                const int32_t column = 16 * tile + local_column;
#pragma unroll
                for (int s3 = 0; s3 < 4; s3++) {
                    const int32_t m3 = 4 * s3 + q;
                    g_columns[s3] = G.load(
                        (static_cast<uint32_t>(node) * g_block_bytes +
                         static_cast<uint32_t>(min(m3, p.n3 - 1)) * row_bytes +
                         static_cast<uint32_t>(min(column, p.L - 1)) * ELEMENT) |
                            unless(m3 < p.n3 && column < p.L),
                        0
                    );
                }
                typename M::Acc z[NB];
#pragma unroll
                for (int c = 0; c < NB; c++) {
                    z[c] = M::zero();
                }
#pragma unroll
                for (int s3 = 0; s3 < 4; s3++) {
                    if (s3 < steps3_now()) {
#pragma unroll
                        for (int c = 0; c < NB; c++) {
                            if (has_row(c)) {
                                z[c] = M::mma(g_columns[s3], table[(c * steps3_now() + s3) * WAVE + lane], z[c]);
                            }
                        }
                    }
                }
                const int32_t first_column = 16 * tile + 4 * q; // of this lane's four
                const int32_t inside = p.L - first_column;      // columns from there on that exist
#pragma unroll
                for (int t = 0; t < TILES; t++) {
                    if (t < n_tiles) { // (uniform)
                        const bool usable = my_edge[t] >= 0 && in_bounds(my_sender[t], p.n_nodes);
                        T b[4];
                        load_four<T, VECTORS>(
                            b, B,
                            static_cast<uint32_t>(max(my_edge[t], 0)) * row_bytes +
                                static_cast<uint32_t>(min(first_column, p.L - 1)) * ELEMENT,
                            0, inside, unless(usable)
                        );
                        const uint32_t from = static_cast<uint32_t>(usable ? my_sender[t] : 0) * w_block_bytes +
                                              static_cast<uint32_t>(min(first_column, p.L - 1)) * ELEMENT;
                        T w[NB][4];
#pragma unroll
                        for (int c = 0; c < NB; c++) {
                            load_four<T, VECTORS>(
                                w[c], W, from, fresh(static_cast<uint32_t>(EXACT ? c : min(c, p.n2 - 1))) * row_bytes, inside,
                                unless(usable)
                            );
                        }
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int c = 0; c < NB; c++) {
                            if (has_row(c)) {
#pragma unroll
                                for (int r = 0; r < 4; r++) {
                                    sums[t] = M::mma(z[c][r], w[c][r] * b[r], sums[t]);
                                }
                            }
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
#pragma unroll
            for (int t = 0; t < TILES; t++) {
                if (t < n_tiles && my_edge[t] >= 0) {
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const int32_t m1 = M::row(lane, r);
                        if (m1 < p.nA) {
                            T* target = p.grad_A + static_cast<size_t>(my_edge[t]) * (GENERAL ? p.lda : p.nA) + m1;
                            T value = sums[t][r];
                            if constexpr (GENERAL) {
                                if (p.add_to_A) { // (uniform)
                                    value += *target;
                                }
                            }
                            *target = value;
                        }
                    }
                }
            }
        }
    }
};

/// grad_A, grad_B and grad_W in one persistent launch (see contract_kernel for
/// how the units of work are dealt out): the per-edge gradients of the segments
/// that start in a chunk of 16, 32 or 64 positions, one unit for grad_A and one for
/// every 16 columns of grad_B, then grad_W of a node from its slots, one unit for
/// every 16 columns. Three wavefronts build the three layouts of the table side
/// by side.
/// Wavefronts per SIMD of the gradient kernel (it needs more registers than
/// contract_kernel: Z' of a node, the rows of W of 16 edges and the sums).
template <typename T, int NB> constexpr int gradient_waves_per_simd() { return sizeof(T) == 4 && NB <= 9 ? 3 : 2; }
template <typename T, int NB> constexpr int gradient_group_threads() {
    return 4 * gradient_waves_per_simd<T, NB>() * WAVE;
}

/// EXACT: n2 = n3 = NB, no row of a block is padding (otherwise the block rows are
/// compared with n2 / n3 as the loops go).
template <typename T, int NB, bool EXACT, bool VECTORS, bool ARRIVALS, bool GENERAL = false>
__global__ __launch_bounds__((gradient_group_threads<T, NB>())) void gradients_kernel(const GradientArgs<T> args) {
    constexpr int THREADS = gradient_group_threads<T, NB>();
    constexpr int GROUP_WAVES = THREADS / WAVE;
    static_assert(GROUP_WAVES >= 3, "a wavefront per layout of the table");
    extern __shared__ __align__(16) char lds_raw[];
    // the three layouts of the table, then an array of owners for each (build_table)
    T* const table_W = reinterpret_cast<T*>(lds_raw);
    T* const table_alpha = table_W + args.table_W.slots();
    T* const table_beta = table_alpha + args.table_alpha.slots();
    int32_t* const owner_W = reinterpret_cast<int32_t*>(table_beta + args.table_beta.slots());
    int32_t* const owner_alpha = owner_W + args.table_W.slots();
    int32_t* const owner_beta = owner_alpha + args.table_alpha.slots();
    int32_t* next_turn = owner_beta + args.table_beta.slots();
    int32_t* table_ready = next_turn + 1; // [3]: W, alpha, beta

    const int lane = threadIdx.x & (WAVE - 1);
    const int32_t wave = threadIdx.x >> 6;
    int32_t* const sorting_area = table_ready + 3 + wave * SLOT_CAPACITY; // (arrivals_in_order)
    const int32_t group = static_cast<int32_t>(blockIdx.x);
    const int32_t n_groups = static_cast<int32_t>(gridDim.x);
    const bool want_W = args.grad_W != nullptr, want_A = args.grad_A != nullptr, want_B = args.grad_B != nullptr;

    Contraction<T> contraction;
    contraction.A = args.A;
    contraction.B = args.B;
    contraction.rows = args.G;
    contraction.gather_index = args.receivers;
    contraction.result = args.grad_W;
    contraction.n_edges = args.n_edges;
    contraction.n_blocks = args.n_nodes;
    contraction.nA = args.nA;
    contraction.L = args.L;
    contraction.ld = args.L;
    contraction.n_red = args.n3;
    contraction.n_out = args.n2;
    contraction.column_tiles = args.column_tiles;
    contraction.lda = GENERAL ? args.lda : args.nA;
    contraction.rows_stride = GENERAL ? args.g_stride_rows : args.n3;
    contraction.out_stride = GENERAL ? args.w_stride_rows : args.n2;
    contraction.accumulate = GENERAL && args.add_to_W;
    NodeSum<T, NB, EXACT, true, GENERAL> sum(contraction, args.table_W.registers);
    EdgeGradients<T, NB, EXACT, VECTORS, GENERAL> edges(args);

    // Turn k of this workgroup is unit group + k * n_groups: the roles of a chunk
    // go to neighbouring workgroups. (Giving them to the wavefronts of one
    // workgroup, so that the rows they share come from memory once, takes a
    // third off the bytes read and is SLOWER: 65 -> 66 us in float, 104 -> 112 us
    // in double at 60 000 edges. Roles of different length then end side by side.)
    auto unit_of_turn = [&](int32_t turn) { return group + turn * n_groups; };
    auto take_turn = [&]() {
        int32_t turn = 0;
        if (lane == 0) {
            turn = atomicAdd(next_turn, 1);
        }
        return __builtin_amdgcn_readfirstlane(turn);
    };
    // what is asked for ahead of a unit: of a chunk, the index values around
    // it and the senders of the 128 positions from its first; of a node, its slots
    struct Ahead {
        int32_t v[6];
    };
    auto look_ahead = [&](Ahead& ahead, int32_t unit) {
        const bool exists = unit < args.n_units;
        if (!exists || unit < args.n_edge_units) {
            const int32_t chunk = exists ? unit / args.edge_roles : 0;
            const ChunkIndex index = load_chunk_index_of(args.receivers, args.n_edges, chunk, args.edge_chunk);
            ahead.v[0] = index.mine;
            ahead.v[1] = index.before;
            ahead.v[2] = index.ahead;
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int32_t position = chunk * args.edge_chunk + h * WAVE + lane;
                const int32_t sender =
                    load_or_zero(args.senders, static_cast<size_t>(position), position < args.n_edges);
                ahead.v[3 + h] = position < args.n_edges ? sender : -1;
            }
            ahead.v[5] = 0;
        } else {
            const int32_t item = unit - args.n_edge_units;
            const int32_t node = item / args.column_tiles;
            const int32_t* mine = args.slot_edges + static_cast<size_t>(node) * SLOT_CAPACITY;
            ahead.v[0] = mine[lane];
            ahead.v[1] = mine[lane + WAVE];
            if constexpr (ARRIVALS) {
                const int32_t tile = item - node * args.column_tiles;
                ahead.v[2] = args.slot_counts[static_cast<size_t>(tile) * args.n_nodes + node];
                ahead.v[3] = 0;
                ahead.v[4] = 0;
                ahead.v[5] = 0;
            } else {
                const int4 counts = reinterpret_cast<const int4*>(args.slot_counts)[node];
                ahead.v[2] = counts.x;
                ahead.v[3] = counts.y;
                ahead.v[4] = counts.z;
                ahead.v[5] = counts.w;
            }
        }
    };

    int32_t unit = unit_of_turn(wave);
    Ahead current;
    MyEntries<T> entries;
    // wavefront 0 builds the table of grad_W, 1 that of grad_A, 2 that of grad_B
    const bool builder = (wave == 0 && want_W) || (wave == 1 && want_A) || (wave == 2 && want_B);
    const Table& my_layout = wave == 0 ? args.table_W : wave == 1 ? args.table_alpha : args.table_beta;
    if (builder) {
        load_entries<T>(entries, args.C, my_layout, 0, lane);
    }
    look_ahead(current, unit);
    if (threadIdx.x == 0) {
        *next_turn = GROUP_WAVES;
        table_ready[0] = 0;
        table_ready[1] = 0;
        table_ready[2] = 0;
    }
    __syncthreads(); // (everybody is here at once: nothing has been waited for yet)
    bool seen_W = false, seen_alpha = false, seen_beta = false;
    if (builder) {
        T* my_table = wave == 0 ? table_W : wave == 1 ? table_alpha : table_beta;
        int32_t* my_owner = wave == 0 ? owner_W : wave == 1 ? owner_alpha : owner_beta;
        build_table<T>(my_table, my_owner, entries, args.C, my_layout, lane);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        if (lane == 0) {
            __hip_atomic_store(&table_ready[wave], 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
        seen_W = wave == 0;
        seen_alpha = wave == 1;
        seen_beta = wave == 2;
    }
    // (a builder depends on nobody, so the wait ends)
    auto wait_for = [&](bool& seen, int which) {
        if (!seen) {
            while (__hip_atomic_load(&table_ready[which], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) == 0) {
                __builtin_amdgcn_s_sleep(4);
            }
            seen = true;
        }
    };

    while (unit < args.n_units) {
        const int32_t next_unit = unit_of_turn(take_turn());
        Ahead next;
        look_ahead(next, next_unit);

        if (unit < args.n_edge_units) {
            const int32_t chunk = unit / args.edge_roles;
            const int32_t role = unit - chunk * args.edge_roles;
            const bool for_A = want_A && role == 0;
            const int32_t tile = role - (want_A ? 1 : 0);
            const ChunkIndex index{current.v[0], current.v[1], current.v[2]};
            const int32_t near_source[2] = {current.v[3], current.v[4]};
            if (for_A) {
                wait_for(seen_alpha, 1);
            } else {
                wait_for(seen_beta, 2);
            }
            walk_pieces_of<0>(
                args.receivers, args.n_edges, args.n_nodes, chunk, args.edge_chunk, index,
                [&](int32_t node, int32_t first, int32_t last, bool, bool) {
                    if (for_A) {
                        edges.grad_A_of_segment(table_alpha, node, first, last, near_source, chunk * args.edge_chunk);
                    } else {
                        edges.grad_B_of_segment(table_beta, node, first, last, tile, near_source, chunk * args.edge_chunk);
                    }
                },
                [&](int32_t, int32_t) {}
            );
        } else {
            const int32_t item = unit - args.n_edge_units;
            const int32_t node = item / args.column_tiles;
            const int32_t tile = item - node * args.column_tiles;
            sum.set_column_tile(tile);
            bool any;
            if constexpr (ARRIVALS) {
                const int32_t count = __builtin_amdgcn_readfirstlane(current.v[2]);
                if (lane == 0) {
                    // (nobody else reads this counter in this launch: zero again for the next one)
                    args.slot_counts[static_cast<size_t>(tile) * args.n_nodes + node] = 0;
                }
                any = sum_over_arrivals(sum, current.v[0], current.v[1], count, sorting_area, args.senders, node, lane);
            } else {
                const int4 counts = make_int4(current.v[2], current.v[3], current.v[4], current.v[5]);
                any = sum_over_slots(sum, current.v[0], current.v[1], counts, args.senders, node, lane);
            }
            if (any) {
                wait_for(seen_W, 0);
                sum.finish(table_W, args.table_W.registers, node);
            } else {
                sum.clear_rows(node, node + 1);
            }
        }
        unit = next_unit;
        current = next;
    }
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
    t.layout = Layout::RESULT;
    t.bucket = n_red;
    t.m1_begin = 0;
    t.red_begin = 0;
    t.out_begin = 0;
    return t;
}

/// Accumulator tiles: the block rows themselves when they are 1, 4, 9 or 16 (the
/// numbers of components of spherical harmonics up to some degree), otherwise
/// rounded up to one of those.
template <typename Launch> void with_block_rows(int32_t n_red, Launch&& launch) {
#ifdef MOPS_SEG_DEV
    launch(std::integral_constant<int, 9>{}, std::true_type{}); // (development builds: one size only)
#else
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
#endif
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
/// unit (measured at 60 000 edges, 2 column tiles: float, 4096 wavefronts: 25 us
/// with 16, 22 with 32, 29 with 64; double, 2048 wavefronts: 41, 36, 31.5).
int32_t chunk_for(int32_t n_edges, int32_t column_tiles, int64_t resident_waves) {
    for (int32_t chunk : {16, 32}) {
        if ((static_cast<int64_t>(n_edges) + chunk - 1) / chunk * column_tiles <= resident_waves) {
            return chunk;
        }
    }
    return 64;
}

template <typename T> void launch_contract(ContractArgs<T> args, hipStream_t stream, bool general = false) {
    const Contraction<T>& p = args.contraction;
    const size_t lds = table_lds(args.table, sizeof(T));
    with_block_rows(p.n_red, [&](auto block_rows, auto exact) {
        constexpr int NB = decltype(block_rows)::value;
        constexpr bool EXACT = decltype(exact)::value;
        constexpr int64_t GROUP_WAVES = group_threads<T, NB>() / WAVE;
        auto go = [&](auto chunk_constant, auto general_constant) {
            constexpr int CHUNK = decltype(chunk_constant)::value;
            const int64_t units = (static_cast<int64_t>(p.n_edges) + CHUNK - 1) / CHUNK * p.column_tiles;
            args.n_units = narrow_i32(static_cast<size_t>(units), "units of work");
            // one workgroup per compute unit, fewer when there is not a unit per wavefront
            // (a workgroup takes all column tiles of a chunk)
            const int64_t chunks = units / p.column_tiles;
            const int64_t chunks_per_round = std::max<int64_t>(GROUP_WAVES / p.column_tiles, 1);
            const unsigned grid = static_cast<unsigned>(
                std::min<int64_t>(compute_units(), (chunks + chunks_per_round - 1) / chunks_per_round)
            );
            auto kernel = contract_kernel<T, NB, EXACT, CHUNK, decltype(general_constant)::value>;
            allow_lds(kernel, lds);
            kernel<<<grid, group_threads<T, NB>(), lds, stream>>>(args);
        };
        if (general) {
            // (parts of larger tensors: one size of chunk, the one of the shapes the kernel was tuned on)
            go(std::integral_constant<int, 32>{}, std::true_type{});
            return;
        }
        switch (chunk_for(p.n_edges, p.column_tiles, GROUP_WAVES * compute_units())) {
        case 16:
            go(std::integral_constant<int, 16>{}, std::false_type{});
            break;
        case 32:
            go(std::integral_constant<int, 32>{}, std::false_type{});
            break;
        default:
            go(std::integral_constant<int, 64>{}, std::false_type{});
            break;
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
    c.lda = s.nA;
    c.rows_stride = n_red;
    c.out_stride = n_out;
    c.accumulate = false;
    return c;
}

} // namespace

static bool offsets_fit(const Shape& s, size_t element_size) {
    // 32-bit byte offsets into every tensor
    const uint64_t limit = uint64_t(1) << 32;
    const uint64_t widest = static_cast<uint64_t>(std::max(std::max(s.n2, s.n3), 1)) * s.L * element_size;
    return static_cast<uint64_t>(s.n_nodes) * widest < limit &&
           static_cast<uint64_t>(s.n_edges) * std::max(s.nA, s.L) * element_size < limit;
}

bool supports(const Shape& s, size_t element_size) {
    if (s.n_nodes < 1 || s.n_edges < 1 || s.N < 1 || s.N > MAX_TABLE || s.L < 1) {
        return false;
    }
    if (s.nA < 1 || s.nA > MAX_INDEX || s.n2 < 1 || s.n2 > MAX_INDEX || s.n3 < 1 || s.n3 > MAX_INDEX) {
        return false;
    }
    return offsets_fit(s, element_size);
}

// More than 16 values of a component index (forward pass): the sums over m1 and over the block
// rows are taken in parts of 16 each, a launch per pair of parts that adds to what the one before
// left, and the rows of the result in blocks of 16 inside a launch, as many as the table in LDS
// has room for (then the next launches). Every launch walks all edges again, so the parts are
// limited: MAX_PARTS launches.
constexpr int32_t MAX_PARTS = thresholds::SASAW_MAX_PARTS;
constexpr size_t GENERAL_TABLE_LDS = 144 * 1024; // of the 160 KB of a compute unit

/// Rows of the result per launch: whole blocks of 16, as many as fit the LDS with a table of
/// 4 registers x 16 block rows per block.
static int32_t result_rows_per_launch(const Shape& s, size_t element_size) {
    const size_t per_block = static_cast<size_t>(4) * std::min(s.n2, MAX_INDEX) * WAVE * (element_size + sizeof(int32_t));
    const int32_t blocks = static_cast<int32_t>(std::max<size_t>(1, (GENERAL_TABLE_LDS - 64) / per_block));
    return 16 * std::min(blocks, (s.n3 + 15) / 16);
}

bool supports_forward(const Shape& s, size_t element_size) {
    if (sasaw_segments::supports(s, element_size)) {
        return true;
    }
    if (s.n_nodes < 1 || s.n_edges < 1 || s.N < 1 || s.N > MAX_TABLE || s.L < 1 || s.nA < 1 || s.n2 < 1 || s.n3 < 1) {
        return false;
    }
    const int64_t parts = static_cast<int64_t>((s.nA + MAX_INDEX - 1) / MAX_INDEX) * ((s.n2 + MAX_INDEX - 1) / MAX_INDEX) *
                          ((s.n3 + result_rows_per_launch(s, element_size) - 1) / result_rows_per_launch(s, element_size));
    return parts <= MAX_PARTS && offsets_fit(s, element_size);
}

template <typename T>
void forward(
    T* output, const T* A, const T* B, const T* C, const T* W, const Indices& indices, const Shape& s,
    hipStream_t stream
) {
    MainKernelTimer timer(stream);
    if (sasaw_segments::supports(s, sizeof(T))) {
        ContractArgs<T> args{};
        args.contraction = contraction_of<T>(s, A, B, W, indices.W_1, output, s.n2, s.n3);
        args.table = table_of(s, indices.A, indices.W_2, indices.output_2, s.n2, s.n3);
        args.C = C;
        args.sorted_index = indices.output_1;
        launch_contract<T>(args, stream);
        return;
    }
    const int32_t rows_per_launch = result_rows_per_launch(s, sizeof(T));
    for (int32_t out_begin = 0; out_begin < s.n3; out_begin += rows_per_launch) {
        const int32_t n_out = std::min(rows_per_launch, s.n3 - out_begin);
        bool first = true;
        for (int32_t m1_begin = 0; m1_begin < s.nA; m1_begin += MAX_INDEX) {
            const int32_t nA = std::min(MAX_INDEX, s.nA - m1_begin);
            for (int32_t red_begin = 0; red_begin < s.n2; red_begin += MAX_INDEX) {
                const int32_t n_red = std::min(MAX_INDEX, s.n2 - red_begin);
                ContractArgs<T> args{};
                Contraction<T>& c = args.contraction;
                c = contraction_of<T>(s, A + m1_begin, B, W + static_cast<size_t>(red_begin) * s.L, indices.W_1,
                                      output + static_cast<size_t>(out_begin) * s.L, n_red, n_out);
                c.nA = nA;
                c.lda = s.nA;
                c.rows_stride = s.n2;
                c.out_stride = s.n3;
                c.accumulate = !first;
                args.table = table_of(s, indices.A, indices.W_2, indices.output_2, n_red, n_out);
                args.table.nA = nA;
                args.table.registers = (nA + 3) / 4;
                args.table.m1_begin = m1_begin;
                args.table.red_begin = red_begin;
                args.table.out_begin = out_begin;
                args.C = C;
                args.sorted_index = indices.output_1;
                launch_contract<T>(args, stream, true);
                first = false;
            }
        }
    }
}

/// Whether the persistent gradient kernel serves this vjp: the senders' edges
/// fit the slots on average (sparse graphs), which grad_W needs.
/// Whether the senders' edges are listed by arrival (one look at every edge,
/// an atomic for each) rather than in slots (every 16 senders look at the whole
/// index, which costs edges x nodes). Measured at 30 edges per node, whole vjp
/// in float, by arrival / in slots: 2000 nodes 66.7 / 60.7 us, 3000: 93.8 /
/// 92.8, 4000: 113.7 / 114.0, 6000: 170 / 179, 8000: 233 / 255, 20 000: 682 /
/// 820 (double alike). Graphs with 48 to 64 edges per node on average overflow the
/// slots (32 places per quarter of the index) but not the 128 places of a
/// sender's list by arrival: 1000 nodes with 60 edges each, whole vjp by arrival
/// against the older kernels of sasaw_mfma.hip: 76.6 / 87.6 us (float), 115.3 /
/// 143.8 (double); with 100 edges each the lists overflow too (375 / 101 us).
static bool dense_for_slots(const Shape& s) {
    return static_cast<size_t>(s.n_edges) > static_cast<size_t>(s.n_nodes) * thresholds::SLOT_MEAN_EDGES;
}
static bool lists_by_arrival(const Shape& s) {
    return (s.n_nodes > thresholds::ARRIVAL_NODES || dense_for_slots(s)) &&
           static_cast<size_t>(s.n_nodes) * ((s.L + 15) / 16) <= SCRATCH_COUNTERS;
}

/// Block rows (of W and of grad_output) per launch of the gradient kernel when the index ranges
/// are taken in parts: the kernel with 9 accumulator tiles does a row in less than half the time
/// of the one with 16 (measured on 13 x 7 x 100 components, 60 000 edges, float: 16 rows 222 us,
/// 9 rows 60 us per launch; in double the 16-tile kernel spills and is four times slower still).
constexpr int32_t GRADIENT_PART_ROWS = thresholds::SASAW_GRADIENT_PART_ROWS;

/// Whether the vjp is one launch on the whole index ranges. In double, also a shape with at most
/// 16 values of every index goes in parts when W or grad_output have more than 9 rows: the
/// 16-tile kernel spills its accumulators, and four launches on 9 and 7 rows take 0.83 of its
/// time (16 x 16 x 16 components, 64 columns, 60 000 edges: 784 against 950 us).
static bool vjp_in_one_launch(const Shape& s, size_t element_size) {
    return sasaw_segments::supports(s, element_size) &&
           !(element_size == 8 && std::max(s.n2, s.n3) > GRADIENT_PART_ROWS);
}

bool vjp_supported(const Shape& s, size_t element_size, bool want_grad_W) {
    if (vjp_in_one_launch(s, element_size)) {
        // (more than 48 edges per node on average: only by arrival, see lists_by_arrival)
        return !want_grad_W || !dense_for_slots(s) ||
               (static_cast<size_t>(s.n_edges) <= static_cast<size_t>(s.n_nodes) * thresholds::ARRIVAL_MEAN_EDGES && lists_by_arrival(s));
    }
    // more than 16 values of a component index: in parts (see vjp), every launch with the lists in
    // slots (a sender with more than 32 edges in a quarter of the index is served by a wavefront
    // that reads the whole index: rare up to 64 edges per node on average)
    if (s.n_nodes < 1 || s.n_edges < 1 || s.N < 1 || s.N > MAX_TABLE || s.L < 1 || s.nA < 1 || s.n2 < 1 || s.n3 < 1) {
        return false;
    }
    constexpr int32_t ROWS = GRADIENT_PART_ROWS;
    const int64_t parts =
        static_cast<int64_t>((s.nA + MAX_INDEX - 1) / MAX_INDEX) * ((s.n2 + ROWS - 1) / ROWS) * ((s.n3 + ROWS - 1) / ROWS);
    return parts <= MAX_PARTS && offsets_fit(s, element_size) &&
           (!want_grad_W || static_cast<size_t>(s.n_edges) <= static_cast<size_t>(s.n_nodes) * thresholds::ARRIVAL_MEAN_EDGES);
}

size_t vjp_workspace_bytes(const Shape& s, bool want_grad_W) {
    return want_grad_W ? sender_slots_bytes(s.n_nodes) : 0; // (enough for either way of listing)
}

size_t vjp_counters(const Shape& s, bool want_grad_W) {
    return want_grad_W && lists_by_arrival(s) ? static_cast<size_t>(s.n_nodes) * ((s.L + 15) / 16) : 0;
}

/// Positions of the sorted index per unit of the per-edge gradients: the most
/// of 64, 32, 16 that leave about one unit or more for each of `wanted_units`
/// (the resident wavefronts, twice as many for double, whose units take longer
/// and so even out worse). Measured at 60 000 edges, all three gradients,
/// with 16 / 32 / 64: float 71 / 70 / 66 us, double 111 / 105 / 113 us; grad_A
/// alone: float 34 / 36 / 54 us.
int32_t edge_chunk_for(int32_t n_edges, int32_t edge_roles, int64_t wanted_units) {
    for (int32_t chunk : {64, 32}) {
        const int64_t units = (static_cast<int64_t>(n_edges) + chunk - 1) / chunk * edge_roles;
        if (units * 10 >= wanted_units * 9) {
            return chunk;
        }
    }
    return 16;
}

/// The index ranges one launch of the gradient kernel works on.
struct Part {
    int32_t m1_begin, nA, m2_begin, n2, m3_begin, n3;
};

/// One launch of gradients_kernel for `part` of the shape `s`. `args` holds the tensors (already
/// pointing to the part), the lists of the senders' edges and the flags; `general`: the part is
/// not the whole shape (strides and offsets apply).
template <typename T>
void launch_gradients(
    GradientArgs<T> args, const Shape& s, const Part& part, const Indices& indices, bool general, hipStream_t stream
) {
    args.n_edges = s.n_edges;
    args.n_nodes = s.n_nodes;
    args.nA = part.nA;
    args.L = s.L;
    args.n2 = part.n2;
    args.n3 = part.n3;
    args.column_tiles = (s.L + 15) / 16;
    args.edge_roles = (args.grad_A != nullptr ? 1 : 0) + (args.grad_B != nullptr ? args.column_tiles : 0);
    const int64_t W_units = args.grad_W != nullptr ? static_cast<int64_t>(s.n_nodes) * args.column_tiles : 0;
    args.n_W_units = narrow_i32(static_cast<size_t>(W_units), "units of work");
    // (rows of B and W are read 16 bytes at a time where their alignment allows)
    const bool vectors = s.L % 4 == 0 && reinterpret_cast<uintptr_t>(args.B) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(args.W) % 16 == 0;
    Shape of_part = s;
    of_part.nA = part.nA;
    of_part.n2 = part.n2;
    of_part.n3 = part.n3;
    auto with_offsets = [&](Table table, int32_t red_begin, int32_t out_begin) {
        table.m1_begin = part.m1_begin;
        table.red_begin = red_begin;
        table.out_begin = out_begin;
        return table;
    };

    with_block_rows(std::max(part.n2, part.n3), [&](auto block_rows, auto fits) {
        constexpr int NB = decltype(block_rows)::value;
        // (more than GRADIENT_PART_ROWS rows: whole shapes in float only, see vjp_in_one_launch)
        if constexpr (NB > GRADIENT_PART_ROWS && sizeof(T) == 8) {
            throw std::logic_error("sasaw_segments: a launch on more than 9 rows in double");
        } else {
        // grad_W sums over the rows of grad_output (n3 of them), the others over those of W (n2)
        args.table_W = with_offsets(
            table_of(of_part, indices.A, indices.output_2, indices.W_2, part.n3, part.n2), part.m3_begin, part.m2_begin
        );
        args.table_alpha = with_offsets(
            table_of(of_part, indices.A, indices.W_2, indices.output_2, part.n2, part.n3), part.m2_begin, part.m3_begin
        );
        args.table_alpha.layout = Layout::ALPHA;
        args.table_beta = args.table_alpha;
        args.table_beta.layout = Layout::BETA;
        args.table_beta.bucket = NB;
        const size_t slots = static_cast<size_t>(args.table_W.slots()) + args.table_alpha.slots() + args.table_beta.slots();
        constexpr int GROUP_WAVES = gradient_group_threads<T, NB>() / WAVE;
        // (the tables, a counter and three flags, every wavefront's area for putting a sender's edges in order)
        const size_t lds = slots * (sizeof(T) + sizeof(int32_t)) + 32 +
                           (args.by_arrival ? GROUP_WAVES * SLOT_CAPACITY * sizeof(int32_t) : 0);
        const int64_t resident_waves = static_cast<int64_t>(GROUP_WAVES) * compute_units();
        args.edge_chunk = edge_chunk_for(s.n_edges, args.edge_roles, resident_waves * sizeof(T) / 4);
        const int64_t chunks = (static_cast<int64_t>(s.n_edges) + args.edge_chunk - 1) / args.edge_chunk;
        args.n_edge_units = narrow_i32(static_cast<size_t>(chunks * args.edge_roles), "units of work");
        const int64_t units = W_units + chunks * args.edge_roles;
        args.n_units = narrow_i32(static_cast<size_t>(units), "units of work");
        const unsigned grid =
            static_cast<unsigned>(std::min<int64_t>(compute_units(), (units + GROUP_WAVES - 1) / GROUP_WAVES));
        (void)fits;
        auto launch = [&](auto exact, auto with_vectors, auto arrivals, auto is_general) {
            auto kernel = gradients_kernel<
                T, NB, decltype(exact)::value, decltype(with_vectors)::value, decltype(arrivals)::value,
                decltype(is_general)::value>;
            allow_lds(kernel, lds);
            kernel<<<grid, gradient_group_threads<T, NB>(), lds, stream>>>(args);
        };
        const bool exact = part.n2 == NB && part.n3 == NB;
        if (general) {
            // (parts of larger index ranges: lists in slots only, one variant for rows with and without padding)
            if constexpr (NB > GRADIENT_PART_ROWS) {
                throw std::logic_error("sasaw_segments: a part of more than 9 rows");
            } else {
                if (vectors) {
                    launch(std::false_type{}, std::true_type{}, std::false_type{}, std::true_type{});
                } else {
                    launch(std::false_type{}, std::false_type{}, std::false_type{}, std::true_type{});
                }
                return;
            }
        }
        auto with_lists = [&](auto is_exact, auto with_vectors) {
            if (args.by_arrival) {
                launch(is_exact, with_vectors, std::true_type{}, std::false_type{});
            } else {
                launch(is_exact, with_vectors, std::false_type{}, std::false_type{});
            }
        };
        if (exact && vectors) {
            with_lists(std::true_type{}, std::true_type{});
        } else if (exact) {
            with_lists(std::true_type{}, std::false_type{});
        } else if (vectors) {
            with_lists(std::false_type{}, std::true_type{});
        } else {
            with_lists(std::false_type{}, std::false_type{});
        }
        }
    });
    MOPS_HIP_CHECK(hipGetLastError());
}

template <typename T>
void vjp(
    T* grad_A, T* grad_B, T* grad_W, const T* grad_output, const T* A, const T* B, const T* C, const T* W,
    const Indices& indices, const Shape& s, void* workspace, int32_t* counters, bool counters_are_zero,
    hipStream_t stream
) {
    GradientArgs<T> args{};
    args.A = A;
    args.B = B;
    args.W = W;
    args.G = grad_output;
    args.C = C;
    args.grad_A = grad_A;
    args.grad_B = grad_B;
    args.grad_W = grad_W;
    args.receivers = indices.output_1;
    args.senders = indices.W_1;
    args.lda = s.nA;
    args.w_stride_rows = s.n2;
    args.g_stride_rows = s.n3;
    const bool whole = vjp_in_one_launch(s, sizeof(T));
    if (grad_W != nullptr) {
        // the edges of every sender, listed by a launch of its own in front
        args.by_arrival = whole && lists_by_arrival(s);
        if (args.by_arrival) {
            if (!counters_are_zero) {
                clear_counters(counters, vjp_counters(s, true), stream);
            }
            const SenderArrivals lists = list_edges_by_arrival(
                indices.W_1, s.n_edges, s.n_nodes, (s.L + 15) / 16, workspace, counters, stream
            );
            args.slot_edges = lists.edges;
            args.slot_counts = lists.counts;
            test_failure_point("sasaw_vjp_after_listing");
        } else {
            const SenderSlots slots = list_edges_in_slots(indices.W_1, s.n_edges, s.n_nodes, workspace, stream);
            args.slot_edges = slots.edges;
            args.slot_counts = const_cast<int32_t*>(slots.counts);
        }
    }
    MainKernelTimer timer(stream);
    if (whole) {
        launch_gradients<T>(args, s, Part{0, s.nA, 0, s.n2, 0, s.n3}, indices, false, stream);
        return;
    }
    // More than 16 values of a component index: the ranges in parts, a launch per triple of
    // parts; a gradient is a sum over the parts of the two ranges it does not have as an index
    // (grad_B: of all three), so all launches but the first of such a sum add to what is there.
    for (int32_t m1_begin = 0; m1_begin < s.nA; m1_begin += MAX_INDEX) {
        for (int32_t m2_begin = 0; m2_begin < s.n2; m2_begin += GRADIENT_PART_ROWS) {
            for (int32_t m3_begin = 0; m3_begin < s.n3; m3_begin += GRADIENT_PART_ROWS) {
                const Part part{
                    m1_begin, std::min(MAX_INDEX, s.nA - m1_begin), m2_begin,
                    std::min(GRADIENT_PART_ROWS, s.n2 - m2_begin), m3_begin,
                    std::min(GRADIENT_PART_ROWS, s.n3 - m3_begin)};
                GradientArgs<T> of_part = args;
                of_part.A = A + m1_begin;
                of_part.W = W + static_cast<size_t>(m2_begin) * s.L;
                of_part.G = grad_output + static_cast<size_t>(m3_begin) * s.L;
                of_part.grad_A = grad_A != nullptr ? grad_A + m1_begin : nullptr;
                of_part.grad_W = grad_W != nullptr ? grad_W + static_cast<size_t>(m2_begin) * s.L : nullptr;
                of_part.add_to_A = m2_begin > 0 || m3_begin > 0;
                of_part.add_to_B = m1_begin > 0 || m2_begin > 0 || m3_begin > 0;
                of_part.add_to_W = m1_begin > 0 || m3_begin > 0;
                launch_gradients<T>(of_part, s, part, indices, true, stream);
            }
        }
    }
}

template void forward<float>(
    float*, const float*, const float*, const float*, const float*, const Indices&, const Shape&, hipStream_t
);
template void forward<double>(
    double*, const double*, const double*, const double*, const double*, const Indices&, const Shape&, hipStream_t
);
template void vjp<float>(
    float*, float*, float*, const float*, const float*, const float*, const float*, const float*, const Indices&,
    const Shape&, void*, int32_t*, bool, hipStream_t
);
template void vjp<double>(
    double*, double*, double*, const double*, const double*, const double*, const double*, const double*,
    const Indices&, const Shape&, void*, int32_t*, bool, hipStream_t
);

} // namespace mops::amd::sasaw_segments
