// SAP on the matrix cores of gfx950.
//
//   O[i, PO[k]] += C[k] * A[i, PA[k]] * B[i, PB[k]]
//
// (semantics: mops/src/sap/cpu.tpp:10-255 of lab-cosmo/mops). When the three
// index ranges are small the table is a small dense tensor
//
//   M[a, b, o] = sum of C[k] over entries with (PA[k], PB[k], PO[k]) == (a, b, o)
//
// and all three functions are products of a matrix of per-row pair products
// with a reshaping of M, done 16 rows at a time with v_mfma_*_16x16x4:
//
//   O[i, o]      = sum_{(a, b)} (A[i, a] * B[i, b])  * M[(a, b), o]
//   grad_A[i, a] = sum_{(b, o)} (B[i, b] * gO[i, o]) * M[a, (b, o)]
//   grad_B[i, b] = sum_{(a, o)} (A[i, a] * gO[i, o]) * M[b, (a, o)]
//
// The pairs are enumerated as (x, 4 g + q): x runs over the first index of the
// pair ("outer"), g over groups of four values of the second ("inner") and
// q = lane >> 4 is the position of a lane's quarter of the wavefront in the
// reduction dimension of the matrix instruction. A lane keeps the inner values
// of its row in registers and fetches the outer value once per x; a pair
// product is one multiplication.
//
// Every workgroup builds the reshaped M it needs in LDS from the raw table
// (build_operand): no second kernel, no table in global memory, and the same
// bits in every workgroup and on every run.
//
// Two sets of kernels. forward_kernel / vjp_kernel: a workgroup for every 128
// rows, two wavefronts per tile of 16 rows; what launches of up to a few
// tiles per wavefront of the device take. forward_walk_kernel /
// vjp_walk_kernel: as many workgroups as the device holds, each builds M once
// and its wavefronts then walk over tiles of their own; what launches of
// hundreds of thousands of rows take (walks() has the measured thresholds).
#include "sap_mfma.hpp"

#include <algorithm>
#include <stdexcept>
#include <type_traits>

#include <hip/hip_ext.h>

#include "device_common.hpp"
#include "dispatch_thresholds.hpp"
#include "mfma.hpp"
#include "runtime.hpp"

namespace mops::amd::sap_mfma {
namespace {

constexpr int WAVES = 8;          // wavefronts per workgroup
constexpr int ROW_TILES = 1;      // tiles of 16 rows per wavefront
constexpr int ROWS_PER_WAVE = 16 * ROW_TILES;
constexpr int ROWS_PER_GROUP = WAVES * ROWS_PER_WAVE;
constexpr int THREADS = 2 * WAVES * WAVE; // two wavefronts per tile of 16 rows
constexpr int MAX_INNER_GROUPS_FORWARD = 4; // nB <= 16
constexpr int MAX_INNER_GROUPS_VJP = 16;    // nO <= 64
constexpr int MAX_OUTER = 16;
constexpr int MAX_ENTRIES = 8192;
constexpr size_t LDS_BUDGET = 156 * 1024; // of the 160 KB of a compute unit (16 values of every index in double need 153 KB for the vjp)
constexpr size_t LDS_WITHOUT_ASKING = 64 * 1024;

__host__ __device__ constexpr size_t align16(size_t bytes) { return (bytes + 15) & ~static_cast<size_t>(15); }

/// How a reshaped M is laid out as right operand:
///   operand[((x * n_groups + g) * n_tiles + t) * 64 + 16 q + j]
///     = M[outer = x, inner = 4 g + q, column = 16 t + j]
struct OperandShape {
    int32_t n_outer, n_inner, n_columns;
    int32_t n_groups; // ceil(n_inner / 4)
    int32_t n_tiles;  // ceil(n_columns / 16)

    __host__ __device__ int32_t size() const { return n_outer * n_groups * n_tiles * WAVE; }
    __device__ int32_t slot(int32_t outer, int32_t inner, int32_t column) const {
        if (!in_bounds(outer, n_outer) || !in_bounds(inner, n_inner) || !in_bounds(column, n_columns)) {
            return -1;
        }
        return ((outer * n_groups + (inner >> 2)) * n_tiles + (column >> 4)) * WAVE + ((inner & 3) << 4) +
               (column & 15);
    }
};

OperandShape operand_shape(int32_t n_outer, int32_t n_inner, int32_t n_columns) {
    OperandShape s;
    s.n_outer = n_outer;
    s.n_inner = n_inner;
    s.n_columns = n_columns;
    s.n_groups = (n_inner + 3) / 4;
    s.n_tiles = (n_columns + 15) / 16;
    return s;
}

// Table entries per thread of the build: 2 for tables of up to 2048 entries (what real
// Clebsch-Gordan tables of up to 16 x 16 x 16 cells mostly are), 8 beyond (more registers while
// the table is built). The kernels after the build do not depend on the number of entries.
constexpr int FEW_ENTRIES_PER_THREAD = 2;
constexpr int MANY_ENTRIES_PER_THREAD = MAX_ENTRIES / THREADS;
constexpr int FEW_ENTRIES = FEW_ENTRIES_PER_THREAD * THREADS;
constexpr int32_t NOBODY = 0x7fffffff;

/// The table entries a thread looks after (entry k = thread + e * THREADS),
/// loaded once, before anything waits for memory.
template <typename T, int ENTRIES_PER_THREAD> struct MyEntries {
    int32_t index_A[ENTRIES_PER_THREAD];
    int32_t index_B[ENTRIES_PER_THREAD];
    int32_t index_O[ENTRIES_PER_THREAD];
    T coefficient[ENTRIES_PER_THREAD];

    __device__ __forceinline__ void load(
        const T* __restrict__ C, const int32_t* __restrict__ PA, const int32_t* __restrict__ PB,
        const int32_t* __restrict__ PO, int32_t K
    ) {
#pragma unroll
        for (int e = 0; e < ENTRIES_PER_THREAD; e++) {
            const int32_t k = threadIdx.x + e * THREADS;
            const bool exists = k < K;
            // entries beyond the table get an index no range contains
            index_A[e] = exists ? PA[exists ? k : 0] : -1;
            index_B[e] = load_or_zero(PB, k, exists);
            index_O[e] = load_or_zero(PO, k, exists);
            coefficient[e] = load_or_zero(C, k, exists);
        }
    }
};

/// build_operands, called by all threads of the workgroup, fills up to
/// TARGETS operands in LDS with the dense table, each in its own layout.
/// `heads` is an LDS array of nA * nB * nO integers, `next` one of K integers
/// and `coefficients` one of K values.
///
/// Entries that name the same triple must be added in an order that does not
/// depend on timing for the sum to be the same everywhere and on every run.
/// Every entry pushes itself onto the list of its triple (one atomic
/// exchange); the entry that found the list empty then walks the finished
/// list and adds the coefficients of its members in ascending entry order,
/// smallest remaining entry first. Lists have one or two members for real
/// tables.
template <typename T> struct OperandTarget {
    T* operand; // LDS, null: not wanted
    OperandShape shape;
    int role[3]; // which of (A, B, O) is outer, inner, column
};

template <typename T> struct BuildAreas {
    int32_t* heads;
    int32_t* next;
    T* coefficients;
};

template <typename T, int TARGETS, int ENTRIES_PER_THREAD>
__device__ __forceinline__ void build_operands(
    const OperandTarget<T> (&targets)[TARGETS], const BuildAreas<T>& areas, int32_t nA, int32_t nB,
    int32_t nO, const MyEntries<T, ENTRIES_PER_THREAD>& entries
) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int w = 0; w < TARGETS; w++) {
        if (targets[w].operand != nullptr) {
            const int32_t operand_size = targets[w].shape.size();
            for (int32_t at = tid; at < operand_size; at += THREADS) {
                targets[w].operand[at] = T(0);
            }
        }
    }
    const int32_t n_dense = nA * nB * nO;
    for (int32_t at = tid; at < n_dense; at += THREADS) {
        areas.heads[at] = NOBODY;
    }
    int32_t dense[ENTRIES_PER_THREAD]; // -1: no such entry
#pragma unroll
    for (int e = 0; e < ENTRIES_PER_THREAD; e++) {
        const int32_t a = entries.index_A[e];
        const int32_t b = entries.index_B[e];
        const int32_t o = entries.index_O[e];
        const bool valid = in_bounds(a, nA) && in_bounds(b, nB) && in_bounds(o, nO);
        dense[e] = valid ? (a * nB + b) * nO + o : -1;
        if (valid) {
            areas.coefficients[tid + e * THREADS] = entries.coefficient[e];
        }
    }
    __syncthreads();
    bool first_of_list[ENTRIES_PER_THREAD];
#pragma unroll
    for (int e = 0; e < ENTRIES_PER_THREAD; e++) {
        first_of_list[e] = false;
        if (dense[e] >= 0) {
            const int32_t k = tid + e * THREADS;
            const int32_t previous = atomicExch(&areas.heads[dense[e]], k);
            areas.next[k] = previous;
            first_of_list[e] = previous == NOBODY;
        }
    }
    __syncthreads();
#pragma unroll
    for (int e = 0; e < ENTRIES_PER_THREAD; e++) {
        if (first_of_list[e]) {
            const int32_t head = areas.heads[dense[e]];
            T sum = T(0);
            // Short lists (all of them, in practice) are read once, sorted in
            // registers and added up in ascending entry order; NOBODY is larger
            // than any entry number. The wavefront reads until all its lists
            // have ended: at most four members each is the usual case and has
            // its own, shorter code; up to eight are sorted likewise; longer
            // lists are walked once per member.
            int32_t member[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                member[j] = NOBODY;
            }
            int32_t cursor = head;
            auto walk = [&](int from, int to) {
#pragma unroll
                for (int j = from; j < to; j++) {
                    if (__ballot(cursor != NOBODY) == 0) {
                        break;
                    }
                    member[j] = cursor;
                    if (cursor != NOBODY) {
                        cursor = areas.next[cursor];
                    }
                }
            };
            auto order = [&](int j, int k) {
                const int32_t low = min(member[j], member[k]);
                const int32_t high = max(member[j], member[k]);
                member[j] = low;
                member[k] = high;
            };
            auto add_members = [&](auto count) {
                constexpr int COUNT = decltype(count)::value;
                T value[COUNT];
#pragma unroll
                for (int j = 0; j < COUNT; j++) {
                    value[j] = load_or_zero(areas.coefficients, member[j], member[j] != NOBODY);
                }
#pragma unroll
                for (int j = 0; j < COUNT; j++) {
                    if (member[j] != NOBODY) {
                        sum += value[j];
                    }
                }
            };
            walk(0, 4);
            if (__ballot(cursor != NOBODY) == 0) {
                order(0, 1), order(2, 3), order(0, 2), order(1, 3), order(1, 2);
                add_members(std::integral_constant<int, 4>{});
            } else {
                walk(4, 8);
                if (cursor == NOBODY) {
#pragma unroll
                    for (int pass = 0; pass < 8; pass++) {
#pragma unroll
                        for (int j = pass & 1; j + 1 < 8; j += 2) { // odd-even transposition sort
                            order(j, j + 1);
                        }
                    }
                    add_members(std::integral_constant<int, 8>{});
                } else {
                    int32_t last = -1;
                    for (;;) {
                        // the smallest member above `last`
                        int32_t smallest = NOBODY;
                        for (int32_t k = head; k != NOBODY; k = areas.next[k]) {
                            if (k > last && k < smallest) {
                                smallest = k;
                            }
                        }
                        if (smallest == NOBODY) {
                            break;
                        }
                        sum += areas.coefficients[smallest];
                        last = smallest;
                    }
                }
            }
            // (selects, not an array indexed by role: that would live in scratch memory)
            auto index = [&](int role) {
                return role == 0 ? entries.index_A[e] : (role == 1 ? entries.index_B[e] : entries.index_O[e]);
            };
#pragma unroll
            for (int w = 0; w < TARGETS; w++) {
                if (targets[w].operand != nullptr) {
                    targets[w].operand[targets[w].shape.slot(
                        index(targets[w].role[0]), index(targets[w].role[1]), index(targets[w].role[2])
                    )] = sum;
                }
            }
        }
    }
    __syncthreads();
}

/// acc[r][t] += sum over x < n_outer, g < GROUPS of
///   (outer_r[x] * inner[r][g]) (x) operand[(x, g), t]
/// for the ROW_TILES row tiles of a wavefront. `outer_rows` points at this
/// lane's row of the outer values in LDS, row tile r is `outer_tile_stride`
/// elements further. The LDS reads of step x + 1 are issued before the matrix
/// instructions of step x; nothing inside the loop is conditional.
/// The operand has NT_TOTAL column tiles per (x, g), of which this call uses
/// the NT from `first_tile` on.
template <typename T, int NT, int GROUPS, int NT_TOTAL = NT>
__device__ __forceinline__ void pair_products(
    typename Mfma<T>::Acc (&acc)[ROW_TILES][NT],
    const T* __restrict__ outer_rows,
    int32_t outer_tile_stride,
    int32_t n_outer,
    const T (&inner)[ROW_TILES][GROUPS],
    const T* __restrict__ operand,
    int lane,
    int first_tile = 0
) {
    using M = Mfma<T>;
    struct Step {
        T outer[ROW_TILES];
        T right[GROUPS][NT];
    };
    constexpr int STEP_ELEMENTS = GROUPS * NT_TOTAL * WAVE;
    auto fetch = [&](Step& to, int32_t x) {
        const T* right = operand + lane + x * STEP_ELEMENTS + first_tile * WAVE;
#pragma unroll
        for (int r = 0; r < ROW_TILES; r++) {
            to.outer[r] = outer_rows[r * outer_tile_stride + x];
        }
#pragma unroll
        for (int g = 0; g < GROUPS; g++) {
#pragma unroll
            for (int t = 0; t < NT; t++) {
                to.right[g][t] = right[(g * NT_TOTAL + t) * WAVE];
            }
        }
    };
    // Two sets of accumulators, used in turn and added at the end: a matrix
    // instruction that continues the sum of the one before it waits for it.
    typename M::Acc other[ROW_TILES][NT];
#pragma unroll
    for (int r = 0; r < ROW_TILES; r++) {
#pragma unroll
        for (int t = 0; t < NT; t++) {
            other[r][t] = M::zero();
        }
    }
    auto multiply = [&](const Step& from) {
#pragma unroll
        for (int g = 0; g < GROUPS; g++) {
#pragma unroll
            for (int r = 0; r < ROW_TILES; r++) {
                const T product = from.outer[r] * inner[r][g];
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    if (g % 2 == 0) {
                        acc[r][t] = M::mma(product, from.right[g][t], acc[r][t]);
                    } else {
                        other[r][t] = M::mma(product, from.right[g][t], other[r][t]);
                    }
                }
            }
        }
    };
    Step even;
    Step odd;
    fetch(even, 0);
    int32_t x = 0;
    for (; x + 1 < n_outer; x += 2) {
        fetch(odd, x + 1);
        multiply(even);
        fetch(even, min(x + 2, n_outer - 1));
        multiply(odd);
    }
    if (x < n_outer) {
        multiply(even);
    }
#pragma unroll
    for (int r = 0; r < ROW_TILES; r++) {
#pragma unroll
        for (int t = 0; t < NT; t++) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                acc[r][t][e] += other[r][t][e];
            }
        }
    }
}

/// Copies `rows` x `width` contiguous values from global memory to LDS (same
/// layout), zeros beyond `valid_rows`. Loads are issued eight at a time.
template <typename T>
__device__ __forceinline__ void stage_rows(
    T* __restrict__ lds, const T* __restrict__ global, int32_t width, int32_t valid_rows, int32_t rows, int lane
) {
    constexpr int BATCH = 8;
    const int32_t total = rows * width;
    const int32_t valid = max(valid_rows, 0) * width;
    for (int32_t base = 0; base < total; base += BATCH * WAVE) {
        T values[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; u++) {
            const int32_t at = base + u * WAVE + lane;
            values[u] = load_or_zero(global, at, at < valid);
        }
#pragma unroll
        for (int u = 0; u < BATCH; u++) {
            const int32_t at = base + u * WAVE + lane;
            if (at < total) {
                lds[at] = values[u];
            }
        }
    }
}

/// Writes NT column tiles of accumulators, from tile `first_tile` on, to LDS
/// [16][width].
template <typename T, int NT>
__device__ __forceinline__ void stage_tiles(
    T* __restrict__ lds, const typename Mfma<T>::Acc (&acc)[ROW_TILES][NT], int first_tile, int32_t width, int lane
) {
    using M = Mfma<T>;
    const int j = lane & 15;
#pragma unroll
    for (int r = 0; r < ROW_TILES; r++) {
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const int32_t column = 16 * (first_tile + t) + j;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                if (column < width) {
                    lds[(16 * r + M::row(lane, e)) * width + column] = acc[r][t][e];
                }
            }
        }
    }
}

/// Writes a wavefront's accumulators (rows x columns tile by tile) to LDS
/// [32][width] and from there, contiguously, to global memory.
template <typename T, int NT>
__device__ __forceinline__ void store_rows(
    T* __restrict__ global, T* __restrict__ lds, const typename Mfma<T>::Acc (&acc)[ROW_TILES][NT],
    int32_t width, int32_t valid_rows, int lane
) {
    using M = Mfma<T>;
    const int j = lane & 15;
#pragma unroll
    for (int r = 0; r < ROW_TILES; r++) {
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const int32_t column = 16 * t + j;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                if (column < width) {
                    lds[(16 * r + M::row(lane, e)) * width + column] = acc[r][t][e];
                }
            }
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int32_t total = max(min(valid_rows, ROWS_PER_WAVE), 0) * width;
    for (int32_t at = lane; at < total; at += WAVE) {
        global[at] = lds[at];
    }
}

/// store_rows for the walking kernels: always the same number of store instructions, each a buffer
/// store whose descriptor ends with the rows that exist (the hardware drops what lies beyond), so
/// that a later wait for loads that were asked for before these stores can leave exactly them in
/// flight. With stores under a condition the compiler does not know how many there are and such a
/// wait ends up waiting for younger loads as well.
template <typename T, int NT>
__device__ __forceinline__ void store_rows_counted(
    T* __restrict__ global, T* __restrict__ lds, const typename Mfma<T>::Acc (&acc)[ROW_TILES][NT],
    int32_t width, int32_t valid_rows, int lane
) {
    using M = Mfma<T>;
    const int j = lane & 15;
#pragma unroll
    for (int r = 0; r < ROW_TILES; r++) {
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const int32_t column = 16 * t + j;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                if (column < width) {
                    lds[(16 * r + M::row(lane, e)) * width + column] = acc[r][t][e];
                }
            }
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // (uniform, and said to be: a descriptor that the compiler takes for different from lane to
    // lane costs a loop around every store)
    const int32_t total = __builtin_amdgcn_readfirstlane(max(min(valid_rows, ROWS_PER_WAVE), 0) * width);
    const __amdgpu_buffer_rsrc_t target = __builtin_amdgcn_make_buffer_rsrc(
        global, 0, total * static_cast<int32_t>(sizeof(T)), 0x00020000
    );
    // (ROW_TILES * NT * 4 stores cover 16 rows of up to 16 NT values; the LDS reads stay inside
    // the wavefront's own area, which holds 16 rows of the widest of its tensors)
    const int32_t area = ROWS_PER_WAVE * width;
#pragma unroll
    for (int u = 0; u < ROW_TILES * NT * 4; u++) {
        const int32_t at = u * WAVE + lane;
        const T value = lds[min(at, area - 1)];
        if constexpr (sizeof(T) == 4) {
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, value), target, at * 4, 0, 0);
        } else {
            typedef unsigned int two_words __attribute__((__vector_size__(2 * sizeof(unsigned int))));
            __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(two_words, value), target, at * 8, 0, 0);
        }
    }
}

template <typename T> struct Arguments {
    T* output;  // forward: O; vjp: unused
    T* grad_A;  // vjp, may be null
    T* grad_B;  // vjp, may be null
    const T* A;
    const T* B;
    const T* G; // grad_output (vjp)
    const T* A2; // forward of two pairs: O = sap(A, B) + sap(A2, B2)
    const T* B2;
    const T* C;
    const int32_t* PA;
    const int32_t* PB;
    const int32_t* PO;
    int32_t n_rows, nA, nB, nO, K;
    OperandShape first;  // forward: (a, b) -> o;  vjp: (b, o) -> a
    OperandShape second; // vjp: (a, o) -> b
};

template <typename T>
__device__ __forceinline__ BuildAreas<T> carve_build_areas(char*& cursor, int32_t n_dense, int32_t K) {
    BuildAreas<T> areas;
    areas.heads = reinterpret_cast<int32_t*>(cursor);
    cursor += align16(static_cast<size_t>(n_dense) * 4);
    areas.next = reinterpret_cast<int32_t*>(cursor);
    cursor += align16(static_cast<size_t>(K) * 4);
    areas.coefficients = reinterpret_cast<T*>(cursor);
    cursor += align16(static_cast<size_t>(K) * sizeof(T));
    return areas;
}

size_t build_areas_bytes(const Shape& s, size_t element_size) {
    return align16(static_cast<size_t>(s.nA) * s.nB * s.nO * 4) + align16(static_cast<size_t>(s.K) * 4) +
           align16(static_cast<size_t>(s.K) * element_size);
}

/// Two wavefronts per tile of 16 rows, as in vjp_kernel below: with an even
/// number of column tiles each takes half of them (otherwise the second one
/// only helps with loading and storing).
template <typename T, int NT, int GROUPS, bool TWO_PAIRS = false, int EPT = FEW_ENTRIES_PER_THREAD>
__global__ __launch_bounds__(THREADS) void forward_kernel(const Arguments<T> p) {
    using M = Mfma<T>;
    constexpr bool SPLIT = NT % 2 == 0;
    constexpr int MY_TILES = SPLIT ? NT / 2 : NT;
    extern __shared__ __align__(16) char lds_raw[];
    char* cursor = lds_raw;
    T* operand = reinterpret_cast<T*>(cursor);
    cursor += align16(static_cast<size_t>(p.first.size()) * sizeof(T));
    const BuildAreas<T> areas = carve_build_areas<T>(cursor, p.nA * p.nB * p.nO, p.K);
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x >> 6;
    const int tile = wave & (WAVES - 1);
    const bool second_half = wave >= WAVES; // uniform per wavefront
    const int32_t row_width = p.nA + p.nB;
    MyEntries<T, EPT> entries;
    entries.load(p.C, p.PA, p.PB, p.PO, p.K);
    T* mine = reinterpret_cast<T*>(cursor) + tile * ROWS_PER_WAVE * max(row_width, p.nO);
    T* a_tile = mine;                          // [16][nA]
    T* b_tile = mine + ROWS_PER_WAVE * p.nA;   // [16][nB]

    const int32_t first_row = (blockIdx.x * WAVES + tile) * ROWS_PER_WAVE;
    const int32_t valid_rows = p.n_rows - first_row;
    const int32_t safe_first = valid_rows > 0 ? first_row : 0; // wavefronts beyond the end read row 0
    if (second_half) {
        stage_rows<T>(b_tile, p.B + static_cast<size_t>(safe_first) * p.nB, p.nB, valid_rows, ROWS_PER_WAVE, lane);
    } else {
        stage_rows<T>(a_tile, p.A + static_cast<size_t>(safe_first) * p.nA, p.nA, valid_rows, ROWS_PER_WAVE, lane);
    }
    const OperandTarget<T> targets[1] = {{operand, p.first, {0, 1, 2}}};
    build_operands<T, 1, EPT>(targets, areas, p.nA, p.nB, p.nO, entries); // ends with a barrier: the tiles are there

    const int i = lane & 15;
    const int q = lane >> 4;
    T inner[ROW_TILES][GROUPS];
#pragma unroll
    for (int r = 0; r < ROW_TILES; r++) {
#pragma unroll
        for (int g = 0; g < GROUPS; g++) {
            const int32_t b = 4 * g + q;
            inner[r][g] = load_or_zero(b_tile, (16 * r + i) * p.nB + b, b < p.nB);
        }
    }
    typename M::Acc acc[ROW_TILES][MY_TILES];
#pragma unroll
    for (int r = 0; r < ROW_TILES; r++) {
#pragma unroll
        for (int t = 0; t < MY_TILES; t++) {
            acc[r][t] = M::zero();
        }
    }
    const int first_tile = SPLIT && second_half ? MY_TILES : 0;
    const bool computes = SPLIT || !second_half;
    if (computes) {
        pair_products<T, MY_TILES, GROUPS, NT>(acc, a_tile + i * p.nA, 16 * p.nA, p.nA, inner, operand, lane, first_tile);
    }
    if constexpr (TWO_PAIRS) {
        // the second pair of rows through the same tiles, its products added to the same sums
        __syncthreads();
        if (second_half) {
            stage_rows<T>(b_tile, p.B2 + static_cast<size_t>(safe_first) * p.nB, p.nB, valid_rows, ROWS_PER_WAVE, lane);
        } else {
            stage_rows<T>(a_tile, p.A2 + static_cast<size_t>(safe_first) * p.nA, p.nA, valid_rows, ROWS_PER_WAVE, lane);
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < ROW_TILES; r++) {
#pragma unroll
            for (int g = 0; g < GROUPS; g++) {
                const int32_t b = 4 * g + q;
                inner[r][g] = load_or_zero(b_tile, (16 * r + i) * p.nB + b, b < p.nB);
            }
        }
        if (computes) {
            pair_products<T, MY_TILES, GROUPS, NT>(acc, a_tile + i * p.nA, 16 * p.nA, p.nA, inner, operand, lane, first_tile);
        }
    }
    __syncthreads(); // nobody reads the tiles any more: they become the staging area of the store
    if (computes) {
        stage_tiles<T, MY_TILES>(mine, acc, first_tile, p.nO, lane);
    }
    __syncthreads();
    if (valid_rows > 0) {
        // the 16 output rows are contiguous in memory: both wavefronts copy
        T* target = p.output + static_cast<size_t>(first_row) * p.nO;
        const int32_t total = min(valid_rows, ROWS_PER_WAVE) * p.nO;
        for (int32_t at = lane + (second_half ? WAVE : 0); at < total; at += 2 * WAVE) {
            target[at] = mine[at];
        }
    }
}

/// Two wavefronts per tile of 16 rows: wavefront t computes grad_A of tile t,
/// wavefront t + 8 grad_B, from the same rows in LDS; four wavefronts per SIMD
/// keep the matrix cores busier than two.
template <typename T, int GROUPS, int EPT = FEW_ENTRIES_PER_THREAD>
__global__ __launch_bounds__(THREADS) void vjp_kernel(const Arguments<T> p) {
    using M = Mfma<T>;
    extern __shared__ __align__(16) char lds_raw[];
    char* cursor = lds_raw;
    const bool want_A = p.grad_A != nullptr;
    const bool want_B = p.grad_B != nullptr;
    T* operand_A = reinterpret_cast<T*>(cursor);
    cursor += align16(static_cast<size_t>(want_A ? p.first.size() : 0) * sizeof(T));
    T* operand_B = reinterpret_cast<T*>(cursor);
    cursor += align16(static_cast<size_t>(want_B ? p.second.size() : 0) * sizeof(T));
    const BuildAreas<T> areas = carve_build_areas<T>(cursor, p.nA * p.nB * p.nO, p.K);
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x >> 6;
    const int tile = wave & (WAVES - 1);
    const bool second_half = wave >= WAVES; // uniform per wavefront
    const int32_t row_width = p.nA + p.nB + p.nO;
    MyEntries<T, EPT> entries;
    entries.load(p.C, p.PA, p.PB, p.PO, p.K);
    T* mine = reinterpret_cast<T*>(cursor) + tile * ROWS_PER_WAVE * row_width;
    T* a_tile = mine;                                  // [16][nA]
    T* b_tile = a_tile + ROWS_PER_WAVE * p.nA;         // [16][nB]
    T* g_tile = b_tile + ROWS_PER_WAVE * p.nB;         // [16][nO]

    const int32_t first_row = (blockIdx.x * WAVES + tile) * ROWS_PER_WAVE;
    const int32_t valid_rows = p.n_rows - first_row;
    const int32_t safe_first = valid_rows > 0 ? first_row : 0; // wavefronts beyond the end read row 0
    if (second_half) {
        stage_rows<T>(g_tile, p.G + static_cast<size_t>(safe_first) * p.nO, p.nO, valid_rows, ROWS_PER_WAVE, lane);
    } else {
        stage_rows<T>(a_tile, p.A + static_cast<size_t>(safe_first) * p.nA, p.nA, valid_rows, ROWS_PER_WAVE, lane);
        stage_rows<T>(b_tile, p.B + static_cast<size_t>(safe_first) * p.nB, p.nB, valid_rows, ROWS_PER_WAVE, lane);
    }
    const OperandTarget<T> targets[2] = {
        {want_A ? operand_A : nullptr, p.first, {1, 2, 0}},
        {want_B ? operand_B : nullptr, p.second, {0, 2, 1}},
    };
    build_operands<T, 2, EPT>(targets, areas, p.nA, p.nB, p.nO, entries); // ends with a barrier: the tiles are there

    const int i = lane & 15;
    const int q = lane >> 4;
    T inner[ROW_TILES][GROUPS]; // grad_output[row][4 g + q]
#pragma unroll
    for (int r = 0; r < ROW_TILES; r++) {
#pragma unroll
        for (int g = 0; g < GROUPS; g++) {
            const int32_t o = 4 * g + q;
            inner[r][g] = load_or_zero(g_tile, (16 * r + i) * p.nO + o, o < p.nO);
        }
    }
    typename M::Acc acc[ROW_TILES][1];
#pragma unroll
    for (int r = 0; r < ROW_TILES; r++) {
        acc[r][0] = M::zero();
    }
    if (second_half) {
        if (want_B) {
            pair_products<T, 1, GROUPS>(acc, a_tile + i * p.nA, 16 * p.nA, p.nA, inner, operand_B, lane);
        }
    } else if (want_A) {
        pair_products<T, 1, GROUPS>(acc, b_tile + i * p.nB, 16 * p.nB, p.nB, inner, operand_A, lane);
    }
    __syncthreads(); // nobody reads the tiles any more: they become the staging areas of the stores
    if (valid_rows > 0) {
        if (second_half) {
            if (want_B) {
                store_rows<T, 1>(p.grad_B + static_cast<size_t>(first_row) * p.nB, b_tile, acc, p.nB, valid_rows, lane);
            }
        } else if (want_A) {
            store_rows<T, 1>(p.grad_A + static_cast<size_t>(first_row) * p.nA, a_tile, acc, p.nA, valid_rows, lane);
        }
    }
}

// ---------------------------------------------------------------------------
// Many rows (more tiles of 16 rows than a few for every wavefront the device
// holds): workgroups that stay, build the table once and then let every
// wavefront walk over tiles of its own, all the work of a tile in one
// wavefront. After the build no wavefront waits for another; the rows of a
// wavefront's next tile are asked for before the products of this one.

constexpr int WALK_WAVES = 16;                  // wavefronts per workgroup
constexpr int WALK_THREADS = WALK_WAVES * WAVE; // (= THREADS: build_operands counts on it)
static_assert(WALK_THREADS == THREADS, "the table build is written for THREADS threads");
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

/// The `valid_rows` x `width` values from `global` on (at most N * 64: N loads per lane); after them
/// comes a repeat of the first value, which the rows of a tile that do not exist may hold: every row
/// of the results depends on its own row of the operands only, and rows that do not exist are not
/// stored. (No zero is put in their place: a choice that follows a load is a wait for that load
/// wherever the compiler moves it, and it moved all of them to the end of the loop, behind the
/// loads of the tile after the next.)
template <typename T, int N>
__device__ __forceinline__ void fetch_rows(
    T (&values)[N], const T* __restrict__ global, int32_t width, int32_t valid_rows, int lane
) {
    const int32_t valid = max(min(valid_rows, ROWS_PER_WAVE), 0) * width;
    // (no branch around a load either, not even a uniform one: every load would wait for the one before)
#pragma unroll
    for (int u = 0; u < N; u++) {
        const int32_t at = u * WAVE + lane;
        values[u] = global[at < valid ? at : 0];
    }
}

template <typename T, int N>
__device__ __forceinline__ void place_rows(T* __restrict__ lds, const T (&values)[N], int32_t total, int lane) {
#pragma unroll
    for (int u = 0; u < N; u++) {
        const int32_t at = u * WAVE + lane;
        if (at < total) {
            lds[at] = values[u];
        }
    }
}

/// Loads per lane for a tile of 16 rows of up to 16 values (A and B of the vjp, A of the forward pass).
constexpr int SHORT_ROW_LOADS = 4;

template <typename T, int NT, int GROUPS, int EPT = FEW_ENTRIES_PER_THREAD>
__global__ __launch_bounds__(WALK_THREADS) void forward_walk_kernel(const Arguments<T> p) {
    using M = Mfma<T>;
    extern __shared__ __align__(16) char lds_raw[];
    char* cursor = lds_raw;
    T* operand = reinterpret_cast<T*>(cursor);
    cursor += align16(static_cast<size_t>(p.first.size()) * sizeof(T));
    const BuildAreas<T> areas = carve_build_areas<T>(cursor, p.nA * p.nB * p.nO, p.K);
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x >> 6;
    MyEntries<T, EPT> entries;
    entries.load(p.C, p.PA, p.PB, p.PO, p.K);
    T* mine = reinterpret_cast<T*>(cursor) + wave * ROWS_PER_WAVE * max(p.nA + p.nB, p.nO);
    T* a_tile = mine;                        // [16][nA]
    T* b_tile = mine + ROWS_PER_WAVE * p.nA; // [16][nB]

    const int32_t n_tiles = (p.n_rows + ROWS_PER_WAVE - 1) / ROWS_PER_WAVE;
    const int32_t stride = static_cast<int32_t>(gridDim.x) * WALK_WAVES;
    int32_t tile = static_cast<int32_t>(blockIdx.x) * WALK_WAVES + wave;
    // the rows of the next two tiles of this wavefront are on their way while it works on one
    struct Rows {
        T a[SHORT_ROW_LOADS];
        T b[GROUPS];
    };
    auto fetch = [&](Rows& rows, int32_t which) {
        const int32_t first_row = min(which, n_tiles - 1) * ROWS_PER_WAVE; // (beyond the end: a tile that exists, no rows of it)
        const int32_t valid_rows = which < n_tiles ? p.n_rows - first_row : 0;
        fetch_rows<T, SHORT_ROW_LOADS>(rows.a, p.A + static_cast<size_t>(first_row) * p.nA, p.nA, valid_rows, lane);
        fetch_rows<T, GROUPS>(rows.b, p.B + static_cast<size_t>(first_row) * p.nB, p.nB, valid_rows, lane);
    };
    Rows even, odd;
    fetch(even, tile);
    fetch(odd, tile + stride);
    const OperandTarget<T> targets[1] = {{operand, p.first, {0, 1, 2}}};
    build_operands<T, 1, EPT>(targets, areas, p.nA, p.nB, p.nO, entries); // ends with a barrier

    const int i = lane & 15;
    const int q = lane >> 4;
    auto work = [&](Rows& rows) {
        place_rows<T, SHORT_ROW_LOADS>(a_tile, rows.a, ROWS_PER_WAVE * p.nA, lane);
        place_rows<T, GROUPS>(b_tile, rows.b, ROWS_PER_WAVE * p.nB, lane);
        wave_sync();
        fetch(rows, tile + 2 * stride);
        T inner[ROW_TILES][GROUPS];
#pragma unroll
        for (int r = 0; r < ROW_TILES; r++) {
#pragma unroll
            for (int g = 0; g < GROUPS; g++) {
                const int32_t b = 4 * g + q;
                inner[r][g] = load_or_zero(b_tile, (16 * r + i) * p.nB + b, b < p.nB);
            }
        }
        typename M::Acc acc[ROW_TILES][NT];
#pragma unroll
        for (int r = 0; r < ROW_TILES; r++) {
#pragma unroll
            for (int t = 0; t < NT; t++) {
                acc[r][t] = M::zero();
            }
        }
        pair_products<T, NT, GROUPS>(acc, a_tile + i * p.nA, 16 * p.nA, p.nA, inner, operand, lane);
        wave_sync(); // the tile has been read: its place becomes the staging area of the store
        // (the same in all lanes, which the compiler cannot know: a wavefront's number comes from threadIdx)
        const int32_t first_row = __builtin_amdgcn_readfirstlane(tile) * ROWS_PER_WAVE;
        store_rows_counted<T, NT>(p.output + static_cast<size_t>(first_row) * p.nO, mine, acc, p.nO, p.n_rows - first_row, lane);
        wave_sync();
        tile += stride;
    };
    while (tile < n_tiles) {
        work(even);
        if (tile >= n_tiles) {
            break;
        }
        work(odd);
    }
}

template <typename T, int GROUPS, int EPT = FEW_ENTRIES_PER_THREAD>
__global__ __launch_bounds__(WALK_THREADS) void vjp_walk_kernel(const Arguments<T> p) {
    using M = Mfma<T>;
    extern __shared__ __align__(16) char lds_raw[];
    char* cursor = lds_raw;
    const bool want_A = p.grad_A != nullptr;
    const bool want_B = p.grad_B != nullptr;
    T* operand_A = reinterpret_cast<T*>(cursor);
    cursor += align16(static_cast<size_t>(want_A ? p.first.size() : 0) * sizeof(T));
    T* operand_B = reinterpret_cast<T*>(cursor);
    cursor += align16(static_cast<size_t>(want_B ? p.second.size() : 0) * sizeof(T));
    const BuildAreas<T> areas = carve_build_areas<T>(cursor, p.nA * p.nB * p.nO, p.K);
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x >> 6;
    MyEntries<T, EPT> entries;
    entries.load(p.C, p.PA, p.PB, p.PO, p.K);
    T* mine = reinterpret_cast<T*>(cursor) + wave * ROWS_PER_WAVE * (p.nA + p.nB + p.nO);
    T* a_tile = mine;                          // [16][nA]
    T* b_tile = a_tile + ROWS_PER_WAVE * p.nA; // [16][nB]
    T* g_tile = b_tile + ROWS_PER_WAVE * p.nB; // [16][nO]

    const int32_t n_tiles = (p.n_rows + ROWS_PER_WAVE - 1) / ROWS_PER_WAVE;
    const int32_t stride = static_cast<int32_t>(gridDim.x) * WALK_WAVES;
    int32_t tile = static_cast<int32_t>(blockIdx.x) * WALK_WAVES + wave;
    // the rows of the next two tiles of this wavefront are on their way while it works on one
    struct Rows {
        T a[SHORT_ROW_LOADS];
        T b[SHORT_ROW_LOADS];
        T g[GROUPS];
    };
    auto fetch = [&](Rows& rows, int32_t which) {
        const int32_t first_row = min(which, n_tiles - 1) * ROWS_PER_WAVE;
        const int32_t valid_rows = which < n_tiles ? p.n_rows - first_row : 0;
        fetch_rows<T, SHORT_ROW_LOADS>(rows.a, p.A + static_cast<size_t>(first_row) * p.nA, p.nA, valid_rows, lane);
        fetch_rows<T, SHORT_ROW_LOADS>(rows.b, p.B + static_cast<size_t>(first_row) * p.nB, p.nB, valid_rows, lane);
        fetch_rows<T, GROUPS>(rows.g, p.G + static_cast<size_t>(first_row) * p.nO, p.nO, valid_rows, lane);
    };
    Rows even, odd;
    fetch(even, tile);
    fetch(odd, tile + stride);
    const OperandTarget<T> targets[2] = {
        {want_A ? operand_A : nullptr, p.first, {1, 2, 0}},
        {want_B ? operand_B : nullptr, p.second, {0, 2, 1}},
    };
    build_operands<T, 2, EPT>(targets, areas, p.nA, p.nB, p.nO, entries); // ends with a barrier

    const int i = lane & 15;
    const int q = lane >> 4;
    auto work = [&](Rows& rows) {
        place_rows<T, SHORT_ROW_LOADS>(a_tile, rows.a, ROWS_PER_WAVE * p.nA, lane);
        place_rows<T, SHORT_ROW_LOADS>(b_tile, rows.b, ROWS_PER_WAVE * p.nB, lane);
        place_rows<T, GROUPS>(g_tile, rows.g, ROWS_PER_WAVE * p.nO, lane);
        wave_sync();
        fetch(rows, tile + 2 * stride);
        T inner[ROW_TILES][GROUPS]; // grad_output[row][4 g + q]
#pragma unroll
        for (int r = 0; r < ROW_TILES; r++) {
#pragma unroll
            for (int g = 0; g < GROUPS; g++) {
                const int32_t o = 4 * g + q;
                inner[r][g] = load_or_zero(g_tile, (16 * r + i) * p.nO + o, o < p.nO);
            }
        }
        typename M::Acc for_A[ROW_TILES][1], for_B[ROW_TILES][1];
#pragma unroll
        for (int r = 0; r < ROW_TILES; r++) {
            for_A[r][0] = M::zero();
            for_B[r][0] = M::zero();
        }
        if (want_A) {
            pair_products<T, 1, GROUPS>(for_A, b_tile + i * p.nB, 16 * p.nB, p.nB, inner, operand_A, lane);
        }
        if (want_B) {
            pair_products<T, 1, GROUPS>(for_B, a_tile + i * p.nA, 16 * p.nA, p.nA, inner, operand_B, lane);
        }
        wave_sync(); // the tiles have been read: their places become the staging areas of the stores
        const int32_t first_row = __builtin_amdgcn_readfirstlane(tile) * ROWS_PER_WAVE; // (the same in all lanes)
        if (want_A) {
            store_rows_counted<T, 1>(p.grad_A + static_cast<size_t>(first_row) * p.nA, a_tile, for_A, p.nA, p.n_rows - first_row, lane);
        }
        if (want_B) {
            store_rows_counted<T, 1>(p.grad_B + static_cast<size_t>(first_row) * p.nB, b_tile, for_B, p.nB, p.n_rows - first_row, lane);
        }
        wave_sync();
        tile += stride;
    };
    while (tile < n_tiles) {
        work(even);
        if (tile >= n_tiles) {
            break;
        }
        work(odd);
    }
}

size_t forward_lds(const Shape& s, size_t element_size) {
    const OperandShape first = operand_shape(s.nA, s.nB, s.nO);
    return align16(static_cast<size_t>(first.size()) * element_size) +
           build_areas_bytes(s, element_size) +
           static_cast<size_t>(WAVES) * ROWS_PER_WAVE * std::max(s.nA + s.nB, s.nO) * element_size;
}

size_t vjp_lds(const Shape& s, size_t element_size, bool want_A, bool want_B) {
    const OperandShape first = operand_shape(s.nB, s.nO, s.nA);
    const OperandShape second = operand_shape(s.nA, s.nO, s.nB);
    const int32_t size_A = want_A ? first.size() : 0;
    const int32_t size_B = want_B ? second.size() : 0;
    return align16(static_cast<size_t>(size_A) * element_size) + align16(static_cast<size_t>(size_B) * element_size) +
           build_areas_bytes(s, element_size) +
           static_cast<size_t>(WAVES) * ROWS_PER_WAVE * (s.nA + s.nB + s.nO) * element_size;
}

size_t forward_walk_lds(const Shape& s, size_t element_size) {
    return forward_lds(s, element_size) +
           static_cast<size_t>(WALK_WAVES - WAVES) * ROWS_PER_WAVE * std::max(s.nA + s.nB, s.nO) * element_size;
}

size_t vjp_walk_lds(const Shape& s, size_t element_size, bool want_A, bool want_B) {
    return vjp_lds(s, element_size, want_A, want_B) +
           static_cast<size_t>(WALK_WAVES - WAVES) * ROWS_PER_WAVE * (s.nA + s.nB + s.nO) * element_size;
}

/// Workgroups of a walking launch: as many as the device holds at once (two
/// per compute unit by their wavefronts, one when their LDS does not fit twice).
unsigned walking_workgroups(size_t lds) {
    const int64_t per_unit = 2 * lds <= 160 * 1024 ? 2 : 1;
    return static_cast<unsigned>(per_unit * compute_units());
}

/// Whether a launch walks: `tiles_per_wave` tiles or more for every wavefront
/// (below that the builds that are saved do not make up for one wavefront doing
/// all the work of a tile), rows of A (and of B in the vjp) that fit the registers
/// of fetch_rows (the others fit by the limits of these kernels), LDS that fits. Measured with nA, nB, nO = 13, 7, 20 over 65 000 to 560 000 rows: the
/// forward pass gains from one tile per wavefront on (200 000 rows, f32: 33.3
/// -> 30.0 us; f64 at 100 000: 30.0 -> 25.9), the vjp from two (400 000 rows,
/// f32: 88.9 -> 83.5 us; with one, 140 000 rows take 41.4 instead of 35.9 us).
bool walks(const Shape& s, int32_t widest_short_row, size_t lds, int64_t tiles_per_wave) {
    const int64_t tiles = (static_cast<int64_t>(s.n_rows) + ROWS_PER_WAVE - 1) / ROWS_PER_WAVE;
    return lds <= 160 * 1024 && ROWS_PER_WAVE * widest_short_row <= SHORT_ROW_LOADS * WAVE &&
           tiles >= tiles_per_wave * static_cast<int64_t>(walking_workgroups(lds)) * WALK_WAVES;
}

template <typename T> Arguments<T> arguments(const T* A, const T* B, const Table& table, const Shape& s) {
    Arguments<T> p{};
    p.A = A;
    p.B = B;
    p.C = static_cast<const T*>(table.C);
    p.PA = table.indices_A;
    p.PB = table.indices_B;
    p.PO = table.indices_output;
    p.n_rows = s.n_rows;
    p.nA = s.nA;
    p.nB = s.nB;
    p.nO = s.nO;
    p.K = s.K;
    return p;
}

/// Kernels that use more than 64 KB of LDS have to say so before the launch.
template <typename Kernel> void allow_lds(Kernel kernel, size_t bytes) {
    if (bytes > LDS_WITHOUT_ASKING) {
        MOPS_HIP_CHECK(hipFuncSetAttribute(
            reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
            static_cast<int>(bytes)
        ));
    }
}

/// Calls launch(integral_constant<first>, integral_constant<second>) for
/// 1 <= first <= MAX_FIRST, 1 <= second <= MAX_SECOND given at run time.
template <int MAX_FIRST, int MAX_SECOND, int FIRST = 1, int SECOND = 1, typename Launch>
void with_constants(int first, int second, Launch&& launch) {
    if constexpr (FIRST < MAX_FIRST) {
        if (first > FIRST) {
            with_constants<MAX_FIRST, MAX_SECOND, FIRST + 1, SECOND>(first, second, launch);
            return;
        }
    }
    if constexpr (SECOND < MAX_SECOND) {
        if (second > SECOND) {
            with_constants<MAX_FIRST, MAX_SECOND, FIRST, SECOND + 1>(first, second, launch);
            return;
        }
    }
    launch(std::integral_constant<int, FIRST>{}, std::integral_constant<int, SECOND>{});
}

} // namespace

bool supports_forward(const Shape& s, size_t element_size) {
    if (s.n_rows < 1 || s.nA < 1 || s.nB < 1 || s.nO < 1 || s.K < 1 || s.K > MAX_ENTRIES) {
        return false;
    }
    if (s.nB > 4 * MAX_INNER_GROUPS_FORWARD || s.nO > 64) {
        return false;
    }
    return forward_lds(s, element_size) <= LDS_BUDGET;
}

bool supports_vjp(const Shape& s, size_t element_size) {
    if (s.n_rows < 1 || s.nA < 1 || s.nB < 1 || s.nO < 1 || s.K < 1 || s.K > MAX_ENTRIES) {
        return false;
    }
    if (s.nA > MAX_OUTER || s.nB > MAX_OUTER || s.nO > 4 * MAX_INNER_GROUPS_VJP) {
        return false;
    }
    return vjp_lds(s, element_size, true, true) <= LDS_BUDGET;
}

template <typename T>
void forward(T* output, const T* A, const T* B, const Table& table, const Shape& s, hipStream_t stream) {
    Arguments<T> p = arguments<T>(A, B, table, s);
    p.output = output;
    p.first = operand_shape(s.nA, s.nB, s.nO);
    const size_t walk_lds = forward_walk_lds(s, sizeof(T));
    const bool walk = walks(s, s.nA, walk_lds, thresholds::SAP_FORWARD_WALK_TILES_PER_WAVE);
    const unsigned grid =
        walk ? walking_workgroups(walk_lds) : static_cast<unsigned>((s.n_rows + ROWS_PER_GROUP - 1) / ROWS_PER_GROUP);
    const size_t lds = walk ? walk_lds : forward_lds(s, sizeof(T));
    const LaunchEvents events = launch_events(stream);
    with_constants<4, 4>(p.first.n_tiles, p.first.n_groups, [&](auto tiles, auto groups) {
        constexpr int NT = decltype(tiles)::value, GROUPS = decltype(groups)::value, MANY = MANY_ENTRIES_PER_THREAD;
        auto kernel = s.K <= FEW_ENTRIES
                          ? (walk ? forward_walk_kernel<T, NT, GROUPS> : forward_kernel<T, NT, GROUPS>)
                          : (walk ? forward_walk_kernel<T, NT, GROUPS, MANY> : forward_kernel<T, NT, GROUPS, false, MANY>);
        allow_lds(kernel, lds);
        hipExtLaunchKernelGGL(kernel, dim3(grid), dim3(THREADS), lds, stream, events.start, events.stop, 0, p);
    });
    MOPS_HIP_CHECK(hipGetLastError());
}

bool supports_forward_of_two_pairs(const Shape& s, size_t element_size) {
    return supports_forward(s, element_size) && !walks(s, s.nA, forward_walk_lds(s, element_size), thresholds::SAP_FORWARD_WALK_TILES_PER_WAVE);
}

template <typename T>
void forward_of_two_pairs(
    T* output, const T* A, const T* B, const T* A2, const T* B2, const Table& table, const Shape& s,
    hipStream_t stream
) {
    Arguments<T> p = arguments<T>(A, B, table, s);
    p.A2 = A2;
    p.B2 = B2;
    p.output = output;
    p.first = operand_shape(s.nA, s.nB, s.nO);
    const unsigned grid = static_cast<unsigned>((s.n_rows + ROWS_PER_GROUP - 1) / ROWS_PER_GROUP);
    const size_t lds = forward_lds(s, sizeof(T));
    with_constants<4, 4>(p.first.n_tiles, p.first.n_groups, [&](auto tiles, auto groups) {
        constexpr int NT = decltype(tiles)::value, GROUPS = decltype(groups)::value;
        auto kernel = s.K <= FEW_ENTRIES ? forward_kernel<T, NT, GROUPS, true>
                                         : forward_kernel<T, NT, GROUPS, true, MANY_ENTRIES_PER_THREAD>;
        allow_lds(kernel, lds);
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(THREADS), lds, stream, p);
    });
    MOPS_HIP_CHECK(hipGetLastError());
}

template <typename T>
void vjp(
    T* grad_A, T* grad_B, const T* grad_output, const T* A, const T* B, const Table& table,
    const Shape& s, hipStream_t stream
) {
    Arguments<T> p = arguments<T>(A, B, table, s);
    p.grad_A = grad_A;
    p.grad_B = grad_B;
    p.G = grad_output;
    p.first = operand_shape(s.nB, s.nO, s.nA);
    p.second = operand_shape(s.nA, s.nO, s.nB);
    const size_t walk_lds = vjp_walk_lds(s, sizeof(T), grad_A != nullptr, grad_B != nullptr);
    const bool walk = walks(s, std::max(s.nA, s.nB), walk_lds, thresholds::SAP_VJP_WALK_TILES_PER_WAVE);
    const unsigned grid =
        walk ? walking_workgroups(walk_lds) : static_cast<unsigned>((s.n_rows + ROWS_PER_GROUP - 1) / ROWS_PER_GROUP);
    const size_t lds = walk ? walk_lds : vjp_lds(s, sizeof(T), grad_A != nullptr, grad_B != nullptr);
    const LaunchEvents events = launch_events(stream);
    with_constants<1, 16>(1, p.first.n_groups, [&](auto, auto groups) {
        constexpr int GROUPS = decltype(groups)::value, MANY = MANY_ENTRIES_PER_THREAD;
        auto kernel = s.K <= FEW_ENTRIES ? (walk ? vjp_walk_kernel<T, GROUPS> : vjp_kernel<T, GROUPS>)
                                         : (walk ? vjp_walk_kernel<T, GROUPS, MANY> : vjp_kernel<T, GROUPS, MANY>);
        allow_lds(kernel, lds);
        hipExtLaunchKernelGGL(kernel, dim3(grid), dim3(THREADS), lds, stream, events.start, events.stop, 0, p);
    });
    MOPS_HIP_CHECK(hipGetLastError());
}

template void forward<float>(float*, const float*, const float*, const Table&, const Shape&, hipStream_t);
template void forward<double>(double*, const double*, const double*, const Table&, const Shape&, hipStream_t);
template void forward_of_two_pairs<float>(
    float*, const float*, const float*, const float*, const float*, const Table&, const Shape&, hipStream_t
);
template void forward_of_two_pairs<double>(
    double*, const double*, const double*, const double*, const double*, const Table&, const Shape&, hipStream_t
);
template void vjp<float>(float*, float*, const float*, const float*, const float*, const Table&, const Shape&, hipStream_t);
template void vjp<double>(double*, double*, const double*, const double*, const double*, const Table&, const Shape&, hipStream_t);

} // namespace mops::amd::sap_mfma
