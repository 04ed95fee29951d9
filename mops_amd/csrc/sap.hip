// Sparse accumulation of products (SAP), forward and vector-Jacobian product,
// for gfx950.
//
//   O[i, PO[k]] += C[k] * A[i, PA[k]] * B[i, PB[k]]
//
// Semantics restated from mops/src/sap/cpu.tpp:10-255 of lab-cosmo/mops
// (formula, optional gradients, PO need not be sorted).
//
// Batch-parallel: a lane owns one batch row i, a workgroup 64 consecutive
// rows. Their A, B (and grad_output) rows are loaded with coalesced accesses
// and kept in LDS TRANSPOSED ([feature][row]) so that "feature PA[k] of my
// row" is one conflict-free LDS read whose feature index is the same for the
// whole wavefront.
//
// The table (C, PA, PB, PO) is the same for every row, so all work that
// depends on the table only is done once per call by a small kernel
// (sort_table_kernel): entries with an index out of range are dropped, the
// rest are stably sorted by the column they write to (PO for the forward,
// PA and PB for the two gradients) and packed as {coefficient, LDS byte
// offsets of the operands}. A wavefront of the main kernel then owns whole
// output columns: it walks one column's entries with its sum in a register
// and stores the column once. No flush logic, no partial tiles, no atomics;
// the additions happen in table order, so results are reproducible. The
// packed entries are wave-uniform and come in through the scalar cache four
// at a time, about one scalar-unit instruction per entry: the scalar ALU is
// shared by a whole compute unit and is the first thing this loop would
// otherwise saturate (per-entry bounds checks and offset arithmetic on the
// scalar unit made an earlier version of this kernel six times slower).
//
// Forward only: when there are fewer distinct (PA, PB) pairs than table
// entries (nA * nB <= K), the workgroup first forms all products
// q[pa * nB + pb][row] = A[row, pa] * B[row, pb] in LDS, and an entry costs one
// LDS read and one fused multiply-add. (This evaluates C * (A * B) where the
// reference evaluates (C * A) * B; the last bit can differ.)
//
// Unlike the reference's CUDA kernels (mops/src/sap/sap.cu:41-43, 69-71,
// 300) indices are not packed into 8 bits, and the vjp launches the same grid
// whichever gradients are requested.
#include <algorithm>

#include "mops/sap.hpp"

#include "checks.hpp"
#include "device_common.hpp"
#include "index_validation.hpp"
#include "elementwise.hpp"
#include "runtime.hpp"
#include "sap_mfma.hpp"

namespace mops::amd {
namespace sap { // a name of its own for this file's kernels: profilers print it
namespace {

constexpr int ROWS = WAVE;            // batch rows per workgroup (one per lane)
constexpr int ROW_STRIDE = ROWS + 1;  // odd: transposing stores hit distinct banks
constexpr size_t LDS_BUDGET = 60 * 1024;       // what a workgroup takes by choice
constexpr size_t LARGE_LDS_BUDGET = 150 * 1024; // what it may take before the kernels without LDS are used (160 KB per compute unit)
constexpr int GROUP = 8;              // packed entries fetched together
constexpr int TABLE_PAD = WAVE;       // readable slack after the last packed entry

// ---------------------------------------------------------------------------
// The table, sorted by one of its index columns and packed for the main
// kernels. Arrays have `capacity + TABLE_PAD` elements so that a group load
// that starts inside the table never leaves the allocation.
// ---------------------------------------------------------------------------
// One packed entry: 16 bytes for float and for double, so that a group of
// entries is one aligned scalar load from one running pointer.
template <typename T> struct PackedEntry;
template <> struct alignas(16) PackedEntry<float> {
    float coefficient;
    int32_t first;  // LDS byte offset of the first operand
    int32_t second; // LDS byte offset of the second operand
    int32_t unused;
};
template <> struct alignas(16) PackedEntry<double> {
    double coefficient;
    int32_t first;
    int32_t second;
};

template <typename T> struct PackedTable {
    int32_t* begin;          // [n_buckets + 1] first packed entry of each bucket
    PackedEntry<T>* entries; // [capacity + pad]
};

template <typename T> size_t packed_table_bytes(int32_t n_buckets, int32_t capacity) {
    const size_t slots = static_cast<size_t>(capacity) + TABLE_PAD;
    return align256((static_cast<size_t>(n_buckets) + 1) * 4) + align256(slots * sizeof(PackedEntry<T>));
}

template <typename T>
PackedTable<T> carve_packed_table(char*& cursor, int32_t n_buckets, int32_t capacity) {
    const size_t slots = static_cast<size_t>(capacity) + TABLE_PAD;
    PackedTable<T> table;
    table.begin = reinterpret_cast<int32_t*>(cursor);
    cursor += align256((static_cast<size_t>(n_buckets) + 1) * 4);
    table.entries = reinterpret_cast<PackedEntry<T>*>(cursor);
    cursor += align256(slots * sizeof(PackedEntry<T>));
    return table;
}

// What the bucket and the two operand offsets of a packed entry mean.
constexpr int32_t FORWARD_PRODUCTS = 0; // bucket = po; first = product row of (pa, pb)
constexpr int32_t FORWARD_OPERANDS = 1; // bucket = po; first = a row pa, second = b row pb
constexpr int32_t GRAD_A = 2;           // bucket = pa; first = g row po, second = b row pb
constexpr int32_t GRAD_B = 3;           // bucket = pb; first = g row po, second = a row pa
constexpr int32_t NO_JOB = -1;

constexpr int SORT_THREADS = 1024;
constexpr int SORT_WAVES = SORT_THREADS / WAVE;
constexpr int MAX_BUCKETS = 4096; // LDS counters of the sort kernel
constexpr int WAVE_COUNT_BUCKETS = 256; // up to here the waves of the sort kernel place in parallel

struct SortJob {
    int32_t ordering;
    int32_t n_buckets;
    int32_t* begin;
    void* entries;
};

// One workgroup: stable counting sort of the valid table entries by the
// bucket index of each job, packed output. Stability is obtained by handling
// the 64-entry slices of the table strictly one after the other: inside a
// slice an entry's rank among the entries with the same bucket is the number
// of lower lanes with that bucket.
template <typename T>
__global__ __launch_bounds__(SORT_THREADS) void sort_table_kernel(
    SortJob job0,
    SortJob job1,
    const T* __restrict__ C,
    const int32_t* __restrict__ PA,
    const int32_t* __restrict__ PB,
    const int32_t* __restrict__ PO,
    int32_t n_products,
    int32_t nA,
    int32_t nB,
    int32_t nO,
    int32_t row_bytes,        // LDS bytes between two feature rows of a [feature][65] tile
    int32_t product_row_bytes // LDS bytes between two rows of the product table
) {
    __shared__ int32_t cursor[MAX_BUCKETS + 1];
    __shared__ int32_t wave_count[SORT_WAVES * WAVE_COUNT_BUCKETS];
    __shared__ int32_t scan_tile[SORT_THREADS];
    __shared__ int32_t carry;
    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = tid / WAVE;

    for (int j = 0; j < 2; j++) {
        const SortJob job = j == 0 ? job0 : job1;
        if (job.ordering == NO_JOB) {
            continue; // uniform
        }
        const int32_t ordering = job.ordering;
        const int32_t n_buckets = job.n_buckets;
        PackedEntry<T>* out_entries = static_cast<PackedEntry<T>*>(job.entries);

        __syncthreads();
        for (int32_t b = tid; b <= n_buckets; b += SORT_THREADS) {
            cursor[b] = 0;
        }
        __syncthreads();

        // counts (integer atomics: the totals do not depend on the order)
        for (int32_t k = tid; k < n_products; k += SORT_THREADS) {
            const int32_t pa = PA[k], pb = PB[k], po = PO[k];
            if (in_bounds(pa, nA) && in_bounds(pb, nB) && in_bounds(po, nO)) {
                const int32_t bucket = ordering == GRAD_A ? pa : ordering == GRAD_B ? pb : po;
                atomicAdd(&cursor[bucket], 1);
            }
        }
        __syncthreads();

        // exclusive scan of the counts -> first slot of each bucket
        if (tid == 0) {
            carry = 0;
        }
        __syncthreads();
        for (int32_t base = 0; base <= n_buckets; base += SORT_THREADS) {
            const int32_t b = base + tid;
            const int32_t count = b < n_buckets ? cursor[b] : 0;
            scan_tile[tid] = count;
            __syncthreads();
            for (int distance = 1; distance < SORT_THREADS; distance <<= 1) {
                const int32_t add = tid >= distance ? scan_tile[tid - distance] : 0;
                __syncthreads();
                scan_tile[tid] += add;
                __syncthreads();
            }
            const int32_t exclusive = carry + scan_tile[tid] - count;
            if (b <= n_buckets) {
                cursor[b] = exclusive;
                job.begin[b] = exclusive;
            }
            __syncthreads();
            if (tid == SORT_THREADS - 1) {
                carry += scan_tile[tid];
            }
            __syncthreads();
        }

        // Stable placement. The table is taken in passes of 1024 entries, one
        // 64-entry slice per wave. Inside a slice an entry's rank among the
        // entries with the same bucket is the number of lower lanes with that
        // bucket; between the slices of a pass the order is the wave order.
        // With few buckets every wave first publishes how many entries of
        // each bucket its slice holds, the counts are turned into per-wave
        // start slots, and all waves place their entries at the same time;
        // with many buckets the waves take turns instead.
        const bool parallel = n_buckets <= WAVE_COUNT_BUCKETS;
        for (int32_t base = 0; base < n_products; base += SORT_THREADS) {
            const int32_t k = base + wave * WAVE + lane;
            int32_t pa = 0, pb = 0, po = 0;
            bool valid = false;
            if (k < n_products) {
                pa = PA[k];
                pb = PB[k];
                po = PO[k];
                valid = in_bounds(pa, nA) && in_bounds(pb, nB) && in_bounds(po, nO);
            }
            const int32_t bucket = ordering == GRAD_A ? pa : ordering == GRAD_B ? pb : po;
            int32_t first = 0, second = 0;
            if (ordering == FORWARD_PRODUCTS) {
                first = (pa * nB + pb) * product_row_bytes;
            } else if (ordering == FORWARD_OPERANDS) {
                first = pa * row_bytes;
                second = pb * row_bytes;
            } else if (ordering == GRAD_A) {
                first = po * row_bytes;
                second = pb * row_bytes;
            } else {
                first = po * row_bytes;
                second = pa * row_bytes;
            }
            PackedEntry<T> entry{};
            entry.coefficient = valid ? C[k] : T(0);
            entry.first = first;
            entry.second = second;

            if (parallel) {
                for (int32_t i = tid; i < SORT_WAVES * n_buckets; i += SORT_THREADS) {
                    wave_count[i] = 0;
                }
                __syncthreads();
                // rank inside the slice, and the slice's count per bucket
                int32_t rank = 0;
                unsigned long long todo = __ballot(valid);
                while (todo != 0) {
                    const int leader = __ffsll(static_cast<long long>(todo)) - 1;
                    const int32_t leader_bucket = __shfl(bucket, leader);
                    const bool member = valid && bucket == leader_bucket;
                    const unsigned long long same = __ballot(member);
                    if (member) {
                        rank = __popcll(same & ((1ull << lane) - 1ull));
                    }
                    if (lane == leader) {
                        wave_count[wave * n_buckets + leader_bucket] = __popcll(same);
                    }
                    todo &= ~same;
                }
                __syncthreads();
                // per bucket: start slot of every wave's entries, then advance the cursor
                for (int32_t b = tid; b < n_buckets; b += SORT_THREADS) {
                    int32_t running = cursor[b];
                    for (int w = 0; w < SORT_WAVES; w++) {
                        const int32_t count = wave_count[w * n_buckets + b];
                        wave_count[w * n_buckets + b] = running;
                        running += count;
                    }
                    cursor[b] = running;
                }
                __syncthreads();
                if (valid) {
                    out_entries[wave_count[wave * n_buckets + bucket] + rank] = entry;
                }
                __syncthreads();
            } else {
                for (int turn = 0; turn < SORT_WAVES; turn++) {
                    if (wave == turn) {
                        unsigned long long todo = __ballot(valid);
                        while (todo != 0) {
                            const int leader = __ffsll(static_cast<long long>(todo)) - 1;
                            const int32_t leader_bucket = __shfl(bucket, leader);
                            const bool member = valid && bucket == leader_bucket;
                            const unsigned long long same = __ballot(member);
                            const int32_t slot_base = cursor[leader_bucket];
                            if (member) {
                                out_entries[slot_base + __popcll(same & ((1ull << lane) - 1ull))] = entry;
                            }
                            // every lane has read slot_base before the leader moves the cursor
                            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                            __builtin_amdgcn_wave_barrier();
                            if (lane == leader) {
                                cursor[leader_bucket] = slot_base + __popcll(same);
                            }
                            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                            __builtin_amdgcn_wave_barrier();
                            todo &= ~same;
                        }
                    }
                    __syncthreads();
                }
            }
        }
    }
}

// Copy `rows` x `features` elements starting at `source` (row-major, rows
// contiguous) into LDS as [feature][row].
template <typename T>
__device__ __forceinline__ void stage_transposed(
    T* __restrict__ stage, const T* __restrict__ source, int32_t rows, FastDivisor features
) {
    const int32_t width = static_cast<int32_t>(features.divisor);
    for (int32_t i = threadIdx.x; i < rows * width; i += blockDim.x) {
        int32_t r = static_cast<int32_t>(features.divide(static_cast<uint32_t>(i)));
        int32_t f = i - r * width;
        stage[f * ROW_STRIDE + r] = source[i];
    }
}

// LDS tile [columns][65] -> global rows [rows][columns], coalesced.
template <typename T>
__device__ __forceinline__ void store_transposed(
    T* __restrict__ target, const T* __restrict__ stage, int32_t rows, FastDivisor columns
) {
    const int32_t width = static_cast<int32_t>(columns.divisor);
    for (int32_t i = threadIdx.x; i < rows * width; i += blockDim.x) {
        int32_t r = static_cast<int32_t>(columns.divide(static_cast<uint32_t>(i)));
        int32_t c = i - r * width;
        target[i] = stage[c * ROW_STRIDE + r];
    }
}

template <typename T>
__device__ __forceinline__ T lds_value(const unsigned char* lane_base, int32_t byte_offset) {
    return *reinterpret_cast<const T*>(lane_base + byte_offset);
}

// Broadcast of one lane's value to the whole wavefront through a scalar
// register (v_readlane): no memory access, and the result can feed the next
// instruction as a scalar operand.
__device__ __forceinline__ int32_t broadcast(int32_t value, int lane) {
    return __builtin_amdgcn_readlane(value, lane);
}
__device__ __forceinline__ float broadcast(float value, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(value), lane));
}
__device__ __forceinline__ double broadcast(double value, int lane) {
    const long long bits = __double_as_longlong(value);
    const int32_t low = __builtin_amdgcn_readlane(static_cast<int32_t>(bits), lane);
    const int32_t high = __builtin_amdgcn_readlane(static_cast<int32_t>(bits >> 32), lane);
    return __longlong_as_double(
        (static_cast<long long>(high) << 32) | static_cast<unsigned int>(low)
    );
}

// Sum over the packed entries [k_begin, k_end) of one column, for this lane's
// row. `*_base` point at this lane's element of feature row 0 of the operand
// tiles; the byte offsets in the table are relative to that.
//   ONE operand : sum += c * first
//   TWO operands: sum += (c * first) * second
//
// The entries are wave-uniform data. They are fetched 64 at a time with one
// coalesced vector load (lane j holds entry j) and then handed out to all
// lanes one after the other with v_readlane, so the inner loop has no memory
// access besides the LDS reads of the operands and uses neither the scalar
// cache nor the scalar ALU (which a whole compute unit shares). Slots past
// the end of the column get a zero coefficient and the offset of a cell that
// holds zero (`zero_offset_*`), so the loop runs in whole groups without a
// test per entry and 0 * x can never meet a non-finite x.
template <typename T, bool TWO_OPERANDS>
__device__ __forceinline__ T column_sum(
    const PackedTable<T>& table,
    int32_t k_begin,
    int32_t k_end,
    const unsigned char* first_base,
    const unsigned char* second_base,
    int32_t zero_offset_first,
    int32_t zero_offset_second
) {
    const int lane = threadIdx.x & (WAVE - 1);
    T sum = T(0);
    for (int32_t chunk = k_begin; chunk < k_end; chunk += WAVE) {
        const int32_t n = min(WAVE, k_end - chunk);
        const bool mine = lane < n;
        // the table is padded, so the load itself is always in bounds
        const PackedEntry<T> loaded = table.entries[chunk + (mine ? lane : 0)];
        const T coefficient = mine ? loaded.coefficient : T(0);
        const int32_t first = mine ? loaded.first : zero_offset_first;
        const int32_t second = mine ? loaded.second : zero_offset_second;
        for (int32_t j = 0; j < n; j += GROUP) {
            T x[GROUP], y[GROUP], c[GROUP];
#pragma unroll
            for (int u = 0; u < GROUP; u++) {
                c[u] = broadcast(coefficient, j + u);
                x[u] = lds_value<T>(first_base, broadcast(first, j + u));
                y[u] = TWO_OPERANDS ? lds_value<T>(second_base, broadcast(second, j + u)) : T(1);
            }
#pragma unroll
            for (int u = 0; u < GROUP; u++) {
                if (TWO_OPERANDS) {
                    sum += (c[u] * x[u]) * y[u];
                } else {
                    sum += c[u] * x[u];
                }
            }
        }
    }
    return sum;
}

// ---------------------------------------------------------------------------
// forward. LDS: a[nA][65] b[nB][65] out[nO][65] (products[nA*nB][64])
// ---------------------------------------------------------------------------
template <typename T, bool USE_PRODUCTS>
__global__ __launch_bounds__(1024) void forward_kernel(
    T* __restrict__ output,
    const T* __restrict__ A,
    const T* __restrict__ B,
    PackedTable<T> table,
    int32_t n_rows,
    FastDivisor div_A,
    FastDivisor div_B,
    FastDivisor div_O
) {
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    const int32_t nA = static_cast<int32_t>(div_A.divisor);
    const int32_t nB = static_cast<int32_t>(div_B.divisor);
    const int32_t nO = static_cast<int32_t>(div_O.divisor);
    T* a_stage = reinterpret_cast<T*>(lds_bytes);
    T* b_stage = a_stage + static_cast<size_t>(nA) * ROW_STRIDE;
    T* out_stage = b_stage + static_cast<size_t>(nB) * ROW_STRIDE;
    T* zero_row = out_stage + static_cast<size_t>(nO) * ROW_STRIDE; // [64] zeros
    T* products = zero_row + ROWS;

    const int32_t row0 = blockIdx.x * ROWS;
    const int32_t rows = min(ROWS, n_rows - row0);
    const int lane = threadIdx.x % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int waves = blockDim.x / WAVE;

    stage_transposed(a_stage, A + static_cast<size_t>(row0) * nA, rows, div_A);
    stage_transposed(b_stage, B + static_cast<size_t>(row0) * nB, rows, div_B);
    if (threadIdx.x < ROWS) {
        zero_row[threadIdx.x] = T(0);
    }
    __syncthreads();
    if (USE_PRODUCTS) {
        for (int32_t pair = wave; pair < nA * nB; pair += waves) {
            const int32_t pa = static_cast<int32_t>(div_B.divide(static_cast<uint32_t>(pair)));
            const int32_t pb = pair - pa * nB;
            products[pair * ROWS + lane] =
                a_stage[pa * ROW_STRIDE + lane] * b_stage[pb * ROW_STRIDE + lane];
        }
        __syncthreads();
    }

    const unsigned char* first_base =
        reinterpret_cast<const unsigned char*>((USE_PRODUCTS ? products : a_stage) + lane);
    const unsigned char* second_base = reinterpret_cast<const unsigned char*>(b_stage + lane);
    const unsigned char* zero_base = reinterpret_cast<const unsigned char*>(zero_row + lane);
    const int32_t zero_first = static_cast<int32_t>(zero_base - first_base);
    const int32_t zero_second = static_cast<int32_t>(zero_base - second_base);
    for (int32_t column = wave; column < nO; column += waves) {
        const int32_t k_begin = table.begin[column];
        const int32_t k_end = table.begin[column + 1];
        out_stage[column * ROW_STRIDE + lane] = column_sum<T, !USE_PRODUCTS>(
            table, k_begin, k_end, first_base, second_base, zero_first, zero_second
        );
    }
    __syncthreads();
    store_transposed(output + static_cast<size_t>(row0) * nO, out_stage, rows, div_O);
}

// ---------------------------------------------------------------------------
// vjp
//   grad_A[i, pa] = sum over entries with PA = pa of (C * G[i, PO]) * B[i, PB]
//   grad_B[i, pb] = sum over entries with PB = pb of (C * G[i, PO]) * A[i, PA]
// LDS: g[nO][65] a[nA][65] b[nB][65] out_A[nA][65] out_B[nB][65]
// The nA + nB output columns are dealt to the waves round-robin.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(1024) void vjp_kernel(
    T* __restrict__ grad_A,
    T* __restrict__ grad_B,
    const T* __restrict__ grad_output,
    const T* __restrict__ A,
    const T* __restrict__ B,
    PackedTable<T> by_A,
    PackedTable<T> by_B,
    int32_t n_rows,
    FastDivisor div_A,
    FastDivisor div_B,
    FastDivisor div_O
) {
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    const int32_t nA = static_cast<int32_t>(div_A.divisor);
    const int32_t nB = static_cast<int32_t>(div_B.divisor);
    const int32_t nO = static_cast<int32_t>(div_O.divisor);
    const bool want_A = grad_A != nullptr;
    const bool want_B = grad_B != nullptr;

    T* g_stage = reinterpret_cast<T*>(lds_bytes);
    T* a_stage = g_stage + static_cast<size_t>(nO) * ROW_STRIDE;
    T* b_stage = a_stage + static_cast<size_t>(nA) * ROW_STRIDE;
    T* out_A = b_stage + static_cast<size_t>(nB) * ROW_STRIDE;
    T* out_B = out_A + static_cast<size_t>(nA) * ROW_STRIDE;
    T* zero_row = out_B + static_cast<size_t>(nB) * ROW_STRIDE; // [64] zeros

    const int32_t row0 = blockIdx.x * ROWS;
    const int32_t rows = min(ROWS, n_rows - row0);
    const int lane = threadIdx.x % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int waves = blockDim.x / WAVE;

    stage_transposed(g_stage, grad_output + static_cast<size_t>(row0) * nO, rows, div_O);
    stage_transposed(a_stage, A + static_cast<size_t>(row0) * nA, rows, div_A);
    stage_transposed(b_stage, B + static_cast<size_t>(row0) * nB, rows, div_B);
    if (threadIdx.x < ROWS) {
        zero_row[threadIdx.x] = T(0);
    }
    __syncthreads();

    const unsigned char* g_base = reinterpret_cast<const unsigned char*>(g_stage + lane);
    const unsigned char* a_base = reinterpret_cast<const unsigned char*>(a_stage + lane);
    const unsigned char* b_base = reinterpret_cast<const unsigned char*>(b_stage + lane);
    const unsigned char* zero_base = reinterpret_cast<const unsigned char*>(zero_row + lane);
    const int32_t zero_g = static_cast<int32_t>(zero_base - g_base);
    const int32_t zero_a = static_cast<int32_t>(zero_base - a_base);
    const int32_t zero_b = static_cast<int32_t>(zero_base - b_base);

    // the columns of grad_B hold more entries each than those of grad_A when
    // nB < nA: deal them out first so that the long tasks start first
    const int32_t tasks_B = want_B ? nB : 0;
    const int32_t tasks = tasks_B + (want_A ? nA : 0);
    for (int32_t task = wave; task < tasks; task += waves) {
        if (task < tasks_B) {
            const int32_t column = task;
            out_B[column * ROW_STRIDE + lane] = column_sum<T, true>(
                by_B, by_B.begin[column], by_B.begin[column + 1], g_base, a_base, zero_g, zero_a
            );
        } else {
            const int32_t column = task - tasks_B;
            out_A[column * ROW_STRIDE + lane] = column_sum<T, true>(
                by_A, by_A.begin[column], by_A.begin[column + 1], g_base, b_base, zero_g, zero_b
            );
        }
    }
    __syncthreads();
    if (want_A) {
        store_transposed(grad_A + static_cast<size_t>(row0) * nA, out_A, rows, div_A);
    }
    if (want_B) {
        store_transposed(grad_B + static_cast<size_t>(row0) * nB, out_B, rows, div_B);
    }
}

// ---------------------------------------------------------------------------
// Fallbacks for feature counts whose tiles do not fit in LDS (or more output
// columns than the sort kernel has counters): one thread per batch row,
// accumulating straight into the row of the result in global memory (a row
// belongs to one thread, so there is no race and the order of additions is
// the table order).
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void forward_global_kernel(
    T* output,
    const T* __restrict__ A,
    const T* __restrict__ B,
    const T* __restrict__ C,
    const int32_t* __restrict__ PA,
    const int32_t* __restrict__ PB,
    const int32_t* __restrict__ PO,
    int32_t n_rows,
    int32_t nA,
    int32_t nB,
    int32_t nO,
    int32_t n_products
) {
    const int32_t row = blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= n_rows) {
        return;
    }
    T* o = output + static_cast<size_t>(row) * nO;
    const T* a = A + static_cast<size_t>(row) * nA;
    const T* b = B + static_cast<size_t>(row) * nB;
    for (int32_t column = 0; column < nO; column++) {
        o[column] = T(0);
    }
    for (int32_t k = 0; k < n_products; k++) {
        const int32_t pa = PA[k], pb = PB[k], po = PO[k];
        if (in_bounds(pa, nA) && in_bounds(pb, nB) && in_bounds(po, nO)) {
            o[po] += (C[k] * a[pa]) * b[pb];
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void vjp_global_kernel(
    T* grad_A,
    T* grad_B,
    const T* __restrict__ grad_output,
    const T* __restrict__ A,
    const T* __restrict__ B,
    const T* __restrict__ C,
    const int32_t* __restrict__ PA,
    const int32_t* __restrict__ PB,
    const int32_t* __restrict__ PO,
    int32_t n_rows,
    int32_t nA,
    int32_t nB,
    int32_t nO,
    int32_t n_products
) {
    const int32_t row = blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= n_rows) {
        return;
    }
    const T* g = grad_output + static_cast<size_t>(row) * nO;
    const T* a = A + static_cast<size_t>(row) * nA;
    const T* b = B + static_cast<size_t>(row) * nB;
    T* ga = grad_A != nullptr ? grad_A + static_cast<size_t>(row) * nA : nullptr;
    T* gb = grad_B != nullptr ? grad_B + static_cast<size_t>(row) * nB : nullptr;
    if (ga != nullptr) {
        for (int32_t column = 0; column < nA; column++) {
            ga[column] = T(0);
        }
    }
    if (gb != nullptr) {
        for (int32_t column = 0; column < nB; column++) {
            gb[column] = T(0);
        }
    }
    for (int32_t k = 0; k < n_products; k++) {
        const int32_t pa = PA[k], pb = PB[k], po = PO[k];
        if (in_bounds(pa, nA) && in_bounds(pb, nB) && in_bounds(po, nO)) {
            const T common = C[k] * g[po];
            if (ga != nullptr) {
                ga[pa] += common * b[pb];
            }
            if (gb != nullptr) {
                gb[pb] += common * a[pa];
            }
        }
    }
}

// Waves per workgroup: columns are dealt round-robin, so pick the smallest
// wave count that still gives every wave the same maximum number of columns
// (20 columns on 16 waves would leave 12 waves idle half of the time; 10
// waves with two columns each do the same work with fewer resources).
int pick_waves(size_t n_blocks, int32_t columns) {
    size_t wanted = std::max<size_t>(2, ceil_div(8192, std::max<size_t>(n_blocks, 1)));
    size_t limit = std::min<size_t>(wanted, 16);
    size_t count = static_cast<size_t>(std::max(columns, 1));
    size_t per_wave = ceil_div(count, limit);
    return static_cast<int>(ceil_div(count, per_wave));
}

} // namespace
} // namespace sap
using namespace sap;
} // namespace mops::amd

namespace mops::cuda {

template <typename scalar_t>
void sparse_accumulation_of_products(MOPS_SAP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using namespace mops::amd;
    const char* operation = "cuda_sparse_accumulation_of_products";
    checks::Validator validator(operation);
    checks::sap(validator, output, A, B, C, indices_A, indices_B, indices_output);
    validate_gather_index(indices_A, A.shape[1], "indices_A", operation);
    validate_gather_index(indices_B, B.shape[1], "indices_B", operation);
    validate_gather_index(indices_output, output.shape[1], "indices_output", operation);

    const int32_t n_rows = narrow_i32(A.shape[0], "A.shape[0]");
    const int32_t nA = narrow_i32(A.shape[1], "A.shape[1]");
    const int32_t nB = narrow_i32(B.shape[1], "B.shape[1]");
    const int32_t nO = narrow_i32(output.shape[1], "output.shape[1]");
    const int32_t n_products = narrow_i32(C.shape[0], "C.shape[0]");
    if (n_rows == 0 || nO == 0) {
        return;
    }
    hipStream_t stream = current_stream();
    const sap_mfma::Shape dense_shape{n_rows, nA, nB, nO, n_products};
    if (sap_mfma::supports_forward(dense_shape, sizeof(scalar_t))) {
        const sap_mfma::Table dense_table{C.data, indices_A.data, indices_B.data, indices_output.data};
        sap_mfma::forward<scalar_t>(output.data, A.data, B.data, dense_table, dense_shape, stream);
        finish_call(operation);
        return;
    }
    const size_t n_blocks = ceil_div(static_cast<size_t>(n_rows), ROWS);
    const size_t tile_elements = (static_cast<size_t>(nA) + nB + nO) * ROW_STRIDE + ROWS;
    const size_t product_elements = static_cast<size_t>(nA) * nB * ROWS;
    const bool fits = tile_elements * sizeof(scalar_t) <= LARGE_LDS_BUDGET && nO <= MAX_BUCKETS;
    if (!fits) {
        unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<size_t>(n_rows), 256));
        forward_global_kernel<scalar_t><<<blocks, 256, 0, stream>>>(
            output.data, A.data, B.data, C.data, indices_A.data, indices_B.data, indices_output.data,
            n_rows, nA, nB, nO, n_products
        );
        finish_call(operation);
        return;
    }
    const bool use_products = product_elements <= static_cast<size_t>(n_products) * ROWS &&
                              (tile_elements + product_elements) * sizeof(scalar_t) <= LDS_BUDGET;

    char* cursor = static_cast<char*>(scratch(packed_table_bytes<scalar_t>(nO, n_products)));
    PackedTable<scalar_t> table = carve_packed_table<scalar_t>(cursor, nO, n_products);
    SortJob job{use_products ? FORWARD_PRODUCTS : FORWARD_OPERANDS, nO, table.begin, table.entries};
    SortJob none{NO_JOB, 0, nullptr, nullptr};
    sort_table_kernel<scalar_t><<<1, SORT_THREADS, 0, stream>>>(
        job, none, C.data, indices_A.data, indices_B.data, indices_output.data, n_products, nA, nB, nO,
        static_cast<int32_t>(ROW_STRIDE * sizeof(scalar_t)), static_cast<int32_t>(ROWS * sizeof(scalar_t))
    );

    const int waves = pick_waves(n_blocks, nO);
    const size_t lds = (tile_elements + (use_products ? product_elements : 0)) * sizeof(scalar_t);
    MainKernelTimer timer(stream);
    if (lds > 64 * 1024) {
        // (only without the product table: with it the tiles stay below LDS_BUDGET)
        MOPS_HIP_CHECK(hipFuncSetAttribute(
            reinterpret_cast<const void*>(forward_kernel<scalar_t, false>),
            hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)
        ));
    }
    if (use_products) {
        forward_kernel<scalar_t, true><<<static_cast<unsigned>(n_blocks), waves * WAVE, lds, stream>>>(
            output.data, A.data, B.data, table, n_rows, FastDivisor::make(nA), FastDivisor::make(nB),
            FastDivisor::make(nO)
        );
    } else {
        forward_kernel<scalar_t, false><<<static_cast<unsigned>(n_blocks), waves * WAVE, lds, stream>>>(
            output.data, A.data, B.data, table, n_rows, FastDivisor::make(nA), FastDivisor::make(nB),
            FastDivisor::make(nO)
        );
    }
    finish_call(operation);
}

template <typename scalar_t>
void sparse_accumulation_of_products_vjp(MOPS_SAP_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using namespace mops::amd;
    const char* operation = "cuda_sparse_accumulation_of_products_vjp";
    checks::Validator validator(operation);
    checks::sap_vjp(validator, grad_A, grad_B, grad_output, A, B, C, indices_A, indices_B, indices_output);
    const bool want_A = grad_A.data != nullptr;
    const bool want_B = grad_B.data != nullptr;
    if (!want_A && !want_B) {
        return;
    }
    validate_gather_index(indices_A, A.shape[1], "indices_A", operation);
    validate_gather_index(indices_B, B.shape[1], "indices_B", operation);
    validate_gather_index(indices_output, grad_output.shape[1], "indices_output", operation);

    const int32_t n_rows = narrow_i32(A.shape[0], "A.shape[0]");
    const int32_t nA = narrow_i32(A.shape[1], "A.shape[1]");
    const int32_t nB = narrow_i32(B.shape[1], "B.shape[1]");
    const int32_t nO = narrow_i32(grad_output.shape[1], "grad_output.shape[1]");
    const int32_t n_products = narrow_i32(C.shape[0], "C.shape[0]");
    if (n_rows == 0) {
        return;
    }
    hipStream_t stream = current_stream();
    const sap_mfma::Shape dense_shape{n_rows, nA, nB, nO, n_products};
    if (sap_mfma::supports_vjp(dense_shape, sizeof(scalar_t))) {
        const sap_mfma::Table dense_table{C.data, indices_A.data, indices_B.data, indices_output.data};
        sap_mfma::vjp<scalar_t>(
            grad_A.data, grad_B.data, grad_output.data, A.data, B.data, dense_table, dense_shape, stream
        );
        finish_call(operation);
        return;
    }
    const size_t n_blocks = ceil_div(static_cast<size_t>(n_rows), ROWS);
    const size_t tile_elements =
        (static_cast<size_t>(nO) + 2 * (static_cast<size_t>(nA) + nB)) * ROW_STRIDE + ROWS;
    const bool fits =
        tile_elements * sizeof(scalar_t) <= LARGE_LDS_BUDGET && nA <= MAX_BUCKETS && nB <= MAX_BUCKETS;
    if (!fits) {
        unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<size_t>(n_rows), 256));
        vjp_global_kernel<scalar_t><<<blocks, 256, 0, stream>>>(
            grad_A.data, grad_B.data, grad_output.data, A.data, B.data, C.data, indices_A.data,
            indices_B.data, indices_output.data, n_rows, nA, nB, nO, n_products
        );
        finish_call(operation);
        return;
    }

    char* cursor = static_cast<char*>(scratch(
        packed_table_bytes<scalar_t>(nA, n_products) + packed_table_bytes<scalar_t>(nB, n_products)
    ));
    PackedTable<scalar_t> by_A = carve_packed_table<scalar_t>(cursor, nA, n_products);
    PackedTable<scalar_t> by_B = carve_packed_table<scalar_t>(cursor, nB, n_products);
    SortJob none{NO_JOB, 0, nullptr, nullptr};
    SortJob job_A = want_A ? SortJob{GRAD_A, nA, by_A.begin, by_A.entries} : none;
    SortJob job_B = want_B ? SortJob{GRAD_B, nB, by_B.begin, by_B.entries} : none;
    sort_table_kernel<scalar_t><<<1, SORT_THREADS, 0, stream>>>(
        job_A, job_B, C.data, indices_A.data, indices_B.data, indices_output.data, n_products, nA, nB,
        nO, static_cast<int32_t>(ROW_STRIDE * sizeof(scalar_t)), static_cast<int32_t>(ROWS * sizeof(scalar_t))
    );

    // A column is summed by one wave in table order, so the bits of a
    // gradient do not depend on the wave count or on whether the other
    // gradient is computed alongside.
    const int waves = pick_waves(n_blocks, (want_A ? nA : 0) + (want_B ? nB : 0));
    const size_t lds = tile_elements * sizeof(scalar_t);
    MainKernelTimer timer(stream);
    if (lds > 64 * 1024) {
        MOPS_HIP_CHECK(hipFuncSetAttribute(
            reinterpret_cast<const void*>(vjp_kernel<scalar_t>), hipFuncAttributeMaxDynamicSharedMemorySize,
            static_cast<int>(lds)
        ));
    }
    vjp_kernel<scalar_t><<<static_cast<unsigned>(n_blocks), waves * WAVE, lds, stream>>>(
        grad_A.data, grad_B.data, grad_output.data, A.data, B.data, by_A, by_B, n_rows,
        FastDivisor::make(nA), FastDivisor::make(nB), FastDivisor::make(nO)
    );
    finish_call(operation);
}

// Second order (semantics of mops/src/sap/cpu.tpp:257-541). The operation is
// bilinear in A and B, so every output is a first-order call with one operand
// replaced by a cotangent:
//   grad_grad_output = forward(grad_grad_A, B) + forward(A, grad_grad_B)
//   grad_A_2         = vjp's grad_A with B := grad_grad_B
//   grad_B_2         = vjp's grad_B with A := grad_grad_A
// A cotangent that is not given counts as zero.
template <typename scalar_t>
void sparse_accumulation_of_products_vjp_vjp(MOPS_SAP_VJP_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using namespace mops::amd;
    const char* operation = "cuda_sparse_accumulation_of_products_vjp_vjp";
    checks::Validator validator(operation);
    checks::sap_vjp_vjp(
        validator, grad_grad_output, grad_A_2, grad_B_2, grad_grad_A, grad_grad_B, grad_output, A, B, C,
        indices_A, indices_B, indices_output
    );
    validate_gather_index(indices_A, A.shape[1], "indices_A", operation);
    validate_gather_index(indices_B, B.shape[1], "indices_B", operation);
    validate_gather_index(indices_output, grad_output.shape[1], "indices_output", operation);
    const bool have_A = grad_grad_A.data != nullptr, have_B = grad_grad_B.data != nullptr;
    const Tensor<scalar_t, 2> nothing{nullptr, {0, 0}};
    hipStream_t stream = current_stream();
    const size_t output_count = grad_output.shape[0] * grad_output.shape[1];

    if (grad_grad_output.data != nullptr) {
        const sap_mfma::Shape dense_shape{
            narrow_i32(A.shape[0], "A.shape[0]"), narrow_i32(A.shape[1], "A.shape[1]"),
            narrow_i32(B.shape[1], "B.shape[1]"), narrow_i32(grad_output.shape[1], "grad_output.shape[1]"),
            narrow_i32(C.shape[0], "C.shape[0]")};
        if (have_A && have_B && sap_mfma::supports_forward_of_two_pairs(dense_shape, sizeof(scalar_t))) {
            // both terms in the sums of one launch
            const sap_mfma::Table dense_table{C.data, indices_A.data, indices_B.data, indices_output.data};
            sap_mfma::forward_of_two_pairs<scalar_t>(
                grad_grad_output.data, grad_grad_A.data, B.data, A.data, grad_grad_B.data, dense_table,
                dense_shape, stream
            );
        } else if (have_A && have_B) {
            ::mops::cuda::sparse_accumulation_of_products<scalar_t>(
                grad_grad_output, grad_grad_A, B, C, indices_A, indices_B, indices_output
            );
            StreamTemporary<scalar_t> second(output_count, stream);
            ::mops::cuda::sparse_accumulation_of_products<scalar_t>(
                Tensor<scalar_t, 2>{second.data(), {grad_output.shape[0], grad_output.shape[1]}}, A,
                grad_grad_B, C, indices_A, indices_B, indices_output
            );
            add_in_place<scalar_t>(grad_grad_output.data, second.data(), output_count, stream);
        } else if (have_B) {
            ::mops::cuda::sparse_accumulation_of_products<scalar_t>(
                grad_grad_output, A, grad_grad_B, C, indices_A, indices_B, indices_output
            );
        } else if (have_A) {
            ::mops::cuda::sparse_accumulation_of_products<scalar_t>(
                grad_grad_output, grad_grad_A, B, C, indices_A, indices_B, indices_output
            );
        } else {
            fill_zero<scalar_t>(grad_grad_output.data, output_count, stream);
        }
    }
    if (grad_A_2.data != nullptr && grad_B_2.data != nullptr && have_A && have_B) {
        // grad_A_2 is the vjp's grad_A with grad_grad_B for B, grad_B_2 its grad_B with
        // grad_grad_A for A, and neither gradient of the vjp reads its own tensor: one call
        ::mops::cuda::sparse_accumulation_of_products_vjp<scalar_t>(
            grad_A_2, grad_B_2, grad_output, grad_grad_A, grad_grad_B, C, indices_A, indices_B, indices_output
        );
        finish_call(operation);
        return;
    }
    if (grad_A_2.data != nullptr) {
        if (have_B) {
            ::mops::cuda::sparse_accumulation_of_products_vjp<scalar_t>(
                grad_A_2, nothing, grad_output, A, grad_grad_B, C, indices_A, indices_B, indices_output
            );
        } else {
            fill_zero<scalar_t>(grad_A_2.data, A.shape[0] * A.shape[1], stream);
        }
    }
    if (grad_B_2.data != nullptr) {
        if (have_A) {
            ::mops::cuda::sparse_accumulation_of_products_vjp<scalar_t>(
                nothing, grad_B_2, grad_output, grad_grad_A, B, C, indices_A, indices_B, indices_output
            );
        } else {
            fill_zero<scalar_t>(grad_B_2.data, B.shape[0] * B.shape[1], stream);
        }
    }
    finish_call(operation);
}

MOPS_CXX_INSTANTIATE(sparse_accumulation_of_products, MOPS_SAP_PARAMS)
MOPS_CXX_INSTANTIATE(sparse_accumulation_of_products_vjp, MOPS_SAP_VJP_PARAMS)
MOPS_CXX_INSTANTIATE(sparse_accumulation_of_products_vjp_vjp, MOPS_SAP_VJP_VJP_PARAMS)

} // namespace mops::cuda
