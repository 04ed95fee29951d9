// Homogeneous polynomial evaluation (HPE), forward and vector-Jacobian
// product, for gfx950.
//
//   O[i] = sum_j C[j] * prod_k A[i, P[j, k]]
//   grad_A[i, P[j, f]] += C[j] * grad_O[i] * prod_{k != f} A[i, P[j, k]]
//
// Semantics restated from mops/src/hpe/cpu.tpp:13-272 of lab-cosmo/mops:
// each monomial's product starts from C[j] and multiplies the factors left
// to right; a polynomial of order 0 gives O[i] = sum_j C[j]; the vjp is a
// no-op when grad_A is not requested. (The CPU reference stops at order 10;
// there is no such limit here.)
//
// Work split: a workgroup takes `R` consecutive batch rows (R a power of two,
// 1..64) and G = blockDim / R monomial groups; thread (r, g) evaluates the
// monomials j = g, g + G, ... for row r. The rows' A values sit in LDS as
// [feature][row]. Small batches get R = 1 (the whole workgroup shares one row
// and spreads over the monomials), large batches R = 64 (one row per lane,
// the table read once per wavefront), so that there are always enough
// workgroups to fill the device.
//
// The partial sums of the G groups are combined in group order, so results
// are reproducible from run to run. The reference's CUDA vjp accumulates
// with shared-memory float atomics (mops/src/hpe/hpe.cu:288) and is not.
#include <algorithm>
#include <type_traits>

#include "mops/hpe.hpp"

#include "checks.hpp"
#include "device_common.hpp"
#include "dispatch_thresholds.hpp"
#include "index_validation.hpp"
#include "elementwise.hpp"
#include "runtime.hpp"
#include "sender_buckets.hpp"

namespace mops::amd {
namespace hpe { // a name of its own for this file's kernels: profilers print it
namespace {

constexpr size_t LDS_BUDGET = 60 * 1024;
constexpr int32_t MANY_ROWS = thresholds::HPE_VJP_BY_FEATURE_ROWS;            // from here on the vjp goes by feature
constexpr int32_t FORWARD_MANY_ROWS = thresholds::HPE_FORWARD_LANE_PER_ROW_ROWS; // from here on the forward pass has a lane per row
constexpr size_t BY_FEATURE_LDS_BUDGET = 140 * 1024;    // its two tiles, of the 160 KB of a compute unit

// ---------------------------------------------------------------------------
// forward. LDS: a[nA][R] partial[G][R]
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void forward_kernel(
    T* __restrict__ output,
    const T* __restrict__ A,
    const T* __restrict__ C,
    const int32_t* __restrict__ P,
    int32_t n_rows,
    int32_t nA,
    int32_t n_monomials,
    int32_t order,
    int32_t R
) {
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    T* a_stage = reinterpret_cast<T*>(lds_bytes);
    T* partial = a_stage + static_cast<size_t>(nA) * R;

    const int tid = threadIdx.x;
    const int G = blockDim.x / R;
    const int r = tid % R;
    const int g = tid / R;
    const int32_t row0 = blockIdx.x * R;
    const int32_t rows = min(R, n_rows - row0);

    const T* a_src = A + static_cast<size_t>(row0) * nA;
    for (int32_t i = tid; i < rows * nA; i += blockDim.x) {
        int32_t row = i / nA;
        a_stage[(i - row * nA) * R + row] = a_src[i];
    }
    __syncthreads();

    T sum = T(0);
    if (r < rows) {
        for (int32_t j = g; j < n_monomials; j += G) {
            const int32_t* factors = P + static_cast<size_t>(j) * order;
            T product = C[j];
            for (int32_t k = 0; k < order; k++) {
                int32_t feature = factors[k];
                product *= in_bounds(feature, nA) ? a_stage[feature * R + r] : T(0);
            }
            sum += product;
        }
    }
    partial[g * R + r] = sum;
    __syncthreads();
    if (g == 0 && r < rows) {
        T total = T(0);
        for (int group = 0; group < G; group++) {
            total += partial[group * R + r];
        }
        output[row0 + r] = total;
    }
}

// ---------------------------------------------------------------------------
// forward with the order known at compile time: factors and the values they
// select in registers, the next monomial fetched while the current one is
// multiplied, and the partial sums of the groups combined by a fixed tree
// (shuffles inside a wavefront, then the wavefronts in order) instead of one
// thread walking over all of them. R is a power of two.
// ---------------------------------------------------------------------------
template <typename T, int ORDER>
__global__ __launch_bounds__(256) void forward_ordered_kernel(
    T* __restrict__ output,
    const T* __restrict__ A,
    const T* __restrict__ C,
    const int32_t* __restrict__ P,
    int32_t n_rows,
    int32_t nA,
    int32_t n_monomials,
    int32_t R
) {
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    // a[nA + 1][R]: the row after the last stays zero, a factor outside [0, nA)
    // reads it, and the loop over the monomials has no branch in it
    T* a_stage = reinterpret_cast<T*>(lds_bytes);
    T* partial = a_stage + static_cast<size_t>(nA + 1) * R;

    const int tid = threadIdx.x;
    const int G = blockDim.x / R;
    const int r = tid % R;
    const int g = tid / R;
    const int32_t row0 = blockIdx.x * R;
    const int32_t rows = min(R, n_rows - row0);

    const T* a_src = A + static_cast<size_t>(row0) * nA;
    for (int32_t i = tid; i < rows * nA; i += blockDim.x) {
        int32_t row = i / nA;
        a_stage[(i - row * nA) * R + row] = a_src[i];
    }
    if (tid < R) {
        a_stage[nA * R + tid] = T(0);
    }
    __syncthreads();

    struct Monomial {
        int32_t factor[ORDER > 0 ? ORDER : 1];
        T coefficient;
    };
    auto fetch = [&](Monomial& to, int32_t j) {
        const int32_t safe = min(j, n_monomials - 1);
        const int32_t* factors = P + static_cast<size_t>(safe) * ORDER;
#pragma unroll
        for (int k = 0; k < ORDER; k++) {
            to.factor[k] = factors[k];
        }
        to.coefficient = C[safe];
    };
    // BATCH monomials at a time: their factors asked for together, then their
    // values of A, then the products (independent chains); a monomial beyond
    // the last counts with coefficient zero.
    T sum = T(0);
    if (r < rows && n_monomials > 0) {
        constexpr int BATCH = 4;
        const uint32_t features = static_cast<uint32_t>(nA);
        const T* my_a = a_stage + r;
        Monomial next[BATCH];
#pragma unroll
        for (int d = 0; d < BATCH; d++) {
            fetch(next[d], g + d * G);
        }
        for (int32_t j0 = g; j0 < n_monomials; j0 += BATCH * G) {
            Monomial now[BATCH];
            T value[BATCH][ORDER > 0 ? ORDER : 1];
#pragma unroll
            for (int d = 0; d < BATCH; d++) {
                now[d] = next[d];
#pragma unroll
                for (int k = 0; k < ORDER; k++) {
                    // (as unsigned, a negative factor is a large one)
                    value[d][k] = my_a[min(static_cast<uint32_t>(now[d].factor[k]), features) * R];
                }
            }
#pragma unroll
            for (int d = 0; d < BATCH; d++) {
                fetch(next[d], j0 + (d + BATCH) * G);
            }
#pragma unroll
            for (int d = 0; d < BATCH; d++) {
                T product = j0 + d * G < n_monomials ? now[d].coefficient : T(0);
#pragma unroll
                for (int k = 0; k < ORDER; k++) {
                    product *= value[d][k];
                }
                sum += product;
            }
        }
    }
    // lanes with the same r inside a wavefront, then the wavefronts
    for (int offset = WAVE / 2; offset >= R; offset >>= 1) {
        sum += __shfl_xor(sum, offset);
    }
    const int wave = tid / WAVE;
    const int lane = tid % WAVE;
    if (R <= WAVE) {
        if (lane < R) {
            partial[wave * R + lane] = sum;
        }
    } else {
        partial[g * R + r] = sum;
    }
    __syncthreads();
    const int copies = R <= WAVE ? static_cast<int>(blockDim.x) / WAVE : G;
    if (tid < rows) {
        T total = T(0);
        for (int copy = 0; copy < copies; copy++) {
            total += partial[copy * R + tid];
        }
        output[row0 + tid] = total;
    }
}

// ---------------------------------------------------------------------------
// vjp. One wavefront per workgroup. LDS: a[nA][R] accumulator[G][span][R]
// Thread (r, g) adds its monomials' terms into its private accumulator row
// set; afterwards the G copies are added in group order.
// `span` = nA when the accumulators of all features fit in LDS; otherwise the
// features are split into ranges of `span`, blockIdx.y picks the range, and a
// workgroup walks all monomials but keeps only the terms for its range.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(WAVE) void vjp_kernel(
    T* __restrict__ grad_A,
    const T* __restrict__ grad_output,
    const T* __restrict__ A,
    const T* __restrict__ C,
    const int32_t* __restrict__ P,
    int32_t n_rows,
    int32_t nA,
    int32_t n_monomials,
    int32_t order,
    int32_t R,
    int32_t span
) {
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    T* a_stage = reinterpret_cast<T*>(lds_bytes);
    T* accumulator = a_stage + static_cast<size_t>(nA) * R;
    const int32_t feature_begin = blockIdx.y * span;
    const int32_t feature_count = min(span, nA - feature_begin);

    const int tid = threadIdx.x;
    const int G = WAVE / R;
    const int r = tid % R;
    const int g = tid / R;
    const int32_t row0 = blockIdx.x * R;
    const int32_t rows = min(R, n_rows - row0);

    const T* a_src = A + static_cast<size_t>(row0) * nA;
    for (int32_t i = tid; i < rows * nA; i += WAVE) {
        int32_t row = i / nA;
        a_stage[(i - row * nA) * R + row] = a_src[i];
    }
    for (int32_t i = tid; i < G * feature_count * R; i += WAVE) {
        accumulator[i] = T(0);
    }
    __syncthreads();

    if (r < rows) {
        T* mine = accumulator + static_cast<size_t>(g) * feature_count * R + r;
        const T upstream = grad_output[row0 + r];
        for (int32_t j = g; j < n_monomials; j += G) {
            const int32_t* factors = P + static_cast<size_t>(j) * order;
            const T base = C[j] * upstream;
            for (int32_t f = 0; f < order; f++) {
                int32_t target = factors[f] - feature_begin;
                if (!in_bounds(target, feature_count)) {
                    continue;
                }
                T term = base;
                for (int32_t k = 0; k < order; k++) {
                    if (k == f) {
                        continue;
                    }
                    int32_t feature = factors[k];
                    term *= in_bounds(feature, nA) ? a_stage[feature * R + r] : T(0);
                }
                mine[target * R] += term;
            }
        }
    }
    __syncthreads();

    T* dst = grad_A + static_cast<size_t>(row0) * nA + feature_begin;
    for (int32_t i = tid; i < rows * feature_count; i += WAVE) {
        int32_t row = i / feature_count;
        int32_t feature = i - row * feature_count;
        T total = T(0);
        for (int group = 0; group < G; group++) {
            total += accumulator[(static_cast<size_t>(group) * feature_count + feature) * R + row];
        }
        dst[static_cast<size_t>(row) * nA + feature] = total;
    }
}

// ---------------------------------------------------------------------------
// vjp with the order known at compile time: same layout as vjp_kernel, but a
// monomial's factors, the values they select and the K partial products
// (prefix * suffix, 3 K multiplications instead of K^2) live in registers, and
// the factors of the next monomial are fetched while the current one is used.
// ---------------------------------------------------------------------------
constexpr int ORDERED_VJP_THREADS = 4 * WAVE; // one wavefront that walks the monomials and three helpers

template <typename T, int ORDER, bool ALL_FEATURES>
__global__ __launch_bounds__(ORDERED_VJP_THREADS) void vjp_ordered_kernel(
    T* __restrict__ grad_A,
    const T* __restrict__ grad_output,
    const T* __restrict__ A,
    const T* __restrict__ C,
    const int32_t* __restrict__ P,
    int32_t n_rows,
    int32_t nA,
    int32_t n_monomials,
    int32_t log2_R,
    int32_t span
) {
    // LDS: a[nA + 1][R] accumulator[G][feature_count + 1][R]. The extra row of
    // `a` stays zero and the extra accumulator row is never read: a factor
    // outside [0, nA) reads the one, a term that is not to be kept (a feature
    // of another range, a monomial beyond the last) goes to the other, and
    // the loop over the monomials has no branch in it.
    // ALL_FEATURES: span == nA, the workgroup keeps the terms of all features.
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    const int32_t R = 1 << log2_R;
    T* a_stage = reinterpret_cast<T*>(lds_bytes);
    T* accumulator = a_stage + static_cast<size_t>(nA + 1) * R;
    const int32_t feature_begin = ALL_FEATURES ? 0 : blockIdx.y * span;
    const int32_t feature_count = ALL_FEATURES ? nA : min(span, nA - feature_begin);

    // Thread (r, g) of the FIRST wavefront walks the monomials; the other
    // wavefronts of the workgroup only help to stage the rows, to clear the
    // accumulators and to add up the copies, which a single wavefront would
    // spend a third of the launch on.
    const int tid = threadIdx.x;
    const bool walks = tid < WAVE;
    const int G = WAVE >> log2_R;
    const int r = tid & (R - 1);
    const int g = (tid & (WAVE - 1)) >> log2_R;
    const int32_t row0 = blockIdx.x * R;
    const int32_t rows = min(R, n_rows - row0);

    struct Monomial {
        int32_t factor[ORDER];
        T coefficient;
    };
    auto fetch = [&](Monomial& to, int32_t j) {
        const int32_t safe = min(j, n_monomials - 1);
        const int32_t* factors = P + static_cast<size_t>(safe) * ORDER;
#pragma unroll
        for (int k = 0; k < ORDER; k++) {
            to.factor[k] = factors[k];
        }
        to.coefficient = C[safe];
    };
    // A compute unit holds three of these wavefronts (their accumulators fill
    // its LDS), so nobody else covers a thread's waits and every instruction
    // counts. A thread works on BATCH monomials at a time, in three phases:
    // all their values of A are asked for from LDS together, then all their
    // terms are multiplied up in registers (BATCH independent chains), then
    // all terms are added to the accumulators, in the order of the
    // monomials. The factors of the next batch are on their way from global
    // memory meanwhile, those of the first one while the tiles are set up.
    constexpr int BATCH = 8;
    Monomial queue[BATCH];
    T upstream = T(0);
    if (walks) {
#pragma unroll
        for (int d = 0; d < BATCH; d++) {
            fetch(queue[d], g + d * G);
        }
        upstream = grad_output[min(row0 + r, n_rows - 1)];
    }

    // the rows of A, STAGE values per lane asked for together: with one load
    // per turn of a loop, each turn would wait a whole round trip to memory
    const T* a_src = A + static_cast<size_t>(row0) * nA;
    constexpr int STAGE = 8;
    for (int32_t base = 0; base < rows * nA; base += STAGE * ORDERED_VJP_THREADS) {
        T staged[STAGE];
#pragma unroll
        for (int u = 0; u < STAGE; u++) {
            const int32_t i = base + u * ORDERED_VJP_THREADS + tid;
            staged[u] = a_src[min(i, rows * nA - 1)];
        }
#pragma unroll
        for (int u = 0; u < STAGE; u++) {
            const int32_t i = base + u * ORDERED_VJP_THREADS + tid;
            if (i < rows * nA) {
                const int32_t row = i / nA;
                a_stage[((i - row * nA) << log2_R) + row] = staged[u];
            }
        }
    }
    if (tid < R) {
        a_stage[nA * R + tid] = T(0);
    }
    // (G * R = 64: the accumulators are feature_count + 1 rows of 64 values, one
    // per lane; wavefront w clears rows w, w + 4, ...; unrolled, because a
    // wavefront pays for every instruction of the loop around a store)
    {
        constexpr int HELPERS = ORDERED_VJP_THREADS / WAVE;
        T* clear = accumulator + (tid & (WAVE - 1));
        int32_t k = tid >> 6;
        for (; k + 7 * HELPERS < feature_count + 1; k += 8 * HELPERS) {
#pragma unroll
            for (int u = 0; u < 8; u++) {
                clear[(k + u * HELPERS) * WAVE] = T(0);
            }
        }
        for (; k < feature_count + 1; k += HELPERS) {
            clear[k * WAVE] = T(0);
        }
    }
    __syncthreads();

    if (walks && r < rows) {
        T* mine = accumulator + static_cast<size_t>(g) * (feature_count + 1) * R + r;
        const T* my_a = a_stage + r;
        // a feature's distance in bytes as a shift: address = base + (feature << shift), one
        // instruction (shift-and-add) per LDS access instead of a shift, a scaling and an add
        const int32_t byte_shift = log2_R + (sizeof(T) == 8 ? 3 : 2);
        auto at = [&](auto* base, uint32_t feature) {
            using Pointer = decltype(base);
            using Bytes = std::conditional_t<std::is_const_v<std::remove_pointer_t<Pointer>>, const char*, char*>;
            return reinterpret_cast<Pointer>(reinterpret_cast<Bytes>(base) + (feature << byte_shift));
        };
        const uint32_t features = static_cast<uint32_t>(nA);
        const uint32_t kept = static_cast<uint32_t>(feature_count);
        // `whole`: all monomials of the batch exist
        auto batch = [&](int32_t j0, auto whole) {
            constexpr bool WHOLE = decltype(whole)::value;
            Monomial now[BATCH];
            T value[BATCH][ORDER];
#pragma unroll
            for (int d = 0; d < BATCH; d++) {
                now[d] = queue[d];
#pragma unroll
                for (int k = 0; k < ORDER; k++) {
                    // (as unsigned, a negative factor is a large one)
                    const uint32_t feature = min(static_cast<uint32_t>(now[d].factor[k]), features);
                    value[d][k] = *at(my_a, feature);
                }
            }
            if constexpr (WHOLE) {
#pragma unroll
                for (int d = 0; d < BATCH; d++) {
                    fetch(queue[d], j0 + (d + BATCH) * G);
                }
            }
            // term[f] = base * prod_{k != f} value[k], multiplied left to right
            T term[BATCH][ORDER];
#pragma unroll
            for (int d = 0; d < BATCH; d++) {
                T prefix[ORDER];
                prefix[0] = now[d].coefficient * upstream;
#pragma unroll
                for (int k = 1; k < ORDER; k++) {
                    prefix[k] = prefix[k - 1] * value[d][k - 1];
                }
                T suffix = T(1);
#pragma unroll
                for (int f = ORDER - 1; f >= 0; f--) {
                    term[d][f] = prefix[f] * suffix;
                    suffix *= value[d][f];
                }
            }
#pragma unroll
            for (int d = 0; d < BATCH; d++) {
                const bool exists = WHOLE || j0 + d * G < n_monomials;
#pragma unroll
                for (int f = ORDER - 1; f >= 0; f--) {
                    uint32_t slot = static_cast<uint32_t>(now[d].factor[f]);
                    if constexpr (!ALL_FEATURES) {
                        slot -= static_cast<uint32_t>(feature_begin);
                    }
                    slot = min(slot, kept);
                    T* to = at(mine, exists ? slot : kept);
                    // a slot of my own. In f64 the LDS add instruction, which saves the
                    // round trip of read, add, write; in f32 that instruction is the
                    // slower way here (53 us against 21)
                    if constexpr (sizeof(T) == 8) {
                        unsafeAtomicAdd(to, term[d][f]);
                    } else {
                        *to += term[d][f];
                    }
                }
            }
        };
        int32_t j0 = g;
        for (; j0 + (BATCH - 1) * G < n_monomials; j0 += BATCH * G) {
            batch(j0, std::true_type{});
        }
        if (j0 < n_monomials) {
            batch(j0, std::false_type{});
        }
    }
    __syncthreads();

    // The G copies added up, every (feature, row) by one lane: four running
    // sums over the copies g = 0, 4, ... / 1, 5, ... / 2, 6, ... / 3, 7, ...
    // and then (s0 + s1) + (s2 + s3): one fixed order, and chains of additions
    // a quarter as long as one sum over all copies would be.
    T* dst = grad_A + static_cast<size_t>(row0) * nA + feature_begin;
    const int32_t copy_stride = (feature_count + 1) * R;
    for (int32_t entry = tid; entry < feature_count * R; entry += ORDERED_VJP_THREADS) {
        const int32_t row = entry & (R - 1);
        const int32_t feature = entry >> log2_R;
        const T* from = accumulator + entry;
        T partial[4] = {T(0), T(0), T(0), T(0)};
        int group = 0;
        for (; group + 4 <= G; group += 4) {
#pragma unroll
            for (int u = 0; u < 4; u++) {
                partial[u] += from[(group + u) * copy_stride];
            }
        }
        for (; group < G; group++) {
            partial[group & 3] += from[group * copy_stride];
        }
        if (row < rows) {
            dst[static_cast<size_t>(row) * nA + feature] = (partial[0] + partial[1]) + (partial[2] + partial[3]);
        }
    }
}

// ---------------------------------------------------------------------------
// vjp for MANY rows, by feature. With thousands of rows the kernel above is
// bound by its LDS add instructions (one per factor of every monomial and
// row). Here nothing is scattered: the table is first turned round on the
// device (sender_buckets.hpp, the same counting sort that orders edges by
// sender: for every feature a the list of pairs q = j * ORDER + f with
// P[j, f] = a, in ascending q), and then a wavefront owns (64 rows, one
// feature at a time): a lane is a row, walks the feature's list, multiplies
// up the OTHER factors of its row from an LDS tile of A and adds the terms in
// a register:
//
//   grad_A[i, a] = gO[i] * sum over (j, f) in list(a) of C[j] * prod_{k != f} A[i, P[j, k]]
//
// The list entries are read 64 at a time, one per lane, and handed out to all
// lanes through readlane. One fixed order (ascending q), no atomics.
// LDS: a[nA][ROW_PITCH] out[64][out_pitch]
// ---------------------------------------------------------------------------
constexpr int FEATURE_WAVES = 16;
/// Rows per workgroup when a lane has RPL rows (lane, lane + 64, ...: the table entry a
/// wavefront is at then serves RPL rows per lane for the same readlanes and address)
__host__ __device__ constexpr int feature_rows(int rpl) { return WAVE * rpl; }
/// Distance between features in the tile of A
__host__ __device__ constexpr int feature_row_pitch(int rpl) { return WAVE * rpl + 1; }

template <typename T, int ORDER, int RPL>
__global__ __launch_bounds__(FEATURE_WAVES* WAVE) void vjp_by_feature_kernel(
    T* __restrict__ grad_A,
    const T* __restrict__ grad_output,
    const T* __restrict__ A,
    const T* __restrict__ C,
    const int32_t* __restrict__ P,
    const int32_t* __restrict__ list_begin, // [nA + 1]
    const int32_t* __restrict__ list,       // pairs q = j * ORDER + f, grouped by feature
    int32_t n_rows,
    int32_t nA,
    int32_t features_per_group, // blockIdx.y takes the features [y, y + 1) * features_per_group
    int32_t out_pitch
) {
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    T* a_stage = reinterpret_cast<T*>(lds_bytes);
    T* out = a_stage + static_cast<size_t>(nA) * feature_row_pitch(RPL);
    const int32_t first_feature = blockIdx.y * features_per_group;
    const int32_t n_features = min(features_per_group, nA - first_feature);
    constexpr int THREADS = FEATURE_WAVES * WAVE;
    constexpr int FEATURE_ROWS = feature_rows(RPL);
    constexpr int FEATURE_ROW_PITCH = feature_row_pitch(RPL);
    constexpr int OTHERS = ORDER - 1;

    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int32_t row0 = blockIdx.x * FEATURE_ROWS;
    const int32_t rows = min(FEATURE_ROWS, n_rows - row0);

    const T* a_src = A + static_cast<size_t>(row0) * nA;
    constexpr int STAGE_LOADS = 4;
    for (int32_t i0 = tid; i0 < FEATURE_ROWS * nA; i0 += STAGE_LOADS * THREADS) {
        T value[STAGE_LOADS];
#pragma unroll
        for (int u = 0; u < STAGE_LOADS; u++) {
            const int32_t i = i0 + u * THREADS;
            value[u] = load_or_zero(a_src, static_cast<size_t>(i), i < rows * nA); // rows beyond the end: zeros
        }
#pragma unroll
        for (int u = 0; u < STAGE_LOADS; u++) {
            const int32_t i = i0 + u * THREADS;
            if (i < FEATURE_ROWS * nA) {
                const int32_t row = i / nA;
                a_stage[(i - row * nA) * FEATURE_ROW_PITCH + row] = value[u];
            }
        }
    }
    T upstream[RPL];
#pragma unroll
    for (int r = 0; r < RPL; r++) {
        upstream[r] = load_or_zero(grad_output, static_cast<size_t>(row0 + lane + r * WAVE), lane + r * WAVE < rows);
    }
    __syncthreads();

    const T* mine = a_stage + lane;
    for (int32_t local = wave; local < n_features; local += FEATURE_WAVES) {
        const int32_t feature = first_feature + local;
        const int32_t begin = list_begin[feature];
        const int32_t end = list_begin[feature + 1];
        T sum[RPL];
#pragma unroll
        for (int r = 0; r < RPL; r++) {
            sum[r] = T(0);
        }
        for (int32_t p0 = begin; p0 < end; p0 += WAVE) {
            const int32_t n = min(WAVE, end - p0);
            // my entry of the batch: coefficient (zero: no entry, or a factor out of range) and
            // where the other factors' values are in the tile
            const int32_t q = lane < n ? list[p0 + lane] : 0;
            const int32_t j = q / ORDER;
            const int32_t f = q - j * ORDER;
            T coefficient = lane < n ? C[j] : T(0);
            int32_t other[OTHERS > 0 ? OTHERS : 1];
#pragma unroll
            for (int k = 0; k < OTHERS; k++) {
                const int32_t factor = P[static_cast<size_t>(j) * ORDER + (k < f ? k : k + 1)];
                const bool valid = in_bounds(factor, nA);
                other[k] = (valid ? factor : 0) * FEATURE_ROW_PITCH;
                coefficient = valid ? coefficient : T(0);
            }
            int32_t words[sizeof(T) / 4];
            __builtin_memcpy(words, &coefficient, sizeof(T));
            // BATCH entries at a time: first every LDS read, then the products (a read that
            // is waited for before the next one is asked for costs its whole latency)
            constexpr int BATCH = 8;
            for (int32_t u0 = 0; u0 < n; u0 += BATCH) {
                T term[BATCH];
                T value[BATCH][OTHERS > 0 ? OTHERS : 1][RPL];
#pragma unroll
                for (int b = 0; b < BATCH; b++) {
                    // entries beyond n: lanes beyond n hold coefficient zero and a place that exists
                    const int32_t u = min(u0 + b, WAVE - 1);
                    int32_t uniform[sizeof(T) / 4];
#pragma unroll
                    for (int w = 0; w < static_cast<int>(sizeof(T) / 4); w++) {
                        uniform[w] = __builtin_amdgcn_readlane(words[w], u);
                    }
                    __builtin_memcpy(&term[b], uniform, sizeof(T));
                    if (u0 + b >= WAVE) {
                        term[b] = T(0);
                    }
#pragma unroll
                    for (int k = 0; k < OTHERS; k++) {
                        const T* at = mine + __builtin_amdgcn_readlane(other[k], u);
#pragma unroll
                        for (int r = 0; r < RPL; r++) {
                            value[b][k][r] = at[r * WAVE];
                        }
                    }
                }
#pragma unroll
                for (int b = 0; b < BATCH; b++) {
#pragma unroll
                    for (int r = 0; r < RPL; r++) {
                        T product = term[b];
#pragma unroll
                        for (int k = 0; k < OTHERS; k++) {
                            product *= value[b][k][r];
                        }
                        sum[r] += product;
                    }
                }
            }
        }
#pragma unroll
        for (int r = 0; r < RPL; r++) {
            out[(lane + r * WAVE) * out_pitch + local] = upstream[r] * sum[r];
        }
    }
    __syncthreads();
    // row by row, this group's features next to each other (all of them: one contiguous piece)
    T* target = grad_A + static_cast<size_t>(row0) * nA + first_feature;
    for (int32_t i = tid; i < rows * n_features; i += THREADS) {
        const int32_t row = i / n_features;
        const int32_t local = i - row * n_features;
        target[static_cast<size_t>(row) * nA + local] = out[row * out_pitch + local];
    }
}

// ---------------------------------------------------------------------------
// forward for MANY rows, the same way: a lane is RPL rows, all lanes of a
// wavefront are at the same monomial. The wavefronts of a workgroup share the
// rows and take contiguous shares of the monomials, 64 at a time (lane u
// loads monomial u of the batch, readlane hands it out); their partial sums
// meet in LDS in wave order.
// LDS: a[nA][pitch] partial[FEATURE_WAVES][rows]
// ---------------------------------------------------------------------------
template <typename T, int ORDER, int RPL>
__global__ __launch_bounds__(FEATURE_WAVES* WAVE) void forward_rows_kernel(
    T* __restrict__ output,
    const T* __restrict__ A,
    const T* __restrict__ C,
    const int32_t* __restrict__ P,
    int32_t n_rows,
    int32_t nA,
    int32_t n_monomials
) {
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    constexpr int THREADS = FEATURE_WAVES * WAVE;
    constexpr int ROWS = feature_rows(RPL);
    constexpr int PITCH = feature_row_pitch(RPL);
    T* a_stage = reinterpret_cast<T*>(lds_bytes);
    T* partial = a_stage + static_cast<size_t>(nA) * PITCH;

    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int32_t row0 = blockIdx.x * ROWS;
    const int32_t rows = min(ROWS, n_rows - row0);

    const T* a_src = A + static_cast<size_t>(row0) * nA;
    constexpr int STAGE_LOADS = 4;
    for (int32_t i0 = tid; i0 < ROWS * nA; i0 += STAGE_LOADS * THREADS) {
        T value[STAGE_LOADS];
#pragma unroll
        for (int u = 0; u < STAGE_LOADS; u++) {
            const int32_t i = i0 + u * THREADS;
            value[u] = load_or_zero(a_src, static_cast<size_t>(i), i < rows * nA); // rows beyond the end: zeros
        }
#pragma unroll
        for (int u = 0; u < STAGE_LOADS; u++) {
            const int32_t i = i0 + u * THREADS;
            if (i < ROWS * nA) {
                const int32_t row = i / nA;
                a_stage[(i - row * nA) * PITCH + row] = value[u];
            }
        }
    }
    __syncthreads();

    const int32_t per_wave = (n_monomials + FEATURE_WAVES - 1) / FEATURE_WAVES;
    const int32_t begin = min(wave * per_wave, n_monomials);
    const int32_t end = min(begin + per_wave, n_monomials);
    const T* mine = a_stage + lane;
    T sum[RPL];
#pragma unroll
    for (int r = 0; r < RPL; r++) {
        sum[r] = T(0);
    }
    for (int32_t j0 = begin; j0 < end; j0 += WAVE) {
        const int32_t n = min(WAVE, end - j0);
        // my monomial of the batch: coefficient (zero: none, or a factor out of range) and where
        // its factors' values are in the tile
        const int32_t j = lane < n ? j0 + lane : 0;
        T coefficient = lane < n ? C[j] : T(0);
        int32_t place[ORDER];
#pragma unroll
        for (int k = 0; k < ORDER; k++) {
            const int32_t factor = P[static_cast<size_t>(j) * ORDER + k];
            const bool valid = in_bounds(factor, nA);
            place[k] = (valid ? factor : 0) * PITCH;
            coefficient = valid ? coefficient : T(0);
        }
        int32_t words[sizeof(T) / 4];
        __builtin_memcpy(words, &coefficient, sizeof(T));
        constexpr int BATCH = 8;
        for (int32_t u0 = 0; u0 < n; u0 += BATCH) {
            T term[BATCH];
            T value[BATCH][ORDER][RPL];
#pragma unroll
            for (int b = 0; b < BATCH; b++) {
                const int32_t u = min(u0 + b, WAVE - 1);
                int32_t uniform[sizeof(T) / 4];
#pragma unroll
                for (int w = 0; w < static_cast<int>(sizeof(T) / 4); w++) {
                    uniform[w] = __builtin_amdgcn_readlane(words[w], u);
                }
                __builtin_memcpy(&term[b], uniform, sizeof(T));
                if (u0 + b >= WAVE) {
                    term[b] = T(0);
                }
#pragma unroll
                for (int k = 0; k < ORDER; k++) {
                    const T* at = mine + __builtin_amdgcn_readlane(place[k], u);
#pragma unroll
                    for (int r = 0; r < RPL; r++) {
                        value[b][k][r] = at[r * WAVE];
                    }
                }
            }
#pragma unroll
            for (int b = 0; b < BATCH; b++) {
#pragma unroll
                for (int r = 0; r < RPL; r++) {
                    T product = term[b];
#pragma unroll
                    for (int k = 0; k < ORDER; k++) {
                        product *= value[b][k][r];
                    }
                    sum[r] += product;
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < RPL; r++) {
        partial[wave * ROWS + lane + r * WAVE] = sum[r];
    }
    __syncthreads();
    if (tid < rows) {
        T total = T(0);
        for (int w = 0; w < FEATURE_WAVES; w++) {
            total += partial[w * ROWS + tid];
        }
        output[row0 + tid] = total;
    }
}

// ---------------------------------------------------------------------------
// Fallbacks for feature counts whose tiles do not fit in LDS: one thread per
// batch row, everything in global memory.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void forward_global_kernel(
    T* __restrict__ output,
    const T* __restrict__ A,
    const T* __restrict__ C,
    const int32_t* __restrict__ P,
    int32_t n_rows,
    int32_t nA,
    int32_t n_monomials,
    int32_t order
) {
    const int32_t row = blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= n_rows) {
        return;
    }
    const T* a_row = A + static_cast<size_t>(row) * nA;
    T sum = T(0);
    for (int32_t j = 0; j < n_monomials; j++) {
        const int32_t* factors = P + static_cast<size_t>(j) * order;
        T product = C[j];
        for (int32_t k = 0; k < order; k++) {
            int32_t feature = factors[k];
            product *= in_bounds(feature, nA) ? a_row[feature] : T(0);
        }
        sum += product;
    }
    output[row] = sum;
}

template <typename T>
__global__ __launch_bounds__(256) void vjp_global_kernel(
    T* grad_A,
    const T* __restrict__ grad_output,
    const T* __restrict__ A,
    const T* __restrict__ C,
    const int32_t* __restrict__ P,
    int32_t n_rows,
    int32_t nA,
    int32_t n_monomials,
    int32_t order
) {
    const int32_t row = blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= n_rows) {
        return;
    }
    const T* a_row = A + static_cast<size_t>(row) * nA;
    T* g_row = grad_A + static_cast<size_t>(row) * nA;
    for (int32_t feature = 0; feature < nA; feature++) {
        g_row[feature] = T(0);
    }
    const T upstream = grad_output[row];
    for (int32_t j = 0; j < n_monomials; j++) {
        const int32_t* factors = P + static_cast<size_t>(j) * order;
        const T base = C[j] * upstream;
        for (int32_t f = 0; f < order; f++) {
            int32_t target = factors[f];
            if (!in_bounds(target, nA)) {
                continue;
            }
            T term = base;
            for (int32_t k = 0; k < order; k++) {
                if (k == f) {
                    continue;
                }
                int32_t feature = factors[k];
                term *= in_bounds(feature, nA) ? a_row[feature] : T(0);
            }
            g_row[target] += term;
        }
    }
}

// ---------------------------------------------------------------------------
// Second order: the vjp of the vjp (semantics of mops/src/hpe/cpu.tpp:275-539).
//
//   grad_grad_O[i]      = sum_j C[j] sum_f gg[i, P[j, f]] prod_{k != f} A[i, P[j, k]]
//   grad_A_2[i, P[j,f2]] += gO[i] C[j] sum_{f != f2} gg[i, P[j, f]] prod_{k != f, f2} A[i, P[j, k]]
//
// with gg = grad_grad_A. Same work split as vjp_kernel: one wavefront per
// workgroup, thread (r, g) walks the monomials j = g, g + G, ... of row r and
// adds into private accumulators in LDS, which are then combined in group
// order. LDS: a[nA][R] gg[nA][R] accumulator[G][nA][R] partial[G][R].
// Either output may be null.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(WAVE) void vjp_vjp_kernel(
    T* __restrict__ grad_grad_output,
    T* __restrict__ grad_A_2,
    const T* __restrict__ grad_grad_A,
    const T* __restrict__ grad_output,
    const T* __restrict__ A,
    const T* __restrict__ C,
    const int32_t* __restrict__ P,
    int32_t n_rows,
    int32_t nA,
    int32_t n_monomials,
    int32_t order,
    int32_t R
) {
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    T* a_stage = reinterpret_cast<T*>(lds_bytes);
    T* gg_stage = a_stage + static_cast<size_t>(nA) * R;
    T* accumulator = gg_stage + static_cast<size_t>(nA) * R;
    T* partial = accumulator + static_cast<size_t>(nA) * WAVE;

    const int tid = threadIdx.x;
    const int G = WAVE / R;
    const int r = tid % R;
    const int g = tid / R;
    const int32_t row0 = blockIdx.x * R;
    const int32_t rows = min(R, n_rows - row0);
    const bool want_O = grad_grad_output != nullptr;
    const bool want_A = grad_A_2 != nullptr;

    const T* a_src = A + static_cast<size_t>(row0) * nA;
    const T* gg_src = grad_grad_A + static_cast<size_t>(row0) * nA;
    for (int32_t i = tid; i < rows * nA; i += WAVE) {
        const int32_t row = i / nA;
        a_stage[(i - row * nA) * R + row] = a_src[i];
        gg_stage[(i - row * nA) * R + row] = gg_src[i];
    }
    for (int32_t i = tid; i < nA * WAVE; i += WAVE) {
        accumulator[i] = T(0);
    }
    __syncthreads();

    T sum = T(0);
    if (r < rows) {
        T* mine = accumulator + static_cast<size_t>(g) * nA * R + r;
        const T upstream = grad_output[row0 + r];
        auto value_of = [&](const T* stage, int32_t feature) {
            return in_bounds(feature, nA) ? stage[feature * R + r] : T(0);
        };
        for (int32_t j = g; j < n_monomials; j += G) {
            const int32_t* factors = P + static_cast<size_t>(j) * order;
            const T coefficient = C[j];
            if (want_O) {
                for (int32_t f = 0; f < order; f++) {
                    T term = coefficient * value_of(gg_stage, factors[f]);
                    for (int32_t k = 0; k < order; k++) {
                        if (k != f) {
                            term *= value_of(a_stage, factors[k]);
                        }
                    }
                    sum += term;
                }
            }
            if (want_A) {
                const T base = coefficient * upstream;
                for (int32_t f2 = 0; f2 < order; f2++) {
                    const int32_t target = factors[f2];
                    if (!in_bounds(target, nA)) {
                        continue;
                    }
                    T total = T(0);
                    for (int32_t f = 0; f < order; f++) {
                        if (f == f2) {
                            continue;
                        }
                        T term = base * value_of(gg_stage, factors[f]);
                        for (int32_t k = 0; k < order; k++) {
                            if (k != f && k != f2) {
                                term *= value_of(a_stage, factors[k]);
                            }
                        }
                        total += term;
                    }
                    mine[target * R] += total;
                }
            }
        }
    }
    partial[g * R + r] = sum;
    __syncthreads();

    if (want_O && tid < rows) {
        T total = T(0);
        for (int group = 0; group < G; group++) {
            total += partial[group * R + tid];
        }
        grad_grad_output[row0 + tid] = total;
    }
    if (want_A) {
        T* dst = grad_A_2 + static_cast<size_t>(row0) * nA;
        for (int32_t i = tid; i < rows * nA; i += WAVE) {
            const int32_t row = i / nA;
            const int32_t feature = i - row * nA;
            T total = T(0);
            for (int group = 0; group < G; group++) {
                total += accumulator[(static_cast<size_t>(group) * nA + feature) * R + row];
            }
            dst[i] = total;
        }
    }
}

// ---------------------------------------------------------------------------
// Second order with the order known at compile time. Layout and division of
// labour of vjp_ordered_kernel (the first wavefront walks the monomials, the
// others help to stage, clear and add up), with a tile of grad_grad_A beside
// the tile of A. A monomial costs O(K) instead of O(K^3): with a = A[i, P[j, .]]
// and g = grad_grad_A[i, P[j, .]], the sums above are the derivative of the
// product of the a's along g and that derivative's gradient,
//
//   S      = sum_f g[f] prod_{k != f} a[k]              (into grad_grad_output)
//   D[f2]  = sum_{f != f2} g[f] prod_{k != f, f2} a[k]   (into grad_A_2, times gO)
//
// and both come from products of the factors before and after a position that
// carry their own derivative along g:  p' = p a,  dp' = dp a + p g.
// Then D[f2] = dp[f2] s[f2] + p[f2] ds[f2] and S = dp[K].
// LDS: a[nA + 1][R] gg[nA + 1][R] accumulator[G][nA + 1][R]
// ---------------------------------------------------------------------------
template <typename T, int ORDER>
__global__ __launch_bounds__(ORDERED_VJP_THREADS) void vjp_vjp_ordered_kernel(
    T* __restrict__ grad_grad_output,
    T* __restrict__ grad_A_2,
    const T* __restrict__ grad_grad_A,
    const T* __restrict__ grad_output,
    const T* __restrict__ A,
    const T* __restrict__ C,
    const int32_t* __restrict__ P,
    int32_t n_rows,
    int32_t nA,
    int32_t n_monomials,
    int32_t log2_R
) {
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    const int32_t R = 1 << log2_R;
    T* a_stage = reinterpret_cast<T*>(lds_bytes);
    T* gg_stage = a_stage + static_cast<size_t>(nA + 1) * R;
    T* accumulator = gg_stage + static_cast<size_t>(nA + 1) * R;
    const bool want_O = grad_grad_output != nullptr;
    const bool want_A = grad_A_2 != nullptr;

    const int tid = threadIdx.x;
    const bool walks = tid < WAVE;
    const int G = WAVE >> log2_R;
    const int r = tid & (R - 1);
    const int g = (tid & (WAVE - 1)) >> log2_R;
    const int32_t row0 = blockIdx.x * R;
    const int32_t rows = min(R, n_rows - row0);

    struct Monomial {
        int32_t factor[ORDER];
        T coefficient;
    };
    auto fetch = [&](Monomial& to, int32_t j) {
        const int32_t safe = min(j, n_monomials - 1);
        const int32_t* factors = P + static_cast<size_t>(safe) * ORDER;
#pragma unroll
        for (int k = 0; k < ORDER; k++) {
            to.factor[k] = factors[k];
        }
        to.coefficient = C[safe];
    };
    constexpr int BATCH = 4;
    Monomial queue[BATCH];
    T upstream = T(0);
    if (walks) {
#pragma unroll
        for (int d = 0; d < BATCH; d++) {
            fetch(queue[d], g + d * G);
        }
        upstream = grad_output[min(row0 + r, n_rows - 1)];
    }

    // the rows of A and of grad_grad_A, STAGE values of each per lane asked for together
    const T* a_src = A + static_cast<size_t>(row0) * nA;
    const T* gg_src = grad_grad_A + static_cast<size_t>(row0) * nA;
    constexpr int STAGE = 4;
    for (int32_t base = 0; base < rows * nA; base += STAGE * ORDERED_VJP_THREADS) {
        T staged[2][STAGE];
#pragma unroll
        for (int u = 0; u < STAGE; u++) {
            const int32_t i = min(base + u * ORDERED_VJP_THREADS + tid, rows * nA - 1);
            staged[0][u] = a_src[i];
            staged[1][u] = gg_src[i];
        }
#pragma unroll
        for (int u = 0; u < STAGE; u++) {
            const int32_t i = base + u * ORDERED_VJP_THREADS + tid;
            if (i < rows * nA) {
                const int32_t row = i / nA;
                const int32_t at = ((i - row * nA) << log2_R) + row;
                a_stage[at] = staged[0][u];
                gg_stage[at] = staged[1][u];
            }
        }
    }
    if (tid < R) {
        a_stage[nA * R + tid] = T(0);
        gg_stage[nA * R + tid] = T(0);
    }
    if (want_A) {
        constexpr int HELPERS = ORDERED_VJP_THREADS / WAVE;
        T* clear = accumulator + (tid & (WAVE - 1));
        int32_t k = tid >> 6;
        for (; k + 7 * HELPERS < nA + 1; k += 8 * HELPERS) {
#pragma unroll
            for (int u = 0; u < 8; u++) {
                clear[(k + u * HELPERS) * WAVE] = T(0);
            }
        }
        for (; k < nA + 1; k += HELPERS) {
            clear[k * WAVE] = T(0);
        }
    }
    __syncthreads();

    T sum = T(0);
    if (walks && r < rows) {
        T* mine = accumulator + static_cast<size_t>(g) * (nA + 1) * R + r;
        const int32_t byte_shift = log2_R + (sizeof(T) == 8 ? 3 : 2);
        auto at = [&](auto* base, uint32_t feature) {
            using Pointer = decltype(base);
            using Bytes = std::conditional_t<std::is_const_v<std::remove_pointer_t<Pointer>>, const char*, char*>;
            return reinterpret_cast<Pointer>(reinterpret_cast<Bytes>(base) + (feature << byte_shift));
        };
        const T* my_a = a_stage + r;
        const T* my_gg = gg_stage + r;
        const uint32_t features = static_cast<uint32_t>(nA);
        auto batch = [&](int32_t j0, auto whole) {
            constexpr bool WHOLE = decltype(whole)::value;
            Monomial now[BATCH];
            T a[BATCH][ORDER];
            T gg[BATCH][ORDER];
#pragma unroll
            for (int d = 0; d < BATCH; d++) {
                now[d] = queue[d];
#pragma unroll
                for (int k = 0; k < ORDER; k++) {
                    // (as unsigned, a negative factor is a large one)
                    const uint32_t feature = min(static_cast<uint32_t>(now[d].factor[k]), features);
                    a[d][k] = *at(my_a, feature);
                    gg[d][k] = *at(my_gg, feature);
                }
            }
            if constexpr (WHOLE) {
#pragma unroll
                for (int d = 0; d < BATCH; d++) {
                    fetch(queue[d], j0 + (d + BATCH) * G);
                }
            }
            T term[BATCH][ORDER];
#pragma unroll
            for (int d = 0; d < BATCH; d++) {
                const bool exists = WHOLE || j0 + d * G < n_monomials;
                // products of the factors before a position, and their derivative along gg
                T before[ORDER + 1];
                T d_before[ORDER + 1];
                before[0] = exists ? now[d].coefficient : T(0);
                d_before[0] = T(0);
#pragma unroll
                for (int k = 0; k < ORDER; k++) {
                    before[k + 1] = before[k] * a[d][k];
                    d_before[k + 1] = d_before[k] * a[d][k] + before[k] * gg[d][k];
                }
                sum += d_before[ORDER];
                // the same from the other end, and the two put together
                T after = T(1);
                T d_after = T(0);
#pragma unroll
                for (int f = ORDER - 1; f >= 0; f--) {
                    term[d][f] = upstream * (d_before[f] * after + before[f] * d_after);
                    d_after = d_after * a[d][f] + after * gg[d][f];
                    after *= a[d][f];
                }
            }
            if (want_A) {
#pragma unroll
                for (int d = 0; d < BATCH; d++) {
#pragma unroll
                    for (int f = ORDER - 1; f >= 0; f--) {
                        // (a factor outside [0, nA) and a monomial beyond the last, whose terms
                        // are zero, go to the row that is never read)
                        T* to = at(mine, min(static_cast<uint32_t>(now[d].factor[f]), features));
                        if constexpr (sizeof(T) == 8) {
                            unsafeAtomicAdd(to, term[d][f]);
                        } else {
                            *to += term[d][f];
                        }
                    }
                }
            }
        };
        int32_t j0 = g;
        for (; j0 + (BATCH - 1) * G < n_monomials; j0 += BATCH * G) {
            batch(j0, std::true_type{});
        }
        if (j0 < n_monomials) {
            batch(j0, std::false_type{});
        }
    }
    // grad_grad_output: the lanes of the first wavefront that share a row, by a fixed tree
    if (walks && want_O) {
        for (int offset = WAVE / 2; offset >= R; offset >>= 1) {
            sum += __shfl_xor(sum, offset);
        }
        if (tid < rows) {
            grad_grad_output[row0 + tid] = sum;
        }
    }
    __syncthreads();

    if (want_A) {
        T* dst = grad_A_2 + static_cast<size_t>(row0) * nA;
        const int32_t copy_stride = (nA + 1) * R;
        for (int32_t entry = tid; entry < nA * R; entry += ORDERED_VJP_THREADS) {
            const int32_t row = entry & (R - 1);
            const int32_t feature = entry >> log2_R;
            const T* from = accumulator + entry;
            T partial[4] = {T(0), T(0), T(0), T(0)};
            int group = 0;
            for (; group + 4 <= G; group += 4) {
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    partial[u] += from[(group + u) * copy_stride];
                }
            }
            for (; group < G; group++) {
                partial[group & 3] += from[group * copy_stride];
            }
            if (row < rows) {
                dst[static_cast<size_t>(row) * nA + feature] = (partial[0] + partial[1]) + (partial[2] + partial[3]);
            }
        }
    }
}

// The same with everything in global memory, one thread per batch row, for
// feature counts whose tiles do not fit in LDS.
template <typename T>
__global__ __launch_bounds__(256) void vjp_vjp_global_kernel(
    T* grad_grad_output,
    T* grad_A_2,
    const T* __restrict__ grad_grad_A,
    const T* __restrict__ grad_output,
    const T* __restrict__ A,
    const T* __restrict__ C,
    const int32_t* __restrict__ P,
    int32_t n_rows,
    int32_t nA,
    int32_t n_monomials,
    int32_t order
) {
    const int32_t row = blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= n_rows) {
        return;
    }
    const T* a_row = A + static_cast<size_t>(row) * nA;
    const T* gg_row = grad_grad_A + static_cast<size_t>(row) * nA;
    T* out_row = grad_A_2 != nullptr ? grad_A_2 + static_cast<size_t>(row) * nA : nullptr;
    if (out_row != nullptr) {
        for (int32_t feature = 0; feature < nA; feature++) {
            out_row[feature] = T(0);
        }
    }
    auto value_of = [&](const T* values, int32_t feature) {
        return in_bounds(feature, nA) ? values[feature] : T(0);
    };
    const T upstream = grad_output[row];
    T sum = T(0);
    for (int32_t j = 0; j < n_monomials; j++) {
        const int32_t* factors = P + static_cast<size_t>(j) * order;
        for (int32_t f2 = 0; f2 < order; f2++) {
            // f2 = the factor differentiated last; the f2-th term of the first
            // sum is the product with gg in place of that factor
            T first = C[j] * value_of(gg_row, factors[f2]);
            T second = T(0);
            for (int32_t k = 0; k < order; k++) {
                if (k != f2) {
                    first *= value_of(a_row, factors[k]);
                }
            }
            sum += first;
            if (out_row != nullptr && in_bounds(factors[f2], nA)) {
                for (int32_t f = 0; f < order; f++) {
                    if (f == f2) {
                        continue;
                    }
                    T term = C[j] * upstream * value_of(gg_row, factors[f]);
                    for (int32_t k = 0; k < order; k++) {
                        if (k != f && k != f2) {
                            term *= value_of(a_row, factors[k]);
                        }
                    }
                    second += term;
                }
                out_row[factors[f2]] += second;
            }
        }
    }
    if (grad_grad_output != nullptr) {
        grad_grad_output[row] = sum;
    }
}

// Rows per workgroup: as many as possible (fewer table reads per row) while
// the launch still has about a thousand workgroups and the tiles fit in LDS.
// Returns 0 when even R = 1 does not fit.
int pick_rows(size_t n_rows, size_t bytes_per_row) {
    int R = 64;
    while (R > 1 && (n_rows / R < 1024 || bytes_per_row * R > LDS_BUDGET)) {
        R >>= 1;
    }
    return bytes_per_row * R > LDS_BUDGET ? 0 : R;
}

} // namespace
} // namespace hpe
using namespace hpe;
} // namespace mops::amd

namespace mops::cuda {

template <typename scalar_t>
void homogeneous_polynomial_evaluation(MOPS_HPE_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using namespace mops::amd;
    const char* operation = "cuda_homogeneous_polynomial_evaluation";
    checks::Validator validator(operation);
    checks::hpe(validator, output, A, C, indices_A);
    validate_gather_index(indices_A, A.shape[1], "indices_A", operation);

    const int32_t n_rows = narrow_i32(A.shape[0], "A.shape[0]");
    const int32_t nA = narrow_i32(A.shape[1], "A.shape[1]");
    const int32_t n_monomials = narrow_i32(indices_A.shape[0], "indices_A.shape[0]");
    const int32_t order = narrow_i32(indices_A.shape[1], "indices_A.shape[1]");
    if (n_rows == 0) {
        return;
    }
    hipStream_t stream = current_stream();
    constexpr int THREADS = 256;
    // many rows: a lane per row (forward_rows_kernel), two where the tile of 128 rows fits
    auto rows_bytes = [&](int rpl) {
        return (static_cast<size_t>(nA) * feature_row_pitch(rpl) + static_cast<size_t>(FEATURE_WAVES) * feature_rows(rpl)) *
               sizeof(scalar_t);
    };
    // (a workgroup per 64 or 128 rows: fewer workgroups than about one per compute unit leave the
    // kernel below ahead, 8192 rows: 24 us against 35)
    if (n_rows >= FORWARD_MANY_ROWS && order >= 1 && order <= 6 && n_monomials > 0 &&
        rows_bytes(1) <= BY_FEATURE_LDS_BUDGET) {
        // (two rows per lane also where that halves the workgroups: 20 000 rows, 51 us against 65)
        const int rows_per_lane = rows_bytes(2) <= BY_FEATURE_LDS_BUDGET ? 2 : 1;
        const size_t lds = rows_bytes(rows_per_lane);
        const unsigned blocks =
            static_cast<unsigned>(ceil_div(static_cast<size_t>(n_rows), static_cast<size_t>(feature_rows(rows_per_lane))));
#define MOPS_LAUNCH_ROWS(ORDER)                                                                     \
    {                                                                                              \
        auto kernel = rows_per_lane == 2 ? forward_rows_kernel<scalar_t, ORDER, 2>                 \
                                         : forward_rows_kernel<scalar_t, ORDER, 1>;                \
        if (lds > 64 * 1024) {                                                                     \
            MOPS_HIP_CHECK(hipFuncSetAttribute(                                                    \
                reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, \
                static_cast<int>(lds)                                                              \
            ));                                                                                    \
        }                                                                                          \
        kernel<<<blocks, FEATURE_WAVES * WAVE, lds, stream>>>(                                     \
            output.data, A.data, C.data, indices_A.data, n_rows, nA, n_monomials                   \
        );                                                                                         \
    }
        switch (order) {
        case 1:
            MOPS_LAUNCH_ROWS(1);
            break;
        case 2:
            MOPS_LAUNCH_ROWS(2);
            break;
        case 3:
            MOPS_LAUNCH_ROWS(3);
            break;
        case 4:
            MOPS_LAUNCH_ROWS(4);
            break;
        case 5:
            MOPS_LAUNCH_ROWS(5);
            break;
        default:
            MOPS_LAUNCH_ROWS(6);
            break;
        }
#undef MOPS_LAUNCH_ROWS
        finish_call(operation);
        return;
    }
    // per row: its A values plus one partial sum per group (G <= THREADS)
    int R = pick_rows(n_rows, (static_cast<size_t>(nA) + 1 + THREADS) * sizeof(scalar_t));
    if (R > 0) {
        size_t lds = ((static_cast<size_t>(nA) + 1) * R + THREADS) * sizeof(scalar_t);
        unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<size_t>(n_rows), R));
        MainKernelTimer timer(stream);
#define MOPS_LAUNCH_ORDERED(ORDER)                                                                  \
    forward_ordered_kernel<scalar_t, ORDER><<<blocks, THREADS, lds, stream>>>(                     \
        output.data, A.data, C.data, indices_A.data, n_rows, nA, n_monomials, R                    \
    )
        switch (order) {
        case 0:
            MOPS_LAUNCH_ORDERED(0);
            break;
        case 1:
            MOPS_LAUNCH_ORDERED(1);
            break;
        case 2:
            MOPS_LAUNCH_ORDERED(2);
            break;
        case 3:
            MOPS_LAUNCH_ORDERED(3);
            break;
        case 4:
            MOPS_LAUNCH_ORDERED(4);
            break;
        case 5:
            MOPS_LAUNCH_ORDERED(5);
            break;
        case 6:
            MOPS_LAUNCH_ORDERED(6);
            break;
        default:
            forward_kernel<scalar_t><<<blocks, THREADS, lds, stream>>>(
                output.data, A.data, C.data, indices_A.data, n_rows, nA, n_monomials, order, R
            );
            break;
        }
#undef MOPS_LAUNCH_ORDERED
    } else {
        unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<size_t>(n_rows), THREADS));
        forward_global_kernel<scalar_t><<<blocks, THREADS, 0, stream>>>(
            output.data, A.data, C.data, indices_A.data, n_rows, nA, n_monomials, order
        );
    }
    finish_call(operation);
}

template <typename scalar_t>
void homogeneous_polynomial_evaluation_vjp(MOPS_HPE_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using namespace mops::amd;
    const char* operation = "cuda_homogeneous_polynomial_evaluation_vjp";
    checks::Validator validator(operation);
    checks::hpe_vjp(validator, grad_A, grad_output, A, C, indices_A);
    if (grad_A.data == nullptr) {
        return;
    }
    validate_gather_index(indices_A, A.shape[1], "indices_A", operation);

    const int32_t n_rows = narrow_i32(A.shape[0], "A.shape[0]");
    const int32_t nA = narrow_i32(A.shape[1], "A.shape[1]");
    const int32_t n_monomials = narrow_i32(indices_A.shape[0], "indices_A.shape[0]");
    const int32_t order = narrow_i32(indices_A.shape[1], "indices_A.shape[1]");
    if (n_rows == 0 || nA == 0) {
        return;
    }
    hipStream_t stream = current_stream();
    // many rows: by feature (vjp_by_feature_kernel), after the table has been turned round
    // workgroup = (64 rows, a group of features): groups of 16 features (one per wavefront)
    // while that brings the launch to a few hundred workgroups, all features in one otherwise
    auto by_feature_bytes = [&](int rpl, int32_t pitch) {
        return (static_cast<size_t>(nA) * feature_row_pitch(rpl) + static_cast<size_t>(feature_rows(rpl)) * pitch) *
               sizeof(scalar_t);
    };
    // two rows per lane where the tiles of 128 rows fit
    const int rows_per_lane = by_feature_bytes(2, (FEATURE_WAVES * 4) | 1) <= BY_FEATURE_LDS_BUDGET ? 2 : 1;
    const size_t row_groups = ceil_div(static_cast<size_t>(n_rows), static_cast<size_t>(feature_rows(rows_per_lane)));
    const size_t wanted_groups = std::max<size_t>(1, ceil_div(512, row_groups));
    const size_t feature_groups = std::min(wanted_groups, ceil_div(static_cast<size_t>(nA), FEATURE_WAVES));
    const int32_t features_per_group = static_cast<int32_t>(
        ceil_div(ceil_div(static_cast<size_t>(nA), feature_groups), FEATURE_WAVES) * FEATURE_WAVES
    );
    const int32_t out_pitch = features_per_group | 1;
    const size_t by_feature_lds = by_feature_bytes(rows_per_lane, out_pitch);
    const size_t n_pairs = static_cast<size_t>(n_monomials) * static_cast<size_t>(std::max(order, 0));
    if (n_rows >= MANY_ROWS && order >= 1 && order <= 6 && n_pairs > 0 && n_pairs < (size_t(1) << 30) &&
        by_feature_lds <= BY_FEATURE_LDS_BUDGET) {
        void* workspace = scratch(edges_by_sender_bytes(nA, static_cast<int32_t>(n_pairs)));
        const EdgesBySender lists =
            order_edges_by_sender(indices_A.data, static_cast<int32_t>(n_pairs), nA, workspace, stream);
        const dim3 blocks(
            static_cast<unsigned>(row_groups),
            static_cast<unsigned>(ceil_div(static_cast<size_t>(nA), static_cast<size_t>(features_per_group)))
        );
#define MOPS_LAUNCH_BY_FEATURE(ORDER)                                                               \
    {                                                                                              \
        auto kernel = rows_per_lane == 2 ? vjp_by_feature_kernel<scalar_t, ORDER, 2>               \
                                         : vjp_by_feature_kernel<scalar_t, ORDER, 1>;              \
        if (by_feature_lds > 64 * 1024) {                                                          \
            MOPS_HIP_CHECK(hipFuncSetAttribute(                                                    \
                reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, \
                static_cast<int>(by_feature_lds)                                                   \
            ));                                                                                    \
        }                                                                                          \
        kernel<<<blocks, FEATURE_WAVES * WAVE, by_feature_lds, stream>>>(                          \
            grad_A.data, grad_output.data, A.data, C.data, indices_A.data, lists.offsets, lists.edge, \
            n_rows, nA, features_per_group, out_pitch                                              \
        );                                                                                         \
    }
        switch (order) {
        case 1:
            MOPS_LAUNCH_BY_FEATURE(1);
            break;
        case 2:
            MOPS_LAUNCH_BY_FEATURE(2);
            break;
        case 3:
            MOPS_LAUNCH_BY_FEATURE(3);
            break;
        case 4:
            MOPS_LAUNCH_BY_FEATURE(4);
            break;
        case 5:
            MOPS_LAUNCH_BY_FEATURE(5);
            break;
        default:
            MOPS_LAUNCH_BY_FEATURE(6);
            break;
        }
#undef MOPS_LAUNCH_BY_FEATURE
        finish_call(operation);
        return;
    }
    // LDS holds R rows of A and WAVE private accumulator rows, whatever R is
    const size_t accumulator_bytes = (static_cast<size_t>(nA) + 1) * WAVE * sizeof(scalar_t);
    // Rows per workgroup: the fewest for which all workgroups are on the
    // device at once (256 CUs, as many workgroups per CU as the 160 KB of LDS
    // hold): a second round of workgroups costs more than rows twice as long
    // (c0: 17.8 us with 1000 workgroups of one row, 12.0 us with 500 of two, 17.2 us
    // with 250 of four).
    int R = 0;
    for (int rows = 1; rows <= 64 && R == 0; rows <<= 1) {
        const size_t lds = accumulator_bytes + (static_cast<size_t>(nA) + 1) * rows * sizeof(scalar_t);
        if (lds > LDS_BUDGET) {
            break;
        }
        const size_t resident = 256 * std::max<size_t>(1, (160 * 1024) / lds);
        if (ceil_div(static_cast<size_t>(n_rows), rows) <= resident || rows == 64) {
            R = rows;
        }
    }
    if (R == 0 && accumulator_bytes + (static_cast<size_t>(nA) + 1) * sizeof(scalar_t) <= LDS_BUDGET) {
        // the tiles of 64 rows do not fit: as many rows as do
        R = 1;
        while (accumulator_bytes + (static_cast<size_t>(nA) + 1) * (2 * R) * sizeof(scalar_t) <= LDS_BUDGET && R < 64) {
            R <<= 1;
        }
    }
    int32_t span = nA; // features whose accumulators one workgroup keeps
    if (R == 0 && (static_cast<size_t>(nA) + 1) * sizeof(scalar_t) <= LDS_BUDGET / 2) {
        // the accumulators of all features do not fit: one row per workgroup,
        // the features in ranges that do
        R = 1;
        span = static_cast<int32_t>(
            (LDS_BUDGET - (static_cast<size_t>(nA) + 1) * sizeof(scalar_t)) / (WAVE * sizeof(scalar_t)) - 1
        );
    }
    if (R > 0) {
        // (one row more of each than there are features: see vjp_ordered_kernel)
        size_t lds = (static_cast<size_t>(span) + 1) * WAVE * sizeof(scalar_t) +
                     (static_cast<size_t>(nA) + 1) * R * sizeof(scalar_t);
        int32_t log2_R = 0;
        while ((1 << log2_R) < R) {
            log2_R++;
        }
        const dim3 blocks(
            static_cast<unsigned>(ceil_div(static_cast<size_t>(n_rows), R)),
            static_cast<unsigned>(ceil_div(static_cast<size_t>(nA), span))
        );
        MainKernelTimer timer(stream);
#define MOPS_LAUNCH_ORDERED(ORDER)                                                                  \
    if (span == nA) {                                                                              \
        vjp_ordered_kernel<scalar_t, ORDER, true><<<blocks, ORDERED_VJP_THREADS, lds, stream>>>(                  \
            grad_A.data, grad_output.data, A.data, C.data, indices_A.data, n_rows, nA,             \
            n_monomials, log2_R, span                                                              \
        );                                                                                         \
    } else {                                                                                       \
        vjp_ordered_kernel<scalar_t, ORDER, false><<<blocks, ORDERED_VJP_THREADS, lds, stream>>>(                 \
            grad_A.data, grad_output.data, A.data, C.data, indices_A.data, n_rows, nA,             \
            n_monomials, log2_R, span                                                              \
        );                                                                                         \
    }
        switch (n_monomials > 0 ? order : 0) {
        case 1:
            MOPS_LAUNCH_ORDERED(1);
            break;
        case 2:
            MOPS_LAUNCH_ORDERED(2);
            break;
        case 3:
            MOPS_LAUNCH_ORDERED(3);
            break;
        case 4:
            MOPS_LAUNCH_ORDERED(4);
            break;
        case 5:
            MOPS_LAUNCH_ORDERED(5);
            break;
        case 6:
            MOPS_LAUNCH_ORDERED(6);
            break;
        default:
            vjp_kernel<scalar_t><<<blocks, WAVE, lds, stream>>>(
                grad_A.data, grad_output.data, A.data, C.data, indices_A.data, n_rows, nA, n_monomials,
                order, R, span
            );
            break;
        }
#undef MOPS_LAUNCH_ORDERED
    } else {
        unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<size_t>(n_rows), 256));
        vjp_global_kernel<scalar_t><<<blocks, 256, 0, stream>>>(
            grad_A.data, grad_output.data, A.data, C.data, indices_A.data, n_rows, nA, n_monomials, order
        );
    }
    finish_call(operation);
}

// Second order. The reference has it on the host only
// (mops/src/hpe/cpu.tpp:275-539; device: "Not implemented",
// mops/src/hpe/hpe.cu:402-413) and reads through a null grad_grad_A
// (cpu.tpp:367-388); here a cotangent that is not given counts as zero.
template <typename scalar_t>
void homogeneous_polynomial_evaluation_vjp_vjp(MOPS_HPE_VJP_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using namespace mops::amd;
    const char* operation = "cuda_homogeneous_polynomial_evaluation_vjp_vjp";
    checks::Validator validator(operation);
    checks::hpe_vjp_vjp(validator, grad_grad_output, grad_A_2, grad_grad_A, grad_output, A, C, indices_A);
    if (grad_grad_output.data == nullptr && grad_A_2.data == nullptr) {
        return;
    }
    validate_gather_index(indices_A, A.shape[1], "indices_A", operation);

    const int32_t n_rows = narrow_i32(A.shape[0], "A.shape[0]");
    const int32_t nA = narrow_i32(A.shape[1], "A.shape[1]");
    const int32_t n_monomials = narrow_i32(indices_A.shape[0], "indices_A.shape[0]");
    const int32_t order = narrow_i32(indices_A.shape[1], "indices_A.shape[1]");
    if (n_rows == 0) {
        return;
    }
    hipStream_t stream = current_stream();
    if (grad_grad_A.data == nullptr || nA == 0) {
        if (grad_grad_output.data != nullptr) {
            fill_zero<scalar_t>(grad_grad_output.data, static_cast<size_t>(n_rows), stream);
        }
        if (grad_A_2.data != nullptr) {
            fill_zero<scalar_t>(grad_A_2.data, static_cast<size_t>(n_rows) * nA, stream);
        }
        finish_call(operation);
        return;
    }
    // order known at compile time: the tiles of vjp_ordered_kernel and one more of grad_grad_A;
    // rows per workgroup as there (the fewest for which all workgroups are on the device at once)
    if (order >= 1 && order <= 6 && n_monomials > 0) {
        const size_t accumulator_bytes = (static_cast<size_t>(nA) + 1) * WAVE * sizeof(scalar_t);
        auto ordered_lds = [&](int rows) {
            return accumulator_bytes + 2 * (static_cast<size_t>(nA) + 1) * rows * sizeof(scalar_t);
        };
        int log2_R = -1;
        for (int log2_rows = 0; log2_rows <= 6 && ordered_lds(1 << log2_rows) <= LDS_BUDGET; log2_rows++) {
            log2_R = log2_rows;
            const size_t resident = 256 * std::max<size_t>(1, (160 * 1024) / ordered_lds(1 << log2_rows));
            if (ceil_div(static_cast<size_t>(n_rows), size_t(1) << log2_rows) <= resident) {
                break;
            }
        }
        if (log2_R >= 0) {
            const unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<size_t>(n_rows), size_t(1) << log2_R));
            const size_t lds = ordered_lds(1 << log2_R);
#define MOPS_LAUNCH_ORDERED(ORDER)                                                                  \
    vjp_vjp_ordered_kernel<scalar_t, ORDER><<<blocks, ORDERED_VJP_THREADS, lds, stream>>>(         \
        grad_grad_output.data, grad_A_2.data, grad_grad_A.data, grad_output.data, A.data, C.data,  \
        indices_A.data, n_rows, nA, n_monomials, log2_R                                            \
    )
            switch (order) {
            case 1:
                MOPS_LAUNCH_ORDERED(1);
                break;
            case 2:
                MOPS_LAUNCH_ORDERED(2);
                break;
            case 3:
                MOPS_LAUNCH_ORDERED(3);
                break;
            case 4:
                MOPS_LAUNCH_ORDERED(4);
                break;
            case 5:
                MOPS_LAUNCH_ORDERED(5);
                break;
            default:
                MOPS_LAUNCH_ORDERED(6);
                break;
            }
#undef MOPS_LAUNCH_ORDERED
            finish_call(operation);
            return;
        }
    }
    // LDS: 2 R rows (A and grad_grad_A), WAVE accumulator rows, WAVE partial sums
    const size_t fixed_bytes = (static_cast<size_t>(nA) + 1) * WAVE * sizeof(scalar_t);
    auto lds_for = [&](int rows) { return fixed_bytes + 2 * static_cast<size_t>(nA) * rows * sizeof(scalar_t); };
    int R = 64;
    while (R > 1 && (static_cast<size_t>(n_rows) / R < 1024 || lds_for(R) > LDS_BUDGET)) {
        R >>= 1;
    }
    if (lds_for(R) <= LDS_BUDGET) {
        const unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<size_t>(n_rows), R));
        vjp_vjp_kernel<scalar_t><<<blocks, WAVE, lds_for(R), stream>>>(
            grad_grad_output.data, grad_A_2.data, grad_grad_A.data, grad_output.data, A.data, C.data,
            indices_A.data, n_rows, nA, n_monomials, order, R
        );
    } else {
        const unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<size_t>(n_rows), 256));
        vjp_vjp_global_kernel<scalar_t><<<blocks, 256, 0, stream>>>(
            grad_grad_output.data, grad_A_2.data, grad_grad_A.data, grad_output.data, A.data, C.data,
            indices_A.data, n_rows, nA, n_monomials, order
        );
    }
    finish_call(operation);
}

MOPS_CXX_INSTANTIATE(homogeneous_polynomial_evaluation, MOPS_HPE_PARAMS)
MOPS_CXX_INSTANTIATE(homogeneous_polynomial_evaluation_vjp, MOPS_HPE_VJP_PARAMS)
MOPS_CXX_INSTANTIATE(homogeneous_polynomial_evaluation_vjp_vjp, MOPS_HPE_VJP_VJP_PARAMS)

} // namespace mops::cuda
