// Sparse accumulation + scatter-add with weights (SASAW), forward and
// vector-Jacobian product, for gfx950.
//
//   O[PO1[e], PO2[n], :] += C[n] * A[e, PA[n]] * B[e, :] * W[PW1[e], PW2[n], :]
//
// (e runs over edges, n over the entries of a sparse coupling table; in an
// equivariant message-passing layer A holds spherical harmonics, B radial
// features, W the sender's node features and C Clebsch-Gordan coefficients.)
//
// Semantics restated from mops/src/sasaw/cpu.tpp:8-171 of lab-cosmo/mops.
// The reference loops over all table entries for every edge and every feature
// channel (N*L multiply-adds per edge, three of them per entry in the vjp).
// Here the table is first contracted with the edge's A row into a small dense
// matrix that does not depend on the feature channel,
//
//   T[e, m3, m2] = sum over entries n with (PO2[n], PW2[n]) == (m3, m2) of C[n] * A[e, PA[n]]
//
// after which every quantity is a small dense contraction:
//
//   O[i, m3, l]    = sum_{e in segment i} sum_m2 T[e, m3, m2] * B[e, l] * W[PW1[e], m2, l]
//   grad_B[e, l]   = sum_m3 G[i, m3, l] * sum_m2 T[e, m3, m2] * W[PW1[e], m2, l]
//   U[e, m3, m2]   = sum_l B[e, l] * G[i, m3, l] * W[PW1[e], m2, l]
//   grad_A[e, m1]  = sum over entries n with PA[n] == m1 of C[n] * U[e, PO2[n], PW2[n]]
//   grad_W[w,m2,l] = sum_{e: PW1[e] == w} B[e, l] * sum_m3 T[e, m3, m2] * G[PO1[e], m3, l]
//
// (G = grad_output, i = PO1[e]). This changes the order of the floating-point
// additions with respect to the reference, not the value being computed.
// The table is regrouped once per call by a small kernel (by (m3, m2) cell
// and by m1), in ascending entry order, so all sums have one fixed order.
//
// The receiver index PO1 is sorted: output rows and the grad_A / grad_B rows
// of their edges are owned by one workgroup per receiver (segments from
// first_occurrences). grad_W scatters by the unsorted sender index PW1: edges
// are regrouped by sender (sender_buckets.hpp) and one workgroup per sender
// gathers. No floating-point atomics anywhere.
//
// The reference has no device implementation of this operation
// (mops/src/sasaw/sasaw.cu:1, mops/src/sasaw/cuda.tpp:18).
//
// This file holds the entry points and the GENERAL kernels described above.
// Tables whose component indices have at most 16 values each (equivariant
// message passing) do not get here: the entry points hand them to the
// persistent matrix-core kernels of sasaw_segments.hip (per-node sums of
// rank-one updates; one launch for the forward pass, one for all three
// gradients) and, where those refuse (grad_W on graphs too dense for the
// senders' slots, byte offsets beyond 32 bits), to sasaw_mfma.hip.
#include <algorithm>
#include <optional>
#include <atomic>
#include <stdexcept>
#include <string>

#include "mops/sasaw.hpp"

#include "checks.hpp"
#include "device_common.hpp"
#include "first_occurrences.hpp"
#include "index_validation.hpp"
#include "no_alloc.hpp"
#include "edge_order.hpp"
#include "elementwise.hpp"
#include "runtime.hpp"
#include "sasaw_mfma.hpp"
#include "sasaw_segments.hpp"
#include "sender_buckets.hpp"

namespace mops::amd {
namespace sasaw { // a name of its own for this file's kernels: profilers print it
namespace {

constexpr int MAX_THREADS = 1024;
constexpr size_t STAGING_BYTES = 48 * 1024;

// The coupling table regrouped two ways. Entries keep ascending order inside
// every group; entries with an index outside its range are dropped.
template <typename T> struct CouplingPlan {
    // grouped by cell = m3 * n2 + m2
    const int32_t* cell_begin; // [n3 * n2 + 1]
    const T* cell_coefficient; // [N]
    const int32_t* cell_m1;    // [N]
    // grouped by m1
    const int32_t* m1_begin;   // [nA + 1]
    const T* m1_coefficient;   // [N]
    const int32_t* m1_cell;    // [N]
};

template <typename T> struct CouplingPlanBuffers {
    int32_t* cell_begin;
    T* cell_coefficient;
    int32_t* cell_m1;
    int32_t* m1_begin;
    T* m1_coefficient;
    int32_t* m1_cell;
};

template <typename T> size_t plan_bytes(int32_t N, int32_t n_cells, int32_t nA) {
    size_t entries = static_cast<size_t>(N);
    return align256((static_cast<size_t>(n_cells) + 1) * 4) + align256(entries * sizeof(T)) +
           align256(entries * 4) + align256((static_cast<size_t>(nA) + 1) * 4) +
           align256(entries * sizeof(T)) + align256(entries * 4);
}

template <typename T>
CouplingPlanBuffers<T> carve_plan(void* workspace, int32_t N, int32_t n_cells, int32_t nA) {
    char* base = static_cast<char*>(workspace);
    size_t entries = static_cast<size_t>(N);
    CouplingPlanBuffers<T> plan;
    plan.cell_begin = reinterpret_cast<int32_t*>(base);
    base += align256((static_cast<size_t>(n_cells) + 1) * 4);
    plan.cell_coefficient = reinterpret_cast<T*>(base);
    base += align256(entries * sizeof(T));
    plan.cell_m1 = reinterpret_cast<int32_t*>(base);
    base += align256(entries * 4);
    plan.m1_begin = reinterpret_cast<int32_t*>(base);
    base += align256((static_cast<size_t>(nA) + 1) * 4);
    plan.m1_coefficient = reinterpret_cast<T*>(base);
    base += align256(entries * sizeof(T));
    plan.m1_cell = reinterpret_cast<int32_t*>(base);
    return plan;
}

constexpr int PLAN_THREADS = 256;

// Exclusive prefix sum over `counts[0..n)` -> `begin[0..n]`, one workgroup.
__device__ void block_exclusive_scan(int32_t* begin, int32_t n, int32_t* tile, int32_t* carry) {
    const int tid = threadIdx.x;
    if (tid == 0) {
        *carry = 0;
    }
    __syncthreads();
    for (int32_t base = 0; base < n; base += PLAN_THREADS) {
        int32_t i = base + tid;
        int32_t value = i < n ? begin[i + 1] : 0; // counts are parked one slot up
        tile[tid] = value;
        __syncthreads();
        for (int distance = 1; distance < PLAN_THREADS; distance <<= 1) {
            int32_t add = tid >= distance ? tile[tid - distance] : 0;
            __syncthreads();
            tile[tid] += add;
            __syncthreads();
        }
        int32_t inclusive = *carry + tile[tid];
        __syncthreads();
        if (i < n) {
            begin[i + 1] = inclusive;
        }
        if (tid == PLAN_THREADS - 1) {
            *carry = inclusive;
        }
        __syncthreads();
    }
    if (tid == 0) {
        begin[0] = 0;
    }
    __syncthreads();
}

// One workgroup regroups the N table entries. Every group (a cell or an m1
// value) is handled by one thread that walks the whole table in order: first
// to count its members, then (after a prefix sum) to copy them. Work is
// N * (n_cells + nA) / 256 steps per thread, a few hundred for typical
// tables.
template <typename T>
__global__ __launch_bounds__(PLAN_THREADS) void plan_kernel(
    CouplingPlanBuffers<T> plan,
    const T* __restrict__ C,
    const int32_t* __restrict__ PA,
    const int32_t* __restrict__ PW2,
    const int32_t* __restrict__ PO2,
    int32_t N,
    int32_t nA,
    int32_t n2,
    int32_t n3
) {
    __shared__ int32_t tile[PLAN_THREADS];
    __shared__ int32_t carry;
    const int tid = threadIdx.x;
    const int32_t n_cells = n2 * n3;

    for (int32_t cell = tid; cell < n_cells; cell += PLAN_THREADS) {
        const int32_t m3 = cell / n2;
        const int32_t m2 = cell - m3 * n2;
        int32_t count = 0;
        for (int32_t n = 0; n < N; n++) {
            count += (PO2[n] == m3 && PW2[n] == m2 && in_bounds(PA[n], nA)) ? 1 : 0;
        }
        plan.cell_begin[cell + 1] = count;
    }
    for (int32_t m1 = tid; m1 < nA; m1 += PLAN_THREADS) {
        int32_t count = 0;
        for (int32_t n = 0; n < N; n++) {
            count += (PA[n] == m1 && in_bounds(PW2[n], n2) && in_bounds(PO2[n], n3)) ? 1 : 0;
        }
        plan.m1_begin[m1 + 1] = count;
    }
    __syncthreads();
    block_exclusive_scan(plan.cell_begin, n_cells, tile, &carry);
    block_exclusive_scan(plan.m1_begin, nA, tile, &carry);

    for (int32_t cell = tid; cell < n_cells; cell += PLAN_THREADS) {
        const int32_t m3 = cell / n2;
        const int32_t m2 = cell - m3 * n2;
        int32_t slot = plan.cell_begin[cell];
        for (int32_t n = 0; n < N; n++) {
            if (PO2[n] == m3 && PW2[n] == m2 && in_bounds(PA[n], nA)) {
                plan.cell_coefficient[slot] = C[n];
                plan.cell_m1[slot] = PA[n];
                slot++;
            }
        }
    }
    for (int32_t m1 = tid; m1 < nA; m1 += PLAN_THREADS) {
        int32_t slot = plan.m1_begin[m1];
        for (int32_t n = 0; n < N; n++) {
            if (PA[n] == m1 && in_bounds(PW2[n], n2) && in_bounds(PO2[n], n3)) {
                plan.m1_coefficient[slot] = C[n];
                plan.m1_cell[slot] = PO2[n] * n2 + PW2[n];
                slot++;
            }
        }
    }
}

template <typename T> CouplingPlan<T> as_const(const CouplingPlanBuffers<T>& buffers) {
    return CouplingPlan<T>{buffers.cell_begin, buffers.cell_coefficient, buffers.cell_m1,
                           buffers.m1_begin,   buffers.m1_coefficient,   buffers.m1_cell};
}

// T[e, cell] for the `n` edges whose A rows are staged in `a_stage`
// ([n, nA], row-major) -> t_stage [n, n_cells]. All threads participate.
template <typename T>
__device__ __forceinline__ void contract_table(
    T* __restrict__ t_stage,
    const T* __restrict__ a_stage,
    const CouplingPlan<T>& plan,
    int32_t n,
    int32_t nA,
    int32_t n_cells
) {
    for (int32_t i = threadIdx.x; i < n * n_cells; i += blockDim.x) {
        int32_t e = i / n_cells;
        int32_t cell = i - e * n_cells;
        const T* a_row = a_stage + e * nA;
        T sum = 0;
        for (int32_t p = plan.cell_begin[cell]; p < plan.cell_begin[cell + 1]; p++) {
            sum += plan.cell_coefficient[p] * a_row[plan.cell_m1[p]];
        }
        t_stage[i] = sum;
    }
}

// ---------------------------------------------------------------------------
// forward: one workgroup per receiver row; thread t owns output element
// (m3, l). Per chunk of edges the workgroup stages A rows, the products
// Z[e, m2, l] = B[e, l] * W[PW1[e], m2, l] and the contracted table T in LDS.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(MAX_THREADS) void forward_kernel(
    T* __restrict__ output,
    const T* __restrict__ A,
    const T* __restrict__ B,
    const T* __restrict__ W,
    const int32_t* __restrict__ PW1,
    CouplingPlan<T> plan,
    const int32_t* __restrict__ segments,
    int32_t n_nodes,
    int32_t nA,
    int32_t L,
    int32_t n2,
    int32_t n3,
    int32_t chunk
) {
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    const int32_t n_cells = n2 * n3;
    T* a_stage = reinterpret_cast<T*>(lds_bytes);
    T* t_stage = a_stage + static_cast<size_t>(chunk) * nA;
    T* z_stage = t_stage + static_cast<size_t>(chunk) * n_cells;

    const int32_t row = blockIdx.x;
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int32_t first = segments[row];
    const int32_t last = segments[n_nodes + row];
    const int32_t row_elements = n3 * L;
    const int32_t z_per_edge = n2 * L;
    T* out_row = output + static_cast<size_t>(row) * row_elements;

    for (int32_t tile = 0; tile < row_elements; tile += nthreads) {
        const int32_t element = tile + tid;
        const bool active = element < row_elements;
        const int32_t m3 = active ? element / L : 0;
        const int32_t l = active ? element - m3 * L : 0;
        T sum = 0;

        for (int32_t c0 = first; c0 < last; c0 += chunk) {
            const int32_t n = min(chunk, last - c0);
            __syncthreads();
            const T* a_src = A + static_cast<size_t>(c0) * nA;
            for (int32_t i = tid; i < n * nA; i += nthreads) {
                a_stage[i] = a_src[i];
            }
            for (int32_t i = tid; i < n * z_per_edge; i += nthreads) {
                int32_t e = i / z_per_edge;
                int32_t rest = i - e * z_per_edge; // m2 * L + col
                int32_t col = rest % L;
                int32_t sender = PW1[c0 + e];
                T value = T(0);
                if (in_bounds(sender, n_nodes)) {
                    value = B[static_cast<size_t>(c0 + e) * L + col] *
                            W[static_cast<size_t>(sender) * z_per_edge + rest];
                }
                z_stage[i] = value;
            }
            __syncthreads();
            contract_table(t_stage, a_stage, plan, n, nA, n_cells);
            __syncthreads();
            if (active) {
                for (int32_t e = 0; e < n; e++) {
                    const T* t_row = t_stage + e * n_cells + m3 * n2;
                    const T* z_col = z_stage + e * z_per_edge + l;
                    for (int32_t m2 = 0; m2 < n2; m2++) {
                        sum += t_row[m2] * z_col[m2 * L];
                    }
                }
            }
        }
        if (active) {
            out_row[element] = sum;
        }
    }
}

// ---------------------------------------------------------------------------
// vjp, receiver side: grad_A and grad_B rows of the edges of one receiver.
// The receiver's grad_output tile G [n3, L] is staged once (odd row stride).
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(MAX_THREADS) void vjp_edges_kernel(
    T* __restrict__ grad_A,
    T* __restrict__ grad_B,
    const T* __restrict__ grad_output,
    const T* __restrict__ A,
    const T* __restrict__ B,
    const T* __restrict__ W,
    const int32_t* __restrict__ PW1,
    CouplingPlan<T> plan,
    const int32_t* __restrict__ segments,
    int32_t n_nodes,
    int32_t nA,
    int32_t L,
    int32_t n2,
    int32_t n3,
    int32_t chunk
) {
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    const int32_t row = blockIdx.x;
    const int32_t first = segments[row];
    const int32_t last = segments[n_nodes + row];
    if (first < 0) {
        return;
    }
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int32_t n_cells = n2 * n3;
    const int32_t Ls = odd_stride(L);
    const int32_t w_per_edge = n2 * Ls;

    T* g_stage = reinterpret_cast<T*>(lds_bytes);                 // [n3, Ls]
    T* a_stage = g_stage + static_cast<size_t>(n3) * Ls;          // [chunk, nA]
    T* b_stage = a_stage + static_cast<size_t>(chunk) * nA;       // [chunk, L]
    T* t_stage = b_stage + static_cast<size_t>(chunk) * L;        // [chunk, n_cells]  T, later U
    T* w_stage = t_stage + static_cast<size_t>(chunk) * n_cells;  // [chunk, n2, Ls]

    const T* g_src = grad_output + static_cast<size_t>(row) * n3 * L;
    for (int32_t i = tid; i < n3 * L; i += nthreads) {
        int32_t m3 = i / L;
        g_stage[m3 * Ls + (i - m3 * L)] = g_src[i];
    }

    for (int32_t c0 = first; c0 < last; c0 += chunk) {
        const int32_t n = min(chunk, last - c0);
        __syncthreads();
        const T* a_src = A + static_cast<size_t>(c0) * nA;
        for (int32_t i = tid; i < n * nA; i += nthreads) {
            a_stage[i] = a_src[i];
        }
        const T* b_src = B + static_cast<size_t>(c0) * L;
        for (int32_t i = tid; i < n * L; i += nthreads) {
            b_stage[i] = b_src[i];
        }
        for (int32_t i = tid; i < n * n2 * L; i += nthreads) {
            int32_t e = i / (n2 * L);
            int32_t rest = i - e * (n2 * L);
            int32_t m2 = rest / L;
            int32_t col = rest - m2 * L;
            int32_t sender = PW1[c0 + e];
            w_stage[e * w_per_edge + m2 * Ls + col] =
                in_bounds(sender, n_nodes) ? W[static_cast<size_t>(sender) * n2 * L + rest] : T(0);
        }
        __syncthreads();

        if (grad_B != nullptr) {
            contract_table(t_stage, a_stage, plan, n, nA, n_cells);
            __syncthreads();
            T* dst = grad_B + static_cast<size_t>(c0) * L;
            for (int32_t i = tid; i < n * L; i += nthreads) {
                int32_t e = i / L;
                int32_t l = i - e * L;
                const T* t_edge = t_stage + e * n_cells;
                const T* w_col = w_stage + e * w_per_edge + l;
                T sum = 0;
                for (int32_t m3 = 0; m3 < n3; m3++) {
                    T inner = 0;
                    for (int32_t m2 = 0; m2 < n2; m2++) {
                        inner += t_edge[m3 * n2 + m2] * w_col[m2 * Ls];
                    }
                    sum += g_stage[m3 * Ls + l] * inner;
                }
                dst[i] = sum;
            }
            __syncthreads();
        }

        if (grad_A != nullptr) {
            // U[e, cell] over the feature channel
            for (int32_t i = tid; i < n * n_cells; i += nthreads) {
                int32_t e = i / n_cells;
                int32_t cell = i - e * n_cells;
                int32_t m3 = cell / n2;
                int32_t m2 = cell - m3 * n2;
                const T* b_row = b_stage + e * L;
                const T* g_row = g_stage + m3 * Ls;
                const T* w_row = w_stage + e * w_per_edge + m2 * Ls;
                T sum = 0;
                for (int32_t l = 0; l < L; l++) {
                    sum += b_row[l] * g_row[l] * w_row[l];
                }
                t_stage[i] = sum;
            }
            __syncthreads();
            T* dst = grad_A + static_cast<size_t>(c0) * nA;
            for (int32_t i = tid; i < n * nA; i += nthreads) {
                int32_t e = i / nA;
                int32_t m1 = i - e * nA;
                const T* u_edge = t_stage + e * n_cells;
                T sum = 0;
                for (int32_t p = plan.m1_begin[m1]; p < plan.m1_begin[m1 + 1]; p++) {
                    sum += plan.m1_coefficient[p] * u_edge[plan.m1_cell[p]];
                }
                dst[i] = sum;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// vjp, sender side: grad_W[w] gathers over the edges that name w as sender,
// in ascending edge order. Thread t owns element (m2, l) of the row.
// Staged per chunk: A rows, T, and GB[e, m3, l] = G[PO1[e], m3, l] * B[e, l].
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(MAX_THREADS) void vjp_weights_kernel(
    T* __restrict__ grad_W,
    const T* __restrict__ grad_output,
    const T* __restrict__ A,
    const T* __restrict__ B,
    const int32_t* __restrict__ PO1,
    CouplingPlan<T> plan,
    SenderBuckets buckets,
    int32_t n_nodes,
    int32_t nA,
    int32_t L,
    int32_t n2,
    int32_t n3,
    int32_t chunk
) {
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    __shared__ int32_t bucket_lds[BUCKET_LDS_CAPACITY];
    const int32_t node = blockIdx.x;
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int32_t n_cells = n2 * n3;
    const int32_t g_per_edge = n3 * L;

    T* a_stage = reinterpret_cast<T*>(lds_bytes);                 // [chunk, nA]
    T* t_stage = a_stage + static_cast<size_t>(chunk) * nA;       // [chunk, n_cells]
    T* gb_stage = t_stage + static_cast<size_t>(chunk) * n_cells; // [chunk, n3, L]

    SortedBucket bucket = sorted_bucket(buckets, node, bucket_lds);
    const int32_t row_elements = n2 * L;
    T* out_row = grad_W + static_cast<size_t>(node) * row_elements;

    for (int32_t tile = 0; tile < row_elements; tile += nthreads) {
        const int32_t element = tile + tid;
        const bool active = element < row_elements;
        const int32_t m2 = active ? element / L : 0;
        const int32_t l = active ? element - m2 * L : 0;
        T sum = 0;

        for (int32_t c0 = 0; c0 < bucket.count; c0 += chunk) {
            const int32_t n = min(chunk, bucket.count - c0);
            __syncthreads();
            for (int32_t i = tid; i < n * nA; i += nthreads) {
                int32_t e = i / nA;
                int32_t edge = bucket.edges[c0 + e];
                a_stage[i] = A[static_cast<size_t>(edge) * nA + (i - e * nA)];
            }
            for (int32_t i = tid; i < n * g_per_edge; i += nthreads) {
                int32_t e = i / g_per_edge;
                int32_t rest = i - e * g_per_edge; // m3 * L + col
                int32_t col = rest % L;
                int32_t edge = bucket.edges[c0 + e];
                int32_t receiver = PO1[edge];
                T value = T(0);
                if (in_bounds(receiver, n_nodes)) {
                    value = grad_output[static_cast<size_t>(receiver) * g_per_edge + rest] *
                            B[static_cast<size_t>(edge) * L + col];
                }
                gb_stage[i] = value;
            }
            __syncthreads();
            contract_table(t_stage, a_stage, plan, n, nA, n_cells);
            __syncthreads();
            if (active) {
                for (int32_t e = 0; e < n; e++) {
                    const T* t_col = t_stage + e * n_cells + m2;
                    const T* gb_col = gb_stage + e * g_per_edge + l;
                    for (int32_t m3 = 0; m3 < n3; m3++) {
                        sum += t_col[m3 * n2] * gb_col[m3 * L];
                    }
                }
            }
        }
        if (active) {
            out_row[element] = sum;
        }
    }
}

template <typename T> int32_t pick_chunk(size_t per_edge, size_t fixed, int32_t cap) {
    size_t budget = STAGING_BYTES / sizeof(T);
    size_t available = budget > fixed ? budget - fixed : 0;
    size_t chunk = per_edge > 0 ? available / per_edge : static_cast<size_t>(cap);
    chunk = std::min<size_t>(chunk, static_cast<size_t>(cap));
    return static_cast<int32_t>(chunk);
}

struct Sizes {
    int32_t n_nodes, n_edges, nA, L, N, n2, n3, n_cells;
};

template <typename T>
Sizes sizes_of(Tensor<T, 3> output, Tensor<T, 2> A, Tensor<T, 2> B, Tensor<T, 1> C, Tensor<T, 3> W) {
    Sizes s;
    s.n_nodes = narrow_i32(output.shape[0], "output.shape[0]");
    s.n_edges = narrow_i32(A.shape[0], "A.shape[0]");
    s.nA = narrow_i32(A.shape[1], "A.shape[1]");
    s.L = narrow_i32(B.shape[1], "B.shape[1]");
    s.N = narrow_i32(C.shape[0], "C.shape[0]");
    s.n2 = narrow_i32(W.shape[1], "W.shape[1]");
    s.n3 = narrow_i32(output.shape[1], "output.shape[1]");
    s.n_cells = narrow_i32(W.shape[1] * output.shape[1], "W.shape[1] * output.shape[1]");
    narrow_i32(W.shape[1] * W.shape[2], "W.shape[1] * W.shape[2]");
    narrow_i32(output.shape[1] * output.shape[2], "output.shape[1] * output.shape[2]");
    return s;
}

[[noreturn]] void too_large(const char* operation) {
    throw std::runtime_error(
        std::string(operation) +
        ": the per-edge working set (size_A, size_B, W.shape[1], output.shape[1]) does not fit "
        "the LDS staging area of the device kernel"
    );
}

template <typename T>
CouplingPlan<T> enqueue_plan(
    void* workspace,
    const Sizes& s,
    Tensor<T, 1> C,
    Tensor<int32_t, 1> indices_A,
    Tensor<int32_t, 1> indices_W_2,
    Tensor<int32_t, 1> indices_output_2,
    hipStream_t stream
) {
    CouplingPlanBuffers<T> buffers = carve_plan<T>(workspace, s.N, s.n_cells, s.nA);
    plan_kernel<T><<<1, PLAN_THREADS, 0, stream>>>(
        buffers, C.data, indices_A.data, indices_W_2.data, indices_output_2.data, s.N, s.nA, s.n2, s.n3
    );
    MOPS_HIP_CHECK(hipGetLastError());
    return as_const(buffers);
}

} // namespace
} // namespace sasaw
using namespace sasaw;
} // namespace mops::amd

namespace mops::cuda {

template <typename scalar_t>
void sparse_accumulation_scatter_add_with_weights(MOPS_SASAW_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using namespace mops::amd;
    const char* operation = "cuda_sparse_accumulation_scatter_add_with_weights";
    checks::Validator validator(operation);
    checks::sasaw(
        validator, output, A, B, C, W, indices_A, indices_W_1, indices_W_2, indices_output_1, indices_output_2
    );
    if (accept_unsorted() && !is_sorted_on_device(
                                 indices_output_1.data, narrow_i32(A.shape[0], "A.shape[0]"), current_stream()
                             )) {
        // the same call on the edges in the order of a stable sort by receiver
        hipStream_t stream = current_stream();
        const int32_t n_edges = narrow_i32(A.shape[0], "A.shape[0]");
        const int32_t nA = narrow_i32(A.shape[1], "A.shape[1]"), L = narrow_i32(B.shape[1], "B.shape[1]");
        EdgeOrder order(indices_output_1.data, n_edges, stream);
        StreamTemporary<scalar_t> sorted_A(A.shape[0] * A.shape[1], stream);
        StreamTemporary<scalar_t> sorted_B(B.shape[0] * B.shape[1], stream);
        StreamTemporary<int32_t> sorted_W_1(A.shape[0], stream);
        order.gather_rows(sorted_A.data(), A.data, nA);
        order.gather_rows(sorted_B.data(), B.data, L);
        order.gather_rows(sorted_W_1.data(), indices_W_1.data, 1);
        ::mops::cuda::sparse_accumulation_scatter_add_with_weights<scalar_t>(
            output, {sorted_A.data(), {A.shape[0], A.shape[1]}}, {sorted_B.data(), {B.shape[0], B.shape[1]}}, C, W,
            indices_A, {sorted_W_1.data(), {A.shape[0]}}, indices_W_2,
            {const_cast<int32_t*>(order.sorted_index()), {A.shape[0]}}, indices_output_2
        );
        return;
    }
    validate_gather_index(indices_A, A.shape[1], "indices_A", operation);
    validate_gather_index(indices_W_1, output.shape[0], "indices_W_1", operation);
    validate_gather_index(indices_W_2, W.shape[1], "indices_W_2", operation);
    validate_scatter_index(indices_output_1, output.shape[0], "indices_output_1", operation);
    validate_gather_index(indices_output_2, output.shape[1], "indices_output_2", operation);

    const Sizes s = sizes_of(output, A, B, C, W);
    if (s.n_nodes == 0 || s.n3 == 0 || s.L == 0) {
        return;
    }
    hipStream_t stream = current_stream();

    const sasaw_mfma::Shape shape{s.n_nodes, s.n_edges, s.nA, s.L, s.N, s.n2, s.n3};
    if (sasaw_segments::supports_forward(shape, sizeof(scalar_t))) {
        const sasaw_mfma::Indices indices{
            indices_A.data, indices_W_1.data, indices_W_2.data, indices_output_1.data, indices_output_2.data
        };
        sasaw_segments::forward<scalar_t>(output.data, A.data, B.data, C.data, W.data, indices, shape, stream);
        finish_call(operation);
        return;
    }
    if (sasaw_mfma::supports(shape, sizeof(scalar_t))) {
        const sasaw_mfma::Indices indices{
            indices_A.data, indices_W_1.data, indices_W_2.data, indices_output_1.data, indices_output_2.data
        };
        void* workspace = scratch(sasaw_mfma::workspace_bytes(shape, sizeof(scalar_t)));
        sasaw_mfma::forward<scalar_t>(
            output.data, A.data, B.data, C.data, W.data, indices, shape, workspace, stream
        );
        finish_call(operation);
        return;
    }

    const size_t segments_bytes = align256(static_cast<size_t>(s.n_nodes) * 2 * sizeof(int32_t));
    char* workspace = static_cast<char*>(
        scratch(segments_bytes + plan_bytes<scalar_t>(s.N, s.n_cells, s.nA))
    );
    auto* segments = reinterpret_cast<int32_t*>(workspace);
    first_occurrences(indices_output_1.data, s.n_edges, s.n_nodes, segments, stream);
    CouplingPlan<scalar_t> plan = enqueue_plan<scalar_t>(
        workspace + segments_bytes, s, C, indices_A, indices_W_2, indices_output_2, stream
    );

    const size_t per_edge =
        static_cast<size_t>(s.nA) + s.n_cells + static_cast<size_t>(s.n2) * s.L;
    int32_t chunk = pick_chunk<scalar_t>(per_edge, 0, 16);
    if (chunk < 1) {
        too_large(operation);
    }
    size_t lds = static_cast<size_t>(chunk) * per_edge * sizeof(scalar_t);
    int threads = std::min(MAX_THREADS, round_up_wave(std::min(s.n3 * s.L, MAX_THREADS)));
    forward_kernel<scalar_t><<<s.n_nodes, threads, lds, stream>>>(
        output.data, A.data, B.data, W.data, indices_W_1.data, plan, segments, s.n_nodes, s.nA, s.L,
        s.n2, s.n3, chunk
    );
    finish_call(operation);
}

template <typename scalar_t>
void sparse_accumulation_scatter_add_with_weights_vjp(MOPS_SASAW_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using namespace mops::amd;
    const char* operation = "cuda_sparse_accumulation_scatter_add_with_weights_vjp";
    checks::Validator validator(operation);
    checks::sasaw_vjp(
        validator, grad_A, grad_B, grad_W, grad_output, A, B, C, W, indices_A, indices_W_1, indices_W_2,
        indices_output_1, indices_output_2
    );
    const bool want_A = grad_A.data != nullptr;
    const bool want_B = grad_B.data != nullptr;
    const bool want_W = grad_W.data != nullptr;
    if (!want_A && !want_B && !want_W) {
        return;
    }
    if (accept_unsorted() && !is_sorted_on_device(
                                 indices_output_1.data, narrow_i32(A.shape[0], "A.shape[0]"), current_stream()
                             )) {
        // the same call on the edges in the order of a stable sort by receiver;
        // the per-edge gradients go back to their own rows afterwards
        hipStream_t stream = current_stream();
        const int32_t n_edges = narrow_i32(A.shape[0], "A.shape[0]");
        const int32_t nA = narrow_i32(A.shape[1], "A.shape[1]"), L = narrow_i32(B.shape[1], "B.shape[1]");
        EdgeOrder order(indices_output_1.data, n_edges, stream);
        StreamTemporary<scalar_t> sorted_A(A.shape[0] * A.shape[1], stream);
        StreamTemporary<scalar_t> sorted_B(B.shape[0] * B.shape[1], stream);
        StreamTemporary<int32_t> sorted_W_1(A.shape[0], stream);
        StreamTemporary<scalar_t> sorted_grad_A(want_A ? A.shape[0] * A.shape[1] : 0, stream);
        StreamTemporary<scalar_t> sorted_grad_B(want_B ? B.shape[0] * B.shape[1] : 0, stream);
        order.gather_rows(sorted_A.data(), A.data, nA);
        order.gather_rows(sorted_B.data(), B.data, L);
        order.gather_rows(sorted_W_1.data(), indices_W_1.data, 1);
        ::mops::cuda::sparse_accumulation_scatter_add_with_weights_vjp<scalar_t>(
            {sorted_grad_A.data(), {want_A ? A.shape[0] : 0, want_A ? A.shape[1] : 0}},
            {sorted_grad_B.data(), {want_B ? B.shape[0] : 0, want_B ? B.shape[1] : 0}}, grad_W, grad_output,
            {sorted_A.data(), {A.shape[0], A.shape[1]}}, {sorted_B.data(), {B.shape[0], B.shape[1]}}, C, W,
            indices_A, {sorted_W_1.data(), {A.shape[0]}}, indices_W_2,
            {const_cast<int32_t*>(order.sorted_index()), {A.shape[0]}}, indices_output_2
        );
        if (want_A) {
            order.scatter_rows(grad_A.data, sorted_grad_A.data(), nA);
        }
        if (want_B) {
            order.scatter_rows(grad_B.data, sorted_grad_B.data(), L);
        }
        finish_call(operation);
        return;
    }
    // the reference repeats the gradient shape tests here under the operation
    // name "sasaw_vjp" (mops/src/sasaw/cpu.tpp:99-110); they cannot fail after
    // the validation above but are kept for the same observable behaviour
    if (want_A) {
        checks::same_shape(grad_A, "grad_A", A, "A", "sasaw_vjp");
    }
    if (want_B) {
        checks::same_shape(grad_B, "grad_B", B, "B", "sasaw_vjp");
    }
    if (want_W) {
        checks::same_shape(grad_W, "grad_W", W, "W", "sasaw_vjp");
    }
    validate_gather_index(indices_A, A.shape[1], "indices_A", operation);
    validate_gather_index(indices_W_1, grad_output.shape[0], "indices_W_1", operation);
    validate_gather_index(indices_W_2, W.shape[1], "indices_W_2", operation);
    validate_scatter_index(indices_output_1, grad_output.shape[0], "indices_output_1", operation);
    validate_gather_index(indices_output_2, grad_output.shape[1], "indices_output_2", operation);

    const Sizes s = sizes_of(grad_output, A, B, C, W);
    hipStream_t stream = current_stream();

    const sasaw_mfma::Shape shape{s.n_nodes, s.n_edges, s.nA, s.L, s.N, s.n2, s.n3};
    if (s.L > 0 && sasaw_segments::vjp_supported(shape, sizeof(scalar_t), want_W)) {
        const sasaw_mfma::Indices indices{
            indices_A.data, indices_W_1.data, indices_W_2.data, indices_output_1.data, indices_output_2.data
        };
        const size_t bytes = sasaw_segments::vjp_workspace_bytes(shape, want_W);
        void* workspace = bytes > 0 ? scratch(bytes) : nullptr;
        std::optional<ScratchCounters> taken; // (until the end of this call, finish_call included)
        if (bytes > 0) {
            taken.emplace();
        }
        int32_t* counters = taken ? taken->data() : nullptr;
        sasaw_segments::vjp<scalar_t>(
            grad_A.data, grad_B.data, grad_W.data, grad_output.data, A.data, B.data, C.data, W.data, indices,
            shape, workspace, counters, true, stream
        );
        finish_call(operation);
        return;
    }
    if (sasaw_mfma::supports(shape, sizeof(scalar_t))) {
        const sasaw_mfma::Indices indices{
            indices_A.data, indices_W_1.data, indices_W_2.data, indices_output_1.data, indices_output_2.data
        };
        void* workspace = scratch(sasaw_mfma::workspace_bytes(shape, sizeof(scalar_t)));
        sasaw_mfma::vjp<scalar_t>(
            grad_A.data, grad_B.data, grad_W.data, grad_output.data, A.data, B.data, C.data, W.data, indices,
            shape, workspace, stream
        );
        finish_call(operation);
        return;
    }

    const size_t segments_bytes = align256(static_cast<size_t>(s.n_nodes) * 2 * sizeof(int32_t));
    const size_t table_bytes = plan_bytes<scalar_t>(s.N, s.n_cells, s.nA);
    const size_t buckets_bytes = want_W ? sender_buckets_bytes(s.n_nodes, s.n_edges) : 0;
    char* workspace = static_cast<char*>(scratch(segments_bytes + table_bytes + buckets_bytes));
    auto* segments = reinterpret_cast<int32_t*>(workspace);
    CouplingPlan<scalar_t> plan = enqueue_plan<scalar_t>(
        workspace + segments_bytes, s, C, indices_A, indices_W_2, indices_output_2, stream
    );

    if ((want_A || want_B) && s.n_nodes > 0 && s.n_edges > 0 && (s.nA > 0 || s.L > 0)) {
        first_occurrences(indices_output_1.data, s.n_edges, s.n_nodes, segments, stream);
        const int32_t Ls = odd_stride(s.L);
        const size_t fixed = static_cast<size_t>(s.n3) * Ls;
        const size_t per_edge = static_cast<size_t>(s.nA) + s.L + s.n_cells +
                                static_cast<size_t>(s.n2) * Ls;
        int32_t chunk = pick_chunk<scalar_t>(per_edge, fixed, 16);
        if (chunk < 1) {
            too_large(operation);
        }
        size_t lds = (fixed + static_cast<size_t>(chunk) * per_edge) * sizeof(scalar_t);
        int widest = std::max(std::max(s.L, s.n_cells), s.nA) * chunk;
        int threads = std::min(512, round_up_wave(std::max(widest, 1)));
        vjp_edges_kernel<scalar_t><<<s.n_nodes, threads, lds, stream>>>(
            grad_A.data, grad_B.data, grad_output.data, A.data, B.data, W.data, indices_W_1.data, plan,
            segments, s.n_nodes, s.nA, s.L, s.n2, s.n3, chunk
        );
    }

    if (want_W && s.n_nodes > 0 && s.n2 > 0 && s.L > 0) {
        SenderBuckets buckets = build_sender_buckets(
            indices_W_1.data, s.n_edges, s.n_nodes, workspace + segments_bytes + table_bytes, stream
        );
        const size_t per_edge =
            static_cast<size_t>(s.nA) + s.n_cells + static_cast<size_t>(s.n3) * s.L;
        int32_t chunk = pick_chunk<scalar_t>(per_edge, 0, 16);
        if (chunk < 1) {
            too_large(operation);
        }
        size_t lds = static_cast<size_t>(chunk) * per_edge * sizeof(scalar_t);
        int threads = std::min(MAX_THREADS, round_up_wave(std::min(s.n2 * s.L, MAX_THREADS)));
        vjp_weights_kernel<scalar_t><<<s.n_nodes, threads, lds, stream>>>(
            grad_W.data, grad_output.data, A.data, B.data, indices_output_1.data, plan, buckets,
            s.n_nodes, s.nA, s.L, s.n2, s.n3, chunk
        );
    }
    finish_call(operation);
}

template <typename scalar_t>
void sparse_accumulation_scatter_add_with_weights_vjp_vjp(MOPS_SASAW_VJP_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    // no double backward exists for this operation on any device
    // (mops/src/sasaw/cpu.tpp:173-194)
    throw std::runtime_error("Not implemented");
}

MOPS_CXX_INSTANTIATE(sparse_accumulation_scatter_add_with_weights, MOPS_SASAW_PARAMS)
MOPS_CXX_INSTANTIATE(sparse_accumulation_scatter_add_with_weights_vjp, MOPS_SASAW_VJP_PARAMS)
MOPS_CXX_INSTANTIATE(sparse_accumulation_scatter_add_with_weights_vjp_vjp, MOPS_SASAW_VJP_VJP_PARAMS)

} // namespace mops::cuda

// ---------------------------------------------------------------------------
// the entry point that allocates nothing

namespace mops::amd {
namespace {

// Temporary memory of the no-allocation entry point: part of the code object,
// so every GPU the library runs on holds its own copy from the moment the
// code object is loaded there until the process ends. In host code this name
// is only a handle for hipGetSymbolAddress, never an address.
static __device__ __align__(256) unsigned char no_alloc_scratch[NO_ALLOC_SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;
std::atomic<void*> no_alloc_scratch_address[MAX_DEVICES];

/// Address of the array on the current device (asked for once per device).
void* no_alloc_scratch_of_current_device() {
    int device = 0;
    MOPS_HIP_CHECK(hipGetDevice(&device));
    if (device < 0 || device >= MAX_DEVICES) {
        throw std::runtime_error("mops: device number " + std::to_string(device) + " is beyond the no-allocation entry point's table");
    }
    void* address = no_alloc_scratch_address[device].load(std::memory_order_acquire);
    if (address == nullptr) {
        MOPS_HIP_CHECK(hipGetSymbolAddress(&address, HIP_SYMBOL(no_alloc_scratch)));
        if (address == nullptr) {
            throw std::runtime_error("mops: hipGetSymbolAddress gave no address for the no-allocation scratch array");
        }
        // (two threads may both ask: they get the same answer)
        no_alloc_scratch_address[device].store(address, std::memory_order_release);
    }
    return address;
}

} // namespace

void sasaw_vjp_no_alloc(
    Tensor<float, 2> grad_A,
    Tensor<float, 2> grad_B,
    Tensor<float, 3> grad_W,
    Tensor<float, 3> grad_output,
    Tensor<float, 2> A,
    Tensor<float, 2> B,
    Tensor<float, 1> C,
    Tensor<float, 3> W,
    Tensor<int32_t, 1> indices_A,
    Tensor<int32_t, 1> indices_W_1,
    Tensor<int32_t, 1> indices_W_2,
    Tensor<int32_t, 1> indices_output_1,
    Tensor<int32_t, 1> indices_output_2
) {
    const char* operation = "cuda_sparse_accumulation_scatter_add_with_weights_vjp";
    checks::Validator validator(operation);
    checks::sasaw_vjp(
        validator, grad_A, grad_B, grad_W, grad_output, A, B, C, W, indices_A, indices_W_1, indices_W_2,
        indices_output_1, indices_output_2
    );
    const bool want_edges = grad_A.data != nullptr || grad_B.data != nullptr;
    const bool want_W = grad_W.data != nullptr;
    if (!want_edges && !want_W) {
        return;
    }
    // (with MOPS_AMD_CHECK_INDICES=1 these copy the indices to the host and wait for the stream,
    // as in the existing entry point: a debugging aid, not for a stream that is being captured)
    validate_gather_index(indices_A, A.shape[1], "indices_A", operation);
    validate_gather_index(indices_W_1, grad_output.shape[0], "indices_W_1", operation);
    validate_gather_index(indices_W_2, W.shape[1], "indices_W_2", operation);
    validate_scatter_index(indices_output_1, grad_output.shape[0], "indices_output_1", operation);
    validate_gather_index(indices_output_2, grad_output.shape[1], "indices_output_2", operation);
    // Kernel timing (mops_amd_kernel_timing) takes HIP events from a pool that it fills with
    // hipEventCreate: not in a call that promises to create nothing. Off for the length of it.
    struct TimingOff {
        bool was = set_kernel_timing(false);
        ~TimingOff() { set_kernel_timing(was); }
    } timing_off;
    const Sizes s = sizes_of(grad_output, A, B, C, W);
    hipStream_t stream = current_stream();
    if (s.L == 0 || s.N == 0 || s.n_edges == 0 || s.n_nodes == 0 || s.nA == 0 || s.n2 == 0 || s.n3 == 0) {
        // every sum is over nothing: the gradients that have elements are zero (as the existing
        // entry point gives them)
        if (grad_A.data != nullptr) {
            fill_zero(grad_A.data, static_cast<size_t>(s.n_edges) * s.nA, stream);
        }
        if (grad_B.data != nullptr) {
            fill_zero(grad_B.data, static_cast<size_t>(s.n_edges) * s.L, stream);
        }
        if (want_W) {
            fill_zero(grad_W.data, static_cast<size_t>(s.n_nodes) * s.n2 * s.L, stream);
        }
        finish_call(operation);
        return;
    }
    const sasaw_mfma::Shape shape{s.n_nodes, s.n_edges, s.nA, s.L, s.N, s.n2, s.n3};
    const char* who = "mops_amd_sparse_accumulation_scatter_add_with_weights_vjp_no_alloc_f32: ";
    const sasaw_mfma::Indices indices{
        indices_A.data, indices_W_1.data, indices_W_2.data, indices_output_1.data, indices_output_2.data
    };
    if (s.L > 0 && sasaw_segments::vjp_supported(shape, sizeof(float), want_W)) {
        // (the same kernels as the existing entry point takes for these shapes)
        // (the places of the senders' edges, then their counters; the array is shared with the
        // kernels of other shapes, so the counters are cleared by a launch in front)
        const size_t places = sasaw_segments::vjp_workspace_bytes(shape, want_W);
        const size_t needed = places + sasaw_segments::vjp_counters(shape, want_W) * sizeof(int32_t);
        if (needed > NO_ALLOC_SCRATCH_BYTES) {
            throw std::runtime_error(
                std::string(who) + "these shapes need " + std::to_string(needed) + " bytes of temporary memory, the "
                "built-in array holds " + std::to_string(NO_ALLOC_SCRATCH_BYTES) + " (about " +
                std::to_string(NO_ALLOC_SCRATCH_BYTES / 528 - 64) + " nodes); use "
                "mops_cuda_sparse_accumulation_scatter_add_with_weights_vjp_f32"
            );
        }
        char* const array = static_cast<char*>(no_alloc_scratch_of_current_device());
        sasaw_segments::vjp<float>(
            grad_A.data, grad_B.data, grad_W.data, grad_output.data, A.data, B.data, C.data, W.data, indices, shape,
            array, reinterpret_cast<int32_t*>(array + places), false, stream
        );
        finish_call(operation);
        return;
    }
    if (!sasaw_mfma::supports(shape, sizeof(float))) {
        throw std::runtime_error(
            std::string(who) + "only the shapes of the matrix-core kernels are served without allocation (at least "
            "one node, edge and table entry; A.shape[1], W.shape[1] and output.shape[1] between 1 and 16); use "
            "mops_cuda_sparse_accumulation_scatter_add_with_weights_vjp_f32"
        );
    }
    if (want_W && sasaw_mfma::orders_edges_by_sender(shape, sizeof(float))) {
        throw std::runtime_error(
            std::string(who) + "for a graph of this size with more than 48 edges per node on average grad_W needs "
            "the edges put in the order of their senders first, by a counting sort on a second stream, which this "
            "entry point cannot create; use mops_cuda_sparse_accumulation_scatter_add_with_weights_vjp_f32"
        );
    }
    if (!sasaw_mfma::vjp_allocates_nothing(shape, sizeof(float), want_edges, want_W)) {
        throw std::runtime_error(
            std::string(who) + "for this graph (more than 48 edges per node on average) grad_W is computed beside "
            "the other gradients on a second stream, which this entry point cannot create; use "
            "mops_cuda_sparse_accumulation_scatter_add_with_weights_vjp_f32, or ask for grad_W in a call of its own"
        );
    }
    const size_t needed = sasaw_mfma::workspace_bytes(shape, sizeof(float));
    if (needed > NO_ALLOC_SCRATCH_BYTES) {
        throw std::runtime_error(
            std::string(who) + "these shapes need " + std::to_string(needed) + " bytes of temporary memory, the "
            "built-in array holds " + std::to_string(NO_ALLOC_SCRATCH_BYTES) + " (about " +
            std::to_string(NO_ALLOC_SCRATCH_BYTES / 528 - 64) + " nodes); use "
            "mops_cuda_sparse_accumulation_scatter_add_with_weights_vjp_f32"
        );
    }
    void* workspace = no_alloc_scratch_of_current_device();
    sasaw_mfma::vjp<float>(
        grad_A.data, grad_B.data, grad_W.data, grad_output.data, A.data, B.data, C.data, W.data, indices, shape,
        workspace, stream
    );
    finish_call(operation);
}

} // namespace mops::amd

