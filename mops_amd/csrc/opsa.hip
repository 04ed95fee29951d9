// Outer-product scatter-add, without (OPSA) and with (OPSAW) per-sender
// weights, forward and vector-Jacobian product, for gfx950.
//
//   OPSA   O[P[j], k, l]  += A[j, k] * B[j, l]
//   OPSAW  O[PO[e], k, l] += A[e, k] * B[e, l] * W[PW[e], l]
//
// The scatter index is sorted, so the edges of one output row are one
// contiguous segment [first, last) given by first_occurrences. Each output
// row is owned by one workgroup that reduces its segment in registers and
// writes the row once: no atomics, a fixed summation order (ascending edge
// number, the order of the reference's CPU loops), and rows without edges
// are written as exact zeros.
//
// Reference semantics restated here: mops/src/opsa/cpu.tpp:9-112 and
// mops/src/opsaw/cpu.tpp:9-131 of lab-cosmo/mops (formulas, optional
// gradients, zero rows); the reference's CUDA OPSA kernels
// (mops/src/opsa/opsa.cu:14-284) use the same one-block-per-row split but
// read A and B from global memory once per output element; OPSAW has no
// reference device code at all (mops/src/opsaw/opsaw.cu:1).
#include <algorithm>
#include <vector>

#include "mops/opsa.hpp"
#include "mops/opsaw.hpp"

#include "checks.hpp"
#include "device_common.hpp"
#include "first_occurrences.hpp"
#include "index_validation.hpp"
#include "runtime.hpp"
#include "sender_buckets.hpp"

namespace mops::amd {
namespace {

// LDS the staging buffers of one workgroup may use. Well below the 160 KB of
// a gfx950 CU so that several workgroups stay resident per CU.
constexpr size_t STAGING_BYTES = 32 * 1024;
constexpr int MAX_THREADS = 1024;

// ---------------------------------------------------------------------------
// forward
//
// grid: one workgroup per output row; thread t owns output element
// (k, l) = (t / L, t % L) (and t + blockDim, ... when K*L > blockDim).
// The segment is streamed through LDS in chunks of `chunk` edges with
// coalesced loads of the contiguous rows A[first..], B[first..]; for OPSAW the
// weight row W[PW[e]] is folded into the staged copy of B, so the inner loop
// is the same two LDS reads and one FMA per edge for both operations.
// ---------------------------------------------------------------------------
template <typename T, bool WEIGHTED>
__global__ __launch_bounds__(MAX_THREADS) void forward_kernel(
    T* __restrict__ output,
    const T* __restrict__ A,
    const T* __restrict__ B,
    const T* __restrict__ W,
    const int32_t* __restrict__ indices_W,
    const int32_t* __restrict__ segments,
    int32_t n_output,
    int32_t n_weights,
    int32_t K,
    int32_t L,
    int32_t chunk
) {
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    T* a_stage = reinterpret_cast<T*>(lds_bytes);
    T* b_stage = a_stage + static_cast<size_t>(chunk) * K;

    const int32_t row = blockIdx.x;
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int32_t first = segments[row];
    const int32_t last = segments[n_output + row];
    const int32_t KL = K * L;
    T* out_row = output + static_cast<size_t>(row) * KL;

    for (int32_t tile = 0; tile < KL; tile += nthreads) {
        const int32_t element = tile + tid;
        const bool active = element < KL;
        const int32_t k = active ? element / L : 0;
        const int32_t l = active ? element - k * L : 0;
        T sum = 0;

        for (int32_t c0 = first; c0 < last; c0 += chunk) {
            const int32_t n = min(chunk, last - c0);
            __syncthreads();
            const T* a_src = A + static_cast<size_t>(c0) * K;
            for (int32_t i = tid; i < n * K; i += nthreads) {
                a_stage[i] = a_src[i];
            }
            const T* b_src = B + static_cast<size_t>(c0) * L;
            for (int32_t i = tid; i < n * L; i += nthreads) {
                T value = b_src[i];
                if (WEIGHTED) {
                    int32_t e = i / L;
                    int32_t col = i - e * L;
                    int32_t w_row = indices_W[c0 + e];
                    value = in_bounds(w_row, n_weights)
                                ? value * W[static_cast<size_t>(w_row) * L + col]
                                : T(0);
                }
                b_stage[i] = value;
            }
            __syncthreads();
            if (active) {
                const T* a_ptr = a_stage + k;
                const T* b_ptr = b_stage + l;
                for (int32_t e = 0; e < n; e++) {
                    sum += a_ptr[e * K] * b_ptr[e * L];
                }
            }
        }
        if (active) {
            out_row[element] = sum;
        }
    }
}

// ---------------------------------------------------------------------------
// vjp with respect to A and B (and, for OPSAW, the per-edge term of grad_W)
//
// grid: one workgroup per output row. The row's grad_output tile [K, L] is
// staged once in LDS (row stride padded to an odd length so that walking a
// column is conflict-free) and reused by every edge of the segment:
//
//   S[e, l]      = sum_k G[k, l] * A[e, k]
//   grad_A[e, k] = sum_l G[k, l] * B[e, l] (* W[PW[e], l])
//   grad_B[e, l] = S[e, l]                 (* W[PW[e], l])
//   edge_W[e, l] = S[e, l] * B[e, l]        -> summed per sender afterwards
//
// Results are written with consecutive threads on consecutive addresses
// (the edges of a segment are contiguous rows of grad_A / grad_B).
// STAGE_G = false is the fallback for tiles too large for LDS: G is then read
// from global memory.
// ---------------------------------------------------------------------------
template <typename T, bool WEIGHTED, bool STAGE_G>
__global__ __launch_bounds__(MAX_THREADS) void vjp_kernel(
    T* __restrict__ grad_A,
    T* __restrict__ grad_B,
    T* __restrict__ edge_W,
    const T* __restrict__ grad_output,
    const T* __restrict__ A,
    const T* __restrict__ B,
    const T* __restrict__ W,
    const int32_t* __restrict__ indices_W,
    const int32_t* __restrict__ segments,
    int32_t n_output,
    int32_t n_weights,
    int32_t K,
    int32_t L,
    int32_t chunk
) {
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    const int32_t row = blockIdx.x;
    const int32_t first = segments[row];
    const int32_t last = segments[n_output + row];
    if (first < 0) {
        return; // no edge reads this row of grad_output
    }
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;

    const int32_t g_stride = STAGE_G ? odd_stride(L) : L;
    T* cursor = reinterpret_cast<T*>(lds_bytes);
    T* g_stage = cursor;
    if (STAGE_G) {
        cursor += static_cast<size_t>(K) * g_stride;
    }
    T* a_stage = cursor;
    cursor += static_cast<size_t>(chunk) * K;
    T* b_stage = cursor; // B, or B * W when weighted
    cursor += static_cast<size_t>(chunk) * L;
    T* w_stage = cursor; // only when weighted
    if (WEIGHTED) {
        cursor += static_cast<size_t>(chunk) * L;
    }
    T* braw_stage = cursor; // unweighted B, only when weighted

    const T* g_global = grad_output + static_cast<size_t>(row) * K * L;
    if (STAGE_G) {
        for (int32_t i = tid; i < K * L; i += nthreads) {
            int32_t k = i / L;
            g_stage[k * g_stride + (i - k * L)] = g_global[i];
        }
    }
    const T* G = STAGE_G ? g_stage : g_global;

    for (int32_t c0 = first; c0 < last; c0 += chunk) {
        const int32_t n = min(chunk, last - c0);
        __syncthreads();
        const T* a_src = A + static_cast<size_t>(c0) * K;
        for (int32_t i = tid; i < n * K; i += nthreads) {
            a_stage[i] = a_src[i];
        }
        const T* b_src = B + static_cast<size_t>(c0) * L;
        for (int32_t i = tid; i < n * L; i += nthreads) {
            T value = b_src[i];
            if (WEIGHTED) {
                int32_t e = i / L;
                int32_t col = i - e * L;
                int32_t w_row = indices_W[c0 + e];
                T weight =
                    in_bounds(w_row, n_weights) ? W[static_cast<size_t>(w_row) * L + col] : T(0);
                w_stage[i] = weight;
                braw_stage[i] = value;
                value *= weight;
            }
            b_stage[i] = value;
        }
        __syncthreads();

        if (grad_A != nullptr) {
            T* dst = grad_A + static_cast<size_t>(c0) * K;
            for (int32_t i = tid; i < n * K; i += nthreads) {
                int32_t e = i / K;
                int32_t k = i - e * K;
                const T* g_row = G + k * g_stride;
                const T* b_row = b_stage + e * L;
                T sum = 0;
                for (int32_t l = 0; l < L; l++) {
                    sum += g_row[l] * b_row[l];
                }
                dst[i] = sum;
            }
        }
        if (grad_B != nullptr || (WEIGHTED && edge_W != nullptr)) {
            for (int32_t i = tid; i < n * L; i += nthreads) {
                int32_t e = i / L;
                int32_t l = i - e * L;
                const T* g_col = G + l;
                const T* a_row = a_stage + e * K;
                T sum = 0;
                for (int32_t k = 0; k < K; k++) {
                    sum += g_col[k * g_stride] * a_row[k];
                }
                if (WEIGHTED) {
                    if (grad_B != nullptr) {
                        grad_B[static_cast<size_t>(c0) * L + i] = sum * w_stage[i];
                    }
                    if (edge_W != nullptr) {
                        edge_W[static_cast<size_t>(c0) * L + i] = sum * braw_stage[i];
                    }
                } else {
                    grad_B[static_cast<size_t>(c0) * L + i] = sum;
                }
            }
        }
    }
}

// An edge whose scatter index lies outside [0, n_output) belongs to no segment:
// its rows of grad_A / grad_B are then left unwritten (such input is invalid;
// the reference's device path does not define it either). Nothing is ever read
// or written out of bounds because of it.

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

// Edges per LDS chunk such that `per_edge` elements per edge plus `fixed`
// elements fit the staging budget.
template <typename T> int32_t pick_chunk(size_t per_edge, size_t fixed) {
    size_t budget = STAGING_BYTES / sizeof(T);
    size_t available = budget > fixed ? budget - fixed : 0;
    size_t chunk = per_edge > 0 ? available / per_edge : 64;
    chunk = std::min<size_t>(chunk, 64);
    return static_cast<int32_t>(std::max<size_t>(chunk, 1));
}

constexpr size_t LDS_LIMIT = 64 * 1024; // stay within the default dynamic-LDS limit

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
    auto* segments = static_cast<int32_t*>(scratch(static_cast<size_t>(n_output) * 2 * sizeof(int32_t)));
    first_occurrences(indices_output.data, n_edges, n_output, segments, stream);

    const size_t per_edge = static_cast<size_t>(K) + L;
    if (per_edge * sizeof(T) > LDS_LIMIT) {
        throw std::runtime_error(
            std::string(operation) + ": size_A + size_B = " + std::to_string(per_edge) +
            " is too large for the device kernel (one row of A and B must fit in 64 KiB of LDS)"
        );
    }
    int32_t chunk = pick_chunk<T>(per_edge, 0);
    size_t lds = static_cast<size_t>(chunk) * per_edge * sizeof(T);
    int threads = std::min(MAX_THREADS, round_up_wave(K * L > 0 ? std::min(K * L, MAX_THREADS) : 1));

    forward_kernel<T, WEIGHTED><<<n_output, threads, lds, stream>>>(
        output.data,
        A.data,
        B.data,
        W,
        indices_W,
        segments,
        n_output,
        n_output,
        K,
        L,
        chunk
    );
    finish_call(operation);
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

    // scratch: segments | edge_W (weighted, grad_W wanted) | sender buckets
    const size_t segments_bytes = align256(static_cast<size_t>(n_output) * 2 * sizeof(int32_t));
    const size_t edge_w_bytes =
        want_W ? align256(static_cast<size_t>(n_edges) * L * sizeof(T)) : 0;
    const size_t buckets_bytes = want_W ? sender_buckets_bytes(n_output, n_edges) : 0;
    char* workspace = static_cast<char*>(scratch(segments_bytes + edge_w_bytes + buckets_bytes));
    auto* segments = reinterpret_cast<int32_t*>(workspace);
    T* edge_W = want_W ? reinterpret_cast<T*>(workspace + segments_bytes) : nullptr;

    if (n_output > 0 && n_edges > 0 && K > 0 && L > 0) {
        first_occurrences(indices_output.data, n_edges, n_output, segments, stream);

        const size_t g_elements = static_cast<size_t>(K) * odd_stride(L);
        const bool stage_g = g_elements * sizeof(T) <= STAGING_BYTES;
        const size_t per_edge = static_cast<size_t>(K) + (WEIGHTED ? 3 : 1) * static_cast<size_t>(L);
        if (per_edge * sizeof(T) > LDS_LIMIT / 2) {
            throw std::runtime_error(
                std::string(operation) + ": size_A and size_B are too large for the device kernel"
            );
        }
        int32_t chunk = pick_chunk<T>(per_edge, 0);
        size_t lds = (static_cast<size_t>(chunk) * per_edge + (stage_g ? g_elements : 0)) * sizeof(T);
        int widest = std::max(K, L) * chunk;
        int threads = std::min(256, round_up_wave(std::max(widest, 1)));

        if (stage_g) {
            vjp_kernel<T, WEIGHTED, true><<<n_output, threads, lds, stream>>>(
                grad_A.data, grad_B.data, edge_W, grad_output.data, A.data, B.data, W, indices_W,
                segments, n_output, n_output, K, L, chunk
            );
        } else {
            vjp_kernel<T, WEIGHTED, false><<<n_output, threads, lds, stream>>>(
                grad_A.data, grad_B.data, edge_W, grad_output.data, A.data, B.data, W, indices_W,
                segments, n_output, n_output, K, L, chunk
            );
        }
    }

    if (want_W && n_output > 0 && L > 0) {
        SenderBuckets buckets = build_sender_buckets(
            indices_W, n_edges, n_output, workspace + segments_bytes + edge_w_bytes, stream
        );
        int threads = std::min(256, round_up_wave(L));
        gather_weights_kernel<T><<<n_output, threads, 0, stream>>>(grad_W.data, edge_W, buckets, L);
    }
    finish_call(operation);
}

} // namespace
} // namespace mops::amd

// ------------------------------------------------------------ C++ API ----
namespace mops::cuda {

template <typename scalar_t>
void outer_product_scatter_add(MOPS_OPSA_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    const char* operation = "cuda_outer_product_scatter_add";
    checks::Validator validator(operation);
    checks::opsa(validator, output, A, B, indices_output);
    amd::validate_scatter_index(indices_output, output.shape[0], "indices_output", operation);
    amd::launch_forward<scalar_t, false>(output, A, B, nullptr, nullptr, indices_output, operation);
}

template <typename scalar_t>
void outer_product_scatter_add_vjp(MOPS_OPSA_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    const char* operation = "cuda_outer_product_scatter_add_vjp";
    checks::Validator validator(operation);
    checks::opsa_vjp(validator, grad_A, grad_B, grad_output, A, B, indices_output);
    amd::validate_scatter_index(indices_output, grad_output.shape[0], "indices_output", operation);
    amd::launch_vjp<scalar_t, false>(
        grad_A, grad_B, Tensor<scalar_t, 2>{nullptr, {0, 0}}, grad_output, A, B, nullptr, nullptr,
        indices_output, operation
    );
}

template <typename scalar_t>
void outer_product_scatter_add_vjp_vjp(MOPS_OPSA_VJP_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    // same state as the reference's device path (mops/src/opsa/opsa.cu:305-318)
    throw std::runtime_error("Not implemented");
}

template <typename scalar_t>
void outer_product_scatter_add_with_weights(MOPS_OPSAW_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    const char* operation = "cuda_outer_product_scatter_add_with_weights";
    checks::Validator validator(operation);
    checks::opsaw(validator, output, A, B, W, indices_W, indices_output);
    amd::validate_scatter_index(indices_output, output.shape[0], "indices_output", operation);
    amd::validate_gather_index(indices_W, output.shape[0], "indices_W", operation);
    amd::launch_forward<scalar_t, true>(output, A, B, W.data, indices_W.data, indices_output, operation);
}

template <typename scalar_t>
void outer_product_scatter_add_with_weights_vjp(MOPS_OPSAW_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    const char* operation = "cuda_outer_product_scatter_add_with_weights_vjp";
    checks::Validator validator(operation);
    checks::opsaw_vjp(validator, grad_A, grad_B, grad_W, grad_output, A, B, W, indices_W, indices_output);
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
