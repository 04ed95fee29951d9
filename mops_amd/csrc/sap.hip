// Sparse accumulation of products (SAP), forward and vector-Jacobian product,
// for gfx950.
//
//   O[i, PO[k]] += C[k] * A[i, PA[k]] * B[i, PB[k]]
//
// Semantics restated from mops/src/sap/cpu.tpp:10-255 of lab-cosmo/mops
// (formula, evaluation as (C*A)*B, optional gradients, PO need not be sorted).
//
// Batch-parallel: a lane owns one batch row i. A workgroup takes 64
// consecutive rows; their A, B (and grad_output) rows are loaded with
// coalesced accesses and kept in LDS TRANSPOSED ([feature][row], odd row
// stride) so that "feature PA[k] of my row" is one conflict-free LDS read
// whose feature index is the same for the whole wavefront. The table entries
// (C, PA, PB, PO) are wave-uniform and are fetched through the scalar cache.
// The waves of a workgroup split the table into contiguous ranges and keep
// private partial results in LDS, which are added in wave order at the end,
// so the result does not depend on scheduling. Unlike the reference's CUDA
// kernel (mops/src/sap/sap.cu:41-43,69-71) indices are not packed into 8
// bits, so feature counts above 255 work.
#include <algorithm>

#include "mops/sap.hpp"

#include "checks.hpp"
#include "device_common.hpp"
#include "index_validation.hpp"
#include "runtime.hpp"

namespace mops::amd {
namespace {

constexpr int ROWS = WAVE;            // batch rows per workgroup (one per lane)
constexpr int ROW_STRIDE = ROWS + 1;  // odd: transposing stores hit distinct banks
constexpr size_t LDS_BUDGET = 60 * 1024;

// Copy `rows` x `features` elements starting at `source` (row-major, rows
// contiguous) into LDS as [feature][row].
template <typename T>
__device__ __forceinline__ void stage_transposed(
    T* __restrict__ stage, const T* __restrict__ source, int32_t rows, int32_t features
) {
    for (int32_t i = threadIdx.x; i < rows * features; i += blockDim.x) {
        int32_t r = i / features;
        int32_t f = i - r * features;
        stage[f * ROW_STRIDE + r] = source[i];
    }
}

// ---------------------------------------------------------------------------
// forward
// LDS: a[nA][65] b[nB][65] partial[waves][nO][64]
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(1024) void forward_kernel(
    T* __restrict__ output,
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
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    T* a_stage = reinterpret_cast<T*>(lds_bytes);
    T* b_stage = a_stage + static_cast<size_t>(nA) * ROW_STRIDE;
    T* partial = b_stage + static_cast<size_t>(nB) * ROW_STRIDE;

    const int32_t row0 = blockIdx.x * ROWS;
    const int32_t rows = min(ROWS, n_rows - row0);
    const int lane = threadIdx.x % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int waves = blockDim.x / WAVE;

    stage_transposed(a_stage, A + static_cast<size_t>(row0) * nA, rows, nA);
    stage_transposed(b_stage, B + static_cast<size_t>(row0) * nB, rows, nB);
    T* mine = partial + static_cast<size_t>(wave) * nO * ROWS;
    for (int32_t i = lane; i < nO * ROWS; i += WAVE) {
        mine[i] = T(0);
    }
    __syncthreads();

    // contiguous share of the table for this wave
    const int32_t per_wave = (n_products + waves - 1) / waves;
    const int32_t k_begin = min(wave * per_wave, n_products);
    const int32_t k_end = min(k_begin + per_wave, n_products);

    // Entries are applied in ascending k. While consecutive entries name the
    // same output column the sum stays in a register.
    T running = T(0);
    int32_t running_column = -1;
    for (int32_t k = k_begin; k < k_end; k++) {
        const int32_t pa = PA[k];
        const int32_t pb = PB[k];
        const int32_t po = PO[k];
        if (!(in_bounds(pa, nA) && in_bounds(pb, nB) && in_bounds(po, nO))) {
            continue; // wave-uniform
        }
        if (po != running_column) {
            if (running_column >= 0) {
                mine[running_column * ROWS + lane] += running;
            }
            running = T(0);
            running_column = po;
        }
        const T a = a_stage[pa * ROW_STRIDE + lane];
        const T b = b_stage[pb * ROW_STRIDE + lane];
        running += (C[k] * a) * b;
    }
    if (running_column >= 0) {
        mine[running_column * ROWS + lane] += running;
    }
    __syncthreads();

    // add the waves' partial tiles in wave order and write [row][column]
    for (int32_t i = threadIdx.x; i < rows * nO; i += blockDim.x) {
        int32_t r = i / nO;
        int32_t column = i - r * nO;
        T sum = T(0);
        for (int w = 0; w < waves; w++) {
            sum += partial[(static_cast<size_t>(w) * nO + column) * ROWS + r];
        }
        output[static_cast<size_t>(row0) * nO + i] = sum;
    }
}

// ---------------------------------------------------------------------------
// vjp
//   grad_A[i, PA[k]] += (C[k] * G[i, PO[k]]) * B[i, PB[k]]
//   grad_B[i, PB[k]] += (C[k] * G[i, PO[k]]) * A[i, PA[k]]
// LDS: g[nO][65] a[nA][65] b[nB][65] partial_A[waves][nA][64] partial_B[waves][nB][64]
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(1024) void vjp_kernel(
    T* __restrict__ grad_A,
    T* __restrict__ grad_B,
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
    extern __shared__ __align__(16) unsigned char lds_bytes[];
    const bool want_A = grad_A != nullptr;
    const bool want_B = grad_B != nullptr;
    const int waves = blockDim.x / WAVE;

    T* g_stage = reinterpret_cast<T*>(lds_bytes);
    T* a_stage = g_stage + static_cast<size_t>(nO) * ROW_STRIDE;
    T* b_stage = a_stage + static_cast<size_t>(nA) * ROW_STRIDE;
    T* partial_A = b_stage + static_cast<size_t>(nB) * ROW_STRIDE;
    T* partial_B = partial_A + (want_A ? static_cast<size_t>(waves) * nA * ROWS : 0);

    const int32_t row0 = blockIdx.x * ROWS;
    const int32_t rows = min(ROWS, n_rows - row0);
    const int lane = threadIdx.x % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);

    stage_transposed(g_stage, grad_output + static_cast<size_t>(row0) * nO, rows, nO);
    stage_transposed(a_stage, A + static_cast<size_t>(row0) * nA, rows, nA);
    stage_transposed(b_stage, B + static_cast<size_t>(row0) * nB, rows, nB);
    T* mine_A = partial_A + static_cast<size_t>(wave) * nA * ROWS;
    T* mine_B = partial_B + static_cast<size_t>(wave) * nB * ROWS;
    if (want_A) {
        for (int32_t i = lane; i < nA * ROWS; i += WAVE) {
            mine_A[i] = T(0);
        }
    }
    if (want_B) {
        for (int32_t i = lane; i < nB * ROWS; i += WAVE) {
            mine_B[i] = T(0);
        }
    }
    __syncthreads();

    const int32_t per_wave = (n_products + waves - 1) / waves;
    const int32_t k_begin = min(wave * per_wave, n_products);
    const int32_t k_end = min(k_begin + per_wave, n_products);

    for (int32_t k = k_begin; k < k_end; k++) {
        const int32_t pa = PA[k];
        const int32_t pb = PB[k];
        const int32_t po = PO[k];
        if (!(in_bounds(pa, nA) && in_bounds(pb, nB) && in_bounds(po, nO))) {
            continue;
        }
        const T common = C[k] * g_stage[po * ROW_STRIDE + lane];
        if (want_A) {
            mine_A[pa * ROWS + lane] += common * b_stage[pb * ROW_STRIDE + lane];
        }
        if (want_B) {
            mine_B[pb * ROWS + lane] += common * a_stage[pa * ROW_STRIDE + lane];
        }
    }
    __syncthreads();

    if (want_A) {
        for (int32_t i = threadIdx.x; i < rows * nA; i += blockDim.x) {
            int32_t r = i / nA;
            int32_t column = i - r * nA;
            T sum = T(0);
            for (int w = 0; w < waves; w++) {
                sum += partial_A[(static_cast<size_t>(w) * nA + column) * ROWS + r];
            }
            grad_A[static_cast<size_t>(row0) * nA + i] = sum;
        }
    }
    if (want_B) {
        for (int32_t i = threadIdx.x; i < rows * nB; i += blockDim.x) {
            int32_t r = i / nB;
            int32_t column = i - r * nB;
            T sum = T(0);
            for (int w = 0; w < waves; w++) {
                sum += partial_B[(static_cast<size_t>(w) * nB + column) * ROWS + r];
            }
            grad_B[static_cast<size_t>(row0) * nB + i] = sum;
        }
    }
}

// ---------------------------------------------------------------------------
// Fallbacks for feature counts whose tiles do not fit in LDS: one thread per
// batch row, accumulating straight into the row of the result in global
// memory (a row belongs to one thread, so there is no race and the order of
// additions is the table order).
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

// Waves per workgroup: enough that the whole launch has a few thousand
// waves in flight, limited by the LDS the private partial tiles need.
template <typename T>
int pick_waves(size_t n_blocks, size_t shared_elements, size_t per_wave_elements) {
    if ((shared_elements + per_wave_elements) * sizeof(T) > LDS_BUDGET) {
        return 0; // does not fit: use the global-memory kernel
    }
    size_t by_lds = (LDS_BUDGET - shared_elements * sizeof(T)) / (per_wave_elements * sizeof(T));
    size_t wanted = std::max<size_t>(1, 4096 / std::max<size_t>(n_blocks, 1));
    size_t waves = std::min<size_t>({wanted, by_lds, 16});
    return static_cast<int>(std::max<size_t>(waves, 1));
}

} // namespace
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
    const size_t n_blocks = ceil_div(static_cast<size_t>(n_rows), ROWS);
    const size_t shared_elements = (static_cast<size_t>(nA) + nB) * ROW_STRIDE;
    const size_t per_wave = static_cast<size_t>(nO) * ROWS;
    int waves = pick_waves<scalar_t>(n_blocks, shared_elements, std::max<size_t>(per_wave, 1));
    if (waves > 0) {
        size_t lds = (shared_elements + waves * per_wave) * sizeof(scalar_t);
        forward_kernel<scalar_t><<<static_cast<unsigned>(n_blocks), waves * WAVE, lds, current_stream()>>>(
            output.data, A.data, B.data, C.data, indices_A.data, indices_B.data, indices_output.data,
            n_rows, nA, nB, nO, n_products
        );
    } else {
        unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<size_t>(n_rows), 256));
        forward_global_kernel<scalar_t><<<blocks, 256, 0, current_stream()>>>(
            output.data, A.data, B.data, C.data, indices_A.data, indices_B.data, indices_output.data,
            n_rows, nA, nB, nO, n_products
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
    const size_t n_blocks = ceil_div(static_cast<size_t>(n_rows), ROWS);
    const size_t shared_elements = (static_cast<size_t>(nO) + nA + nB) * ROW_STRIDE;
    const size_t per_wave =
        ((want_A ? static_cast<size_t>(nA) : 0) + (want_B ? static_cast<size_t>(nB) : 0)) * ROWS;
    // how the table is split over waves fixes the order of the additions: size
    // the split as if both gradients were requested, so that a gradient has
    // the same bits whether or not the other one is computed alongside
    const size_t per_wave_both = (static_cast<size_t>(nA) + nB) * ROWS;
    int waves = pick_waves<scalar_t>(n_blocks, shared_elements, std::max<size_t>(per_wave_both, 1));
    // the grid depends on the batch size only, whichever gradients are
    // requested (the reference sizes it from grad_A and launches nothing when
    // only grad_B is wanted, mops/src/sap/sap.cu:300)
    if (waves > 0) {
        size_t lds = (shared_elements + waves * per_wave) * sizeof(scalar_t);
        vjp_kernel<scalar_t><<<static_cast<unsigned>(n_blocks), waves * WAVE, lds, current_stream()>>>(
            grad_A.data, grad_B.data, grad_output.data, A.data, B.data, C.data, indices_A.data,
            indices_B.data, indices_output.data, n_rows, nA, nB, nO, n_products
        );
    } else {
        unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<size_t>(n_rows), 256));
        vjp_global_kernel<scalar_t><<<blocks, 256, 0, current_stream()>>>(
            grad_A.data, grad_B.data, grad_output.data, A.data, B.data, C.data, indices_A.data,
            indices_B.data, indices_output.data, n_rows, nA, nB, nO, n_products
        );
    }
    finish_call(operation);
}

template <typename scalar_t>
void sparse_accumulation_of_products_vjp_vjp(MOPS_SAP_VJP_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    throw std::runtime_error("Not implemented");
}

MOPS_CXX_INSTANTIATE(sparse_accumulation_of_products, MOPS_SAP_PARAMS)
MOPS_CXX_INSTANTIATE(sparse_accumulation_of_products_vjp, MOPS_SAP_VJP_PARAMS)
MOPS_CXX_INSTANTIATE(sparse_accumulation_of_products_vjp_vjp, MOPS_SAP_VJP_VJP_PARAMS)

} // namespace mops::cuda
