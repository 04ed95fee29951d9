// TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
//
// A CPU restatement of the reference's host algorithms for the five mops
// operations and their vector-Jacobian products. It exists so that the HIP
// kernels can be checked against an independent implementation of the same
// mathematics on the machine that has the GPU, and so that a CPU baseline
// can be timed next to them. Only the test-suite, the smoke test and the
// benchmark's CPU-baseline leg may load it; the product library never does.
//
// What it follows (lab-cosmo/mops, paths relative to that repository):
//   bucket_rows            mops/src/internal/utils.cpp:7-14   (get_write_list)
//   interleave/deinterleave mops/src/internal/utils.hpp:33-94
//   hpe / hpe_vjp          mops/src/hpe/cpu.tpp:13-74, 133-215
//   sap / sap_vjp          mops/src/sap/cpu.tpp:10-92, 95-255
//   opsa / opsa_vjp        mops/src/opsa/cpu.tpp:9-53, 55-112
//   opsaw / opsaw_vjp      mops/src/opsaw/cpu.tpp:9-54, 57-131
//   sasaw / sasaw_vjp      mops/src/sasaw/cpu.tpp:8-72, 75-171
//   hpe / sap / opsa _vjp_vjp   mops/src/hpe/cpu.tpp:275-539, sap/cpu.tpp:257-541,
//                               opsa/cpu.tpp:114-246
// The loop structure is the reference's: HPE and SAP re-lay the batch axis
// into blocks of `lanes` rows ([block][feature][lane], lanes = 256 bits /
// element size) and run an OpenMP loop over blocks with a serial remainder;
// the scatter operations bucket the input rows by destination and run an
// OpenMP loop over destinations, visiting each bucket in ascending row order;
// the vjps of OPSAW and SASAW bucket by the weight index instead. Products are
// associated as in the reference ((c*a)*b, (g*c)*b*w, ...), so results agree
// with it to rounding of the last bit on the same inputs.
//
// How it is pinned (tests/test_oracle.py): against closed forms that do not
// share code with it -- dense einsum / index_add formulations in numpy,
// order-0 and order-1 polynomials, single-segment inputs that reduce to a
// matrix product, finite differences and the adjoint identity for every vjp,
// and empty segments; the second-order functions against central differences
// of the (pinned) vjps through the adjoint identity, and against torch's double
// backward of the dense formulations (golden vectors). The compiled reference itself is not available to this
// build (it needs a CMake-generated header), so "equal to the reference" is
// established through those mathematical pins, not by running it.
//
// The C entry points mirror the product's C ABI with the prefix
// "mops_oracle_" in place of "mops_" (same by-value tensor structs, same
// argument order, same status convention), so one ctypes marshalling layer
// serves both libraries.
#include <algorithm>
#include <cstddef>
#include <cstdint>
#include <exception>
#include <stdexcept>
#include <string>
#include <vector>

#include "mops/detail/signatures.h"
#include "mops/tensor.h"
#include "mops/tensor.hpp"

namespace oracle {

using mops::Tensor;

// ---- row buckets: for each destination, the input rows that go there -------
struct Buckets {
    std::vector<size_t> begin; // [n_buckets + 1]
    std::vector<size_t> rows;  // input row numbers, ascending inside a bucket
};

static Buckets bucket_rows(const int32_t* destination, size_t n_rows, size_t n_buckets) {
    Buckets b;
    b.begin.assign(n_buckets + 1, 0);
    for (size_t j = 0; j < n_rows; j++) {
        b.begin[static_cast<size_t>(destination[j]) + 1]++;
    }
    for (size_t v = 0; v < n_buckets; v++) {
        b.begin[v + 1] += b.begin[v];
    }
    b.rows.resize(n_rows);
    std::vector<size_t> cursor(b.begin.begin(), b.begin.end() - 1);
    for (size_t j = 0; j < n_rows; j++) {
        b.rows[cursor[static_cast<size_t>(destination[j])]++] = j;
    }
    return b;
}

// ---- batch re-layout --------------------------------------------------------
template <typename T> constexpr size_t lanes_of() { return 32 / sizeof(T); }

// [n, f] -> blocks [n / lanes][f][lanes] and a remainder [f][n % lanes]
template <typename T> struct Blocked {
    size_t n, f, full, rest;
    std::vector<T> blocks, tail;

    Blocked(size_t n_, size_t f_) : n(n_), f(f_) {
        constexpr size_t w = lanes_of<T>();
        full = n / w;
        rest = n % w;
        blocks.assign(full * f * w, T(0));
        tail.assign(rest * f, T(0));
    }

    void load(const T* source) {
        constexpr size_t w = lanes_of<T>();
#pragma omp parallel for
        for (size_t b = 0; b < full; b++) {
            for (size_t c = 0; c < f; c++) {
                for (size_t lane = 0; lane < w; lane++) {
                    blocks[(b * f + c) * w + lane] = source[(b * w + lane) * f + c];
                }
            }
        }
        for (size_t c = 0; c < f; c++) {
            for (size_t lane = 0; lane < rest; lane++) {
                tail[c * rest + lane] = source[(full * w + lane) * f + c];
            }
        }
    }

    void store(T* target) const {
        constexpr size_t w = lanes_of<T>();
#pragma omp parallel for
        for (size_t b = 0; b < full; b++) {
            for (size_t c = 0; c < f; c++) {
                for (size_t lane = 0; lane < w; lane++) {
                    target[(b * w + lane) * f + c] = blocks[(b * f + c) * w + lane];
                }
            }
        }
        for (size_t c = 0; c < f; c++) {
            for (size_t lane = 0; lane < rest; lane++) {
                target[(full * w + lane) * f + c] = tail[c * rest + lane];
            }
        }
    }
};

// ---------------------------------------------------------------- HPE -------
template <typename scalar_t>
void homogeneous_polynomial_evaluation(MOPS_HPE_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using T = scalar_t;
    constexpr size_t w = lanes_of<T>();
    const size_t n = A.shape[0], nA = A.shape[1];
    const size_t J = indices_A.shape[0], K = indices_A.shape[1];
    if (K > 10) {
        throw std::runtime_error(
            "Only up to polynomial order 10 is supported at the moment. Please contact the "
            "developers for more"
        );
    }
    Blocked<T> a(n, nA);
    a.load(A.data);
    const int32_t* P = indices_A.data;

#pragma omp parallel for
    for (size_t b = 0; b < a.full; b++) {
        T acc[w];
        for (size_t lane = 0; lane < w; lane++) {
            acc[lane] = T(0);
        }
        const T* ab = a.blocks.data() + b * nA * w;
        for (size_t j = 0; j < J; j++) {
            T term[w];
            for (size_t lane = 0; lane < w; lane++) {
                term[lane] = C.data[j];
            }
            for (size_t k = 0; k < K; k++) {
                const T* factor = ab + static_cast<size_t>(P[j * K + k]) * w;
                for (size_t lane = 0; lane < w; lane++) {
                    term[lane] *= factor[lane];
                }
            }
            for (size_t lane = 0; lane < w; lane++) {
                acc[lane] += term[lane];
            }
        }
        for (size_t lane = 0; lane < w; lane++) {
            output.data[b * w + lane] = acc[lane];
        }
    }
    for (size_t lane = 0; lane < a.rest; lane++) {
        T acc = T(0);
        for (size_t j = 0; j < J; j++) {
            T term = C.data[j];
            for (size_t k = 0; k < K; k++) {
                term *= a.tail[static_cast<size_t>(P[j * K + k]) * a.rest + lane];
            }
            acc += term;
        }
        output.data[a.full * w + lane] = acc;
    }
}

template <typename scalar_t>
void homogeneous_polynomial_evaluation_vjp(MOPS_HPE_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using T = scalar_t;
    if (grad_A.data == nullptr) {
        return;
    }
    constexpr size_t w = lanes_of<T>();
    const size_t n = A.shape[0], nA = A.shape[1];
    const size_t J = indices_A.shape[0], K = indices_A.shape[1];
    if (K > 10) {
        throw std::runtime_error(
            "Only up to polynomial order 10 is supported at the moment. Please contact the "
            "developers for more"
        );
    }
    Blocked<T> a(n, nA), g(n, nA);
    a.load(A.data);
    const int32_t* P = indices_A.data;

#pragma omp parallel for
    for (size_t b = 0; b < a.full; b++) {
        const T* ab = a.blocks.data() + b * nA * w;
        T* gb = g.blocks.data() + b * nA * w;
        const T* upstream = grad_output.data + b * w;
        for (size_t j = 0; j < J; j++) {
            T base[w];
            for (size_t lane = 0; lane < w; lane++) {
                base[lane] = C.data[j] * upstream[lane];
            }
            for (size_t f = 0; f < K; f++) {
                T term[w];
                for (size_t lane = 0; lane < w; lane++) {
                    term[lane] = base[lane];
                }
                for (size_t k = 0; k < K; k++) {
                    if (k == f) {
                        continue;
                    }
                    const T* factor = ab + static_cast<size_t>(P[j * K + k]) * w;
                    for (size_t lane = 0; lane < w; lane++) {
                        term[lane] *= factor[lane];
                    }
                }
                T* target = gb + static_cast<size_t>(P[j * K + f]) * w;
                for (size_t lane = 0; lane < w; lane++) {
                    target[lane] += term[lane];
                }
            }
        }
    }
    const T* upstream = grad_output.data + a.full * w;
    for (size_t j = 0; j < J; j++) {
        for (size_t f = 0; f < K; f++) {
            for (size_t lane = 0; lane < a.rest; lane++) {
                T term = C.data[j] * upstream[lane];
                for (size_t k = 0; k < K; k++) {
                    if (k == f) {
                        continue;
                    }
                    term *= a.tail[static_cast<size_t>(P[j * K + k]) * a.rest + lane];
                }
                g.tail[static_cast<size_t>(P[j * K + f]) * a.rest + lane] += term;
            }
        }
    }
    g.store(grad_A.data);
}

// Second-order functions (mops/src/hpe/cpu.tpp:275-460, sap/cpu.tpp:257-541,
// opsa/cpu.tpp:114-246): the vjp of the vjp. Inputs are those of the vjp plus
// the cotangents of its outputs (grad_grad_*); outputs are the cotangents of
// grad_output (grad_grad_output) and of A, B (grad_*_2). They are written row
// by row here (the reference blocks the batch axis as above, which changes
// which rows share a vector register but not the order of any row's sums):
// monomials / table entries / bucket members in ascending order, and inside
// one of them the grad_grad_A term before the grad_grad_B term. A cotangent
// that is not given counts as zero; the reference reads through the null
// pointer in HPE in that case (hpe/cpu.tpp:367-388), which is not followed.
template <typename scalar_t>
void homogeneous_polynomial_evaluation_vjp_vjp(MOPS_HPE_VJP_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using T = scalar_t;
    const size_t n = A.shape[0], nA = A.shape[1];
    const size_t J = indices_A.shape[0], K = indices_A.shape[1];
    if (K > 10) {
        throw std::runtime_error(
            "Only up to polynomial order 10 is supported at the moment. Please contact the "
            "developers for more"
        );
    }
    const bool have = grad_grad_A.data != nullptr;
    const bool want_O = grad_grad_output.data != nullptr, want_A = grad_A_2.data != nullptr;
    const int32_t* P = indices_A.data;
#pragma omp parallel for
    for (size_t i = 0; i < n; i++) {
        const T* a = A.data + i * nA;
        const T* gg = have ? grad_grad_A.data + i * nA : nullptr;
        if (want_O) {
            T sum = T(0);
            for (size_t j = 0; have && j < J; j++) {
                for (size_t f = 0; f < K; f++) {
                    T term = C.data[j] * gg[P[j * K + f]];
                    for (size_t k = 0; k < K; k++) {
                        if (k != f) {
                            term *= a[P[j * K + k]];
                        }
                    }
                    sum += term;
                }
            }
            grad_grad_output.data[i] = sum;
        }
        if (want_A) {
            T* out = grad_A_2.data + i * nA;
            std::fill(out, out + nA, T(0));
            for (size_t j = 0; have && j < J; j++) {
                const T base = C.data[j] * grad_output.data[i];
                for (size_t f2 = 0; f2 < K; f2++) {
                    for (size_t f = 0; f < K; f++) {
                        if (f == f2) {
                            continue;
                        }
                        T term = base * gg[P[j * K + f]];
                        for (size_t k = 0; k < K; k++) {
                            if (k != f && k != f2) {
                                term *= a[P[j * K + k]];
                            }
                        }
                        out[P[j * K + f2]] += term;
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------- SAP -------
template <typename scalar_t>
void sparse_accumulation_of_products(MOPS_SAP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using T = scalar_t;
    constexpr size_t w = lanes_of<T>();
    const size_t n = A.shape[0], nA = A.shape[1], nB = B.shape[1], nO = output.shape[1];
    const size_t K = C.shape[0];
    Blocked<T> a(n, nA), b(n, nB), o(n, nO);
    a.load(A.data);
    b.load(B.data);
    const int32_t *PA = indices_A.data, *PB = indices_B.data, *PO = indices_output.data;

#pragma omp parallel for
    for (size_t blk = 0; blk < a.full; blk++) {
        const T* ab = a.blocks.data() + blk * nA * w;
        const T* bb = b.blocks.data() + blk * nB * w;
        T* ob = o.blocks.data() + blk * nO * w;
        for (size_t k = 0; k < K; k++) {
            const T* av = ab + static_cast<size_t>(PA[k]) * w;
            const T* bv = bb + static_cast<size_t>(PB[k]) * w;
            T* ov = ob + static_cast<size_t>(PO[k]) * w;
            const T c = C.data[k];
            for (size_t lane = 0; lane < w; lane++) {
                ov[lane] += c * av[lane] * bv[lane];
            }
        }
    }
    for (size_t k = 0; k < K; k++) {
        const T c = C.data[k];
        for (size_t lane = 0; lane < a.rest; lane++) {
            o.tail[static_cast<size_t>(PO[k]) * a.rest + lane] +=
                c * a.tail[static_cast<size_t>(PA[k]) * a.rest + lane] *
                b.tail[static_cast<size_t>(PB[k]) * a.rest + lane];
        }
    }
    o.store(output.data);
}

template <typename scalar_t>
void sparse_accumulation_of_products_vjp(MOPS_SAP_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using T = scalar_t;
    const bool want_A = grad_A.data != nullptr, want_B = grad_B.data != nullptr;
    if (!want_A && !want_B) {
        return;
    }
    constexpr size_t w = lanes_of<T>();
    const size_t n = A.shape[0], nA = A.shape[1], nB = B.shape[1], nO = grad_output.shape[1];
    const size_t K = C.shape[0];
    Blocked<T> go(n, nO), a(n, nA), b(n, nB), ga(n, nA), gb(n, nB);
    go.load(grad_output.data);
    a.load(A.data);
    b.load(B.data);
    const int32_t *PA = indices_A.data, *PB = indices_B.data, *PO = indices_output.data;

#pragma omp parallel for
    for (size_t blk = 0; blk < a.full; blk++) {
        const T* gob = go.blocks.data() + blk * nO * w;
        const T* ab = a.blocks.data() + blk * nA * w;
        const T* bb = b.blocks.data() + blk * nB * w;
        T* gab = ga.blocks.data() + blk * nA * w;
        T* gbb = gb.blocks.data() + blk * nB * w;
        for (size_t k = 0; k < K; k++) {
            T common[w];
            const T c = C.data[k];
            const T* gov = gob + static_cast<size_t>(PO[k]) * w;
            for (size_t lane = 0; lane < w; lane++) {
                common[lane] = c * gov[lane];
            }
            if (want_A) {
                T* target = gab + static_cast<size_t>(PA[k]) * w;
                const T* other = bb + static_cast<size_t>(PB[k]) * w;
                for (size_t lane = 0; lane < w; lane++) {
                    target[lane] += common[lane] * other[lane];
                }
            }
            if (want_B) {
                T* target = gbb + static_cast<size_t>(PB[k]) * w;
                const T* other = ab + static_cast<size_t>(PA[k]) * w;
                for (size_t lane = 0; lane < w; lane++) {
                    target[lane] += common[lane] * other[lane];
                }
            }
        }
    }
    const size_t rest = a.rest;
    for (size_t k = 0; k < K; k++) {
        for (size_t lane = 0; lane < rest; lane++) {
            // the remainder loop of the reference associates (g * c)
            const T common = go.tail[static_cast<size_t>(PO[k]) * rest + lane] * C.data[k];
            if (want_A) {
                ga.tail[static_cast<size_t>(PA[k]) * rest + lane] +=
                    common * b.tail[static_cast<size_t>(PB[k]) * rest + lane];
            }
            if (want_B) {
                gb.tail[static_cast<size_t>(PB[k]) * rest + lane] +=
                    common * a.tail[static_cast<size_t>(PA[k]) * rest + lane];
            }
        }
    }
    if (want_A) {
        ga.store(grad_A.data);
    }
    if (want_B) {
        gb.store(grad_B.data);
    }
}

template <typename scalar_t>
void sparse_accumulation_of_products_vjp_vjp(MOPS_SAP_VJP_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using T = scalar_t;
    const size_t n = A.shape[0], nA = A.shape[1], nB = B.shape[1], nO = grad_output.shape[1];
    const size_t K = C.shape[0];
    const bool have_A = grad_grad_A.data != nullptr, have_B = grad_grad_B.data != nullptr;
    const bool want_O = grad_grad_output.data != nullptr;
    const bool want_A = grad_A_2.data != nullptr, want_B = grad_B_2.data != nullptr;
    const int32_t *PA = indices_A.data, *PB = indices_B.data, *PO = indices_output.data;
#pragma omp parallel for
    for (size_t i = 0; i < n; i++) {
        const T* a = A.data + i * nA;
        const T* b = B.data + i * nB;
        const T* g = grad_output.data + i * nO;
        const T* gga = have_A ? grad_grad_A.data + i * nA : nullptr;
        const T* ggb = have_B ? grad_grad_B.data + i * nB : nullptr;
        T* ggo = want_O ? grad_grad_output.data + i * nO : nullptr;
        T* ga2 = want_A ? grad_A_2.data + i * nA : nullptr;
        T* gb2 = want_B ? grad_B_2.data + i * nB : nullptr;
        if (want_O) {
            std::fill(ggo, ggo + nO, T(0));
        }
        if (want_A) {
            std::fill(ga2, ga2 + nA, T(0));
        }
        if (want_B) {
            std::fill(gb2, gb2 + nB, T(0));
        }
        for (size_t k = 0; k < K; k++) {
            const T c = C.data[k];
            if (have_A) {
                if (want_O) {
                    ggo[PO[k]] += c * gga[PA[k]] * b[PB[k]];
                }
                if (want_B) {
                    gb2[PB[k]] += c * gga[PA[k]] * g[PO[k]];
                }
            }
            if (have_B) {
                if (want_O) {
                    ggo[PO[k]] += c * ggb[PB[k]] * a[PA[k]];
                }
                if (want_A) {
                    ga2[PA[k]] += c * ggb[PB[k]] * g[PO[k]];
                }
            }
        }
    }
}

// --------------------------------------------------------------- OPSA -------
template <typename scalar_t>
void outer_product_scatter_add(MOPS_OPSA_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using T = scalar_t;
    const size_t n_out = output.shape[0], K = A.shape[1], L = B.shape[1];
    Buckets buckets = bucket_rows(indices_output.data, A.shape[0], n_out);
    std::fill(output.data, output.data + n_out * K * L, T(0));

#pragma omp parallel for
    for (size_t i = 0; i < n_out; i++) {
        T* o = output.data + i * K * L;
        for (size_t p = buckets.begin[i]; p < buckets.begin[i + 1]; p++) {
            const size_t j = buckets.rows[p];
            const T* a = A.data + j * K;
            const T* b = B.data + j * L;
            for (size_t k = 0; k < K; k++) {
                const T ak = a[k];
                for (size_t l = 0; l < L; l++) {
                    o[k * L + l] += ak * b[l];
                }
            }
        }
    }
}

template <typename scalar_t>
void outer_product_scatter_add_vjp(MOPS_OPSA_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using T = scalar_t;
    const bool want_A = grad_A.data != nullptr, want_B = grad_B.data != nullptr;
    if (!want_A && !want_B) {
        return;
    }
    const size_t J = A.shape[0], K = A.shape[1], L = B.shape[1];
    if (want_A) {
        std::fill(grad_A.data, grad_A.data + J * K, T(0));
    }
    if (want_B) {
        std::fill(grad_B.data, grad_B.data + J * L, T(0));
    }
#pragma omp parallel for
    for (size_t j = 0; j < J; j++) {
        const T* g = grad_output.data + static_cast<size_t>(indices_output.data[j]) * K * L;
        const T* a = A.data + j * K;
        const T* b = B.data + j * L;
        for (size_t k = 0; k < K; k++) {
            for (size_t l = 0; l < L; l++) {
                if (want_A) {
                    grad_A.data[j * K + k] += g[k * L + l] * b[l];
                }
                if (want_B) {
                    grad_B.data[j * L + l] += g[k * L + l] * a[k];
                }
            }
        }
    }
}

template <typename scalar_t>
void outer_product_scatter_add_vjp_vjp(MOPS_OPSA_VJP_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using T = scalar_t;
    const size_t J = A.shape[0], K = A.shape[1], L = B.shape[1], n_out = grad_output.shape[0];
    const bool have_A = grad_grad_A.data != nullptr, have_B = grad_grad_B.data != nullptr;
    const bool want_O = grad_grad_output.data != nullptr;
    const bool want_A = grad_A_2.data != nullptr, want_B = grad_B_2.data != nullptr;
    if (want_A) {
        std::fill(grad_A_2.data, grad_A_2.data + J * K, T(0));
    }
    if (want_B) {
        std::fill(grad_B_2.data, grad_B_2.data + J * L, T(0));
    }
    if (want_O) {
        std::fill(grad_grad_output.data, grad_grad_output.data + n_out * K * L, T(0));
    }
    Buckets buckets = bucket_rows(indices_output.data, J, n_out);
#pragma omp parallel for
    for (size_t i = 0; i < n_out; i++) {
        T* ggo = want_O ? grad_grad_output.data + i * K * L : nullptr;
        const T* g = grad_output.data + i * K * L;
        for (size_t p = buckets.begin[i]; p < buckets.begin[i + 1]; p++) {
            const size_t j = buckets.rows[p];
            const T* a = A.data + j * K;
            const T* b = B.data + j * L;
            if (have_A) {
                const T* gga = grad_grad_A.data + j * K;
                for (size_t k = 0; k < K; k++) {
                    for (size_t l = 0; l < L; l++) {
                        if (want_O) {
                            ggo[k * L + l] += gga[k] * b[l];
                        }
                        if (want_B) {
                            grad_B_2.data[j * L + l] += gga[k] * g[k * L + l];
                        }
                    }
                }
            }
            if (have_B) {
                const T* ggb = grad_grad_B.data + j * L;
                for (size_t k = 0; k < K; k++) {
                    for (size_t l = 0; l < L; l++) {
                        if (want_O) {
                            ggo[k * L + l] += ggb[l] * a[k];
                        }
                        if (want_A) {
                            grad_A_2.data[j * K + k] += ggb[l] * g[k * L + l];
                        }
                    }
                }
            }
        }
    }
}

// -------------------------------------------------------------- OPSAW -------
template <typename scalar_t>
void outer_product_scatter_add_with_weights(MOPS_OPSAW_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using T = scalar_t;
    const size_t n_out = output.shape[0], K = A.shape[1], L = B.shape[1];
    Buckets buckets = bucket_rows(indices_output.data, A.shape[0], n_out);
    std::fill(output.data, output.data + n_out * K * L, T(0));

#pragma omp parallel for
    for (size_t i = 0; i < n_out; i++) {
        T* o = output.data + i * K * L;
        for (size_t p = buckets.begin[i]; p < buckets.begin[i + 1]; p++) {
            const size_t e = buckets.rows[p];
            const T* a = A.data + e * K;
            const T* b = B.data + e * L;
            const T* wt = W.data + static_cast<size_t>(indices_W.data[e]) * L;
            for (size_t k = 0; k < K; k++) {
                const T ak = a[k];
                for (size_t l = 0; l < L; l++) {
                    o[k * L + l] += ak * b[l] * wt[l];
                }
            }
        }
    }
}

template <typename scalar_t>
void outer_product_scatter_add_with_weights_vjp(MOPS_OPSAW_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using T = scalar_t;
    const bool want_A = grad_A.data != nullptr, want_B = grad_B.data != nullptr,
               want_W = grad_W.data != nullptr;
    if (!want_A && !want_B && !want_W) {
        return;
    }
    const size_t E = A.shape[0], K = A.shape[1], L = B.shape[1], n_nodes = W.shape[0];
    if (want_A) {
        std::fill(grad_A.data, grad_A.data + E * K, T(0));
    }
    if (want_B) {
        std::fill(grad_B.data, grad_B.data + E * L, T(0));
    }
    if (want_W) {
        std::fill(grad_W.data, grad_W.data + n_nodes * L, T(0));
    }
    // bucketed by the weight row, so that one thread owns grad_W[j]
    Buckets buckets = bucket_rows(indices_W.data, E, n_nodes);
#pragma omp parallel for
    for (size_t j = 0; j < n_nodes; j++) {
        const T* wt = W.data + j * L;
        for (size_t p = buckets.begin[j]; p < buckets.begin[j + 1]; p++) {
            const size_t e = buckets.rows[p];
            const T* g = grad_output.data + static_cast<size_t>(indices_output.data[e]) * K * L;
            const T* a = A.data + e * K;
            const T* b = B.data + e * L;
            for (size_t k = 0; k < K; k++) {
                const T ak = a[k];
                for (size_t l = 0; l < L; l++) {
                    const T gv = g[k * L + l];
                    if (want_A) {
                        grad_A.data[e * K + k] += gv * b[l] * wt[l];
                    }
                    if (want_B) {
                        grad_B.data[e * L + l] += gv * ak * wt[l];
                    }
                    if (want_W) {
                        grad_W.data[j * L + l] += gv * ak * b[l];
                    }
                }
            }
        }
    }
}

// -------------------------------------------------------------- SASAW -------
template <typename scalar_t>
void sparse_accumulation_scatter_add_with_weights(MOPS_SASAW_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using T = scalar_t;
    const size_t n_nodes = output.shape[0], n3 = output.shape[1], L = output.shape[2];
    const size_t nA = A.shape[1], n2 = W.shape[1], N = C.shape[0];
    Buckets buckets = bucket_rows(indices_output_1.data, A.shape[0], n_nodes);
    std::fill(output.data, output.data + n_nodes * n3 * L, T(0));

#pragma omp parallel for
    for (size_t i = 0; i < n_nodes; i++) {
        for (size_t p = buckets.begin[i]; p < buckets.begin[i + 1]; p++) {
            const size_t e = buckets.rows[p];
            T* o = output.data + static_cast<size_t>(indices_output_1.data[e]) * n3 * L;
            const T* a = A.data + e * nA;
            const T* b = B.data + e * L;
            const T* wt = W.data + static_cast<size_t>(indices_W_1.data[e]) * n2 * L;
            for (size_t n = 0; n < N; n++) {
                const T ca = C.data[n] * a[indices_A.data[n]];
                T* on = o + static_cast<size_t>(indices_output_2.data[n]) * L;
                const T* wn = wt + static_cast<size_t>(indices_W_2.data[n]) * L;
                for (size_t l = 0; l < L; l++) {
                    on[l] += ca * b[l] * wn[l];
                }
            }
        }
    }
}

template <typename scalar_t>
void sparse_accumulation_scatter_add_with_weights_vjp(MOPS_SASAW_VJP_PARAMS(MOPS_CXX_FIRST, MOPS_CXX_NEXT)) {
    using T = scalar_t;
    const bool want_A = grad_A.data != nullptr, want_B = grad_B.data != nullptr,
               want_W = grad_W.data != nullptr;
    if (!want_A && !want_B && !want_W) {
        return;
    }
    const size_t n_nodes = grad_output.shape[0], n3 = grad_output.shape[1], L = grad_output.shape[2];
    const size_t E = A.shape[0], nA = A.shape[1], n2 = W.shape[1], N = C.shape[0];
    if (want_A) {
        std::fill(grad_A.data, grad_A.data + E * nA, T(0));
    }
    if (want_B) {
        std::fill(grad_B.data, grad_B.data + E * L, T(0));
    }
    if (want_W) {
        std::fill(grad_W.data, grad_W.data + n_nodes * n2 * L, T(0));
    }
    Buckets buckets = bucket_rows(indices_W_1.data, E, n_nodes);
#pragma omp parallel for
    for (size_t j = 0; j < n_nodes; j++) {
        const T* wt = W.data + j * n2 * L;
        for (size_t p = buckets.begin[j]; p < buckets.begin[j + 1]; p++) {
            const size_t e = buckets.rows[p];
            const T* g = grad_output.data + static_cast<size_t>(indices_output_1.data[e]) * n3 * L;
            const T* a = A.data + e * nA;
            const T* b = B.data + e * L;
            for (size_t n = 0; n < N; n++) {
                const T c = C.data[n];
                const size_t m1 = static_cast<size_t>(indices_A.data[n]);
                const size_t m2 = static_cast<size_t>(indices_W_2.data[n]);
                const T ca = c * a[m1];
                const T* gn = g + static_cast<size_t>(indices_output_2.data[n]) * L;
                const T* wn = wt + m2 * L;
                for (size_t l = 0; l < L; l++) {
                    const T gv = gn[l];
                    if (want_A) {
                        grad_A.data[e * nA + m1] += gv * c * b[l] * wn[l];
                    }
                    if (want_B) {
                        grad_B.data[e * L + l] += gv * ca * wn[l];
                    }
                    if (want_W) {
                        grad_W.data[(j * n2 + m2) * L + l] += gv * ca * b[l];
                    }
                }
            }
        }
    }
}

// No second-order function exists for the two weighted operations
// (mops/src/opsaw/cpu.tpp:133-150, mops/src/sasaw/cpu.tpp:173-194: "Not implemented").

} // namespace oracle

// ---- C entry points ---------------------------------------------------------
namespace {

thread_local std::string LAST_ERROR;

#define ORACLE_DEFINE_VIEW(STRUCT, ELEMENT)                                                        \
    [[maybe_unused]] mops::Tensor<ELEMENT, sizeof(STRUCT::shape) / sizeof(int64_t)> view(STRUCT t) { \
        constexpr size_t N = sizeof(STRUCT::shape) / sizeof(int64_t);                              \
        mops::Tensor<ELEMENT, N> result;                                                           \
        result.data = t.data;                                                                      \
        for (size_t d = 0; d < N; d++) {                                                           \
            result.shape[d] = static_cast<size_t>(t.shape[d]);                                     \
        }                                                                                          \
        return result;                                                                             \
    }

ORACLE_DEFINE_VIEW(mops_tensor_1d_f32_t, float)
ORACLE_DEFINE_VIEW(mops_tensor_2d_f32_t, float)
ORACLE_DEFINE_VIEW(mops_tensor_3d_f32_t, float)
ORACLE_DEFINE_VIEW(mops_tensor_1d_f64_t, double)
ORACLE_DEFINE_VIEW(mops_tensor_2d_f64_t, double)
ORACLE_DEFINE_VIEW(mops_tensor_3d_f64_t, double)
ORACLE_DEFINE_VIEW(mops_tensor_1d_i32_t, int32_t)
ORACLE_DEFINE_VIEW(mops_tensor_2d_i32_t, int32_t)

} // namespace

#define ORACLE_EXPORT extern "C" __attribute__((visibility("default")))
#define ORACLE_FIRST(KIND, NAME) view(NAME)
#define ORACLE_NEXT(KIND, NAME) , view(NAME)

#define ORACLE_C_DEFINE(NAME, S, T, PARAMS)                                                        \
    ORACLE_EXPORT int mops_oracle_##NAME##_##S(PARAMS(MOPS_C_FIRST_##S, MOPS_C_NEXT_##S)) {        \
        try {                                                                                      \
            oracle::NAME<T>(PARAMS(ORACLE_FIRST, ORACLE_NEXT));                                    \
            return 0;                                                                              \
        } catch (const std::exception& caught) {                                                   \
            LAST_ERROR = caught.what();                                                            \
            return 1;                                                                              \
        } catch (...) {                                                                            \
            LAST_ERROR = "unknown error";                                                          \
            return 2;                                                                              \
        }                                                                                          \
    }

#define ORACLE_C_DEFINE_BOTH(NAME, PARAMS)                                                         \
    ORACLE_C_DEFINE(NAME, f32, float, PARAMS)                                                      \
    ORACLE_C_DEFINE(NAME, f64, double, PARAMS)

ORACLE_C_DEFINE_BOTH(homogeneous_polynomial_evaluation, MOPS_HPE_PARAMS)
ORACLE_C_DEFINE_BOTH(homogeneous_polynomial_evaluation_vjp, MOPS_HPE_VJP_PARAMS)
ORACLE_C_DEFINE_BOTH(sparse_accumulation_of_products, MOPS_SAP_PARAMS)
ORACLE_C_DEFINE_BOTH(sparse_accumulation_of_products_vjp, MOPS_SAP_VJP_PARAMS)
ORACLE_C_DEFINE_BOTH(outer_product_scatter_add, MOPS_OPSA_PARAMS)
ORACLE_C_DEFINE_BOTH(outer_product_scatter_add_vjp, MOPS_OPSA_VJP_PARAMS)
ORACLE_C_DEFINE_BOTH(outer_product_scatter_add_with_weights, MOPS_OPSAW_PARAMS)
ORACLE_C_DEFINE_BOTH(outer_product_scatter_add_with_weights_vjp, MOPS_OPSAW_VJP_PARAMS)
ORACLE_C_DEFINE_BOTH(sparse_accumulation_scatter_add_with_weights, MOPS_SASAW_PARAMS)
ORACLE_C_DEFINE_BOTH(sparse_accumulation_scatter_add_with_weights_vjp, MOPS_SASAW_VJP_PARAMS)
ORACLE_C_DEFINE_BOTH(homogeneous_polynomial_evaluation_vjp_vjp, MOPS_HPE_VJP_VJP_PARAMS)
ORACLE_C_DEFINE_BOTH(sparse_accumulation_of_products_vjp_vjp, MOPS_SAP_VJP_VJP_PARAMS)
ORACLE_C_DEFINE_BOTH(outer_product_scatter_add_vjp_vjp, MOPS_OPSA_VJP_VJP_PARAMS)

ORACLE_EXPORT const char* mops_oracle_get_last_error_message(void) { return LAST_ERROR.c_str(); }

// first_occurrences on the host, by definition: lower/upper bound of every
// value in the sorted vector, -1/-1 when absent (the contract documented at
// mops/src/internal/cuda_first_occurences.cu:82-117 and .cuh:7-9).
ORACLE_EXPORT int mops_oracle_first_occurrences(
    const int32_t* sorted_indices, int64_t n_input, int64_t n_output, int32_t* result
) {
    for (int64_t v = 0; v < n_output; v++) {
        const int32_t* lo =
            std::lower_bound(sorted_indices, sorted_indices + n_input, static_cast<int32_t>(v));
        const int32_t* hi =
            std::upper_bound(sorted_indices, sorted_indices + n_input, static_cast<int32_t>(v));
        if (lo == hi) {
            result[v] = -1;
            result[n_output + v] = -1;
        } else {
            result[v] = static_cast<int32_t>(lo - sorted_indices);
            result[n_output + v] = static_cast<int32_t>(hi - sorted_indices);
        }
    }
    return 0;
}

// OpenMP threads the oracle will use (for the benchmark's "cores" field).
#ifdef _OPENMP
#include <omp.h>
ORACLE_EXPORT int mops_oracle_num_threads(void) { return omp_get_max_threads(); }
ORACLE_EXPORT void mops_oracle_set_num_threads(int threads) { omp_set_num_threads(threads < 1 ? 1 : threads); }
#else
ORACLE_EXPORT int mops_oracle_num_threads(void) { return 1; }
ORACLE_EXPORT void mops_oracle_set_num_threads(int) {}
#endif
