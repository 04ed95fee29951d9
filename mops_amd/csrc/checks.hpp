// Argument validation for the fifteen operations.
//
// The wording and the ORDER of the tests are part of the interface: callers'
// test suites match the message text (python/mops/tests/opsa.py:66-90 of
// lab-cosmo/mops and its siblings). The rules below restate
// mops/src/internal/checks/utils.hpp:21-103 and
// mops/src/internal/checks/{hpe,sap,opsa,opsaw,sasaw}.hpp:
//
//  * extents are compared pairwise in a fixed sequence, first failure wins;
//  * index tensors are range-checked only when the operation name does not
//    start with "cuda_" (the values of a device tensor are not readable from
//    the host without a copy);
//  * an optional gradient is checked only when its data pointer is non-null.
//
// Known oddities that are kept because the text is observable:
//  * HPE reports its output under the name "grad_output" (checks/hpe.hpp:16);
//  * SASAW bounds indices_W_2 by B.shape[1] (checks/sasaw.hpp:33);
//  * OPSAW and SASAW require W.shape[0] == output.shape[0];
//  * the negative-index message has no blank in "negative-valuedindices".
#ifndef MOPS_AMD_CHECKS_HPP
#define MOPS_AMD_CHECKS_HPP

#include <algorithm>
#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>

#include "mops/tensor.hpp"

namespace mops::checks {

/// One axis of a named tensor.
struct Axis {
    const char* tensor;
    size_t axis;
    size_t extent;
};

template <typename T, size_t N> Axis axis_of(const Tensor<T, N>& tensor, const char* name, size_t axis) {
    return Axis{name, axis, tensor.shape[axis]};
}

class Validator {
  public:
    explicit Validator(std::string operation) : operation_(std::move(operation)) {}

    /// Index values can be inspected from the host.
    bool host_indices() const { return operation_.rfind("cuda_", 0) != 0; }

    const std::string& operation() const { return operation_; }

    void same_extent(Axis first, Axis second) const {
        if (first.extent != second.extent) {
            throw std::runtime_error(
                std::string("Dimension mismatch: the sizes of ") + first.tensor +
                " along dimension " + std::to_string(first.axis) + " and " + second.tensor +
                " along dimension " + std::to_string(second.axis) + " must match in " + operation_
            );
        }
    }

    /// Every element of `indices` must lie in [0, bound).
    template <size_t N>
    void index_range(const Tensor<int32_t, N>& indices, const char* name, size_t bound) const {
        size_t count = 1;
        for (size_t d = 0; d < N; d++) {
            count *= indices.shape[d];
        }
        if (count == 0) {
            return;
        }
        auto extremes = std::minmax_element(indices.data, indices.data + count);
        int32_t smallest = *extremes.first;
        int32_t largest = *extremes.second;
        if (largest >= static_cast<int32_t>(bound)) {
            throw std::runtime_error(
                std::string("Index array ") + name + " in operation " + operation_ +
                " contains elements up to " + std::to_string(largest) +
                "; this would cause out-of-bounds accesses. With the " +
                "provided parameters, it can only contain elements up to " +
                std::to_string(bound - 1)
            );
        }
        if (smallest < 0) {
            throw std::runtime_error(
                std::string("Index array ") + name + " in operation " + operation_ +
                " contains negative-valued" + "indices"
            );
        }
    }

    /// A requested gradient must have the shape of the tensor it belongs to.
    template <typename T, size_t N>
    void gradient_like(
        const Tensor<T, N>& gradient, const char* gradient_name, const Tensor<T, N>& tensor, const char* name
    ) const {
        if (gradient.data == nullptr) {
            return;
        }
        for (size_t d = 0; d < N; d++) {
            same_extent(axis_of(gradient, gradient_name, d), axis_of(tensor, name, d));
        }
    }

  private:
    std::string operation_;
};

/// Element-wise shape equality with the long-form message of
/// mops/src/internal/checks/utils.hpp:86-101.
template <typename T, size_t N>
void same_shape(
    const Tensor<T, N>& first,
    const std::string& first_name,
    const Tensor<T, N>& second,
    const std::string& second_name,
    const std::string& operation
) {
    for (size_t d = 0; d < N; d++) {
        if (first.shape[d] != second.shape[d]) {
            throw std::runtime_error(
                "Dimension mismatch: the sizes of " + first_name + " and " + second_name +
                " must match in " + operation + ", but they are " + std::to_string(first.shape[d]) +
                " and " + std::to_string(second.shape[d]) + " respectively" + " along dimension " +
                std::to_string(d)
            );
        }
    }
}

// ---------------------------------------------------------------- HPE ----
template <typename T>
void hpe(
    const Validator& v, Tensor<T, 1> output, Tensor<T, 2> A, Tensor<T, 1> C, Tensor<int32_t, 2> indices_A
) {
    v.same_extent(axis_of(A, "A", 0), axis_of(output, "grad_output", 0));
    v.same_extent(axis_of(C, "C", 0), axis_of(indices_A, "indices_A", 0));
    if (v.host_indices()) {
        v.index_range(indices_A, "indices_A", A.shape[1]);
    }
}

template <typename T>
void hpe_vjp(
    const Validator& v,
    Tensor<T, 2> grad_A,
    Tensor<T, 1> grad_output,
    Tensor<T, 2> A,
    Tensor<T, 1> C,
    Tensor<int32_t, 2> indices_A
) {
    v.gradient_like(grad_A, "grad_A", A, "A");
    hpe(v, grad_output, A, C, indices_A);
}

template <typename T>
void hpe_vjp_vjp(
    const Validator& v,
    Tensor<T, 1> grad_grad_output,
    Tensor<T, 2> grad_A_2,
    Tensor<T, 2> grad_grad_A,
    Tensor<T, 1> grad_output,
    Tensor<T, 2> A,
    Tensor<T, 1> C,
    Tensor<int32_t, 2> indices_A
) {
    v.gradient_like(grad_grad_output, "grad_grad_output", grad_output, "grad_output");
    v.gradient_like(grad_A_2, "grad_A_2", A, "A");
    v.gradient_like(grad_grad_A, "grad_grad_A", A, "A");
    // the reference revalidates with grad_grad_A in the grad_A slot
    // (checks/hpe.hpp:63), which repeats the same comparison under the name
    // "grad_A"; it can no longer fail here.
    hpe(v, grad_output, A, C, indices_A);
}

// ---------------------------------------------------------------- SAP ----
template <typename T>
void sap(
    const Validator& v,
    Tensor<T, 2> output,
    Tensor<T, 2> A,
    Tensor<T, 2> B,
    Tensor<T, 1> C,
    Tensor<int32_t, 1> indices_A,
    Tensor<int32_t, 1> indices_B,
    Tensor<int32_t, 1> indices_output
) {
    v.same_extent(axis_of(A, "A", 0), axis_of(B, "B", 0));
    v.same_extent(axis_of(A, "A", 0), axis_of(output, "output", 0));
    v.same_extent(axis_of(C, "C", 0), axis_of(indices_A, "indices_A", 0));
    v.same_extent(axis_of(C, "C", 0), axis_of(indices_B, "indices_B", 0));
    v.same_extent(axis_of(C, "C", 0), axis_of(indices_output, "indices_output", 0));
    if (v.host_indices()) {
        v.index_range(indices_A, "indices_A", A.shape[1]);
        v.index_range(indices_B, "indices_B", B.shape[1]);
        v.index_range(indices_output, "indices_output", output.shape[1]);
    }
}

template <typename T>
void sap_vjp(
    const Validator& v,
    Tensor<T, 2> grad_A,
    Tensor<T, 2> grad_B,
    Tensor<T, 2> grad_output,
    Tensor<T, 2> A,
    Tensor<T, 2> B,
    Tensor<T, 1> C,
    Tensor<int32_t, 1> indices_A,
    Tensor<int32_t, 1> indices_B,
    Tensor<int32_t, 1> indices_output
) {
    v.gradient_like(grad_A, "grad_A", A, "A");
    v.gradient_like(grad_B, "grad_B", B, "B");
    sap(v, grad_output, A, B, C, indices_A, indices_B, indices_output);
}

template <typename T>
void sap_vjp_vjp(
    const Validator& v,
    Tensor<T, 2> grad_grad_output,
    Tensor<T, 2> grad_A_2,
    Tensor<T, 2> grad_B_2,
    Tensor<T, 2> grad_grad_A,
    Tensor<T, 2> grad_grad_B,
    Tensor<T, 2> grad_output,
    Tensor<T, 2> A,
    Tensor<T, 2> B,
    Tensor<T, 1> C,
    Tensor<int32_t, 1> indices_A,
    Tensor<int32_t, 1> indices_B,
    Tensor<int32_t, 1> indices_output
) {
    v.gradient_like(grad_grad_output, "grad_grad_output", grad_output, "grad_output");
    v.gradient_like(grad_A_2, "grad_A_2", A, "A");
    v.gradient_like(grad_B_2, "grad_B_2", B, "B");
    v.gradient_like(grad_grad_A, "grad_grad_A", A, "A");
    v.gradient_like(grad_grad_B, "grad_grad_B", B, "B");
    sap(v, grad_output, A, B, C, indices_A, indices_B, indices_output);
}

// --------------------------------------------------------------- OPSA ----
template <typename T>
void opsa(
    const Validator& v, Tensor<T, 3> output, Tensor<T, 2> A, Tensor<T, 2> B, Tensor<int32_t, 1> indices_output
) {
    v.same_extent(axis_of(A, "A", 0), axis_of(B, "B", 0));
    v.same_extent(axis_of(A, "A", 1), axis_of(output, "output", 1));
    v.same_extent(axis_of(B, "B", 1), axis_of(output, "output", 2));
    v.same_extent(axis_of(A, "A", 0), axis_of(indices_output, "indices_output", 0));
    if (v.host_indices()) {
        v.index_range(indices_output, "indices_output", output.shape[0]);
    }
}

template <typename T>
void opsa_vjp(
    const Validator& v,
    Tensor<T, 2> grad_A,
    Tensor<T, 2> grad_B,
    Tensor<T, 3> grad_output,
    Tensor<T, 2> A,
    Tensor<T, 2> B,
    Tensor<int32_t, 1> indices_output
) {
    v.gradient_like(grad_A, "grad_A", A, "A");
    v.gradient_like(grad_B, "grad_B", B, "B");
    opsa(v, grad_output, A, B, indices_output);
}

template <typename T>
void opsa_vjp_vjp(
    const Validator& v,
    Tensor<T, 3> grad_grad_output,
    Tensor<T, 2> grad_A_2,
    Tensor<T, 2> grad_B_2,
    Tensor<T, 2> grad_grad_A,
    Tensor<T, 2> grad_grad_B,
    Tensor<T, 3> grad_output,
    Tensor<T, 2> A,
    Tensor<T, 2> B,
    Tensor<int32_t, 1> indices_output
) {
    v.gradient_like(grad_grad_output, "grad_grad_output", grad_output, "grad_output");
    v.gradient_like(grad_A_2, "grad_A_2", A, "A");
    v.gradient_like(grad_B_2, "grad_B_2", B, "B");
    v.gradient_like(grad_grad_A, "grad_grad_A", A, "A");
    v.gradient_like(grad_grad_B, "grad_grad_B", B, "B");
    opsa(v, grad_output, A, B, indices_output);
}

// -------------------------------------------------------------- OPSAW ----
template <typename T>
void opsaw(
    const Validator& v,
    Tensor<T, 3> output,
    Tensor<T, 2> A,
    Tensor<T, 2> B,
    Tensor<T, 2> W,
    Tensor<int32_t, 1> indices_W,
    Tensor<int32_t, 1> indices_output
) {
    v.same_extent(axis_of(A, "A", 0), axis_of(B, "B", 0));
    v.same_extent(axis_of(A, "A", 1), axis_of(output, "output", 1));
    v.same_extent(axis_of(B, "B", 1), axis_of(output, "output", 2));
    v.same_extent(axis_of(A, "A", 0), axis_of(indices_output, "indices_output", 0));
    v.same_extent(axis_of(A, "A", 0), axis_of(indices_W, "indices_W", 0));
    v.same_extent(axis_of(W, "W", 0), axis_of(output, "output", 0));
    v.same_extent(axis_of(B, "B", 1), axis_of(W, "W", 1));
    if (v.host_indices()) {
        v.index_range(indices_output, "indices_output", output.shape[0]);
        v.index_range(indices_W, "indices_W", output.shape[0]);
    }
}

template <typename T>
void opsaw_vjp(
    const Validator& v,
    Tensor<T, 2> grad_A,
    Tensor<T, 2> grad_B,
    Tensor<T, 2> grad_W,
    Tensor<T, 3> grad_output,
    Tensor<T, 2> A,
    Tensor<T, 2> B,
    Tensor<T, 2> W,
    Tensor<int32_t, 1> indices_W,
    Tensor<int32_t, 1> indices_output
) {
    v.gradient_like(grad_A, "grad_A", A, "A");
    v.gradient_like(grad_B, "grad_B", B, "B");
    v.gradient_like(grad_W, "grad_W", W, "W");
    opsaw(v, grad_output, A, B, W, indices_W, indices_output);
}

// -------------------------------------------------------------- SASAW ----
template <typename T>
void sasaw(
    const Validator& v,
    Tensor<T, 3> output,
    Tensor<T, 2> A,
    Tensor<T, 2> B,
    Tensor<T, 1> C,
    Tensor<T, 3> W,
    Tensor<int32_t, 1> indices_A,
    Tensor<int32_t, 1> indices_W_1,
    Tensor<int32_t, 1> indices_W_2,
    Tensor<int32_t, 1> indices_output_1,
    Tensor<int32_t, 1> indices_output_2
) {
    v.same_extent(axis_of(A, "A", 0), axis_of(B, "B", 0));
    v.same_extent(axis_of(W, "W", 0), axis_of(output, "output", 0));
    v.same_extent(axis_of(B, "B", 1), axis_of(W, "W", 2));
    v.same_extent(axis_of(C, "C", 0), axis_of(indices_A, "indices_A", 0));
    v.same_extent(axis_of(C, "C", 0), axis_of(indices_W_2, "indices_W_2", 0));
    v.same_extent(axis_of(C, "C", 0), axis_of(indices_output_2, "indices_output_2", 0));
    v.same_extent(axis_of(A, "A", 0), axis_of(indices_output_1, "indices_output_1", 0));
    v.same_extent(axis_of(A, "A", 0), axis_of(indices_W_1, "indices_W_1", 0));
    if (v.host_indices()) {
        v.index_range(indices_A, "indices_A", A.shape[1]);
        v.index_range(indices_W_1, "indices_W_1", output.shape[0]);
        v.index_range(indices_W_2, "indices_W_2", B.shape[1]);
        v.index_range(indices_output_1, "indices_output_1", output.shape[0]);
        v.index_range(indices_output_2, "indices_output_2", output.shape[1]);
    }
}

template <typename T>
void sasaw_vjp(
    const Validator& v,
    Tensor<T, 2> grad_A,
    Tensor<T, 2> grad_B,
    Tensor<T, 3> grad_W,
    Tensor<T, 3> grad_output,
    Tensor<T, 2> A,
    Tensor<T, 2> B,
    Tensor<T, 1> C,
    Tensor<T, 3> W,
    Tensor<int32_t, 1> indices_A,
    Tensor<int32_t, 1> indices_W_1,
    Tensor<int32_t, 1> indices_W_2,
    Tensor<int32_t, 1> indices_output_1,
    Tensor<int32_t, 1> indices_output_2
) {
    v.gradient_like(grad_A, "grad_A", A, "A");
    v.gradient_like(grad_B, "grad_B", B, "B");
    v.gradient_like(grad_W, "grad_W", W, "W");
    sasaw(
        v, grad_output, A, B, C, W, indices_A, indices_W_1, indices_W_2, indices_output_1, indices_output_2
    );
}

} // namespace mops::checks

#endif
