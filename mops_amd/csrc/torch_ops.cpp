// torch.ops.mops.* in C++: the five operations as PyTorch operators with
// autograd, for callers that cannot afford (or do not have) an interpreter
// around every call: eager-mode training loops, scripted modules loaded from
// C++.
//
// Operator names and schemas are those of the reference's TorchScript
// extension (mops-torch/src/register.cpp:5-38 of lab-cosmo/mops). What is
// behind them is this library only: every operator checks its tensors, makes
// them contiguous, points the library at PyTorch's current stream and calls
// the `mops::cuda::` templates of <mops.hpp>; ROCm tensors are the only ones
// accepted (host tensors: "device path only", as everywhere in this library).
//
// Autograd: one torch::autograd::Function per operation whose backward is the
// library's vjp, computing only the gradients that are asked for. For the
// three operations that have a second derivative (HPE, SAP, OPSA, as in the
// reference) the vjp is itself a Function whose backward is the library's
// vjp_vjp. There is no gradient with respect to C or to index tensors.
//
// mops_amd/torch.py loads this library when it has been built and registers
// the same operators from Python otherwise.
#include <array>
#include <stdexcept>
#include <string>
#include <vector>

#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/script.h>

#include "mops.hpp"
#include "mops/amd.h"

namespace {

using torch::autograd::AutogradContext;
using torch::autograd::Function;
using torch::autograd::variable_list;

// ------------------------------------------------------------ arguments --
void require_device(const at::Tensor& tensor, const char* name, const char* operation) {
    if (!tensor.is_cuda()) { // ROCm tensors carry the CUDA device type
        throw std::runtime_error(
            std::string("mops::") + operation + ": " + name +
            " must be on a ROCm device; this library implements the device path only"
        );
    }
}

at::Tensor values(const at::Tensor& tensor, const at::Tensor& like, const char* name, const char* operation) {
    require_device(tensor, name, operation);
    if (tensor.scalar_type() != at::kFloat && tensor.scalar_type() != at::kDouble) {
        throw std::runtime_error(std::string("mops::") + operation + ": " + name + " must be float32 or float64");
    }
    if (tensor.scalar_type() != like.scalar_type() || tensor.device() != like.device()) {
        throw std::runtime_error(
            std::string("mops::") + operation + ": " + name + " must have the dtype and the device of A"
        );
    }
    return tensor.contiguous();
}

at::Tensor indices(const at::Tensor& tensor, const at::Tensor& like, const char* name, const char* operation) {
    require_device(tensor, name, operation);
    if (tensor.device() != like.device()) {
        throw std::runtime_error(std::string("mops::") + operation + ": " + name + " must be on the device of A");
    }
    if (!at::isIntegralType(tensor.scalar_type(), /*includeBool=*/false)) {
        throw std::runtime_error(std::string("mops::") + operation + ": " + name + " must hold integers");
    }
    return tensor.to(at::kInt).contiguous();
}

template <typename T, size_t N> mops::Tensor<T, N> view(const at::Tensor& tensor, const char* name) {
    mops::Tensor<T, N> result{nullptr, {}};
    for (size_t d = 0; d < N; d++) {
        result.shape[d] = 0;
    }
    if (!tensor.defined()) {
        return result; // "not wanted" / "not given": a null view
    }
    if (static_cast<size_t>(tensor.dim()) != N) {
        throw std::runtime_error(
            std::string(name) + " must have " + std::to_string(N) + " dimensions, got " + std::to_string(tensor.dim())
        );
    }
    result.data = tensor.data_ptr<T>();
    for (size_t d = 0; d < N; d++) {
        result.shape[d] = static_cast<size_t>(tensor.size(static_cast<int64_t>(d)));
    }
    return result;
}

/// The library's launches go to PyTorch's current stream of the tensors' device, without blocking.
/// (In a ROCm build of PyTorch the HIP device type goes under the name of CUDA: these are the
/// guard and the stream of that build.)
struct OnTorchStream {
    c10::hip::HIPGuardMasqueradingAsCUDA guard;
    explicit OnTorchStream(const at::Tensor& tensor) : guard(tensor.device()) {
        mops_amd_set_stream(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream());
        mops_amd_set_synchronous(0);
    }
};

template <typename Body> void by_dtype(const at::Tensor& like, Body&& body) {
    if (like.scalar_type() == at::kFloat) {
        body(float{});
    } else {
        body(double{});
    }
}

at::Tensor nothing(const at::Tensor& like) { return at::empty({0}, like.options()); }
at::Tensor or_undefined(const at::Tensor& tensor, bool wanted) { return wanted ? tensor : at::Tensor(); }

// ------------------------------------------------------------------ HPE --
at::Tensor hpe_forward(const at::Tensor& A_, const at::Tensor& C_, const at::Tensor& P_) {
    const char* op = "homogeneous_polynomial_evaluation";
    const at::Tensor A = values(A_, A_, "A", op), C = values(C_, A_, "C", op), P = indices(P_, A_, "indices_A", op);
    OnTorchStream stream(A);
    at::Tensor output = at::empty({A.dim() == 2 ? A.size(0) : 0}, A.options());
    by_dtype(A, [&](auto zero) {
        using T = decltype(zero);
        mops::cuda::homogeneous_polynomial_evaluation<T>(
            view<T, 1>(output, "output"), view<T, 2>(A, "A"), view<T, 1>(C, "C"), view<int32_t, 2>(P, "indices_A")
        );
    });
    return output;
}

at::Tensor hpe_vjp(const at::Tensor& gO_, const at::Tensor& A_, const at::Tensor& C_, const at::Tensor& P_) {
    const char* op = "homogeneous_polynomial_evaluation_vjp";
    const at::Tensor A = values(A_, A_, "A", op), C = values(C_, A_, "C", op), P = indices(P_, A_, "indices_A", op);
    const at::Tensor gO = values(gO_, A_, "grad_output", op);
    OnTorchStream stream(A);
    at::Tensor grad_A = at::empty_like(A);
    by_dtype(A, [&](auto zero) {
        using T = decltype(zero);
        mops::cuda::homogeneous_polynomial_evaluation_vjp<T>(
            view<T, 2>(grad_A, "grad_A"), view<T, 1>(gO, "grad_output"), view<T, 2>(A, "A"), view<T, 1>(C, "C"),
            view<int32_t, 2>(P, "indices_A")
        );
    });
    return grad_A;
}

std::array<at::Tensor, 2> hpe_vjp_vjp(
    const at::Tensor& ggA_, const at::Tensor& gO_, const at::Tensor& A_, const at::Tensor& C_, const at::Tensor& P_,
    bool want_ggO, bool want_A2
) {
    const char* op = "homogeneous_polynomial_evaluation_vjp_vjp";
    const at::Tensor A = values(A_, A_, "A", op), C = values(C_, A_, "C", op), P = indices(P_, A_, "indices_A", op);
    const at::Tensor gO = values(gO_, A_, "grad_output", op);
    const at::Tensor ggA = ggA_.defined() ? values(ggA_, A_, "grad_grad_A", op) : at::Tensor();
    OnTorchStream stream(A);
    at::Tensor ggO = want_ggO ? at::empty_like(gO) : at::Tensor();
    at::Tensor A2 = want_A2 ? at::empty_like(A) : at::Tensor();
    by_dtype(A, [&](auto zero) {
        using T = decltype(zero);
        mops::cuda::homogeneous_polynomial_evaluation_vjp_vjp<T>(
            view<T, 1>(ggO, "grad_grad_output"), view<T, 2>(A2, "grad_A_2"), view<T, 2>(ggA, "grad_grad_A"),
            view<T, 1>(gO, "grad_output"), view<T, 2>(A, "A"), view<T, 1>(C, "C"), view<int32_t, 2>(P, "indices_A")
        );
    });
    return {ggO, A2};
}

struct HpeVjp : public Function<HpeVjp> {
    static at::Tensor forward(AutogradContext* ctx, at::Tensor gO, at::Tensor A, at::Tensor C, at::Tensor P) {
        ctx->save_for_backward({gO, A, C, P});
        return hpe_vjp(gO, A, C, P);
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        const auto saved = ctx->get_saved_variables();
        if (ctx->needs_input_grad(2)) {
            throw std::runtime_error("gradients with respect to C are not supported");
        }
        const bool want_ggO = ctx->needs_input_grad(0), want_A2 = ctx->needs_input_grad(1);
        const auto second = hpe_vjp_vjp(grads[0], saved[0], saved[1], saved[2], saved[3], want_ggO, want_A2);
        return {second[0], second[1], at::Tensor(), at::Tensor()};
    }
};

struct Hpe : public Function<Hpe> {
    static at::Tensor forward(AutogradContext* ctx, at::Tensor A, at::Tensor C, at::Tensor P) {
        ctx->save_for_backward({A, C, P});
        return hpe_forward(A, C, P);
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        const auto saved = ctx->get_saved_variables();
        if (ctx->needs_input_grad(1)) {
            throw std::runtime_error("gradients with respect to C are not supported");
        }
        at::Tensor grad_A;
        if (ctx->needs_input_grad(0)) {
            grad_A = HpeVjp::apply(grads[0], saved[0], saved[1], saved[2]);
        }
        return {grad_A, at::Tensor(), at::Tensor()};
    }
};

// ------------------------------------------------------------ OPSA, SAP --
// Both have two differentiable inputs (A, B) and a second derivative; they differ in
// their other arguments, which `Extra` carries: OPSA {indices_output}, SAP {C, indices_A,
// indices_B, indices_output}.
struct Opsa {
    static constexpr const char* name = "outer_product_scatter_add";
    static constexpr size_t n_extra = 1;
    static std::vector<at::Tensor> prepare(const std::vector<at::Tensor>& extra, const at::Tensor& A, const char* op) {
        return {indices(extra[0], A, "indices_output", op)};
    }
    static at::Tensor output_like(const at::Tensor& A, const at::Tensor& B, int64_t output_size) {
        return at::empty({output_size, A.dim() == 2 ? A.size(1) : 0, B.dim() == 2 ? B.size(1) : 0}, A.options());
    }
    template <typename T>
    static void forward(at::Tensor& O, const at::Tensor& A, const at::Tensor& B, const std::vector<at::Tensor>& e) {
        mops::cuda::outer_product_scatter_add<T>(
            view<T, 3>(O, "output"), view<T, 2>(A, "A"), view<T, 2>(B, "B"), view<int32_t, 1>(e[0], "indices_output")
        );
    }
    template <typename T>
    static void vjp(
        at::Tensor& gA, at::Tensor& gB, const at::Tensor& gO, const at::Tensor& A, const at::Tensor& B,
        const std::vector<at::Tensor>& e
    ) {
        mops::cuda::outer_product_scatter_add_vjp<T>(
            view<T, 2>(gA, "grad_A"), view<T, 2>(gB, "grad_B"), view<T, 3>(gO, "grad_output"), view<T, 2>(A, "A"),
            view<T, 2>(B, "B"), view<int32_t, 1>(e[0], "indices_output")
        );
    }
    template <typename T>
    static void vjp_vjp(
        at::Tensor& ggO, at::Tensor& A2, at::Tensor& B2, const at::Tensor& ggA, const at::Tensor& ggB,
        const at::Tensor& gO, const at::Tensor& A, const at::Tensor& B, const std::vector<at::Tensor>& e
    ) {
        mops::cuda::outer_product_scatter_add_vjp_vjp<T>(
            view<T, 3>(ggO, "grad_grad_output"), view<T, 2>(A2, "grad_A_2"), view<T, 2>(B2, "grad_B_2"),
            view<T, 2>(ggA, "grad_grad_A"), view<T, 2>(ggB, "grad_grad_B"), view<T, 3>(gO, "grad_output"),
            view<T, 2>(A, "A"), view<T, 2>(B, "B"), view<int32_t, 1>(e[0], "indices_output")
        );
    }
    template <typename T> static mops::Tensor<T, 3> grad_output_view(const at::Tensor& gO) {
        return view<T, 3>(gO, "grad_output");
    }
};

struct Sap {
    static constexpr const char* name = "sparse_accumulation_of_products";
    static constexpr size_t n_extra = 4;
    static std::vector<at::Tensor> prepare(const std::vector<at::Tensor>& extra, const at::Tensor& A, const char* op) {
        return {
            values(extra[0], A, "C", op), indices(extra[1], A, "indices_A", op), indices(extra[2], A, "indices_B", op),
            indices(extra[3], A, "indices_output", op)};
    }
    static at::Tensor output_like(const at::Tensor& A, const at::Tensor&, int64_t output_size) {
        return at::empty({A.dim() == 2 ? A.size(0) : 0, output_size}, A.options());
    }
    template <typename T>
    static void forward(at::Tensor& O, const at::Tensor& A, const at::Tensor& B, const std::vector<at::Tensor>& e) {
        mops::cuda::sparse_accumulation_of_products<T>(
            view<T, 2>(O, "output"), view<T, 2>(A, "A"), view<T, 2>(B, "B"), view<T, 1>(e[0], "C"),
            view<int32_t, 1>(e[1], "indices_A"), view<int32_t, 1>(e[2], "indices_B"),
            view<int32_t, 1>(e[3], "indices_output")
        );
    }
    template <typename T>
    static void vjp(
        at::Tensor& gA, at::Tensor& gB, const at::Tensor& gO, const at::Tensor& A, const at::Tensor& B,
        const std::vector<at::Tensor>& e
    ) {
        mops::cuda::sparse_accumulation_of_products_vjp<T>(
            view<T, 2>(gA, "grad_A"), view<T, 2>(gB, "grad_B"), view<T, 2>(gO, "grad_output"), view<T, 2>(A, "A"),
            view<T, 2>(B, "B"), view<T, 1>(e[0], "C"), view<int32_t, 1>(e[1], "indices_A"),
            view<int32_t, 1>(e[2], "indices_B"), view<int32_t, 1>(e[3], "indices_output")
        );
    }
    template <typename T>
    static void vjp_vjp(
        at::Tensor& ggO, at::Tensor& A2, at::Tensor& B2, const at::Tensor& ggA, const at::Tensor& ggB,
        const at::Tensor& gO, const at::Tensor& A, const at::Tensor& B, const std::vector<at::Tensor>& e
    ) {
        mops::cuda::sparse_accumulation_of_products_vjp_vjp<T>(
            view<T, 2>(ggO, "grad_grad_output"), view<T, 2>(A2, "grad_A_2"), view<T, 2>(B2, "grad_B_2"),
            view<T, 2>(ggA, "grad_grad_A"), view<T, 2>(ggB, "grad_grad_B"), view<T, 2>(gO, "grad_output"),
            view<T, 2>(A, "A"), view<T, 2>(B, "B"), view<T, 1>(e[0], "C"), view<int32_t, 1>(e[1], "indices_A"),
            view<int32_t, 1>(e[2], "indices_B"), view<int32_t, 1>(e[3], "indices_output")
        );
    }
};

/// grad_A, grad_B of a bilinear operation; a gradient that is not wanted comes back undefined.
template <typename Op>
std::array<at::Tensor, 2> bilinear_vjp(
    const at::Tensor& gO_, const at::Tensor& A_, const at::Tensor& B_, const std::vector<at::Tensor>& extra_,
    bool want_A, bool want_B
) {
    const std::string op = std::string(Op::name) + "_vjp";
    const at::Tensor A = values(A_, A_, "A", op.c_str()), B = values(B_, A_, "B", op.c_str());
    const at::Tensor gO = values(gO_, A_, "grad_output", op.c_str());
    const std::vector<at::Tensor> extra = Op::prepare(extra_, A, op.c_str());
    OnTorchStream stream(A);
    at::Tensor gA = want_A ? at::empty_like(A) : at::Tensor();
    at::Tensor gB = want_B ? at::empty_like(B) : at::Tensor();
    by_dtype(A, [&](auto zero) { Op::template vjp<decltype(zero)>(gA, gB, gO, A, B, extra); });
    return {gA, gB};
}

template <typename Op> struct BilinearVjp : public Function<BilinearVjp<Op>> {
    // inputs: grad_output, A, B, extra tensors..., then which gradients are wanted
    static variable_list forward(
        AutogradContext* ctx, at::Tensor gO, at::Tensor A, at::Tensor B, at::TensorList extra_list, bool want_A,
        bool want_B
    ) {
        // (a TensorList, not a vector: only that makes the tensors in it inputs of the Function)
        const variable_list extra = extra_list.vec();
        variable_list saved = {gO, A, B};
        saved.insert(saved.end(), extra.begin(), extra.end());
        ctx->save_for_backward(saved);
        ctx->saved_data["want_A"] = want_A;
        ctx->saved_data["want_B"] = want_B;
        const auto gradients = bilinear_vjp<Op>(gO, A, B, extra, want_A, want_B);
        // a Function's outputs must be defined: an empty tensor stands for "not computed"
        return {want_A ? gradients[0] : nothing(A), want_B ? gradients[1] : nothing(B)};
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        const auto saved = ctx->get_saved_variables();
        const at::Tensor &gO_ = saved[0], &A_ = saved[1], &B_ = saved[2];
        const std::vector<at::Tensor> extra_(saved.begin() + 3, saved.end());
        const std::string op = std::string(Op::name) + "_vjp_vjp";
        // the inputs of forward(): grad_output 0, A 1, B 2, the list of extra tensors from 3 on
        for (size_t at = 0; at < Op::n_extra; at++) {
            if (at::isFloatingType(extra_[at].scalar_type()) && ctx->needs_input_grad(3 + at)) {
                throw std::runtime_error("gradients with respect to C are not supported");
            }
        }
        const bool have_A = ctx->saved_data["want_A"].toBool() && grads[0].defined();
        const bool have_B = ctx->saved_data["want_B"].toBool() && grads[1].defined();
        const bool want_ggO = ctx->needs_input_grad(0), want_A2 = ctx->needs_input_grad(1),
                   want_B2 = ctx->needs_input_grad(2);
        const at::Tensor A = values(A_, A_, "A", op.c_str()), B = values(B_, A_, "B", op.c_str());
        const at::Tensor gO = values(gO_, A_, "grad_output", op.c_str());
        const at::Tensor ggA = have_A ? values(grads[0], A_, "grad_grad_A", op.c_str()) : at::Tensor();
        const at::Tensor ggB = have_B ? values(grads[1], A_, "grad_grad_B", op.c_str()) : at::Tensor();
        const std::vector<at::Tensor> extra = Op::prepare(extra_, A, op.c_str());
        OnTorchStream stream(A);
        at::Tensor ggO = want_ggO ? at::empty_like(gO) : at::Tensor();
        at::Tensor A2 = want_A2 ? at::empty_like(A) : at::Tensor();
        at::Tensor B2 = want_B2 ? at::empty_like(B) : at::Tensor();
        by_dtype(A, [&](auto zero) {
            Op::template vjp_vjp<decltype(zero)>(ggO, A2, B2, ggA, ggB, gO, A, B, extra);
        });
        variable_list result = {ggO, A2, B2};
        result.resize(3 + Op::n_extra + 2); // nothing for the extra tensors and the two flags
        return result;
    }
};

template <typename Op> struct Bilinear : public Function<Bilinear<Op>> {
    static at::Tensor forward(
        AutogradContext* ctx, at::Tensor A_, at::Tensor B_, at::TensorList extra_list, int64_t output_size
    ) {
        const variable_list extra_ = extra_list.vec();
        variable_list saved = {A_, B_};
        saved.insert(saved.end(), extra_.begin(), extra_.end());
        ctx->save_for_backward(saved);
        const at::Tensor A = values(A_, A_, "A", Op::name), B = values(B_, A_, "B", Op::name);
        const std::vector<at::Tensor> extra = Op::prepare(extra_, A, Op::name);
        OnTorchStream stream(A);
        at::Tensor output = Op::output_like(A, B, output_size);
        by_dtype(A, [&](auto zero) { Op::template forward<decltype(zero)>(output, A, B, extra); });
        return output;
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        const auto saved = ctx->get_saved_variables();
        const std::vector<at::Tensor> extra(saved.begin() + 2, saved.end());
        for (size_t at = 0; at < Op::n_extra; at++) {
            if (at::isFloatingType(extra[at].scalar_type()) && ctx->needs_input_grad(2 + at)) {
                throw std::runtime_error("gradients with respect to C are not supported");
            }
        }
        const bool want_A = ctx->needs_input_grad(0), want_B = ctx->needs_input_grad(1);
        variable_list result(2 + Op::n_extra + 1);
        if (want_A || want_B) {
            const auto gradients =
                BilinearVjp<Op>::apply(grads[0], saved[0], saved[1], at::TensorList(extra), want_A, want_B);
            result[0] = or_undefined(gradients[0], want_A);
            result[1] = or_undefined(gradients[1], want_B);
        }
        return result;
    }
};

// ------------------------------------------------------- OPSAW, SASAW --
// Three differentiable inputs (A, B, W), no second derivative (the reference has none:
// mops/src/opsaw/cpu.tpp:133-150, mops/src/sasaw/cpu.tpp:173-194).
struct OpsawFunction : public Function<OpsawFunction> {
    static at::Tensor forward(
        AutogradContext* ctx, at::Tensor A_, at::Tensor B_, at::Tensor W_, at::Tensor PW_, at::Tensor PO_
    ) {
        const char* op = "outer_product_scatter_add_with_weights";
        ctx->save_for_backward({A_, B_, W_, PW_, PO_});
        const at::Tensor A = values(A_, A_, "A", op), B = values(B_, A_, "B", op), W = values(W_, A_, "W", op);
        const at::Tensor PW = indices(PW_, A_, "indices_W", op), PO = indices(PO_, A_, "indices_output", op);
        OnTorchStream stream(A);
        at::Tensor output = at::empty(
            {W.dim() == 2 ? W.size(0) : 0, A.dim() == 2 ? A.size(1) : 0, B.dim() == 2 ? B.size(1) : 0}, A.options()
        );
        by_dtype(A, [&](auto zero) {
            using T = decltype(zero);
            mops::cuda::outer_product_scatter_add_with_weights<T>(
                view<T, 3>(output, "output"), view<T, 2>(A, "A"), view<T, 2>(B, "B"), view<T, 2>(W, "W"),
                view<int32_t, 1>(PW, "indices_W"), view<int32_t, 1>(PO, "indices_output")
            );
        });
        return output;
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        const char* op = "outer_product_scatter_add_with_weights_vjp";
        const auto saved = ctx->get_saved_variables();
        const bool want_A = ctx->needs_input_grad(0), want_B = ctx->needs_input_grad(1),
                   want_W = ctx->needs_input_grad(2);
        const at::Tensor A = values(saved[0], saved[0], "A", op), B = values(saved[1], saved[0], "B", op),
                         W = values(saved[2], saved[0], "W", op);
        const at::Tensor PW = indices(saved[3], saved[0], "indices_W", op),
                         PO = indices(saved[4], saved[0], "indices_output", op);
        const at::Tensor gO = values(grads[0], saved[0], "grad_output", op);
        OnTorchStream stream(A);
        at::Tensor gA = want_A ? at::empty_like(A) : at::Tensor();
        at::Tensor gB = want_B ? at::empty_like(B) : at::Tensor();
        at::Tensor gW = want_W ? at::empty_like(W) : at::Tensor();
        by_dtype(A, [&](auto zero) {
            using T = decltype(zero);
            mops::cuda::outer_product_scatter_add_with_weights_vjp<T>(
                view<T, 2>(gA, "grad_A"), view<T, 2>(gB, "grad_B"), view<T, 2>(gW, "grad_W"),
                view<T, 3>(gO, "grad_output"), view<T, 2>(A, "A"), view<T, 2>(B, "B"), view<T, 2>(W, "W"),
                view<int32_t, 1>(PW, "indices_W"), view<int32_t, 1>(PO, "indices_output")
            );
        });
        return {gA, gB, gW, at::Tensor(), at::Tensor()};
    }
};

struct SasawFunction : public Function<SasawFunction> {
    static at::Tensor forward(
        AutogradContext* ctx, at::Tensor A_, at::Tensor B_, at::Tensor C_, at::Tensor W_, at::Tensor PA_,
        at::Tensor PW1_, at::Tensor PW2_, at::Tensor PO1_, at::Tensor PO2_, int64_t output_size
    ) {
        const char* op = "sparse_accumulation_scatter_add_with_weights";
        ctx->save_for_backward({A_, B_, C_, W_, PA_, PW1_, PW2_, PO1_, PO2_});
        const at::Tensor A = values(A_, A_, "A", op), B = values(B_, A_, "B", op), C = values(C_, A_, "C", op),
                         W = values(W_, A_, "W", op);
        const at::Tensor PA = indices(PA_, A_, "indices_A", op), PW1 = indices(PW1_, A_, "indices_W_1", op),
                         PW2 = indices(PW2_, A_, "indices_W_2", op), PO1 = indices(PO1_, A_, "indices_output_1", op),
                         PO2 = indices(PO2_, A_, "indices_output_2", op);
        OnTorchStream stream(A);
        at::Tensor output =
            at::empty({W.dim() == 3 ? W.size(0) : 0, output_size, B.dim() == 2 ? B.size(1) : 0}, A.options());
        by_dtype(A, [&](auto zero) {
            using T = decltype(zero);
            mops::cuda::sparse_accumulation_scatter_add_with_weights<T>(
                view<T, 3>(output, "output"), view<T, 2>(A, "A"), view<T, 2>(B, "B"), view<T, 1>(C, "C"),
                view<T, 3>(W, "W"), view<int32_t, 1>(PA, "indices_A"), view<int32_t, 1>(PW1, "indices_W_1"),
                view<int32_t, 1>(PW2, "indices_W_2"), view<int32_t, 1>(PO1, "indices_output_1"),
                view<int32_t, 1>(PO2, "indices_output_2")
            );
        });
        return output;
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        const char* op = "sparse_accumulation_scatter_add_with_weights_vjp";
        const auto saved = ctx->get_saved_variables();
        if (ctx->needs_input_grad(2)) {
            throw std::runtime_error("gradients with respect to C are not supported");
        }
        const bool want_A = ctx->needs_input_grad(0), want_B = ctx->needs_input_grad(1),
                   want_W = ctx->needs_input_grad(3);
        const at::Tensor& like = saved[0];
        const at::Tensor A = values(saved[0], like, "A", op), B = values(saved[1], like, "B", op),
                         C = values(saved[2], like, "C", op), W = values(saved[3], like, "W", op);
        const at::Tensor PA = indices(saved[4], like, "indices_A", op), PW1 = indices(saved[5], like, "indices_W_1", op),
                         PW2 = indices(saved[6], like, "indices_W_2", op),
                         PO1 = indices(saved[7], like, "indices_output_1", op),
                         PO2 = indices(saved[8], like, "indices_output_2", op);
        const at::Tensor gO = values(grads[0], like, "grad_output", op);
        OnTorchStream stream(A);
        at::Tensor gA = want_A ? at::empty_like(A) : at::Tensor();
        at::Tensor gB = want_B ? at::empty_like(B) : at::Tensor();
        at::Tensor gW = want_W ? at::empty_like(W) : at::Tensor();
        by_dtype(A, [&](auto zero) {
            using T = decltype(zero);
            mops::cuda::sparse_accumulation_scatter_add_with_weights_vjp<T>(
                view<T, 2>(gA, "grad_A"), view<T, 2>(gB, "grad_B"), view<T, 3>(gW, "grad_W"),
                view<T, 3>(gO, "grad_output"), view<T, 2>(A, "A"), view<T, 2>(B, "B"), view<T, 1>(C, "C"),
                view<T, 3>(W, "W"), view<int32_t, 1>(PA, "indices_A"), view<int32_t, 1>(PW1, "indices_W_1"),
                view<int32_t, 1>(PW2, "indices_W_2"), view<int32_t, 1>(PO1, "indices_output_1"),
                view<int32_t, 1>(PO2, "indices_output_2")
            );
        });
        variable_list result(10);
        result[0] = gA;
        result[1] = gB;
        result[3] = gW;
        return result;
    }
};

// ------------------------------------------------------------ operators --
at::Tensor homogeneous_polynomial_evaluation(at::Tensor A, at::Tensor C, at::Tensor indices_A) {
    return Hpe::apply(A, C, indices_A);
}

at::Tensor outer_product_scatter_add(at::Tensor A, at::Tensor B, at::Tensor indices_output, int64_t output_size) {
    const variable_list extra = {indices_output};
    return Bilinear<Opsa>::apply(A, B, at::TensorList(extra), output_size);
}

at::Tensor sparse_accumulation_of_products(
    at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor indices_A, at::Tensor indices_B, at::Tensor indices_output,
    int64_t output_size
) {
    const variable_list extra = {C, indices_A, indices_B, indices_output};
    return Bilinear<Sap>::apply(A, B, at::TensorList(extra), output_size);
}

at::Tensor outer_product_scatter_add_with_weights(
    at::Tensor A, at::Tensor B, at::Tensor W, at::Tensor indices_W, at::Tensor indices_output
) {
    return OpsawFunction::apply(A, B, W, indices_W, indices_output);
}

at::Tensor sparse_accumulation_scatter_add_with_weights(
    at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor W, at::Tensor indices_A, at::Tensor indices_W_1,
    at::Tensor indices_W_2, at::Tensor indices_output_1, at::Tensor indices_output_2, int64_t output_size
) {
    return SasawFunction::apply(
        A, B, C, W, indices_A, indices_W_1, indices_W_2, indices_output_1, indices_output_2, output_size
    );
}

} // namespace

TORCH_LIBRARY(mops, m) {
    m.def(
        "homogeneous_polynomial_evaluation(Tensor A, Tensor C, Tensor indices_A) -> Tensor",
        homogeneous_polynomial_evaluation
    );
    m.def(
        "outer_product_scatter_add(Tensor A, Tensor B, Tensor indices_output, int output_size) -> Tensor",
        outer_product_scatter_add
    );
    m.def(
        "sparse_accumulation_of_products(Tensor A, Tensor B, Tensor C, Tensor indices_A, Tensor indices_B, "
        "Tensor indices_output, int output_size) -> Tensor",
        sparse_accumulation_of_products
    );
    m.def(
        "outer_product_scatter_add_with_weights(Tensor A, Tensor B, Tensor W, Tensor indices_W, "
        "Tensor indices_output) -> Tensor",
        outer_product_scatter_add_with_weights
    );
    m.def(
        "sparse_accumulation_scatter_add_with_weights(Tensor A, Tensor B, Tensor C, Tensor W, Tensor indices_A, "
        "Tensor indices_W_1, Tensor indices_W_2, Tensor indices_output_1, Tensor indices_output_2, "
        "int output_size) -> Tensor",
        sparse_accumulation_scatter_add_with_weights
    );
}
