// The torch extension over the C ABI of libmegagemm_hip.so: host-only C++ (no device code
// here), taking the place of the reference's pytorch_binding/binding.cpp.
//
//   rmsnorm_forward / rmsnorm_backward   the reference's two module functions
//       (binding.cpp:136-139), same checks and messages (binding.cpp:9-11,17-24,62-65),
//       outputs allocated here (binding.cpp:29-30,89-90); the dtype ladders collapse into one
//       C call each.
//   rmsnorm_backward_f32                 the same backward with dW also kept in fp32
//   swiglu_forward / swiglu_backward     tensor-level form of the two Triton launches
//       (megagemm/swiglu.py:89-131)
//   rmsnorm / swiglu                     the two operators as autograd nodes written in C++,
//       doing what RMSNormFunction (megagemm/rmsnorm.py:18-48) and MegaGemmFunction
//       (megagemm/swiglu.py:86-131) do, without a round trip through Python in backward
//
// Everything runs on torch's current stream of the tensors' device and never synchronises.
#include <torch/extension.h>
// torch on ROCm presents its devices as "cuda": the guard and stream types that go with that
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <tuple>
#include <vector>

#include "megagemm_hip.h"

namespace {

using torch::Tensor;

void check_input(const Tensor& t, const char* name) {
    TORCH_CHECK(t.is_cuda(), name, " must be a CUDA tensor");
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}

int dtype_code(at::ScalarType t) {
    switch (t) {
        case at::kFloat: return MG_F32;
        case at::kHalf: return MG_F16;
        case at::kBFloat16: return MG_BF16;
        default: TORCH_CHECK(false, "Unsupported dtype ", t, ". Use float32, float16, or bfloat16."); return -1;
    }
}

void check_pair(const Tensor& input, const Tensor& weight) {
    TORCH_CHECK(input.dim() == 2, "Input must be 2D");
    TORCH_CHECK(weight.dim() == 1 && weight.size(0) == input.size(1), "Weight size must match hidden size");
    TORCH_CHECK(weight.scalar_type() == input.scalar_type(), "weight dtype (", weight.scalar_type(),
                ") must equal input dtype (", input.scalar_type(),
                "); cast the module, e.g. model.half() or model.to(torch.bfloat16)");
    TORCH_CHECK(weight.device() == input.device(), "input and weight must be on the same device");
}

void* current_stream() { return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }

std::vector<Tensor> rmsnorm_forward(const Tensor& input, const Tensor& weight, double epsilon) {
    check_input(input, "input");
    check_input(weight, "weight");
    check_pair(input, weight);
    const int64_t rows = input.size(0), cols = input.size(1);
    TORCH_CHECK(cols >= 1, "hidden size must be >= 1");
    const int code = dtype_code(input.scalar_type());
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
    auto output = torch::empty_like(input);
    auto inv_rms = torch::empty({rows}, input.options().dtype(torch::kFloat32));
    const int rc = mg_rmsnorm_fwd(output.data_ptr(), inv_rms.data_ptr<float>(), input.data_ptr(), weight.data_ptr(),
                                  rows, cols, (float)epsilon, code, current_stream());
    TORCH_CHECK(rc == MG_OK, "RMSNorm forward failed (code ", rc, "): ", mg_last_error());
    return {output, inv_rms};
}

// (grad_input, grad_weight in fp32, grad_weight in the weight's dtype); the last two are
// undefined tensors when need_weight_grad is false, and the same tensor for fp32 weights.
std::tuple<Tensor, Tensor, Tensor> backward_impl(const Tensor& grad_output, const Tensor& input, const Tensor& weight,
                                                 const Tensor& inv_rms, bool need_weight_grad, bool want_f32) {
    check_input(grad_output, "grad_output");
    check_input(input, "input");
    check_input(weight, "weight");
    check_input(inv_rms, "inv_rms");
    check_pair(input, weight);
    const int64_t rows = input.size(0), cols = input.size(1);
    TORCH_CHECK(grad_output.sizes() == input.sizes() && grad_output.scalar_type() == input.scalar_type(),
                "grad_output must have the shape and dtype of input");
    TORCH_CHECK(inv_rms.scalar_type() == at::kFloat && inv_rms.dim() == 1 && inv_rms.size(0) == rows,
                "inv_rms must be a float32 vector with one entry per row");
    const int code = dtype_code(input.scalar_type());
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
    int64_t num_partials = 0, ld = 0;
    TORCH_CHECK(mg_rmsnorm_bwd_workspace(rows, cols, code, &num_partials, &ld) == MG_OK,
                "RMSNorm backward (workspace query) failed: ", mg_last_error());
    const auto f32 = input.options().dtype(torch::kFloat32);
    auto grad_input = torch::empty_like(input);
    auto partial = torch::empty({num_partials, ld}, f32);
    void* stream = current_stream();
    int rc = mg_rmsnorm_bwd(grad_input.data_ptr(), partial.data_ptr<float>(), grad_output.data_ptr(),
                            input.data_ptr(), weight.data_ptr(), inv_rms.data_ptr<float>(), rows, cols, code,
                            num_partials, ld, stream);
    TORCH_CHECK(rc == MG_OK, "RMSNorm backward failed (code ", rc, "): ", mg_last_error());
    Tensor dw_f32, dw_cast;
    if (need_weight_grad) {
        if (want_f32 || code == MG_F32) dw_f32 = torch::empty({cols}, f32);
        dw_cast = code == MG_F32 ? dw_f32 : torch::empty_like(weight);   // weight dtype, as binding.cpp:90
        rc = mg_rmsnorm_dw_reduce(dw_f32.defined() ? dw_f32.data_ptr<float>() : nullptr,
                                  code == MG_F32 ? nullptr : dw_cast.data_ptr(), code, partial.data_ptr<float>(),
                                  num_partials, ld, cols, stream);
        TORCH_CHECK(rc == MG_OK, "RMSNorm backward (dW reduction) failed (code ", rc, "): ", mg_last_error());
    }
    return {grad_input, dw_f32, dw_cast};
}

std::tuple<Tensor, Tensor, Tensor> rmsnorm_backward_f32(const Tensor& grad_output, const Tensor& input,
                                                        const Tensor& weight, const Tensor& inv_rms,
                                                        bool need_weight_grad) {
    return backward_impl(grad_output, input, weight, inv_rms, need_weight_grad, true);
}

std::vector<Tensor> rmsnorm_backward(const Tensor& grad_output, const Tensor& input, const Tensor& weight,
                                     const Tensor& inv_rms) {
    auto r = backward_impl(grad_output, input, weight, inv_rms, true, false);
    return {std::get<0>(r), std::get<2>(r)};
}

Tensor swiglu_forward(const Tensor& gate_up, int64_t hidden_dim) {
    check_input(gate_up, "w12_out");
    TORCH_CHECK(gate_up.dim() == 2 && gate_up.size(1) == 2 * hidden_dim, "expected a [M, ", 2 * hidden_dim,
                "] matrix, got ", gate_up.sizes());
    const int code = dtype_code(gate_up.scalar_type());
    const int64_t M = gate_up.size(0);
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(gate_up.device());
    auto out = torch::empty({M, hidden_dim}, gate_up.options());
    const int rc = mg_swiglu_fwd(out.data_ptr(), gate_up.data_ptr(), M, hidden_dim, code, current_stream());
    TORCH_CHECK(rc == MG_OK, "SwiGLU forward failed (code ", rc, "): ", mg_last_error());
    return out;
}

Tensor swiglu_backward(const Tensor& grad_out, const Tensor& gate_up, int64_t hidden_dim) {
    check_input(grad_out, "grad_output");
    check_input(gate_up, "w12_out");
    TORCH_CHECK(gate_up.dim() == 2 && gate_up.size(1) == 2 * hidden_dim, "expected a [M, ", 2 * hidden_dim,
                "] matrix, got ", gate_up.sizes());
    const int64_t M = gate_up.size(0);
    TORCH_CHECK(grad_out.dim() == 2 && grad_out.size(0) == M && grad_out.size(1) == hidden_dim &&
                    grad_out.scalar_type() == gate_up.scalar_type(),
                "grad_output must be [M, hidden_dim] with the dtype of the forward input");
    const int code = dtype_code(gate_up.scalar_type());
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(gate_up.device());
    auto grad_in = torch::empty_like(gate_up);
    const int rc = mg_swiglu_bwd(grad_in.data_ptr(), grad_out.data_ptr(), gate_up.data_ptr(), M, hidden_dim, code,
                                 current_stream());
    TORCH_CHECK(rc == MG_OK, "SwiGLU backward failed (code ", rc, "): ", mg_last_error());
    return grad_in;
}

// ---- autograd nodes ----
// Neither backward can be differentiated again (the kernels record no graph); asking for a
// second derivative raises, like torch's once_differentiable.
void refuse_double_backward(const Tensor& grad, const char* what) {
    TORCH_CHECK(!(torch::GradMode::is_enabled() && grad.requires_grad()), what,
                ": trying to differentiate twice a function whose backward is not differentiable");
}

struct RMSNormNode : public torch::autograd::Function<RMSNormNode> {
    static Tensor forward(torch::autograd::AutogradContext* ctx, const Tensor& input, const Tensor& weight,
                          double epsilon) {
        TORCH_CHECK(input.dim() >= 1, "RMSNorm needs at least one dimension");
        const auto shape = input.sizes().vec();
        auto x2d = input.contiguous().view({-1, shape.back()});
        auto w = weight.contiguous();
        auto out = rmsnorm_forward(x2d, w, epsilon);
        ctx->save_for_backward({x2d, w, out[1]});
        ctx->saved_data["shape"] = shape;
        return out[0].view(shape);
    }

    static torch::autograd::tensor_list backward(torch::autograd::AutogradContext* ctx,
                                                 torch::autograd::tensor_list grads) {
        refuse_double_backward(grads[0], "RMSNorm");
        torch::NoGradGuard no_grad;
        const auto saved = ctx->get_saved_variables();
        const Tensor &x2d = saved[0], &w = saved[1], &inv_rms = saved[2];
        auto dy = grads[0].contiguous().view(x2d.sizes());
        if (dy.scalar_type() != x2d.scalar_type()) dy = dy.to(x2d.scalar_type());
        auto r = backward_impl(dy, x2d, w, inv_rms, ctx->needs_input_grad(1), false);
        return {std::get<0>(r).view(ctx->saved_data["shape"].toIntVector()), std::get<2>(r), Tensor()};
    }
};

struct SwigluNode : public torch::autograd::Function<SwigluNode> {
    static Tensor forward(torch::autograd::AutogradContext* ctx, const Tensor& w12_out, int64_t hidden_dim) {
        TORCH_CHECK(w12_out.dim() >= 1 && w12_out.size(-1) == 2 * hidden_dim, "last dimension must be 2*hidden_dim = ",
                    2 * hidden_dim, ", got ", w12_out.dim() >= 1 ? w12_out.size(-1) : 0);
        auto fused = w12_out.contiguous();
        ctx->save_for_backward({fused});
        ctx->saved_data["hidden_dim"] = hidden_dim;
        auto shape = fused.sizes().vec();
        shape.back() = hidden_dim;
        return swiglu_forward(fused.view({-1, 2 * hidden_dim}), hidden_dim).view(shape);
    }

    static torch::autograd::tensor_list backward(torch::autograd::AutogradContext* ctx,
                                                 torch::autograd::tensor_list grads) {
        refuse_double_backward(grads[0], "SwiGLU");
        torch::NoGradGuard no_grad;
        const auto saved = ctx->get_saved_variables();
        const Tensor& fused = saved[0];
        const int64_t hidden_dim = ctx->saved_data["hidden_dim"].toInt();
        auto dh = grads[0].contiguous().view({-1, hidden_dim});
        if (dh.scalar_type() != fused.scalar_type()) dh = dh.to(fused.scalar_type());
        auto grad = swiglu_backward(dh, fused.view({-1, 2 * hidden_dim}), hidden_dim);
        return {grad.view(fused.sizes()), Tensor()};
    }
};

// y = x * rsqrt(mean(x^2, -1) + epsilon) * weight over the last dimension, differentiable.
Tensor rmsnorm(const Tensor& input, const Tensor& weight, double epsilon) {
    if (torch::GradMode::is_enabled() && (input.requires_grad() || weight.requires_grad()))
        return RMSNormNode::apply(input, weight, epsilon);
    // nothing to differentiate: same kernel, no node, no saved tensors and no per-row scale
    // (the C ABI takes a null inv_rms); the output keeps the input's shape, so no views either
    TORCH_CHECK(input.dim() >= 1, "RMSNorm needs at least one dimension");
    TORCH_CHECK(input.is_cuda(), "input must be a CUDA tensor");
    TORCH_CHECK(weight.is_cuda(), "weight must be a CUDA tensor");
    const Tensor x = input.contiguous(), w = weight.contiguous();   // themselves when they already are
    const int64_t cols = x.size(-1);
    TORCH_CHECK(cols >= 1, "hidden size must be >= 1");
    TORCH_CHECK(w.dim() == 1 && w.size(0) == cols, "Weight size must match hidden size");
    TORCH_CHECK(w.scalar_type() == x.scalar_type(), "weight dtype (", w.scalar_type(), ") must equal input dtype (",
                x.scalar_type(), "); cast the module, e.g. model.half() or model.to(torch.bfloat16)");
    TORCH_CHECK(w.device() == x.device(), "input and weight must be on the same device");
    const int code = dtype_code(x.scalar_type());
    const int64_t rows = x.numel() / cols;
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    auto output = torch::empty_like(x);
    const int rc = mg_rmsnorm_fwd(output.data_ptr(), nullptr, x.data_ptr(), w.data_ptr(), rows, cols, (float)epsilon,
                                  code, current_stream());
    TORCH_CHECK(rc == MG_OK, "RMSNorm forward failed (code ", rc, "): ", mg_last_error());
    return output;
}

// silu(gate) * up on a fused [..., 2*hidden_dim] tensor, differentiable.
Tensor swiglu(const Tensor& w12_out, int64_t hidden_dim) {
    if (torch::GradMode::is_enabled() && w12_out.requires_grad()) return SwigluNode::apply(w12_out, hidden_dim);
    TORCH_CHECK(w12_out.dim() >= 1 && w12_out.size(-1) == 2 * hidden_dim, "last dimension must be 2*hidden_dim = ",
                2 * hidden_dim, ", got ", w12_out.dim() >= 1 ? w12_out.size(-1) : 0);
    auto fused = w12_out.contiguous();
    auto shape = fused.sizes().vec();
    shape.back() = hidden_dim;
    return swiglu_forward(fused.view({-1, 2 * hidden_dim}), hidden_dim).view(shape);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "torch extension over libmegagemm_hip.so (C ABI version " + std::to_string(MG_ABI_VERSION) + ")";
    m.def("abi_version", [] { return mg_abi_version(); }, "ABI version of the loaded libmegagemm_hip.so");
    m.def("built_abi_version", [] { return MG_ABI_VERSION; },
          "MG_ABI_VERSION of the header this extension was compiled against");
    m.def("rmsnorm_forward", &rmsnorm_forward, "RMSNorm forward: [output, inv_rms]", py::arg("input"),
          py::arg("weight"), py::arg("epsilon"));
    m.def("rmsnorm_backward", &rmsnorm_backward, "RMSNorm backward: [grad_input, grad_weight]",
          py::arg("grad_output"), py::arg("input"), py::arg("weight"), py::arg("inv_rms"));
    m.def("rmsnorm_backward_f32", &rmsnorm_backward_f32,
          "RMSNorm backward: (grad_input, grad_weight fp32, grad_weight in the weight's dtype)", py::arg("grad_output"),
          py::arg("input"), py::arg("weight"), py::arg("inv_rms"), py::arg("need_weight_grad") = true);
    m.def("swiglu_forward", &swiglu_forward, "silu(gate) * up on [M, 2H] -> [M, H]", py::arg("gate_up"),
          py::arg("hidden_dim"));
    m.def("swiglu_backward", &swiglu_backward, "[d_gate | d_up] from grad_out [M, H] and gate_up [M, 2H]",
          py::arg("grad_out"), py::arg("gate_up"), py::arg("hidden_dim"));
    m.def("rmsnorm", &rmsnorm, "differentiable RMSNorm over the last dimension", py::arg("input"), py::arg("weight"),
          py::arg("epsilon") = 1e-5);
    m.def("swiglu", &swiglu, "differentiable silu(gate) * up over the last dimension", py::arg("w12_out"),
          py::arg("hidden_dim"));
}
