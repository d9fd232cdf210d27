// A compiled torch extension over the C ABI of libmegagemm_hip.so: what a maintainer of the
// reference would put in place of pytorch_binding/binding.cpp.  Same module functions
// (binding.cpp:136-139), same checks and messages (binding.cpp:9-11,17-24,62-65), outputs
// allocated by the binding (binding.cpp:29-30,89-90); the dtype ladders collapse into one
// call each.  Built and exercised by the test-suite as proof that the recipe in the
// integration notes compiles and runs; the package itself binds the library with ctypes.
#include <torch/extension.h>
// torch on ROCm presents its devices as "cuda": the guard and stream types that go with that
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <vector>

#include "megagemm_hip.h"

namespace {

void check_input(const torch::Tensor& t, const char* name) {
    TORCH_CHECK(t.is_cuda(), name, " must be a CUDA tensor");
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}

int dtype_code(at::ScalarType t) {
    switch (t) {
        case at::kFloat: return MG_F32;
        case at::kHalf: return MG_F16;
        case at::kBFloat16: return MG_BF16;
        default: TORCH_CHECK(false, "Unsupported dtype. Use float32, float16, or bfloat16."); return -1;
    }
}

std::vector<torch::Tensor> rmsnorm_forward(torch::Tensor input, torch::Tensor weight, double epsilon) {
    check_input(input, "input");
    check_input(weight, "weight");
    TORCH_CHECK(input.dim() == 2, "Input must be 2D");
    const int64_t rows = input.size(0), cols = input.size(1);
    TORCH_CHECK(weight.dim() == 1 && weight.size(0) == cols, "Weight size must match hidden size");
    TORCH_CHECK(weight.scalar_type() == input.scalar_type(), "weight dtype must equal input dtype");
    const int code = dtype_code(input.scalar_type());
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
    auto output = torch::empty_like(input);
    auto inv_rms = torch::empty({rows}, input.options().dtype(torch::kFloat32));
    void* stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    const int rc = mg_rmsnorm_fwd(output.data_ptr(), inv_rms.data_ptr<float>(), input.data_ptr(), weight.data_ptr(),
                                  rows, cols, (float)epsilon, code, stream);
    TORCH_CHECK(rc == MG_OK, "RMSNorm forward failed: ", mg_last_error());
    return {output, inv_rms};
}

std::vector<torch::Tensor> rmsnorm_backward(torch::Tensor grad_output, torch::Tensor input, torch::Tensor weight,
                                            torch::Tensor inv_rms) {
    check_input(grad_output, "grad_output");
    check_input(input, "input");
    check_input(weight, "weight");
    check_input(inv_rms, "inv_rms");
    TORCH_CHECK(input.dim() == 2, "Input must be 2D");
    const int64_t rows = input.size(0), cols = input.size(1);
    TORCH_CHECK(weight.dim() == 1 && weight.size(0) == cols, "Weight size must match hidden size");
    TORCH_CHECK(grad_output.sizes() == input.sizes() && grad_output.scalar_type() == input.scalar_type(),
                "grad_output must have the shape and dtype of input");
    TORCH_CHECK(inv_rms.scalar_type() == at::kFloat && inv_rms.numel() == rows,
                "inv_rms must be a float32 vector with one entry per row");
    const int code = dtype_code(input.scalar_type());
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
    int64_t num_partials = 0, ld = 0;
    TORCH_CHECK(mg_rmsnorm_bwd_workspace(rows, cols, code, &num_partials, &ld) == MG_OK, mg_last_error());
    auto grad_input = torch::empty_like(input);
    auto grad_weight = torch::empty_like(weight);   // weight dtype, as binding.cpp:90
    auto partial = torch::empty({num_partials, ld}, input.options().dtype(torch::kFloat32));
    void* stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    int rc = mg_rmsnorm_bwd(grad_input.data_ptr(), partial.data_ptr<float>(), grad_output.data_ptr(),
                            input.data_ptr(), weight.data_ptr(), inv_rms.data_ptr<float>(), rows, cols, code,
                            num_partials, ld, stream);
    TORCH_CHECK(rc == MG_OK, "RMSNorm backward failed: ", mg_last_error());
    rc = mg_rmsnorm_dw_reduce(nullptr, grad_weight.data_ptr(), code, partial.data_ptr<float>(), num_partials, ld,
                              cols, stream);
    TORCH_CHECK(rc == MG_OK, "RMSNorm backward (dW reduction) failed: ", mg_last_error());
    return {grad_input, grad_weight};
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.def("rmsnorm_forward", &rmsnorm_forward, "RMSNorm forward over libmegagemm_hip.so");
    m.def("rmsnorm_backward", &rmsnorm_backward, "RMSNorm backward over libmegagemm_hip.so");
}
