// Python-free check of the C ABI: RMSNorm forward and backward on the GPU against the CPU
// oracle (oracle/mg_oracle.c), in the spirit of the reference's standalone executable
// (rmsnorm_standalone.cu:32-94: 2048 x 4096 fp32, mt19937(1234), uniform(-1,1) for input
// and weight, eps 1e-5, max-abs tolerance 1e-4).  Unlike the reference's, the exit code
// reports the outcome.  Build and run with `make run` from the repository root.
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "megagemm_hip.h"

extern "C" {
void oracle_rmsnorm_fwd_f32(float* y, float* inv_rms, const float* x, const float* w, int64_t rows, int64_t cols,
                            float eps);
void oracle_rmsnorm_bwd_f64(double* dx, double* dw, const float* dy, const float* x, const float* w, int64_t rows,
                            int64_t cols, double eps);
}

#define HIP_OK(call)                                                                             \
    do {                                                                                         \
        hipError_t err_ = (call);                                                                \
        if (err_ != hipSuccess) {                                                                \
            std::fprintf(stderr, "HIP error at %s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(err_)); \
            return 2;                                                                            \
        }                                                                                        \
    } while (0)

#define MG_OK_OR_DIE(call)                                                             \
    do {                                                                               \
        if ((call) != MG_OK) {                                                         \
            std::fprintf(stderr, "library call failed: %s\n", mg_last_error());        \
            return 3;                                                                  \
        }                                                                              \
    } while (0)

int main() {
    const int64_t rows = 2048, cols = 4096;
    const float eps = 1e-5f;
    const size_t n = (size_t)rows * cols;

    std::vector<float> x(n), dy(n), w(cols), y_cpu(n), s_cpu(rows), y_gpu(n), dx_gpu(n), dw_gpu(cols);
    std::vector<double> dx_cpu(n), dw_cpu(cols);
    std::mt19937 gen(1234);
    std::uniform_real_distribution<float> dist(-1.0f, 1.0f);
    for (auto& v : x) v = dist(gen);
    for (auto& v : w) v = dist(gen);
    for (auto& v : dy) v = dist(gen);

    std::printf("CPU oracle ...\n");
    oracle_rmsnorm_fwd_f32(y_cpu.data(), s_cpu.data(), x.data(), w.data(), rows, cols, eps);
    oracle_rmsnorm_bwd_f64(dx_cpu.data(), dw_cpu.data(), dy.data(), x.data(), w.data(), rows, cols, eps);

    float *d_x, *d_dy, *d_w, *d_y, *d_dx, *d_s, *d_part, *d_dw;
    int64_t P = 0, ld = 0;
    MG_OK_OR_DIE(mg_rmsnorm_bwd_workspace(rows, cols, MG_F32, &P, &ld));
    HIP_OK(hipMalloc((void**)&d_x, n * 4));
    HIP_OK(hipMalloc((void**)&d_dy, n * 4));
    HIP_OK(hipMalloc((void**)&d_y, n * 4));
    HIP_OK(hipMalloc((void**)&d_dx, n * 4));
    HIP_OK(hipMalloc((void**)&d_w, cols * 4));
    HIP_OK(hipMalloc((void**)&d_dw, cols * 4));
    HIP_OK(hipMalloc((void**)&d_s, rows * 4));
    HIP_OK(hipMalloc((void**)&d_part, (size_t)P * ld * 4));
    HIP_OK(hipMemcpy(d_x, x.data(), n * 4, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_dy, dy.data(), n * 4, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_w, w.data(), cols * 4, hipMemcpyHostToDevice));

    std::printf("GPU kernels (ABI %d, %lld partial rows) ...\n", mg_abi_version(), (long long)P);
    MG_OK_OR_DIE(mg_rmsnorm_fwd(d_y, d_s, d_x, d_w, rows, cols, eps, MG_F32, nullptr));
    MG_OK_OR_DIE(mg_rmsnorm_bwd(d_dx, d_part, d_dy, d_x, d_w, d_s, rows, cols, MG_F32, P, ld, nullptr));
    MG_OK_OR_DIE(mg_rmsnorm_dw_reduce(d_dw, nullptr, MG_F32, d_part, P, ld, cols, nullptr));
    HIP_OK(hipDeviceSynchronize());
    HIP_OK(hipMemcpy(y_gpu.data(), d_y, n * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(dx_gpu.data(), d_dx, n * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(dw_gpu.data(), d_dw, cols * 4, hipMemcpyDeviceToHost));

    double max_y = 0, max_dx = 0, max_dw = 0, scale_dw = 0;
    for (size_t i = 0; i < n; ++i) {
        max_y = std::fmax(max_y, std::fabs((double)y_cpu[i] - y_gpu[i]));
        max_dx = std::fmax(max_dx, std::fabs(dx_cpu[i] - dx_gpu[i]));
    }
    for (int64_t j = 0; j < cols; ++j) {
        max_dw = std::fmax(max_dw, std::fabs(dw_cpu[j] - dw_gpu[j]));
        scale_dw = std::fmax(scale_dw, std::fabs(dw_cpu[j]));
    }
    std::printf("forward  max |cpu - gpu| = %.3e (tolerance 1e-4)\n", max_y);
    std::printf("backward max |cpu - gpu| = %.3e for dx (tolerance 1e-4), %.3e for dW (tolerance 1e-3 of max |dW| = %.3e)\n",
                max_dx, max_dw, scale_dw);
    const bool ok = max_y < 1e-4 && max_dx < 1e-4 && max_dw < 1e-3 * scale_dw;
    std::printf(ok ? "Validation PASSED\n" : "Validation FAILED\n");

    for (float* p : {d_x, d_dy, d_y, d_dx, d_w, d_dw, d_s, d_part}) (void)hipFree(p);
    return ok ? 0 : 1;
}
