/*
 * mg_oracle.c -- CPU restatement of the reference's RMSNorm and SwiGLU arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing that ships (the mgrrmsnorm_amd package, the HIP
 * library) may call, link or import this file; it exists so that tests, the smoke check
 * and the CPU leg of the benchmark have an independent answer to compare against.
 *
 * Two flavours of every function:
 *   *_f32  follows the reference's own arithmetic literally (fp32 accumulation in index
 *          order), and is what the CPU baseline timing runs;
 *   *_f64  evaluates the same formulas in double precision from fp32 inputs and returns
 *          doubles: the "exact" answer that kernel outputs are compared with after one
 *          rounding to the output type.
 *
 * Reference lines restated:
 *   RMSNorm forward   rmsnorm_standalone.cu:17-30 (rmsnorm_cpu), test_rmsnorm.py:55-56
 *   RMSNorm backward  src/rmsnorm_kernel.cu:258-312 (A, term2, dx, dW), README.md:114-123
 *   SwiGLU forward    megagemm/swiglu.py:35-41, benchmark_swiglu.py:57
 *   SwiGLU backward   megagemm/swiglu.py:64-79
 *
 * Pinned by (tests/test_oracle_*.py): Decimal-arithmetic golden vectors with finite-
 * difference gradients (tests/golden/), closed-form known answers, torch float64
 * autograd, torch.nn.functional.rms_norm / silu, and brute-force loops on tiny inputs.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

/* ---------------------------------------------------------------- RMSNorm forward */

/* rmsnorm_standalone.cu:17-30: sum_sq in fp32 in column order, rms = 1/sqrtf(sum/cols+eps),
 * out = in * rms * weight.  inv_rms (may be NULL) receives rms per row, as the kernel's
 * side output does (src/rmsnorm_kernel.cu:83). */
void oracle_rmsnorm_fwd_f32(float* y, float* inv_rms, const float* x, const float* w,
                            int64_t rows, int64_t cols, float eps) {
    for (int64_t i = 0; i < rows; ++i) {
        const float* xr = x + i * cols;
        float sum_sq = 0.0f;
        for (int64_t j = 0; j < cols; ++j) sum_sq += xr[j] * xr[j];
        const float rms = 1.0f / sqrtf(sum_sq / (float)cols + eps);
        if (inv_rms) inv_rms[i] = rms;
        for (int64_t j = 0; j < cols; ++j) y[i * cols + j] = xr[j] * rms * w[j];
    }
}

void oracle_rmsnorm_fwd_f64(double* y, double* inv_rms, const float* x, const float* w,
                            int64_t rows, int64_t cols, double eps) {
    for (int64_t i = 0; i < rows; ++i) {
        const float* xr = x + i * cols;
        double sum_sq = 0.0;
        for (int64_t j = 0; j < cols; ++j) sum_sq += (double)xr[j] * (double)xr[j];
        const double rms = 1.0 / sqrt(sum_sq / (double)cols + eps);
        if (inv_rms) inv_rms[i] = rms;
        for (int64_t j = 0; j < cols; ++j) y[i * cols + j] = (double)xr[j] * rms * (double)w[j];
    }
}

/* --------------------------------------------------------------- RMSNorm backward */

/* src/rmsnorm_kernel.cu:258-312 with the row's inv_rms taken as an input, exactly as the
 * kernel takes it:  A = sum dy*w*x;  term2 = A*s*s/cols;  dx = s*(dy*w - x*term2);
 * dW[j] += dy*x*s.  dW must hold `cols` floats and is overwritten. */
void oracle_rmsnorm_bwd_f32(float* dx, float* dw, const float* dy, const float* x, const float* w,
                            const float* inv_rms, int64_t rows, int64_t cols) {
    for (int64_t j = 0; j < cols; ++j) dw[j] = 0.0f;
    for (int64_t i = 0; i < rows; ++i) {
        const float* xr = x + i * cols;
        const float* gr = dy + i * cols;
        const float s = inv_rms[i];
        float a = 0.0f;
        for (int64_t j = 0; j < cols; ++j) {
            a += gr[j] * w[j] * xr[j];
            dw[j] += gr[j] * xr[j] * s;
        }
        const float term2 = a * (s * s) / (float)cols;
        for (int64_t j = 0; j < cols; ++j) dx[i * cols + j] = s * (gr[j] * w[j] - xr[j] * term2);
    }
}

/* Same algebra in double, with s recomputed from x and eps in double (so the result does
 * not inherit the forward pass's fp32 rounding of inv_rms). */
void oracle_rmsnorm_bwd_f64(double* dx, double* dw, const float* dy, const float* x, const float* w,
                            int64_t rows, int64_t cols, double eps) {
    for (int64_t j = 0; j < cols; ++j) dw[j] = 0.0;
    for (int64_t i = 0; i < rows; ++i) {
        const float* xr = x + i * cols;
        const float* gr = dy + i * cols;
        double sum_sq = 0.0, a = 0.0;
        for (int64_t j = 0; j < cols; ++j) sum_sq += (double)xr[j] * (double)xr[j];
        const double s = 1.0 / sqrt(sum_sq / (double)cols + eps);
        for (int64_t j = 0; j < cols; ++j) {
            const double g = (double)gr[j], xv = (double)xr[j];
            a += g * (double)w[j] * xv;
            dw[j] += g * xv * s;
        }
        const double term2 = a * (s * s) / (double)cols;
        for (int64_t j = 0; j < cols; ++j)
            dx[i * cols + j] = s * ((double)gr[j] * (double)w[j] - (double)xr[j] * term2);
    }
}

/* ------------------------------------------------------------------------ SwiGLU */

/* megagemm/swiglu.py:35-41: row m of gu is [gate(0..H-1) | up(0..H-1)];
 * h = (gate * sigmoid(gate)) * up. */
void oracle_swiglu_fwd_f32(float* h, const float* gu, int64_t M, int64_t H) {
    for (int64_t m = 0; m < M; ++m) {
        const float* g = gu + m * 2 * H;
        const float* u = g + H;
        for (int64_t j = 0; j < H; ++j) {
            const float sig = 1.0f / (1.0f + expf(-g[j]));
            h[m * H + j] = (g[j] * sig) * u[j];
        }
    }
}

void oracle_swiglu_fwd_f64(double* h, const float* gu, int64_t M, int64_t H) {
    for (int64_t m = 0; m < M; ++m) {
        const float* g = gu + m * 2 * H;
        const float* u = g + H;
        for (int64_t j = 0; j < H; ++j) {
            const double gd = (double)g[j];
            const double sig = 1.0 / (1.0 + exp(-gd));
            h[m * H + j] = (gd * sig) * (double)u[j];
        }
    }
}

/* megagemm/swiglu.py:64-79: d_up = dh * gate*sig;  d_gate = dh * up * sig*(1 + gate*(1-sig));
 * output row = [d_gate | d_up]. */
void oracle_swiglu_bwd_f32(float* dgu, const float* dh, const float* gu, int64_t M, int64_t H) {
    for (int64_t m = 0; m < M; ++m) {
        const float* g = gu + m * 2 * H;
        const float* u = g + H;
        float* dg = dgu + m * 2 * H;
        float* du = dg + H;
        for (int64_t j = 0; j < H; ++j) {
            const float d = dh[m * H + j];
            const float sig = 1.0f / (1.0f + expf(-g[j]));
            du[j] = d * (g[j] * sig);
            dg[j] = d * u[j] * (sig * (1.0f + g[j] * (1.0f - sig)));
        }
    }
}

void oracle_swiglu_bwd_f64(double* dgu, const float* dh, const float* gu, int64_t M, int64_t H) {
    for (int64_t m = 0; m < M; ++m) {
        const float* g = gu + m * 2 * H;
        const float* u = g + H;
        double* dg = dgu + m * 2 * H;
        double* du = dg + H;
        for (int64_t j = 0; j < H; ++j) {
            const double d = (double)dh[m * H + j], gd = (double)g[j];
            const double sig = 1.0 / (1.0 + exp(-gd));
            du[j] = d * (gd * sig);
            dg[j] = d * (double)u[j] * (sig * (1.0 + gd * (1.0 - sig)));
        }
    }
}
