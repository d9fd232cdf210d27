/*
 * megagemm_hip.h -- C ABI of libmegagemm_hip.so (gfx950 / MI355X).
 *
 * The library is the device side of two operators: RMSNorm forward/backward and the
 * SwiGLU activation silu(gate)*up forward/backward.  It replaces, for those operators,
 *   - the CUDA host launchers declared in the reference's src/rmsnorm_kernel.h:9-78,
 *   - the pybind11 module rmsnorm_cuda_ops (pytorch_binding/binding.cpp:16-139),
 *   - the Triton launches in megagemm/swiglu.py:100-107 and :122-129.
 *
 * Conventions (all entry points):
 *   - plain C, no C++ or torch types; every pointer is a DEVICE pointer unless it is
 *     marked "host";
 *   - the caller owns every buffer (inputs, outputs and the dW workspace); the library
 *     never allocates, frees, memsets or synchronises;
 *   - work is enqueued on `stream` (a hipStream_t passed as void*; NULL = the null
 *     stream) of the CURRENT HIP device, asynchronously;
 *   - matrices are row-major and contiguous: element (r, c) of a [rows, cols] matrix is at
 *     index r*cols + c;
 *   - the return value is MG_OK (0) or a negative MG_ERR_* code; on error nothing was
 *     launched and mg_last_error() returns a thread-local, human-readable message;
 *   - arguments are validated before any HIP call, so argument errors are reported on a
 *     machine without a GPU too;
 *   - rows == 0 (or M == 0) is valid and launches no work on x (backward still zeroes dW);
 *   - callable from any thread (the autograd engine calls backward from its own device
 *     thread) and re-entrant: the functions declared here keep no state of their own
 *     between calls except the partials array of mg_rmsnorm_bwd_noalloc, documented
 *     there.  The launch shapes they choose can be overridden for the
 *     whole process through megagemm_hip_tuning.h; nothing else is process-wide.
 */
#ifndef MEGAGEMM_HIP_H
#define MEGAGEMM_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MG_ABI_VERSION 2

/* element types; the reference encodes these in function-name suffixes
 * (_fp32/_fp16/_bf16, src/rmsnorm_kernel.h:9-67) */
enum mg_dtype { MG_F32 = 0, MG_F16 = 1, MG_BF16 = 2 };

enum mg_status {
    MG_OK = 0,
    MG_ERR_INVALID_ARG = -1, /* null pointer, negative size, unknown dtype, misaligned base pointer */
    MG_ERR_UNSUPPORTED = -2, /* size beyond what the kernels index (see each entry point) */
    MG_ERR_HIP = -3          /* a HIP runtime call or the launch itself failed */
};

/* Version of this ABI (MG_ABI_VERSION of the header the library was built from). */
int mg_abi_version(void);

/* Message of the last failing call on the calling thread ("" if none).  Replaces the
 * reference's fprintf(stderr, ...) + `return false` (src/rmsnorm_kernel.cu:533-548). */
const char* mg_last_error(void);

/*
 * RMSNorm forward.  Replaces rmsnorm_cuda_{fp32,fp16,bf16} (src/rmsnorm_kernel.h:9-15,
 * 30-36,51-57; launchers src/rmsnorm_kernel.cu:529-550,577-594,621-638).
 *
 *   s[r]    = 1 / sqrt(mean_c(x[r,c]^2) + eps)        (fp32 accumulation)
 *   y[r,c]  = (x[r,c] * s[r]) * w[c]                  (fp32, rounded once, to nearest even)
 *   inv_rms[r] = s[r]                                 (fp32; pointer may be NULL)
 *
 * x, y: [rows, cols] of `dtype`; w: [cols] of the same dtype.  Any cols >= 1 is accepted
 * (the reference requires cols % 4 == 0 for fp32 and cols % 2 == 0 otherwise and skips a
 * remainder).  Base pointers must be aligned to the element size; nothing more is needed
 * for the fast path.
 * Limits: cols * sizeof(element) < 2^31, rows < 2^31.
 */
int mg_rmsnorm_fwd(void* y, float* inv_rms, const void* x, const void* w,
                   int64_t rows, int64_t cols, float eps, int dtype, void* stream);

/*
 * Workspace shape for mg_rmsnorm_bwd on the current device.  The backward pass writes one
 * fp32 partial dW row per workgroup instead of the reference's atomicAdd epilogue
 * (src/rmsnorm_kernel.cu:315-325,415-425,513-521) and its cudaMemset of dW (:562,606,650).
 *
 *   *num_partials (host, out): number P of partial rows the backward pass should use
 *   *ld           (host, out): leading dimension of the workspace in floats (>= cols)
 *
 * The caller allocates P * ld floats of device memory; it need not be initialised.
 */
int mg_rmsnorm_bwd_workspace(int64_t rows, int64_t cols, int dtype,
                             int64_t* num_partials, int64_t* ld);

/*
 * RMSNorm backward, pass 1.  Replaces rmsnorm_backward_cuda_{fp32,fp16,bf16}
 * (src/rmsnorm_kernel.h:17-25,38-46,59-67; launchers src/rmsnorm_kernel.cu:552-574,
 * 596-618,640-662) together with mg_rmsnorm_dw_reduce.
 *
 *   A[r]      = sum_c dy[r,c] * w[c] * x[r,c]
 *   dx[r,c]   = s[r] * (dy[r,c]*w[c] - x[r,c] * s[r]^2 * A[r] / cols)
 *   dw_partial[p, c] = sum over the rows r that workgroup p owns of dy[r,c] * x[r,c] * s[r]
 *
 * with s = inv_rms as written by mg_rmsnorm_fwd.  dy, x, dx: [rows, cols] of `dtype`;
 * w: [cols]; inv_rms: [rows] fp32; dw_partial: [num_partials, ld] fp32 with ld >= cols and
 * ld % 64 == 0 (mg_rmsnorm_bwd_workspace gives suitable values; any num_partials in
 * [1, 65535] is accepted).  Every element of dw_partial[:, 0:cols] is written, in a fixed
 * order that depends only on (rows, cols, dtype, num_partials) -- and on the launch-shape
 * overrides of megagemm_hip_tuning.h, if a process sets any: results are bit-identical from
 * run to run.  With rows == 0 the workspace is zero-filled.
 * Limits as for mg_rmsnorm_fwd (the reference caps cols at 16384 / 32768).
 * Rows of more than 32 KiB (2-byte types: more than 24 KiB) use a kernel with more than
 * 64 KiB of dynamic LDS, for which the library asks once per GPU on the first such call
 * (hipFuncSetAttribute): make that call before the first stream capture rather than inside it.
 */
int mg_rmsnorm_bwd(void* dx, float* dw_partial, const void* dy, const void* x, const void* w,
                   const float* inv_rms, int64_t rows, int64_t cols, int dtype,
                   int64_t num_partials, int64_t ld, void* stream);

/*
 * RMSNorm backward, pass 2: dW[c] = sum_p dw_partial[p, c], summed in a fixed order in
 * fp32.  Writes dw_f32 ([cols] fp32) when non-NULL and dw_cast ([cols] of `cast_dtype`,
 * rounded to nearest even) when non-NULL; at least one must be given.  dw_cast is what the
 * reference returns as grad_weight (weight dtype, pytorch_binding/binding.cpp:90).
 */
int mg_rmsnorm_dw_reduce(float* dw_f32, void* dw_cast, int cast_dtype, const float* dw_partial,
                         int64_t num_partials, int64_t ld, int64_t cols, void* stream);

/*
 * RMSNorm backward for callers that cannot allocate device memory (code under HIP graph
 * capture, serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  It does what mg_rmsnorm_bwd followed by mg_rmsnorm_dw_reduce does -- dx, and dW
 * as dw_f32 ([cols] fp32) and/or dw_cast ([cols] of `dtype`); at least one of the two -- but
 * keeps the dW partials in a device array of MG_NOALLOC_SCRATCH_BYTES that belongs to the
 * library (one copy per GPU the library runs on, held until the process ends) instead of a
 * workspace of the caller's.  That array is part of the library's code object, so its cost --
 * 16 MiB of device memory on every GPU on which the process uses the library -- is paid by every
 * user of the library from the moment the code object is loaded, whether or not this entry
 * point is ever called.  It calls no allocating routine.  The number of partial rows is
 * the one mg_rmsnorm_bwd_workspace reports, capped at MG_NOALLOC_SCRATCH_BYTES / (4 * ld);
 * results are bit-identical to the two-call sequence with that number of partial rows.
 * cols above MG_NOALLOC_MAX_COLS is rejected with MG_ERR_UNSUPPORTED.
 * All calls on one GPU share that GPU's array, which keeps the last call's contents: nothing
 * in it has to start at zero, because every partial sum a call reads was written by that same
 * call first.  Calls that overlap in time on one GPU (two streams, two threads) race on it;
 * calls ordered by a stream or by events do not.
 * The first call on a GPU looks the array's address up (hipGetSymbolAddress: no allocation,
 * but it may make the runtime load the library's code object); make one call per GPU before
 * the first stream capture rather than inside it.
 */
#define MG_NOALLOC_SCRATCH_BYTES (16 << 20)
#define MG_NOALLOC_MAX_COLS 65536
int mg_rmsnorm_bwd_noalloc(void* dx, float* dw_f32, void* dw_cast, const void* dy, const void* x,
                           const void* w, const float* inv_rms, int64_t rows, int64_t cols, int dtype,
                           void* stream);

/*
 * SwiGLU activation forward.  Replaces the launch of _mg_swiglu_fwd_kernel
 * (megagemm/swiglu.py:18-43, launch :100-107).
 *
 *   gu: [M, 2*H] of `dtype`, each row = [gate(0..H-1) | up(0..H-1)]
 *   h : [M, H],  h[m,j] = (g * sigmoid(g)) * u   with g = gu[m,j], u = gu[m,H+j]  (fp32 math)
 *
 * Any H >= 1.  Limits: M*H < 2^40 elements, H < 2^30.
 */
int mg_swiglu_fwd(void* h, const void* gu, int64_t M, int64_t H, int dtype, void* stream);

/*
 * SwiGLU activation backward.  Replaces the launch of _mg_swiglu_bwd_kernel
 * (megagemm/swiglu.py:46-79, launch :122-129).
 *
 *   dh : [M, H];  gu: [M, 2*H] (the forward input);  dgu: [M, 2*H] = [d_gate | d_up]
 *   sig = sigmoid(g);  d_up = dh * g * sig;  d_gate = dh * u * sig * (1 + g * (1 - sig))
 */
int mg_swiglu_bwd(void* dgu, const void* dh, const void* gu, int64_t M, int64_t H, int dtype,
                  void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MEGAGEMM_HIP_H */
