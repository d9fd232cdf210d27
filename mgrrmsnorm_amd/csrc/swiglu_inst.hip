// SwiGLU activation launchers (all element types) and the dW second pass.
#include "megagemm_hip.h"
#include "mg_launch.hpp"
#include "rmsnorm_kernels.hpp"
#include "swiglu_kernels.hpp"

#include <atomic>

namespace mg {
namespace {

// Zero-fill of the partial matrix for rows == 0 (a kernel rather than a memset node, so
// that the call behaves the same under stream capture).
__global__ void __launch_bounds__(256) fill_zero_f32(float* __restrict__ p, long n) {
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) p[i] = 0.0f;
}

// Plain 16-byte copy, one vector per thread: the yardstick the HBM traffic counters are
// calibrated against (its traffic is exactly 2 * bytes).
__global__ void __launch_bounds__(256) copy_vec16(u32x4* __restrict__ dst, const u32x4* __restrict__ src, long n) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = src[i];
}

// Streaming yardsticks with the accesses the operators use (16-byte buffer loads/stores with
// the non-temporal bit, 4 KiB per workgroup): a copy (b == nullptr) or dst = a + b word by
// word (two reads, one write).  What these reach at a given size bounds any kernel with the
// same read/write mix.
template <bool TWO_READS>
__global__ void __launch_bounds__(256) stream_probe(char* __restrict__ dst, const char* __restrict__ a,
                                                    const char* __restrict__ b, long bytes, int xcd_group) {
    const long chunk = 256L * 16;
    const long c = xcd_remap(blockIdx.x, gridDim.x, xcd_group);
    const long left = bytes - c * chunk;
    const u32 n = left >= chunk ? (u32)chunk : (u32)left;
    const u32 off = threadIdx.x * 16u;
    Words<4> v = buf_load<4, kStream>(make_rsrc(a + c * chunk, n), off);
    if constexpr (TWO_READS) {
        const Words<4> w = buf_load<4, kStream>(make_rsrc(b + c * chunk, n), off);
#pragma unroll
        for (int j = 0; j < 4; ++j) v.v[j] += w.v[j];
    }
    buf_store<4, kStream>(make_rsrc(dst + c * chunk, n), off, v);
}

// The same traffic with the operators' work split: a workgroup of BLOCK threads (256 for rows of
// up to 4 KiB, 512 up to 16 KiB, 1024 beyond) owns whole rows of `row_bytes` (at most 64 KiB), ITEMS vectors per
// thread, and walks the rows blockIdx.x,
// blockIdx.x + gridDim.x, ... with the next row requested before the current one is stored --
// a grid of `rows` workgroups takes one row each, a smaller grid is persistent like backward
// pass 1.  What this reaches bounds a kernel that must see a whole row before it can store.
template <bool TWO_READS, int BLOCK, int ITEMS>
__global__ void __launch_bounds__(BLOCK) row_probe(char* __restrict__ dst, const char* __restrict__ a,
                                                    const char* __restrict__ b, long rows, u32 row_bytes) {
    const u32 tid = threadIdx.x;
    Words<4> av[ITEMS], bv[ITEMS];
    auto request = [&](long row, Words<4> (&x)[ITEMS], Words<4> (&y)[ITEMS]) {
        const bool live = row < rows;
        const long base = live ? row * (long)row_bytes : 0;
        const rsrc_t ra = make_rsrc(a + base, live ? row_bytes : 0u);
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) x[i] = buf_load<4, kStream>(ra, (tid + i * (u32)BLOCK) * 16u);
        if constexpr (TWO_READS) {
            const rsrc_t rb = make_rsrc(b + base, live ? row_bytes : 0u);
#pragma unroll
            for (int i = 0; i < ITEMS; ++i) y[i] = buf_load<4, kStream>(rb, (tid + i * (u32)BLOCK) * 16u);
        }
    };
    long row = blockIdx.x;
    request(row, av, bv);
    for (; row < rows; row += gridDim.x) {
        Words<4> na[ITEMS], nb[ITEMS];
        request(row + gridDim.x, na, nb);
        const rsrc_t rd = make_rsrc(dst + row * (long)row_bytes, row_bytes);
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            if constexpr (TWO_READS) {
#pragma unroll
                for (int j = 0; j < 4; ++j) av[i].v[j] += bv[i].v[j];
            }
            buf_store<4, kStream>(rd, (tid + i * (u32)BLOCK) * 16u, av[i]);
        }
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) { av[i] = na[i]; if constexpr (TWO_READS) bv[i] = nb[i]; }
    }
}

// units handled by one launch stay below 2^31 so that 32-bit indices cannot wrap
constexpr long kMaxUnitsPerLaunchDefault = 1L << 31;
std::atomic<long> g_max_units{kMaxUnitsPerLaunchDefault};

// rows one launch may cover when a row has `units_per_row` units (at least one row)
long rows_per_launch_for(long units_per_row) {
    const long r = g_max_units.load(std::memory_order_relaxed) / units_per_row;
    return r < 1 ? 1 : r;
}

template <typename T, int UNROLL>
hipError_t fwd_vec(int xg, void* h, const void* gu, long M, long H, hipStream_t s) {
    const long nvr = H * (long)sizeof(T) / 16;
    const long rows_per_launch = rows_per_launch_for(nvr);
    const FastDiv fd = make_fastdiv((uint32_t)nvr);
    for (long r0 = 0; r0 < M; r0 += rows_per_launch) {
        const long m = (M - r0) < rows_per_launch ? (M - r0) : rows_per_launch;
        const uint32_t total = (uint32_t)(m * nvr);
        const unsigned grid = (unsigned)((total + 256u * UNROLL - 1) / (256u * UNROLL));
        hipError_t e = launch(swiglu_fwd_vec<T, UNROLL>, dim3(grid), dim3(256), 0, s,
            (T*)h + r0 * H, (const T*)gu + r0 * 2 * H, total, fd, xg);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

template <typename T, int UNROLL>
hipError_t bwd_vec(int xg, void* dgu, const void* dh, const void* gu, long M, long H, hipStream_t s) {
    const long nvr = H * (long)sizeof(T) / 16;
    const long rows_per_launch = rows_per_launch_for(nvr);
    const FastDiv fd = make_fastdiv((uint32_t)nvr);
    for (long r0 = 0; r0 < M; r0 += rows_per_launch) {
        const long m = (M - r0) < rows_per_launch ? (M - r0) : rows_per_launch;
        const uint32_t total = (uint32_t)(m * nvr);
        const unsigned grid = (unsigned)((total + 256u * UNROLL - 1) / (256u * UNROLL));
        hipError_t e = launch(swiglu_bwd_vec<T, UNROLL>, dim3(grid), dim3(256), 0, s,
            (T*)dgu + r0 * 2 * H, (const T*)dh + r0 * H, (const T*)gu + r0 * 2 * H, total, fd, xg);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

// rows one launch of the ragged kernels may cover: as above, and all byte offsets below 2^31
long ragged_rows_per_launch(long nvr, long half_bytes) {
    long r = rows_per_launch_for(nvr);
    const long by_bytes = (1L << 31) / (2 * half_bytes);
    if (r > by_bytes) r = by_bytes;
    return r < 1 ? 1 : r;
}

template <typename T>
hipError_t fwd_ragged(int xg, void* h, const void* gu, long M, long H, hipStream_t s) {
    const long half_bytes = H * (long)sizeof(T);
    const long nvr = (half_bytes + 15) / 16;
    const long rows_per_launch = ragged_rows_per_launch(nvr, half_bytes);
    const FastDiv fd = make_fastdiv((uint32_t)nvr);
    for (long r0 = 0; r0 < M; r0 += rows_per_launch) {
        const long m = (M - r0) < rows_per_launch ? (M - r0) : rows_per_launch;
        const uint32_t total = (uint32_t)(m * nvr);
        hipError_t e = launch(swiglu_fwd_ragged<T>, dim3((total + 255u) / 256u), dim3(256), 0, s,
            (T*)h + r0 * H, (const T*)gu + r0 * 2 * H, (uint32_t)m, total, (uint32_t)half_bytes, fd, xg);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

template <typename T>
hipError_t bwd_ragged(int xg, void* dgu, const void* dh, const void* gu, long M, long H, hipStream_t s) {
    const long half_bytes = H * (long)sizeof(T);
    const long nvr = (half_bytes + 15) / 16;
    const long rows_per_launch = ragged_rows_per_launch(nvr, half_bytes);
    const FastDiv fd = make_fastdiv((uint32_t)nvr);
    for (long r0 = 0; r0 < M; r0 += rows_per_launch) {
        const long m = (M - r0) < rows_per_launch ? (M - r0) : rows_per_launch;
        const uint32_t total = (uint32_t)(m * nvr);
        hipError_t e = launch(swiglu_bwd_ragged<T>, dim3((total + 255u) / 256u), dim3(256), 0, s,
            (T*)dgu + r0 * 2 * H, (const T*)dh + r0 * H, (const T*)gu + r0 * 2 * H, (uint32_t)m, total,
            (uint32_t)half_bytes, fd, xg);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

template <typename T>
hipError_t fwd_gen(void* h, const void* gu, long M, long H, hipStream_t s) {
    const long rows_per_launch = rows_per_launch_for(H);
    const FastDiv fd = make_fastdiv((uint32_t)H);
    for (long r0 = 0; r0 < M; r0 += rows_per_launch) {
        const long m = (M - r0) < rows_per_launch ? (M - r0) : rows_per_launch;
        const uint32_t total = (uint32_t)(m * H);
        hipError_t e = launch(swiglu_fwd_generic<T>, dim3((total + 255u) / 256u), dim3(256), 0, s,
            (T*)h + r0 * H, (const T*)gu + r0 * 2 * H, total, fd);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

template <typename T>
hipError_t bwd_gen(void* dgu, const void* dh, const void* gu, long M, long H, hipStream_t s) {
    const long rows_per_launch = rows_per_launch_for(H);
    const FastDiv fd = make_fastdiv((uint32_t)H);
    for (long r0 = 0; r0 < M; r0 += rows_per_launch) {
        const long m = (M - r0) < rows_per_launch ? (M - r0) : rows_per_launch;
        const uint32_t total = (uint32_t)(m * H);
        hipError_t e = launch(swiglu_bwd_generic<T>, dim3((total + 255u) / 256u), dim3(256), 0, s,
            (T*)dgu + r0 * 2 * H, (const T*)dh + r0 * H, (const T*)gu + r0 * 2 * H, total, fd);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

template <typename T>
hipError_t fwd_t(int mode, int unroll, int xg, void* h, const void* gu, long M, long H, hipStream_t s) {
    if (mode == kSwigluElementwise) return fwd_gen<T>(h, gu, M, H, s);
    if (mode == kSwigluRagged) return fwd_ragged<T>(xg, h, gu, M, H, s);
    switch (unroll) {
        case 1: return fwd_vec<T, 1>(xg, h, gu, M, H, s);
        case 2: return fwd_vec<T, 2>(xg, h, gu, M, H, s);
        case 4: return fwd_vec<T, 4>(xg, h, gu, M, H, s);
        case 8: return fwd_vec<T, 8>(xg, h, gu, M, H, s);
        default: return hipErrorInvalidValue;
    }
}

template <typename T>
hipError_t bwd_t(int mode, int unroll, int xg, void* dgu, const void* dh, const void* gu, long M, long H,
                 hipStream_t s) {
    if (mode == kSwigluElementwise) return bwd_gen<T>(dgu, dh, gu, M, H, s);
    if (mode == kSwigluRagged) return bwd_ragged<T>(xg, dgu, dh, gu, M, H, s);
    switch (unroll) {
        case 1: return bwd_vec<T, 1>(xg, dgu, dh, gu, M, H, s);
        case 2: return bwd_vec<T, 2>(xg, dgu, dh, gu, M, H, s);
        case 4: return bwd_vec<T, 4>(xg, dgu, dh, gu, M, H, s);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

void set_swiglu_max_units(long units) {
    g_max_units.store(units >= 1 && units <= kMaxUnitsPerLaunchDefault ? units : kMaxUnitsPerLaunchDefault);
}

hipError_t launch_swiglu_fwd(int dtype, int mode, int unroll, int xg, void* h, const void* gu, long M, long H,
                             hipStream_t s) {
    switch (dtype) {
        case MG_F32: return fwd_t<float>(mode, unroll, xg, h, gu, M, H, s);
        case MG_F16: return fwd_t<half_t>(mode, unroll, xg, h, gu, M, H, s);
        case MG_BF16: return fwd_t<bf16_t>(mode, unroll, xg, h, gu, M, H, s);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_swiglu_bwd(int dtype, int mode, int unroll, int xg, void* dgu, const void* dh, const void* gu,
                             long M, long H, hipStream_t s) {
    switch (dtype) {
        case MG_F32: return bwd_t<float>(mode, unroll, xg, dgu, dh, gu, M, H, s);
        case MG_F16: return bwd_t<half_t>(mode, unroll, xg, dgu, dh, gu, M, H, s);
        case MG_BF16: return bwd_t<bf16_t>(mode, unroll, xg, dgu, dh, gu, M, H, s);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_dw_reduce(float* dw_f32, void* dw_cast, int cast_dtype, const float* part, int P, int ld,
                            int cols, hipStream_t s) {
    const dim3 grid((unsigned)((cols + kReduceCols - 1) / kReduceCols)), block(256);
    if (dw_cast == nullptr || cast_dtype == MG_F32)
        return launch(rmsnorm_dw_reduce<float>, grid, block, 0, s, dw_f32, (float*)dw_cast, part, P, ld, cols);
    if (cast_dtype == MG_F16)
        return launch(rmsnorm_dw_reduce<half_t>, grid, block, 0, s, dw_f32, (half_t*)dw_cast, part, P, ld, cols);
    if (cast_dtype == MG_BF16)
        return launch(rmsnorm_dw_reduce<bf16_t>, grid, block, 0, s, dw_f32, (bf16_t*)dw_cast, part, P, ld, cols);
    return hipErrorInvalidValue;
}

hipError_t launch_copy(void* dst, const void* src, long bytes, hipStream_t s) {
    const long n = bytes / 16;
    if (n <= 0) return hipSuccess;
    return launch(copy_vec16, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (u32x4*)dst, (const u32x4*)src, n);
}

hipError_t launch_stream_probe(void* dst, const void* a, const void* b, long bytes, int xcd_group, hipStream_t s) {
    const long n = (bytes + 4095) / 4096;
    if (n <= 0) return hipSuccess;
    if (b == nullptr)
        return launch(stream_probe<false>, dim3((unsigned)n), dim3(256), 0, s, (char*)dst, (const char*)a,
                      (const char*)nullptr, bytes, xcd_group);
    return launch(stream_probe<true>, dim3((unsigned)n), dim3(256), 0, s, (char*)dst, (const char*)a, (const char*)b,
                  bytes, xcd_group);
}

template <bool TWO_READS>
hipError_t row_probe_by_shape(unsigned grid, void* dst, const void* a, const void* b, long rows, u32 row_bytes,
                              hipStream_t s) {
#define MG_ROW_PROBE(B, I) \
    return launch(row_probe<TWO_READS, B, I>, dim3(grid), dim3(B), 0, s, (char*)dst, (const char*)a, (const char*)b, rows, row_bytes)
    const u32 nvec = row_bytes / 16u;
    if (nvec <= 256) MG_ROW_PROBE(256, 1);
    else if (nvec <= 512) MG_ROW_PROBE(512, 1);
    else if (nvec <= 1024) MG_ROW_PROBE(512, 2);
    else if (nvec <= 2048) MG_ROW_PROBE(1024, 2);
    else MG_ROW_PROBE(1024, 4);
#undef MG_ROW_PROBE
}

hipError_t launch_row_probe(void* dst, const void* a, const void* b, long rows, long row_bytes, long workgroups,
                            hipStream_t s) {
    if (rows <= 0) return hipSuccess;
    const unsigned grid = (unsigned)(workgroups > 0 && workgroups < rows ? workgroups : rows);
    return b == nullptr ? row_probe_by_shape<false>(grid, dst, a, b, rows, (u32)row_bytes, s)
                        : row_probe_by_shape<true>(grid, dst, a, b, rows, (u32)row_bytes, s);
}

hipError_t launch_fill_zero(float* p, long n, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    const long blocks = (n + 255) / 256;
    return launch(fill_zero_f32, dim3((unsigned)(blocks < (1L << 20) ? blocks : (1L << 20))), dim3(256), 0, s, p, n);
}

}  // namespace mg
