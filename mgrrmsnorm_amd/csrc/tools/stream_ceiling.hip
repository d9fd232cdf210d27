// stream_ceiling: what can this GPU stream?  Plain read / write / copy / 2-reads-1-write
// kernels built from the same 16-byte buffer accesses as the RMSNorm and SwiGLU kernels,
// over buffers that rotate so that nothing is cache resident.  The figures bound what any
// kernel with the same read/write mix can reach and are what the operators' GB/s should be
// judged against on a given machine.
//
//   hipcc -O3 --offload-arch=gfx950 -Xclang -target-feature -Xclang -packed-fp32-ops \
//         mgrrmsnorm_amd/csrc/tools/stream_ceiling.hip -o stream_ceiling && ./stream_ceiling
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <vector>

typedef unsigned int u32;
typedef u32 u32x4 __attribute__((ext_vector_type(4)));

#define CK(x)                                                                        \
    do {                                                                             \
        hipError_t e_ = (x);                                                         \
        if (e_ != hipSuccess) {                                                      \
            std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
            std::exit(1);                                                            \
        }                                                                            \
    } while (0)

__device__ inline __amdgpu_buffer_rsrc_t rsrc(const void* p, u32 bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}

enum Mode { COPY = 0, READ = 1, WRITE = 2, READ2_WRITE1 = 3 };

// One workgroup of 256 threads moves one contiguous chunk of 256*U*16 bytes.
template <int U, int POLICY, int MODE>
__global__ void __launch_bounds__(256)
stream_kernel(const char* __restrict__ a, const char* __restrict__ b, char* __restrict__ d, long nchunks, u32* sink) {
    const long chunk = 256L * U * 16;
    const long c = blockIdx.x;
    if (c >= nchunks) return;
    const auto ra = rsrc(a + c * chunk, (u32)chunk);
    const auto rb = rsrc(b + c * chunk, (u32)chunk);
    const auto rd = rsrc(d + c * chunk, (u32)chunk);
    u32x4 v[U], w[U];
#pragma unroll
    for (int i = 0; i < U; ++i) {
        const int off = (threadIdx.x + i * 256) * 16;
        v[i] = (MODE == WRITE) ? u32x4{(u32)c, 1u, 2u, 3u} : __builtin_amdgcn_raw_buffer_load_b128(ra, off, 0, POLICY);
        if (MODE == READ2_WRITE1) w[i] = __builtin_amdgcn_raw_buffer_load_b128(rb, off, 0, POLICY);
    }
    u32 acc = 0;
#pragma unroll
    for (int i = 0; i < U; ++i) {
        const int off = (threadIdx.x + i * 256) * 16;
        if (MODE == READ2_WRITE1) v[i] += w[i];
        if (MODE == READ) acc += v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
        else __builtin_amdgcn_raw_buffer_store_b128(v[i], rd, off, 0, POLICY);
    }
    if (MODE == READ && acc == 0x12345678u) sink[0] = acc;  // keeps the loads alive
}

struct Buffers {
    std::vector<char*> a, b, d;
    size_t bytes;
};

template <int U, int POLICY, int MODE>
double time_us(const Buffers& B, hipStream_t st, u32* sink) {
    const long nchunks = (long)(B.bytes / (256L * U * 16));
    const int n = (int)B.a.size();
    const int iters = B.bytes >= (256u << 20) ? 20 : 200;
    auto launch = [&](int i) {
        stream_kernel<U, POLICY, MODE><<<dim3((unsigned)nchunks), dim3(256), 0, st>>>(B.a[i % n], B.b[i % n], B.d[i % n], nchunks, sink);
    };
    for (int i = 0; i < 5; ++i) launch(i);
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    double best = 1e30;
    for (int r = 0; r < 3; ++r) {
        CK(hipEventRecord(e0, st));
        for (int i = 0; i < iters; ++i) launch(i);
        CK(hipEventRecord(e1, st));
        CK(hipEventSynchronize(e1));
        float ms = 0;
        CK(hipEventElapsedTime(&ms, e0, e1));
        if (ms * 1e3 / iters < best) best = ms * 1e3 / iters;
    }
    CK(hipGetLastError());
    CK(hipEventDestroy(e0));
    CK(hipEventDestroy(e1));
    return best;
}

template <int U, int POLICY>
void report(const Buffers& B, hipStream_t st, u32* sink) {
    const double mb = B.bytes / 1e6;
    const double tc = time_us<U, POLICY, COPY>(B, st, sink), tr = time_us<U, POLICY, READ>(B, st, sink),
                 tw = time_us<U, POLICY, WRITE>(B, st, sink), t3 = time_us<U, POLICY, READ2_WRITE1>(B, st, sink);
    std::printf("  %4d B/thread %-12s read %8.1f us %5.0f GB/s | write %8.1f us %5.0f GB/s | copy %8.1f us %5.0f GB/s | 2r+1w %8.1f us %5.0f GB/s\n",
                U * 16, POLICY == 2 ? "non-temporal" : "default", tr, mb / tr * 1e3, tw, mb / tw * 1e3, tc, 2 * mb / tc * 1e3,
                t3, 3 * mb / t3 * 1e3);
    std::fflush(stdout);
}

int main() {
    hipStream_t st;
    CK(hipStreamCreate(&st));
    u32* sink;
    CK(hipMalloc(&sink, 4));
    for (size_t bytes : {size_t(32) << 20, size_t(256) << 20, size_t(1) << 30}) {
        Buffers B;
        B.bytes = bytes;
        const int n = bytes >= (size_t(1) << 30) ? 2 : bytes >= (256u << 20) ? 3 : 12;  // >= 1 GiB in rotation
        for (int i = 0; i < n; ++i) {
            char *p, *q, *r;
            CK(hipMalloc(&p, bytes)); CK(hipMalloc(&q, bytes)); CK(hipMalloc(&r, bytes));
            CK(hipMemset(p, 1, bytes)); CK(hipMemset(q, 2, bytes)); CK(hipMemset(r, 3, bytes));
            B.a.push_back(p); B.b.push_back(q); B.d.push_back(r);
        }
        CK(hipDeviceSynchronize());
        std::printf("%zu MiB per tensor, %d buffer sets in rotation\n", bytes >> 20, n);
        report<1, 0>(B, st, sink);
        report<2, 0>(B, st, sink);
        report<4, 0>(B, st, sink);
        report<1, 2>(B, st, sink);
        report<2, 2>(B, st, sink);
        report<4, 2>(B, st, sink);
        for (auto p : B.a) CK(hipFree(p));
        for (auto p : B.b) CK(hipFree(p));
        for (auto p : B.d) CK(hipFree(p));
    }
    return 0;
}
