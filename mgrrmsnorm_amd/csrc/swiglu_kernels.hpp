// SwiGLU activation kernels for gfx950: h = silu(gate) * up over a fused [M, 2H] =
// [gate | up] matrix, and its backward.  Pure streaming work: every thread handles
// UNROLL independent 16-byte vectors of the flat [M, H] index space, all loads issued
// before the first use; (row, column) come from one multiply-high division.
#pragma once
#include "mg_device.hpp"
#include "mg_divmod.hpp"

namespace mg {

// 16-byte global accesses with the non-temporal hint: every element is touched once.
__device__ __forceinline__ Words<4> gload4(const void* p) {
    u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    Words<4> o; o.v[0] = t.x; o.v[1] = t.y; o.v[2] = t.z; o.v[3] = t.w; return o;
}
__device__ __forceinline__ void gstore4(void* p, const Words<4>& w) {
    u32x4 t = {w.v[0], w.v[1], w.v[2], w.v[3]};
    __builtin_nontemporal_store(t, reinterpret_cast<u32x4*>(p));
}

// total = M * nvr vectors, nvr = H * sizeof(T) / 16 vectors per half row.
template <typename T, int UNROLL>
__global__ void __launch_bounds__(256)
swiglu_fwd_vec(T* __restrict__ h, const T* __restrict__ gu, uint32_t total, FastDiv nvr, int xcd_group) {
    constexpr int EPV = 16 / (int)sizeof(T);
    const uint32_t v0 = (uint32_t)xcd_remap(blockIdx.x, gridDim.x, xcd_group) * (256u * UNROLL) + threadIdx.x;
    const char* in = reinterpret_cast<const char*>(gu);
    char* out = reinterpret_cast<char*>(h);

    Words<4> g[UNROLL], u[UNROLL];
    bool ok[UNROLL];
#pragma unroll
    for (int k = 0; k < UNROLL; ++k) {
        const uint32_t v = v0 + k * 256u;
        ok[k] = v < total;
        if (ok[k]) {
            const uint32_t row = fastdiv(v, nvr);
            const uint32_t col = v - row * nvr.d;
            const uint64_t gi = (uint64_t)row * (2ull * nvr.d) + col;
            g[k] = gload4(in + gi * 16);
            u[k] = gload4(in + (gi + nvr.d) * 16);
        }
    }
#pragma unroll
    for (int k = 0; k < UNROLL; ++k) {
        if (ok[k]) {
            float gf[EPV], uf[EPV], o[EPV];
            unpack_vec<T, 4>(g[k], gf);
            unpack_vec<T, 4>(u[k], uf);
#pragma unroll
            for (int e = 0; e < EPV; ++e) o[e] = (gf[e] * fast_sigmoid(gf[e])) * uf[e];
            gstore4(out + (uint64_t)(v0 + k * 256u) * 16, pack_vec<T, 4>(o));
        }
    }
}

template <typename T, int UNROLL>
__global__ void __launch_bounds__(256)
swiglu_bwd_vec(T* __restrict__ dgu, const T* __restrict__ dh, const T* __restrict__ gu, uint32_t total,
               FastDiv nvr, int xcd_group) {
    constexpr int EPV = 16 / (int)sizeof(T);
    const uint32_t v0 = (uint32_t)xcd_remap(blockIdx.x, gridDim.x, xcd_group) * (256u * UNROLL) + threadIdx.x;
    const char* in = reinterpret_cast<const char*>(gu);
    const char* din = reinterpret_cast<const char*>(dh);
    char* out = reinterpret_cast<char*>(dgu);

    Words<4> g[UNROLL], u[UNROLL], d[UNROLL];
    uint64_t gi[UNROLL];
    bool ok[UNROLL];
#pragma unroll
    for (int k = 0; k < UNROLL; ++k) {
        const uint32_t v = v0 + k * 256u;
        ok[k] = v < total;
        gi[k] = 0;
        if (ok[k]) {
            const uint32_t row = fastdiv(v, nvr);
            const uint32_t col = v - row * nvr.d;
            gi[k] = (uint64_t)row * (2ull * nvr.d) + col;
            g[k] = gload4(in + gi[k] * 16);
            u[k] = gload4(in + (gi[k] + nvr.d) * 16);
            d[k] = gload4(din + (uint64_t)v * 16);
        }
    }
#pragma unroll
    for (int k = 0; k < UNROLL; ++k) {
        if (ok[k]) {
            float gf[EPV], uf[EPV], df[EPV], og[EPV], ou[EPV];
            unpack_vec<T, 4>(g[k], gf);
            unpack_vec<T, 4>(u[k], uf);
            unpack_vec<T, 4>(d[k], df);
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                const float sg = fast_sigmoid(gf[e]);
                ou[e] = df[e] * (gf[e] * sg);
                og[e] = (df[e] * uf[e]) * (sg * __builtin_fmaf(gf[e], 1.0f - sg, 1.0f));
            }
            gstore4(out + gi[k] * 16, pack_vec<T, 4>(og));
            gstore4(out + (gi[k] + nvr.d) * 16, pack_vec<T, 4>(ou));
        }
    }
}

// Any H and any element-aligned base: 16-byte buffer accesses at whatever alignment the row
// gives them.  A half row of H elements is cut into nvr = ceil(H * sizeof(T) / 16) vectors;
// the last one reaches past the half row (into the `up` half, the next row, or -- at the end
// of the launch's rows -- out of the buffer, where loads return 0), which is harmless for
// loads since nothing is reduced, and is stored in pieces (store_row_vector).  Only an
// element in a half dword that the range check drops at the very end of the buffer needs a
// 2-byte load of its own.  total = rows * nvr vectors per launch; all byte offsets of a
// launch stay below 2^31.  Outputs take the default cache policy: rows share cache lines
// between store instructions, which the L2 merges.
template <typename T>
__device__ __forceinline__ Words<4> load_half_row_vector(rsrc_t r, u32 off, u32 rem) {
    Words<4> v = buf_load<4, kStream>(r, off);
    if (sizeof(T) == 2 && rem < 16u && (rem & 2u)) {
        const u32 bits = load_b16<kStream>(r, off + (rem & ~3u));
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if ((u32)j == rem / 4u) v.v[j] = bits;
    }
    return v;
}

template <typename T>
__global__ void __launch_bounds__(256)
swiglu_fwd_ragged(T* __restrict__ h, const T* __restrict__ gu, uint32_t rows, uint32_t total, uint32_t half_bytes,
                  FastDiv nvr, int xcd_group) {
    constexpr int EPV = 16 / (int)sizeof(T);
    const uint32_t v = (uint32_t)xcd_remap(blockIdx.x, gridDim.x, xcd_group) * 256u + threadIdx.x;
    if (v >= total) return;
    const rsrc_t rin = make_rsrc(gu, rows * 2u * half_bytes);
    const rsrc_t rout = make_rsrc(h, rows * half_bytes);
    const uint32_t row = fastdiv(v, nvr);
    const uint32_t pos = (v - row * nvr.d) * 16u;
    const uint32_t rem = half_bytes - pos;
    const uint32_t gi = row * 2u * half_bytes + pos;
    const Words<4> g = load_half_row_vector<T>(rin, gi, rem);
    const Words<4> u = load_half_row_vector<T>(rin, gi + half_bytes, rem);
    float gf[EPV], uf[EPV], o[EPV];
    unpack_vec<T, 4>(g, gf);
    unpack_vec<T, 4>(u, uf);
#pragma unroll
    for (int e = 0; e < EPV; ++e) o[e] = (gf[e] * fast_sigmoid(gf[e])) * uf[e];
    store_row_vector<kKeep>(rout, row * half_bytes + pos, rem, pack_vec<T, 4>(o));
}

template <typename T>
__global__ void __launch_bounds__(256)
swiglu_bwd_ragged(T* __restrict__ dgu, const T* __restrict__ dh, const T* __restrict__ gu, uint32_t rows,
                  uint32_t total, uint32_t half_bytes, FastDiv nvr, int xcd_group) {
    constexpr int EPV = 16 / (int)sizeof(T);
    const uint32_t v = (uint32_t)xcd_remap(blockIdx.x, gridDim.x, xcd_group) * 256u + threadIdx.x;
    if (v >= total) return;
    const rsrc_t rin = make_rsrc(gu, rows * 2u * half_bytes);
    const rsrc_t rdh = make_rsrc(dh, rows * half_bytes);
    const rsrc_t rout = make_rsrc(dgu, rows * 2u * half_bytes);
    const uint32_t row = fastdiv(v, nvr);
    const uint32_t pos = (v - row * nvr.d) * 16u;
    const uint32_t rem = half_bytes - pos;
    const uint32_t gi = row * 2u * half_bytes + pos;
    const Words<4> g = load_half_row_vector<T>(rin, gi, rem);
    const Words<4> u = load_half_row_vector<T>(rin, gi + half_bytes, rem);
    const Words<4> d = load_half_row_vector<T>(rdh, row * half_bytes + pos, rem);
    float gf[EPV], uf[EPV], df[EPV], og[EPV], ou[EPV];
    unpack_vec<T, 4>(g, gf);
    unpack_vec<T, 4>(u, uf);
    unpack_vec<T, 4>(d, df);
#pragma unroll
    for (int e = 0; e < EPV; ++e) {
        const float sg = fast_sigmoid(gf[e]);
        ou[e] = df[e] * (gf[e] * sg);
        og[e] = (df[e] * uf[e]) * (sg * __builtin_fmaf(gf[e], 1.0f - sg, 1.0f));
    }
    store_row_vector<kKeep>(rout, gi, rem, pack_vec<T, 4>(og));
    store_row_vector<kKeep>(rout, gi + half_bytes, rem, pack_vec<T, 4>(ou));
}

// Element-wise variants, kept for comparison (the "force_generic" option).
// total = M * H elements (< 2^32 per launch), hdiv divides by H.
template <typename T>
__global__ void __launch_bounds__(256)
swiglu_fwd_generic(T* __restrict__ h, const T* __restrict__ gu, uint32_t total, FastDiv hdiv) {
    const uint32_t v = blockIdx.x * 256u + threadIdx.x;
    if (v >= total) return;
    const uint32_t row = fastdiv(v, hdiv);
    const uint32_t col = v - row * hdiv.d;
    const uint64_t gi = (uint64_t)row * (2ull * hdiv.d) + col;
    const float g = Elem<T>::load1(gu + gi);
    const float u = Elem<T>::load1(gu + gi + hdiv.d);
    Elem<T>::store1(h + v, (g * fast_sigmoid(g)) * u);
}

template <typename T>
__global__ void __launch_bounds__(256)
swiglu_bwd_generic(T* __restrict__ dgu, const T* __restrict__ dh, const T* __restrict__ gu, uint32_t total,
                   FastDiv hdiv) {
    const uint32_t v = blockIdx.x * 256u + threadIdx.x;
    if (v >= total) return;
    const uint32_t row = fastdiv(v, hdiv);
    const uint32_t col = v - row * hdiv.d;
    const uint64_t gi = (uint64_t)row * (2ull * hdiv.d) + col;
    const float g = Elem<T>::load1(gu + gi);
    const float u = Elem<T>::load1(gu + gi + hdiv.d);
    const float d = Elem<T>::load1(dh + v);
    const float sg = fast_sigmoid(g);
    Elem<T>::store1(dgu + gi + hdiv.d, d * (g * sg));
    Elem<T>::store1(dgu + gi, (d * u) * (sg * __builtin_fmaf(g, 1.0f - sg, 1.0f)));
}

}  // namespace mg
