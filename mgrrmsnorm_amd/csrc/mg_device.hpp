// Device-side building blocks shared by the gfx950 kernels: 128/64-bit raw buffer
// loads and stores, element packing for fp32/fp16/bf16, wave64 DPP reduction.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mg {

typedef unsigned int u32;
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

typedef _Float16 half_t;
typedef __bf16 bf16_t;

constexpr int kWave = 64;

// ---------------------------------------------------------------------------------
// Raw buffer resources.  A resource describes [base, base + bytes): loads whose byte
// offset falls outside return 0 and stores outside are dropped, which gives branch-free
// row tails and lets a wave that has no row left run with bytes == 0.
// Word 3 = 0x00020000 selects the untyped 32-bit data format on gfx9-family parts.
// ---------------------------------------------------------------------------------
typedef __amdgpu_buffer_rsrc_t rsrc_t;

__device__ __forceinline__ rsrc_t make_rsrc(const void* base, u32 bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

// NW 32-bit words per vector (4 -> dwordx4, 2 -> dwordx2).
template <int NW> struct Words { u32 v[NW]; };

// Cache policy of a buffer access (the instruction's nt bit).  kStream marks data that is
// touched once (activations and their gradients): measured on MI355X, non-temporal loads
// stream about 8 % faster than default ones at sizes beyond the caches and non-temporal
// stores about 20 % faster at tens of MiB.  kKeep is for what every row re-reads (weights).
constexpr int kKeep = 0;
constexpr int kStream = 2;

template <int NW, int POLICY = kKeep>
__device__ __forceinline__ Words<NW> buf_load(rsrc_t r, u32 byte_off) {
    static_assert(NW == 4 || NW == 2, "vector loads are 16 or 8 bytes");
    Words<NW> o;
    if constexpr (NW == 4) {
        u32x4 t = __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_off, 0, POLICY);
        o.v[0] = t.x; o.v[1] = t.y; o.v[2] = t.z; o.v[3] = t.w;
    } else {
        u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(r, (int)byte_off, 0, POLICY);
        o.v[0] = t.x; o.v[1] = t.y;
    }
    return o;
}

template <int NW, int POLICY = kKeep>
__device__ __forceinline__ void buf_store(rsrc_t r, u32 byte_off, const Words<NW>& w) {
    static_assert(NW == 4 || NW == 2, "vector stores are 16 or 8 bytes");
    if constexpr (NW == 4) {
        u32x4 t = {w.v[0], w.v[1], w.v[2], w.v[3]};
        __builtin_amdgcn_raw_buffer_store_b128(t, r, (int)byte_off, 0, POLICY);
    } else {
        u32x2 t = {w.v[0], w.v[1]};
        __builtin_amdgcn_raw_buffer_store_b64(t, r, (int)byte_off, 0, POLICY);
    }
}

// ---------------------------------------------------------------------------------
// Rows of an odd number of 2-byte elements end in half a dword.  The per-dword range check
// drops that last dword (it loads as 0 and its store is discarded), so the one lane whose
// vector holds the last element fetches and stores it with 2-byte accesses and patches it
// into the low half of the right word; the high half stays 0, i.e. an element of value 0
// beyond the end of the row, which adds nothing to any sum.
// ---------------------------------------------------------------------------------
struct RowTail {
    bool any;    // the row has such a half dword (uniform over the launch)
    int lane;    // lane (within the row's TPR threads) that owns it
    int item;    // which of that lane's vectors
    int word;    // which 32-bit word of the vector
    u32 off;     // byte offset of the element in the row
};

template <typename T, int TPR>
__device__ __forceinline__ RowTail row_tail(int cols, u32 row_bytes) {
    RowTail t = {false, 0, 0, 0, 0};
    if constexpr (sizeof(T) == 2) {
        t.any = (row_bytes & 3u) != 0;
        const u32 vec = (u32)(cols - 1) / 8u;   // 8 two-byte elements per 16-byte vector
        t.lane = (int)(vec % TPR);
        t.item = (int)(vec / TPR);
        t.word = (int)(((u32)(cols - 1) % 8u) / 2u);
        t.off = row_bytes - 2u;
    }
    return t;
}

// All ITEMS vectors of one row for this lane (vector i of lane l is vector l + i*TPR of the
// row), plus the half-dword tail if this lane owns it.
template <int NW, int ITEMS, int TPR, int POLICY>
__device__ __forceinline__ void load_row(Words<NW> (&v)[ITEMS], rsrc_t r, int lir, const RowTail& t) {
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) v[i] = buf_load<NW, POLICY>(r, (u32)(lir + i * TPR) * (NW * 4));
    if (t.any && lir == t.lane) {
        const u32 bits = __builtin_amdgcn_raw_buffer_load_b16(r, (int)t.off, 0, POLICY);
#pragma unroll
        for (int i = 0; i < ITEMS; ++i)
#pragma unroll
            for (int j = 0; j < NW; ++j)
                if (i == t.item && j == t.word) v[i].v[j] = bits;
    }
}

// The same in two steps, for rows that are requested long before they are used (the next
// row of a persistent kernel): request_row() issues the loads and leaves the tail element in
// `tail_bits` untouched; patch_row_tail() puts it into its word when the row is used, so that
// no wait for the loads sits between the request and the work it is meant to overlap.
template <int NW, int ITEMS, int TPR, int POLICY>
__device__ __forceinline__ void request_row(Words<NW> (&v)[ITEMS], u32& tail_bits, rsrc_t r, int lir, const RowTail& t) {
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) v[i] = buf_load<NW, POLICY>(r, (u32)(lir + i * TPR) * (NW * 4));
    tail_bits = 0;
    if (t.any)   // uniform over the launch; lanes that do not own the tail ask for nothing
        tail_bits = __builtin_amdgcn_raw_buffer_load_b16(r, (int)(lir == t.lane ? t.off : 0xFFFFFFF0u), 0, POLICY);
}

template <int NW, int ITEMS>
__device__ __forceinline__ void patch_row_tail(Words<NW> (&v)[ITEMS], u32 tail_bits, int lir, const RowTail& t) {
    if (t.any) {
#pragma unroll
        for (int i = 0; i < ITEMS; ++i)
#pragma unroll
            for (int j = 0; j < NW; ++j)
                v[i].v[j] = (lir == t.lane && i == t.item && j == t.word) ? tail_bits : v[i].v[j];
    }
}

// Store vector `i` of this lane; the owner of the half-dword tail also stores that element.
template <int NW, int TPR, int POLICY>
__device__ __forceinline__ void store_item(rsrc_t r, int lir, int i, const Words<NW>& w, const RowTail& t) {
    buf_store<NW, POLICY>(r, (u32)(lir + i * TPR) * (NW * 4), w);
    if (t.any && lir == t.lane && i == t.item) {
        u32 bits = 0;
#pragma unroll
        for (int j = 0; j < NW; ++j)
            if (j == t.word) bits = w.v[j];
        __builtin_amdgcn_raw_buffer_store_b16((unsigned short)(bits & 0xffffu), r, (int)t.off, 0, POLICY);
    }
}

// ---------------------------------------------------------------------------------
// Rows packed back to back under one buffer resource (several rows per wave): a 16-byte
// vector that starts `pos` bytes into a row of `row_bytes` may run past the end of its row
// into the next one.  `rem` = row_bytes - pos is what the row still holds from there (as an
// unsigned difference it wraps to a huge value for a lane that has no vector in the row,
// which reads as "nothing to trim": such a lane's offset is out of range anyway).
// trim_row_vector() zeroes the words beyond the row after a plain 16-byte load -- it only
// touches registers, so it can run long after the load was issued -- and puts in `tail_bits`
// where a row of an odd number of 2-byte elements ends in half a dword (the lane holding that
// word fetches the element with a 2-byte load of its own).  store_row_vector() stores only
// what belongs to the row.
// ---------------------------------------------------------------------------------
__device__ __forceinline__ void trim_row_vector(Words<4>& v, u32 rem, u32 tail_bits) {
    const int r = rem < 16u ? (int)rem : 16;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int left = r - 4 * j;
        v.v[j] = left >= 4 ? v.v[j] : (left == 2 ? tail_bits : 0u);
    }
}

template <int POLICY>
__device__ __forceinline__ void store_row_vector(rsrc_t r, u32 off, u32 rem, const Words<4>& w) {
    if (rem >= 16u) {
        buf_store<4, POLICY>(r, off, w);
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int left = (int)rem - 4 * j;
            if (left >= 4) __builtin_amdgcn_raw_buffer_store_b32(w.v[j], r, (int)(off + 4u * j), 0, POLICY);
            else if (left == 2)
                __builtin_amdgcn_raw_buffer_store_b16((unsigned short)(w.v[j] & 0xffffu), r, (int)(off + 4u * j), 0, POLICY);
        }
    }
}

template <int POLICY>
__device__ __forceinline__ u32 load_b16(rsrc_t r, u32 off) {
    return (u32)__builtin_amdgcn_raw_buffer_load_b16(r, (int)off, 0, POLICY);
}

// ---------------------------------------------------------------------------------
// Element traits: PER_WORD elements per 32-bit word, conversion to/from fp32.
// fp32 -> fp16/bf16 uses the hardware round-to-nearest-even converts
// (v_cvt_pk_f16_f32 / v_cvt_pk_bf16_f32); never the round-toward-zero pack.
// ---------------------------------------------------------------------------------
template <typename T> struct Elem;

template <> struct Elem<float> {
    static constexpr int PER_WORD = 1;
    static __device__ __forceinline__ void unpack(u32 w, float* f) { f[0] = __builtin_bit_cast(float, w); }
    static __device__ __forceinline__ u32 pack(const float* f) { return __builtin_bit_cast(u32, f[0]); }
    static __device__ __forceinline__ float load1(const float* p) { return *p; }
    static __device__ __forceinline__ void store1(float* p, float f) { *p = f; }
};

template <> struct Elem<half_t> {
    static constexpr int PER_WORD = 2;
    static __device__ __forceinline__ void unpack(u32 w, float* f) {
        f16x2 h = __builtin_bit_cast(f16x2, w);
        f[0] = (float)h.x; f[1] = (float)h.y;
    }
    static __device__ __forceinline__ u32 pack(const float* f) {
        f32x2 p = {f[0], f[1]};
        return __builtin_bit_cast(u32, __builtin_convertvector(p, f16x2));
    }
    static __device__ __forceinline__ float load1(const half_t* p) { return (float)*p; }
    static __device__ __forceinline__ void store1(half_t* p, float f) { *p = (half_t)f; }
};

template <> struct Elem<bf16_t> {
    static constexpr int PER_WORD = 2;
    static __device__ __forceinline__ void unpack(u32 w, float* f) {
        f[0] = __builtin_bit_cast(float, w << 16);
        f[1] = __builtin_bit_cast(float, w & 0xffff0000u);
    }
    static __device__ __forceinline__ u32 pack(const float* f) {
        f32x2 p = {f[0], f[1]};
        return __builtin_bit_cast(u32, __builtin_convertvector(p, bf16x2));
    }
    static __device__ __forceinline__ float load1(const bf16_t* p) {
        unsigned short b = *reinterpret_cast<const unsigned short*>(p);
        return __builtin_bit_cast(float, (u32)b << 16);
    }
    static __device__ __forceinline__ void store1(bf16_t* p, float f) { *p = (bf16_t)f; }
};

// Unpack / pack a whole vector of NW words = NW * PER_WORD elements.
template <typename T, int NW>
__device__ __forceinline__ void unpack_vec(const Words<NW>& w, float* f) {
#pragma unroll
    for (int i = 0; i < NW; ++i) Elem<T>::unpack(w.v[i], f + i * Elem<T>::PER_WORD);
}
template <typename T, int NW>
__device__ __forceinline__ Words<NW> pack_vec(const float* f) {
    Words<NW> w;
#pragma unroll
    for (int i = 0; i < NW; ++i) w.v[i] = Elem<T>::pack(f + i * Elem<T>::PER_WORD);
    return w;
}

// ---------------------------------------------------------------------------------
// wave64 all-reduce (sum).  Four DPP steps make every lane of each 16-lane row hold that
// row's sum (xor-1, xor-2 inside quads, then rotate-by-4 and rotate-by-8 inside the row);
// the four row sums are then read with v_readlane and added in a fixed order, so the
// result is identical in all 64 lanes and from run to run.
// ---------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float read_lane(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_mov<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_mov<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_mov<0x124>(v);  // row_ror:4
    v += dpp_mov<0x128>(v);  // row_ror:8
    return (read_lane(v, 0) + read_lane(v, 16)) + (read_lane(v, 32) + read_lane(v, 48));
}

// Workgroups are handed to the 8 XCDs round-robin by workgroup id, so consecutive ids land
// on different dies.  This bijection makes each die work on `group` consecutive logical
// ids at a time (workgroups id, id+8, id+16, ... of a block of 8*group ids become
// consecutive), which keeps a die's address translations and open DRAM pages local:
// measured +6 % on plain streaming reads, +2.6 % on copies, +11 % on the forward pass over
// 2 GiB tensors.  group == 0, or a ragged last block, leaves ids unchanged.
__device__ __forceinline__ long xcd_remap(long id, long count, int group) {
    if (group <= 0) return id;
    const long span = 8L * group;
    const long base = id / span * span;
    if (base + span > count) return id;
    const long within = id - base;
    return base + (within & 7) * group + (within >> 3);
}

// Sum over groups of 1, 2, 4, 8, 16 or 32 adjacent lanes (rows narrower than a wave): every
// lane ends up with its group's total.  xor-1 and xor-2 inside quads, then mirror inside half
// rows (8) and inside 16-lane rows; for 32 the two row sums of each half wave are read with
// v_readlane and added.  A fixed order, no LDS.
template <int GROUP>
__device__ __forceinline__ float group_sum(float v) {
    static_assert(GROUP == 1 || GROUP == 2 || GROUP == 4 || GROUP == 8 || GROUP == 16 || GROUP == 32,
                  "sub-wave rows are 1 to 32 lanes wide");
    if constexpr (GROUP >= 2) v += dpp_mov<0xB1>(v);   // quad_perm [1,0,3,2]
    if constexpr (GROUP >= 4) v += dpp_mov<0x4E>(v);   // quad_perm [2,3,0,1]
    if constexpr (GROUP >= 8) v += dpp_mov<0x141>(v);  // row_half_mirror: lane i <-> 7 - i of each 8
    if constexpr (GROUP >= 16) v += dpp_mov<0x140>(v);  // row_mirror: lane i <-> 15 - i of each 16
    if constexpr (GROUP == 32) {
        const float lo = read_lane(v, 0) + read_lane(v, 16);
        const float hi = read_lane(v, 32) + read_lane(v, 48);
        v = (__lane_id() & 32) ? hi : lo;
    }
    return v;
}

// 1/sqrt(v): the hardware estimate (about 1 ulp) refined by one Newton step, so that the
// per-row scale, which the backward pass uses cubed, is good to about half an ulp.
// v = +inf (a row holding an infinity, or squares that overflow fp32) gives 0 like rsqrtf:
// the refinement would form inf * 0 there, so it is skipped.
__device__ __forceinline__ float fast_rsqrt(float v) {
    const float y = __builtin_amdgcn_rsqf(v);
    const float e = __builtin_fmaf(-(v * y), y, 1.0f);  // 1 - v*y^2
    const float r = __builtin_fmaf(0.5f * y, e, y);
    return v < __builtin_inff() ? r : y;
}

// sigmoid(g) = 1 / (1 + 2^(-g*log2(e))).  For g << 0 the power overflows to +inf and the
// reciprocal gives +0, the correct limit.
__device__ __forceinline__ float fast_sigmoid(float g) {
    float e = __builtin_amdgcn_exp2f(g * -1.4426950408889634f);
    return __builtin_amdgcn_rcpf(1.0f + e);
}

}  // namespace mg
