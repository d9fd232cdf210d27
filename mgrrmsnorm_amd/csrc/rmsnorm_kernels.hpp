// RMSNorm forward / backward kernels for gfx950.
//
// Register-resident family ("rows" kernels): a row of `cols` elements is split into
// vectors of VEC = 16 bytes; TPR threads (a multiple of the 64-lane wave) share one row
// and each holds ITEMS vectors of it in VGPRs, vector i of thread t being vector t + i*TPR
// of the row.  All of a row's loads are issued before the first use.  Row sums are reduced
// with DPP inside a wave and through a few floats of LDS across the waves of a row.
// Rows need no alignment beyond that of an element: buffer_load/store_dwordx4 work at any
// byte offset, and the range check against the row's byte length is made per dword, so a
// row whose length is not a multiple of 16 simply ends inside its last vector (the lanes
// and dwords beyond it load 0 and store nothing).  A row of an odd number of 2-byte
// elements ends in half a dword, which one lane moves with 2-byte accesses (RowTail).
//
// Narrow family: rows of at most 128 vectors put 8, 16 or 32 lanes on a row, so that one
// wave carries 8, 4 or 2 consecutive rows, with up to 4 vectors per lane (see below).
//
// Row-group family: rows of at most 64 vectors put 1 ... 64 lanes on a row with one vector
// per lane, and a wave keeps several groups of 64/lanes consecutive rows in flight; every
// load or store instruction then covers one contiguous piece of memory (see below).
//
// Streaming family: rows that do not fit registers are read twice by one 1024-thread
// workgroup per row, with the same 16-byte accesses.
//
// Generic family: one 256-thread workgroup per row, element-wise loads, two passes over
// the row; nothing selects it by itself, it runs on request only (the force_generic option).
#pragma once
#include "mg_device.hpp"

namespace mg {

// A byte offset no buffer resource holds (rows stay below 2^31 bytes): a load there returns 0,
// a store there is dropped.
constexpr u32 kOutOfRange = 0xFFFFFFF0u;

// =================================================================================
// Forward, register-resident.
//   grid  = ceil(rows / RPB) workgroups, RPB = BLOCK / TPR rows per workgroup
//   block = BLOCK = max(TPR, 256) threads
// =================================================================================
template <typename T, int VEC, int TPR, int ITEMS>
__global__ void __launch_bounds__((TPR > 256 ? TPR : 256))
rmsnorm_fwd_rows(T* __restrict__ y, float* __restrict__ inv_rms, const T* __restrict__ x,
                 const T* __restrict__ w, long rows, int cols, float eps, float inv_cols, int xcd_group) {
    constexpr int BLOCK = TPR > 256 ? TPR : 256;
    constexpr int RPB = BLOCK / TPR;
    constexpr int WPR = TPR / kWave;
    constexpr int NW = VEC / 4;
    constexpr int EPV = VEC / (int)sizeof(T);

    const int tid = threadIdx.x;
    const int rg = __builtin_amdgcn_readfirstlane(tid / TPR);  // row slot inside the workgroup
    const int lir = tid - rg * TPR;                            // lane inside the row
    const long row = xcd_remap(blockIdx.x, gridDim.x, xcd_group) * RPB + rg;
    const bool live = row < rows;
    const u32 row_bytes = (u32)cols * (u32)sizeof(T);
    const long base = live ? row * (long)cols : 0;

    const rsrc_t rx = make_rsrc(x + base, live ? row_bytes : 0u);
    const rsrc_t ry = make_rsrc(y + base, live ? row_bytes : 0u);
    const rsrc_t rw = make_rsrc(w, row_bytes);

    const RowTail tail = row_tail<T, TPR>(cols, row_bytes);
    Words<NW> xv[ITEMS];
    Words<NW> wv[ITEMS];
    u32 x_tail, w_tail;
    request_row<NW, ITEMS, TPR, kStream>(xv, x_tail, rx, lir, tail);
    request_row<NW, ITEMS, TPR, kKeep>(wv, w_tail, rw, lir, tail);
    patch_row_tail<NW, ITEMS>(xv, x_tail, lir, tail);
    patch_row_tail<NW, ITEMS>(wv, w_tail, lir, tail);

    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        float f[EPV];
        unpack_vec<T, NW>(xv[i], f);
#pragma unroll
        for (int k = 0; k < EPV; ++k) ss = __builtin_fmaf(f[k], f[k], ss);
    }
    ss = wave_sum(ss);
    if constexpr (WPR > 1) {
        __shared__ float part[RPB][WPR];
        const int wir = __builtin_amdgcn_readfirstlane(lir / kWave);  // wave inside the row
        if ((tid & (kWave - 1)) == 0) part[rg][wir] = ss;
        __syncthreads();
        float t = 0.0f;
#pragma unroll
        for (int k = 0; k < WPR; ++k) t += part[rg][k];
        ss = t;
    }
    const float s = fast_rsqrt(ss * inv_cols + eps);
    if (live && lir == 0 && inv_rms != nullptr) inv_rms[row] = s;

#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        float xf[EPV], wf[EPV], o[EPV];
        unpack_vec<T, NW>(xv[i], xf);
        unpack_vec<T, NW>(wv[i], wf);
#pragma unroll
        for (int k = 0; k < EPV; ++k) o[k] = (xf[k] * s) * wf[k];
        store_item<NW, TPR, kStream>(ry, lir, i, pack_vec<T, NW>(o), tail);
    }
}

// =================================================================================
// Forward, register-resident, vectors on the 128-byte lines of y ("lines" layout): for row
// pitches that are multiples of 8 but not of 128 bytes.  With vector j of a row at the row's
// first byte + 16 j (the layout above) every store instruction of a wave begins and ends
// inside a 128-byte line, so every line of y is written in two pieces by two instructions;
// here slot k of a row covers bytes [16 k, 16 k + 16) counted from the start of the line that
// holds the row's first byte, i.e. row bytes [16 k - a, 16 k - a + 16) with a = (address of the
// row in y) mod 128, so a wave's instruction covers whole lines and only the first and last
// line of a row are shared with its neighbours.  Slots in front of the row get an
// out-of-range offset (they load 0 and store nothing), the row's end is clipped by the
// buffer's range check as everywhere.  When a is 8 mod 16 -- every other row of a pitch that
// is 8 mod 16 -- the row's first 8 bytes are the upper half of slot (a - 8) / 16, which is
// always a slot of a thread's first vector: that lane moves them with an 8-byte access of
// its own into and out of the upper two words (the lower two stay 0 and are not stored).
// x and w are read at the same offsets as y is written, so a thread holds x, w and y of the
// same columns whatever a is.  Runs on request only: measured on MI355X (bf16, against the
// layout above) it gains 2-7 % at 2052, 2056, 5000 and 8200 columns and loses 1-10 % at 4100,
// 12292 and 16380 columns and at 4096 rows (the figures are where the host chooses).
//   needs: row pitch and the address of y multiples of 8 bytes (a is then a multiple of 8);
//          TPR * ITEMS >= ceil((120 + row bytes) / 16) slots
//   grid / block as rmsnorm_fwd_rows
// =================================================================================
template <typename T, int VEC, int TPR, int ITEMS>
__global__ void __launch_bounds__((TPR > 256 ? TPR : 256))
rmsnorm_fwd_rows_lines(T* __restrict__ y, float* __restrict__ inv_rms, const T* __restrict__ x,
                       const T* __restrict__ w, long rows, int cols, float eps, float inv_cols, int xcd_group) {
    static_assert(VEC == 16, "slots are 16 bytes");
    constexpr int BLOCK = TPR > 256 ? TPR : 256;
    constexpr int RPB = BLOCK / TPR;
    constexpr int WPR = TPR / kWave;
    constexpr int NW = VEC / 4;
    constexpr int EPV = VEC / (int)sizeof(T);

    const int tid = threadIdx.x;
    const int rg = __builtin_amdgcn_readfirstlane(tid / TPR);
    const int lir = tid - rg * TPR;
    const long row = xcd_remap(blockIdx.x, gridDim.x, xcd_group) * RPB + rg;
    const bool live = row < rows;
    const u32 row_bytes = (u32)cols * (u32)sizeof(T);
    const long base = live ? row * (long)cols : 0;

    const rsrc_t rx = make_rsrc(x + base, live ? row_bytes : 0u);
    const rsrc_t ry = make_rsrc(y + base, live ? row_bytes : 0u);
    const rsrc_t rw = make_rsrc(w, row_bytes);

    // a row belongs to whole waves, so its skew is uniform over a wave
    const u32 a = (u32)__builtin_amdgcn_readfirstlane((int)(reinterpret_cast<unsigned long long>(y + base) & 127ull));
    const bool half = (a & 8u) != 0;
    const u32 head_off = (half && (u32)lir * (u32)VEC + 8u == a) ? 0u : kOutOfRange;
    u32 off[ITEMS];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        const u32 slot_byte = (u32)(lir + i * TPR) * (u32)VEC;
        off[i] = slot_byte >= a ? slot_byte - a : kOutOfRange;
    }

    Words<NW> xv[ITEMS];
    Words<NW> wv[ITEMS];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) xv[i] = buf_load<NW, kStream>(rx, off[i]);
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) wv[i] = buf_load<NW, kKeep>(rw, off[i]);
    if (half) {   // the lane whose first slot straddles the row's first byte: that slot's own load was out of range
        const Words<2> hx = buf_load<2, kStream>(rx, head_off);
        const Words<2> hw = buf_load<2, kKeep>(rw, head_off);
        xv[0].v[2] |= hx.v[0];
        xv[0].v[3] |= hx.v[1];
        wv[0].v[2] |= hw.v[0];
        wv[0].v[3] |= hw.v[1];
    }

    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        float f[EPV];
        unpack_vec<T, NW>(xv[i], f);
#pragma unroll
        for (int k = 0; k < EPV; ++k) ss = __builtin_fmaf(f[k], f[k], ss);
    }
    ss = wave_sum(ss);
    if constexpr (WPR > 1) {
        __shared__ float part[RPB][WPR];
        const int wir = __builtin_amdgcn_readfirstlane(lir / kWave);
        if ((tid & (kWave - 1)) == 0) part[rg][wir] = ss;
        __syncthreads();
        float t = 0.0f;
#pragma unroll
        for (int k = 0; k < WPR; ++k) t += part[rg][k];
        ss = t;
    }
    const float s = fast_rsqrt(ss * inv_cols + eps);
    if (live && lir == 0 && inv_rms != nullptr) inv_rms[row] = s;

#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        float xf[EPV], wf[EPV], o[EPV];
        unpack_vec<T, NW>(xv[i], xf);
        unpack_vec<T, NW>(wv[i], wf);
#pragma unroll
        for (int k = 0; k < EPV; ++k) o[k] = (xf[k] * s) * wf[k];
        const Words<NW> ov = pack_vec<T, NW>(o);
        buf_store<NW, kStream>(ry, off[i], ov);
        if (i == 0 && half) {
            const Words<2> h = {{ov.v[2], ov.v[3]}};
            buf_store<2, kStream>(ry, head_off, h);
        }
    }
}

// =================================================================================
// Narrow rows (at most 4 vectors per lane): TPR = 8, 16 or 32 lanes per row, so a wave
// carries 64/TPR consecutive rows and a 256-thread workgroup 256/TPR.  One buffer resource
// spans the wave's rows; lanes past the end of a row, and rows past the end of the matrix,
// get an out-of-range offset (loads 0, stores nothing).  Row sums stay inside the wave (DPP,
// plus v_readlane for 32 lanes): no LDS, no barrier.  RAGGED = the row pitch is not a
// multiple of 16 bytes: the last vector of a row then reaches into the next row and is
// trimmed to its own row on load and on store (load_row_vector / store_row_vector).
// =================================================================================

// Activations of ragged rows take the default cache policy: a row's last vector is stored in
// pieces, and lines shared by two rows are written by two instructions; the L2 merges those
// writes, whereas non-temporal ones reach memory piecemeal (measured: 2.2 against 4.7 TB/s
// at 100 bf16 columns).
template <bool RAGGED> constexpr int kNarrowPolicy = RAGGED ? kKeep : kStream;

// Where this lane's vectors sit in a narrow row, fixed for the whole kernel.
template <int TPR, int ITEMS>
struct NarrowLane {
    u32 off[ITEMS];   // byte offset under the wave's buffer resource, or out of range
    u32 woff[ITEMS];  // byte offset in the weight row, or out of range
    u32 rem[ITEMS];   // bytes the row still holds from the vector's start (ragged rows)
    u32 tail_off;     // where the row's last 2-byte element is, for the lane that patches it in
    bool owns_tail;   // the row ends in half a dword and this lane holds that word
};

template <typename T, int TPR, int ITEMS, bool RAGGED>
__device__ __forceinline__ NarrowLane<TPR, ITEMS> narrow_lane(int sub, int lir, u32 row_bytes) {
    NarrowLane<TPR, ITEMS> p;
    const u32 nvec = (row_bytes + 15u) / 16u;
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        const u32 vec = (u32)(lir + i * TPR);
        p.off[i] = vec < nvec ? (u32)sub * row_bytes + vec * 16u : kOutOfRange;
        p.woff[i] = vec < nvec ? vec * 16u : kOutOfRange;
        p.rem[i] = row_bytes - vec * 16u;
    }
    p.owns_tail = false;
    p.tail_off = row_bytes - 2u;
    if constexpr (RAGGED && sizeof(T) == 2)
        p.owns_tail = (row_bytes & 2u) != 0 && (u32)lir == ((row_bytes - 1u) / 16u) % TPR;
    return p;
}

template <typename T, int TPR, int ITEMS, bool RAGGED>
__global__ void __launch_bounds__(256)
rmsnorm_fwd_narrow(T* __restrict__ y, float* __restrict__ inv_rms, const T* __restrict__ x,
                   const T* __restrict__ w, long rows, int cols, float eps, float inv_cols, int xcd_group) {
    constexpr int RPW = kWave / TPR;   // rows per wave
    constexpr int RPB = 256 / TPR;     // rows per workgroup
    constexpr int EPV = 16 / (int)sizeof(T);
    constexpr int POL = kNarrowPolicy<RAGGED>;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int lane = tid & (kWave - 1);
    const int sub = lane / TPR;        // row inside the wave
    const int lir = lane % TPR;        // lane inside the row
    const long row0 = xcd_remap(blockIdx.x, gridDim.x, xcd_group) * RPB + (long)wave * RPW;
    const long left = rows - row0;
    const u32 live_rows = left <= 0 ? 0u : (left < RPW ? (u32)left : (u32)RPW);
    const u32 row_bytes = (u32)cols * (u32)sizeof(T);
    const long base = live_rows ? row0 * (long)cols : 0;
    const rsrc_t rx = make_rsrc(x + base, live_rows * row_bytes);
    const rsrc_t ry = make_rsrc(y + base, live_rows * row_bytes);
    const rsrc_t rw = make_rsrc(w, row_bytes);
    const NarrowLane<TPR, ITEMS> p = narrow_lane<T, TPR, ITEMS, RAGGED>(sub, lir, row_bytes);

    Words<4> xv[ITEMS], wv[ITEMS];
    u32 x_tail = 0, w_tail = 0;
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) xv[i] = buf_load<4, POL>(rx, p.off[i]);
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) wv[i] = buf_load<4, kKeep>(rw, p.woff[i]);
    if constexpr (RAGGED) {
        if (p.owns_tail) {
            x_tail = load_b16<POL>(rx, (u32)sub * row_bytes + p.tail_off);
            w_tail = load_b16<kKeep>(rw, p.tail_off);
        }
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            trim_row_vector(xv[i], p.rem[i], x_tail);
            trim_row_vector(wv[i], p.rem[i], w_tail);
        }
    }
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        float f[EPV];
        unpack_vec<T, 4>(xv[i], f);
#pragma unroll
        for (int k = 0; k < EPV; ++k) ss = __builtin_fmaf(f[k], f[k], ss);
    }
    ss = group_sum<TPR>(ss);
    const float s = fast_rsqrt(ss * inv_cols + eps);
    if (lir == 0 && (u32)sub < live_rows && inv_rms != nullptr) inv_rms[row0 + sub] = s;
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        float xf[EPV], wf[EPV], o[EPV];
        unpack_vec<T, 4>(xv[i], xf);
        unpack_vec<T, 4>(wv[i], wf);
#pragma unroll
        for (int k = 0; k < EPV; ++k) o[k] = (xf[k] * s) * wf[k];
        if constexpr (RAGGED) store_row_vector<POL>(ry, p.off[i], p.rem[i], pack_vec<T, 4>(o));
        else buf_store<4, POL>(ry, p.off[i], pack_vec<T, 4>(o));
    }
}

// Narrow rows, one vector per lane ("row groups"): TPR = 1, 2, 4 ... 64 lanes per row with
// TPR >= the row's vectors, and G groups of 64/TPR consecutive rows per wave in flight.
// Every load or store instruction of a wave then covers one contiguous piece of memory (the
// idle lanes of a row map to nothing), whatever the row pitch -- the layout for pitches that
// are not multiples of 128 bytes, where the several-vectors-per-lane layout above writes
// cache lines in pieces.  Ragged rows as above; POL = cache policy of the activations.
template <int TPR>
__device__ __forceinline__ float lanes_sum(float v) {
    if constexpr (TPR == kWave) return wave_sum(v);
    else return group_sum<TPR>(v);
}

template <typename T, int TPR, int G, bool RAGGED, int POL>
__global__ void __launch_bounds__(256)
rmsnorm_fwd_groups(T* __restrict__ y, float* __restrict__ inv_rms, const T* __restrict__ x,
                   const T* __restrict__ w, long rows, int cols, float eps, float inv_cols, int xcd_group) {
    constexpr int RPG = kWave / TPR;   // rows per group
    constexpr int RPW = G * RPG;       // rows per wave
    constexpr int RPB = 4 * RPW;       // rows per workgroup
    constexpr int EPV = 16 / (int)sizeof(T);
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int lane = tid & (kWave - 1);
    const int sub = lane / TPR;
    const int lir = lane % TPR;
    const long row0 = xcd_remap(blockIdx.x, gridDim.x, xcd_group) * RPB + (long)wave * RPW;
    const long left = rows - row0;
    const u32 live_rows = left <= 0 ? 0u : (left < RPW ? (u32)left : (u32)RPW);
    const u32 row_bytes = (u32)cols * (u32)sizeof(T);
    const u32 nvec = (row_bytes + 15u) / 16u;
    const long base = live_rows ? row0 * (long)cols : 0;
    const rsrc_t rx = make_rsrc(x + base, live_rows * row_bytes);
    const rsrc_t ry = make_rsrc(y + base, live_rows * row_bytes);
    const rsrc_t rw = make_rsrc(w, row_bytes);
    const bool mine = (u32)lir < nvec;
    const u32 pos = (u32)lir * 16u;             // where this lane's vector starts in its row
    const u32 rem = row_bytes - pos;            // what the row holds from there (wraps when !mine)
    const u32 tail_off = row_bytes - 2u;
    bool owns_tail = false;
    if constexpr (RAGGED && sizeof(T) == 2) owns_tail = (row_bytes & 2u) != 0 && (u32)lir == (row_bytes - 1u) / 16u;
    u32 off[G];
#pragma unroll
    for (int g = 0; g < G; ++g) off[g] = mine ? (u32)(g * RPG + sub) * row_bytes + pos : kOutOfRange;

    Words<4> xv[G];
    u32 x_tail[G];
#pragma unroll
    for (int g = 0; g < G; ++g) xv[g] = buf_load<4, POL>(rx, off[g]);
    Words<4> wv = buf_load<4, kKeep>(rw, mine ? pos : kOutOfRange);
    if constexpr (RAGGED) {
        u32 w_tail = 0;
#pragma unroll
        for (int g = 0; g < G; ++g) x_tail[g] = 0;
        if (owns_tail) {
#pragma unroll
            for (int g = 0; g < G; ++g) x_tail[g] = load_b16<POL>(rx, (u32)(g * RPG + sub) * row_bytes + tail_off);
            w_tail = load_b16<kKeep>(rw, tail_off);
        }
        trim_row_vector(wv, rem, w_tail);
    }
    float wf[EPV];
    unpack_vec<T, 4>(wv, wf);
#pragma unroll
    for (int g = 0; g < G; ++g) {
        if constexpr (RAGGED) trim_row_vector(xv[g], rem, x_tail[g]);
        float f[EPV], o[EPV];
        unpack_vec<T, 4>(xv[g], f);
        float ss = 0.0f;
#pragma unroll
        for (int k = 0; k < EPV; ++k) ss = __builtin_fmaf(f[k], f[k], ss);
        ss = lanes_sum<TPR>(ss);
        const float s = fast_rsqrt(ss * inv_cols + eps);
        const u32 r = (u32)(g * RPG + sub);
        if (lir == 0 && r < live_rows && inv_rms != nullptr) inv_rms[row0 + r] = s;
#pragma unroll
        for (int k = 0; k < EPV; ++k) o[k] = (f[k] * s) * wf[k];
        if constexpr (RAGGED) store_row_vector<POL>(ry, off[g], rem, pack_vec<T, 4>(o));
        else buf_store<4, POL>(ry, off[g], pack_vec<T, 4>(o));
    }
}

// Backward pass 1 in the same layout: persistent grid of 512-thread workgroups; wave q walks
// the blocks of G * 64/TPR consecutive rows q, q + Q, q + 2Q ... (Q = all waves), with the
// next block requested before the current one is reduced.  dW: 4 or 8 sums per lane (all row
// groups put the same columns on a lane), then across the rows of a wave by lane shuffles,
// then across the 8 waves in wave order through LDS; one partial row per workgroup.
template <typename T, int TPR, int G, bool RAGGED, int POL>
__global__ void __launch_bounds__(512)
rmsnorm_bwd_groups(T* __restrict__ dx, float* __restrict__ dw_part, int ld, const T* __restrict__ dy,
                   const T* __restrict__ x, const T* __restrict__ w, const float* __restrict__ inv_rms,
                   long rows, int cols, float inv_cols) {
    constexpr int BLOCK = 512;
    constexpr int WAVES = BLOCK / kWave;
    constexpr int RPG = kWave / TPR;
    constexpr int RPW = G * RPG;
    constexpr int EPV = 16 / (int)sizeof(T);
    constexpr int COVER = TPR * EPV;   // columns one row's lanes cover (>= cols)
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int lane = tid & (kWave - 1);
    const int sub = lane / TPR;
    const int lir = lane % TPR;
    const long nwaves = (long)gridDim.x * WAVES;
    const long q = (long)blockIdx.x * WAVES + wave;
    const long nblocks = (rows + RPW - 1) / RPW;
    const long n_it = (nblocks + nwaves - 1) / nwaves;
    const u32 row_bytes = (u32)cols * (u32)sizeof(T);
    const u32 nvec = (row_bytes + 15u) / 16u;
    const bool mine = (u32)lir < nvec;
    const u32 pos = (u32)lir * 16u;
    const u32 rem = row_bytes - pos;
    const u32 tail_off = row_bytes - 2u;
    bool owns_tail = false;
    if constexpr (RAGGED && sizeof(T) == 2) owns_tail = (row_bytes & 2u) != 0 && (u32)lir == (row_bytes - 1u) / 16u;
    u32 off[G];
#pragma unroll
    for (int g = 0; g < G; ++g) off[g] = mine ? (u32)(g * RPG + sub) * row_bytes + pos : kOutOfRange;

    float acc[EPV];
#pragma unroll
    for (int k = 0; k < EPV; ++k) acc[k] = 0.0f;

    float wf[EPV];
    {
        const rsrc_t rw = make_rsrc(w, row_bytes);
        Words<4> wv = buf_load<4, kKeep>(rw, mine ? pos : kOutOfRange);
        if constexpr (RAGGED) {
            u32 w_tail = 0;
            if (owns_tail) w_tail = load_b16<kKeep>(rw, tail_off);
            trim_row_vector(wv, rem, w_tail);
        }
        unpack_vec<T, 4>(wv, wf);
    }

    auto live_rows_of = [&](long row0) -> u32 {
        const long left = rows - row0;
        return left <= 0 ? 0u : (left < RPW ? (u32)left : (u32)RPW);
    };
    auto request = [&](long row0, u32 live, Words<4> (&xo)[G], Words<4> (&go)[G], u32 (&xt)[G], u32 (&gt)[G], float (&so)[G]) {
        const long base = live ? row0 * (long)cols : 0;
        const rsrc_t rx = make_rsrc(x + base, live * row_bytes);
        const rsrc_t rg = make_rsrc(dy + base, live * row_bytes);
#pragma unroll
        for (int g = 0; g < G; ++g) xo[g] = buf_load<4, POL>(rx, off[g]);
#pragma unroll
        for (int g = 0; g < G; ++g) go[g] = buf_load<4, POL>(rg, off[g]);
#pragma unroll
        for (int g = 0; g < G; ++g) {
            xt[g] = 0; gt[g] = 0; so[g] = 0.0f;
            if constexpr (RAGGED) {
                if (owns_tail) {
                    const u32 at = (u32)(g * RPG + sub) * row_bytes + tail_off;
                    xt[g] = load_b16<POL>(rx, at);
                    gt[g] = load_b16<POL>(rg, at);
                }
            }
            const u32 r = (u32)(g * RPG + sub);
            if (r < live) so[g] = inv_rms[row0 + r];
        }
    };

    Words<4> xv[G], gv[G];
    u32 x_tail[G], g_tail[G];
    float s[G];
    long row0 = q * RPW;
    u32 live = live_rows_of(row0);
    request(row0, live, xv, gv, x_tail, g_tail, s);

    for (long it = 0; it < n_it; ++it) {
        const long nrow0 = row0 + nwaves * RPW;
        const u32 nlive = live_rows_of(nrow0);
        Words<4> nxv[G], ngv[G];
        u32 nx_tail[G], ng_tail[G];
        float ns[G];
        request(nrow0, nlive, nxv, ngv, nx_tail, ng_tail, ns);

        const long base = live ? row0 * (long)cols : 0;
        const rsrc_t rd = make_rsrc(dx + base, live * row_bytes);
#pragma unroll
        for (int g = 0; g < G; ++g) {
            if constexpr (RAGGED) {
                trim_row_vector(xv[g], rem, x_tail[g]);
                trim_row_vector(gv[g], rem, g_tail[g]);
            }
            float xf[EPV], gf[EPV], o[EPV];
            unpack_vec<T, 4>(xv[g], xf);
            unpack_vec<T, 4>(gv[g], gf);
            float a = 0.0f;
#pragma unroll
            for (int k = 0; k < EPV; ++k) {
                const float t = gf[k] * xf[k];
                a = __builtin_fmaf(t, wf[k], a);
                acc[k] = __builtin_fmaf(t, s[g], acc[k]);
            }
            a = lanes_sum<TPR>(a);
            const float c2 = a * (s[g] * s[g]) * s[g] * inv_cols;
#pragma unroll
            for (int k = 0; k < EPV; ++k) o[k] = __builtin_fmaf(gf[k] * wf[k], s[g], -(xf[k] * c2));
            if constexpr (RAGGED) store_row_vector<POL>(rd, off[g], rem, pack_vec<T, 4>(o));
            else buf_store<4, POL>(rd, off[g], pack_vec<T, 4>(o));
        }
#pragma unroll
        for (int g = 0; g < G; ++g) {
            xv[g] = nxv[g]; gv[g] = ngv[g];
            x_tail[g] = nx_tail[g]; g_tail[g] = ng_tail[g];
            s[g] = ns[g];
        }
        row0 = nrow0; live = nlive;
    }

    // rows of one group: lanes lir, lir + TPR, lir + 2*TPR, ... hold the same columns
#pragma unroll
    for (int k = 0; k < EPV; ++k)
#pragma unroll
        for (int d = TPR; d < kWave; d *= 2) acc[k] += __shfl_xor(acc[k], d);

    // waves of the workgroup, in wave order
    __shared__ float dwbuf[COVER];
    for (int g = 0; g < WAVES; ++g) {
        if (wave == g && sub == 0) {
#pragma unroll
            for (int k = 0; k < EPV; ++k) {
                if (g == 0) dwbuf[lir * EPV + k] = acc[k];
                else dwbuf[lir * EPV + k] += acc[k];
            }
        }
        __syncthreads();
    }
    float* out = dw_part + (long)blockIdx.x * ld;
    const int lim = ld < COVER ? ld : COVER;
    for (int c = tid * 4; c < lim; c += BLOCK * 4) {
        f32x4 v = {dwbuf[c], dwbuf[c + 1], dwbuf[c + 2], dwbuf[c + 3]};
        *reinterpret_cast<f32x4*>(out + c) = v;
    }
    // columns between COVER and ld (COVER can be as small as 32) belong to no lane
    for (int c = COVER + tid; c < ld; c += BLOCK) out[c] = 0.0f;
}

// Backward pass 1 for narrow rows: persistent grid of 512-thread workgroups; each wave walks
// groups of 64/TPR consecutive rows (group g of wave q: rows (g*Q + q)*RPW ..., Q = all waves),
// prefetching the next group (ragged rows are trimmed when the data is used, not when it is
// requested, so the prefetch stays in flight).  dW: per lane in registers, then across the
// rows of a wave by lane shuffles, then across the 8 waves in wave order through LDS; one
// partial row per workgroup.
template <typename T, int TPR, int ITEMS, bool RAGGED>
__global__ void __launch_bounds__(512)
rmsnorm_bwd_narrow(T* __restrict__ dx, float* __restrict__ dw_part, int ld, const T* __restrict__ dy,
                   const T* __restrict__ x, const T* __restrict__ w, const float* __restrict__ inv_rms,
                   long rows, int cols, float inv_cols) {
    constexpr int BLOCK = 512;
    constexpr int WAVES = BLOCK / kWave;
    constexpr int RPW = kWave / TPR;
    constexpr int EPV = 16 / (int)sizeof(T);
    constexpr int COVER = TPR * ITEMS * EPV;   // columns one row's lanes cover (>= cols)
    constexpr int POL = kNarrowPolicy<RAGGED>;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int lane = tid & (kWave - 1);
    const int sub = lane / TPR;
    const int lir = lane % TPR;
    const long nwaves = (long)gridDim.x * WAVES;
    const long q = (long)blockIdx.x * WAVES + wave;
    const long ngroups = (rows + RPW - 1) / RPW;            // groups of RPW rows in the matrix
    const long n_it = (ngroups + nwaves - 1) / nwaves;
    const u32 row_bytes = (u32)cols * (u32)sizeof(T);
    const NarrowLane<TPR, ITEMS> p = narrow_lane<T, TPR, ITEMS, RAGGED>(sub, lir, row_bytes);
    const u32 tail_at = (u32)sub * row_bytes + p.tail_off;

    float acc[ITEMS][EPV];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i)
#pragma unroll
        for (int k = 0; k < EPV; ++k) acc[i][k] = 0.0f;

    Words<4> wv[ITEMS];
    {
        const rsrc_t rw = make_rsrc(w, row_bytes);
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) wv[i] = buf_load<4, kKeep>(rw, p.woff[i]);
        if constexpr (RAGGED) {
            u32 w_tail = 0;
            if (p.owns_tail) w_tail = load_b16<kKeep>(rw, p.tail_off);
#pragma unroll
            for (int i = 0; i < ITEMS; ++i) trim_row_vector(wv[i], p.rem[i], w_tail);
        }
    }

    auto live_rows_of = [&](long row0) -> u32 {
        const long left = rows - row0;
        return left <= 0 ? 0u : (left < RPW ? (u32)left : (u32)RPW);
    };
    // requests the x and dy vectors (and the odd last elements) of the rows from row0 on
    auto request = [&](long row0, u32 live, Words<4> (&xo)[ITEMS], Words<4> (&go)[ITEMS], u32& xt, u32& gt, float& so) {
        const long base = live ? row0 * (long)cols : 0;
        const rsrc_t rx = make_rsrc(x + base, live * row_bytes);
        const rsrc_t rg = make_rsrc(dy + base, live * row_bytes);
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) xo[i] = buf_load<4, POL>(rx, p.off[i]);
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) go[i] = buf_load<4, POL>(rg, p.off[i]);
        xt = 0; gt = 0;
        if constexpr (RAGGED) {
            if (p.owns_tail) { xt = load_b16<POL>(rx, tail_at); gt = load_b16<POL>(rg, tail_at); }
        }
        so = 0.0f;
        if ((u32)sub < live) so = inv_rms[row0 + sub];
    };

    Words<4> xv[ITEMS], gv[ITEMS];
    u32 x_tail, g_tail;
    long row0 = q * RPW;
    u32 live = live_rows_of(row0);
    float s;
    request(row0, live, xv, gv, x_tail, g_tail, s);

    for (long it = 0; it < n_it; ++it) {
        const long nrow0 = row0 + nwaves * RPW;
        const u32 nlive = live_rows_of(nrow0);
        Words<4> nxv[ITEMS], ngv[ITEMS];
        u32 nx_tail, ng_tail;
        float ns;
        request(nrow0, nlive, nxv, ngv, nx_tail, ng_tail, ns);

        if constexpr (RAGGED) {
#pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                trim_row_vector(xv[i], p.rem[i], x_tail);
                trim_row_vector(gv[i], p.rem[i], g_tail);
            }
        }
        float a = 0.0f;
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            float xf[EPV], gf[EPV], wf[EPV];
            unpack_vec<T, 4>(xv[i], xf);
            unpack_vec<T, 4>(gv[i], gf);
            unpack_vec<T, 4>(wv[i], wf);
#pragma unroll
            for (int k = 0; k < EPV; ++k) {
                const float t = gf[k] * xf[k];
                a = __builtin_fmaf(t, wf[k], a);
                acc[i][k] = __builtin_fmaf(t, s, acc[i][k]);
            }
        }
        a = group_sum<TPR>(a);
        const float c2 = a * (s * s) * s * inv_cols;
        {
            const long base = live ? row0 * (long)cols : 0;
            const rsrc_t rd = make_rsrc(dx + base, live * row_bytes);
#pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                float xf[EPV], gf[EPV], wf[EPV], o[EPV];
                unpack_vec<T, 4>(xv[i], xf);
                unpack_vec<T, 4>(gv[i], gf);
                unpack_vec<T, 4>(wv[i], wf);
#pragma unroll
                for (int k = 0; k < EPV; ++k) o[k] = __builtin_fmaf(gf[k] * wf[k], s, -(xf[k] * c2));
                if constexpr (RAGGED) store_row_vector<POL>(rd, p.off[i], p.rem[i], pack_vec<T, 4>(o));
                else buf_store<4, POL>(rd, p.off[i], pack_vec<T, 4>(o));
            }
        }
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) { xv[i] = nxv[i]; gv[i] = ngv[i]; }
        x_tail = nx_tail; g_tail = ng_tail;
        row0 = nrow0; live = nlive; s = ns;
    }

    // rows of one wave: lanes lir, lir + TPR, lir + 2*TPR, ... hold the same columns
#pragma unroll
    for (int i = 0; i < ITEMS; ++i)
#pragma unroll
        for (int k = 0; k < EPV; ++k)
#pragma unroll
            for (int d = TPR; d < kWave; d *= 2) acc[i][k] += __shfl_xor(acc[i][k], d);

    // waves of the workgroup, in wave order
    __shared__ float dwbuf[COVER];
    for (int g = 0; g < WAVES; ++g) {
        if (wave == g && sub == 0) {
#pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                const int c0 = (lir + i * TPR) * EPV;
#pragma unroll
                for (int k = 0; k < EPV; ++k) {
                    if (g == 0) dwbuf[c0 + k] = acc[i][k];
                    else dwbuf[c0 + k] += acc[i][k];
                }
            }
        }
        __syncthreads();
    }
    float* out = dw_part + (long)blockIdx.x * ld;
    const int lim = ld < COVER ? ld : COVER;
    for (int c = tid * 4; c < lim; c += BLOCK * 4) {
        f32x4 v = {dwbuf[c], dwbuf[c + 1], dwbuf[c + 2], dwbuf[c + 3]};
        *reinterpret_cast<f32x4*>(out + c) = v;
    }
    // columns between COVER and ld (COVER can be as small as 32) belong to no lane
    for (int c = COVER + tid; c < ld; c += BLOCK) out[c] = 0.0f;
}

// =================================================================================
// Forward, generic: one workgroup of 256 threads per row, any cols, any alignment.
// =================================================================================
template <typename T>
__global__ void __launch_bounds__(256)
rmsnorm_fwd_generic(T* __restrict__ y, float* __restrict__ inv_rms, const T* __restrict__ x,
                    const T* __restrict__ w, long rows, int cols, float eps, float inv_cols) {
    const long row = blockIdx.x;
    if (row >= rows) return;
    const T* xr = x + row * (long)cols;
    T* yr = y + row * (long)cols;
    float ss = 0.0f;
    for (int c = threadIdx.x; c < cols; c += 256) {
        float v = Elem<T>::load1(xr + c);
        ss = __builtin_fmaf(v, v, ss);
    }
    ss = wave_sum(ss);
    __shared__ float part[4];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    ss = (part[0] + part[1]) + (part[2] + part[3]);
    const float s = fast_rsqrt(ss * inv_cols + eps);
    if (threadIdx.x == 0 && inv_rms != nullptr) inv_rms[row] = s;
    for (int c = threadIdx.x; c < cols; c += 256) {
        float v = Elem<T>::load1(xr + c);
        float wv = Elem<T>::load1(w + c);
        Elem<T>::store1(yr + c, (v * s) * wv);
    }
}

// =================================================================================
// Backward pass 1, register-resident and persistent.
//   block = BLOCK threads (1024 or 512) = RG row slots of TPR threads; grid = P workgroups.
//   Row slot q = wg*RG + rg (wg = the workgroup's logical id) handles rows q, q + P*RG, q + 2*P*RG, ... and keeps
//   the dW contributions of its columns in fp32 registers; the next row's x and dy are
//   requested before the current row is reduced, so loads stay in flight across the
//   per-row barrier.  At the end the RG slots of a workgroup are added in slot order
//   through LDS and the workgroup writes row wg of the [P, ld] partial matrix.
// =================================================================================
template <typename T, int VEC, int TPR, int ITEMS, int BLOCK, bool PREFETCH>
__global__ void __launch_bounds__(BLOCK)
rmsnorm_bwd_rows(T* __restrict__ dx, float* __restrict__ dw_part, int ld, const T* __restrict__ dy,
                 const T* __restrict__ x, const T* __restrict__ w, const float* __restrict__ inv_rms,
                 long rows, int cols, float inv_cols, int xcd_group) {
    static_assert(BLOCK % TPR == 0 && TPR % kWave == 0, "row slots must tile the workgroup");
    constexpr int RG = BLOCK / TPR;
    constexpr int WPR = TPR / kWave;
    constexpr int NW = VEC / 4;
    constexpr int EPV = VEC / (int)sizeof(T);
    constexpr int COVER = TPR * ITEMS * EPV;  // columns covered by one row slot (>= cols)
    static_assert(RG == 1 || COVER * 4 <= 65536, "LDS combine buffer limited to 64 KiB");

    const int tid = threadIdx.x;
    const int rg = __builtin_amdgcn_readfirstlane(tid / TPR);
    const int lir = tid - rg * TPR;
    const long nslots = (long)gridDim.x * RG;
    const long wg = xcd_remap(blockIdx.x, gridDim.x, xcd_group);  // logical workgroup: owns partial row wg
    const long slot = wg * RG + rg;
    const long n_it = (rows + nslots - 1) / nslots;
    const u32 row_bytes = (u32)cols * (u32)sizeof(T);

    __shared__ float red[2][RG][WPR > 1 ? WPR : 1];

    float acc[ITEMS][EPV];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i)
#pragma unroll
        for (int k = 0; k < EPV; ++k) acc[i][k] = 0.0f;

    const RowTail tail = row_tail<T, TPR>(cols, row_bytes);
    Words<NW> wv[ITEMS];
    load_row<NW, ITEMS, TPR, kKeep>(wv, make_rsrc(w, row_bytes), lir, tail);

    Words<NW> xv[ITEMS], gv[ITEMS];
    u32 x_tail, g_tail;   // the odd last element of a 2-byte row, patched in when the row is used
    long row = slot;
    bool live = row < rows;
    float s = 0.0f;
    {
        const long base = live ? row * (long)cols : 0;
        const rsrc_t rx = make_rsrc(x + base, live ? row_bytes : 0u);
        const rsrc_t rg_ = make_rsrc(dy + base, live ? row_bytes : 0u);
        request_row<NW, ITEMS, TPR, kStream>(xv, x_tail, rx, lir, tail);
        request_row<NW, ITEMS, TPR, kStream>(gv, g_tail, rg_, lir, tail);
        if (live) s = inv_rms[row];
    }

    for (long it = 0; it < n_it; ++it) {
        const long nrow = row + nslots;
        const bool nlive = nrow < rows;
        Words<NW> nxv[PREFETCH ? ITEMS : 1], ngv[PREFETCH ? ITEMS : 1];
        u32 nx_tail = 0, ng_tail = 0;
        float ns = 0.0f;
        if constexpr (PREFETCH) {
            // request the next row of this slot now (nothing is fetched when there is none)
            const long nbase = nlive ? nrow * (long)cols : 0;
            const rsrc_t rx = make_rsrc(x + nbase, nlive ? row_bytes : 0u);
            const rsrc_t rg_ = make_rsrc(dy + nbase, nlive ? row_bytes : 0u);
            request_row<NW, ITEMS, TPR, kStream>(nxv, nx_tail, rx, lir, tail);
            request_row<NW, ITEMS, TPR, kStream>(ngv, ng_tail, rg_, lir, tail);
            if (nlive) ns = inv_rms[nrow];
        }
        patch_row_tail<NW, ITEMS>(xv, x_tail, lir, tail);
        patch_row_tail<NW, ITEMS>(gv, g_tail, lir, tail);

        // A = sum dy*w*x over the row; dW += dy*x*s
        float a = 0.0f;
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            float xf[EPV], gf[EPV], wf[EPV];
            unpack_vec<T, NW>(xv[i], xf);
            unpack_vec<T, NW>(gv[i], gf);
            unpack_vec<T, NW>(wv[i], wf);
#pragma unroll
            for (int k = 0; k < EPV; ++k) {
                const float t = gf[k] * xf[k];
                a = __builtin_fmaf(t, wf[k], a);
                acc[i][k] = __builtin_fmaf(t, s, acc[i][k]);
            }
        }
        a = wave_sum(a);
        if constexpr (WPR > 1) {
            const int wir = __builtin_amdgcn_readfirstlane(lir / kWave);
            const int buf = (int)(it & 1);
            if ((tid & (kWave - 1)) == 0) red[buf][rg][wir] = a;
            __syncthreads();
            float t = 0.0f;
#pragma unroll
            for (int k = 0; k < WPR; ++k) t += red[buf][rg][k];
            a = t;
        }
        // dx = s*dy*w - x * (A * s^3 / cols)
        const float c2 = a * (s * s) * s * inv_cols;
        {
            const long base = live ? row * (long)cols : 0;
            const rsrc_t rd = make_rsrc(dx + base, live ? row_bytes : 0u);
#pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                float xf[EPV], gf[EPV], wf[EPV], o[EPV];
                unpack_vec<T, NW>(xv[i], xf);
                unpack_vec<T, NW>(gv[i], gf);
                unpack_vec<T, NW>(wv[i], wf);
#pragma unroll
                for (int k = 0; k < EPV; ++k) o[k] = __builtin_fmaf(gf[k] * wf[k], s, -(xf[k] * c2));
                store_item<NW, TPR, kStream>(rd, lir, i, pack_vec<T, NW>(o), tail);
            }
        }
        if constexpr (PREFETCH) {
#pragma unroll
            for (int i = 0; i < ITEMS; ++i) { xv[i] = nxv[i]; gv[i] = ngv[i]; }
            x_tail = nx_tail; g_tail = ng_tail;
        } else {
            // wide rows: no second copy of the row in registers; the next row is requested
            // once this one is stored, and a second workgroup on the CU covers the wait
            const long nbase = nlive ? nrow * (long)cols : 0;
            const rsrc_t rx = make_rsrc(x + nbase, nlive ? row_bytes : 0u);
            const rsrc_t rg_ = make_rsrc(dy + nbase, nlive ? row_bytes : 0u);
            request_row<NW, ITEMS, TPR, kStream>(xv, x_tail, rx, lir, tail);
            request_row<NW, ITEMS, TPR, kStream>(gv, g_tail, rg_, lir, tail);
            if (nlive) ns = inv_rms[nrow];
        }
        row = nrow; live = nlive; s = ns;
    }

    // ---- combine the RG row slots in slot order, write this workgroup's partial row ----
    float* out = dw_part + wg * ld;
    if constexpr (RG == 1) {
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            const int c0 = (lir + i * TPR) * EPV;
#pragma unroll
            for (int k = 0; k < EPV; ++k)
                if (c0 + k < ld) out[c0 + k] = acc[i][k];
        }
    } else {
        __shared__ float dwbuf[COVER];
        for (int g = 0; g < RG; ++g) {
            if (rg == g) {
#pragma unroll
                for (int i = 0; i < ITEMS; ++i) {
                    const int c0 = (lir + i * TPR) * EPV;
#pragma unroll
                    for (int k = 0; k < EPV; ++k) {
                        if (g == 0) dwbuf[c0 + k] = acc[i][k];
                        else dwbuf[c0 + k] += acc[i][k];
                    }
                }
            }
            __syncthreads();
        }
        const int lim = ld < COVER ? ld : COVER;  // ld % 4 == 0 and COVER % 4 == 0
        for (int c = tid * 4; c < lim; c += BLOCK * 4) {
            f32x4 v = {dwbuf[c], dwbuf[c + 1], dwbuf[c + 2], dwbuf[c + 3]};
            *reinterpret_cast<f32x4*>(out + c) = v;
        }
    }
}

// =================================================================================
// Backward pass 1 over a ring of DEPTH register buffers per row slot, for rows whose pitch is
// a multiple of 16 bytes (no ragged last vector, no half-dword tail).  The same persistent
// grid, row slots and partial rows as rmsnorm_bwd_rows; what differs is how the next rows are
// kept in flight.  There the prefetched row is copied into the working registers at the end of
// an iteration, which makes every wave wait for it before it may request another; here the
// loop is unrolled DEPTH times over DEPTH register buffers, buffer (d + DEPTH - 1) % DEPTH is
// requested right before buffer d is worked on, and the only waits are the partial ones in
// front of a buffer's first use, so a slot always has DEPTH - 1 rows requested ahead and no
// register copies.  With one vector per thread (twice the threads per row) this measures
// 1-5 % faster than the copying loop on rows that fill their lanes (MI355X, bf16, 65536 rows:
// 2048 columns 124.3 against 129.0 us, 8192 columns at 16384 rows 126.4 against 130.0,
// 4096 x 4096 18.4-18.6 against 18.85), and slower where the last vector of a thread is mostly
// empty (5120 columns: 335 against 319 us) or the pitch is not a multiple of 16 bytes (4100
// columns: 277-299 against 267), which therefore stay with rmsnorm_bwd_rows.
// Iterations past the last row of a slot (the loop runs a multiple of DEPTH) work on an empty
// buffer resource: loads return 0, stores are dropped, the row scale is 0.
//
// TRACE = true is the same kernel with time stamps (the 100 MHz constant clock): thread 0 of
// every workgroup writes a record of kTimelineWords 64-bit words to `timeline` -- [0] start,
// [1 + i] end of iteration i (the first kTimelineIters of them), [kTimelineWords - 3] end of the
// row loop, [kTimelineWords - 2] end of the workgroup, [kTimelineWords - 1] the die (XCC) it ran
// on -- which is what mg_rmsnorm_bwd_timeline returns.  Without TRACE `timeline` is not touched.
// =================================================================================
constexpr int kTimelineWords = 32;
constexpr int kTimelineIters = 24;

template <typename T, int VEC, int TPR, int ITEMS, int BLOCK, int DEPTH, bool TRACE = false, int PARTIAL_POLICY = 0>
__global__ void __launch_bounds__(BLOCK)
rmsnorm_bwd_rows_ring(T* __restrict__ dx, float* __restrict__ dw_part, int ld, const T* __restrict__ dy,
                      const T* __restrict__ x, const T* __restrict__ w, const float* __restrict__ inv_rms,
                      long rows, int cols, float inv_cols, unsigned long long* __restrict__ timeline) {
    static_assert(BLOCK % TPR == 0 && TPR % kWave == 0, "row slots must tile the workgroup");
    static_assert(DEPTH >= 2 && DEPTH <= 4, "2 to 4 register buffers per row slot");
    constexpr int RG = BLOCK / TPR;
    constexpr int WPR = TPR / kWave;
    constexpr int NW = VEC / 4;
    constexpr int EPV = VEC / (int)sizeof(T);
    constexpr int COVER = TPR * ITEMS * EPV;
    static_assert(RG == 1 || COVER * 4 <= 65536, "LDS combine buffer limited to 64 KiB");

    const int tid = threadIdx.x;
    const int rg = __builtin_amdgcn_readfirstlane(tid / TPR);
    const int lir = tid - rg * TPR;
    const long nslots = (long)gridDim.x * RG;
    const long wg = blockIdx.x;
    const long slot = wg * RG + rg;
    const int n_it = (int)((rows + nslots - 1) / nslots);   // rows < 2^31
    const u32 row_bytes = (u32)cols * (u32)sizeof(T);

    __shared__ float red[2][RG][WPR > 1 ? WPR : 1];
    unsigned long long t_start = 0;
    if constexpr (TRACE) t_start = wall_clock64();

    float acc[ITEMS][EPV];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i)
#pragma unroll
        for (int k = 0; k < EPV; ++k) acc[i][k] = 0.0f;

    float wf[ITEMS][EPV];   // the weights stay unpacked for the whole kernel
    {
        const rsrc_t rw = make_rsrc(w, row_bytes);
#pragma unroll
        for (int i = 0; i < ITEMS; ++i)
            unpack_vec<T, NW>(buf_load<NW, kKeep>(rw, (u32)(lir + i * TPR) * VEC), wf[i]);
    }

    Words<NW> bx[DEPTH][ITEMS], bg[DEPTH][ITEMS];
    float bs[DEPTH];
    auto request = [&](int d, long row) {
        const bool live = row < rows;
        const long base = live ? row * (long)cols : 0;
        const rsrc_t rx = make_rsrc(x + base, live ? row_bytes : 0u);
        const rsrc_t rgd = make_rsrc(dy + base, live ? row_bytes : 0u);
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) bx[d][i] = buf_load<NW, kStream>(rx, (u32)(lir + i * TPR) * VEC);
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) bg[d][i] = buf_load<NW, kStream>(rgd, (u32)(lir + i * TPR) * VEC);
        bs[d] = live ? inv_rms[row] : 0.0f;
    };

#pragma unroll
    for (int d = 0; d < DEPTH - 1; ++d) request(d, slot + d * nslots);

    for (int it0 = 0; it0 < n_it; it0 += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int it = it0 + d;
            const long row = slot + (long)it * nslots;
            const bool live = row < rows;
            request((d + DEPTH - 1) % DEPTH, row + (DEPTH - 1) * nslots);
            const float s = bs[d];

            // A = sum dy*w*x over the row; dW += dy*x*s
            float a = 0.0f;
#pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                float xf[EPV], gf[EPV];
                unpack_vec<T, NW>(bx[d][i], xf);
                unpack_vec<T, NW>(bg[d][i], gf);
#pragma unroll
                for (int k = 0; k < EPV; ++k) {
                    const float t = gf[k] * xf[k];
                    a = __builtin_fmaf(t, wf[i][k], a);
                    acc[i][k] = __builtin_fmaf(t, s, acc[i][k]);
                }
            }
            a = wave_sum(a);
            if constexpr (WPR > 1) {
                const int wir = __builtin_amdgcn_readfirstlane(lir / kWave);
                const int buf = it & 1;
                if ((tid & (kWave - 1)) == 0) red[buf][rg][wir] = a;
                __syncthreads();
                float t = 0.0f;
#pragma unroll
                for (int k = 0; k < WPR; ++k) t += red[buf][rg][k];
                a = t;
            }
            // dx = s*dy*w - x * (A * s^3 / cols)
            const float c2 = a * (s * s) * s * inv_cols;
            const long base = live ? row * (long)cols : 0;
            const rsrc_t rd = make_rsrc(dx + base, live ? row_bytes : 0u);
#pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                float xf[EPV], gf[EPV], o[EPV];
                unpack_vec<T, NW>(bx[d][i], xf);
                unpack_vec<T, NW>(bg[d][i], gf);
#pragma unroll
                for (int k = 0; k < EPV; ++k) o[k] = __builtin_fmaf(gf[k] * wf[i][k], s, -(xf[k] * c2));
                buf_store<NW, kStream>(rd, (u32)(lir + i * TPR) * VEC, pack_vec<T, NW>(o));
            }
            if constexpr (TRACE) {
                if (tid == 0 && it < kTimelineIters) timeline[wg * kTimelineWords + 1 + it] = wall_clock64();
            }
        }
    }
    unsigned long long t_loop = 0;
    if constexpr (TRACE) t_loop = wall_clock64();

    // ---- combine the RG row slots in slot order, write this workgroup's partial row ----
    // PARTIAL_POLICY (one slot per workgroup only): the cache-policy bits of the partial row's
    // stores -- 0 default (the row stays in this die's L2 until the end-of-kernel write-back),
    // kStream non-temporal, 17 (sc0 sc1) written through to memory at once.  Measured at
    // 4096 x 4096 bf16 they differ by less than the run-to-run spread, so 0 is what runs; the
    // other two exist for the "bwd_partial_policy" option.
    float* out = dw_part + wg * ld;
    if constexpr (RG == 1) {
        const rsrc_t rp = make_rsrc(out, (u32)ld * 4u);   // ld < 2^29 floats: cols < 2^31 bytes per row
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            const int c0 = (lir + i * TPR) * EPV;   // ld % 4 == 0 and EPV % 4 == 0
#pragma unroll
            for (int h = 0; h < EPV / 4; ++h) {
                const f32x4 v = {acc[i][4 * h], acc[i][4 * h + 1], acc[i][4 * h + 2], acc[i][4 * h + 3]};
                if constexpr (PARTIAL_POLICY == 0) {
                    if (c0 + 4 * h < ld) *reinterpret_cast<f32x4*>(out + c0 + 4 * h) = v;
                } else {   // out-of-range offsets are dropped by the buffer's range check
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), rp, (c0 + 4 * h) * 4, 0, PARTIAL_POLICY);
                }
            }
        }
    } else {
        __shared__ float dwbuf[COVER];
        for (int g = 0; g < RG; ++g) {
            if (rg == g) {
#pragma unroll
                for (int i = 0; i < ITEMS; ++i) {
                    const int c0 = (lir + i * TPR) * EPV;
#pragma unroll
                    for (int k = 0; k < EPV; ++k) {
                        if (g == 0) dwbuf[c0 + k] = acc[i][k];
                        else dwbuf[c0 + k] += acc[i][k];
                    }
                }
            }
            __syncthreads();
        }
        const int lim = ld < COVER ? ld : COVER;  // ld % 4 == 0 and COVER % 4 == 0
        for (int c = tid * 4; c < lim; c += BLOCK * 4) {
            f32x4 v = {dwbuf[c], dwbuf[c + 1], dwbuf[c + 2], dwbuf[c + 3]};
            *reinterpret_cast<f32x4*>(out + c) = v;
        }
    }
    if constexpr (TRACE) {
        if (tid == 0) {
            u32 xcc = 0;
            asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
            unsigned long long* rec = timeline + wg * kTimelineWords;
            rec[0] = t_start;
            rec[kTimelineWords - 3] = t_loop;
            rec[kTimelineWords - 2] = wall_clock64();
            rec[kTimelineWords - 1] = xcc & 0xfu;
        }
    }
}

// =================================================================================
// Backward pass 1 for rows of up to 4096 vectors on 1024 threads (used from 2049 vectors on,
// and from 1537 for the 2-byte types): the same persistent scheme with one row slot per
// workgroup, but the dW sums -- 8 floats per vector of a 2-byte type, which registers no
// longer hold next to the row itself once a thread has more than two vectors (with 5-8
// vectors per thread at 512 threads the register kernel spills: 4.8 TB/s at 20 480 bf16
// columns, 1.2 at 32 768) -- live in LDS.  Each thread owns fixed 16-byte slices of it, so no
// synchronisation is needed.
//   block = TPR = 1024 threads; grid = P workgroups, one per compute unit (two for 2 vectors of
//   a 2-byte type); dynamic LDS = ITEMS * 1024 * (16 / sizeof(T)) floats (32 ... 128 KiB)
// =================================================================================
template <typename T, int ITEMS>
__global__ void __launch_bounds__(1024)
rmsnorm_bwd_rows_lds(T* __restrict__ dx, float* __restrict__ dw_part, int ld, const T* __restrict__ dy,
                     const T* __restrict__ x, const T* __restrict__ w, const float* __restrict__ inv_rms,
                     long rows, int cols, float inv_cols, int xcd_group) {
    constexpr int TPR = 1024;
    constexpr int WPR = TPR / kWave;
    constexpr int EPV = 16 / (int)sizeof(T);
    constexpr int QPV = EPV / 4;              // 16-byte slices of fp32 sums per vector of T
    static_assert(ITEMS * TPR * EPV * 4 <= 160 * 1024 - 1024, "the dW sums of a workgroup must fit the LDS of a compute unit");

    const int tid = threadIdx.x;
    const long nslots = gridDim.x;
    const long wg = xcd_remap(blockIdx.x, gridDim.x, xcd_group);
    const long n_it = (rows + nslots - 1) / nslots;
    const u32 row_bytes = (u32)cols * (u32)sizeof(T);

    __shared__ float red[2][WPR];
    // slice (i, h) of thread t: columns (t + i*TPR)*EPV + 4h .. +3, at sums[(i*QPV + h)*TPR + t];
    // consecutive threads are 16 bytes apart, so the accesses are free of bank conflicts
    extern __shared__ f32x4 sums[];
#pragma unroll
    for (int j = 0; j < ITEMS * QPV; ++j) sums[j * TPR + tid] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    const RowTail tail = row_tail<T, TPR>(cols, row_bytes);
    Words<4> wv[ITEMS];
    load_row<4, ITEMS, TPR, kKeep>(wv, make_rsrc(w, row_bytes), tid, tail);

    for (long it = 0; it < n_it; ++it) {
        const long row = wg + it * nslots;
        const bool live = row < rows;
        const long base = live ? row * (long)cols : 0;
        Words<4> xv[ITEMS], gv[ITEMS];
        u32 x_tail, g_tail;
        request_row<4, ITEMS, TPR, kStream>(xv, x_tail, make_rsrc(x + base, live ? row_bytes : 0u), tid, tail);
        request_row<4, ITEMS, TPR, kStream>(gv, g_tail, make_rsrc(dy + base, live ? row_bytes : 0u), tid, tail);
        patch_row_tail<4, ITEMS>(xv, x_tail, tid, tail);
        patch_row_tail<4, ITEMS>(gv, g_tail, tid, tail);
        const float s = live ? inv_rms[row] : 0.0f;

        float a = 0.0f;
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            float xf[EPV], gf[EPV], wf[EPV];
            unpack_vec<T, 4>(xv[i], xf);
            unpack_vec<T, 4>(gv[i], gf);
            unpack_vec<T, 4>(wv[i], wf);
#pragma unroll
            for (int h = 0; h < QPV; ++h) {
                f32x4 acc = sums[(i * QPV + h) * TPR + tid];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const float t = gf[4 * h + k] * xf[4 * h + k];
                    a = __builtin_fmaf(t, wf[4 * h + k], a);
                    acc[k] = __builtin_fmaf(t, s, acc[k]);
                }
                sums[(i * QPV + h) * TPR + tid] = acc;
            }
        }
        a = wave_sum(a);
        {
            const int wir = __builtin_amdgcn_readfirstlane(tid / kWave);
            const int buf = (int)(it & 1);
            if ((tid & (kWave - 1)) == 0) red[buf][wir] = a;
            __syncthreads();
            float t = 0.0f;
#pragma unroll
            for (int k = 0; k < WPR; ++k) t += red[buf][k];
            a = t;
        }
        const float c2 = a * (s * s) * s * inv_cols;
        const rsrc_t rd = make_rsrc(dx + base, live ? row_bytes : 0u);
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            float xf[EPV], gf[EPV], wf[EPV], o[EPV];
            unpack_vec<T, 4>(xv[i], xf);
            unpack_vec<T, 4>(gv[i], gf);
            unpack_vec<T, 4>(wv[i], wf);
#pragma unroll
            for (int k = 0; k < EPV; ++k) o[k] = __builtin_fmaf(gf[k] * wf[k], s, -(xf[k] * c2));
            store_item<4, TPR, kStream>(rd, tid, i, pack_vec<T, 4>(o), tail);
        }
    }

    // every thread writes its own slices of this workgroup's partial row
    float* out = dw_part + wg * ld;
#pragma unroll
    for (int i = 0; i < ITEMS; ++i)
#pragma unroll
        for (int h = 0; h < QPV; ++h) {
            const int c0 = (tid + i * TPR) * EPV + 4 * h;     // ld % 4 == 0
            if (c0 < ld) *reinterpret_cast<f32x4*>(out + c0) = sums[(i * QPV + h) * TPR + tid];
        }
}

// =================================================================================
// Backward, generic (any cols / alignment): dx per row, then dW partials per column.
// =================================================================================
template <typename T>
__global__ void __launch_bounds__(256)
rmsnorm_bwd_dx_generic(T* __restrict__ dx, const T* __restrict__ dy, const T* __restrict__ x,
                       const T* __restrict__ w, const float* __restrict__ inv_rms, long rows, int cols,
                       float inv_cols) {
    const long row = blockIdx.x;
    if (row >= rows) return;
    const T* xr = x + row * (long)cols;
    const T* gr = dy + row * (long)cols;
    T* dr = dx + row * (long)cols;
    const float s = inv_rms[row];
    float a = 0.0f;
    for (int c = threadIdx.x; c < cols; c += 256) {
        const float t = Elem<T>::load1(gr + c) * Elem<T>::load1(xr + c);
        a = __builtin_fmaf(t, Elem<T>::load1(w + c), a);
    }
    a = wave_sum(a);
    __shared__ float part[4];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = a;
    __syncthreads();
    a = (part[0] + part[1]) + (part[2] + part[3]);
    const float c2 = a * (s * s) * s * inv_cols;
    for (int c = threadIdx.x; c < cols; c += 256) {
        const float g = Elem<T>::load1(gr + c) * Elem<T>::load1(w + c);
        Elem<T>::store1(dr + c, __builtin_fmaf(g, s, -(Elem<T>::load1(xr + c) * c2)));
    }
}

// grid = (ceil(cols/256), P); thread owns one column and the rows p, p+P, p+2P, ...
template <typename T>
__global__ void __launch_bounds__(256)
rmsnorm_bwd_dw_generic(float* __restrict__ dw_part, int ld, const T* __restrict__ dy,
                       const T* __restrict__ x, const float* __restrict__ inv_rms, long rows, int cols) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    const int p = blockIdx.y;
    const int P = gridDim.y;
    if (c >= cols) return;
    float acc = 0.0f;
    for (long r = p; r < rows; r += P) {
        const float t = Elem<T>::load1(dy + r * (long)cols + c) * Elem<T>::load1(x + r * (long)cols + c);
        acc = __builtin_fmaf(t, inv_rms[r], acc);
    }
    dw_part[(long)p * ld + c] = acc;
}

// =================================================================================
// Rows too wide for registers: one 1024-thread workgroup
// per row streams the row twice with 16-byte buffer accesses -- once for the row sum, once
// for the output; the second read of a row that fits the L2 comes from there.  Four vectors
// per thread are in flight at a time; offsets past the row load 0 and store nothing.
// =================================================================================
constexpr int kWideBlock = 1024;
constexpr int kWideInFlight = 4;

// Sum over the 1024 threads of a workgroup, identical in every thread: DPP inside the waves,
// then the 16 wave sums through LDS in wave order.
__device__ __forceinline__ float wide_block_sum(float v, float* lds16) {
    v = wave_sum(v);
    __syncthreads();   // lds16 may still be read from a previous sum
    if ((threadIdx.x & (kWave - 1)) == 0) lds16[threadIdx.x / kWave] = v;
    __syncthreads();
    float t = 0.0f;
#pragma unroll
    for (int k = 0; k < kWideBlock / kWave; ++k) t += lds16[k];
    return t;
}

template <typename T>
__global__ void __launch_bounds__(kWideBlock)
rmsnorm_fwd_wide(T* __restrict__ y, float* __restrict__ inv_rms, const T* __restrict__ x,
                 const T* __restrict__ w, long rows, int cols, float eps, float inv_cols) {
    constexpr int EPV = 16 / (int)sizeof(T);
    __shared__ float lds16[kWideBlock / kWave];
    const long row = blockIdx.x;
    const u32 row_bytes = (u32)cols * (u32)sizeof(T);
    const u32 nvec = (row_bytes + 15u) / 16u;
    const rsrc_t rx = make_rsrc(x + row * (long)cols, row_bytes);
    const rsrc_t ry = make_rsrc(y + row * (long)cols, row_bytes);
    const rsrc_t rw = make_rsrc(w, row_bytes);
    const u32 stride = kWideBlock * kWideInFlight;

    float ss = 0.0f;
    for (u32 v0 = threadIdx.x; v0 < nvec; v0 += stride) {
        Words<4> xv[kWideInFlight];
#pragma unroll
        for (int k = 0; k < kWideInFlight; ++k) xv[k] = buf_load<4, kKeep>(rx, (v0 + k * kWideBlock) * 16u);
#pragma unroll
        for (int k = 0; k < kWideInFlight; ++k) {
            float f[EPV];
            unpack_vec<T, 4>(xv[k], f);
#pragma unroll
            for (int e = 0; e < EPV; ++e) ss = __builtin_fmaf(f[e], f[e], ss);
        }
    }
    // a row of an odd number of 2-byte elements ends in half a dword, which the range check
    // drops from the vectors: thread 0 carries that element by itself
    const bool odd_tail = sizeof(T) == 2 && (row_bytes & 2u) != 0 && threadIdx.x == 0;
    float x_last = 0.0f;
    if (odd_tail) {
        x_last = Elem<T>::load1(x + row * (long)cols + (cols - 1));
        ss = __builtin_fmaf(x_last, x_last, ss);
    }
    ss = wide_block_sum(ss, lds16);
    const float s = fast_rsqrt(ss * inv_cols + eps);
    if (threadIdx.x == 0 && inv_rms != nullptr) inv_rms[row] = s;
    if (odd_tail) Elem<T>::store1(y + row * (long)cols + (cols - 1), (x_last * s) * Elem<T>::load1(w + (cols - 1)));

    for (u32 v0 = threadIdx.x; v0 < nvec; v0 += stride) {
        Words<4> xv[kWideInFlight], wv[kWideInFlight];
#pragma unroll
        for (int k = 0; k < kWideInFlight; ++k) xv[k] = buf_load<4, kStream>(rx, (v0 + k * kWideBlock) * 16u);
#pragma unroll
        for (int k = 0; k < kWideInFlight; ++k) wv[k] = buf_load<4, kKeep>(rw, (v0 + k * kWideBlock) * 16u);
#pragma unroll
        for (int k = 0; k < kWideInFlight; ++k) {
            float xf[EPV], wf[EPV], o[EPV];
            unpack_vec<T, 4>(xv[k], xf);
            unpack_vec<T, 4>(wv[k], wf);
#pragma unroll
            for (int e = 0; e < EPV; ++e) o[e] = (xf[e] * s) * wf[e];
            buf_store<4, kStream>(ry, (v0 + k * kWideBlock) * 16u, pack_vec<T, 4>(o));
        }
    }
}

// dx for rows too wide for registers: pass 1 sums dy*w*x over the row, pass 2 writes dx.
template <typename T>
__global__ void __launch_bounds__(kWideBlock)
rmsnorm_bwd_dx_wide(T* __restrict__ dx, const T* __restrict__ dy, const T* __restrict__ x,
                    const T* __restrict__ w, const float* __restrict__ inv_rms, long rows, int cols,
                    float inv_cols) {
    constexpr int EPV = 16 / (int)sizeof(T);
    __shared__ float lds16[kWideBlock / kWave];
    const long row = blockIdx.x;
    const u32 row_bytes = (u32)cols * (u32)sizeof(T);
    const u32 nvec = (row_bytes + 15u) / 16u;
    const rsrc_t rx = make_rsrc(x + row * (long)cols, row_bytes);
    const rsrc_t rg = make_rsrc(dy + row * (long)cols, row_bytes);
    const rsrc_t rd = make_rsrc(dx + row * (long)cols, row_bytes);
    const rsrc_t rw = make_rsrc(w, row_bytes);
    const u32 stride = kWideBlock * kWideInFlight;
    const float s = inv_rms[row];

    float a = 0.0f;
    for (u32 v0 = threadIdx.x; v0 < nvec; v0 += stride) {
        Words<4> xv[kWideInFlight], gv[kWideInFlight], wv[kWideInFlight];
#pragma unroll
        for (int k = 0; k < kWideInFlight; ++k) xv[k] = buf_load<4, kKeep>(rx, (v0 + k * kWideBlock) * 16u);
#pragma unroll
        for (int k = 0; k < kWideInFlight; ++k) gv[k] = buf_load<4, kKeep>(rg, (v0 + k * kWideBlock) * 16u);
#pragma unroll
        for (int k = 0; k < kWideInFlight; ++k) wv[k] = buf_load<4, kKeep>(rw, (v0 + k * kWideBlock) * 16u);
#pragma unroll
        for (int k = 0; k < kWideInFlight; ++k) {
            float xf[EPV], gf[EPV], wf[EPV];
            unpack_vec<T, 4>(xv[k], xf);
            unpack_vec<T, 4>(gv[k], gf);
            unpack_vec<T, 4>(wv[k], wf);
#pragma unroll
            for (int e = 0; e < EPV; ++e) a = __builtin_fmaf(gf[e] * xf[e], wf[e], a);
        }
    }
    // the element in the half dword that ends a row of an odd number of 2-byte elements
    const bool odd_tail = sizeof(T) == 2 && (row_bytes & 2u) != 0 && threadIdx.x == 0;
    float x_last = 0.0f, gw_last = 0.0f;
    if (odd_tail) {
        const long at = row * (long)cols + (cols - 1);
        x_last = Elem<T>::load1(x + at);
        gw_last = Elem<T>::load1(dy + at) * Elem<T>::load1(w + (cols - 1));
        a = __builtin_fmaf(gw_last, x_last, a);
    }
    a = wide_block_sum(a, lds16);
    const float c2 = a * (s * s) * s * inv_cols;
    if (odd_tail) Elem<T>::store1(dx + row * (long)cols + (cols - 1), __builtin_fmaf(gw_last, s, -(x_last * c2)));

    for (u32 v0 = threadIdx.x; v0 < nvec; v0 += stride) {
        Words<4> xv[kWideInFlight], gv[kWideInFlight], wv[kWideInFlight];
#pragma unroll
        for (int k = 0; k < kWideInFlight; ++k) xv[k] = buf_load<4, kStream>(rx, (v0 + k * kWideBlock) * 16u);
#pragma unroll
        for (int k = 0; k < kWideInFlight; ++k) gv[k] = buf_load<4, kStream>(rg, (v0 + k * kWideBlock) * 16u);
#pragma unroll
        for (int k = 0; k < kWideInFlight; ++k) wv[k] = buf_load<4, kKeep>(rw, (v0 + k * kWideBlock) * 16u);
#pragma unroll
        for (int k = 0; k < kWideInFlight; ++k) {
            float xf[EPV], gf[EPV], wf[EPV], o[EPV];
            unpack_vec<T, 4>(xv[k], xf);
            unpack_vec<T, 4>(gv[k], gf);
            unpack_vec<T, 4>(wv[k], wf);
#pragma unroll
            for (int e = 0; e < EPV; ++e) o[e] = __builtin_fmaf(gf[e] * wf[e], s, -(xf[e] * c2));
            buf_store<4, kStream>(rd, (v0 + k * kWideBlock) * 16u, pack_vec<T, 4>(o));
        }
    }
}

// dW partials for rows too wide for registers: grid = (ceil(nvec / 256), P); a thread owns
// one 16-byte vector of columns and the rows p, p + P, p + 2P, ... (four rows in flight).
template <typename T>
__global__ void __launch_bounds__(256)
rmsnorm_bwd_dw_wide(float* __restrict__ dw_part, int ld, const T* __restrict__ dy, const T* __restrict__ x,
                    const float* __restrict__ inv_rms, long rows, int cols) {
    constexpr int EPV = 16 / (int)sizeof(T);
    const u32 row_bytes = (u32)cols * (u32)sizeof(T);
    const u32 vec = blockIdx.x * 256u + threadIdx.x;
    const u32 off = vec * 16u;          // past the row for the lanes beyond it: loads 0
    const long p = blockIdx.y, P = gridDim.y;
    // the thread whose vector holds the half dword that ends an odd row of 2-byte elements
    // fetches that element with 2-byte loads and puts it where the vector load left 0
    const bool odd_tail = sizeof(T) == 2 && (row_bytes & 2u) != 0 && vec == (row_bytes - 1u) / 16u;
    const int tail_word = (int)(((row_bytes - 2u) % 16u) / 4u);
    float acc[EPV];
#pragma unroll
    for (int e = 0; e < EPV; ++e) acc[e] = 0.0f;
    for (long r0 = p; r0 < rows; r0 += 4 * P) {
        Words<4> xv[4], gv[4];
        float sr[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const long r = r0 + k * P;
            const bool live = r < rows;
            const long base = live ? r * (long)cols : 0;
            const rsrc_t rx = make_rsrc(x + base, live ? row_bytes : 0u);
            const rsrc_t rg = make_rsrc(dy + base, live ? row_bytes : 0u);
            xv[k] = buf_load<4, kStream>(rx, off);
            gv[k] = buf_load<4, kStream>(rg, off);
            if (odd_tail) {
                const u32 xb = load_b16<kStream>(rx, row_bytes - 2u), gb = load_b16<kStream>(rg, row_bytes - 2u);
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (j == tail_word) { xv[k].v[j] = xb; gv[k].v[j] = gb; }
            }
            sr[k] = live ? inv_rms[r] : 0.0f;
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            float xf[EPV], gf[EPV];
            unpack_vec<T, 4>(xv[k], xf);
            unpack_vec<T, 4>(gv[k], gf);
#pragma unroll
            for (int e = 0; e < EPV; ++e) acc[e] = __builtin_fmaf(gf[e] * xf[e], sr[k], acc[e]);
        }
    }
    float* out = dw_part + p * (long)ld;
#pragma unroll
    for (int e = 0; e < EPV; ++e) {
        const long c = (long)vec * EPV + e;
        if (c < ld) out[c] = acc[e];
    }
}

// =================================================================================
// Backward pass 2: dW[c] = sum_p part[p, c] in a fixed order.
//   block = 256 threads = 8 column quads (32 columns = one 128-byte line per partial row)
//   x 32 row subsets; thread (q, sub) adds rows sub, sub+32, ... with eight independent
//   loads in flight; the 32 subsets are then added in subset order through LDS.  The partial
//   rows are read once, with non-temporal loads (4096 columns x 256 rows: 3.15 against 3.4 us).
//   grid = ceil(cols / 32).
// =================================================================================
constexpr int kReduceCols = 32;

template <typename TC>
__global__ void __launch_bounds__(256)
rmsnorm_dw_reduce(float* __restrict__ dw_f32, TC* __restrict__ dw_cast, const float* __restrict__ part,
                  int P, int ld, int cols) {
    constexpr int QUADS = kReduceCols / 4;  // 8
    constexpr int SUBS = 256 / QUADS;       // 32
    const int q = threadIdx.x % QUADS;
    const int sub = threadIdx.x / QUADS;
    const int c0 = blockIdx.x * kReduceCols + q * 4;  // < ld: ld % 64 == 0 and the grid covers cols
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    if (c0 < ld) {
        int p = sub;
        for (; p + 7 * SUBS < P; p += 8 * SUBS) {   // 8 independent loads in flight per thread
            f32x4 v[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) v[k] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(part + (long)(p + k * SUBS) * ld + c0));
#pragma unroll
            for (int k = 0; k < 8; ++k) acc += v[k];
        }
        for (; p < P; p += SUBS) acc += __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(part + (long)p * ld + c0));
    }
    __shared__ f32x4 sm[SUBS][QUADS];
    sm[sub][q] = acc;
    __syncthreads();
    if (threadIdx.x < kReduceCols) {
        const int qq = threadIdx.x >> 2, k = threadIdx.x & 3;
        float t = 0.0f;
#pragma unroll
        for (int j = 0; j < SUBS; ++j) t += sm[j][qq][k];
        const int c = blockIdx.x * kReduceCols + threadIdx.x;
        if (c < cols) {
            if (dw_f32 != nullptr) dw_f32[c] = t;
            if (dw_cast != nullptr) Elem<TC>::store1(dw_cast + c, t);
        }
    }
}

}  // namespace mg
