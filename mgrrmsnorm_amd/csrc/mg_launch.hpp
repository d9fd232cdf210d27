// Internal interface between the C ABI (mg_api.hip) and the per-dtype kernel
// translation units.  Everything here is host code.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <tuple>
#include <utility>

namespace mg {

// Kernel launch whose return value is this launch's own status.  hipLaunchKernel reports it
// directly, so nothing has to be read from the thread's last-error slot, which other users of
// the HIP runtime in the process (torch) share: an error they left there stays where it is.
// When our launch fails, the runtime has put that error into the slot as well; it is ours and
// is taken out again, so that it does not surface in somebody else's next check.
template <typename... P, size_t... I>
hipError_t launch_unpacked(void (*kernel)(P...), dim3 grid, dim3 block, size_t lds_bytes, hipStream_t s,
                           std::tuple<P...>& vals, std::index_sequence<I...>) {
    void* ptrs[] = {static_cast<void*>(&std::get<I>(vals))...};
    const hipError_t e = hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, ptrs, lds_bytes, s);
    if (e != hipSuccess) (void)hipGetLastError();
    return e;
}
template <typename... P, typename... A>
hipError_t launch(void (*kernel)(P...), dim3 grid, dim3 block, size_t lds_bytes, hipStream_t s, A... args) {
    static_assert(sizeof...(P) == sizeof...(A), "one argument per kernel parameter");
    std::tuple<P...> vals{static_cast<P>(args)...};
    return launch_unpacked(kernel, grid, block, lds_bytes, s, vals, std::index_sequence_for<P...>{});
}

// How a row is spread over threads in the register-resident RMSNorm kernels.
struct RowCfg {
    int vec;    // bytes per vector load (16)
    int tpr;    // threads per row: 64, 128, 256, 512, 1024; 8, 16 or 32 = several rows per wave
    int items;  // vectors per thread
    int block;  // backward only: threads per workgroup, 1024 or 512
    int family; // kFamilyResident (rows held in registers), kFamilyStreaming (rows read twice) or
                // kFamilyGroups (narrow rows, one vector per lane; `items` = row groups in flight) or
                // kFamilyLdsSums (backward: rows in registers, dW sums in LDS) or
                // kFamilyRing (backward: a ring of `depth` register buffers per row slot) or
                // kFamilyLines (forward: rows in registers, vectors on the 128-byte lines of y)
    int depth;  // kFamilyRing only: register buffers per row slot (2 or 4); 0 = chosen per call
};
constexpr int kFamilyResident = 0, kFamilyStreaming = 1;
// Rows of at most 64 vectors can also go one vector per lane, `items` groups of 64/tpr rows
// per wave in flight ("row groups"); `tpr` is then a power of two from 1 to 64 and at least the
// row's vectors (below 8 lanes per row only with 2 or 4 groups).
constexpr int kFamilyGroups = 2;
// Backward only: rows of 1025-4096 vectors on 1024 threads with 2, 3 or 4 vectors each and the
// dW sums in LDS (32 KiB of dynamic LDS per vector of a thread for the 2-byte types, 16 KiB for fp32).
constexpr int kFamilyLdsSums = 3;
constexpr bool bwd_lds_ok(int esize, long nvec, int items) {
    return (esize == 2 || esize == 4) && nvec > 1024 && nvec <= 4096 && (items == 2 || items == 3 || items == 4) && nvec <= 1024L * items;
}
// Backward only: rows whose pitch is a multiple of 16 bytes, one vector per thread on 64 ... 1024
// threads (512-thread workgroups, 1024 for 1024 threads per row), or two vectors on 1024
// threads, with the rows of a slot kept in flight through a ring of register buffers.
constexpr int kFamilyRing = 4;
constexpr bool bwd_ring_ok(long row_bytes, int tpr, int items, int depth) {
    const long nvec = (row_bytes + 15) / 16;
    const bool shape = (items == 1 && (tpr == 64 || tpr == 128 || tpr == 256 || tpr == 512 || tpr == 1024)) ||
                       (items == 2 && tpr == 1024);
    return shape && row_bytes % 16 == 0 && nvec <= (long)tpr * items && (depth == 2 || depth == 4);
}
// Forward only, on request: the register-resident layout with the vectors on the 128-byte lines of y, for
// row pitches that are multiples of 8 but not of 128 bytes and rows of more than 256 vectors
// (4 KiB; measured from there on).
// The slots of a row start at the line that holds its first byte, so up to 120 bytes of slots
// lie in front of the row: `fwd_lines_shape` gives the threads per row and vectors per thread
// for ceil((120 + row bytes) / 16) slots by the rule of the plain layout (the fewest threads at
// two vectors each; half the threads at three when the second vector would be mostly empty;
// 512 x 3 for 1025-1536 slots), 0 threads = the row does not take this layout.
constexpr int kFamilyLines = 5;
constexpr bool fwd_lines_pitch(long row_bytes) { return row_bytes % 8 == 0 && row_bytes % 128 != 0 && row_bytes > 256 * 16; }
struct LinesShape { int tpr, items; };
constexpr LinesShape fwd_lines_shape(long row_bytes) {
    if (!fwd_lines_pitch(row_bytes)) return {0, 0};
    const long slots = (row_bytes + 120 + 15) / 16;
    if (slots > 1024 && slots <= 1536) return {512, 3};
    for (int t = 128; t <= 1024; t *= 2) {
        int need = (int)((slots + t - 1) / t);
        if (need == 7) need = 8;
        if (need <= 2 || (t == 1024 && need <= 8)) {
            if (need == 2 && t >= 256 && slots * 10 < (long)t * 12) { t /= 2; need = (int)((slots + t - 1) / t); }
            return {t, need};
        }
    }
    return {0, 0};
}
constexpr bool fwd_lines_ok(long row_bytes, int tpr, int items) {
    const bool shape = (tpr == 128 || tpr == 256 || tpr == 512 || tpr == 1024) && items >= 1 && items <= 8 && items != 7;
    return shape && fwd_lines_pitch(row_bytes) && (row_bytes + 120 + 15) / 16 <= (long)tpr * items;
}
constexpr bool groups_ok(long row_bytes, int tpr, int groups) {
    const bool lanes = tpr == 1 || tpr == 2 || tpr == 4 || tpr == 8 || tpr == 16 || tpr == 32 || tpr == 64;
    return lanes && (row_bytes + 15) / 16 <= tpr && (groups == 2 || groups == 4 || (groups == 1 && tpr >= 8));
}
constexpr int groups_tpr(long row_bytes) {   // 0 = the row has more than 64 vectors
    const long nvec = (row_bytes + 15) / 16;
    int t = 1;
    while (t < nvec && t < 128) t *= 2;
    return t <= 64 ? t : 0;
}
// Which rows take the row-group layout by default, and with how many groups in flight
// (0 = the several-vectors-per-lane layout).  From sweeps over 4...512 columns of all three
// types at 2^18...2^20 rows on MI355X:
//  - pitch a multiple of 16 bytes: the row-group layout whenever the pitch is not a multiple of
//    128 bytes (there the other layout writes cache lines in pieces: 80 bf16 columns forward
//    3.9 -> 5.8 TB/s, backward 4.8 -> 5.7; 200 columns 3.7 -> 5.8 and 5.3 -> 6.0), and for rows
//    of up to 16 vectors in any case (128 columns: 6.0 -> 6.2 and 6.0 -> 6.1); four groups
//    forward, two backward (which also keeps the next block's two in flight);
//  - other pitches: only while a row fills three quarters of its lanes or has at most 8
//    vectors, and up to 32 vectors (100 bf16 columns: 4.6 -> 5.1 and 4.6 -> 5.1; 129 columns,
//    17 of 32 lanes: backward 4.2 -> 3.0, so not there).
constexpr int groups_default(long row_bytes, bool backward) {
    const long nvec = (row_bytes + 15) / 16;
    const int tpr = groups_tpr(row_bytes);
    if (tpr == 0) return 0;
    if (row_bytes % 16 == 0) {
        if (row_bytes % 128 == 0 && nvec > 16) return 0;
        return backward ? 2 : 4;
    }
    if (tpr > 32 || !(nvec <= 8 || 4 * nvec >= 3 * tpr)) return 0;
    return backward ? (nvec <= 16 ? 4 : 2) : 2;
}
// Rows that do not fit registers stream through 1024-thread workgroups.

constexpr int kVec = 16;

// Largest ITEMS instantiated.
constexpr int kFwdMaxItems = 8;
constexpr int kBwdMaxItems = 8;

// Forward: ITEMS in {1,2,3,4,5,6,8}.
constexpr bool fwd_items_ok(int items) { return items >= 1 && items <= 8 && items != 7; }
// Backward: 1024-thread workgroups (128 VGPRs per thread) hold up to 2 vectors per
// thread without spilling, 512-thread workgroups (256 VGPRs) up to 8 (ITEMS in
// {1,2,3,4,6,8}).  When several row slots share a workgroup their combine buffer
// (tpr * items * elements-per-vector floats) must fit 64 KiB of LDS.
// 256-thread workgroups (one row slot of 256 threads, up to 2 vectors each, several workgroups per
// compute unit) exist on request only ("bwd_block" = 256): they measure slower than two slots in
// one 512-thread workgroup, and every workgroup adds a partial row.
constexpr bool bwd_cfg_ok(int esize, int tpr, int items, int block) {
    if (block == 256) return tpr == 256 && (items == 1 || items == 2);
    return (block == 1024 || block == 512) && tpr <= block &&
           items >= 1 && items <= (block == 1024 ? 2 : kBwdMaxItems) && items != 5 && items != 7 &&
           (tpr == block || tpr * items * (kVec / esize) * 4 <= 65536);
}
constexpr bool tpr_ok(int tpr) { return tpr == 64 || tpr == 128 || tpr == 256 || tpr == 512 || tpr == 1024; }

// Rows of at most 128 vectors can share a wave: 8, 16 or 32 lanes per row and up to 4
// vectors per lane.
constexpr bool narrow_tpr(int tpr) { return tpr == 8 || tpr == 16 || tpr == 32; }
constexpr int narrow_items(long row_bytes, int tpr) {   // 0 = does not fit
    if (!narrow_tpr(tpr)) return 0;
    const long need = ((row_bytes + kVec - 1) / kVec + tpr - 1) / tpr;
    return need <= 4 ? (int)need : 0;
}
// Default use, from sweeps over row widths on MI355X (0 = one or more waves per row).
// Pitch a multiple of 16 bytes -- forward: the fewest lanes that hold the row in 4 vectors
// each, up to 128 vectors; backward (which also carries dy, a prefetched row and the dW
// sums): 2 vectors each, up to 56 vectors; from there on one wave per row is as fast.
// Other pitches (a row's last vector is moved in pieces and rows share cache lines) gain
// only while a row is short: up to 40 vectors, with the split that measured best.
constexpr int narrow_default_tpr(long row_bytes, bool backward) {
    const long nvec = (row_bytes + kVec - 1) / kVec;
    if (row_bytes % kVec != 0) return nvec <= 24 ? 8 : (nvec <= 32 ? 32 : (nvec <= 40 ? 16 : 0));
    if (backward) return nvec <= 16 ? 8 : (nvec <= 32 ? 16 : (nvec <= 56 ? 32 : 0));
    // 65-128 vectors: only pitches that are multiples of 128 bytes (others measure 6-11 %
    // faster with a wave per row and two vectors per lane: 1000 bf16 columns 5.1 -> 5.7 TB/s)
    return nvec <= 32 ? 8 : (nvec <= 64 ? 16 : (nvec <= 128 && row_bytes % 128 == 0 ? 32 : 0));
}

struct FwdArgs {
    void* y; float* inv_rms; const void* x; const void* w;
    long rows; int cols; float eps;
    int xcd_group;  // see xcd_remap(); 0 = workgroup ids used as they come
};
struct BwdArgs {
    void* dx; float* dw_part; int ld; const void* dy; const void* x; const void* w; const float* inv_rms;
    long rows; int cols; int num_partials;
    int xcd_group;
    bool prefetch;  // request row i+1 before reducing row i (costs a second copy of the row in VGPRs)
    unsigned long long* timeline;  // kFamilyRing with 512 threads per row only: per-workgroup time stamps, or null
    int partial_policy;  // kFamilyRing with 512 threads per row only: 0 default stores of the partial row,
                         // 1 non-temporal, 2 write-through to memory
};

// One set of launchers per element type (T = float, _Float16, __bf16), each defined in
// its own translation unit.  `generic` selects the element-wise kernels.
template <typename T> hipError_t launch_rmsnorm_fwd(const RowCfg& cfg, bool generic, const FwdArgs& a, hipStream_t s);
template <typename T> hipError_t launch_rmsnorm_bwd(const RowCfg& cfg, bool generic, const BwdArgs& a, hipStream_t s);

hipError_t launch_dw_reduce(float* dw_f32, void* dw_cast, int cast_dtype, const float* part, int P, int ld,
                            int cols, hipStream_t s);
hipError_t launch_fill_zero(float* p, long n, hipStream_t s);
hipError_t launch_copy(void* dst, const void* src, long bytes, hipStream_t s);
hipError_t launch_stream_probe(void* dst, const void* a, const void* b, long bytes, int xcd_group, hipStream_t s);
hipError_t launch_row_probe(void* dst, const void* a, const void* b, long rows, long row_bytes, long workgroups,
                            hipStream_t s);

// SwiGLU kernel families: aligned 16-byte vectors (needs H*sizeof(T) % 16 == 0 and 16-byte
// aligned bases), 16-byte vectors at any alignment with ragged half rows, or one element per
// thread.  rows*H per launch stays below 2^31 units (vectors or elements); larger inputs are
// split by rows, as are inputs above the "swiglu_max_units" option.
constexpr int kSwigluElementwise = 0, kSwigluAligned = 1, kSwigluRagged = 2;
void set_swiglu_max_units(long units);
hipError_t launch_swiglu_fwd(int dtype, int mode, int unroll, int xcd_group, void* h, const void* gu, long M, long H,
                             hipStream_t s);
hipError_t launch_swiglu_bwd(int dtype, int mode, int unroll, int xcd_group, void* dgu, const void* dh, const void* gu,
                             long M, long H, hipStream_t s);

}  // namespace mg
