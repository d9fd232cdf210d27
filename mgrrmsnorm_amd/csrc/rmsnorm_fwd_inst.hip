// RMSNorm forward launchers for one element type; compile with -DMG_DTYPE=0|1|2
// (fp32 | fp16 | bf16).
#include "mg_launch.hpp"
#include "rmsnorm_kernels.hpp"

#ifndef MG_DTYPE
#error "compile with -DMG_DTYPE=0 (fp32), 1 (fp16) or 2 (bf16)"
#endif

namespace mg {
namespace {

#if MG_DTYPE == 0
typedef float elem_t;
#elif MG_DTYPE == 1
typedef half_t elem_t;
#else
typedef bf16_t elem_t;
#endif

template <int VEC, int TPR, int ITEMS>
hipError_t run(const FwdArgs& a, hipStream_t s) {
    constexpr int BLOCK = TPR > 256 ? TPR : 256;
    constexpr int RPB = BLOCK / TPR;
    const long grid = (a.rows + RPB - 1) / RPB;
    return launch(rmsnorm_fwd_rows<elem_t, VEC, TPR, ITEMS>, dim3((unsigned)grid), dim3(BLOCK), 0, s,
            (elem_t*)a.y, a.inv_rms, (const elem_t*)a.x, (const elem_t*)a.w, a.rows, a.cols, a.eps,
        1.0f / (float)a.cols, a.xcd_group);
}

template <int VEC, int TPR>
hipError_t by_items(int items, const FwdArgs& a, hipStream_t s) {
    switch (items) {
        case 1: return run<VEC, TPR, 1>(a, s);
        case 2: return run<VEC, TPR, 2>(a, s);
        case 3: return run<VEC, TPR, 3>(a, s);
        case 4: return run<VEC, TPR, 4>(a, s);
        case 5: return run<VEC, TPR, 5>(a, s);
        case 6: return run<VEC, TPR, 6>(a, s);
        case 8: return run<VEC, TPR, 8>(a, s);
        default: return hipErrorInvalidValue;
    }
}

template <int TPR, int ITEMS>
hipError_t run_lines(const FwdArgs& a, hipStream_t s) {
    constexpr int BLOCK = TPR > 256 ? TPR : 256;
    constexpr int RPB = BLOCK / TPR;
    const long grid = (a.rows + RPB - 1) / RPB;
    return launch(rmsnorm_fwd_rows_lines<elem_t, kVec, TPR, ITEMS>, dim3((unsigned)grid), dim3(BLOCK), 0, s,
            (elem_t*)a.y, a.inv_rms, (const elem_t*)a.x, (const elem_t*)a.w, a.rows, a.cols, a.eps,
        1.0f / (float)a.cols, a.xcd_group);
}

template <int TPR>
hipError_t lines_by_items(int items, const FwdArgs& a, hipStream_t s) {
    switch (items) {
        case 1: return run_lines<TPR, 1>(a, s);
        case 2: return run_lines<TPR, 2>(a, s);
        case 3: return run_lines<TPR, 3>(a, s);
        case 4: return run_lines<TPR, 4>(a, s);
        case 5: return run_lines<TPR, 5>(a, s);
        case 6: return run_lines<TPR, 6>(a, s);
        case 8: return run_lines<TPR, 8>(a, s);
        default: return hipErrorInvalidValue;
    }
}

template <int TPR, int ITEMS, bool RAGGED>
hipError_t run_narrow(const FwdArgs& a, hipStream_t s) {
    constexpr int RPB = 256 / TPR;
    const long grid = (a.rows + RPB - 1) / RPB;
    return launch(rmsnorm_fwd_narrow<elem_t, TPR, ITEMS, RAGGED>, dim3((unsigned)grid), dim3(256), 0, s,
            (elem_t*)a.y, a.inv_rms, (const elem_t*)a.x, (const elem_t*)a.w, a.rows, a.cols, a.eps,
        1.0f / (float)a.cols, a.xcd_group);
}

template <int TPR, int G, bool RAGGED, int POL>
hipError_t run_groups(const FwdArgs& a, hipStream_t s) {
    constexpr int RPB = 4 * G * (kWave / TPR);
    const long grid = (a.rows + RPB - 1) / RPB;
    return launch(rmsnorm_fwd_groups<elem_t, TPR, G, RAGGED, POL>, dim3((unsigned)grid), dim3(256), 0, s,
            (elem_t*)a.y, a.inv_rms, (const elem_t*)a.x, (const elem_t*)a.w, a.rows, a.cols, a.eps,
        1.0f / (float)a.cols, a.xcd_group);
}

// ragged rows (pitch not a multiple of 16 bytes) take the default cache policy, as in the
// several-vectors-per-lane kernels; the others stream
template <int TPR, int G>
hipError_t groups_by_pitch(const FwdArgs& a, hipStream_t s) {
    const bool ragged = ((long)a.cols * (long)sizeof(elem_t)) % kVec != 0;
    return ragged ? run_groups<TPR, G, true, kKeep>(a, s) : run_groups<TPR, G, false, kStream>(a, s);
}

template <int TPR>
hipError_t groups_by_g(int g, const FwdArgs& a, hipStream_t s) {
    switch (g) {
        case 1:
            if constexpr (TPR >= 8) return groups_by_pitch<TPR, 1>(a, s);
            else return hipErrorInvalidValue;
        case 2: return groups_by_pitch<TPR, 2>(a, s);
        case 4: return groups_by_pitch<TPR, 4>(a, s);
        default: return hipErrorInvalidValue;
    }
}

template <int TPR>
hipError_t narrow_by_items(int items, const FwdArgs& a, hipStream_t s) {
    if (narrow_items((long)a.cols * (long)sizeof(elem_t), TPR) != items) return hipErrorInvalidValue;
    const bool ragged = ((long)a.cols * (long)sizeof(elem_t)) % kVec != 0;
    switch (items) {
        case 1: return ragged ? run_narrow<TPR, 1, true>(a, s) : run_narrow<TPR, 1, false>(a, s);
        case 2: return ragged ? run_narrow<TPR, 2, true>(a, s) : run_narrow<TPR, 2, false>(a, s);
        case 3: return ragged ? run_narrow<TPR, 3, true>(a, s) : run_narrow<TPR, 3, false>(a, s);
        case 4: return ragged ? run_narrow<TPR, 4, true>(a, s) : run_narrow<TPR, 4, false>(a, s);
        default: return hipErrorInvalidValue;
    }
}

template <int VEC>
hipError_t by_tpr(int tpr, int items, const FwdArgs& a, hipStream_t s) {
    switch (tpr) {
        case 8: return narrow_by_items<8>(items, a, s);
        case 16: return narrow_by_items<16>(items, a, s);
        case 32: return narrow_by_items<32>(items, a, s);
        case 64: return by_items<VEC, 64>(items, a, s);
        case 128: return by_items<VEC, 128>(items, a, s);
        case 256: return by_items<VEC, 256>(items, a, s);
        case 512: return by_items<VEC, 512>(items, a, s);
        case 1024: return by_items<VEC, 1024>(items, a, s);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

template <>
hipError_t launch_rmsnorm_fwd<elem_t>(const RowCfg& cfg, bool generic, const FwdArgs& a, hipStream_t s) {
    if (generic) {
        return launch(rmsnorm_fwd_generic<elem_t>, dim3((unsigned)a.rows), dim3(256), 0, s,
            (elem_t*)a.y, a.inv_rms, (const elem_t*)a.x, (const elem_t*)a.w, a.rows, a.cols, a.eps,
            1.0f / (float)a.cols);
    }
    if (cfg.family == kFamilyStreaming) {
        return launch(rmsnorm_fwd_wide<elem_t>, dim3((unsigned)a.rows), dim3(kWideBlock), 0, s,
            (elem_t*)a.y, a.inv_rms, (const elem_t*)a.x, (const elem_t*)a.w, a.rows, a.cols, a.eps,
            1.0f / (float)a.cols);
    }
    if (cfg.family == kFamilyGroups) {
        if (!groups_ok((long)a.cols * (long)sizeof(elem_t), cfg.tpr, cfg.items)) return hipErrorInvalidValue;
        switch (cfg.tpr) {
            case 1: return groups_by_g<1>(cfg.items, a, s);
            case 2: return groups_by_g<2>(cfg.items, a, s);
            case 4: return groups_by_g<4>(cfg.items, a, s);
            case 8: return groups_by_g<8>(cfg.items, a, s);
            case 16: return groups_by_g<16>(cfg.items, a, s);
            case 32: return groups_by_g<32>(cfg.items, a, s);
            default: return groups_by_g<64>(cfg.items, a, s);
        }
    }
    if (cfg.family == kFamilyLines) {
        // the kernel's own conditions, checked where it is launched: the pitch, enough slots, and an
        // output whose rows start at multiples of 8 bytes
        if (!fwd_lines_ok((long)a.cols * (long)sizeof(elem_t), cfg.tpr, cfg.items) ||
            reinterpret_cast<uintptr_t>(a.y) % 8 != 0)
            return hipErrorInvalidValue;
        switch (cfg.tpr) {
            case 128: return lines_by_items<128>(cfg.items, a, s);
            case 256: return lines_by_items<256>(cfg.items, a, s);
            case 512: return lines_by_items<512>(cfg.items, a, s);
            default: return lines_by_items<1024>(cfg.items, a, s);
        }
    }
    if (cfg.vec == kVec) return by_tpr<kVec>(cfg.tpr, cfg.items, a, s);
    return hipErrorInvalidValue;
}

}  // namespace mg
