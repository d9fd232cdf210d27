// RMSNorm backward (pass 1) launchers for one element type; compile with
// -DMG_DTYPE=0|1|2 (fp32 | fp16 | bf16).
#include <atomic>

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

template <int TPR, int ITEMS, int BLOCK>
hipError_t run(const BwdArgs& a, hipStream_t s) {
    if constexpr (bwd_cfg_ok((int)sizeof(elem_t), TPR, ITEMS, BLOCK)) {
        auto kernel = a.prefetch ? rmsnorm_bwd_rows<elem_t, kVec, TPR, ITEMS, BLOCK, true>
                                 : rmsnorm_bwd_rows<elem_t, kVec, TPR, ITEMS, BLOCK, false>;
        return launch(kernel, dim3((unsigned)a.num_partials), dim3(BLOCK), 0, s,
            (elem_t*)a.dx, a.dw_part, a.ld, (const elem_t*)a.dy, (const elem_t*)a.x, (const elem_t*)a.w,
                a.inv_rms, a.rows, a.cols, 1.0f / (float)a.cols, a.xcd_group);
    } else {
        return hipErrorInvalidValue;
    }
}

// dW sums in LDS: more dynamic LDS than the 64 KiB a kernel gets without asking
template <int ITEMS>
hipError_t run_lds_sums(const BwdArgs& a, hipStream_t s) {
    if constexpr (sizeof(elem_t) == 2 || sizeof(elem_t) == 4) {
        constexpr int kLdsBytes = ITEMS * 1024 * (kVec / (int)sizeof(elem_t)) * 4;
        auto kernel = rmsnorm_bwd_rows_lds<elem_t, ITEMS>;
        // asked for once per device (the first call on a device should not sit inside a stream capture)
        static std::atomic<bool> allowed[64];
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return e;
        if (dev < 0 || dev >= 64 || !allowed[dev].load(std::memory_order_acquire)) {
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    kLdsBytes);
            if (e != hipSuccess) return e;
            if (dev >= 0 && dev < 64) allowed[dev].store(true, std::memory_order_release);
        }
        return launch(kernel, dim3((unsigned)a.num_partials), dim3(1024), kLdsBytes, s,
            (elem_t*)a.dx, a.dw_part, a.ld, (const elem_t*)a.dy, (const elem_t*)a.x, (const elem_t*)a.w, a.inv_rms,
            a.rows, a.cols, 1.0f / (float)a.cols, a.xcd_group);
    } else {
        return hipErrorInvalidValue;
    }
}

template <int TPR, int ITEMS, int DEPTH>
hipError_t run_ring(const BwdArgs& a, hipStream_t s) {
    constexpr int BLOCK = TPR > 512 ? TPR : 512;
    if (a.timeline != nullptr) {
        // the time-stamped build exists for the 512-thread layout only (the 4096-column shapes)
        if constexpr (TPR == 512 && ITEMS == 1)
            return launch(rmsnorm_bwd_rows_ring<elem_t, kVec, TPR, ITEMS, BLOCK, DEPTH, true>,
                          dim3((unsigned)a.num_partials), dim3(BLOCK), 0, s, (elem_t*)a.dx, a.dw_part, a.ld,
                          (const elem_t*)a.dy, (const elem_t*)a.x, (const elem_t*)a.w, a.inv_rms, a.rows, a.cols,
                          1.0f / (float)a.cols, a.timeline);
        else
            return hipErrorNotSupported;
    }
    if constexpr (TPR == 512 && ITEMS == 1) {   // the partial row's store policy, on request
        if (a.partial_policy == 1)
            return launch(rmsnorm_bwd_rows_ring<elem_t, kVec, TPR, ITEMS, BLOCK, DEPTH, false, kStream>,
                          dim3((unsigned)a.num_partials), dim3(BLOCK), 0, s, (elem_t*)a.dx, a.dw_part, a.ld,
                          (const elem_t*)a.dy, (const elem_t*)a.x, (const elem_t*)a.w, a.inv_rms, a.rows, a.cols,
                          1.0f / (float)a.cols, (unsigned long long*)nullptr);
        if (a.partial_policy == 2)
            return launch(rmsnorm_bwd_rows_ring<elem_t, kVec, TPR, ITEMS, BLOCK, DEPTH, false, 17>,
                          dim3((unsigned)a.num_partials), dim3(BLOCK), 0, s, (elem_t*)a.dx, a.dw_part, a.ld,
                          (const elem_t*)a.dy, (const elem_t*)a.x, (const elem_t*)a.w, a.inv_rms, a.rows, a.cols,
                          1.0f / (float)a.cols, (unsigned long long*)nullptr);
    }
    return launch(rmsnorm_bwd_rows_ring<elem_t, kVec, TPR, ITEMS, BLOCK, DEPTH>, dim3((unsigned)a.num_partials),
                  dim3(BLOCK), 0, s, (elem_t*)a.dx, a.dw_part, a.ld, (const elem_t*)a.dy, (const elem_t*)a.x,
                  (const elem_t*)a.w, a.inv_rms, a.rows, a.cols, 1.0f / (float)a.cols, (unsigned long long*)nullptr);
}

template <int TPR, int ITEMS>
hipError_t ring_by_depth(int depth, const BwdArgs& a, hipStream_t s) {
    return depth == 4 ? run_ring<TPR, ITEMS, 4>(a, s) : run_ring<TPR, ITEMS, 2>(a, s);
}

hipError_t ring_by_shape(const RowCfg& cfg, const BwdArgs& a, hipStream_t s) {
    if (!bwd_ring_ok((long)a.cols * (long)sizeof(elem_t), cfg.tpr, cfg.items, cfg.depth)) return hipErrorInvalidValue;
    if (cfg.items == 2) return cfg.depth == 2 ? run_ring<1024, 2, 2>(a, s) : hipErrorInvalidValue;   // four buffers would spill
    switch (cfg.tpr) {
        case 64: return ring_by_depth<64, 1>(cfg.depth, a, s);
        case 128: return ring_by_depth<128, 1>(cfg.depth, a, s);
        case 256: return ring_by_depth<256, 1>(cfg.depth, a, s);
        case 512: return ring_by_depth<512, 1>(cfg.depth, a, s);
        default: return ring_by_depth<1024, 1>(cfg.depth, a, s);
    }
}

template <int TPR, int BLOCK>
hipError_t by_items(int items, const BwdArgs& a, hipStream_t s) {
    switch (items) {
        case 1: return run<TPR, 1, BLOCK>(a, s);
        case 2: return run<TPR, 2, BLOCK>(a, s);
        case 3: return run<TPR, 3, BLOCK>(a, s);
        case 4: return run<TPR, 4, BLOCK>(a, s);
        case 6: return run<TPR, 6, BLOCK>(a, s);
        case 8: return run<TPR, 8, BLOCK>(a, s);
        default: return hipErrorInvalidValue;
    }
}

template <int TPR, int ITEMS, bool RAGGED>
hipError_t run_narrow(const BwdArgs& a, hipStream_t s) {
    return launch(rmsnorm_bwd_narrow<elem_t, TPR, ITEMS, RAGGED>, dim3((unsigned)a.num_partials), dim3(512), 0, s,
            (elem_t*)a.dx, a.dw_part, a.ld, (const elem_t*)a.dy, (const elem_t*)a.x, (const elem_t*)a.w, a.inv_rms,
        a.rows, a.cols, 1.0f / (float)a.cols);
}

template <int TPR, int G, bool RAGGED, int POL>
hipError_t run_groups(const BwdArgs& a, hipStream_t s) {
    return launch(rmsnorm_bwd_groups<elem_t, TPR, G, RAGGED, POL>, dim3((unsigned)a.num_partials), dim3(512), 0, s,
            (elem_t*)a.dx, a.dw_part, a.ld, (const elem_t*)a.dy, (const elem_t*)a.x, (const elem_t*)a.w, a.inv_rms,
        a.rows, a.cols, 1.0f / (float)a.cols);
}

// ragged rows (pitch not a multiple of 16 bytes) take the default cache policy, as in the
// several-vectors-per-lane kernels; the others stream
template <int TPR, int G>
hipError_t groups_by_pitch(const BwdArgs& a, hipStream_t s) {
    const bool ragged = ((long)a.cols * (long)sizeof(elem_t)) % kVec != 0;
    return ragged ? run_groups<TPR, G, true, kKeep>(a, s) : run_groups<TPR, G, false, kStream>(a, s);
}

template <int TPR>
hipError_t groups_by_g(int g, const BwdArgs& a, hipStream_t s) {
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
hipError_t narrow_by_items(int items, const BwdArgs& a, hipStream_t s) {
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

template <int BLOCK>
hipError_t by_tpr(int tpr, int items, const BwdArgs& a, hipStream_t s) {
    switch (tpr) {
        case 64: return by_items<64, BLOCK>(items, a, s);
        case 128: return by_items<128, BLOCK>(items, a, s);
        case 256: return by_items<256, BLOCK>(items, a, s);
        case 512: return by_items<512, BLOCK>(items, a, s);
        case 1024:
            if constexpr (BLOCK == 1024) return by_items<1024, BLOCK>(items, a, s);
            else return hipErrorInvalidValue;
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

template <>
hipError_t launch_rmsnorm_bwd<elem_t>(const RowCfg& cfg, bool generic, const BwdArgs& a, hipStream_t s) {
    if (a.timeline != nullptr && (generic || cfg.family != kFamilyRing)) return hipErrorNotSupported;
    if (generic) {
        hipError_t e = launch(rmsnorm_bwd_dx_generic<elem_t>, dim3((unsigned)a.rows), dim3(256), 0, s,
            (elem_t*)a.dx, (const elem_t*)a.dy, (const elem_t*)a.x, (const elem_t*)a.w, a.inv_rms, a.rows,
            a.cols, 1.0f / (float)a.cols);
        if (e != hipSuccess) return e;
        return launch(rmsnorm_bwd_dw_generic<elem_t>, dim3((unsigned)((a.cols + 255) / 256), (unsigned)a.num_partials), dim3(256), 0, s,
            a.dw_part, a.ld, (const elem_t*)a.dy, (const elem_t*)a.x, a.inv_rms, a.rows, a.cols);
    }
    if (cfg.family == kFamilyStreaming) {
        hipError_t e = launch(rmsnorm_bwd_dx_wide<elem_t>, dim3((unsigned)a.rows), dim3(kWideBlock), 0, s,
            (elem_t*)a.dx, (const elem_t*)a.dy, (const elem_t*)a.x, (const elem_t*)a.w, a.inv_rms, a.rows, a.cols,
            1.0f / (float)a.cols);
        if (e != hipSuccess) return e;
        const long nvec = ((long)a.cols * (long)sizeof(elem_t) + kVec - 1) / kVec;
        return launch(rmsnorm_bwd_dw_wide<elem_t>, dim3((unsigned)((nvec + 255) / 256), (unsigned)a.num_partials), dim3(256), 0, s,
            a.dw_part, a.ld, (const elem_t*)a.dy, (const elem_t*)a.x, a.inv_rms, a.rows, a.cols);
    }
    if (cfg.vec != kVec) return hipErrorInvalidValue;
    if (cfg.family == kFamilyLdsSums) {
        const long nvec = ((long)a.cols * (long)sizeof(elem_t) + kVec - 1) / kVec;
        if (!bwd_lds_ok((int)sizeof(elem_t), nvec, cfg.items)) return hipErrorInvalidValue;
        return cfg.items == 2 ? run_lds_sums<2>(a, s) : (cfg.items == 3 ? run_lds_sums<3>(a, s) : run_lds_sums<4>(a, s));
    }
    if (cfg.family == kFamilyRing) return ring_by_shape(cfg, a, s);
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
    if (cfg.tpr == 8 && cfg.block == 512) return narrow_by_items<8>(cfg.items, a, s);
    if (cfg.tpr == 16 && cfg.block == 512) return narrow_by_items<16>(cfg.items, a, s);
    if (cfg.tpr == 32 && cfg.block == 512) return narrow_by_items<32>(cfg.items, a, s);
    if (cfg.block == 1024) return by_tpr<1024>(cfg.tpr, cfg.items, a, s);
    if (cfg.block == 512) return by_tpr<512>(cfg.tpr, cfg.items, a, s);
    if (cfg.block == 256 && cfg.tpr == 256) return by_items<256, 256>(cfg.items, a, s);
    return hipErrorInvalidValue;
}

}  // namespace mg
