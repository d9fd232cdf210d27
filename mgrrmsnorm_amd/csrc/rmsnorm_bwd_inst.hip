// RMSNorm backward (pass 1) launchers for one element type; compile with
// -DMG_DTYPE=0|1|2 (fp32 | fp16 | bf16).
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
hipError_t run(const BwdArgs& a, hipStream_t s) {
    if constexpr (bwd_cfg_ok((int)sizeof(elem_t), VEC, TPR, ITEMS)) {
        rmsnorm_bwd_rows<elem_t, VEC, TPR, ITEMS><<<dim3((unsigned)a.num_partials), dim3(1024), 0, s>>>(
            (elem_t*)a.dx, a.dw_part, a.ld, (const elem_t*)a.dy, (const elem_t*)a.x, (const elem_t*)a.w,
            a.inv_rms, a.rows, a.cols, 1.0f / (float)a.cols);
        return hipGetLastError();
    } else {
        return hipErrorInvalidValue;
    }
}

template <int VEC, int TPR>
hipError_t by_items(int items, const BwdArgs& a, hipStream_t s) {
    switch (items) {
        case 1: return run<VEC, TPR, 1>(a, s);
        case 2: return run<VEC, TPR, 2>(a, s);
        case 3: return run<VEC, TPR, 3>(a, s);
        case 4: return run<VEC, TPR, 4>(a, s);
        default: return hipErrorInvalidValue;
    }
}

template <int VEC>
hipError_t by_tpr(int tpr, int items, const BwdArgs& a, hipStream_t s) {
    switch (tpr) {
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
hipError_t launch_rmsnorm_bwd<elem_t>(const RowCfg& cfg, bool generic, const BwdArgs& a, hipStream_t s) {
    if (generic) {
        rmsnorm_bwd_dx_generic<elem_t><<<dim3((unsigned)a.rows), dim3(256), 0, s>>>(
            (elem_t*)a.dx, (const elem_t*)a.dy, (const elem_t*)a.x, (const elem_t*)a.w, a.inv_rms, a.rows,
            a.cols, 1.0f / (float)a.cols);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        rmsnorm_bwd_dw_generic<elem_t>
            <<<dim3((unsigned)((a.cols + 255) / 256), (unsigned)a.num_partials), dim3(256), 0, s>>>(
                a.dw_part, a.ld, (const elem_t*)a.dy, (const elem_t*)a.x, a.inv_rms, a.rows, a.cols);
        return hipGetLastError();
    }
    if (cfg.vec == 16) return by_tpr<16>(cfg.tpr, cfg.items, a, s);
    if (cfg.vec == 8) return by_tpr<8>(cfg.tpr, cfg.items, a, s);
    return hipErrorInvalidValue;
}

}  // namespace mg
