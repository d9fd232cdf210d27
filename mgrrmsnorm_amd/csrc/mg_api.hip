// C ABI of libmegagemm_hip.so: argument validation, choice of launch shape, launch.
// Validation happens before any HIP call so that argument errors are reported on hosts
// without a GPU.
#include "megagemm_hip.h"
#include "megagemm_hip_tuning.h"
#include "mg_launch.hpp"
#include "mg_device.hpp"
#include "rmsnorm_kernels.hpp"

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>

namespace mg {
namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int fail_hip(const char* what, hipError_t e) {
    return fail(MG_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

// ---- process-wide tuning overrides (0 / -1 = automatic) ----
std::atomic<int> opt_fwd_tpr{0}, opt_fwd_items{0}, opt_bwd_tpr{0}, opt_bwd_wg_per_cu{0},
    opt_swiglu_unroll{0}, opt_force_generic{0}, opt_bwd_block{0}, opt_xcd_group{-1}, opt_bwd_prefetch{-1}, opt_groups{-1}, opt_bwd_lds{-1}, opt_bwd_ring{-1}, opt_bwd_partials{0}, opt_bwd_partial_policy{0},
    opt_fwd_lines{0};

// Consecutive logical workgroups one die handles at a time in the one-shot streaming
// kernels (see xcd_remap); the "xcd_group" option overrides it (0 switches the remap off).
constexpr int kXcdGroupStreaming = 32;
int xcd_group_or(int dflt) {
    const int v = opt_xcd_group.load();
    return v < 0 ? dflt : v;
}

int esize_of(int dtype) {
    switch (dtype) {
        case MG_F32: return 4;
        case MG_F16: return 2;
        case MG_BF16: return 2;
        default: return 0;
    }
}

const char* dtype_name(int dtype) {
    switch (dtype) {
        case MG_F32: return "fp32";
        case MG_F16: return "fp16";
        case MG_BF16: return "bf16";
        default: return "?";
    }
}

bool aligned(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// Compute units of the current device (cached per device ordinal).
int cu_count(int* out) {
    static std::atomic<int> cache[64];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail_hip("hipGetDevice", e);
    if (dev >= 0 && dev < 64) {
        int c = cache[dev].load(std::memory_order_relaxed);
        if (c > 0) { *out = c; return MG_OK; }
    }
    int n = 0;
    e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return fail_hip("hipDeviceGetAttribute(MultiprocessorCount)", e);
    if (n <= 0) n = 256;
    if (dev >= 0 && dev < 64) cache[dev].store(n, std::memory_order_relaxed);
    *out = n;
    return MG_OK;
}

int ceil_div(long a, long b) { return (int)((a + b - 1) / b); }

// The register-resident kernels take any row pitch and any element-aligned base: 16-byte
// buffer accesses work at every byte alignment (measured at 2-, 4- and 8-byte offsets), the
// range check is per dword, and the half dword that ends a row of an odd number of 2-byte
// elements is handled by the lane that owns it.

int round_items(int items) { return (items == 5 || items == 7) ? items + 1 : items; }

// Forward: the fewest threads per row that keep a thread at or below two vectors (one
// vector per thread leaves too few bytes in flight); when the second vector would be mostly
// empty, half the threads with three vectors each.
bool choose_fwd(long row_bytes, RowCfg* cfg) {
    const long nvec = (row_bytes + kVec - 1) / kVec;
    const int tpr = opt_fwd_tpr.load(), items = opt_fwd_items.load();
    {   // narrow rows, one vector per lane ("narrow_groups": 0 = never, 1 / 2 / 4 = that many groups where it fits)
        const int want = opt_groups.load();
        const int g = want < 0 ? (tpr == 0 && items == 0 ? groups_default(row_bytes, false) : 0) : want;
        if (g > 0 && groups_ok(row_bytes, groups_tpr(row_bytes), g)) {
            *cfg = {kVec, groups_tpr(row_bytes), g, 0, kFamilyGroups};
            return true;
        }
    }
    {   // rows narrower than a wave: several rows per wave (a requested 8, 16 or 32 wins when it fits)
        const int nt = narrow_items(row_bytes, tpr) ? tpr : (tpr == 0 ? narrow_default_tpr(row_bytes, false) : 0);
        if (nt) { *cfg = {kVec, nt, narrow_items(row_bytes, nt), 0}; return true; }
    }
    if (tpr_ok(tpr)) {
        const int need = ceil_div(nvec, tpr) == 7 ? 8 : ceil_div(nvec, tpr);
        if (need <= kFwdMaxItems && fwd_items_ok(need)) { *cfg = {kVec, tpr, need, 0}; return true; }
    }
    const int target = (items > 0 && items <= kFwdMaxItems) ? items : 2;
    // 1025-1536 vectors: 512 threads with three vectors each rather than 1024 with two
    // (10240 bf16 columns: 6.04 against 5.75 TB/s, 12288: 6.03 against 5.87)
    if (items == 0 && nvec > 1024 && nvec <= 1536) { *cfg = {kVec, 512, 3, 0}; return true; }
    for (int t = 64; t <= 1024; t *= 2) {
        int need = ceil_div(nvec, t);
        if (need == 7) need = 8;
        if (need <= target || (t == 1024 && need <= kFwdMaxItems)) {
            if (need == 2 && t >= 128 && nvec * 10 < (long)t * 2 * 6) { t /= 2; need = ceil_div(nvec, t); }
            *cfg = {kVec, t, need, 0};
            return true;
        }
    }
    return false;
}

// On request only ("fwd_lines" = 1): forward rows whose pitch is a multiple of 8 but not of 128
// bytes, with more than 256 vectors and an output whose rows start at multiples of 8 bytes, in
// the register-resident layout with the vectors on the 128-byte lines of y, so that a wave's
// store instruction writes whole lines (a "fwd_tpr" / "fwd_items" override switches it off).
// It is not chosen automatically because it does not win everywhere (bf16, us per launch,
// this layout against vectors counted from the row's first byte): 65536 x 2052 88.8 / 95.4,
// 65536 x 2056 88.5 / 93.3, 32768 x 8200 175.9 / 185.2, 65536 x 5000 219.7 / 225.1, 16384 x 20484
// 228.0 / 232.1, but 65536 x 4100 185.9 / 183.6, 4096 x 4100 14.1 / 13.6, 16384 x 12292 159.1 / 144.5,
// 16384 x 16380 192.9 / 185.7.
bool choose_fwd_lines(long row_bytes, bool y_rows_8_aligned, RowCfg* cfg) {
    if (opt_fwd_lines.load() != 1 || opt_fwd_tpr.load() != 0 || opt_fwd_items.load() != 0 || !y_rows_8_aligned)
        return false;
    const LinesShape sh = fwd_lines_shape(row_bytes);
    if (sh.tpr == 0 || !fwd_lines_ok(row_bytes, sh.tpr, sh.items)) return false;
    *cfg = {kVec, sh.tpr, sh.items, 0, kFamilyLines};
    return true;
}

// Backward: 512-thread workgroups (8 waves, 256 VGPRs per thread).  From sweeps over
// 576...16384 columns on MI355X: the fewest threads per row that keep a thread at or below
// two vectors -- three vectors at half the threads lose 4-23 % (1032 columns: 5.0 against
// 6.1 TB/s, 4104: 5.4 against 6.1), and with the copied prefetch one vector at twice the
// threads loses at the 4096 x 4096 shape (20.5 against 18.9 us; with the ring of register
// buffers, chosen first below where it applies, it wins).  Rows of more than 1024 vectors take
// what fits: 512 x 3, 1024 x 2, 512 x 4...8.
bool choose_bwd(long row_bytes, int esize, RowCfg* cfg) {
    const long nvec = (row_bytes + kVec - 1) / kVec;
    const int tpr = opt_bwd_tpr.load(), block = opt_bwd_block.load();
    {   // narrow rows, one vector per lane
        const int want = opt_groups.load();
        const int g = want < 0 ? (tpr == 0 && block == 0 ? groups_default(row_bytes, true) : 0) : want;
        if (g > 0 && groups_ok(row_bytes, groups_tpr(row_bytes), g)) {
            *cfg = {kVec, groups_tpr(row_bytes), g, 512, kFamilyGroups};
            return true;
        }
    }
    {   // rows narrower than a wave: several rows per wave, always 512-thread workgroups
        const int nt = narrow_items(row_bytes, tpr) ? tpr : (tpr == 0 ? narrow_default_tpr(row_bytes, true) : 0);
        if (nt) { *cfg = {kVec, nt, narrow_items(row_bytes, nt), 512}; return true; }
    }
    // Rows whose pitch is a multiple of 16 bytes and that fill at least three quarters of the lanes
    // of 64 ... 1024 threads at one vector each: one vector per thread and a ring of register
    // buffers ("bwd_ring" = 0: never; 2 or 4: that many buffers).  Against two vectors at half the
    // threads with the copied prefetch (bf16, 65536 rows): 768 columns 49.4 against 50.4 us, 2048
    // 124.3 against 129.0, 4096 250.9 against 256, 8192 at 16384 rows 126.4 against 130.0, 4096 x 4096
    // 18.4 against 18.85.  Rows of 1025-1536 vectors (fp32: up to 2048) take two vectors on 1024
    // threads the same way (10240 bf16 columns 161.8 against 166.2 us, 12288 195.0 against 206.0).
    if (tpr == 0 && block == 0 && opt_bwd_ring.load() != 0 && row_bytes % kVec == 0 && nvec >= 57) {
        if (nvec <= 1024) {
            int t = 64;
            while (t < nvec) t *= 2;
            if (nvec * 4 >= 3L * t) { *cfg = {kVec, t, 1, t > 512 ? 1024 : 512, kFamilyRing, 0}; return true; }
        } else if (nvec * 5 >= 3L * 2048 && nvec <= ((esize == 4 || opt_bwd_ring.load() == 2) ? 2048 : 1536)) {
            *cfg = {kVec, 1024, 2, 1024, kFamilyRing, 0};
            return true;
        }
    }
    if (block == 256) {   // one 256-thread row slot per workgroup, on request only
        const int need = ceil_div(nvec, 256);
        if (bwd_cfg_ok(esize, 256, need, 256)) { *cfg = {kVec, 256, need, 256}; return true; }
    }
    if (tpr_ok(tpr)) {
        const int need = round_items(ceil_div(nvec, tpr));
        for (int b : {block, 512, 1024})
            if (bwd_cfg_ok(esize, tpr, need, b)) { *cfg = {kVec, tpr, need, b}; return true; }
    }
    // Rows of 2049-4096 vectors, and 2-byte rows from 1537 vectors on: 1024 threads with the dW
    // sums in LDS ("bwd_lds" = 0: in registers; 1 = from 1025 vectors on).  Beyond 2048 vectors
    // the register kernel needs 5-8 vectors per thread at 512 threads; with 8 sums per vector
    // (2-byte types) it spills (20480 bf16 columns: 4.8 -> 5.9 TB/s, 32768: 1.2 -> 5.8), with 4
    // (fp32) it merely runs 3-6 % slower (16384 columns: 5.96 -> 6.18 TB/s, 10240: 5.79 -> 6.16).
    // At 1537-2048 vectors of a 2-byte type two such workgroups share a compute unit and gain
    // 1-5 % (16384 x 16384: 5.77 -> 5.98 TB/s); below that, and for fp32 up to 2048 vectors,
    // the register kernel is as fast or faster (10240 bf16 columns: 6.0 against 5.8).
    if (tpr == 0 && block == 0 && opt_bwd_lds.load() != 0) {
        const int need = ceil_div(nvec, 1024);
        if (bwd_lds_ok(esize, nvec, need) && (nvec > 2048 || (nvec > 1536 && esize == 2) || opt_bwd_lds.load() == 1)) {
            *cfg = {kVec, 1024, need, 1024, kFamilyLdsSums};
            return true;
        }
    }
    // 88-128 vectors at a pitch that is a multiple of 16 but not of 128 bytes: two waves per row with one
    // vector per lane, so that every instruction covers contiguous memory, rather than one
    // wave with two (1000 bf16 columns: 6.0 against 5.4 TB/s; 904: 5.9 against 5.3; below 88
    // vectors too many lanes idle: 600 columns 4.8 against 5.5)
    if (tpr == 0 && block == 0 && row_bytes % 128 != 0 && row_bytes % kVec == 0 && nvec >= 88 && nvec <= 128 &&
        bwd_cfg_ok(esize, 128, 1, 512)) {
        *cfg = {kVec, 128, 1, 512};
        return true;
    }
    // rows of 1537-2048 vectors: 1024 threads with 2 vectors each rather than 512 with 4
    // (16384 bf16 columns: 5.85 against 5.67 TB/s)
    if (block != 512 && nvec > 1536 && nvec <= 2048 && bwd_cfg_ok(esize, 1024, 2, 1024)) {
        *cfg = {kVec, 1024, 2, 1024};
        return true;
    }
    for (int b : {block == 1024 ? 1024 : 512, 512}) {
        for (int t = 64; t <= b; t *= 2) {
            const int need = ceil_div(nvec, t);
            if (need <= 2 && bwd_cfg_ok(esize, t, need, b)) { *cfg = {kVec, t, need, b}; return true; }
        }
        const int need = round_items(ceil_div(nvec, b));   // wider than two vectors per thread of a workgroup
        if (bwd_cfg_ok(esize, b, need, b)) { *cfg = {kVec, b, need, b}; return true; }
    }
    return false;
}

// Rows that no register-resident shape holds: 1024 threads stream the row twice
// (vectors_per_thread = 0 in the launch report: it is not fixed).
bool choose_streaming(long row_bytes, RowCfg* cfg) {
    (void)row_bytes;
    *cfg = {kVec, 1024, 0, 1024, kFamilyStreaming};
    return true;
}

// Requesting row i+1 before reducing row i doubles the bytes a workgroup keeps in flight; it
// pays up to about 80 KiB (x and dy, current and next row, all row slots) and costs
// throughput beyond (12288 bf16 columns: 5.75 TB/s with, 6.09 without).
bool bwd_prefetch_default(const RowCfg& cfg, long row_bytes) {
    if (narrow_tpr(cfg.tpr) || cfg.tpr <= 0 || cfg.family != kFamilyResident) return true;
    return (long)(cfg.block / cfg.tpr) * row_bytes * 4 <= 80 * 1024;
}

int check_rmsnorm_dims(const char* fn, int64_t rows, int64_t cols, int dtype) {
    const int es = esize_of(dtype);
    if (es == 0) return fail(MG_ERR_INVALID_ARG, "%s: unknown dtype %d (use 0=fp32, 1=fp16, 2=bf16)", fn, dtype);
    if (rows < 0) return fail(MG_ERR_INVALID_ARG, "%s: rows must be >= 0 (got %lld)", fn, (long long)rows);
    if (cols < 1) return fail(MG_ERR_INVALID_ARG, "%s: cols must be >= 1 (got %lld)", fn, (long long)cols);
    if (cols * es >= (1LL << 31))
        return fail(MG_ERR_UNSUPPORTED, "%s: cols too large (%lld %s elements; a row must stay below 2 GiB)", fn,
                    (long long)cols, dtype_name(dtype));
    if (rows >= (1LL << 31))
        return fail(MG_ERR_UNSUPPORTED, "%s: rows too large (%lld; max 2^31-1)", fn, (long long)rows);
    return MG_OK;
}

template <typename F32, typename F16, typename BF16>
hipError_t by_dtype(int dtype, F32 f32, F16 f16, BF16 bf16) {
    switch (dtype) {
        case MG_F32: return f32();
        case MG_F16: return f16();
        default: return bf16();
    }
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_abi_version(void) { return MG_ABI_VERSION; }

const char* mg_last_error(void) { return g_err; }

// Counts the successful mg_set_option calls of this process: whoever remembers an answer that
// depends on the options (a workspace shape) compares it before trusting the memory.
static std::atomic<int> g_option_generation{0};

int mg_option_generation(void) { return g_option_generation.load(); }

int mg_set_option(const char* key, int value) {
    if (key == nullptr) return fail(MG_ERR_INVALID_ARG, "mg_set_option: key is NULL");
    struct { const char* k; std::atomic<int>* v; } table[] = {
        {"narrow_groups", &opt_groups}, {"bwd_lds", &opt_bwd_lds}, {"fwd_tpr", &opt_fwd_tpr},       {"fwd_items", &opt_fwd_items},
        {"bwd_tpr", &opt_bwd_tpr},
        {"bwd_wg_per_cu", &opt_bwd_wg_per_cu}, {"swiglu_unroll", &opt_swiglu_unroll},
        {"force_generic", &opt_force_generic}, {"bwd_block", &opt_bwd_block}, {"xcd_group", &opt_xcd_group},
        {"bwd_prefetch", &opt_bwd_prefetch}, {"bwd_ring", &opt_bwd_ring}, {"bwd_partials", &opt_bwd_partials}, {"bwd_partial_policy", &opt_bwd_partial_policy},
        {"fwd_lines", &opt_fwd_lines},
    };
    if (strcmp(key, "swiglu_max_units") == 0) {
        set_swiglu_max_units(value);
        g_option_generation.fetch_add(1);
        return MG_OK;
    }
    for (auto& t : table)
        if (strcmp(t.k, key) == 0) {
            t.v->store(value);
            g_option_generation.fetch_add(1);
            return MG_OK;
        }
    return fail(MG_ERR_INVALID_ARG, "mg_set_option: unknown key '%s'", key);
}

int mg_rmsnorm_fwd(void* y, float* inv_rms, const void* x, const void* w, int64_t rows, int64_t cols, float eps,
                   int dtype, void* stream) {
    int rc = check_rmsnorm_dims("mg_rmsnorm_fwd", rows, cols, dtype);
    if (rc != MG_OK) return rc;
    if (rows == 0) return MG_OK;
    if (y == nullptr || x == nullptr || w == nullptr)
        return fail(MG_ERR_INVALID_ARG, "mg_rmsnorm_fwd: y, x and w must not be NULL");
    const int es = esize_of(dtype);
    if (!aligned(y, es) || !aligned(x, es) || !aligned(w, es) || !aligned(inv_rms, 4))
        return fail(MG_ERR_INVALID_ARG, "mg_rmsnorm_fwd: a pointer is not aligned to its element size");

    const long row_bytes = cols * es;
    RowCfg cfg = {0, 0, 0, 0};
    bool generic = opt_force_generic.load() != 0;
    if (!generic && !choose_fwd_lines(row_bytes, aligned(y, 8), &cfg))
        generic = !choose_fwd(row_bytes, &cfg) && !choose_streaming(row_bytes, &cfg);
    const FwdArgs a = {y, inv_rms, x, w, (long)rows, (int)cols, eps, xcd_group_or(kXcdGroupStreaming)};
    hipStream_t s = (hipStream_t)stream;
    hipError_t e = by_dtype(
        dtype, [&] { return launch_rmsnorm_fwd<float>(cfg, generic, a, s); },
        [&] { return launch_rmsnorm_fwd<half_t>(cfg, generic, a, s); },
        [&] { return launch_rmsnorm_fwd<bf16_t>(cfg, generic, a, s); });
    if (e != hipSuccess) return fail_hip("mg_rmsnorm_fwd: launch", e);
    return MG_OK;
}

int mg_rmsnorm_launch_info(int backward, int64_t cols, int dtype, int* generic, int* threads_per_row,
                            int* vectors_per_thread, int* workgroup_threads) {
    int rc = check_rmsnorm_dims("mg_rmsnorm_launch_info", 1, cols, dtype);
    if (rc != MG_OK) return rc;
    if (generic == nullptr || threads_per_row == nullptr || vectors_per_thread == nullptr ||
        workgroup_threads == nullptr)
        return fail(MG_ERR_INVALID_ARG, "mg_rmsnorm_launch_info: output pointers must not be NULL");
    const int es = esize_of(dtype);
    const long row_bytes = cols * es;
    RowCfg cfg = {0, 0, 0, 0};
    bool gen = opt_force_generic.load() != 0;
    // forward: as for an output at a multiple of 8 bytes, which every allocation is
    if (!gen && !(backward == 0 && choose_fwd_lines(row_bytes, true, &cfg)))
        gen = !(backward ? choose_bwd(row_bytes, es, &cfg) : choose_fwd(row_bytes, &cfg)) &&
              !choose_streaming(row_bytes, &cfg);
    *generic = gen ? 1 : 0;
    *threads_per_row = gen ? 256 : cfg.tpr;
    *vectors_per_thread = gen ? 0 : (cfg.family == kFamilyGroups ? -cfg.items : cfg.items);
    *workgroup_threads = gen ? 256 : (backward || cfg.family == kFamilyStreaming ? cfg.block : (cfg.tpr > 256 ? cfg.tpr : 256));
    return MG_OK;
}

int mg_rmsnorm_bwd_workspace(int64_t rows, int64_t cols, int dtype, int64_t* num_partials, int64_t* ld) {
    int rc = check_rmsnorm_dims("mg_rmsnorm_bwd_workspace", rows, cols, dtype);
    if (rc != MG_OK) return rc;
    if (num_partials == nullptr || ld == nullptr)
        return fail(MG_ERR_INVALID_ARG, "mg_rmsnorm_bwd_workspace: output pointers must not be NULL");
    *ld = (cols + 63) / 64 * 64;
    if (rows == 0) { *num_partials = 1; return MG_OK; }
    int cus = 0;
    rc = cu_count(&cus);
    if (rc != MG_OK) return rc;
    // one persistent workgroup per compute unit; four when a thread holds 4 or more vectors:
    // such kernels keep no prefetched copy of the next row (registers) and rely on the other
    // workgroups of the compute unit to cover the wait for it;
    // fewer when there are not enough rows to give every row slot at least one row
    const int es = esize_of(dtype);
    RowCfg cfg = {0, 0, 0, 0};
    int rg = 1, dflt_per_cu = 1;
    if (opt_force_generic.load() == 0 && choose_bwd(cols * es, es, &cfg)) {
        rg = cfg.block / cfg.tpr;
        dflt_per_cu = cfg.items >= 4 ? 4 : 1;
        if (cfg.block == 1024) dflt_per_cu = 2;   // both fit a compute unit; 5.9 against 5.5-5.8 TB/s with one
        if (cfg.block == 256) dflt_per_cu = 2;    // as many row slots as the 512-thread workgroups give
        // one vector per lane leaves half the bytes in flight: a second workgroup makes up for it
        if (narrow_tpr(cfg.tpr)) dflt_per_cu = cfg.items == 1 ? 2 : 1;
        if (cfg.family == kFamilyGroups) { rg = (cfg.block / cfg.tpr) * cfg.items; dflt_per_cu = 1; }
        if (cfg.family == kFamilyLdsSums) dflt_per_cu = (es == 2 && cfg.items == 2) ? 2 : 1;   // 32-128 KiB of LDS each
        if (cfg.family == kFamilyRing) dflt_per_cu = 1;
    }
    int per_cu = opt_bwd_wg_per_cu.load();
    if (per_cu < 1 || per_cu > 8) per_cu = dflt_per_cu;
    int64_t p = (int64_t)cus * per_cu;
    if (opt_bwd_partials.load() > 0) p = opt_bwd_partials.load();   // "bwd_partials": that many workgroups
    const int64_t by_rows = (rows + rg - 1) / rg;
    if (p > by_rows) p = by_rows;
    if (p < 1) p = 1;
    if (p > 65535) p = 65535;
    *num_partials = p;
    return MG_OK;
}

// mg_rmsnorm_bwd, and the same launch with per-workgroup time stamps for mg_rmsnorm_bwd_timeline
static int rmsnorm_bwd_impl(void* dx, float* dw_partial, const void* dy, const void* x, const void* w,
                            const float* inv_rms, int64_t rows, int64_t cols, int dtype, int64_t num_partials,
                            int64_t ld, unsigned long long* timeline, void* stream) {
    int rc = check_rmsnorm_dims("mg_rmsnorm_bwd", rows, cols, dtype);
    if (rc != MG_OK) return rc;
    if (num_partials < 1 || num_partials > 65535)
        return fail(MG_ERR_INVALID_ARG, "mg_rmsnorm_bwd: num_partials must be in [1, 65535] (got %lld)",
                    (long long)num_partials);
    if (ld < cols || ld % 64 != 0 || ld >= (1LL << 31))
        return fail(MG_ERR_INVALID_ARG, "mg_rmsnorm_bwd: ld must be a multiple of 64 and >= cols (got %lld)",
                    (long long)ld);
    if (dw_partial == nullptr || !aligned(dw_partial, 16))
        return fail(MG_ERR_INVALID_ARG, "mg_rmsnorm_bwd: dw_partial must be a 16-byte aligned device pointer");
    hipStream_t s = (hipStream_t)stream;
    if (rows == 0) {
        hipError_t e = launch_fill_zero(dw_partial, (long)(num_partials * ld), s);
        if (e != hipSuccess) return fail_hip("mg_rmsnorm_bwd: zero fill", e);
        return MG_OK;
    }
    if (dx == nullptr || dy == nullptr || x == nullptr || w == nullptr || inv_rms == nullptr)
        return fail(MG_ERR_INVALID_ARG, "mg_rmsnorm_bwd: dx, dy, x, w and inv_rms must not be NULL");
    const int es = esize_of(dtype);
    if (!aligned(dx, es) || !aligned(dy, es) || !aligned(x, es) || !aligned(w, es) || !aligned(inv_rms, 4))
        return fail(MG_ERR_INVALID_ARG, "mg_rmsnorm_bwd: a pointer is not aligned to its element size");

    const long row_bytes = cols * es;
    RowCfg cfg = {0, 0, 0, 0};
    bool generic = opt_force_generic.load() != 0;
    if (!generic) generic = !choose_bwd(row_bytes, es, &cfg) && !choose_streaming(row_bytes, &cfg);
    if (!generic && cfg.family == kFamilyRing) {
        // Two buffers (one row requested ahead) for rows that fill their lanes, four (three rows
        // ahead) for rows that leave up to a quarter of the lanes idle (bf16, 65536 rows, two / four
        // buffers / the copying loop: 2048 columns 125.1 / 128.8 / 127.3 us, 4096 columns 258.4 / 267.6 /
        // 255.9, 768 columns 56.2 / 48.4 / 49.7, 3072 columns 204.5 / 192.2 / 196.2), and four as well
        // while a slot has few rows, where filling the memory pipeline at the start counts: up to 32
        // rows per slot (1024 columns x 32768 rows: 34.4 / 33.1 / 34.0 us), up to 128 with one 512-thread
        // slot per workgroup (4096 x 4096: 19.0 / 18.45 / 18.8; 16384 x 4096: 66.2 / 63.4 / 64.2; 32768 x
        // 4096: 129.6 / 128.9 / 127.8; 65536 x 4096 see above).  Rows on 1024 threads keep two: three rows of
        // 16 KiB requested ahead for x and for dy are more than a compute unit keeps in flight to any
        // gain (4096 x 8192: 34.5 / 35.1 / 37.2; 16384 x 8192: 125.5 / 126.6 / 129.4).  Two vectors per
        // thread: always two buffers (registers).
        const int forced = opt_bwd_ring.load();
        const long nvec = (row_bytes + kVec - 1) / kVec;
        const long slots = num_partials * (cfg.block / cfg.tpr);
        const long rows_per_slot = (rows + slots - 1) / slots;
        const bool full = nvec * 8 > 7L * cfg.tpr;
        if (cfg.items != 1) cfg.depth = 2;
        else if (forced == 2 || forced == 4) cfg.depth = forced;
        else if (!full) cfg.depth = 4;
        else if (cfg.tpr >= 1024) cfg.depth = 2;
        else cfg.depth = rows_per_slot <= (cfg.tpr == 512 ? 128 : 32) ? 4 : 2;
    }
    const int prefetch = opt_bwd_prefetch.load();   // every option is read once per call
    // the persistent grid already walks the rows in order; regrouping its workgroups by die
    // measured within +-2 % either way, so it stays off unless asked for
    const BwdArgs a = {dx, dw_partial, (int)ld, dy, x, w, inv_rms, (long)rows, (int)cols, (int)num_partials,
                       xcd_group_or(0), prefetch < 0 ? bwd_prefetch_default(cfg, row_bytes) : prefetch != 0, timeline,
                       opt_bwd_partial_policy.load()};
    hipError_t e = by_dtype(
        dtype, [&] { return launch_rmsnorm_bwd<float>(cfg, generic, a, s); },
        [&] { return launch_rmsnorm_bwd<half_t>(cfg, generic, a, s); },
        [&] { return launch_rmsnorm_bwd<bf16_t>(cfg, generic, a, s); });
    if (e == hipErrorNotSupported && timeline != nullptr)
        return fail(MG_ERR_UNSUPPORTED, "mg_rmsnorm_bwd_timeline: only rows that take the register-ring kernel on 512 "
                                        "threads (385-512 16-byte vectors at a 16-byte pitch, e.g. 4096 bf16 columns) "
                                        "have a time-stamped build");
    if (e != hipSuccess) return fail_hip("mg_rmsnorm_bwd: launch", e);
    return MG_OK;
}

int mg_rmsnorm_bwd(void* dx, float* dw_partial, const void* dy, const void* x, const void* w, const float* inv_rms,
                   int64_t rows, int64_t cols, int dtype, int64_t num_partials, int64_t ld, void* stream) {
    return rmsnorm_bwd_impl(dx, dw_partial, dy, x, w, inv_rms, rows, cols, dtype, num_partials, ld, nullptr, stream);
}

int mg_rmsnorm_bwd_timeline(void* dx, float* dw_partial, const void* dy, const void* x, const void* w,
                            const float* inv_rms, int64_t rows, int64_t cols, int dtype, int64_t num_partials,
                            int64_t ld, uint64_t* records, void* stream) {
    if (records == nullptr || !aligned(records, 8))
        return fail(MG_ERR_INVALID_ARG, "mg_rmsnorm_bwd_timeline: records must be an 8-byte aligned device pointer");
    if (rows < 1) return fail(MG_ERR_INVALID_ARG, "mg_rmsnorm_bwd_timeline: rows must be >= 1");
    static_assert(MG_TIMELINE_WORDS == kTimelineWords && MG_TIMELINE_ITERATIONS == kTimelineIters, "header and kernel agree");
    return rmsnorm_bwd_impl(dx, dw_partial, dy, x, w, inv_rms, rows, cols, dtype, num_partials, ld,
                            reinterpret_cast<unsigned long long*>(records), stream);
}

int mg_rmsnorm_dw_reduce(float* dw_f32, void* dw_cast, int cast_dtype, const float* dw_partial,
                         int64_t num_partials, int64_t ld, int64_t cols, void* stream) {
    if (cols < 1 || cols >= (1LL << 31))
        return fail(MG_ERR_INVALID_ARG, "mg_rmsnorm_dw_reduce: cols must be in [1, 2^31) (got %lld)", (long long)cols);
    if (num_partials < 1 || num_partials > 65535)
        return fail(MG_ERR_INVALID_ARG, "mg_rmsnorm_dw_reduce: num_partials must be in [1, 65535] (got %lld)",
                    (long long)num_partials);
    if (ld < cols || ld % 64 != 0 || ld >= (1LL << 31))
        return fail(MG_ERR_INVALID_ARG, "mg_rmsnorm_dw_reduce: ld must be a multiple of 64 and >= cols (got %lld)",
                    (long long)ld);
    if (dw_f32 == nullptr && dw_cast == nullptr)
        return fail(MG_ERR_INVALID_ARG, "mg_rmsnorm_dw_reduce: give dw_f32, dw_cast or both");
    if (dw_cast != nullptr && esize_of(cast_dtype) == 0)
        return fail(MG_ERR_INVALID_ARG, "mg_rmsnorm_dw_reduce: unknown cast_dtype %d", cast_dtype);
    if (dw_partial == nullptr || !aligned(dw_partial, 16))
        return fail(MG_ERR_INVALID_ARG, "mg_rmsnorm_dw_reduce: dw_partial must be a 16-byte aligned device pointer");
    if (!aligned(dw_f32, 4) || (dw_cast != nullptr && !aligned(dw_cast, esize_of(cast_dtype))))
        return fail(MG_ERR_INVALID_ARG, "mg_rmsnorm_dw_reduce: an output pointer is not aligned to its element size");
    hipError_t e = launch_dw_reduce(dw_f32, dw_cast, cast_dtype, dw_partial, (int)num_partials, (int)ld, (int)cols,
                                    (hipStream_t)stream);
    if (e != hipSuccess) return fail_hip("mg_rmsnorm_dw_reduce: launch", e);
    return MG_OK;
}

// ---- the entry point that allocates nothing ----
// dW partials live in a device array of the library itself.  The array's name is a host-side
// handle, not a device address: its per-device address is fetched once with
// hipGetSymbolAddress and that pointer is what the kernels get.
constexpr int64_t kScratchFloats = (int64_t)MG_NOALLOC_SCRATCH_BYTES / 4;
static __device__ __align__(256) float scratch[kScratchFloats];

static int scratch_address(float** out) {
    static std::atomic<float*> cache[64];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail_hip("mg_rmsnorm_bwd_noalloc: hipGetDevice", e);
    if (dev >= 0 && dev < 64) {
        float* p = cache[dev].load(std::memory_order_acquire);
        if (p != nullptr) { *out = p; return MG_OK; }
    }
    void* addr = nullptr;
    e = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || addr == nullptr)
        return fail_hip("mg_rmsnorm_bwd_noalloc: hipGetSymbolAddress(scratch)", e == hipSuccess ? hipErrorInvalidSymbol : e);
    if (dev >= 0 && dev < 64) cache[dev].store((float*)addr, std::memory_order_release);
    *out = (float*)addr;
    return MG_OK;
}

int mg_rmsnorm_bwd_noalloc(void* dx, float* dw_f32, void* dw_cast, const void* dy, const void* x, const void* w,
                           const float* inv_rms, int64_t rows, int64_t cols, int dtype, void* stream) {
    int rc = check_rmsnorm_dims("mg_rmsnorm_bwd_noalloc", rows, cols, dtype);
    if (rc != MG_OK) return rc;
    if (cols > MG_NOALLOC_MAX_COLS)
        return fail(MG_ERR_UNSUPPORTED,
                    "mg_rmsnorm_bwd_noalloc: cols = %lld is beyond this entry point's maximum of %d; use "
                    "mg_rmsnorm_bwd with a workspace of the caller's",
                    (long long)cols, MG_NOALLOC_MAX_COLS);
    if (dw_f32 == nullptr && dw_cast == nullptr)
        return fail(MG_ERR_INVALID_ARG, "mg_rmsnorm_bwd_noalloc: give dw_f32, dw_cast or both");
    int64_t num_partials = 0, ld = 0;
    rc = mg_rmsnorm_bwd_workspace(rows, cols, dtype, &num_partials, &ld);
    if (rc != MG_OK) return rc;
    if (num_partials * ld > kScratchFloats) num_partials = kScratchFloats / ld;   // >= 64 rows: ld <= 65536
    float* part = nullptr;
    rc = scratch_address(&part);
    if (rc != MG_OK) return rc;
    rc = mg_rmsnorm_bwd(dx, part, dy, x, w, inv_rms, rows, cols, dtype, num_partials, ld, stream);
    if (rc != MG_OK) return rc;
    return mg_rmsnorm_dw_reduce(dw_f32, dw_cast, dtype, part, num_partials, ld, cols, stream);
}

int mg_copy_bytes(void* dst, const void* src, int64_t bytes, void* stream) {
    if (bytes < 0 || bytes % 16 != 0 || bytes >= (1LL << 40))
        return fail(MG_ERR_INVALID_ARG, "mg_copy_bytes: bytes must be a non-negative multiple of 16 below 2^40 (got %lld)",
                    (long long)bytes);
    if (bytes == 0) return MG_OK;
    if (dst == nullptr || src == nullptr || !aligned(dst, 16) || !aligned(src, 16))
        return fail(MG_ERR_INVALID_ARG, "mg_copy_bytes: dst and src must be 16-byte aligned device pointers");
    hipError_t e = launch_copy(dst, src, (long)bytes, (hipStream_t)stream);
    if (e != hipSuccess) return fail_hip("mg_copy_bytes: launch", e);
    return MG_OK;
}

int mg_stream_probe(void* dst, const void* a, const void* b, int64_t bytes, void* stream) {
    if (bytes < 0 || bytes % 16 != 0 || bytes >= (1LL << 42))
        return fail(MG_ERR_INVALID_ARG, "mg_stream_probe: bytes must be a non-negative multiple of 16 below 2^42 (got %lld)",
                    (long long)bytes);
    if (bytes == 0) return MG_OK;
    if (dst == nullptr || a == nullptr || !aligned(dst, 4) || !aligned(a, 4) || !aligned(b, 4))
        return fail(MG_ERR_INVALID_ARG, "mg_stream_probe: dst, a (and b, if given) must be 4-byte aligned device pointers");
    hipError_t e = launch_stream_probe(dst, a, b, (long)bytes, xcd_group_or(kXcdGroupStreaming), (hipStream_t)stream);
    if (e != hipSuccess) return fail_hip("mg_stream_probe: launch", e);
    return MG_OK;
}

int mg_row_probe(void* dst, const void* a, const void* b, int64_t rows, int64_t row_bytes, int64_t workgroups,
                 void* stream) {
    if (rows < 0 || rows >= (1LL << 31))
        return fail(MG_ERR_INVALID_ARG, "mg_row_probe: rows must be in [0, 2^31) (got %lld)", (long long)rows);
    if (row_bytes < 16 || row_bytes % 16 != 0 || row_bytes > 65536)
        return fail(MG_ERR_INVALID_ARG, "mg_row_probe: row_bytes must be a multiple of 16 from 16 to 65536 (got %lld)",
                    (long long)row_bytes);
    if (workgroups < 0 || workgroups >= (1LL << 31))
        return fail(MG_ERR_INVALID_ARG, "mg_row_probe: workgroups must be in [0, 2^31) (got %lld)", (long long)workgroups);
    if (rows == 0) return MG_OK;
    if (dst == nullptr || a == nullptr || !aligned(dst, 4) || !aligned(a, 4) || !aligned(b, 4))
        return fail(MG_ERR_INVALID_ARG, "mg_row_probe: dst, a (and b, if given) must be 4-byte aligned device pointers");
    hipError_t e = launch_row_probe(dst, a, b, (long)rows, (long)row_bytes, (long)workgroups, (hipStream_t)stream);
    if (e != hipSuccess) return fail_hip("mg_row_probe: launch", e);
    return MG_OK;
}

static int check_swiglu(const char* fn, int64_t M, int64_t H, int dtype) {
    if (esize_of(dtype) == 0)
        return fail(MG_ERR_INVALID_ARG, "%s: unknown dtype %d (use 0=fp32, 1=fp16, 2=bf16)", fn, dtype);
    if (M < 0) return fail(MG_ERR_INVALID_ARG, "%s: M must be >= 0 (got %lld)", fn, (long long)M);
    if (H < 1) return fail(MG_ERR_INVALID_ARG, "%s: H must be >= 1 (got %lld)", fn, (long long)H);
    if (H >= (1LL << 30)) return fail(MG_ERR_UNSUPPORTED, "%s: H too large (%lld; max 2^30-1)", fn, (long long)H);
    if (M > (1LL << 40) / H)
        return fail(MG_ERR_UNSUPPORTED, "%s: M*H too large (%lld x %lld; max 2^40 elements)", fn, (long long)M,
                    (long long)H);
    return MG_OK;
}

// Aligned 16-byte vectors when the half-row pitch and every base allow it; otherwise 16-byte
// vectors at any alignment (a row of [gate | up] must stay below 2^31 bytes for their 32-bit
// offsets); one element per thread on request or for such enormous rows.
static int swiglu_mode(int64_t half_row_bytes, bool bases_aligned) {
    if (opt_force_generic.load() != 0) return kSwigluElementwise;
    if (half_row_bytes % 16 == 0 && bases_aligned) return kSwigluAligned;
    return 2 * half_row_bytes < (1LL << 31) ? kSwigluRagged : kSwigluElementwise;
}

static int swiglu_unroll(int dflt, int maxv) {
    int u = opt_swiglu_unroll.load();
    if (u == 1 || u == 2 || u == 4 || (u == 8 && maxv >= 8)) return u;
    return dflt;
}

int mg_swiglu_fwd(void* h, const void* gu, int64_t M, int64_t H, int dtype, void* stream) {
    int rc = check_swiglu("mg_swiglu_fwd", M, H, dtype);
    if (rc != MG_OK) return rc;
    if (M == 0) return MG_OK;
    if (h == nullptr || gu == nullptr) return fail(MG_ERR_INVALID_ARG, "mg_swiglu_fwd: h and gu must not be NULL");
    const int es = esize_of(dtype);
    if (!aligned(h, es) || !aligned(gu, es))
        return fail(MG_ERR_INVALID_ARG, "mg_swiglu_fwd: a pointer is not aligned to its element size");
    const int mode = swiglu_mode(H * es, aligned(h, 16) && aligned(gu, 16));
    hipError_t e = launch_swiglu_fwd(dtype, mode, swiglu_unroll(1, 8), xcd_group_or(kXcdGroupStreaming), h, gu, (long)M, (long)H, (hipStream_t)stream);
    if (e != hipSuccess) return fail_hip("mg_swiglu_fwd: launch", e);
    return MG_OK;
}

int mg_swiglu_bwd(void* dgu, const void* dh, const void* gu, int64_t M, int64_t H, int dtype, void* stream) {
    int rc = check_swiglu("mg_swiglu_bwd", M, H, dtype);
    if (rc != MG_OK) return rc;
    if (M == 0) return MG_OK;
    if (dgu == nullptr || dh == nullptr || gu == nullptr)
        return fail(MG_ERR_INVALID_ARG, "mg_swiglu_bwd: dgu, dh and gu must not be NULL");
    const int es = esize_of(dtype);
    if (!aligned(dgu, es) || !aligned(dh, es) || !aligned(gu, es))
        return fail(MG_ERR_INVALID_ARG, "mg_swiglu_bwd: a pointer is not aligned to its element size");
    const int mode = swiglu_mode(H * es, aligned(dgu, 16) && aligned(dh, 16) && aligned(gu, 16));
    hipError_t e =
        launch_swiglu_bwd(dtype, mode, swiglu_unroll(1, 4), xcd_group_or(kXcdGroupStreaming), dgu, dh, gu, (long)M, (long)H, (hipStream_t)stream);
    if (e != hipSuccess) return fail_hip("mg_swiglu_bwd: launch", e);
    return MG_OK;
}

}  // extern "C"
