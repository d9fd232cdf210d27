// Division of a 32-bit unsigned number by a run-time invariant divisor with one
// multiply-high, after Granlund & Montgomery, "Division by invariant integers using
// multiplication" (1994), figure 4.1.  Usable from host and device code.
#pragma once
#include <stdint.h>

namespace mg {

struct FastDiv {
    uint32_t d;     // divisor (>= 1)
    uint32_t mul;   // floor(2^32 * (2^l - d) / d) + 1, l = ceil(log2 d)
    uint32_t sh1;   // min(l, 1)
    uint32_t sh2;   // max(l - 1, 0)
};

inline FastDiv make_fastdiv(uint32_t d) {
    FastDiv f;
    f.d = d;
    uint32_t l = 0;
    while (l < 32 && (uint64_t(1) << l) < d) ++l;
    const uint64_t two_l = uint64_t(1) << l;
    f.mul = (uint32_t)(((two_l - d) << 32) / d + 1);
    f.sh1 = l < 1 ? l : 1;
    f.sh2 = l > 1 ? l - 1 : 0;
    return f;
}

#if defined(__HIPCC__)
#define MG_HD __host__ __device__ __forceinline__
#else
#define MG_HD inline
#endif

MG_HD uint32_t fastdiv_mulhi(uint32_t a, uint32_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __umulhi(a, b);
#else
    return (uint32_t)(((uint64_t)a * (uint64_t)b) >> 32);
#endif
}

// n / f.d for any 32-bit n
MG_HD uint32_t fastdiv(uint32_t n, const FastDiv& f) {
    const uint32_t t = fastdiv_mulhi(f.mul, n);
    return (t + ((n - t) >> f.sh1)) >> f.sh2;
}

}  // namespace mg
