/* pm_expf.h — a single-precision exp that returns the same bits on the GPU and on the host.
 *
 * Router selection compares f32 scores, so the score transform must be bit-identical to the one the
 * CPU reference computes with its C library (1 / (1 + expf(-x)), expf(x - max); plow
 * runtime/cpu/dev/golden/moe_route.c:33-40). This is the published algorithm of that library's expf
 * (the ARM optimized-routines exp2f-table method glibc >= 2.27 ships: N = 32 table of 2^(i/N),
 * degree-3 polynomial, all arithmetic in binary64, one final rounding to binary32), written with
 * explicit fused multiply-adds in the places where the x86-64 FMA build of the library fuses them.
 * Every step is an IEEE-754 binary64 operation, which gfx950 implements exactly, so device and host
 * agree bit for bit. The host build of this header is compared with the C library's expf over all
 * 2^32 inputs by tests/test_pm_expf.py.
 *
 * Plain C99 (also valid HIP device code): no library calls, no statics.
 */
#ifndef PLOW_PM_EXPF_H
#define PLOW_PM_EXPF_H

#include <stdint.h>

#if defined(__HIPCC__)
#define PM_FN __host__ __device__ static inline
#else
#define PM_FN static inline
#endif

PM_FN uint64_t pm_exp2_tab(uint32_t i) {
    /* bits of 2^(i/32) minus (i << 47), so that adding (k << 47) lands 2^(k/32) for any integer k */
    switch (i & 31u) {
    case 0: return 0x3ff0000000000000ull;  case 1: return 0x3fefd9b0d3158574ull;
    case 2: return 0x3fefb5586cf9890full;  case 3: return 0x3fef9301d0125b51ull;
    case 4: return 0x3fef72b83c7d517bull;  case 5: return 0x3fef54873168b9aaull;
    case 6: return 0x3fef387a6e756238ull;  case 7: return 0x3fef1e9df51fdee1ull;
    case 8: return 0x3fef06fe0a31b715ull;  case 9: return 0x3feef1a7373aa9cbull;
    case 10: return 0x3feedea64c123422ull; case 11: return 0x3feece086061892dull;
    case 12: return 0x3feebfdad5362a27ull; case 13: return 0x3feeb42b569d4f82ull;
    case 14: return 0x3feeab07dd485429ull; case 15: return 0x3feea47eb03a5585ull;
    case 16: return 0x3feea09e667f3bcdull; case 17: return 0x3fee9f75e8ec5f74ull;
    case 18: return 0x3feea11473eb0187ull; case 19: return 0x3feea589994cce13ull;
    case 20: return 0x3feeace5422aa0dbull; case 21: return 0x3feeb737b0cdc5e5ull;
    case 22: return 0x3feec49182a3f090ull; case 23: return 0x3feed503b23e255dull;
    case 24: return 0x3feee89f995ad3adull; case 25: return 0x3feeff76f2fb5e47ull;
    case 26: return 0x3fef199bdd85529cull; case 27: return 0x3fef3720dcef9069ull;
    case 28: return 0x3fef5818dcfba487ull; case 29: return 0x3fef7c97337b9b5full;
    case 30: return 0x3fefa4afa2a490daull; default: return 0x3fefd0765b6e4540ull;
    }
}

/* The body, with the table access as a parameter (TAB(i): entry i & 31) so that the device's second form
 * below is the same arithmetic by construction. The special inputs are decided first and selected last:
 * no lane leaves early, which the second form needs. */
#define PM_EXPF_BODY(x, TAB)                                                                        \
    uint32_t xb;                                                                                    \
    __builtin_memcpy(&xb, &(x), 4);                                                                 \
    const uint32_t abstop = (xb >> 20) & 0x7ffu;                                                    \
    int special = 0;                                                                                \
    float special_value = 0.0f;                                                                     \
    if (abstop >= 0x42bu) { /* |x| >= 88 or NaN */                                                  \
        if (xb == 0xff800000u) special = 1, special_value = 0.0f;                                   \
        else if (abstop >= 0x7f8u) special = 1, special_value = (x) + (x);                          \
        else if ((x) > 0x1.62e42ep6f) special = 1, special_value = __builtin_inff();                \
        else if ((x) < -0x1.9fe368p6f) special = 1, special_value = 0.0f;                           \
    }                                                                                               \
    const double xd = (double)(x);                                                                  \
    const double inv_ln2_n = 0x1.71547652b82fep+0 * 32.0;                                           \
    const double shift = 0x1.8p+52;                                                                 \
    const double z = inv_ln2_n * xd;                                                                \
    double kd = z + shift;                                                                          \
    uint64_t ki;                                                                                    \
    __builtin_memcpy(&ki, &kd, 8);                                                                  \
    kd -= shift;                                                                                    \
    const double r = __builtin_fma(inv_ln2_n, xd, -kd);                                             \
    uint64_t t = TAB((uint32_t)ki) + (ki << 47);                                                    \
    double s;                                                                                       \
    __builtin_memcpy(&s, &t, 8);                                                                    \
    const double c0 = 0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0;                                    \
    const double c1 = 0x1.ebfce50fac4f3p-3 / 32.0 / 32.0;                                           \
    const double c2 = 0x1.62e42ff0c52d6p-1 / 32.0;                                                  \
    const double p = __builtin_fma(c0, r, c1);                                                      \
    const double r2 = r * r;                                                                        \
    double y = __builtin_fma(c2, r, 1.0);                                                           \
    y = __builtin_fma(p, r2, y);                                                                    \
    y = y * s;                                                                                      \
    return special ? special_value : (float)y;

PM_FN float pm_expf(float x) { PM_EXPF_BODY(x, pm_exp2_tab) }

#if defined(__HIPCC__)
/* Second form for code in which a whole wave evaluates the function together: lane l keeps entry l & 31 of
 * the table in registers and an entry is fetched from the lane that holds it (two lane permutes), instead
 * of through the 32-way selection above, which the lanes of a wave take one case after the other. Every lane
 * of the wave must be active at the call (a permute reads nothing from an inactive lane). */
struct PmExpLanes {
    uint32_t lo, hi;
};
__device__ static inline PmExpLanes pm_exp_lanes() {
    const uint64_t t = pm_exp2_tab(threadIdx.x & 31u);
    return PmExpLanes{(uint32_t)t, (uint32_t)(t >> 32)};
}
#define PM_TAB_LANES(i)                                                                             \
    (((uint64_t)(uint32_t)__shfl((int)tab.hi, (int)((i) & 31u), 64) << 32) | (uint64_t)(uint32_t)__shfl((int)tab.lo, (int)((i) & 31u), 64))
__device__ static inline float pm_expf_lanes(float x, const PmExpLanes& tab) { PM_EXPF_BODY(x, PM_TAB_LANES) }
#endif

#endif
