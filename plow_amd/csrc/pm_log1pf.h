/* pm_log1pf.h — a single-precision log1p for arguments in [0, 1] that returns the same bits on the GPU
 * and on the host.
 *
 * The router's sqrt-softplus transform is sqrtf(log1pf(expf(-|l|)) + max(l, 0)) (plow
 * runtime/amd/op_moe.h:485-494); selection compares the resulting f32 scores, so the device has to
 * compute what the CPU restatement computes with its C library. This is the published algorithm of that
 * library's log1pf (the FreeBSD msun / fdlibm single-precision routine glibc ships up to 2.39: argument
 * reduction 1 + x = 2^k (1 + f), a degree-7 polynomial in s^2 with s = f / (2 + f), ln2 split in two
 * words), restricted to 0 <= x <= 1, which is all expf(-|l|) can be. Every step is an IEEE-754 binary32
 * operation with a single rounding (compile without multiply-add contraction and with correctly rounded
 * division), so device and host agree bit for bit. The host build of this header is compared with the C
 * library's log1pf over every float in [0, 1] by tests/test_pm_expf.py.
 *
 * Plain C99 (also valid HIP device code): no library calls, no statics.
 */
#ifndef PLOW_PM_LOG1PF_H
#define PLOW_PM_LOG1PF_H

#include <stdint.h>

#if defined(__HIPCC__)
#define PM_L1_FN __host__ __device__ static inline
#else
#define PM_L1_FN static inline
#endif

/* x in [0, 1] (NaN and anything else: unspecified) */
PM_L1_FN float pm_log1pf_unit(float x) {
    const float ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f;
    const float Lp1 = 6.6666668653e-01f, Lp2 = 4.0000000596e-01f, Lp3 = 2.8571429849e-01f, Lp4 = 2.2222198546e-01f,
                Lp5 = 1.8183572590e-01f, Lp6 = 1.5313838422e-01f, Lp7 = 1.4798198640e-01f;
    uint32_t hx;
    __builtin_memcpy(&hx, &x, 4);
    float f, c = 0.0f;
    int32_t k = 1, hu = 1;
    if (hx < 0x3ed413d7u) { /* x < sqrt(2) - 1: no reduction */
        if (hx < 0x31000000u) { /* x < 2^-29 */
            if (hx < 0x24800000u) return x; /* x < 2^-54 */
            return x - x * x * 0.5f;
        }
        k = 0, f = x;
    } else {
        float u = 1.0f + x;
        uint32_t ub;
        __builtin_memcpy(&ub, &u, 4);
        k = (int32_t)(ub >> 23) - 127;
        c = k > 0 ? 1.0f - (u - x) : x - (u - 1.0f); /* what the sum 1 + x lost */
        c /= u;
        ub &= 0x007fffffu;
        if (ub < 0x3504f7u) {
            ub |= 0x3f800000u; /* u in [1, sqrt 2) */
            hu = (int32_t)(ub & 0x007fffffu);
        } else {
            k += 1;
            hu = (int32_t)((0x00800000u - ub) >> 2);
            ub |= 0x3f000000u; /* u / 2 in [sqrt 2 / 2, 1) */
        }
        __builtin_memcpy(&u, &ub, 4);
        f = u - 1.0f;
    }
    const float fk = (float)k;
    const float hfsq = 0.5f * f * f;
    if (hu == 0) { /* |f| < 2^-20 */
        if (f == 0.0f) {
            if (k == 0) return 0.0f;
            c += fk * ln2_lo;
            return fk * ln2_hi + c;
        }
        const float R0 = hfsq * (1.0f - 0.66666666666666666f * f);
        if (k == 0) return f - R0;
        return fk * ln2_hi - ((R0 - (fk * ln2_lo + c)) - f);
    }
    const float s = f / (2.0f + f);
    const float z = s * s;
    const float R = z * (Lp1 + z * (Lp2 + z * (Lp3 + z * (Lp4 + z * (Lp5 + z * (Lp6 + z * Lp7))))));
    if (k == 0) return f - (hfsq - s * (hfsq + R));
    return fk * ln2_hi - ((hfsq - (s * (hfsq + R) + (fk * ln2_lo + c))) - f);
}

#endif
