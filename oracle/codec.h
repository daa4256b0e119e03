/* codec.h — number formats of the MoE path, restated for the CPU oracle.
 *
 * TEST INFRASTRUCTURE ONLY: the oracle is the checker for the HIP operator; nothing in the shipped
 * library includes or links it.
 *
 * Each function names the plow source it follows:
 *   bf16 <-> f32   runtime/cpu/dev/cpu_dev.h:254-270   (RNE; NaN keeps a payload bit)
 *   e4m3fn         runtime/cpu/dev/fp8_common.h:16-41  (OCP, max 448, RNE, saturating, 0x7f/0xff NaN)
 *   e2m1 / e8m0    runtime/cpu/dev/mxfp4_common.h:15-27 (LUT {0,.5,1,1.5,2,3,4,6}; bitcast(s << 23))
 * Pinned by tests/test_oracle_codecs.py: exhaustive decode tables against closed forms, encode ==
 * nearest-representable (ties to even) by brute force over all 254 finite codes, and bit equality
 * with the compiled reference where oracle/_ref is built.
 */
#ifndef PLOW_ORACLE_CODEC_H
#define PLOW_ORACLE_CODEC_H

#include <math.h>
#include <stdint.h>
#include <string.h>

typedef uint16_t orc_bf16;

static inline uint32_t orc_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float orc_from_bits(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

static inline float orc_bf2f(orc_bf16 h) { return orc_from_bits((uint32_t)h << 16); }

static inline orc_bf16 orc_f2bf(float f) {
    uint32_t u = orc_bits(f);
    if ((u & 0x7F800000u) == 0x7F800000u) /* Inf / NaN: truncate, keep a NaN a NaN */
        return (orc_bf16)((u >> 16) | ((u & 0xFFFFu) ? 0x40u : 0u));
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (orc_bf16)(u >> 16);
}

/* e4m3fn decode: sign | e(4, bias 7) | m(3). e == 0 is subnormal m * 2^-9. */
static inline float orc_e4m3_to_f32(uint8_t b) {
    const uint32_t e = (b >> 3) & 15u, m = b & 7u;
    float v;
    if (e == 15u && m == 7u) v = NAN;
    else if (e == 0u) v = (float)m * 0x1p-9f;
    else v = ldexpf((float)(8u + m), (int)e - 10);
    return (b & 0x80u) ? -v : v;
}

/* e4m3fn encode, round to nearest even, magnitudes >= 448 (Inf included) saturate to 0x7e. */
static inline uint8_t orc_f32_to_e4m3(float x) {
    const uint32_t u = orc_bits(x);
    const uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    const uint32_t mag = u & 0x7FFFFFFFu;
    if (mag > 0x7F800000u) return sign | 0x7Fu;
    const float a = orc_from_bits(mag);
    if (a >= 448.0f) return sign | 0x7Eu;
    if (a < 0x1p-6f) {
        /* subnormal grid: multiples of 2^-9; nearbyintf is RNE in the default rounding mode. A
         * result of 8 is the code of the smallest normal, 0x08, which is what the sum below gives. */
        return sign | (uint8_t)nearbyintf(a * 512.0f);
    }
    int e;
    const float fr = frexpf(a, &e);               /* a = fr * 2^e, fr in [0.5, 1) */
    uint32_t q = (uint32_t)nearbyintf(fr * 16.0f); /* 8..16 : 1.mmm * 8 */
    int E = e - 1;
    if (q == 16u) { q = 8u; E += 1; }
    return sign | (uint8_t)(((uint32_t)(E + 7) << 3) | (q - 8u));
}

static inline float orc_e2m1(uint8_t nib) {
    static const float mag[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
    const float v = mag[nib & 7u];
    return (nib & 8u) ? -v : v;
}

/* E8M0 as the GPU reads it: bitcast(s << 23); s = 0 -> 0, s = 255 -> +Inf. */
static inline float orc_e8m0(uint8_t s) { return orc_from_bits((uint32_t)s << 23); }

/* Element k of an mxfp4 row: low nibble = even k. */
static inline float orc_mxfp4_at(const uint8_t* w, uint32_t k) {
    const uint8_t b = w[k >> 1];
    return orc_e2m1((k & 1u) ? (uint8_t)(b >> 4) : (uint8_t)(b & 15u));
}

/* Monotone f32 -> u32 (runtime/common/moe_route_key.h:35-39). */
static inline uint32_t orc_ord(float x) {
    const uint32_t b = orc_bits(x);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

#endif
