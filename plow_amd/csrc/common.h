/* common.h — shared device helpers of the gfx950 MoE operator (wave64, CDNA4 only). */
#ifndef PLOW_MOE_COMMON_H
#define PLOW_MOE_COMMON_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/plow_moe.h"

#define WAVE 64u

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef unsigned short bf16_t;

/* bf16 <-> f32 with the rounding of plow's plow_f2bf (runtime/cpu/dev/cpu_dev.h:262-270):
 * nearest even, NaN keeps a payload bit. */
__device__ __forceinline__ float bf2f(bf16_t h) { return __uint_as_float((uint32_t)h << 16); }
__device__ __forceinline__ bf16_t f2bf(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7F800000u) == 0x7F800000u) return (bf16_t)((u >> 16) | ((u & 0xFFFFu) ? 0x40u : 0u));
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (bf16_t)(u >> 16);
}

/* Swizzles of LDS operand rows. Direct loads write 64 lanes' 16-byte pieces to consecutive LDS addresses, so rows
 * sit unpadded, and bank conflicts are avoided by permuting the pieces of a row on the GLOBAL side of the load;
 * the reader applies the same permutation. What must not collide is what one clock serves, measured on this
 * part (two lanes of one set on the same banks cost a clock each):
 *   ds_read_b128  16 lanes per clock, not consecutive ones: {0-3, 12-15, 20-23, 24-27}, then
 *                 {4-7, 8-11, 16-19, 28-31}, then the same of lanes 32-63;
 *   ds_read_b64   32 consecutive lanes per clock.
 * In the matrix operand layout (row = lane & 15, k-chunk = lane >> 4) a b128 set therefore holds rows
 * {0-3, 12-15} of one k-chunk and rows {4-11} of the next: the swizzles send those two classes of rows to
 * disjoint halves of the piece range, and an XOR with the k-chunk's piece offset keeps them disjoint.
 * lds_swz8: XOR for the 16-byte piece index (0..7) of row r, rows of 128 bytes (rows r and r ^ 1 differ in
 * bank bit 5 already). lds_swz16: the same for rows of 256 bytes or a multiple (piece index & 15). */
__device__ __forceinline__ uint32_t lds_swz8(uint32_t r) {
    const uint32_t t = (r >> 1) & 7u;
    return t ^ ((t & 2u) << 1);
}
__device__ __forceinline__ uint32_t lds_swz16(uint32_t r) { return (r ^ ((r & 4u) << 1)) & 15u; }

/* Monotone f32 -> u32 (plow runtime/common/moe_route_key.h:35-39). */
__device__ __forceinline__ uint32_t route_ord(float x) {
    const uint32_t b = __float_as_uint(x);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

/* Two f32 -> two OCP e4m3 bytes in the low half of the result: round to nearest even, saturating
 * (the gfx950 conversion; plow runtime/amd/amd_common.h:1228-1235 relies on the same instruction). */
__device__ __forceinline__ uint32_t cvt2_e4m3(float a, float b) {
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false) & 0xFFFFu;
}
__device__ __forceinline__ uint32_t cvt4_e4m3(float a, float b, float c, float d) {
    int v = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    v = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, v, true);
    return (uint32_t)v;
}

/* GLU epilogue as a pair A(gate) * B(up) (plow runtime/amd/op_moe.h:216-241, runtime/cpu/dev/golden/
 * golden.h:110-133), with the C library's exponential and tanh (not the fast intrinsics), as the
 * reference insists. f0 / f1 are the activation's immediates (the descriptor's fj[0], fj[1]):
 *   0 gelu_tanh(g) * u                 1 silu(g) * u
 *   2 situ: f0 * tanh(g / f0) * sigmoid(g)  *  (f1 > 0 ? f1 * tanh(u / f1) : u)
 *   3 swiglu_oai (alpha f0, limit f1 > 0, else poison): g' = min(g, f1), u' = clamp(u, +-f1):
 *     g' * sigmoid(f0 * g') * (u' + 1)
 *   4 clamped SwiGLU (limit f1): silu(min(g, f1)) * clamp(u, +-f1)
 * Anything else poisons. */
__device__ __forceinline__ float moe_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float moe_glu(float g, float u, uint32_t act, float f0, float f1) {
    if (act == PLOW_MOE_ACT_SILU) return (g / (1.0f + expf(-g))) * u;
    if (act == PLOW_MOE_ACT_GELU_TANH) {
        const float c = 0.7978845608028654f * (g + 0.044715f * g * g * g);
        return (0.5f * g * (1.0f + tanhf(c))) * u;
    }
    if (act == PLOW_MOE_ACT_SITU) return (f0 * tanhf(g / f0) * moe_sigmoid(g)) * (f1 > 0.0f ? f1 * tanhf(u / f1) : u);
    if (act == PLOW_MOE_ACT_SWIGLU_OAI) {
        if (!(f1 > 0.0f)) return __builtin_nanf("");
        g = g < f1 ? g : f1;
        u = u < -f1 ? -f1 : (u > f1 ? f1 : u);
        return g * moe_sigmoid(f0 * g) * (u + 1.0f);
    }
    if (act == PLOW_MOE_ACT_SWIGLU_CLAMP) {
        const float gc = fminf(g, f1);
        return (gc / (1.0f + expf(-gc))) * fminf(fmaxf(u, -f1), f1);
    }
    return __builtin_nanf("");
}

/* The order-independent form of the fused down -> combine (plow runtime/amd/op_moe.h:2110-2165): a
 * contribution crosses into the [T][H] accumulator as the integer-valued double rint(clamp(v, +-2^17) *
 * 2^32), added with a device-scope f64 atomic. Every partial sum of up to 16 such values is an integer
 * below 2^53, so every addition is exact and the total does not depend on the order of arrival. A NaN
 * clamps to -2^17 (fmaxf returns its other operand), as in the reference. */
#define PLOW_DET_SCALE 4294967296.0
#define PLOW_DET_UNSCALE 2.3283064365386962890625e-10
#define PLOW_DET_CLAMP 131072.0f
__device__ __forceinline__ double det_q(float v) {
    return __builtin_rint((double)fminf(fmaxf(v, -PLOW_DET_CLAMP), PLOW_DET_CLAMP) * PLOW_DET_SCALE);
}
__device__ __forceinline__ void det_add(double* p, float v) {
    (void)__builtin_amdgcn_global_atomic_fadd_f64((__attribute__((address_space(1))) double*)p, det_q(v));
}

/* The activation quantizer of the fp4 x fp4 arm (plow runtime/amd/amd_common.h:1073-1111, :731-741,
 * :1031-1068): the E8M0 byte that maps a 32-block's amax onto e2m1's top code, its exact inverse scale,
 * and the e2m1 code of a scaled value (nearest on the ladder, exact midpoints away from zero, saturating
 * at 6; NaN gives code 7). */
__device__ __forceinline__ uint32_t mxq_e8m0(float amax) {
    if (!(amax > 0.0f)) return 127u;
    const uint32_t bits = __float_as_uint(amax), E = bits >> 23;
    if (E == 0xFFu || bits < 4u) return 127u;
    int e = (int)E - 1 - (int)((bits & 0x7FFFFFu) < 0x400000u);
    e = e < 1 ? 1 : e;
    e = e > 254 ? 254 : e;
    return (uint32_t)e;
}
__device__ __forceinline__ float mxq_inv(uint32_t b) {
    return b == 254u ? __uint_as_float(0x00400000u) : __uint_as_float((254u - b) << 23);
}
__device__ __forceinline__ uint32_t mxq_fp4(float v) {
    const uint32_t sign = (v < 0.0f) ? 8u : 0u;
    const float a = fabsf(v);
    const uint32_t n = (uint32_t)!(a < 0.25f) + (uint32_t)!(a < 0.75f) + (uint32_t)!(a < 1.25f) + (uint32_t)!(a < 1.75f) +
                       (uint32_t)!(a < 2.5f) + (uint32_t)!(a < 3.5f) + (uint32_t)!(a < 5.0f);
    return sign | n;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

/* Workgroup barrier that orders LDS traffic only. __syncthreads() also drains every outstanding
 * global load (s_waitcnt vmcnt(0)), which would serialise a kernel that keeps loads in flight across
 * the barrier; this one leaves them in flight. Use it when the data exchanged lives in LDS. */
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

/* Cache-policy operand of a direct global -> LDS load for bytes that are read once, in whole 128-byte lines (an
 * expert's weight rows at decode; at prefill those of an expert whose rows fit one row tile): non-temporal.
 * Measured on the DeepSeek-V3 decode GLU, 6.37 GB of weights per launch: 1061 -> 967 us (6.0 -> 6.6 TB/s). Not for
 * bytes that are read again soon (token rows; weight rows that a second row tile of the expert reads: 8 % slower
 * at 4096 tokens with the bit on all of them) and not for lines that come in piecewise (8 bytes of an E8M0 scale
 * row a step: every line fetched sixteen times; 64-byte halves a k-step apart: 13 % slower). */
#define LOAD_NT 2

#endif
