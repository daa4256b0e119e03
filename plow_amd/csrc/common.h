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

/* GLU epilogue (plow runtime/amd/op_moe.h:216-241): act 1 silu, act 0 gelu_tanh, with the C library
 * exponential (not the fast intrinsic), as the reference insists. Other activations poison. */
__device__ __forceinline__ float moe_glu(float g, float u, uint32_t act) {
    if (act == PLOW_MOE_ACT_SILU) return (g / (1.0f + expf(-g))) * u;
    if (act == PLOW_MOE_ACT_GELU_TANH) {
        const float c = 0.7978845608028654f * (g + 0.044715f * g * g * g);
        return (0.5f * g * (1.0f + tanhf(c))) * u;
    }
    return __builtin_nanf("");
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

#endif
