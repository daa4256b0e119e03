/* quant.hip — activation quantizers: 1x128 e4m3 (op 184) and per-row e4m3 (op 32).
 * Compiled with -ffp-contract=off: scale and reciprocal are separately rounded IEEE operations, as in
 * the reference (plow runtime/amd/op_gemm_common.h:2582-2621, runtime/cpu/dev/golden/fp8.c:9-30). */
#include "common.h"
#include "kernels.h"
#include "pm_expf.h"

/* 16 lanes per (row, 128-group), 8 bf16 each. scale[g][row] with row pitch `pitch`. */
__global__ __launch_bounds__(256) void k_quant_block128(uint8_t* __restrict__ xq,
                                                        const bf16_t* __restrict__ x,
                                                        float* __restrict__ scale, uint32_t M,
                                                        uint32_t K, uint32_t pitch) {
    const uint32_t groups = K / 128u, sub = threadIdx.x & 15u;
    const size_t ngroup = (size_t)M * groups;
    for (size_t grp = ((size_t)blockIdx.x * 256u + threadIdx.x) / 16u; grp < ngroup;
         grp += (size_t)gridDim.x * 16u) {
        const uint32_t row = (uint32_t)(grp / groups), g = (uint32_t)(grp % groups);
        const size_t at = (size_t)row * K + g * 128u + sub * 8u;
        const uint4 raw = *(const uint4*)(x + at);
        const uint32_t v[4] = {raw.x, raw.y, raw.z, raw.w};
        float f[8];
        float amax = 1e-10f; /* the amax is floored, not the scale */
#pragma unroll
        for (int j = 0; j < 4; j++) {
            f[2 * j] = __uint_as_float(v[j] << 16);
            f[2 * j + 1] = __uint_as_float(v[j] & 0xFFFF0000u);
            amax = fmaxf(amax, fmaxf(fabsf(f[2 * j]), fabsf(f[2 * j + 1])));
        }
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 16));
        const float s = amax * (1.0f / 448.0f);
        const float inv = 1.0f / s;
        if (sub == 0) scale[(size_t)g * pitch + row] = s;
        uint2 q;
        q.x = cvt4_e4m3(f[0] * inv, f[1] * inv, f[2] * inv, f[3] * inv);
        q.y = cvt4_e4m3(f[4] * inv, f[5] * inv, f[6] * inv, f[7] * inv);
        *(uint2*)(xq + at) = q;
    }
}

int launch_quant_block128(void* xq, const void* x, float* scale, uint32_t M, uint32_t K, uint32_t pitch,
                          hipStream_t st) {
    if (K % 128u || M == 0) return PLOW_MOE_EINVAL;
    const size_t ngroup = (size_t)M * (K / 128u);
    uint32_t blocks = (uint32_t)((ngroup + 15u) / 16u);
    if (blocks > 8192u) blocks = 8192u;
    k_quant_block128<<<blocks, 256, 0, st>>>((uint8_t*)xq, (const bf16_t*)x, scale, M, K, pitch ? pitch : M);
    return 0;
}

/* Op 189 (plow runtime/amd/op_moe_fp8_block128.h:49-55, op_gemm_common.h:2582-2621 with SCATTER,
 * interp.hip:5291-5300): the tilep[E] * 64 aligned bf16 rows, each quantized 1x128 into the row of its
 * routing slot (hq[slot][K], scale[g][slot]; rows whose slot is out of range are skipped), and the bf16
 * layer output [T][H] zeroed for the atomic reduction that follows. 16 lanes per (row, group). */
__global__ __launch_bounds__(256) void k_quant_block128_scatter(uint8_t* __restrict__ hq, const bf16_t* __restrict__ fu,
                                                                float* __restrict__ scale, const int32_t* __restrict__ meta,
                                                                const uint32_t* __restrict__ row_partidx,
                                                                uint2* __restrict__ out, uint32_t K, uint32_t E,
                                                                uint32_t slots, size_t out_words) {
    const uint32_t groups = K / 128u, sub = threadIdx.x & 15u;
    const size_t ngroup = (size_t)((uint32_t)meta[3u * E] * PLOW_MPF_BM) * groups;
    for (size_t grp = ((size_t)blockIdx.x * 256u + threadIdx.x) / 16u; grp < ngroup; grp += (size_t)gridDim.x * 16u) {
        const uint32_t row = (uint32_t)(grp / groups), g = (uint32_t)(grp % groups);
        const uint32_t dst = row_partidx[row];
        if (dst >= slots) continue; /* the same for all 16 lanes of the group */
        const uint4 raw = *(const uint4*)(fu + (size_t)row * K + g * 128u + sub * 8u);
        const uint32_t v[4] = {raw.x, raw.y, raw.z, raw.w};
        float f[8];
        float amax = 1e-10f; /* the amax is floored, not the scale */
#pragma unroll
        for (int j = 0; j < 4; j++) {
            f[2 * j] = __uint_as_float(v[j] << 16);
            f[2 * j + 1] = __uint_as_float(v[j] & 0xFFFF0000u);
            amax = fmaxf(amax, fmaxf(fabsf(f[2 * j]), fabsf(f[2 * j + 1])));
        }
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 16));
        const float s = amax * (1.0f / 448.0f);
        const float inv = 1.0f / s;
        if (sub == 0) scale[(size_t)g * slots + dst] = s;
        uint2 q;
        q.x = cvt4_e4m3(f[0] * inv, f[1] * inv, f[2] * inv, f[3] * inv);
        q.y = cvt4_e4m3(f[4] * inv, f[5] * inv, f[6] * inv, f[7] * inv);
        *(uint2*)(hq + (size_t)dst * K + g * 128u + sub * 8u) = q;
    }
    for (size_t i = (size_t)blockIdx.x * 256u + threadIdx.x; i < out_words; i += (size_t)gridDim.x * 256u)
        out[i] = make_uint2(0u, 0u);
}

int launch_quant_block128_scatter(void* hq, const void* fu, float* scale, const void* meta, const void* row_partidx,
                                  void* out, uint32_t K, uint32_t E, uint32_t topk, uint32_t T, uint32_t H,
                                  hipStream_t st) {
    if (K % 128u || H % 4u || T == 0 || topk == 0 || E == 0) return PLOW_MOE_EINVAL;
    /* the row count lives on the device (meta[3E]); size the grid for its upper bound */
    const size_t rows_max = (size_t)T * topk + (size_t)E * (PLOW_MPF_BM - 1u);
    const size_t ngroup = rows_max * (K / 128u), out_words = (size_t)T * H / 4u;
    size_t want = (ngroup + 15u) / 16u;
    if (want < (out_words + 255u) / 256u) want = (out_words + 255u) / 256u;
    const uint32_t blocks = (uint32_t)(want > 8192u ? 8192u : want);
    k_quant_block128_scatter<<<blocks, 256, 0, st>>>((uint8_t*)hq, (const bf16_t*)fu, scale, (const int32_t*)meta,
                                                     (const uint32_t*)row_partidx, (uint2*)out, K, E, T * topk, out_words);
    return 0;
}

/* e4m3 byte of plow's plow_f32_to_e4m3 (runtime/cpu/dev/fp8_common.h:16-33) for EVERY product
 * prod = x * inv: NaN keeps its sign (0x7f / 0xff), anything at or above 448 in magnitude saturates to
 * the signed 0x7e; in range the hardware conversion rounds as the reference does. A NaN that the
 * multiply itself made (an infinite x times the zero reciprocal of an infinite scale) is the negative
 * default NaN on the reference's x86 host and the positive one here: it takes the reference's byte. */
__device__ __forceinline__ uint32_t e4m3_any(float prod, float x) {
    if (prod != prod && x == x) return 0xFFu;
    const uint32_t u = __float_as_uint(prod), sign = (u >> 24) & 0x80u, mag = u & 0x7FFFFFFFu;
    if (mag > 0x7F800000u) return sign | 0x7Fu;
    if (mag >= 0x43E00000u) return sign | 0x7Eu;
    return cvt2_e4m3(prod, 0.0f) & 0xFFu;
}
__device__ __forceinline__ bool e4m3_in_range(float v) { return (__float_as_uint(v) & 0x7FFFFFFFu) < 0x43E00000u; }

/* activation of the gate alone (plow runtime/cpu/dev/golden/golden.h:103-115): 0 gelu_tanh, 1 silu with
 * the bit-reproducible exponential, anything else poisons */
__device__ __forceinline__ float act_gate_only(float g, uint32_t act) {
    if (act == PLOW_MOE_ACT_SILU) return g / (1.0f + pm_expf(-g));
    if (act == PLOW_MOE_ACT_GELU_TANH) {
        const float c = 0.7978845608028654f * (g + 0.044715f * g * g * g);
        return 0.5f * g * (1.0f + tanhf(c));
    }
    return __builtin_nanf("");
}

/* One workgroup per row (plow runtime/cpu/dev/golden/fp8.c:9-30). With gate / up bound the row is first
 * produced: x = bf16(act(gate) * up), stored, then quantized. amax over K skips NaN (fmaxf) and takes
 * infinities; scale = max(amax / 448, 1e-12), q = e4m3(x * (1 / scale)). VEC: K is a multiple of 8 and
 * every row is 16-byte aligned; otherwise elements are visited one at a time. Each thread quantizes
 * exactly the elements it produced, so no fence is needed between the two passes. */
template <bool VEC>
__global__ __launch_bounds__(256) void k_quant_row(uint8_t* __restrict__ xq, bf16_t* __restrict__ x,
                                                   float* __restrict__ scale, const bf16_t* __restrict__ gate,
                                                   const bf16_t* __restrict__ up, uint32_t act, uint32_t K) {
    __shared__ float red[4];
    const uint32_t row = blockIdx.x, tid = threadIdx.x;
    bf16_t* xr = x + (size_t)row * K;
    float amax = 0.0f;
    if (VEC) {
        for (uint32_t k = tid * 8u; k < K; k += 2048u) {
            uint4 raw;
            if (gate) {
                const uint4 g4 = *(const uint4*)(gate + (size_t)row * K + k);
                const uint4 u4 = *(const uint4*)(up + (size_t)row * K + k);
                const uint32_t gv[4] = {g4.x, g4.y, g4.z, g4.w}, uv[4] = {u4.x, u4.y, u4.z, u4.w};
                uint32_t o[4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const float lo = act_gate_only(__uint_as_float(gv[j] << 16), act) * __uint_as_float(uv[j] << 16);
                    const float hi = act_gate_only(__uint_as_float(gv[j] & 0xFFFF0000u), act) *
                                     __uint_as_float(uv[j] & 0xFFFF0000u);
                    o[j] = (uint32_t)f2bf(lo) | ((uint32_t)f2bf(hi) << 16);
                }
                raw = make_uint4(o[0], o[1], o[2], o[3]);
                *(uint4*)(xr + k) = raw;
            } else {
                raw = *(const uint4*)(xr + k);
            }
            const uint32_t v[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int j = 0; j < 4; j++)
                amax = fmaxf(amax, fmaxf(fabsf(__uint_as_float(v[j] << 16)), fabsf(__uint_as_float(v[j] & 0xFFFF0000u))));
        }
    } else {
        for (uint32_t k = tid; k < K; k += 256u) {
            if (gate)
                xr[k] = f2bf(act_gate_only(bf2f(gate[(size_t)row * K + k]), act) * bf2f(up[(size_t)row * K + k]));
            amax = fmaxf(amax, fabsf(bf2f(xr[k])));
        }
    }
    amax = wave_max(amax);
    if ((tid & 63u) == 0) red[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float s = fmaxf(amax * (1.0f / 448.0f), 1e-12f);
    const float inv = 1.0f / s;
    if (tid == 0) scale[row] = s;
    if (VEC) {
        for (uint32_t k = tid * 8u; k < K; k += 2048u) {
            const uint4 raw = *(const uint4*)(xr + k);
            const uint32_t v[4] = {raw.x, raw.y, raw.z, raw.w};
            float xf[8], f[8];
            bool plain = true;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                xf[2 * j] = __uint_as_float(v[j] << 16);
                xf[2 * j + 1] = __uint_as_float(v[j] & 0xFFFF0000u);
            }
#pragma unroll
            for (int j = 0; j < 8; j++) {
                f[j] = xf[j] * inv;
                plain = plain && e4m3_in_range(f[j]);
            }
            uint2 q;
            if (plain) {
                q.x = cvt4_e4m3(f[0], f[1], f[2], f[3]);
                q.y = cvt4_e4m3(f[4], f[5], f[6], f[7]);
            } else { /* NaN or infinities among the eight: every byte by the total rule */
                q.x = q.y = 0u;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    q.x |= e4m3_any(f[j], xf[j]) << (8 * j);
                    q.y |= e4m3_any(f[4 + j], xf[4 + j]) << (8 * j);
                }
            }
            *(uint2*)(xq + (size_t)row * K + k) = q;
        }
    } else {
        for (uint32_t k = tid; k < K; k += 256u) xq[(size_t)row * K + k] = (uint8_t)e4m3_any(bf2f(xr[k]) * inv, bf2f(xr[k]));
    }
}

int launch_quant_row(void* xq, void* x, float* scale, const void* gate, const void* up, uint32_t act,
                     uint32_t M, uint32_t K, hipStream_t st) {
    if (K == 0 || M == 0 || (gate == nullptr) != (up == nullptr)) return PLOW_MOE_EINVAL;
    const uintptr_t al = (uintptr_t)x | (uintptr_t)gate | (uintptr_t)up;
    if (K % 8u == 0u && al % 16u == 0u && (uintptr_t)xq % 8u == 0u)
        k_quant_row<true><<<M, 256, 0, st>>>((uint8_t*)xq, (bf16_t*)x, scale, (const bf16_t*)gate, (const bf16_t*)up, act, K);
    else
        k_quant_row<false><<<M, 256, 0, st>>>((uint8_t*)xq, (bf16_t*)x, scale, (const bf16_t*)gate, (const bf16_t*)up, act, K);
    return 0;
}
