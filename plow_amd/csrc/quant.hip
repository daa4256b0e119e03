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

__device__ __forceinline__ float e4m3_to_f32(uint32_t byte) { return __builtin_amdgcn_cvt_f32_fp8((int)byte, 0); }

/* Two-term e4m3 rows of the fp8 x fp8 arms 4 / 5 of ops 85 / 86 (plow runtime/amd/moe_pf_w8a8.h:81-92, :420-452):
 * per 1x128 group s = max(amax, 1e-10) / 448, t = v / s, hi = e4m3(t), lo = e4m3((t - hi) * 16); a row is
 * [hi K | lo K] bytes and its scales [K / 128] f32, row-major. The rows are the tilep[E] * 64 aligned rows of
 * `meta`; a pad row (row_token sentinel) leaves as the split of zeros, as the reference writes it. 16 lanes per
 * (row, group), eight values each. */
__global__ __launch_bounds__(256) void k_split_block128(uint8_t* __restrict__ fq, float* __restrict__ fs,
                                                        const bf16_t* __restrict__ fu, const int32_t* __restrict__ meta,
                                                        const uint32_t* __restrict__ row_token, uint32_t K, uint32_t E) {
    const uint32_t groups = K / 128u, sub = threadIdx.x & 15u;
    const size_t ngroup = (size_t)((uint32_t)meta[3u * E] * PLOW_MPF_BM) * groups;
    for (size_t grp = ((size_t)blockIdx.x * 256u + threadIdx.x) / 16u; grp < ngroup; grp += (size_t)gridDim.x * 16u) {
        const uint32_t row = (uint32_t)(grp / groups), g = (uint32_t)(grp % groups);
        const bool live = row_token[row] != PLOW_EXPERT_UNUSED;
        uint4 raw = make_uint4(0u, 0u, 0u, 0u);
        if (live) raw = *(const uint4*)(fu + (size_t)row * K + g * 128u + sub * 8u);
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
        if (sub == 0) fs[(size_t)row * groups + g] = s;
        float t[8], d[8];
#pragma unroll
        for (int j = 0; j < 8; j++) t[j] = f[j] * inv;
        uint2 hi, lo;
        hi.x = cvt4_e4m3(t[0], t[1], t[2], t[3]);
        hi.y = cvt4_e4m3(t[4], t[5], t[6], t[7]);
#pragma unroll
        for (int j = 0; j < 8; j++) d[j] = e4m3_to_f32(((j < 4 ? hi.x : hi.y) >> (8 * (j & 3))) & 0xFFu);
        lo.x = cvt4_e4m3((t[0] - d[0]) * 16.0f, (t[1] - d[1]) * 16.0f, (t[2] - d[2]) * 16.0f, (t[3] - d[3]) * 16.0f);
        lo.y = cvt4_e4m3((t[4] - d[4]) * 16.0f, (t[5] - d[5]) * 16.0f, (t[6] - d[6]) * 16.0f, (t[7] - d[7]) * 16.0f);
        uint8_t* const at = fq + (size_t)row * 2u * K + g * 128u + sub * 8u;
        *(uint2*)at = hi;
        *(uint2*)(at + K) = lo;
    }
}

int launch_split_block128(void* fq, float* fs, const void* fu, const int32_t* meta, const uint32_t* row_token, uint32_t K,
                          uint32_t E, uint32_t rows_bound, hipStream_t st) {
    if (K % 128u || !rows_bound || !fq || !fs || !fu || !meta || !row_token) return PLOW_MOE_EINVAL;
    const size_t ngroup = (size_t)rows_bound * (K / 128u);
    uint32_t blocks = (uint32_t)((ngroup + 15u) / 16u);
    if (blocks > 8192u) blocks = 8192u;
    k_split_block128<<<blocks, 256, 0, st>>>((uint8_t*)fq, fs, (const bf16_t*)fu, meta, row_token, K, E);
    return 0;
}

/* The way back: the aligned rows [hi K | lo K] with their 1x128 scales as bf16 rows s * (hi + lo / 16), which is what
 * the two terms stand for; rows whose slot is the sentinel are skipped. */
__global__ __launch_bounds__(256) void k_join_block128(bf16_t* __restrict__ out, const uint8_t* __restrict__ fq,
                                                       const float* __restrict__ fs, const int32_t* __restrict__ meta,
                                                       const uint32_t* __restrict__ row_partidx, uint32_t K, uint32_t E) {
    const uint32_t groups = K / 128u, sub = threadIdx.x & 15u;
    const size_t ngroup = (size_t)((uint32_t)meta[3u * E] * PLOW_MPF_BM) * groups;
    for (size_t grp = ((size_t)blockIdx.x * 256u + threadIdx.x) / 16u; grp < ngroup; grp += (size_t)gridDim.x * 16u) {
        const uint32_t row = (uint32_t)(grp / groups), g = (uint32_t)(grp % groups);
        if (row_partidx[row] == PLOW_EXPERT_UNUSED) continue;
        const uint8_t* const at = fq + (size_t)row * 2u * K + g * 128u + sub * 8u;
        const uint2 hi = *(const uint2*)at, lo = *(const uint2*)(at + K);
        const float s = fs[(size_t)row * groups + g];
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float v[2];
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int e = 2 * j + h;
                const float a = e4m3_to_f32(((e < 4 ? hi.x : hi.y) >> (8 * (e & 3))) & 0xFFu);
                const float b = e4m3_to_f32(((e < 4 ? lo.x : lo.y) >> (8 * (e & 3))) & 0xFFu);
                v[h] = s * fmaf(b, 0.0625f, a);
            }
            o[j] = (uint32_t)f2bf(v[0]) | ((uint32_t)f2bf(v[1]) << 16);
        }
        *(uint4*)(out + (size_t)row * K + g * 128u + sub * 8u) = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

int launch_join_block128(void* out, const void* fq, const float* fs, const int32_t* meta, const uint32_t* row_partidx,
                         uint32_t K, uint32_t E, uint32_t rows_bound, hipStream_t st) {
    if (K % 128u || !rows_bound || !out || !fq || !fs || !meta || !row_partidx) return PLOW_MOE_EINVAL;
    const size_t ngroup = (size_t)rows_bound * (K / 128u);
    uint32_t blocks = (uint32_t)((ngroup + 15u) / 16u);
    if (blocks > 8192u) blocks = 8192u;
    k_join_block128<<<blocks, 256, 0, st>>>((bf16_t*)out, (const uint8_t*)fq, fs, meta, row_partidx, K, E);
    return 0;
}

/* bf16 rows -> mxfp4 rows with one E8M0 byte per 32 values: the activation quantizer of the fp4 x fp4 arm
 * of ops 85 / 86 (plow runtime/amd/op_moe.h:4132-4179, amd_common.h:1031-1111). Four lanes per 32-block,
 * eight values each; value 2i sits in the low nibble of byte i. */
__global__ __launch_bounds__(256) void k_quant_mx_act(uint8_t* __restrict__ out, uint8_t* __restrict__ scales,
                                                      const bf16_t* __restrict__ x, size_t n_blocks) {
    const uint32_t sub = threadIdx.x & 3u;
    for (size_t b = ((size_t)blockIdx.x * 256u + threadIdx.x) / 4u; b < n_blocks; b += (size_t)gridDim.x * 64u) {
        const uint4 raw = *(const uint4*)(x + b * 32u + sub * 8u);
        const uint32_t v[4] = {raw.x, raw.y, raw.z, raw.w};
        float f[8];
        float amax = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            f[2 * j] = __uint_as_float(v[j] << 16);
            f[2 * j + 1] = __uint_as_float(v[j] & 0xFFFF0000u);
            amax = fmaxf(amax, fmaxf(fabsf(f[2 * j]), fabsf(f[2 * j + 1])));
        }
        amax = fmaxf(amax, __shfl_xor(amax, 1, 4));
        amax = fmaxf(amax, __shfl_xor(amax, 2, 4));
        const uint32_t sb = mxq_e8m0(amax);
        const float inv = mxq_inv(sb);
        uint32_t code = 0u;
#pragma unroll
        for (int j = 0; j < 8; j++) code |= mxq_fp4(f[j] * inv) << (4 * j);
        *(uint32_t*)(out + b * 16u + sub * 4u) = code;
        if (sub == 0) scales[b] = (uint8_t)sb;
    }
}

int launch_quant_mx_act(uint8_t* out, uint8_t* scales, const void* x, uint32_t rows, uint32_t K, hipStream_t st) {
    if (K % 32u || rows == 0 || !out || !scales || !x) return PLOW_MOE_EINVAL;
    const size_t n_blocks = (size_t)rows * (K / 32u);
    uint32_t blocks = (uint32_t)((n_blocks + 63u) / 64u > 16384u ? 16384u : (n_blocks + 63u) / 64u);
    k_quant_mx_act<<<blocks, 256, 0, st>>>(out, scales, (const bf16_t*)x, n_blocks);
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
    /* eight elements at k: produced (act(gate) * up, stored) or loaded; their |max| joins amax */
    auto first_pass = [&](uint32_t k) -> uint4 {
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
        return raw;
    };
    /* VEC: a thread's pieces of the row stay in registers between the two passes when the row has at most four
     * per thread (K <= 8192): the second pass then starts without another trip to memory */
    const bool hold = VEC && K <= 8192u;
    uint4 held[4];
    if (VEC) {
        if (hold) {
#pragma unroll
            for (uint32_t it = 0; it < 4u; it++) {
                const uint32_t k = tid * 8u + it * 2048u;
                held[it] = make_uint4(0u, 0u, 0u, 0u);
                if (k < K) held[it] = first_pass(k);
            }
        } else {
            for (uint32_t k = tid * 8u; k < K; k += 2048u) (void)first_pass(k);
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
    auto second_pass = [&](uint32_t k, const uint4 raw) {
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
    };
    if (VEC) {
        if (hold) {
#pragma unroll
            for (uint32_t it = 0; it < 4u; it++) {
                const uint32_t k = tid * 8u + it * 2048u;
                if (k < K) second_pass(k, held[it]);
            }
        } else {
            for (uint32_t k = tid * 8u; k < K; k += 2048u) second_pass(k, *(const uint4*)(xr + k));
        }
    } else {
        for (uint32_t k = tid; k < K; k += 256u) xq[(size_t)row * K + k] = (uint8_t)e4m3_any(bf2f(xr[k]) * inv, bf2f(xr[k]));
    }
}

/* Rows of at most 2048 elements that only need quantizing (no gate / up): one wave per row, four rows per
 * workgroup. A lane holds its up to four 8-element pieces between the two passes, the row's maximum is a wave
 * reduction, and there is no barrier and no LDS: the same values in the same order as k_quant_row<true>
 * (a maximum does not depend on the order of its operands). */
__global__ __launch_bounds__(256) void k_quant_row_wave(uint8_t* __restrict__ xq, const bf16_t* __restrict__ x,
                                                        float* __restrict__ scale, uint32_t M, uint32_t K) {
    const uint32_t lane = threadIdx.x & 63u, row = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (row >= M) return; /* the whole wave */
    const bf16_t* xr = x + (size_t)row * K;
    uint4 held[4];
    float amax = 0.0f;
#pragma unroll
    for (uint32_t it = 0; it < 4u; it++) {
        const uint32_t k = lane * 8u + it * 512u;
        held[it] = make_uint4(0u, 0u, 0u, 0u);
        if (k < K) held[it] = *(const uint4*)(xr + k);
        const uint32_t v[4] = {held[it].x, held[it].y, held[it].z, held[it].w};
#pragma unroll
        for (int j = 0; j < 4; j++)
            amax = fmaxf(amax, fmaxf(fabsf(__uint_as_float(v[j] << 16)), fabsf(__uint_as_float(v[j] & 0xFFFF0000u))));
    }
    amax = wave_max(amax);
    const float s = fmaxf(amax * (1.0f / 448.0f), 1e-12f);
    const float inv = 1.0f / s;
    if (lane == 0) scale[row] = s;
#pragma unroll
    for (uint32_t it = 0; it < 4u; it++) {
        const uint32_t k = lane * 8u + it * 512u;
        if (k >= K) continue;
        const uint32_t v[4] = {held[it].x, held[it].y, held[it].z, held[it].w};
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
}

int launch_quant_row(void* xq, void* x, float* scale, const void* gate, const void* up, uint32_t act,
                     uint32_t M, uint32_t K, hipStream_t st) {
    if (K == 0 || M == 0 || (gate == nullptr) != (up == nullptr)) return PLOW_MOE_EINVAL;
    const uintptr_t al = (uintptr_t)x | (uintptr_t)gate | (uintptr_t)up;
    if (!gate && K % 8u == 0u && K <= 2048u && al % 16u == 0u && (uintptr_t)xq % 8u == 0u && M >= 64u) {
        k_quant_row_wave<<<(M + 3u) / 4u, 256, 0, st>>>((uint8_t*)xq, (const bf16_t*)x, scale, M, K);
        return 0;
    }
    if (K % 8u == 0u && al % 16u == 0u && (uintptr_t)xq % 8u == 0u)
        k_quant_row<true><<<M, 256, 0, st>>>((uint8_t*)xq, (bf16_t*)x, scale, (const bf16_t*)gate, (const bf16_t*)up, act, K);
    else
        k_quant_row<false><<<M, 256, 0, st>>>((uint8_t*)xq, (bf16_t*)x, scale, (const bf16_t*)gate, (const bf16_t*)up, act, K);
    return 0;
}


/* Op 1, RMSNorm with its fused activation quantizers (plow runtime/cpu/dev/golden/norm.c:15-43,
 * runtime/amd/op_norm.h:486-551): out[row0 + r] = bf16(x[r] * inv * gamma) with
 * inv = 1 / sqrt(mean(x^2) + eps) in f32 (the sum of squares in a fixed tree order, as plow's GPU kernel
 * does; its CPU kernel sums in index order, a difference of rounding only), gamma optional. MODE 1: the
 * rounded row is also quantized per row like op 32 (scale = max(amax / 448, 1e-12)); MODE 2: per 1x128
 * group like op 184 (amax floored at 1e-10, scale [feat / 128][rows]) - in both cases exactly what the
 * separate quantizer produces from `out`. One workgroup per row; a thread keeps its share of the row
 * (8 elements per 256-thread stride, feat <= 16384) in registers between the passes. */
#define RN_MAXV 8
template <int MODE>
__global__ __launch_bounds__(256) void k_rmsnorm(bf16_t* __restrict__ out, const bf16_t* __restrict__ x,
                                                 const bf16_t* __restrict__ gamma, uint8_t* __restrict__ xq,
                                                 float* __restrict__ scale, uint32_t rows, uint32_t feat,
                                                 uint32_t out_row0, float eps) {
    __shared__ float red[4];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wv = tid >> 6;
    auto block_reduce = [&](float v, bool is_max) -> float {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float other = __shfl_xor(v, o, 64);
            v = is_max ? fmaxf(v, other) : v + other;
        }
        __syncthreads(); /* the previous reduction's values have been read */
        if (lane == 0) red[wv] = v;
        __syncthreads();
        return is_max ? fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])) : (red[0] + red[1]) + (red[2] + red[3]);
    };
    for (uint32_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const bf16_t* xr = x + (size_t)row * feat;
        bf16_t* orow = out + (size_t)(out_row0 + row) * feat;
        float f[RN_MAXV][8];
        float ss = 0.0f;
#pragma unroll
        for (int c = 0; c < RN_MAXV; c++) {
            const uint32_t i = ((uint32_t)c * 256u + tid) * 8u;
#pragma unroll
            for (int j = 0; j < 8; j++) f[c][j] = 0.0f;
            if (i < feat) {
                const uint4 raw = *(const uint4*)(xr + i);
                const uint32_t v[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    f[c][2 * j] = __uint_as_float(v[j] << 16);
                    f[c][2 * j + 1] = __uint_as_float(v[j] & 0xFFFF0000u);
                }
#pragma unroll
                for (int j = 0; j < 8; j++) ss += f[c][j] * f[c][j];
            }
        }
        ss = block_reduce(ss, false);
        const float inv = 1.0f / sqrtf(ss / (float)feat + eps);
        float amax_row = 0.0f;
#pragma unroll
        for (int c = 0; c < RN_MAXV; c++) {
            const uint32_t i = ((uint32_t)c * 256u + tid) * 8u;
            float amax = 1e-10f; /* MODE 2: the amax is floored, not the scale */
            if (i < feat) {
                uint4 graw = make_uint4(0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u); /* ones */
                if (gamma) graw = *(const uint4*)(gamma + i);
                const uint32_t gv[4] = {graw.x, graw.y, graw.z, graw.w};
                uint32_t o[8];
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const float g = (j & 1) ? __uint_as_float(gv[j >> 1] & 0xFFFF0000u) : __uint_as_float(gv[j >> 1] << 16);
                    o[j] = f2bf(gamma ? f[c][j] * inv * g : f[c][j] * inv * 1.0f);
                    f[c][j] = bf2f((bf16_t)o[j]); /* the quantizers read the rounded row */
                    amax = fmaxf(amax, fabsf(f[c][j]));
                }
                *(uint4*)(orow + i) = make_uint4(o[0] | (o[1] << 16), o[2] | (o[3] << 16), o[4] | (o[5] << 16), o[6] | (o[7] << 16));
            }
            if (MODE == 2) { /* a 128-group is 16 consecutive threads' 8 elements; feat % 128 == 0 keeps groups whole */
#pragma unroll
                for (int o2 = 8; o2 > 0; o2 >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o2, 16));
                if (i < feat) {
                    const float sc = amax * (1.0f / 448.0f), qi = 1.0f / sc;
                    if ((tid & 15u) == 0u) scale[(size_t)(i / 128u) * rows + row] = sc;
                    uint2 q;
                    q.x = cvt4_e4m3(f[c][0] * qi, f[c][1] * qi, f[c][2] * qi, f[c][3] * qi);
                    q.y = cvt4_e4m3(f[c][4] * qi, f[c][5] * qi, f[c][6] * qi, f[c][7] * qi);
                    *(uint2*)(xq + (size_t)row * feat + i) = q;
                }
            }
            if (MODE == 1 && i < feat) {
#pragma unroll
                for (int j = 0; j < 8; j++) amax_row = fmaxf(amax_row, fabsf(f[c][j]));
            }
        }
        if (MODE == 1) {
            amax_row = block_reduce(amax_row, true);
            const float sc = fmaxf(amax_row * (1.0f / 448.0f), 1e-12f), qi = 1.0f / sc;
            if (tid == 0) scale[row] = sc;
#pragma unroll
            for (int c = 0; c < RN_MAXV; c++) {
                const uint32_t i = ((uint32_t)c * 256u + tid) * 8u;
                if (i < feat) {
                    uint2 q = make_uint2(0u, 0u);
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        q.x |= e4m3_any(f[c][j] * qi, f[c][j]) << (8 * j);
                        q.y |= e4m3_any(f[c][4 + j] * qi, f[c][4 + j]) << (8 * j);
                    }
                    *(uint2*)(xq + (size_t)row * feat + i) = q;
                }
            }
        }
    }
}

int launch_rmsnorm(void* out, const void* x, const void* gamma, void* xq, float* scale, uint32_t rows, uint32_t feat,
                   uint32_t out_row0, float eps, uint32_t mode, hipStream_t st) {
    if (rows == 0 || feat == 0 || feat % 8u || feat > RN_MAXV * 256u * 8u) return PLOW_MOE_EINVAL;
    if (mode == 2u && feat % 128u) return PLOW_MOE_EINVAL;
    const uint32_t blocks = rows < 65535u ? rows : 65535u;
    if (mode == 2u) k_rmsnorm<2><<<blocks, 256, 0, st>>>((bf16_t*)out, (const bf16_t*)x, (const bf16_t*)gamma, (uint8_t*)xq, scale, rows, feat, out_row0, eps);
    else if (mode == 1u) k_rmsnorm<1><<<blocks, 256, 0, st>>>((bf16_t*)out, (const bf16_t*)x, (const bf16_t*)gamma, (uint8_t*)xq, scale, rows, feat, out_row0, eps);
    else k_rmsnorm<0><<<blocks, 256, 0, st>>>((bf16_t*)out, (const bf16_t*)x, (const bf16_t*)gamma, nullptr, nullptr, rows, feat, out_row0, eps);
    return 0;
}
