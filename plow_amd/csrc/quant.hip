/* quant.hip — activation quantizers: 1x128 e4m3 (op 184) and per-row e4m3 (op 32).
 * Compiled with -ffp-contract=off: scale and reciprocal are separately rounded IEEE operations, as in
 * the reference (plow runtime/amd/op_gemm_common.h:2582-2621, runtime/cpu/dev/golden/fp8.c:9-30). */
#include "common.h"
#include "kernels.h"

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

/* One workgroup per row: amax over K, scale = max(amax / 448, 1e-12), q = e4m3(x * (1 / scale)). */
__global__ __launch_bounds__(256) void k_quant_row(uint8_t* __restrict__ xq, const bf16_t* __restrict__ x,
                                                   float* __restrict__ scale, uint32_t K) {
    __shared__ float red[4];
    const uint32_t row = blockIdx.x, tid = threadIdx.x;
    const bf16_t* xr = x + (size_t)row * K;
    float amax = 0.0f;
    for (uint32_t k = tid * 8u; k < K; k += 2048u) {
        const uint4 raw = *(const uint4*)(xr + k);
        const uint32_t v[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int j = 0; j < 4; j++)
            amax = fmaxf(amax, fmaxf(fabsf(__uint_as_float(v[j] << 16)), fabsf(__uint_as_float(v[j] & 0xFFFF0000u))));
    }
    amax = wave_max(amax);
    if ((tid & 63u) == 0) red[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float s = fmaxf(amax * (1.0f / 448.0f), 1e-12f);
    const float inv = 1.0f / s;
    if (tid == 0) scale[row] = s;
    for (uint32_t k = tid * 8u; k < K; k += 2048u) {
        const uint4 raw = *(const uint4*)(xr + k);
        const uint32_t v[4] = {raw.x, raw.y, raw.z, raw.w};
        float f[8];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            f[2 * j] = __uint_as_float(v[j] << 16);
            f[2 * j + 1] = __uint_as_float(v[j] & 0xFFFF0000u);
        }
        uint2 q;
        q.x = cvt4_e4m3(f[0] * inv, f[1] * inv, f[2] * inv, f[3] * inv);
        q.y = cvt4_e4m3(f[4] * inv, f[5] * inv, f[6] * inv, f[7] * inv);
        *(uint2*)(xq + (size_t)row * K + k) = q;
    }
}

int launch_quant_row(void* xq, const void* x, float* scale, uint32_t M, uint32_t K, hipStream_t st) {
    if (K % 8u || M == 0) return PLOW_MOE_EINVAL;
    k_quant_row<<<M, 256, 0, st>>>((uint8_t*)xq, (const bf16_t*)x, scale, K);
    return 0;
}
