/* combine_body.h — the combine's device body (ops 87 / 43), shared by the library's kernels and by the
 * code object plowrt loads for its combine segments. */
#pragma once
#include "common.h"

/* out[t][h] = bf16(residual? + shared? + sum_{j<k} part[t*k+j][h]), f32, that order
 * (plow runtime/cpu/dev/golden/moe_route.c:130-147). Four consecutive h per thread. */
struct CombineArgs {
    bf16_t* out;
    const bf16_t* residual;
    const bf16_t* shared;
    const void* part;
    uint32_t H, k, T, part16;
};

/* KT > 0: the slot count is known at compile time, so all of a token's partial rows are requested
 * before the first is added (same order of additions); KT = 0: any k, one load at a time. */
template <uint32_t KT>
__device__ __forceinline__ void combine_body(const CombineArgs& a) {
    const uint32_t H4 = a.H / 4u;
    const size_t total = (size_t)a.T * H4;
    const uint32_t k = KT ? KT : a.k;
    for (size_t i = (size_t)blockIdx.x * 256u + threadIdx.x; i < total; i += (size_t)gridDim.x * 256u) {
        const uint32_t tok = (uint32_t)(i / H4), h = (uint32_t)(i % H4) * 4u;
        const size_t o = (size_t)tok * a.H + h;
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        uint2 rr = make_uint2(0u, 0u), rs = make_uint2(0u, 0u);
        if (a.residual) rr = *(const uint2*)(a.residual + o);
        if (a.shared) rs = *(const uint2*)(a.shared + o);
        if (KT && !a.part16) {
            float4 v[KT ? KT : 1u];
#pragma unroll
            for (uint32_t j = 0; j < KT; j++) {
                typedef float f4v __attribute__((ext_vector_type(4)));
                const f4v t = __builtin_nontemporal_load((const f4v*)((const float*)a.part + ((size_t)tok * KT + j) * a.H + h));
                v[j] = make_float4(t[0], t[1], t[2], t[3]);
            }
            if (a.residual) {
                acc[0] = __uint_as_float(rr.x << 16); acc[1] = __uint_as_float(rr.x & 0xFFFF0000u);
                acc[2] = __uint_as_float(rr.y << 16); acc[3] = __uint_as_float(rr.y & 0xFFFF0000u);
            }
            if (a.shared) {
                acc[0] += __uint_as_float(rs.x << 16); acc[1] += __uint_as_float(rs.x & 0xFFFF0000u);
                acc[2] += __uint_as_float(rs.y << 16); acc[3] += __uint_as_float(rs.y & 0xFFFF0000u);
            }
#pragma unroll
            for (uint32_t j = 0; j < KT; j++) { acc[0] += v[j].x; acc[1] += v[j].y; acc[2] += v[j].z; acc[3] += v[j].w; }
        } else {
            if (a.residual) {
                acc[0] = __uint_as_float(rr.x << 16); acc[1] = __uint_as_float(rr.x & 0xFFFF0000u);
                acc[2] = __uint_as_float(rr.y << 16); acc[3] = __uint_as_float(rr.y & 0xFFFF0000u);
            }
            if (a.shared) {
                acc[0] += __uint_as_float(rs.x << 16); acc[1] += __uint_as_float(rs.x & 0xFFFF0000u);
                acc[2] += __uint_as_float(rs.y << 16); acc[3] += __uint_as_float(rs.y & 0xFFFF0000u);
            }
            for (uint32_t j = 0; j < k; j++) {
                const size_t p = ((size_t)tok * k + j) * a.H + h;
                if (a.part16) {
                    const uint2 r = *(const uint2*)((const bf16_t*)a.part + p);
                    acc[0] += __uint_as_float(r.x << 16); acc[1] += __uint_as_float(r.x & 0xFFFF0000u);
                    acc[2] += __uint_as_float(r.y << 16); acc[3] += __uint_as_float(r.y & 0xFFFF0000u);
                } else {
                    const float4 v = *(const float4*)((const float*)a.part + p);
                    acc[0] += v.x; acc[1] += v.y; acc[2] += v.z; acc[3] += v.w;
                }
            }
        }
        uint2 w;
        w.x = (uint32_t)f2bf(acc[0]) | ((uint32_t)f2bf(acc[1]) << 16);
        w.y = (uint32_t)f2bf(acc[2]) | ((uint32_t)f2bf(acc[3]) << 16);
        *(uint2*)(a.out + o) = w;
    }
}
