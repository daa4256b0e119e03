/* experts_w8a8.hip — grouped expert GEMMs over aligned rows, block-fp8 weights (128x128 f32 scales)
 * times 1x128-scaled e4m3 activations (ops 85 / 86, arm 2 / 3).
 *
 * Arithmetic (plow runtime/amd/moe_pf_w8a8.h:368-379, :401-473): per 128-K block one fp8 x fp8
 * matrix product t accumulated in f32, promoted with acc = fmaf(t, a_scale[row][kb] * w_scale[nb][kb],
 * acc) in ascending kb. GLU: SwiGLU in f32, then per (row, 128 columns) amax = max(1e-10, |v|),
 * fs = amax / 448, fq = e4m3(v * (1 / fs)). DOWN: part[row_partidx[r]] = row_gate[r] * acc.
 *
 * WEIGHT-STREAMING KERNEL (few rows per expert; the decode shape). The job is to pull every weight
 * byte of every hit expert through the chip exactly once at HBM speed; the matrix cores are nearly
 * idle. One workgroup = (expert, 128 output channels), 8 waves, each wave 16 channels. The weights
 * are the A operand of v_mfma_f32_16x16x128_f8f6f4 (lane = (channel c, k-chunk q) holds 32 bytes of
 * one weight row) and go from global memory straight into the operand registers, DEPTH k-steps
 * ahead of their use; an expert's few activation rows are the B operand (lane = (row c, k-chunk q))
 * and come through the vector L1, since all 8 waves of the workgroup read the same rows. A lane's
 * 32 operand bytes are two 16-byte loads; k is permuted inside the 128 block (the same way for both
 * operands, which leaves the dot product unchanged) so that the four lanes of a row cover 64
 * contiguous bytes per load: lane q holds bytes [16q, 16q+16) and [64+16q, 64+16q+16).
 * The accumulator holds D[channel 4q+i][row c], so gate and up of one output element sit in the same
 * lane and the GLU epilogue needs no exchange; only the per-row amax crosses waves (through LDS).
 */
#include "common.h"
#include "kernels.h"
#include "tuning.h"

#include <cstdlib>
#include <cstring>

#define SK_WAVES 8u
#define SK_THREADS (SK_WAVES * WAVE)
#define SK_BN 128u /* output channels per workgroup */
#ifndef SK_DEPTH
#define SK_DEPTH 3 /* k-steps of weight loads in flight per wave */
#endif


__device__ __forceinline__ v4i ldg16(const uint8_t* p) { return *(const v4i*)p; }
/* weight bytes of the register forms: a row's 128-byte line is read as two 64-byte halves a k-step apart, so the
 * line has to stay cached between them (non-temporal loads here: DeepSeek-V3 decode DOWN 557 -> 630 us) */
__device__ __forceinline__ v4i ldg16_stream(const uint8_t* p) { return *(const v4i*)p; }

typedef short sk_bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void sk_atomic_add_bf16x2(bf16_t* p, float a, float b) {
    const uint32_t pk = (uint32_t)f2bf(a) | ((uint32_t)f2bf(b) << 16);
    __builtin_amdgcn_global_atomic_fadd_v2bf16((sk_bf16x2*)p, __builtin_bit_cast(sk_bf16x2, pk));
}

/* WIDE (DOWN, block mode only): a wave owns 32 channels as two 16-channel streams, a workgroup 256
 * channels; the short K loop of the down projection then amortises its prologue over twice the bytes.
 * NW: waves in the workgroup. The work item is always that of eight waves (128 channels, 256 WIDE);
 * with NW = 4 a wave runs the shares of logical waves wv and wv + 4 one after the other and keeps the
 * first share's GLU values until the amax over all 128 channels is known.
 * AQ (GLU, block mode): g.a holds the bf16 rows themselves and every 1x128 group is quantized where it
 * is loaded: amax floored at 1e-10, scale amax / 448, e4m3 of x * (1 / scale), the arithmetic of the
 * separate quantizer op, so the result equals quantizer + plain GLU bit for bit
 * (plow runtime/amd/moe_pf_w8a8.h:118-121, :255-283). */
template <int RT, bool GLU, int D, bool PC, bool WIDE, uint32_t NW = SK_WAVES, bool AQ = false, bool DET = false>
__device__ __forceinline__ void sk_body(const GroupW8A8& g, uint32_t e, uint32_t ct, uint32_t r0,
                                        uint32_t rb, uint32_t cnt, float* s_red) {
    static_assert(NW == 8u || NW == 4u, "eight waves, or four running two shares each");
    static_assert(!AQ || (GLU && !PC), "in-place activation quantization is a block-mode GLU form");
    constexpr uint32_t SUBS = SK_WAVES / NW;
    const uint32_t lane = threadIdx.x & 63u, wv = threadIdx.x >> 6, c = lane & 15u, q = lane >> 4;
    const uint32_t K = g.K, KB = K / 128u, N = g.N;
    constexpr bool TWO = GLU || WIDE; /* two weight streams per wave */
    /* block mode: {gate, up, down} tables, scale rows [N/128][KB]; per-channel mode: {gate_up fused,
     * down} tables (up rows follow the N gate rows), one f32 scale per weight row */
    const uint32_t wcols = PC ? 2u : 3u, sel0 = PC ? (GLU ? 0u : 1u) : (GLU ? 0u : 2u), sel1 = PC ? 0u : 1u;
    const uint8_t* const wbase0 = (const uint8_t*)(uintptr_t)g.wtab[(size_t)e * wcols + sel0];
    const uint8_t* const wbase1 = GLU ? (const uint8_t*)(uintptr_t)g.wtab[(size_t)e * wcols + sel1] : nullptr;
    const float* const sbase0 = (const float*)(uintptr_t)g.stab[(size_t)e * wcols + sel0];
    const float* const sbase1 = GLU ? (const float*)(uintptr_t)g.stab[(size_t)e * wcols + sel1] : nullptr;

    /* B operand rows of this lane, one per row tile */
    const uint8_t* ap[RT];
    const float* asp[RT];
    uint32_t as_stride;
    bool valid[RT];
    uint32_t rowidx[RT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
        const uint32_t off = rb + (uint32_t)rt * 16u + c;
        rowidx[rt] = r0 + off;
        valid[rt] = off < cnt;
        if (GLU) {
            const uint32_t tok = valid[rt] ? g.row_token[rowidx[rt]] : PLOW_EXPERT_UNUSED;
            valid[rt] = tok != PLOW_EXPERT_UNUSED && (g.T == 0u || tok < g.T);
            const uint32_t t = valid[rt] ? tok : 0u;
            ap[rt] = (const uint8_t*)g.a + ((size_t)t * K + 16u * q) * (AQ ? 2u : 1u);
            asp[rt] = AQ ? nullptr : g.a_scale + t;
        } else if (PC) {
            const uint32_t pi = valid[rt] ? g.row_partidx[rowidx[rt]] : PLOW_EXPERT_UNUSED;
            valid[rt] = pi != PLOW_EXPERT_UNUSED;
            const uint32_t r = valid[rt] ? rowidx[rt] : r0;
            ap[rt] = (const uint8_t*)g.a + (size_t)r * K + 16u * q;
            asp[rt] = g.a_scale + r;
        } else if (g.a_slots) { /* rows and scales stored by slot: [slot][K], [KB][a_slots] */
            const uint32_t pi = valid[rt] ? g.row_partidx[rowidx[rt]] : PLOW_EXPERT_UNUSED;
            valid[rt] = pi < g.a_slots;
            const uint32_t r = valid[rt] ? pi : 0u;
            ap[rt] = (const uint8_t*)g.a + (size_t)r * K + 16u * q;
            asp[rt] = g.a_scale + r;
        } else {
            const uint32_t pi = valid[rt] ? g.row_partidx[rowidx[rt]] : PLOW_EXPERT_UNUSED;
            valid[rt] = pi != PLOW_EXPERT_UNUSED;
            const uint32_t r = valid[rt] ? rowidx[rt] : r0;
            ap[rt] = (const uint8_t*)g.a + (size_t)r * K + 16u * q;
            asp[rt] = g.a_scale + (size_t)r * KB;
        }
    }
    as_stride = GLU ? g.pitch : (!PC && g.a_slots ? g.a_slots : 1u);

    float vkeep[SUBS][RT][4]; /* block-mode GLU: a share's values until the group's amax is known */
#pragma unroll
    for (uint32_t sub = 0; sub < SUBS; sub++) {
    const uint32_t lw = wv + NW * sub; /* the logical wave (of eight) whose share this is */
    const uint32_t ch = WIDE ? ct * 256u + lw * 32u + c : ct * SK_BN + lw * 16u + c; /* this lane's weight row */
    const uint8_t* w0 = wbase0 + (size_t)ch * K + 16u * q;
    const uint8_t* w1 = GLU ? wbase1 + (size_t)(ch + (PC ? N : 0u)) * K + 16u * q
                            : (WIDE ? w0 + (size_t)16u * K : nullptr);
    const float* s0 = sbase0 + (PC ? 0u : (WIDE ? (size_t)(ct * 2u + (lw >> 2)) * KB : (size_t)ct * KB));
    const float* s1 = GLU ? sbase1 + (PC ? (size_t)N : (size_t)ct * KB) : nullptr;

    v4i wa[D][2], wb[D][2], xa[D][RT][AQ ? 4 : 2];
    float xs[D][RT], sa[D], sb[D];
    auto issue = [&](int d, uint32_t kb) {
        const uint32_t ko = kb * 128u;
        wa[d][0] = ldg16_stream(w0 + ko);
        wa[d][1] = ldg16_stream(w0 + ko + 64u);
        if (TWO) {
            wb[d][0] = ldg16_stream(w1 + ko);
            wb[d][1] = ldg16_stream(w1 + ko + 64u);
        }
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
#pragma unroll
            for (int j = 0; j < (AQ ? 4 : 2); j++) xa[d][rt][j] = (v4i){0, 0, 0, 0};
            xs[d][rt] = 0.0f;
            if (valid[rt]) {
                if (AQ) { /* bf16 elements ko + 16q .. + 15 and ko + 64 + 16q .. + 15 */
                    xa[d][rt][0] = ldg16(ap[rt] + 2u * ko);
                    xa[d][rt][1] = ldg16(ap[rt] + 2u * ko + 16u);
                    xa[d][rt][2] = ldg16(ap[rt] + 2u * ko + 128u);
                    xa[d][rt][3] = ldg16(ap[rt] + 2u * ko + 144u);
                } else {
                    xa[d][rt][0] = ldg16(ap[rt] + ko);
                    xa[d][rt][1] = ldg16(ap[rt] + ko + 64u);
                    if (!PC) xs[d][rt] = asp[rt][(size_t)kb * as_stride];
                }
            }
        }
        if (!PC) {
            sa[d] = s0[kb];
            if (GLU) sb[d] = s1[kb];
        }
    };

    v4f acc0[RT], acc1[RT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
        acc0[rt] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
        acc1[rt] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
    }
#pragma unroll
    for (int d = 0; d < D; d++)
        if ((uint32_t)d < KB) issue(d, (uint32_t)d);
    for (uint32_t kb0 = 0; kb0 < KB; kb0 += D) {
#pragma unroll
        for (int d = 0; d < D; d++) {
            const uint32_t kb = kb0 + (uint32_t)d;
            if (kb < KB) {
                const v8i A0 = __builtin_shufflevector(wa[d][0], wa[d][1], 0, 1, 2, 3, 4, 5, 6, 7);
                v8i A1;
                if (TWO) A1 = __builtin_shufflevector(wb[d][0], wb[d][1], 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
                for (int rt = 0; rt < RT; rt++) {
                    v8i B;
                    float xsc;
                    if (AQ) {
                        /* the lane's 32 bf16 of the row's 128-group; the group's other lanes are q ^ 1, 2, 3 */
                        float f[32];
#pragma unroll
                        for (int j = 0; j < 4; j++)
#pragma unroll
                            for (int i = 0; i < 4; i++) {
                                const uint32_t w = (uint32_t)xa[d][rt][j][i];
                                f[8 * j + 2 * i] = __uint_as_float(w << 16);
                                f[8 * j + 2 * i + 1] = __uint_as_float(w & 0xFFFF0000u);
                            }
                        float amax = 1e-10f; /* the amax is floored, not the scale */
#pragma unroll
                        for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(f[i]));
                        amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
                        amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
                        xsc = amax * (1.0f / 448.0f);
                        const float inv = 1.0f / xsc;
#pragma unroll
                        for (int i = 0; i < 8; i++)
                            B[i] = (int)cvt4_e4m3(f[4 * i] * inv, f[4 * i + 1] * inv, f[4 * i + 2] * inv, f[4 * i + 3] * inv);
                    } else {
                        B = __builtin_shufflevector(xa[d][rt][0], xa[d][rt][1], 0, 1, 2, 3, 4, 5, 6, 7);
                        xsc = xs[d][rt];
                    }
                    if (PC) { /* scales are outside the K reduction: accumulate straight through */
                        acc0[rt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A0, B, acc0[rt], 0, 0, 0, 0, 0, 0);
                        if (GLU) acc1[rt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A1, B, acc1[rt], 0, 0, 0, 0, 0, 0);
                    } else {
                        const v4f z = {0.0f, 0.0f, 0.0f, 0.0f};
                        const v4f t0 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A0, B, z, 0, 0, 0, 0, 0, 0);
                        const float sc0 = xsc * sa[d];
#pragma unroll
                        for (int i = 0; i < 4; i++) acc0[rt][i] = fmaf(t0[i], sc0, acc0[rt][i]);
                        if (TWO) {
                            const v4f t1 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A1, B, z, 0, 0, 0, 0, 0, 0);
                            const float sc1 = xsc * (WIDE ? sa[d] : sb[d]);
#pragma unroll
                            for (int i = 0; i < 4; i++) acc1[rt][i] = fmaf(t1[i], sc1, acc1[rt][i]);
                        }
                    }
                }
                if (kb + D < KB) issue(d, kb + D);
            }
        }
    }

    /* ---- epilogue: lane holds channels ct*128 + lw*16 + 4q + i (i = 0..3) of row c ---- */
    const uint32_t col = WIDE ? ct * 256u + lw * 32u + 4u * q : ct * SK_BN + lw * 16u + 4u * q;
    if (PC) {
        /* per-channel arm (plow runtime/amd/op_moe.h:6655-6700): g = acc * (as * wsc[n]); GLU stores
         * bf16(act(g) * u) and zeroes pad rows, DOWN stores gate * acc, then * (as * wsc[h]) */
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
            const uint32_t off = rb + (uint32_t)rt * 16u + c;
            if (GLU) {
                if (!valid[rt]) {
                    if (off < ((cnt + PLOW_MPF_BM - 1u) / PLOW_MPF_BM) * PLOW_MPF_BM)
                        *(uint2*)((bf16_t*)g.out + (size_t)rowidx[rt] * N + col) = make_uint2(0u, 0u);
                    continue;
                }
                const float as = asp[rt][0];
                float o[4];
#pragma unroll
                for (int i = 0; i < 4; i++)
                    o[i] = moe_glu(acc0[rt][i] * (as * s0[col + i]), acc1[rt][i] * (as * s1[col + i]), g.act, g.f0, g.f1);
                uint2 pk;
                pk.x = (uint32_t)f2bf(o[0]) | ((uint32_t)f2bf(o[1]) << 16);
                pk.y = (uint32_t)f2bf(o[2]) | ((uint32_t)f2bf(o[3]) << 16);
                *(uint2*)((bf16_t*)g.out + (size_t)rowidx[rt] * N + col) = pk;
            } else {
                if (!valid[rt]) continue;
                const uint32_t pidx = g.row_partidx[rowidx[rt]];
                const float gate = g.row_gate[rowidx[rt]], as = asp[rt][0];
                float o[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    o[i] = gate * acc0[rt][i];
                    o[i] *= as * s0[col + i];
                }
                *(float4*)((float*)g.out + (size_t)pidx * N + col) = make_float4(o[0], o[1], o[2], o[3]);
            }
        }
    } else if (GLU && g.out_bf16) {
        /* bf16 intermediate (op 188): bf16(act(g) * u) for live rows, zeros for the other rows of the tile */
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
            const uint32_t off = rb + (uint32_t)rt * 16u + c;
            uint2 pk = make_uint2(0u, 0u);
            if (valid[rt]) {
                float o[4];
#pragma unroll
                for (int i = 0; i < 4; i++) o[i] = moe_glu(acc0[rt][i], acc1[rt][i], g.act, g.f0, g.f1);
                pk.x = (uint32_t)f2bf(o[0]) | ((uint32_t)f2bf(o[1]) << 16);
                pk.y = (uint32_t)f2bf(o[2]) | ((uint32_t)f2bf(o[3]) << 16);
            }
            if (off < ((cnt + PLOW_MPF_BM - 1u) / PLOW_MPF_BM) * PLOW_MPF_BM)
                *(uint2*)((bf16_t*)g.out + (size_t)rowidx[rt] * N + col) = pk;
        }
    } else if (GLU) {
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
            float m = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                vkeep[sub][rt][i] = moe_glu(acc0[rt][i], acc1[rt][i], g.act, g.f0, g.f1);
                m = fmaxf(m, fabsf(vkeep[sub][rt][i]));
            }
            m = fmaxf(m, __shfl_xor(m, 16, 64));
            m = fmaxf(m, __shfl_xor(m, 32, 64));
            if (q == 0) s_red[lw * 64u + (uint32_t)rt * 16u + c] = m;
        }
    } else {
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
            if (!valid[rt]) continue;
            const uint32_t pidx = g.row_partidx[rowidx[rt]];
            const float gate = g.row_gate[rowidx[rt]];
            const float y0 = gate * acc0[rt][0], y1 = gate * acc0[rt][1], y2 = gate * acc0[rt][2], y3 = gate * acc0[rt][3];
            if (DET && g.det_k) { /* order-independent: fixed-point f64 atomics into the token's accumulator row */
                double* arow = (double*)g.out + (size_t)(pidx / g.det_k) * N + col;
                det_add(arow, y0), det_add(arow + 1, y1), det_add(arow + 2, y2), det_add(arow + 3, y3);
                if (WIDE) {
                    det_add(arow + 16, gate * acc1[rt][0]), det_add(arow + 17, gate * acc1[rt][1]);
                    det_add(arow + 18, gate * acc1[rt][2]), det_add(arow + 19, gate * acc1[rt][3]);
                }
                continue;
            }
            if (g.acc_topk) { /* add into the layer output row of the slot's token, packed bf16 atomics */
                bf16_t* orow = (bf16_t*)g.out + (size_t)(pidx / g.acc_topk) * N + col;
                sk_atomic_add_bf16x2(orow, y0, y1);
                sk_atomic_add_bf16x2(orow + 2, y2, y3);
                if (WIDE) {
                    sk_atomic_add_bf16x2(orow + 16, gate * acc1[rt][0], gate * acc1[rt][1]);
                    sk_atomic_add_bf16x2(orow + 18, gate * acc1[rt][2], gate * acc1[rt][3]);
                }
                continue;
            }
            if (g.part16) {
                uint2 o;
                o.x = (uint32_t)f2bf(y0) | ((uint32_t)f2bf(y1) << 16);
                o.y = (uint32_t)f2bf(y2) | ((uint32_t)f2bf(y3) << 16);
                *(uint2*)((bf16_t*)g.out + (size_t)pidx * N + col) = o;
            } else {
                *(float4*)((float*)g.out + (size_t)pidx * N + col) = make_float4(y0, y1, y2, y3);
            }
            if (WIDE) { /* the second 16-channel stream */
                const float z0 = gate * acc1[rt][0], z1 = gate * acc1[rt][1], z2 = gate * acc1[rt][2], z3 = gate * acc1[rt][3];
                if (g.part16) {
                    uint2 o;
                    o.x = (uint32_t)f2bf(z0) | ((uint32_t)f2bf(z1) << 16);
                    o.y = (uint32_t)f2bf(z2) | ((uint32_t)f2bf(z3) << 16);
                    *(uint2*)((bf16_t*)g.out + (size_t)pidx * N + col + 16u) = o;
                } else {
                    *(float4*)((float*)g.out + (size_t)pidx * N + col + 16u) = make_float4(z0, z1, z2, z3);
                }
            }
        }
    }
    } /* sub */

    if (GLU && !PC && !g.out_bf16) {
        __syncthreads();
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
            float amax = 1e-10f;
#pragma unroll
            for (uint32_t w = 0; w < SK_WAVES; w++) amax = fmaxf(amax, s_red[w * 64u + (uint32_t)rt * 16u + c]);
            const float s = amax * (1.0f / 448.0f);
            const float inv = 1.0f / s;
            if (valid[rt]) {
#pragma unroll
                for (uint32_t sub = 0; sub < SUBS; sub++) {
                    const uint32_t col = ct * SK_BN + (wv + NW * sub) * 16u + 4u * q;
                    const float* v = vkeep[sub][rt];
                    *(uint32_t*)((uint8_t*)g.out + (size_t)rowidx[rt] * N + col) = cvt4_e4m3(v[0] * inv, v[1] * inv, v[2] * inv, v[3] * inv);
                }
                if (wv == 0 && q == 0) g.out_scale[(size_t)rowidx[rt] * (N / 128u) + ct] = s;
            }
        }
        __syncthreads(); /* s_red is reused by the next row block */
    }
}

/* DET: the deterministic accumulate epilogue (g.det_k) is compiled only into the launches that ask for
 * it; in the plain kernel its f64 address arithmetic costs the registers of a fourth wave per SIMD */
template <bool GLU, int D, bool PC, bool WIDE = false, bool AQ = false, bool DET = false>
__global__ __launch_bounds__(SK_THREADS) void k_group_w8a8_stream(GroupW8A8 g) {
    __shared__ float s_red[SK_WAVES * 64u];
    const uint32_t tiles = g.N / (WIDE ? 256u : SK_BN);
    /* highest expert id first: a folded shared expert (id E-1, every token routed to it) is the one
     * segment that needs several passes, so it must start early instead of forming the tail */
    const uint32_t e = g.E - 1u - blockIdx.x / tiles, ct = blockIdx.x % tiles;
    const uint32_t cnt = (uint32_t)g.meta[g.E + e];
    if (cnt == 0u || !form_is_mine(g)) return;
    const uint32_t r0 = (uint32_t)g.meta[e];
    const bool bf16_mid = GLU && (PC || g.out_bf16); /* the GLU owns every row of its 64-row tiles */
    const uint32_t padded = ((cnt + PLOW_MPF_BM - 1u) / PLOW_MPF_BM) * PLOW_MPF_BM;
    bool resident = g.wtab[(size_t)e * (PC ? 2u : 3u) + (PC ? (GLU ? 0u : 1u) : (GLU ? 0u : 2u))] != 0ull;
    if (GLU && !PC && g.out_bf16) resident = resident && g.wtab[(size_t)e * 3u + 1u] != 0ull;
    if (!resident) {
        if (GLU && !PC && g.out_bf16) /* op 188 zeroes the rows of an expert it cannot compute */
            for (uint32_t i = threadIdx.x; i < padded * (SK_BN / 4u); i += SK_THREADS)
                *(uint2*)((bf16_t*)g.out + (size_t)(r0 + i / (SK_BN / 4u)) * g.N + ct * SK_BN + (i % (SK_BN / 4u)) * 4u) = make_uint2(0u, 0u);
        return;
    }
    /* 16 rows a pass; an expert with more rows streams its weights once per pass (the tiled
     * kernel, not this one, is the tool for many rows per expert) */
    for (uint32_t rb = 0; rb < cnt; rb += 16u) sk_body<1, GLU, D, PC, WIDE, SK_WAVES, AQ, DET>(g, e, ct, r0, rb, cnt, s_red);
    if (bf16_mid) {
        /* a GLU with a bf16 intermediate zeroes the pad rows of its 64-row tile (the partial 16-row pass
         * above did its own); the row quantizer that follows reads every aligned row */
        const uint32_t first = ((cnt + 15u) / 16u) * 16u;
        for (uint32_t i = threadIdx.x; i < (padded - first) * (SK_BN / 4u); i += SK_THREADS) {
            const uint32_t r = r0 + first + i / (SK_BN / 4u), col = ct * SK_BN + (i % (SK_BN / 4u)) * 4u;
            *(uint2*)((bf16_t*)g.out + (size_t)r * g.N + col) = make_uint2(0u, 0u);
        }
    }
}


/* ---------------------------------------------------------------------------------------------------
 * GLU, block mode, second form: every load goes global -> LDS directly (global_load_lds_dwordx4) with
 * 8 consecutive lanes on one 128-byte line, into a ring that is PRIVATE to the wave, and the operands
 * are read back from LDS in the matrix layout. The "lane = weight row" loads of the first form cost
 * the vector memory pipeline four times as much per instruction, which shows at the gate|up shape
 * (two matrices, rows 7 KB apart). No workgroup barrier in the K loop: a wave waits for its own loads
 * (s_waitcnt vmcnt) and nobody else's. Pad rows read the pass's first row and carry a zero scale.
 * LDS pieces are swizzled on the global side: piece p of row r holds global piece p ^ lds_swz8(r). */
#ifndef SD_STAGES
#define SD_STAGES 3
#endif
#define SD_NLOAD 7 /* per wave and 128-k block: 1 scale, 2 activation-row, 4 weight-row direct loads */
struct SdSlot {
    uint8_t w[32u * 128u]; /* rows 0..15 gate, 16..31 up of this wave's 16 channels */
    uint8_t x[16u * 128u]; /* the pass's 16 activation rows */
    float xs[64];          /* their scales (lanes 16..63 write copies) */
};
struct SdLds {
    SdSlot ring[SK_WAVES][SD_STAGES];
    float red[SK_WAVES * 16u];
    float wsc[2][128]; /* the tile's weight block scales (gate, up), all of K: K <= 16384 */
};
typedef __attribute__((address_space(3))) void sd_lds_void;
__device__ __forceinline__ uint32_t sd_lds_off(const void* p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}
template <uint32_t OFF>
__device__ __forceinline__ v4i sd_read16(uint32_t addr) {
    v4i r;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF) : "memory");
    return r;
}
__device__ __forceinline__ float sd_read4(uint32_t addr) {
    float r;
    asm volatile("ds_read_b32 %0, %1" : "=v"(r) : "v"(addr) : "memory");
    return r;
}
#define SD_WAIT_VM(n) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(n) : "memory")

__global__ __launch_bounds__(SK_THREADS) void k_group_glu_w8a8_dma(GroupW8A8 g) {
    extern __shared__ __attribute__((aligned(16))) uint8_t sd_raw[];
    SdLds& L = *(SdLds*)sd_raw;
    const uint32_t tiles = g.N / SK_BN;
    const uint32_t e = g.E - 1u - blockIdx.x / tiles, ct = blockIdx.x % tiles; /* heavy (folded shared) expert first */
    /* A workgroup fills its CU alone, so every trip to memory before its first block is time the CU streams
     * nothing. Everything that depends on the expert alone is asked for at once, before the first of it is
     * used (count, row offset, weight and scale pointers: one trip) ... */
    const uint32_t cnt = (uint32_t)g.meta[g.E + e];
    const uint32_t r0 = (uint32_t)g.meta[e];
    const uint64_t wp0 = g.wtab[(size_t)e * 3u], wp1 = g.wtab[(size_t)e * 3u + 1u];
    const uint64_t sp0 = g.stab[(size_t)e * 3u], sp1 = g.stab[(size_t)e * 3u + 1u];
    const bool mine = form_is_mine(g);
    asm volatile("" ::"s"(r0), "s"(wp0), "s"(wp1), "s"(sp0), "s"(sp1)); /* the loads stay above the branch */
    if (cnt == 0u || !mine) return;
    const uint32_t padded = ((cnt + PLOW_MPF_BM - 1u) / PLOW_MPF_BM) * PLOW_MPF_BM;
    if (wp0 == 0ull || (g.out_bf16 && wp1 == 0ull)) { /* not resident; the bf16 form zeroes what it cannot compute */
        if (g.out_bf16)
            for (uint32_t i = threadIdx.x; i < padded * (SK_BN / 4u); i += SK_THREADS)
                *(uint2*)((bf16_t*)g.out + (size_t)(r0 + i / (SK_BN / 4u)) * g.N + ct * SK_BN + (i % (SK_BN / 4u)) * 4u) = make_uint2(0u, 0u);
        return;
    }
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wv = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint32_t c = lane & 15u, q = lane >> 4; /* operand layout: row / channel c, 32-byte chunk q */
    const uint32_t lr = lane >> 3, p = lane & 7u; /* load layout: row lr of a group of 8, piece p */
    const uint32_t K = g.K, KB = K / 128u, N = g.N;
    const uint32_t chw = ct * SK_BN + wv * 16u;   /* this wave's first channel */
    const float* s0 = (const float*)(uintptr_t)sp0 + (size_t)ct * KB;
    const float* s1 = (const float*)(uintptr_t)sp1 + (size_t)ct * KB;
    /* ... and what depends on those — the tile's weight block scales and the tokens of the first pass's 16
     * rows (lane l: row l & 15) — in a second trip, together */
    const uint32_t tok_first = (lane & 15u) < cnt ? g.row_token[r0 + (lane & 15u)] : PLOW_EXPERT_UNUSED;

    /* weight rows: load j covers LDS rows 8j .. 8j + 7 (j < 2 gate, else up) */
    const uint8_t* wsrc[4];
#pragma unroll
    for (uint32_t j = 0; j < 4u; j++) {
        const uint32_t R = 8u * j + lr;
        const uint8_t* base = (const uint8_t*)(uintptr_t)(j < 2u ? wp0 : wp1);
        wsrc[j] = base + (size_t)(chw + (R & 15u)) * K + ((p ^ lds_swz8(R)) << 4);
    }
    /* the weight block scales go to LDS once: an ordinary load inside the K loop would make the
     * compiler wait for every outstanding load of the ring */
    for (uint32_t i = threadIdx.x; i < KB; i += SK_THREADS) {
        L.wsc[0][i] = s0[i];
        L.wsc[1][i] = s1[i];
    }
    __syncthreads();
    const uint32_t wsc_base = sd_lds_off(&L.wsc[0][0]);
    SdSlot* const ring = L.ring[wv];
    const uint32_t swz = lds_swz8(c);
    const uint32_t o_lo = c * 128u + (((2u * q) ^ swz) << 4), o_hi = c * 128u + (((2u * q + 1u) ^ swz) << 4);

    for (uint32_t rb = 0; rb < cnt; rb += 16u) {
        /* the token of row `idx` of the pass (PLOW_EXPERT_UNUSED past the expert's rows): the first pass has
         * them in registers already, a later pass (an expert with more than 16 rows) reads them now */
        auto tok_at = [&](uint32_t idx) -> uint32_t {
            if (rb == 0u) return (uint32_t)__shfl((int)tok_first, (int)idx, 64);
            return rb + idx < cnt ? g.row_token[r0 + rb + idx] : PLOW_EXPERT_UNUSED;
        };
        /* activation rows of the pass: load i covers rows 8i .. 8i + 7 */
        uint32_t tok0 = tok_at(0u);
        if (g.T != 0u && tok0 >= g.T) tok0 = 0u; /* any readable row: its scale is zeroed below */
        const uint8_t* xsrc[2];
#pragma unroll
        for (uint32_t i = 0; i < 2u; i++) {
            const uint32_t row = 8u * i + lr;
            uint32_t tok = tok_at(row);
            if (tok == PLOW_EXPERT_UNUSED || (g.T != 0u && tok >= g.T)) tok = tok0;
            xsrc[i] = (const uint8_t*)g.a + (size_t)tok * K + ((p ^ lds_swz8(row)) << 4);
        }
        const float* ssrc;
        uint32_t sstep;
        const uint32_t tok_c = tok_at(c);
        const bool valid = tok_c != PLOW_EXPERT_UNUSED && (g.T == 0u || tok_c < g.T);
        ssrc = valid ? g.a_scale + tok_c : (const float*)(g.meta + 2u * g.E); /* tilep[0] = 0 */
        sstep = valid ? g.pitch : 0u;
        auto issue = [&](uint32_t kb) {
            SdSlot* s = ring + kb % SD_STAGES;
            __builtin_amdgcn_global_load_lds((const void*)(ssrc + (size_t)kb * sstep), (sd_lds_void*)&s->xs[0], 4, 0, 0);
#pragma unroll
            for (uint32_t i = 0; i < 2u; i++)
                __builtin_amdgcn_global_load_lds((const void*)(xsrc[i] + (size_t)kb * 128u),
                                                 (sd_lds_void*)&s->x[8u * i * 128u], 16, 0, 0);
#pragma unroll
            for (uint32_t j = 0; j < 4u; j++)
                __builtin_amdgcn_global_load_lds((const void*)(wsrc[j] + (size_t)kb * 128u),
                                                 (sd_lds_void*)&s->w[8u * j * 128u], 16, 0, LOAD_NT);
        };
        v4f acc0 = {0.0f, 0.0f, 0.0f, 0.0f}, acc1 = acc0;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); /* the row maps above are loaded; the count starts at zero */
        issue(0);
        if (KB > 1u) issue(1);
        for (uint32_t kb = 0; kb < KB; kb++) {
            /* loads return in order: block kb has landed once at most block kb + 1's are outstanding */
            if (kb + 1u < KB) SD_WAIT_VM(SD_NLOAD); else SD_WAIT_VM(0);
            const uint32_t base = sd_lds_off(ring + kb % SD_STAGES);
            v4i a0l = sd_read16<0>(base + o_lo), a0h = sd_read16<0>(base + o_hi);
            v4i a1l = sd_read16<2048>(base + o_lo), a1h = sd_read16<2048>(base + o_hi);
            v4i bl = sd_read16<4096>(base + o_lo), bh = sd_read16<4096>(base + o_hi);
            float xs = sd_read4(base + 6144u + c * 4u);
            float sa = sd_read4(wsc_base + kb * 4u), sb = sd_read4(wsc_base + 512u + kb * 4u);
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a0l), "+v"(a0h), "+v"(a1l), "+v"(a1h));
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(bl), "+v"(bh), "+v"(xs), "+v"(sa), "+v"(sb));
            /* block kb - 1's slot is free (its reads were waited for one iteration ago): refill it */
            if (kb + 2u < KB) issue(kb + 2u);
            const v8i A0 = __builtin_shufflevector(a0l, a0h, 0, 1, 2, 3, 4, 5, 6, 7);
            const v8i A1 = __builtin_shufflevector(a1l, a1h, 0, 1, 2, 3, 4, 5, 6, 7);
            const v8i B = __builtin_shufflevector(bl, bh, 0, 1, 2, 3, 4, 5, 6, 7);
            const v4f z = {0.0f, 0.0f, 0.0f, 0.0f};
            const v4f t0 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A0, B, z, 0, 0, 0, 0, 0, 0);
            const v4f t1 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A1, B, z, 0, 0, 0, 0, 0, 0);
            const float sc0 = xs * sa, sc1 = xs * sb;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                acc0[i] = fmaf(t0[i], sc0, acc0[i]);
                acc1[i] = fmaf(t1[i], sc1, acc1[i]);
            }
        }
        /* ---- epilogue: lane holds channels chw + 4q + i (i = 0..3) of row rb + c ---- */
        if (g.out_bf16) { /* bf16 intermediate: live rows get bf16(act(g) * u), the tile's other rows zeros */
            uint2 pk = make_uint2(0u, 0u);
            if (valid) {
                float o[4];
#pragma unroll
                for (int i = 0; i < 4; i++) o[i] = moe_glu(acc0[i], acc1[i], g.act, g.f0, g.f1);
                pk.x = (uint32_t)f2bf(o[0]) | ((uint32_t)f2bf(o[1]) << 16);
                pk.y = (uint32_t)f2bf(o[2]) | ((uint32_t)f2bf(o[3]) << 16);
            }
            if (rb + c < padded) *(uint2*)((bf16_t*)g.out + (size_t)(r0 + rb + c) * N + chw + 4u * q) = pk;
            continue;
        }
        float v[4], m = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            v[i] = moe_glu(acc0[i], acc1[i], g.act, g.f0, g.f1);
            m = fmaxf(m, fabsf(v[i]));
        }
        m = fmaxf(m, __shfl_xor(m, 16, 64));
        m = fmaxf(m, __shfl_xor(m, 32, 64));
        if (q == 0) L.red[wv * 16u + c] = m;
        __syncthreads();
        float amax = 1e-10f;
#pragma unroll
        for (uint32_t w = 0; w < SK_WAVES; w++) amax = fmaxf(amax, L.red[w * 16u + c]);
        const float s = amax * (1.0f / 448.0f), inv = 1.0f / s;
        if (valid) {
            const uint32_t row = r0 + rb + c, col = chw + 4u * q;
            *(uint32_t*)((uint8_t*)g.out + (size_t)row * N + col) = cvt4_e4m3(v[0] * inv, v[1] * inv, v[2] * inv, v[3] * inv);
            if (wv == 0 && q == 0) g.out_scale[(size_t)row * (N / 128u) + ct] = s;
        }
        __syncthreads(); /* L.red is reused by the next pass */
    }
    if (g.out_bf16) { /* pad rows of the last 64-row tile that no 16-row pass covered */
        const uint32_t first = ((cnt + 15u) / 16u) * 16u;
        for (uint32_t i = threadIdx.x; i < (padded - first) * (SK_BN / 4u); i += SK_THREADS)
            *(uint2*)((bf16_t*)g.out + (size_t)(r0 + first + i / (SK_BN / 4u)) * N + ct * SK_BN + (i % (SK_BN / 4u)) * 4u) = make_uint2(0u, 0u);
    }
}

/* DOWN, block mode, the same direct-to-LDS form: a wave owns 32 output channels (two 16-row operands that share
 * the activation operand and the weight block scale) and a private ring of the same slots; the weight rows are
 * read once, whole 128-byte lines per row and block, with non-temporal loads (the register form reads a line as
 * two halves a k-step apart and has to keep it cached: 5.7 TB/s against the 6.6 of the GLU above). Four waves
 * and 128 channels per workgroup: 77 KB of LDS, so a CU holds two workgroups and one's set-up trips to memory
 * (count and pointers, then row maps and block scales) pass under the other's stream. e4m3 rows by aligned row;
 * f32 or bf16 partials by row_partidx, or the deterministic accumulate. Rows past the expert's count read its first row with a
 * zero scale; a row whose slot is unused is computed and not stored. */
#define SDD_WAVES 4u
struct SddLds {
    SdSlot ring[SDD_WAVES][SD_STAGES];
    float wsc[128]; /* the tile's weight block scales, all of K: K <= 16384 */
};
__global__ __launch_bounds__(SDD_WAVES* WAVE) void k_group_down_w8a8_dma(GroupW8A8 g) {
    extern __shared__ __attribute__((aligned(16))) uint8_t sdd_raw[];
    SddLds& L = *(SddLds*)sdd_raw;
    const uint32_t tiles = g.N / 128u;
    const uint32_t e = g.E - 1u - blockIdx.x / tiles, ct = blockIdx.x % tiles; /* heavy (folded shared) expert first */
    const uint32_t cnt = (uint32_t)g.meta[g.E + e];
    const uint32_t r0 = (uint32_t)g.meta[e];
    const uint64_t wp = g.wtab[(size_t)e * 3u + 2u], sp = g.stab[(size_t)e * 3u + 2u];
    const bool mine = form_is_mine(g);
    asm volatile("" ::"s"(r0), "s"(wp), "s"(sp)); /* the loads stay above the branch */
    if (cnt == 0u || wp == 0ull || !mine) return;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wv = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint32_t c = lane & 15u, q = lane >> 4; /* operand layout: row / channel c, 32-byte chunk q */
    const uint32_t lr = lane >> 3, p = lane & 7u; /* load layout: row lr of a group of 8, piece p */
    const uint32_t K = g.K, KB = K / 128u, N = g.N;
    const uint32_t chw = ct * 128u + wv * 32u; /* this wave's first channel */
    const float* const sc = (const float*)(uintptr_t)sp + (size_t)ct * KB;
    /* weight rows: load j covers LDS rows 8j .. 8j + 7 = channels chw + 8j .. */
    const uint8_t* wsrc[4];
#pragma unroll
    for (uint32_t j = 0; j < 4u; j++) {
        const uint32_t R = 8u * j + lr;
        wsrc[j] = (const uint8_t*)(uintptr_t)wp + (size_t)(chw + R) * K + ((p ^ lds_swz8(R)) << 4);
    }
    for (uint32_t i = threadIdx.x; i < KB; i += SDD_WAVES * WAVE) L.wsc[i] = sc[i];
    __syncthreads();
    const uint32_t wsc_base = sd_lds_off(&L.wsc[0]);
    SdSlot* const ring = L.ring[wv];
    const uint32_t swz = lds_swz8(c);
    const uint32_t o_lo = c * 128u + (((2u * q) ^ swz) << 4), o_hi = c * 128u + (((2u * q + 1u) ^ swz) << 4);

    for (uint32_t rb = 0; rb < cnt; rb += 16u) {
        /* activation rows of the pass: load i covers rows 8i .. 8i + 7; aligned rows need no map */
        const uint8_t* xsrc[2];
#pragma unroll
        for (uint32_t i = 0; i < 2u; i++) {
            const uint32_t idx = 8u * i + lr;
            const uint32_t row = rb + idx < cnt ? r0 + rb + idx : r0;
            xsrc[i] = (const uint8_t*)g.a + (size_t)row * K + ((p ^ lds_swz8(idx)) << 4);
        }
        const bool live = rb + c < cnt;
        const float* const ssrc = live ? g.a_scale + (size_t)(r0 + rb + c) * KB : (const float*)(g.meta + 2u * g.E); /* tilep[0] = 0 */
        const uint32_t sstep = live ? 1u : 0u;
        uint32_t pidx = live ? g.row_partidx[r0 + rb + c] : PLOW_EXPERT_UNUSED;
        float gate = live ? g.row_gate[r0 + rb + c] : 0.0f;
        auto issue = [&](uint32_t kb) {
            SdSlot* s = ring + kb % SD_STAGES;
            __builtin_amdgcn_global_load_lds((const void*)(ssrc + (size_t)kb * sstep), (sd_lds_void*)&s->xs[0], 4, 0, 0);
#pragma unroll
            for (uint32_t i = 0; i < 2u; i++)
                __builtin_amdgcn_global_load_lds((const void*)(xsrc[i] + (size_t)kb * 128u),
                                                 (sd_lds_void*)&s->x[8u * i * 128u], 16, 0, 0);
#pragma unroll
            for (uint32_t j = 0; j < 4u; j++)
                __builtin_amdgcn_global_load_lds((const void*)(wsrc[j] + (size_t)kb * 128u),
                                                 (sd_lds_void*)&s->w[8u * j * 128u], 16, 0, LOAD_NT);
        };
        v4f acc0 = {0.0f, 0.0f, 0.0f, 0.0f}, acc1 = acc0;
        asm volatile("s_waitcnt vmcnt(0)" : "+v"(pidx), "+v"(gate) : : "memory"); /* the row maps are loaded; the count starts at zero */
        issue(0);
        if (KB > 1u) issue(1);
        for (uint32_t kb = 0; kb < KB; kb++) {
            /* loads return in order: block kb has landed once at most block kb + 1's are outstanding */
            if (kb + 1u < KB) SD_WAIT_VM(SD_NLOAD); else SD_WAIT_VM(0);
            const uint32_t base = sd_lds_off(ring + kb % SD_STAGES);
            v4i a0l = sd_read16<0>(base + o_lo), a0h = sd_read16<0>(base + o_hi);
            v4i a1l = sd_read16<2048>(base + o_lo), a1h = sd_read16<2048>(base + o_hi);
            v4i bl = sd_read16<4096>(base + o_lo), bh = sd_read16<4096>(base + o_hi);
            float xs = sd_read4(base + 6144u + c * 4u);
            float sa = sd_read4(wsc_base + kb * 4u);
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a0l), "+v"(a0h), "+v"(a1l), "+v"(a1h));
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(bl), "+v"(bh), "+v"(xs), "+v"(sa));
            /* block kb - 1's slot is free (its reads were waited for one iteration ago): refill it */
            if (kb + 2u < KB) issue(kb + 2u);
            const v8i A0 = __builtin_shufflevector(a0l, a0h, 0, 1, 2, 3, 4, 5, 6, 7);
            const v8i A1 = __builtin_shufflevector(a1l, a1h, 0, 1, 2, 3, 4, 5, 6, 7);
            const v8i B = __builtin_shufflevector(bl, bh, 0, 1, 2, 3, 4, 5, 6, 7);
            const v4f z = {0.0f, 0.0f, 0.0f, 0.0f};
            const v4f t0 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A0, B, z, 0, 0, 0, 0, 0, 0);
            const v4f t1 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A1, B, z, 0, 0, 0, 0, 0, 0);
            const float s01 = xs * sa;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                acc0[i] = fmaf(t0[i], s01, acc0[i]);
                acc1[i] = fmaf(t1[i], s01, acc1[i]);
            }
        }
        /* ---- epilogue: lane holds channels chw + 4q + i and chw + 16 + 4q + i (i = 0..3) of row rb + c ---- */
        if (pidx == PLOW_EXPERT_UNUSED) continue;
        const size_t o = (size_t)pidx * N + chw + 4u * q;
        const float y0 = gate * acc0[0], y1 = gate * acc0[1], y2 = gate * acc0[2], y3 = gate * acc0[3];
        const float z0 = gate * acc1[0], z1 = gate * acc1[1], z2 = gate * acc1[2], z3 = gate * acc1[3];
        if (g.det_k) { /* order-independent: fixed-point f64 atomics into the token's accumulator row */
            double* const arow = (double*)g.out + (size_t)(pidx / g.det_k) * N + chw + 4u * q;
            det_add(arow, y0), det_add(arow + 1, y1), det_add(arow + 2, y2), det_add(arow + 3, y3);
            det_add(arow + 16, z0), det_add(arow + 17, z1), det_add(arow + 18, z2), det_add(arow + 19, z3);
            continue;
        }
        if (g.part16) {
            uint2 a, b;
            a.x = (uint32_t)f2bf(y0) | ((uint32_t)f2bf(y1) << 16), a.y = (uint32_t)f2bf(y2) | ((uint32_t)f2bf(y3) << 16);
            b.x = (uint32_t)f2bf(z0) | ((uint32_t)f2bf(z1) << 16), b.y = (uint32_t)f2bf(z2) | ((uint32_t)f2bf(z3) << 16);
            *(uint2*)((bf16_t*)g.out + o) = a;
            *(uint2*)((bf16_t*)g.out + o + 16u) = b;
        } else {
            *(float4*)((float*)g.out + o) = make_float4(y0, y1, y2, y3);
            *(float4*)((float*)g.out + o + 16u) = make_float4(z0, z1, z2, z3);
        }
    }
}

/* dynamic-LDS limit of the direct-to-LDS form, once per device (plow_moe_device_setup) */
int plow_moe_w8a8_setup() {
    return hipFuncSetAttribute((const void*)k_group_glu_w8a8_dma, hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)sizeof(SdLds)) == hipSuccess &&
           hipFuncSetAttribute((const void*)k_group_down_w8a8_dma, hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)sizeof(SddLds)) == hipSuccess ? 0 : PLOW_MOE_EDEVICE;
}

/* The device-side choice between the streaming and the tiled form of a grouped op whose caller states no row
 * count: one workgroup adds up the experts' row counts. */
__global__ __launch_bounds__(256) void k_pick_form(uint32_t* word, const int32_t* meta, uint32_t E) {
    __shared__ uint32_t part[4];
    uint32_t s = 0;
    for (uint32_t e = threadIdx.x; e < E; e += 256u) s += (uint32_t)meta[E + e];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
    if ((threadIdx.x & 63u) == 0u) part[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0u) *word = (part[0] + part[1] + part[2] + part[3] >= 16u * E) ? 1u : 0u;
}
int launch_pick_form(uint32_t* word, const int32_t* meta, uint32_t E, hipStream_t st) {
    if (!word || !meta || !E) return PLOW_MOE_EINVAL;
    k_pick_form<<<1, 256, 0, st>>>(word, meta, E);
    return 0;
}

static int check_w8a8(const GroupW8A8& g) {
    if (g.N == 0 || g.K == 0 || g.E == 0) return PLOW_MOE_EINVAL;
    if (g.N % SK_BN || g.K % 128u) return PLOW_MOE_EINVAL;
    if ((uint64_t)g.E * (g.N / SK_BN) > 0x7FFFFFFFull) return PLOW_MOE_EINVAL;
    return 0;
}

int launch_group_glu_w8a8(const GroupW8A8& g, hipStream_t st) {
    const int rc = check_w8a8(g);
    if (rc) return rc;
    const dim3 grid(g.E * (g.N / SK_BN));
    if (g.per_channel) { k_group_w8a8_stream<true, 3, true><<<grid, SK_THREADS, 0, st>>>(g); return 0; }
    const PlowMoeTuning& tune = plow_moe_tuning();
    if (g.out_bf16 && tune.sk_glu_regs) { /* bf16 intermediate on the register form */
        k_group_w8a8_stream<true, 3, false><<<grid, SK_THREADS, 0, st>>>(g);
        return 0;
    }
    if (g.a_bf16) { /* bf16 rows, quantized where they are loaded */
        k_group_w8a8_stream<true, 3, false, false, true><<<grid, SK_THREADS, 0, st>>>(g);
        return 0;
    }
    /* the direct-to-LDS form keeps the block scales of all of K in LDS (K <= 16384); longer rows take the
     * register form, which reads them as it goes */
    if (!tune.sk_glu_regs && g.K <= 16384u) {
        k_group_glu_w8a8_dma<<<grid, SK_THREADS, sizeof(SdLds), st>>>(g);
        return 0;
    }
    switch (plow_moe_tuning().sk_depth) {
    case 2: k_group_w8a8_stream<true, 2, false><<<grid, SK_THREADS, 0, st>>>(g); break;
    case 4: k_group_w8a8_stream<true, 4, false><<<grid, SK_THREADS, 0, st>>>(g); break;
    default: k_group_w8a8_stream<true, 3, false><<<grid, SK_THREADS, 0, st>>>(g); break;
    }
    return 0;
}

int launch_group_down_w8a8(const GroupW8A8& g, hipStream_t st) {
    const int rc = check_w8a8(g);
    if (rc) return rc;
    const dim3 grid(g.E * (g.N / SK_BN));
    if (g.per_channel) { k_group_w8a8_stream<false, 3, true><<<grid, SK_THREADS, 0, st>>>(g); return 0; }
    const bool dma_ok = !g.acc_topk && !g.a_slots && !g.a_bf16 && g.K <= 16384u && !plow_moe_tuning().sk_down_regs;
    if (g.det_k && !dma_ok) { /* deterministic accumulate on the register form: its own instantiations */
        if (g.N % 256u == 0u && !plow_moe_tuning().sk_narrow) {
            k_group_w8a8_stream<false, 3, false, true, false, true><<<dim3(g.E * (g.N / 256u)), SK_THREADS, 0, st>>>(g);
        } else {
            k_group_w8a8_stream<false, 3, false, false, false, true><<<grid, SK_THREADS, 0, st>>>(g);
        }
        return 0;
    }
    /* the plain arm on the direct-to-LDS form (the block scales of all of K sit in LDS: K <= 16384) */
    if (dma_ok) {
        k_group_down_w8a8_dma<<<grid, SDD_WAVES * WAVE, sizeof(SddLds), st>>>(g);
        return 0;
    }
    if (g.N % 256u == 0u && !plow_moe_tuning().sk_narrow) {
        const dim3 wgrid(g.E * (g.N / 256u));
        switch (plow_moe_tuning().sk_depth) {
        case 2: k_group_w8a8_stream<false, 2, false, true><<<wgrid, SK_THREADS, 0, st>>>(g); break;
        case 4: k_group_w8a8_stream<false, 4, false, true><<<wgrid, SK_THREADS, 0, st>>>(g); break;
        default: k_group_w8a8_stream<false, 3, false, true><<<wgrid, SK_THREADS, 0, st>>>(g); break;
        }
        return 0;
    }
    switch (plow_moe_tuning().sk_depth) {
    case 2: k_group_w8a8_stream<false, 2, false><<<grid, SK_THREADS, 0, st>>>(g); break;
    case 4: k_group_w8a8_stream<false, 4, false><<<grid, SK_THREADS, 0, st>>>(g); break;
    default: k_group_w8a8_stream<false, 3, false><<<grid, SK_THREADS, 0, st>>>(g); break;
    }
    return 0;
}
