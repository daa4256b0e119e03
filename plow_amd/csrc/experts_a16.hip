/* experts_a16.hip — grouped expert GEMMs with bf16 activations: bf16 weights (enc 0), block-fp8
 * weights with 128x128 f32 scales (enc 1, arm 0), mxfp4 weights (enc 2, arm 8) and per-output-channel
 * fp8 weights (ops 65 / 66). Also serves the dense bf16 shared expert (ops 20 / 8) as a one-expert
 * group.
 *
 * Arithmetic, per weight encoding (the weight is decoded EXACTLY to bf16, the product runs on the bf16
 * matrix cores with f32 accumulation):
 *   bf16        acc = sum_k w * x                      plow runtime/cpu/dev/golden/moe_gemma.c:35-39
 *   block-fp8   per 128-K block t = sum w * x, acc += t * S[n/128][kb]
 *                                                       plow runtime/amd/op_moe.h:3299-3310, :674-702
 *   mxfp4       w = e2m1 * 2^(s-127) folded exactly into the bf16 operand (one E8M0 per 32 k)
 *                                                       plow runtime/cpu/dev/mxfp4_common.h:30-40,
 *                                                       runtime/amd/op_moe.h:843-964
 *   fp8 / chan  acc = (sum_k w * x) * sc[n]             plow runtime/cpu/dev/golden/fp8.c:33-41, :173-214
 * GLU: out = bf16(act(gate) * up); DOWN: out = gate_r * acc as f32 (or bf16 for the dense op 8).
 *
 * WEIGHT-STREAMING KERNEL, same shape as the fp8 x fp8 one: workgroup = (expert, 128 output channels),
 * 8 waves x 16 channels, weights are the A operand of v_mfma_f32_16x16x32_bf16 (lane = (channel c,
 * k-chunk q)), read from global memory DEPTH 128-k steps ahead and decoded in registers; the
 * expert's rows are the B operand. A 128-k step is four matrix instructions of 32 k. The k order
 * inside a step is permuted identically for both operands so that every load is 16 bytes per lane:
 *   bf16 weights  instruction j of the step uses k = 32 j + 8 q .. + 8
 *   fp8 weights   the lane's 32 bytes are [16q, 16q+16) and [64+16q, 64+16q+16); instruction j uses
 *                 its bytes 8 j .. 8 j + 8
 *   mxfp4         the lane's 16 bytes are one whole MX block, k = 32 q .. 32 q + 32; instruction j
 *                 uses values 8 j .. 8 j + 8
 * Rows are addressed through two index arrays so that one kernel serves the gathered (ops 85 / 86)
 * and the slot-major (ops 48 / 49 / 65 / 66, after an internal sort by expert) layouts:
 * a_idx[r] = row of `a` feeding aligned row r, o_idx[r] = output row; ~0 marks a pad row.
 */
#include "common.h"
#include "kernels.h"
#include "tuning.h"
#include <string.h>

#define AK_WAVES 8u
#define AK_THREADS (AK_WAVES * WAVE)
#define AK_BN 128u

enum { AENC_BF16 = 0, AENC_FP8BLK = 1, AENC_MXFP4 = 2, AENC_FP8PC = 3 };

template <int ENC> struct WStep;                 /* registers one lane loads per stream and 128-k step */
template <> struct WStep<AENC_BF16> { v4i r[4]; };
template <> struct WStep<AENC_FP8BLK> { v4i r[2]; };
template <> struct WStep<AENC_FP8PC> { v4i r[2]; };
template <> struct WStep<AENC_MXFP4> { v4i r[1]; };

/* byte offset inside the 128-k step of the activation piece instruction j needs (16 bytes, 8 bf16) */
template <int ENC>
__device__ __forceinline__ uint32_t x_off(uint32_t q, int j) {
    if (ENC == AENC_BF16) return (32u * j + 8u * q) * 2u;
    if (ENC == AENC_MXFP4) return (32u * q + 8u * j) * 2u;
    return ((j < 2 ? 16u * q + 8u * j : 64u + 16u * q + 8u * (j - 2))) * 2u;
}

template <int ENC>
__device__ __forceinline__ void w_issue(WStep<ENC>& d, const uint8_t* w, const uint8_t* s, uint32_t kb,
                                        uint32_t q) {
    if (ENC == AENC_BF16) {
#pragma unroll
        for (int j = 0; j < 4; j++) d.r[j] = *(const v4i*)(w + (size_t)kb * 256u + (32u * j + 8u * q) * 2u);
    } else if (ENC == AENC_MXFP4) {
        d.r[0] = *(const v4i*)(w + (size_t)kb * 64u + 16u * q);
    } else {
        d.r[0] = *(const v4i*)(w + (size_t)kb * 128u + 16u * q);
        d.r[1] = *(const v4i*)(w + (size_t)kb * 128u + 64u + 16u * q);
    }
}

/* 8 bf16 operand values of instruction j from a lane's step registers */
template <int ENC>
__device__ __forceinline__ v8bf w_operand(const WStep<ENC>& d, int j, uint32_t e8m0 = 0) {
    if (ENC == AENC_BF16) {
        return __builtin_bit_cast(v8bf, d.r[j]);
    } else if (ENC == AENC_MXFP4) {
        const float sc = __uint_as_float(e8m0 << 23); /* E8M0: 2^(s-127) */
        const uint32_t wd = (uint32_t)d.r[0][j];                                 /* 8 nibbles, low = even k */
        const v2bf p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(wd, sc, 0);
        const v2bf p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(wd, sc, 1);
        const v2bf p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(wd, sc, 2);
        const v2bf p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(wd, sc, 3);
        return (v8bf){p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
    } else {
        const uint32_t lo = (uint32_t)d.r[j >> 1][(j & 1) * 2], hi = (uint32_t)d.r[j >> 1][(j & 1) * 2 + 1];
        const v2bf p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, false);
        const v2bf p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, true);
        const v2bf p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, false);
        const v2bf p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, true);
        return (v8bf){p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
    }
}

template <int ENC> struct DepthA { static constexpr int v = 2; };
template <> struct DepthA<AENC_MXFP4> { static constexpr int v = 4; }; /* = the scale group below */

template <int ENC, bool GLU>
__device__ __forceinline__ void ak_body(const GroupA16& g, uint32_t e, uint32_t ct, uint32_t r0,
                                        uint32_t rb, uint32_t cnt) {
    constexpr int D = DepthA<ENC>::v;
    const uint32_t lane = threadIdx.x & 63u, wv = threadIdx.x >> 6, c = lane & 15u, q = lane >> 4;
    const uint32_t K = g.K, KB = K / 128u, N = g.N;
    const uint32_t ch = ct * AK_BN + wv * 16u + c; /* this lane's weight row */
    /* bytes per weight row and per scale row */
    const size_t wrow = ENC == AENC_BF16 ? (size_t)K * 2u : (ENC == AENC_MXFP4 ? K / 2u : K);
    const uint64_t* wt = g.wtab ? g.wtab + (size_t)e * g.wcols : nullptr;
    const uint64_t* stt = g.stab ? g.stab + (size_t)e * g.wcols : nullptr;
    const uint8_t* wbase0 = wt ? (const uint8_t*)(uintptr_t)wt[g.wsel0] : (const uint8_t*)g.wdirect[0];
    const uint8_t* wbase1 = wt ? (const uint8_t*)(uintptr_t)wt[g.wsel1] : (const uint8_t*)g.wdirect[1];
    const uint32_t wmul = g.wmul ? g.wmul : 1u;
    const uint32_t wr0 = ch * wmul + g.wrow0, wr1 = ch * wmul + g.wrow1; /* this lane's weight rows */
    const uint8_t* w0 = wbase0 + (size_t)wr0 * wrow;
    const uint8_t* w1 = GLU ? wbase1 + (size_t)wr1 * wrow : nullptr;
    const uint8_t* sb0 = stt ? (const uint8_t*)(uintptr_t)stt[g.wsel0] : nullptr;
    const uint8_t* sb1 = (GLU && stt) ? (const uint8_t*)(uintptr_t)stt[g.wsel1] : nullptr;
    const uint8_t *ms0 = nullptr, *ms1 = nullptr; /* mxfp4: this row's E8M0 bytes */
    const float *bs0 = nullptr, *bs1 = nullptr;   /* block-fp8: this channel block's scale row */
    if (ENC == AENC_MXFP4) {
        ms0 = sb0 + (size_t)wr0 * (K / 32u);
        if (GLU) ms1 = sb1 + (size_t)wr1 * (K / 32u);
    }
    if (ENC == AENC_FP8BLK) {
        bs0 = (const float*)sb0 + (size_t)((ct * AK_BN + g.wrow0) / 128u) * KB;
        if (GLU) bs1 = (const float*)sb1 + (size_t)((ct * AK_BN + g.wrow1) / 128u) * KB;
    }

    /* the B-operand row of this lane */
    const uint32_t off = rb + c, r = r0 + off;
    bool valid = off < cnt;
    const uint32_t ai = valid ? (g.a_idx ? g.a_idx[r] : r) : PLOW_EXPERT_UNUSED;
    valid = ai != PLOW_EXPERT_UNUSED;
    const uint8_t* ap = (const uint8_t*)g.a + (size_t)(valid ? ai : 0u) * K * 2u;

    WStep<ENC> wa[D], wb[D];
    constexpr int DX = 2; /* the rows come from L1 / L2: two steps ahead is enough, and it halves their registers */
    v4i xa[DX][4];
    float sa[D], sbv[D];
    /* mxfp4: the E8M0 bytes of a row are read 16 at a time (four 128-k steps x four k-chunks), one load
     * per stream and four steps instead of one byte load per step: a load instruction costs the memory
     * pipeline the same whatever its width. Step d of a group uses byte 4 d + q. */
    v4i sg0[2] = {}, sg1[2] = {};
    auto issue_scales = [&](int slot, uint32_t kb) { /* kb a multiple of 4; the row's tail reads what exists */
        if (ENC != AENC_MXFP4) return;
        const uint32_t nb = K / 32u; /* bytes per scale row */
        if (kb * 4u + 16u <= nb) {
            sg0[slot] = *(const v4i*)(ms0 + kb * 4u);
            if (GLU) sg1[slot] = *(const v4i*)(ms1 + kb * 4u);
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                sg0[slot][i] = kb * 4u + 4u * i < nb ? *(const int*)(ms0 + kb * 4u + 4u * i) : 0;
                if (GLU) sg1[slot][i] = kb * 4u + 4u * i < nb ? *(const int*)(ms1 + kb * 4u + 4u * i) : 0;
            }
        }
    };
    auto issue = [&](int d, uint32_t kb) {
        w_issue<ENC>(wa[d], w0, ms0, kb, q);
        if (GLU) w_issue<ENC>(wb[d], w1, ms1, kb, q);
        if (ENC == AENC_FP8BLK) {
            sa[d] = bs0[kb];
            if (GLU) sbv[d] = bs1[kb];
        }
    };

    auto issue_x = [&](int dx, uint32_t kb) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            xa[dx][j] = (v4i){0, 0, 0, 0};
            if (valid) xa[dx][j] = *(const v4i*)(ap + (size_t)kb * 256u + x_off<ENC>(q, j));
        }
    };

    v4f acc0 = {0.0f, 0.0f, 0.0f, 0.0f}, acc1 = {0.0f, 0.0f, 0.0f, 0.0f};
    issue_scales(0, 0u);
#pragma unroll
    for (int d = 0; d < D; d++)
        if ((uint32_t)d < KB) issue(d, (uint32_t)d);
#pragma unroll
    for (int d = 0; d < DX; d++)
        if ((uint32_t)d < KB) issue_x(d, (uint32_t)d);
    static_assert(D % DX == 0, "the row ring must divide the weight ring");
    for (uint32_t kb0 = 0; kb0 < KB; kb0 += D) {
        if (ENC == AENC_MXFP4 && kb0 + D < KB) issue_scales(1, kb0 + D); /* the next group's scales */
#pragma unroll
        for (int d = 0; d < D; d++) {
            const uint32_t kb = kb0 + (uint32_t)d;
            if (kb < KB) {
                const uint32_t e0 = ENC == AENC_MXFP4 ? ((uint32_t)sg0[0][d] >> (8u * q)) & 0xFFu : 0u;
                const uint32_t e1 = (ENC == AENC_MXFP4 && GLU) ? ((uint32_t)sg1[0][d] >> (8u * q)) & 0xFFu : 0u;
                v4f t0 = ENC == AENC_FP8BLK ? (v4f){0.0f, 0.0f, 0.0f, 0.0f} : acc0;
                v4f t1 = ENC == AENC_FP8BLK ? (v4f){0.0f, 0.0f, 0.0f, 0.0f} : acc1;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const v8bf B = __builtin_bit_cast(v8bf, xa[d % DX][j]);
                    t0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_operand<ENC>(wa[d], j, e0), B, t0, 0, 0, 0);
                    if (GLU) t1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_operand<ENC>(wb[d], j, e1), B, t1, 0, 0, 0);
                }
                if (ENC == AENC_FP8BLK) {
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        acc0[i] = fmaf(t0[i], sa[d], acc0[i]);
                        if (GLU) acc1[i] = fmaf(t1[i], sbv[d], acc1[i]);
                    }
                } else {
                    acc0 = t0;
                    if (GLU) acc1 = t1;
                }
                if (kb + D < KB) issue(d, kb + D);
                if (kb + DX < KB) issue_x(d % DX, kb + DX);
            }
        }
        if (ENC == AENC_MXFP4) sg0[0] = sg0[1], sg1[0] = sg1[1];
    }

    /* ---- epilogue: lane holds channels ct*128 + wv*16 + 4q + i of row c ---- */
    if (!valid) return;
    const uint32_t col = ct * AK_BN + wv * 16u + 4u * q;
    if (g.bias) { /* flat-tensor ops: per-expert bias rows laid out like the weight rows */
        const bf16_t* be = (const bf16_t*)g.bias + (size_t)e * g.bias_rows;
#pragma unroll
        for (uint32_t i = 0; i < 4u; i++) {
            acc0[i] += bf2f(be[(col + i) * wmul + g.wrow0]);
            if (GLU) acc1[i] += bf2f(be[(col + i) * wmul + g.wrow1]);
        }
    }
    if (ENC == AENC_FP8PC) {
        const float* sc0 = (const float*)sb0 + g.wrow0 + col;
#pragma unroll
        for (int i = 0; i < 4; i++) acc0[i] *= sc0[i];
        if (GLU) {
            const float* sc1 = (const float*)sb1 + g.wrow1 + col;
#pragma unroll
            for (int i = 0; i < 4; i++) acc1[i] *= sc1[i];
        }
    }
    const uint32_t oi = g.o_idx ? g.o_idx[r] : r;
    if (oi == PLOW_EXPERT_UNUSED) return;
    if (GLU) {
        uint2 o;
        o.x = (uint32_t)f2bf(moe_glu(acc0[0], acc1[0], g.act, g.f0, g.f1)) | ((uint32_t)f2bf(moe_glu(acc0[1], acc1[1], g.act, g.f0, g.f1)) << 16);
        o.y = (uint32_t)f2bf(moe_glu(acc0[2], acc1[2], g.act, g.f0, g.f1)) | ((uint32_t)f2bf(moe_glu(acc0[3], acc1[3], g.act, g.f0, g.f1)) << 16);
        *(uint2*)((bf16_t*)g.out + (size_t)oi * N + col) = o;
    } else {
        const float gate = g.gate ? g.gate[r] : 1.0f;
        const float y0 = gate * acc0[0], y1 = gate * acc0[1], y2 = gate * acc0[2], y3 = gate * acc0[3];
        if (g.out_bf16) {
            uint2 o;
            o.x = (uint32_t)f2bf(g.gate ? y0 : acc0[0]) | ((uint32_t)f2bf(g.gate ? y1 : acc0[1]) << 16);
            o.y = (uint32_t)f2bf(g.gate ? y2 : acc0[2]) | ((uint32_t)f2bf(g.gate ? y3 : acc0[3]) << 16);
            *(uint2*)((bf16_t*)g.out + (size_t)oi * N + col) = o;
        } else {
            *(float4*)((float*)g.out + (size_t)oi * N + col) = make_float4(y0, y1, y2, y3);
        }
    }
}

template <int ENC, bool GLU>
__global__ __launch_bounds__(AK_THREADS, GLU ? 2 : 4) void k_group_a16_stream(GroupA16 g) {
    const uint32_t tiles = g.N / AK_BN;
    const uint32_t e = g.E - 1u - blockIdx.x / tiles, ct = blockIdx.x % tiles; /* heavy (folded shared) expert first */
    const uint32_t cnt = g.meta ? (uint32_t)g.meta[g.E + e] : g.dense_rows;
    if (cnt == 0u || !form_is_mine(g)) return;
    if (g.wtab && g.wtab[(size_t)e * g.wcols + g.wsel0] == 0ull) return; /* expert not resident: skipped */
    if (g.stab && ENC != AENC_BF16 && g.stab[(size_t)e * g.wcols + g.wsel0] == 0ull) return;
    const uint32_t r0 = g.meta ? (uint32_t)g.meta[e] : 0u;
    for (uint32_t rb = 0; rb < cnt; rb += 16u) ak_body<ENC, GLU>(g, e, ct, r0, rb, cnt);
}

/* ---- second form: every load goes global -> LDS in the coalesced shape -------------------------------
 * The kernel above reads its operands the way the matrix instruction wants them (lane = row), which the
 * vector memory pipeline serves at a quarter of its rate: 16 rows, so 16 or more cache lines, per load
 * instruction. That instruction rate, not memory, bounds it. Here a step is one whole 128-byte line per
 * weight row (256 k of mxfp4, 128 k of fp8, 64 k of bf16), and
 *   weights   per wave and stream 16 rows x 128 B = two direct loads (8 consecutive lanes per line) into a
 *             wave-private ring; mxfp4: the E8M0 bytes of four steps (32 per row) by one 16-byte direct load
 *             per wave (8 per row and step by a 4-byte load per stream where rows are not whole 16-byte
 *             pieces); block-fp8: the tile's block scales sit in LDS for all of K;
 *   rows      the 16 activation rows of the pass are the same for all eight waves: 16 rows x 2 bytes per k
 *             of the step, in a ring shared by the workgroup and loaded 1 KB per wave (the first 8, 4 or 2
 *             waves); experts of a handful of rows: a copy per wave instead (PRIV below);
 *   sync      rings of three steps, loads two steps ahead; per step each wave waits for its own loads
 *             (s_waitcnt vmcnt) and all meet at one barrier, after which the step before is free (none
 *             with per-wave rows);
 *   DOWN      tiles of 128 channels, 16 per wave, or of 256 with two weight operands per wave (WIDE below);
 *   swizzle   direct loads write LDS contiguously, so bank conflicts are avoided on the global side:
 *             LDS piece p of weight row r holds global piece p ^ lds_swz8(r), and likewise for
 *             activation rows of 128 B; piece p of a longer activation row r holds global piece
 *             (p & ~15) | ((p ^ lds_swz16(r)) & 15).
 * Same arithmetic as the first form, and the same order of additions except with per-wave rows, where a wave
 * starts its walk over K at a column of its own. */
/* ring depth: four steps (loads three ahead) where the rings leave room in the CU's 160 KB — one row group per
 * pass and 4 KB of weight rows per wave and step — three steps otherwise (mxfp4's step carries 8 KB of
 * activation rows and the E8M0 bytes; several row groups per pass multiply the activation ring) */
template <int ENC, int RG> struct DmDepth { static constexpr uint32_t v = (ENC != AENC_MXFP4 && RG == 1) ? 4u : 3u; };
#ifndef DM_MX_DOWN_STAGES1
#define DM_MX_DOWN_STAGES1 6u
#endif
#ifndef DM_MX_DOWN_STAGES2
#define DM_MX_DOWN_STAGES2 4u
#endif
/* Ring slots in use; loads are in flight for one step fewer. The GLU's two weight streams keep twice the bytes in
 * flight per step and measured no faster at a fourth slot (the DOWN gained 3 %), so it stays at three. The mxfp4
 * DOWN's step is 16 KB of weight rows per workgroup (one CU): two steps in flight are 32 KB, which does not keep the
 * CU's share of the memory busy across the per-step barrier; its rings take what the LDS has. */
template <int ENC, bool TWO, int RG> struct DmStages { /* TWO: two weight streams per wave (GLU; the wide DOWN) */
    static constexpr uint32_t v = TWO ? 3u : (ENC == AENC_MXFP4 ? (RG == 1 ? DM_MX_DOWN_STAGES1 : DM_MX_DOWN_STAGES2) : DmDepth<ENC, RG>::v);
};
template <int ENC> struct DmGeom;
template <> struct DmGeom<AENC_MXFP4> { static constexpr uint32_t KSTEP = 256u; };
template <> struct DmGeom<AENC_FP8PC> { static constexpr uint32_t KSTEP = 128u; };
template <> struct DmGeom<AENC_FP8BLK> { static constexpr uint32_t KSTEP = 128u; };
template <> struct DmGeom<AENC_BF16> { static constexpr uint32_t KSTEP = 64u; };
/* mxfp4 scales, two ways. Chunked (MXC, rows of whole 16-byte pieces: K % 512 == 0): a wave brings the E8M0 bytes
 * of FOUR steps, 32 bytes per weight row, with one 16-byte-per-lane direct load for both streams (lane = stream,
 * row, half) into one of two buffers of its own; a row's scale line is then touched once per four steps and not once
 * per step and stream, which matters because a step's weight rows push those lines out of the CU's 32 KB vector
 * cache in between (Kimi-K2 shape, 128 tokens: GLU 1029 -> us). Per step otherwise: 8 bytes per row and stream
 * into the ring slot. */
template <bool SC, int NS> struct DmWSlot;
template <int NS> struct DmWSlot<true, NS> {
    uint8_t w[NS][16u * 128u]; /* [stream][row][128 B] */
    uint8_t sc[NS][256];       /* [stream][row][8 B]; lanes 32..63 write copies behind */
};
template <int NS> struct DmWSlot<false, NS> {
    uint8_t w[NS][16u * 128u];
};
/* A chunk's buffer is written again NB chunks later, when the load cursor, AH steps ahead of the multiplies, starts
 * that chunk; the shortest chunk is two steps (K = 512, or the tail of K = 512 (2 j + 1)), so the multiplies have
 * left it if AH <= 2 (NB - 1). */
template <int NB, int NS> struct DmScaleChunks { uint8_t sch[AK_WAVES][NB][NS * 512]; }; /* [wave][buffer][stream][row][32 B] */
template <int NS> struct DmScaleChunks<0, NS> {};
template <uint32_t AH> struct DmChunkBufs { static constexpr int v = AH <= 2u ? 2 : (AH <= 4u ? 3 : 4); };
template <bool ON> struct DmBlockScales;
template <> struct DmBlockScales<true> { float bsc[4][2][128]; }; /* the weight block scales of the workgroup's tiles, all of K (K <= 16384) */
template <> struct DmBlockScales<false> {};
/* RG = 16-row groups of activation rows per pass over the weights: 1, 2 or 4 (mxfp4: 1 or 2), picked per
 * workgroup from its expert's row count: with more groups the weights are streamed less often and every
 * weight operand read from LDS feeds that many matrix instructions */
/* PRIV: every wave keeps its own copy of the expert's (few) activation rows, DmPrivRows of them, so that nothing in
 * the K loop is shared and no barrier is needed */
template <int ENC> struct DmPrivRows { static constexpr uint32_t v = DmGeom<ENC>::KSTEP * 2u >= 256u ? 4u : 1024u / (DmGeom<ENC>::KSTEP * 2u); };
template <int ENC, bool TWO, int RG, bool MXC = false, bool PRIV = false>
struct DmLds : DmScaleChunks<MXC ? DmChunkBufs<DmStages<ENC, TWO, RG>::v - 1u>::v : 0, TWO ? 2 : 1>, DmBlockScales<ENC == AENC_FP8BLK> { /* bases: empty ones take no room */
    uint8_t x[(PRIV ? AK_WAVES : 1u) * DmStages<ENC, TWO, RG>::v][(PRIV ? DmPrivRows<ENC>::v : RG * 16u) * DmGeom<ENC>::KSTEP * 2u];
    DmWSlot<ENC == AENC_MXFP4 && !MXC, TWO ? 2 : 1> ring[AK_WAVES][DmStages<ENC, TWO, RG>::v];
};
typedef __attribute__((address_space(3))) void dm_lds_void;
__device__ __forceinline__ uint32_t dm_lds_off(const void* p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}
__device__ __forceinline__ v4i dm_read16(uint32_t addr) {
    v4i r;
    asm volatile("ds_read_b128 %0, %1" : "=v"(r) : "v"(addr) : "memory");
    return r;
}
__device__ __forceinline__ uint2 dm_read8(uint32_t addr) {
    uint2 r;
    asm volatile("ds_read_b64 %0, %1" : "=v"(r) : "v"(addr) : "memory");
    return r;
}
__device__ __forceinline__ float dm_read4(uint32_t addr) {
    float r;
    asm volatile("ds_read_b32 %0, %1" : "=v"(r) : "v"(addr) : "memory");
    return r;
}
/* wait until at most n of this wave's loads are outstanding (and its LDS reads are done), then the
 * workgroup barrier */
#define DM_WAIT_BARRIER(n) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(n) : "memory")
#define DM_WAIT_ONLY(n) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(n) : "memory")

/* the wait + barrier for `after` (at most A) steps of PER loads each still allowed in flight */
template <int A, int PER, bool BARRIER = true>
__device__ __forceinline__ void dm_wait_steps(uint32_t after) {
    static_assert(A * PER <= 63, "the load counter holds six bits");
    if constexpr (A == 0) {
        if constexpr (BARRIER) DM_WAIT_BARRIER(0);
        else DM_WAIT_ONLY(0);
    } else {
        if (after == (uint32_t)A) {
            if constexpr (BARRIER) DM_WAIT_BARRIER(A * PER);
            else DM_WAIT_ONLY(A * PER);
        } else {
            dm_wait_steps<A - 1, PER, BARRIER>(after);
        }
    }
}

/* What workgroup index `bid` of a logical grid of E * N / 128 works on: expert e (cnt rows), TPW channel tiles
 * from tile ct. False when it has nothing to do. */
struct DmWork {
    uint32_t e, ct, TPW, cnt;
};
template <int ENC, bool WIDE = false>
__device__ __forceinline__ bool a16_dma_work(const GroupA16& g, uint32_t bid, DmWork& w) {
    const uint32_t tiles = g.N / (WIDE ? 2u * AK_BN : AK_BN);
    /* With plenty of tiles to go round and a short K loop, a workgroup takes TPW consecutive channel tiles
     * of its expert and keeps the load rings running across them, which hides the ramp of the loop. meta[3E], the
     * number of 64-row tiles, is at least the number of experts with rows. The grid has one workgroup per
     * tile; the first E * tiles / TPW of them do the work (consecutive indices, so that they spread over
     * all XCDs) and the rest leave at once. */
    const uint32_t busy = (g.meta ? (uint32_t)g.meta[3u * g.E] : 1u) * tiles;
    const bool short_k = g.K / DmGeom<ENC>::KSTEP <= 16u; /* a long K loop amortises its ramp by itself */
    w.TPW = !short_k ? 1u
            : (ENC == AENC_MXFP4 && busy >= 8192u && tiles % 8u == 0u) ? 8u /* no per-tile tables to hold */
            : (busy >= 4096u && tiles % 4u == 0u) ? 4u : ((busy >= 2048u && tiles % 2u == 0u) ? 2u : 1u);
    const uint32_t wpe = tiles / w.TPW; /* workgroups per expert */
    if (bid >= g.E * wpe) return false;
    w.e = g.E - 1u - bid / wpe, w.ct = (bid % wpe) * w.TPW; /* heavy (folded shared) expert first */
    w.cnt = g.meta ? (uint32_t)g.meta[g.E + w.e] : g.dense_rows;
    return w.cnt != 0u;
}

/* The body takes its LDS as a pointer, so that a kernel with a fixed launch shape (any 1-D grid, static LDS) can
 * walk the logical grid itself. */
/* WIDE (DOWN only): a wave owns 32 channels, two 16-row weight operands that share the activation operand, and the
 * workgroup a tile of 256: the GLU's shape with the second stream 16 channels further down the same matrix. A step
 * is then 32 KB of weight rows per workgroup instead of 16: half the barriers, waits and activation-row reads per
 * weight byte. */
/* PRIV (an expert of at most DmPrivRows rows, two weight streams): the wave loads those rows itself, beside its
 * weights, into a ring of its own (lanes of rows the expert does not have stay out), and waits for nothing but its
 * own loads: no barrier in the K loop, the waves of a workgroup drift apart and their loads and multiplies
 * interleave. The rows cross the L2 -> LDS path once per wave instead of once per workgroup; with three rows that
 * is a third of the weight bytes. */
template <int ENC, bool GLU, int RG, bool MXC = false, bool WIDE = false, bool PRIV = false>
__device__ __forceinline__ void a16_dma_body(const GroupA16& g, uint8_t* dm_raw, const DmWork& work) {
    static_assert(!MXC || ENC == AENC_MXFP4, "chunked scales are the mxfp4 arm's");
    static_assert(!(GLU && WIDE), "the wide form is the DOWN's");
    constexpr bool TWO = GLU || WIDE;                   /* two weight streams per wave */
    static_assert(!PRIV || (RG == 1 && TWO), "private rows: one row group, the two-stream shapes");
    constexpr uint32_t BN = WIDE ? 2u * AK_BN : AK_BN;   /* channels per workgroup tile */
    DmLds<ENC, TWO, RG, MXC, PRIV>& L = *(DmLds<ENC, TWO, RG, MXC, PRIV>*)dm_raw;
    /* ring slots; steps of loads in flight. One slot holds the step being multiplied, the others are in flight; with
     * private rows nobody else reads a wave's slots, a step's operands are in registers before its multiplies start,
     * and its slot takes the next load at once: as many steps in flight as there are slots */
    constexpr uint32_t DM_STAGES = DmStages<ENC, TWO, RG>::v, AH = PRIV ? DM_STAGES : DM_STAGES - 1u;
    typedef DmWSlot<ENC == AENC_MXFP4 && !MXC, TWO ? 2 : 1> Slot;
    constexpr uint32_t KSTEP = DmGeom<ENC>::KSTEP, XROW = KSTEP * 2u; /* activation bytes per row and step */
    constexpr uint32_t NP = XROW / 16u;                              /* 16-byte pieces per activation row */
    constexpr uint32_t PR = DmPrivRows<ENC>::v;                      /* rows of a private ring */
    constexpr uint32_t XROWS = PRIV ? PR : RG * 16u;                 /* rows of a ring stage */
    constexpr uint32_t XL = XROWS * XROW / 1024u;                    /* 1 KB activation loads per step */
    constexpr uint32_t XRPL = 64u / NP;                              /* rows per activation load */
    /* activation loads per wave and step: a share of the workgroup's (wave w: w, w + 8, ..), or all of its own */
    constexpr uint32_t XW = PRIV ? 1u : AK_WAVES;
    constexpr uint32_t NXI = (XL + XW - 1u) / XW;
    static_assert(XL >= 1u && (XL < XW || XL % XW == 0u), "activation loads must split evenly over the waves");
    constexpr int NS = TWO ? 2 : 1;
    /* direct loads per wave and step: weights 2 per stream, mxfp4 scales 1 per stream, rows NXI (waves below XL).
     * Chunked mxfp4 scales are one more load every fourth step and not counted: a wait that allows n loads to be
     * outstanding asks for everything older than the newest n, so an uncounted load makes it stricter by one and
     * never looser. */
    constexpr int NLW = NS * ((ENC == AENC_MXFP4 && !MXC) ? 3 : 2);
    const uint32_t e = work.e, ct = work.ct, TPW = work.TPW, cnt = work.cnt;
    const uint64_t* wt = g.wtab ? g.wtab + (size_t)e * g.wcols : nullptr;
    const uint64_t* stt = g.stab ? g.stab + (size_t)e * g.wcols : nullptr;
    if (wt && wt[g.wsel0] == 0ull) return; /* expert not resident: skipped */
    if (stt && ENC != AENC_BF16 && stt[g.wsel0] == 0ull) return;
    /* K split (dense bf16 ops): slice e % ksplit of tensor e / ksplit; rows 0 .. of the activations, rows
     * e * dense_rows .. of the output */
    const uint32_t ksp = ENC == AENC_BF16 ? g.ksplit : 0u;
    const uint32_t r0 = g.meta ? (uint32_t)g.meta[e] : (ksp ? e * g.dense_rows : 0u);
    const uint32_t xr0 = ksp ? 0u : r0; /* the expert's first activation row */
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wv = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint32_t c = lane & 15u, q = lane >> 4; /* operand layout: row / channel c, k-chunk q */
    const uint32_t K = g.K, KS = K / KSTEP, N = g.N, GS = TPW * KS; /* steps of a pass over all its tiles */
    const uint32_t KP = ksp ? g.kpitch : K;                        /* elements per row in memory */
    const size_t kofs = ksp ? (size_t)(e % ksp) * K * 2u : 0u;     /* the slice's first byte in a row */
    const uint8_t* const abase = (const uint8_t*)g.a + kofs;
    const uint32_t chw = ct * BN + wv * (WIDE ? 32u : 16u); /* this wave's first channel */
    const uint32_t wrow = ENC == AENC_BF16 ? KP * 2u : (ENC == AENC_MXFP4 ? K / 2u : K); /* bytes per weight row */
    const uint32_t wmul = g.wmul ? g.wmul : 1u;

    /* weight loads: load j covers rows 8j .. 8j + 7 of a stream (lane = row lr of the group, piece p) */
    const uint32_t lr = lane >> 3, p = lane & 7u;
    const uint8_t* wsrc[2][2];
    const uint8_t* ssrc[2] = {nullptr, nullptr};
    const float* pcs[2] = {nullptr, nullptr}; /* per-channel fp8: this lane's four output scales per stream */
#pragma unroll
    for (int sidx = 0; sidx < NS; sidx++) {
        /* the wide DOWN's second stream is the same matrix, 16 channels on */
        const uint32_t sel = (sidx && !WIDE) ? g.wsel1 : g.wsel0;
        const uint8_t* wbase = wt ? (const uint8_t*)(uintptr_t)wt[sel]
                                  : (const uint8_t*)g.wdirect[ksp ? e / ksp : (WIDE ? 0 : sidx)] + kofs;
        const uint8_t* sbase = stt ? (const uint8_t*)(uintptr_t)stt[sel] : nullptr;
        const uint32_t wr0 = (sidx && !WIDE) ? g.wrow1 : g.wrow0;
        const uint32_t chs = chw + ((sidx && WIDE) ? 16u : 0u); /* the stream's first channel */
#pragma unroll
        for (uint32_t j = 0; j < 2u; j++) {
            const uint32_t R = 8u * j + lr;
            wsrc[sidx][j] = wbase + (size_t)((chs + R) * wmul + wr0) * wrow + ((p ^ lds_swz8(R)) << 4);
        }
        /* mxfp4 scales: lane -> (row (lane & 31) >> 1, dword lane & 1) of the step's 8 bytes per row */
        if (ENC == AENC_MXFP4 && !MXC)
            ssrc[sidx] = sbase + (size_t)((chs + ((lane & 31u) >> 1)) * wmul + wr0) * (K / 32u) + (lane & 1u) * 4u;
        /* chunked: lanes 0..31 bring the first stream's bytes, lanes 32..63 the second's (one stream: they stay out);
         * lane -> (row (lane & 31) >> 1, 16-byte half lane & 1) of the chunk's 32 bytes per row */
        if (MXC && (sidx == 0 ? (lane < 32u || !TWO) : lane >= 32u))
            ssrc[0] = sbase + (size_t)((chs + ((lane & 31u) >> 1)) * wmul + wr0) * (K / 32u) + (lane & 1u) * 16u;
        if (ENC == AENC_FP8PC) pcs[sidx] = (const float*)sbase + wr0 + chs + 4u * q;
        if (ENC == AENC_FP8BLK) { /* the channel blocks' scale rows go to LDS once (wide: the tile's two blocks) */
            for (uint32_t t = 0; t < TPW; t++) {
                const float* bs = (const float*)sbase + (size_t)(((ct + t) * BN + (WIDE ? 128u * sidx : 0u) + wr0) / 128u) * (K / 128u);
                if constexpr (ENC == AENC_FP8BLK)
                    for (uint32_t i = threadIdx.x; i < K / 128u; i += AK_THREADS) L.bsc[t][sidx][i] = bs[i];
            }
        }
    }
    const uint32_t cx = PRIV ? c % PR : c; /* the ring row that stands for this lane's B-operand row */
    const uint32_t swz = lds_swz8(c), swzx = lds_swz8(cx), swx = lds_swz16(cx);
    const uint32_t x_base = dm_lds_off(&L.x[PRIV ? wv * DM_STAGES : 0u][0]);
    const uint32_t w_base = dm_lds_off(&L.ring[wv][0]);
    uint32_t b_base = 0u, sch_base = 0u;
    if constexpr (ENC == AENC_FP8BLK) b_base = dm_lds_off(&L.bsc[0][0][0]);
    /* scale chunk buffers and their size (private rows: whole chunks of four steps only, K % 1024 == 0, and then
     * a buffer is free when the cursor, AH steps ahead, starts the chunk CKB further on: 4 CKB - AH >= 4) */
    constexpr uint32_t CKB = (uint32_t)DmChunkBufs<DM_STAGES - 1u>::v, CKSZ = NS * 512u;
    static_assert(PRIV ? AH + 4u <= 4u * CKB : AH <= 2u * (CKB - 1u), "a scale buffer must be free when its next chunk is loaded");
    if constexpr (MXC) sch_base = dm_lds_off(&L.sch[wv][0][0]) + c * 32u;
    /* LDS position of logical piece P of activation row c */
    auto xpos = [&](uint32_t P) -> uint32_t { return NP >= 16u ? ((P & ~15u) | ((P ^ swx) & 15u)) : (P ^ swzx); };

    for (uint32_t rb = 0; rb < cnt; rb += 16u * RG) {
        /* this wave's share of the pass's rows: load i covers rows XRPL * (wv + 8 i) .., NP lanes each; a pad
         * row reads the pass's first row and is never stored */
        const uint32_t pc = lane % NP;
        const uint8_t* xsrc[NXI];
        /* A load whose rows all lie past the expert's last row brings four bytes per lane of the pass's first row
         * instead of sixteen of its own rows (one cache line instead of eight; the count of loads per step stays what
         * the waits below assume): the LDS rows it would fill feed only the columns of pad rows in the matrix products
         * (a column of the result depends on its own row alone), and those are never stored. With three rows in a pass
         * of sixteen that is most of the row bytes a step asks of the L2. */
        /* (bf16 weights: a step's rows are 2 KB against 32 KB of weight rows, nothing to win: always loaded) */
        /* (private rings: lanes of rows the expert does not have take no part in the load at all) */
        const uint32_t live = (ENC == AENC_BF16 && !PRIV) ? 0xFFFFFFFFu : cnt - rb;
        const uint8_t* xdummy;
        bool xlane[NXI]; /* private rings: this lane's row exists */
        {
            const uint32_t first = g.a_idx ? g.a_idx[xr0 + rb] : xr0 + rb;
#pragma unroll
            for (uint32_t i = 0; i < NXI; i++) {
                const uint32_t xrow0 = PRIV ? XRPL * i : XRPL * (wv + AK_WAVES * i); /* the load's first row */
                const uint32_t xrow = xrow0 + lane / NP;
                xsrc[i] = nullptr;
                xlane[i] = !PRIV || xrow < live;
                if ((PRIV || wv + AK_WAVES * i < XL) && xrow0 < live) {
                    const uint32_t off = rb + xrow;
                    uint32_t ai = off < cnt ? (g.a_idx ? g.a_idx[xr0 + off] : xr0 + off) : PLOW_EXPERT_UNUSED;
                    if (ai == PLOW_EXPERT_UNUSED) ai = first == PLOW_EXPERT_UNUSED ? 0u : first;
                    const uint32_t gp = NP >= 16u ? ((pc & ~15u) | ((pc ^ lds_swz16(xrow)) & 15u)) : (pc ^ lds_swz8(xrow));
                    xsrc[i] = abase + (size_t)ai * KP * 2u + (gp << 4);
                }
            }
            xdummy = abase + (size_t)(first == PLOW_EXPERT_UNUSED ? 0u : first) * KP * 2u;
        }
        /* the B-operand rows of this lane: row c of each 16-row group */
        bool valid[RG];
        uint32_t oi[RG];
        float gate[RG];
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            const uint32_t off = rb + 16u * (uint32_t)rg + c, r = r0 + off;
            valid[rg] = off < cnt;
            const uint32_t ai_c = valid[rg] ? (g.a_idx ? g.a_idx[r] : r) : PLOW_EXPERT_UNUSED;
            valid[rg] = ai_c != PLOW_EXPERT_UNUSED;
            /* what the epilogues need from memory is read here, before the rings start: an ordinary load
             * inside the stream would make the compiler wait for every outstanding direct load */
            oi[rg] = valid[rg] ? (g.o_idx ? g.o_idx[r] : r) : PLOW_EXPERT_UNUSED;
            gate[rg] = (!GLU && valid[rg] && g.gate) ? g.gate[r] : 1.0f;
        }
        float4 pc0[4], pc1[4];
        if (ENC == AENC_FP8PC) {
#pragma unroll
            for (uint32_t t = 0; t < 4u; t++) {
                pc0[t] = pc1[t] = make_float4(1.0f, 1.0f, 1.0f, 1.0f);
                if (t < TPW) {
                    pc0[t] = *(const float4*)(pcs[0] + t * BN);
                    if (TWO) pc1[t] = *(const float4*)(pcs[1] + t * BN);
                }
            }
        }

        /* a use the compiler cannot move: its own wait for these loads lands here and not behind the
         * first direct loads */
#pragma unroll
        for (int rg = 0; rg < RG; rg++) asm volatile("" ::"v"(oi[rg]), "v"(gate[rg]));
        if (ENC == AENC_FP8PC) {
#pragma unroll
            for (int t = 0; t < 4; t++) asm volatile("" ::"v"(pc0[t].x), "v"(pc0[t].w), "v"(pc1[t].x), "v"(pc1[t].w));
        }

        /* the load cursor walks (tile, step) in order; ring slots follow the running step count */
        /* the cursor's addresses run along: one line on per step, from a tile's last step to the next tile's first */
        /* Private rows: each wave walks K from a start of its own and wraps at the row's end. The 256 weight rows a
         * workgroup asks for in one step are then spread over eight columns of the matrix instead of lying in one,
         * which matters when the row pitch is a power of two and one column means few memory channels (per-channel
         * fp8 at K = 4096: 11 % per byte against K = 3968 or 4224). ld_S is the cursor's place in the row, ld_c
         * its count of steps in the tile. */
        const uint32_t rot = PRIV ? (wv * (ENC == AENC_MXFP4 ? 4u : (KS >= 8u ? KS / 8u : 1u))) % KS : 0u;
        uint32_t ld_S = rot, ld_c = 0, ld_st = 0, ld_ck = 0;
        const uint8_t* wp[2][2] = {{wsrc[0][0] + rot * 128u, wsrc[0][1] + rot * 128u}, {wsrc[1][0] + rot * 128u, wsrc[1][1] + rot * 128u}};
        const uint8_t* sp[2] = {ssrc[0] + rot * 8u, ssrc[1] + rot * 8u};
        const uint8_t* xp[NXI];
#pragma unroll
        for (uint32_t i = 0; i < NXI; i++) xp[i] = xsrc[i] + rot * XROW;
        const size_t w_tile = (size_t)BN * wmul * wrow, s_tile = (size_t)BN * wmul * (K / 32u);
        auto issue = [&]() {
            Slot* slot = &L.ring[wv][ld_st];
            if constexpr (MXC) {
                if ((ld_S & 3u) == 0u) { /* the E8M0 bytes of steps ld_S .. ld_S + 3, ahead of the step's own loads */
                    /* a half whose two steps lie past the row's end reads the first half again */
                    const uint32_t back = (ld_S + 2u * (lane & 1u) < KS) ? 0u : 16u;
                    if (TWO || lane < 32u)
                        __builtin_amdgcn_global_load_lds((const void*)(sp[0] - back), (dm_lds_void*)&L.sch[wv][ld_ck][0], 16, 0, 0);
                    ld_ck = ld_ck + 1u == CKB ? 0u : ld_ck + 1u;
                }
            }
#pragma unroll
            for (int sidx = 0; sidx < NS; sidx++) {
#pragma unroll
                for (uint32_t j = 0; j < 2u; j++) {
                    __builtin_amdgcn_global_load_lds((const void*)wp[sidx][j], (dm_lds_void*)&slot->w[sidx][8u * j * 128u], 16, 0, LOAD_NT);
                    wp[sidx][j] += 128u;
                }
                if constexpr (ENC == AENC_MXFP4 && !MXC)
                    __builtin_amdgcn_global_load_lds((const void*)sp[sidx], (dm_lds_void*)&slot->sc[sidx][0], 4, 0, 0); /* 8 bytes of a line per step: cached */
                if constexpr (ENC == AENC_MXFP4) sp[sidx] += 8u;
            }
#pragma unroll
            for (uint32_t i = 0; i < NXI; i++)
                if (PRIV || wv + AK_WAVES * i < XL) {
                    const uint32_t xrow0 = PRIV ? XRPL * i : XRPL * (wv + AK_WAVES * i);
                    dm_lds_void* const dst = (dm_lds_void*)&L.x[PRIV ? wv * DM_STAGES + ld_st : ld_st][xrow0 * XROW];
                    if (xrow0 < live) {
                        if (xlane[i]) __builtin_amdgcn_global_load_lds((const void*)xp[i], dst, 16, 0, 0);
                        xp[i] += XROW;
                    } else { /* rows past the expert's last: a stand-in that keeps the load count */
                        __builtin_amdgcn_global_load_lds((const void*)xdummy, dst, 4, 0, 0);
                    }
                }
            ld_st = ld_st + 1u == DM_STAGES ? 0u : ld_st + 1u;
            if (++ld_S == KS) { /* the row's end: back to its start */
                ld_S = 0u;
#pragma unroll
                for (int sidx = 0; sidx < NS; sidx++) {
                    wp[sidx][0] -= (size_t)KS * 128u, wp[sidx][1] -= (size_t)KS * 128u;
                    if constexpr (ENC == AENC_MXFP4) sp[sidx] -= (size_t)KS * 8u;
                }
#pragma unroll
                for (uint32_t i = 0; i < NXI; i++) xp[i] = xsrc[i];
            }
            if (++ld_c == KS) { /* on to the next tile of the expert: its weight rows, the same activation rows again */
                ld_c = 0u;
#pragma unroll
                for (int sidx = 0; sidx < NS; sidx++) {
                    wp[sidx][0] += w_tile, wp[sidx][1] += w_tile;
                    if constexpr (ENC == AENC_MXFP4) sp[sidx] += s_tile;
                }
            }
        };
        v4f acc0[RG], acc1[RG];
#pragma unroll
        for (int rg = 0; rg < RG; rg++) acc0[rg] = acc1[rg] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
        /* the row maps above are loaded (the count of outstanding loads starts at zero), and every wave
         * has left the pass before (its ring slots are free; the block scales are written) */
        DM_WAIT_BARRIER(0);
#pragma unroll
        for (uint32_t i = 0; i < AH; i++)
            if (i < GS) issue();
        uint32_t st = 0, ck = CKB - 1u; /* ck: the scale buffer of the chunk being used */
        uint32_t Sr = rot;              /* the multiplies' place in the row (S counts the tile's steps) */
        for (uint32_t G = 0, t = 0, S = 0; G < GS; G++) {
            if (MXC && (S & 3u) == 0u) ck = ck + 1u == CKB ? 0u : ck + 1u;
            /* loads return in order: step G has landed once at most the steps after it that were issued (AH - 1
             * of them, fewer at the end) are outstanding; after the barrier every wave's share of the rows is
             * there and nobody reads step G - 1 any more */
            const uint32_t after = GS - 1u - G < AH - 1u ? GS - 1u - G : AH - 1u; /* steps in flight behind step G */
            const bool loads_x = PRIV || XL >= AK_WAVES || wv < XL;
            if (loads_x) dm_wait_steps<(int)AH - 1, NLW + (int)NXI, !PRIV>(after);
            else dm_wait_steps<(int)AH - 1, NLW, !PRIV>(after);
            /* mxfp4 (twice the multiplies and conversions per weight byte): the step's operand reads go out first and
             * cross the LDS while the loads below are being issued */
            if (ENC != AENC_MXFP4 && !PRIV && G + AH < GS) issue();
            const uint32_t wb = w_base + st * (uint32_t)sizeof(Slot), xb0 = x_base + st * (XROWS * XROW) + cx * XROW;
            /* the weight operands of the step are read once and multiply every row group of the pass */
            if constexpr (ENC == AENC_MXFP4) {
                uint2 e0, e1;
                if constexpr (MXC) {
                    const uint32_t sa8 = sch_base + ck * CKSZ + (S & 3u) * 8u;
                    e0 = dm_read8(sa8), e1 = e0;
                    if (TWO) e1 = dm_read8(sa8 + 512u);
                } else {
                    e0 = dm_read8(wb + NS * 2048u + c * 8u), e1 = e0;
                    if (TWO) e1 = dm_read8(wb + NS * 2048u + 256u + c * 8u);
                }
                v4i wa[2], wbv[2];
#pragma unroll
                for (uint32_t u = 0; u < 2u; u++) {
                    const uint32_t wo = c * 128u + (((4u * u + q) ^ swz) << 4);
                    wa[u] = dm_read16(wb + wo);
                    wbv[u] = wa[u];
                    if (TWO) wbv[u] = dm_read16(wb + 2048u + wo);
                }
                v4i xa[2][4];
#pragma unroll
                for (uint32_t u = 0; u < 2u; u++)
#pragma unroll
                    for (uint32_t j = 0; j < 4u; j++) xa[u][j] = dm_read16(xb0 + (xpos(16u * u + 4u * q + j) << 4));
                if (!PRIV && G + AH < GS) issue();
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(e0), "+v"(e1), "+v"(wa[0]), "+v"(wa[1]), "+v"(wbv[0]), "+v"(wbv[1]));
                if constexpr (PRIV) { /* the step's operands are out of its slot: the slot takes the load AH steps on */
                    asm volatile("" : "+v"(xa[0][0]), "+v"(xa[0][1]), "+v"(xa[0][2]), "+v"(xa[0][3]), "+v"(xa[1][0]), "+v"(xa[1][1]), "+v"(xa[1][2]), "+v"(xa[1][3]));
                    if (G + AH < GS) issue();
                }
#pragma unroll
                for (int rg = 0; rg < RG; rg++) {
                    if (rg) {
                        const uint32_t xb = xb0 + (uint32_t)rg * (16u * XROW);
#pragma unroll
                        for (uint32_t u = 0; u < 2u; u++)
#pragma unroll
                            for (uint32_t j = 0; j < 4u; j++) xa[u][j] = dm_read16(xb + (xpos(16u * u + 4u * q + j) << 4));
                    }
                    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(xa[0][0]), "+v"(xa[0][1]), "+v"(xa[0][2]), "+v"(xa[0][3]));
                    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(xa[1][0]), "+v"(xa[1][1]), "+v"(xa[1][2]), "+v"(xa[1][3]));
#pragma unroll
                    for (uint32_t u = 0; u < 2u; u++) {
                        const uint32_t s0 = ((u ? e0.y : e0.x) >> (8u * q)) & 0xFFu, s1 = ((u ? e1.y : e1.x) >> (8u * q)) & 0xFFu;
                        WStep<AENC_MXFP4> da, db;
                        da.r[0] = wa[u];
                        db.r[0] = wbv[u];
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const v8bf B = __builtin_bit_cast(v8bf, xa[u][j]);
                            acc0[rg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_operand<AENC_MXFP4>(da, j, s0), B, acc0[rg], 0, 0, 0);
                            if (TWO) acc1[rg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_operand<AENC_MXFP4>(db, j, s1), B, acc1[rg], 0, 0, 0);
                        }
                    }
                }
            } else if constexpr (ENC == AENC_BF16) {
                /* 64 k: instruction j uses k = 32 j + 8 q .. + 8 of both operands */
                v4i wa[2], wbv[2];
#pragma unroll
                for (uint32_t j = 0; j < 2u; j++) {
                    const uint32_t wo = c * 128u + (((4u * j + q) ^ swz) << 4);
                    wa[j] = dm_read16(wb + wo);
                    wbv[j] = wa[j];
                    if (TWO) wbv[j] = dm_read16(wb + 2048u + wo);
                }
                v4i xr[2][2];
#pragma unroll
                for (uint32_t j = 0; j < 2u; j++) xr[0][j] = dm_read16(xb0 + (xpos(4u * j + q) << 4));
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(wa[0]), "+v"(wa[1]), "+v"(wbv[0]), "+v"(wbv[1]));
                if constexpr (PRIV) {
                    asm volatile("" : "+v"(xr[0][0]), "+v"(xr[0][1]));
                    if (G + AH < GS) issue();
                }
#pragma unroll
                for (int rg = 0; rg < RG; rg++) {
                    v4i* const xa = xr[rg & 1];
                    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(xa[0]), "+v"(xa[1]));
                    if (rg + 1 < RG) {
                        const uint32_t xb = xb0 + (uint32_t)(rg + 1) * (16u * XROW);
#pragma unroll
                        for (uint32_t j = 0; j < 2u; j++) xr[(rg + 1) & 1][j] = dm_read16(xb + (xpos(4u * j + q) << 4));
                    }
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        const v8bf B = __builtin_bit_cast(v8bf, xa[j]);
                        acc0[rg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, wa[j]), B, acc0[rg], 0, 0, 0);
                        if (TWO) acc1[rg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, wbv[j]), B, acc1[rg], 0, 0, 0);
                    }
                }
            } else {
                /* fp8, 128 k: the lane's weight bytes are [16q, 16q + 16) and [64 + 16q, 64 + 16q + 16);
                 * instruction j uses bytes 8 (j & 1) .. + 8 of half j >> 1 */
                WStep<ENC> da, db;
                float sa = 1.0f, sb = 1.0f;
#pragma unroll
                for (uint32_t h = 0; h < 2u; h++) {
                    const uint32_t wo = c * 128u + (((4u * h + q) ^ swz) << 4);
                    da.r[h] = dm_read16(wb + wo);
                    db.r[h] = da.r[h];
                    if (TWO) db.r[h] = dm_read16(wb + 2048u + wo);
                }
                if (ENC == AENC_FP8BLK) {
                    /* wide: both streams lie in one 128-channel block, the tile's first (waves 0..3) or second */
                    sa = dm_read4(b_base + t * 1024u + (WIDE ? (wv >> 2) * 512u : 0u) + Sr * 4u);
                    sb = sa;
                    if (GLU) sb = dm_read4(b_base + t * 1024u + 512u + Sr * 4u);
                }
                /* the rows of group rg + 1 are read from LDS while group rg multiplies */
                v4i xr[2][4];
#pragma unroll
                for (uint32_t j = 0; j < 4u; j++) xr[0][j] = dm_read16(xb0 + (xpos(8u * (j >> 1) + 2u * q + (j & 1u)) << 4));
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(da.r[0]), "+v"(da.r[1]), "+v"(db.r[0]), "+v"(db.r[1]), "+v"(sa), "+v"(sb));
                if constexpr (PRIV) {
                    asm volatile("" : "+v"(xr[0][0]), "+v"(xr[0][1]), "+v"(xr[0][2]), "+v"(xr[0][3]));
                    if (G + AH < GS) issue();
                }
#pragma unroll
                for (int rg = 0; rg < RG; rg++) {
                    v4i* const xa = xr[rg & 1];
                    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(xa[0]), "+v"(xa[1]), "+v"(xa[2]), "+v"(xa[3]));
                    if (rg + 1 < RG) {
                        const uint32_t xb = xb0 + (uint32_t)(rg + 1) * (16u * XROW);
#pragma unroll
                        for (uint32_t j = 0; j < 4u; j++) xr[(rg + 1) & 1][j] = dm_read16(xb + (xpos(8u * (j >> 1) + 2u * q + (j & 1u)) << 4));
                    }
                    v4f t0 = ENC == AENC_FP8BLK ? (v4f){0.0f, 0.0f, 0.0f, 0.0f} : acc0[rg];
                    v4f t1 = ENC == AENC_FP8BLK ? (v4f){0.0f, 0.0f, 0.0f, 0.0f} : acc1[rg];
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const v8bf B = __builtin_bit_cast(v8bf, xa[j]);
                        t0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_operand<ENC>(da, j), B, t0, 0, 0, 0);
                        if (TWO) t1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_operand<ENC>(db, j), B, t1, 0, 0, 0);
                    }
                    if (ENC == AENC_FP8BLK) {
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            acc0[rg][i] = fmaf(t0[i], sa, acc0[rg][i]);
                            /* (wide: the block's one scale; a copy of sa made before the wait above would hold
                             * what the register held before the read landed) */
                            if (TWO) acc1[rg][i] = fmaf(t1[i], WIDE ? sa : sb, acc1[rg][i]);
                        }
                    } else {
                        acc0[rg] = t0;
                        if (TWO) acc1[rg] = t1;
                    }
                }
            }
            st = st + 1u == DM_STAGES ? 0u : st + 1u;
            Sr = Sr + 1u == KS ? 0u : Sr + 1u;
            if (++S < KS) continue;
            /* ---- a tile is done: lane holds channels chw + 128 t + 4q + i of row rb + c ---- */
            const uint32_t tdone = t;
            S = 0u, t++;
            const uint32_t col = chw + tdone * BN + 4u * q;
            float4 s0 = pc0[0], s1 = pc1[0];
            if (ENC == AENC_FP8PC) {
#pragma unroll
                for (uint32_t t2 = 1; t2 < 4u; t2++)
                    if (tdone == t2) s0 = pc0[t2], s1 = pc1[t2];
            }
#pragma unroll
            for (int rg = 0; rg < RG; rg++) {
                v4f a0 = acc0[rg], a1 = acc1[rg];
                acc0[rg] = acc1[rg] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
                if (!valid[rg] || oi[rg] == PLOW_EXPERT_UNUSED) continue;
                if (ENC == AENC_FP8PC) {
                    a0[0] *= s0.x, a0[1] *= s0.y, a0[2] *= s0.z, a0[3] *= s0.w;
                    if (TWO) a1[0] *= s1.x, a1[1] *= s1.y, a1[2] *= s1.z, a1[3] *= s1.w;
                }
                if (GLU) {
                    uint2 o;
                    o.x = (uint32_t)f2bf(moe_glu(a0[0], a1[0], g.act, g.f0, g.f1)) | ((uint32_t)f2bf(moe_glu(a0[1], a1[1], g.act, g.f0, g.f1)) << 16);
                    o.y = (uint32_t)f2bf(moe_glu(a0[2], a1[2], g.act, g.f0, g.f1)) | ((uint32_t)f2bf(moe_glu(a0[3], a1[3], g.act, g.f0, g.f1)) << 16);
                    *(uint2*)((bf16_t*)g.out + (size_t)oi[rg] * N + col) = o;
                } else {
                    const float gt = gate[rg];
                    auto put = [&](const v4f& a, uint32_t cl) {
                        const float y0 = gt * a[0], y1 = gt * a[1], y2 = gt * a[2], y3 = gt * a[3];
                        if (g.out_bf16) {
                            uint2 o;
                            o.x = (uint32_t)f2bf(g.gate ? y0 : a[0]) | ((uint32_t)f2bf(g.gate ? y1 : a[1]) << 16);
                            o.y = (uint32_t)f2bf(g.gate ? y2 : a[2]) | ((uint32_t)f2bf(g.gate ? y3 : a[3]) << 16);
                            *(uint2*)((bf16_t*)g.out + (size_t)oi[rg] * N + cl) = o;
                        } else {
                            *(float4*)((float*)g.out + (size_t)oi[rg] * N + cl) = make_float4(y0, y1, y2, y3);
                        }
                    };
                    put(a0, col);
                    if (WIDE) put(a1, col + 16u); /* the second stream's channels */
                }
            }
        }
    }
}

template <int ENC, bool GLU, bool WIDE>
__device__ __forceinline__ void a16_dma_pick(const GroupA16& g, uint8_t* dm_raw) {
    DmWork w;
    if (!a16_dma_work<ENC, WIDE>(g, blockIdx.x, w)) return;
    if constexpr ((GLU || WIDE) && ENC != AENC_MXFP4) { /* (mxfp4 measured behind with private rows: the launcher leaves it out) */
        if (g.priv_rows && w.cnt <= DmPrivRows<ENC>::v) { /* a handful of rows: every wave on its own */
            a16_dma_body<ENC, GLU, 1, false, WIDE, true>(g, dm_raw, w);
            return;
        }
    }
    if constexpr (ENC == AENC_MXFP4) {
        if (g.K % 512u == 0u) { /* whole 16-byte pieces of E8M0 bytes per row: scales four steps at a time */
            if (w.cnt <= 16u) a16_dma_body<ENC, GLU, 1, true, WIDE>(g, dm_raw, w);
            else a16_dma_body<ENC, GLU, 2, true, WIDE>(g, dm_raw, w);
        } else {
            if (w.cnt <= 16u) a16_dma_body<ENC, GLU, 1, false, WIDE>(g, dm_raw, w);
            else a16_dma_body<ENC, GLU, 2, false, WIDE>(g, dm_raw, w);
        }
    } else {
        if (w.cnt <= 16u) a16_dma_body<ENC, GLU, 1, false, WIDE>(g, dm_raw, w);
        else if (w.cnt <= 32u) a16_dma_body<ENC, GLU, 2, false, WIDE>(g, dm_raw, w);
        else a16_dma_body<ENC, GLU, 4, false, WIDE>(g, dm_raw, w);
    }
}

/* One kernel, several instances of the body, picked per workgroup from its expert's row count (a16_dma_pick): the
 * private-row form for a handful of rows (fp8 and bf16 weights, two-stream shapes), else the one that covers the
 * rows in the fewest passes over the weights (16, 32 or 64 rows per pass; mxfp4 16 or 32, its rings fill the LDS at
 * 32). Routing is skewed: at 4 rows per expert on average the hot experts hold 30 to 60, and a second pass re-reads
 * the weights from memory (Qwen3 shape, 64 tokens: GLU 325 us with 16-row passes for all, 289 us with 32-row passes
 * for all, which in turn costs the few-row experts 3 % in row loads and multiplies they do not need). The DOWN holds
 * the bodies for tiles of 128 and of 256 channels; the launcher's grid says which (g.down_wide). */
template <int ENC, bool GLU>
__global__ __launch_bounds__(AK_THREADS) void k_group_a16_dma(GroupA16 g) {
    extern __shared__ __attribute__((aligned(16))) uint8_t dm_raw[];
    if (!form_is_mine(g)) return;
    if constexpr (!GLU) {
        /* slot-major DOWN: the f32 rows of slots that no expert serves are zeroed here, a slot per wave (the reference's
         * decode DOWN bodies do it, plow runtime/cpu/dev/golden/moe.c:76-80): one launch less */
        if (g.zs_table && !g.out_bf16) {
            const PlowMoeRoute* const tab = (const PlowMoeRoute*)g.zs_table;
            const uint32_t lane = threadIdx.x & 63u, n_waves = gridDim.x * AK_WAVES;
            for (uint32_t sl = blockIdx.x * AK_WAVES + (threadIdx.x >> 6); sl < g.zs_nslot; sl += n_waves) {
                const uint32_t e = tab[sl].eid;
                const bool served = e < g.E && g.wtab[(size_t)e * g.wcols + g.wsel0] != 0ull &&
                                    (!g.stab || g.stab[(size_t)e * g.wcols + g.wsel0] != 0ull);
                if (served) continue;
                for (uint32_t h = lane; h < g.N; h += WAVE) ((float*)g.out)[(size_t)sl * g.N + h] = 0.0f;
            }
        }
        if (g.down_wide) { /* tiles of 256 channels (the launcher's grid counts them so) */
            a16_dma_pick<ENC, GLU, true>(g, dm_raw);
            return;
        }
    }
    a16_dma_pick<ENC, GLU, false>(g, dm_raw);
}

template <int ENC, bool TWO> struct DmLdsMax2 { /* over the row-group counts and scale forms of one stream count */
    static constexpr bool MX = ENC == AENC_MXFP4;
    static constexpr size_t a = sizeof(DmLds<ENC, TWO, 1, false>), b = sizeof(DmLds<ENC, TWO, 2, false>),
                            c = MX ? sizeof(DmLds<ENC, TWO, 2, MX>) : sizeof(DmLds<ENC, TWO, 4, false>),
                            d = sizeof(DmLds<ENC, TWO, 1, MX>);
    static constexpr size_t e = (TWO && !MX) ? sizeof(DmLds<ENC, true, 1, false, true>) : 0, f = 0;
    static constexpr size_t ab = a > b ? a : b, cd = c > d ? c : d, ef = e > f ? e : f, abcd = ab > cd ? ab : cd, v = abcd > ef ? abcd : ef;
};
template <int ENC, bool GLU> struct DmLdsMax { /* the DOWN kernel holds the one-stream and the wide bodies */
    static constexpr size_t two = DmLdsMax2<ENC, true>::v, one = DmLdsMax2<ENC, false>::v;
    static constexpr size_t v = GLU ? two : (two > one ? two : one);
};
template <int ENC, bool GLU>
static int launch_a16_dma(const GroupA16& g, dim3 grid, hipStream_t st) {
    static_assert(DmLdsMax<ENC, GLU>::v <= 160u * 1024u, "the rings must fit the CU's LDS");
    k_group_a16_dma<ENC, GLU><<<grid, AK_THREADS, DmLdsMax<ENC, GLU>::v, st>>>(g);
    return 0;
}

/* Many rows per expert (16 and more on average): the fp8-weight arms run on the tiled kernel (loader and
 * consumer waves, 128-row tiles, weights decoded to bf16 in registers), which reads an expert's weights
 * once per 128 rows instead of once per 64 and each operand from LDS once per tile. It serves the table
 * layouts plow's ops use: block fp8 {gate, up, down} and per-channel fp8 {gate_up fused, down}; GLU gathers
 * its rows through a_idx (and may scatter through o_idx in per-channel mode: the slot-major ops), DOWN
 * reads aligned rows or, slot-major, the rows a_idx = o_idx names. Returns false when the call is not
 * of that kind (the streaming forms then serve it). */
/* behind_choice: the batch's row count is unknown to the host; the launch goes out behind the device-side choice
 * in g.form_ws and runs only if that names the tiled form */
template <bool GLU>
static bool a16_tiled_try(const GroupA16& g, hipStream_t st, int* rc, bool behind_choice = false) {
    if (!plow_moe_tuning().a16_tiled || !g.meta || g.bias || g.wmul > 1u || g.dense_rows) return false;
    /* mxfp4 DOWN: from 8 rows per expert on average (its streaming form re-streams an expert's weights per 32 rows
     * and decodes every weight once per pass: measured below) */
    const uint32_t per_e = (!GLU && g.enc == AENC_MXFP4) ? 8u : 16u;
    if (behind_choice ? (g.slots_hint != 0u || !g.form_ws || !plow_moe_tuning().form_on_device) : g.slots_hint < per_e * g.E) return false;
    const bool w16 = g.enc == AENC_BF16, w4 = g.enc == AENC_MXFP4;
    if (!w16 && !g.stab) return false;
    /* the table layout: fused pairs {gate_up, down} (per-channel fp8; bf16 through ops 75 / 76) or {gate, up, down} */
    const bool pc = g.enc == AENC_FP8PC || (w16 && g.wcols == 2u);
    if (!pc && !w16 && !w4 && g.enc != AENC_FP8BLK) return false;
    if (w4 && (!plow_moe_tuning().a16_tiled_mx || (!GLU && g.a_idx))) return false; /* aligned rows only */
    if (g.wrow0) return false;
    if (pc) {
        if (g.wcols != 2u || (GLU ? (g.wsel0 != 0u || g.wsel1 != 0u || g.wrow1 != g.N) : g.wsel0 != 1u)) return false;
    } else {
        if (g.wcols != 3u || g.wrow1 || (GLU ? (g.wsel0 != 0u || g.wsel1 != 1u) : g.wsel0 != 2u)) return false;
    }
    GroupW8A8 w = {};
    w.out = g.out, w.a = g.a, w.wtab = g.wtab, w.stab = g.stab, w.meta = g.meta;
    w.N = g.N, w.K = g.K, w.E = g.E, w.act = g.act, w.f0 = g.f0, w.f1 = g.f1;
    w.per_channel = pc ? 1u : 0u;
    w.w_bf16 = w16 ? 1u : 0u;
    w.w_mxfp4 = w4 ? 1u : 0u;
    if (GLU) {
        if (!g.a_idx || (g.o_idx && !pc)) return false;
        w.row_token = g.a_idx, w.row_partidx = g.o_idx, w.out_bf16 = 1u;
    } else {
        if (!g.o_idx || !g.gate || (g.a_idx && g.a_idx != g.o_idx)) return false;
        w.row_partidx = g.o_idx, w.row_gate = g.gate, w.part16 = g.out_bf16;
        w.a_slots = g.a_idx ? g.slots_hint : 0u;
    }
    if (!group_w8a8_tiled_serves(w)) return false;
    if (behind_choice) {
        if (!GLU && g.a_idx) return false; /* slot-major rows need the slot count, which such a caller states */
        *rc = launch_pick_form(g.form_ws, g.meta, g.E, st);
        if (*rc) return true;
        w.form_word = g.form_ws, w.form_want = 1u;
    }
    if (!GLU && g.zs_table) { /* (the streaming forms zero unserved slots themselves) */
        *rc = launch_zero_skipped((float*)g.out, g.zs_table, g.wtab, g.stab, g.wcols, g.wsel0, g.zs_nslot, g.E, g.N, st);
        if (*rc) return true;
    }
    *rc = launch_group_a16_tiled(w, GLU, st);
    return true;
}

/* K split of a dense op, second launch: output row m = the sum over the slices, in slice order, of the partial rows
 * the first launch wrote (part: [mats * S][M][N] f32, matrix-major), through the activation for the GLU (gate =
 * matrix 0, up = matrix 1); a thread takes four channels. */
__global__ __launch_bounds__(64) void k_ksplit_finish(bf16_t* __restrict__ out, const float* __restrict__ part, uint32_t M,
                                                       uint32_t N, uint32_t S, uint32_t glu, uint32_t act, float f0, float f1) {
    const size_t n4 = (size_t)M * (N / 4u), plane = (size_t)M * N;
    /* eight slices' loads go out together; the adds keep the slice order */
    auto sum = [&](const float* p) -> float4 {
        float4 a = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        for (uint32_t s0 = 0; s0 < S; s0 += 8u) {
            float4 t[8];
#pragma unroll
            for (uint32_t j = 0; j < 8u; j++) t[j] = s0 + j < S ? *(const float4*)(p + (size_t)(s0 + j) * plane) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
            for (uint32_t j = 0; j < 8u; j++) {
                if (s0 + j == 0u) a = t[0]; /* (0 + x would turn a -0 sum into +0) */
                else if (s0 + j < S) a.x += t[j].x, a.y += t[j].y, a.z += t[j].z, a.w += t[j].w;
            }
        }
        return a;
    };
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (size_t)gridDim.x * blockDim.x) {
        const float* p = part + i * 4u;
        float4 a = sum(p);
        if (glu) {
            const float4 b = sum(p + S * plane);
            a.x = moe_glu(a.x, b.x, act, f0, f1), a.y = moe_glu(a.y, b.y, act, f0, f1);
            a.z = moe_glu(a.z, b.z, act, f0, f1), a.w = moe_glu(a.w, b.w, act, f0, f1);
        }
        uint2 o;
        o.x = (uint32_t)f2bf(a.x) | ((uint32_t)f2bf(a.y) << 16);
        o.y = (uint32_t)f2bf(a.z) | ((uint32_t)f2bf(a.w) << 16);
        *(uint2*)(out + i * 4u) = o;
    }
}

template <bool GLU>
static int launch_a16(const GroupA16& g_in, hipStream_t st);

/* A dense op (one expert, bf16 weights) of a few rows has N / 128 channel tiles per matrix, a few dozen workgroups
 * on a chip of 256 CUs, each walking the whole K: the op then takes as long as one CU needs for its tile's rows
 * (shared expert of the small bf16 layer, 16 tokens: GLU 22 workgroups). Here K is split S ways: the streaming
 * DOWN kernel runs mats * S "experts" (slice s of matrix m) that write f32 partial rows into the caller's scratch,
 * and a second launch adds the slices up in slice order and applies the epilogue. Returns false when the op is not
 * of that kind or the scratch does not hold the partial rows. */
template <bool GLU>
static bool a16_dense_split_try(const GroupA16& g, hipStream_t st, int* rc) {
    const PlowMoeTuning& tune = plow_moe_tuning();
    if (!tune.a16_dense_split || tune.a16_regs || g.meta || g.wtab || !g.dense_rows || g.dense_rows >= 128u || g.E != 1u ||
        g.enc != AENC_BF16 || g.bias || !g.split_ws || !g.out_bf16 || g.ksplit || g.a_idx || g.o_idx || g.gate || g.wmul > 1u ||
        g.wrow0 || (GLU && g.wrow1))
        return false;
    const uint32_t n_cu = plow_moe_n_cu();
    if (!n_cu) return false;
    const uint32_t mats = GLU ? 2u : 1u, tiles = g.N / AK_BN, steps = g.K / 64u;
    if (g.K % 64u || g.K > 16384u || mats * tiles >= n_cu) return false;
    /* the fewest slices that give every CU a workgroup, each of four steps (256 k) at least; failing that the most */
    uint32_t S = 0u;
    for (uint32_t d = 2u; d * 4u <= steps; d++) {
        if (steps % d || (g.K / d) % 128u) continue; /* (the streaming form takes whole 128-k pairs of steps) */
        if ((uint64_t)mats * d * g.dense_rows * g.N * 4u > g.split_ws_bytes) break;
        S = d;
        if (mats * d * tiles >= n_cu) break;
    }
    if (S < 2u) return false;
    GroupA16 p = g;
    p.out = g.split_ws, p.out_bf16 = 0u, p.act = 0u;
    p.E = mats * S, p.ksplit = S, p.kpitch = g.K, p.K = g.K / S;
    p.split_ws = nullptr;
    *rc = launch_a16<false>(p, st);
    if (*rc) return true;
    const size_t n4 = (size_t)g.dense_rows * (g.N / 4u);
    const uint32_t blocks = (uint32_t)((n4 + 63u) / 64u); /* a wave per workgroup: the op is a handful of rows */
    k_ksplit_finish<<<blocks, 64, 0, st>>>((bf16_t*)g.out, (const float*)g.split_ws, g.dense_rows, g.N, S, GLU ? 1u : 0u, g.act, g.f0, g.f1);
    return true;
}

/* A dense op of many rows as a one-expert batch of the tiled kernel: this launch writes what that kernel reads from
 * memory into the caller's scratch: the expert's pointer row {w0, w1, w0}, its meta {first row 0, M rows} and the
 * identity row maps with gate 1. */
#define DENSE_TAB_BYTES 256u
__global__ __launch_bounds__(256) void k_dense_tables(uint8_t* base, const void* w0, const void* w1, uint32_t M, uint32_t map_bytes) {
    const uint32_t r = blockIdx.x * 256u + threadIdx.x;
    if (r == 0u) {
        uint64_t* const wtab = (uint64_t*)base;
        wtab[0] = (uint64_t)(uintptr_t)w0, wtab[1] = (uint64_t)(uintptr_t)w1, wtab[2] = (uint64_t)(uintptr_t)w0;
        int32_t* const meta = (int32_t*)(base + 64u);
        meta[0] = 0, meta[1] = (int32_t)M;
    }
    if (r < map_bytes / 4u) { /* the maps run on to a multiple of 256 rows: entries past the last row are pad rows */
        ((uint32_t*)(base + DENSE_TAB_BYTES))[r] = r < M ? r : PLOW_EXPERT_UNUSED;
        ((uint32_t*)(base + DENSE_TAB_BYTES + map_bytes))[r] = r < M ? r : PLOW_EXPERT_UNUSED;
        ((float*)(base + DENSE_TAB_BYTES + 2u * (size_t)map_bytes))[r] = r < M ? 1.0f : 0.0f;
    }
}

/* Dense ops beyond the rows the K split takes: the tiled MFMA kernel over bf16 weights, which reads an expert's
 * weights once per 128 rows where the streaming form re-streams them per 64 and has N / 128 workgroups in all. */
template <bool GLU>
static bool a16_dense_tiled_try(const GroupA16& g, hipStream_t st, int* rc) {
    const PlowMoeTuning& tune = plow_moe_tuning();
    if (!tune.a16_tiled || !tune.a16_dense_split || g.meta || g.wtab || g.dense_rows < 128u || g.E != 1u || g.enc != AENC_BF16 ||
        g.bias || !g.split_ws || !g.out_bf16 || g.ksplit || g.a_idx || g.o_idx || g.gate || g.wmul > 1u || g.wrow0 || g.wrow1)
        return false;
    const uint32_t M = g.dense_rows;
    const size_t map_bytes = (((size_t)M + 255u) & ~(size_t)255u) * 4u;
    if (map_bytes > 0x7FFFFFFFull || DENSE_TAB_BYTES + 3u * map_bytes > g.split_ws_bytes) return false;
    uint8_t* const base = (uint8_t*)g.split_ws;
    GroupA16 t = g;
    t.split_ws = nullptr, t.dense_rows = 0u, t.slots_hint = M;
    t.wtab = (const uint64_t*)base, t.meta = (const int32_t*)(base + 64u), t.wcols = 3u;
    if (GLU) t.wsel0 = 0u, t.wsel1 = 1u, t.a_idx = (const uint32_t*)(base + DENSE_TAB_BYTES);
    else t.wsel0 = t.wsel1 = 2u, t.o_idx = (const uint32_t*)(base + DENSE_TAB_BYTES + map_bytes),
         t.gate = (const float*)(base + DENSE_TAB_BYTES + 2u * map_bytes);
    /* would the tiled form take it? (asked before anything is launched) */
    {
        GroupW8A8 w = {};
        w.N = g.N, w.K = g.K, w.E = 1u, w.w_bf16 = 1u, w.meta = t.meta;
        if (!group_w8a8_tiled_serves(w)) return false;
    }
    k_dense_tables<<<(uint32_t)(map_bytes / 1024u), 256, 0, st>>>(base, g.wdirect[0], g.wdirect[1], M, (uint32_t)map_bytes);
    if (!a16_tiled_try<GLU>(t, st, rc, false)) *rc = PLOW_MOE_EINVAL; /* (the checks above are the tiled form's own) */
    return true;
}

template <bool GLU>
static int launch_a16(const GroupA16& g_in, hipStream_t st) {
    GroupA16 g = g_in;
    if (g.N == 0 || g.K == 0 || g.E == 0 || g.N % AK_BN || g.K % 128u) return PLOW_MOE_EINVAL;
    if ((uint64_t)g.E * (g.N / AK_BN) > 0x7FFFFFFFull) return PLOW_MOE_EINVAL;
    {
        int rc = 0;
        if (a16_dense_split_try<GLU>(g, st, &rc)) return rc;
        if (a16_dense_tiled_try<GLU>(g, st, &rc)) return rc;
    }
    if (group_a16_gemv_serves(g)) return launch_group_a16_gemv(g, GLU, st); /* a handful of rows in all */
    {
        int rc = 0;
        if (a16_tiled_try<GLU>(g, st, &rc)) return rc;
        /* no row count from the host: the tiled form goes out behind a choice made on the device from meta, and
         * so does the streaming form below; the one the choice does not name returns at once */
        if (a16_tiled_try<GLU>(g, st, &rc, true)) {
            if (rc) return rc;
            g.form_word = g.form_ws, g.form_want = 0u;
            g.zs_table = nullptr; /* zeroed by a launch of its own ahead of the tiled form */
        }
    }
    dim3 grid(g.E * (g.N / AK_BN));
    /* second form: needs whole steps of K (one 128-byte line per weight row) and the block scales of a
     * tile to fit its LDS table */
    bool dma = !plow_moe_tuning().a16_regs && !g.bias && g.K <= 16384u &&
               g.K % (g.enc == AENC_MXFP4 ? 256u : 128u) == 0u && (g.enc == AENC_BF16 || g.stab);
    if (dma && g.slots_hint) {
        /* The second form fills a CU with one workgroup. With a short K loop and between one and three
         * workgroups per CU in all, the start-up chains of dependent loads (tables, row maps, first steps)
         * run one after the other on a CU, and the first form, four workgroups to a CU, hides them
         * better (mxfp4 DOWN at one token: 39 against 62 microseconds). */
        const uint32_t n_cu = plow_moe_n_cu();
        if (!n_cu) return PLOW_MOE_EDEVICE;
        const uint64_t wgs = (uint64_t)(g.slots_hint < g.E ? g.slots_hint : g.E) * (g.N / AK_BN);
        const uint32_t steps = g.K / (g.enc == AENC_MXFP4 ? 256u : (g.enc == AENC_BF16 ? 64u : 128u));
        if (steps <= 16u && wgs > (uint64_t)n_cu && wgs < 3ull * (uint64_t)n_cu) dma = false;
    }
    g.down_wide = 0u;
    /* per-wave copies of an expert's few rows: ahead on fp8 and bf16 weights (Qwen3 shape, 64 tokens: GLU 261 -> 244 us;
     * small bf16 layer, 16 tokens: 110 -> 103 us), behind on mxfp4, whose step carries twice the row bytes per weight
     * byte (Kimi-K2 shape, 64 tokens: GLU 654 -> 681 us) */
    g.priv_rows = (plow_moe_tuning().a16_private_rows && g.enc != AENC_MXFP4) ? 1u : 0u;
    if (g.ksplit && !dma) return PLOW_MOE_EINVAL; /* (a16_dense_split_try asks for nothing the second form refuses) */
    if (!GLU && dma && g.N % (2u * AK_BN) == 0u && g.meta && plow_moe_tuning().a16_down_wide) {
        /* tiles of 256 channels while they still give every CU two workgroups and more */
        const uint32_t n_cu = plow_moe_n_cu();
        if (!n_cu) return PLOW_MOE_EDEVICE;
        const uint64_t hit = g.slots_hint && g.slots_hint < g.E ? g.slots_hint : g.E;
        if (hit * (g.N / (2u * AK_BN)) >= 2ull * n_cu) g.down_wide = 1u, grid = dim3(g.E * (g.N / (2u * AK_BN)));
    }
    if (!dma && !GLU && g.zs_table) { /* the register form leaves the unserved slots to a launch of their own */
        const int zrc = launch_zero_skipped((float*)g.out, g.zs_table, g.wtab, g.stab, g.wcols, g.wsel0, g.zs_nslot, g.E, g.N, st);
        if (zrc) return zrc;
        g.zs_table = nullptr;
    }
    switch (g.enc) {
    case AENC_BF16:
        if (dma) return launch_a16_dma<AENC_BF16, GLU>(g, grid, st);
        k_group_a16_stream<AENC_BF16, GLU><<<grid, AK_THREADS, 0, st>>>(g);
        break;
    case AENC_FP8BLK:
        if (dma) return launch_a16_dma<AENC_FP8BLK, GLU>(g, grid, st);
        k_group_a16_stream<AENC_FP8BLK, GLU><<<grid, AK_THREADS, 0, st>>>(g);
        break;
    case AENC_MXFP4:
        if (dma) return launch_a16_dma<AENC_MXFP4, GLU>(g, grid, st);
        k_group_a16_stream<AENC_MXFP4, GLU><<<grid, AK_THREADS, 0, st>>>(g);
        break;
    case AENC_FP8PC:
        if (dma) return launch_a16_dma<AENC_FP8PC, GLU>(g, grid, st);
        k_group_a16_stream<AENC_FP8PC, GLU><<<grid, AK_THREADS, 0, st>>>(g);
        break;
    default: return PLOW_MOE_EUNSUPPORTED;
    }
    return 0;
}

/* dynamic-LDS limits of every instance of the direct-to-LDS form, once per device (plow_moe_device_setup) */
template <int ENC, bool GLU>
static bool a16_set_attr() {
    return hipFuncSetAttribute((const void*)k_group_a16_dma<ENC, GLU>, hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)DmLdsMax<ENC, GLU>::v) == hipSuccess;
}
template <int ENC>
static bool a16_set_attrs() {
    return a16_set_attr<ENC, true>() && a16_set_attr<ENC, false>();
}
int plow_moe_a16_setup() {
    return a16_set_attrs<AENC_BF16>() && a16_set_attrs<AENC_FP8BLK>() && a16_set_attrs<AENC_MXFP4>() &&
                   a16_set_attrs<AENC_FP8PC>() ? 0 : PLOW_MOE_EDEVICE;
}

int launch_group_glu_a16(const GroupA16& g, hipStream_t st) { return launch_a16<true>(g, st); }
int launch_group_down_a16(const GroupA16& g, hipStream_t st) { return launch_a16<false>(g, st); }

__global__ void k_flat_tables(uint64_t* wtab, uint64_t* stab, uint64_t W, uint64_t S, uint32_t E, uint64_t w_stride,
                              uint64_t s_stride) {
    const uint32_t e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= E) return;
    for (int j = 0; j < 3; j++) {
        wtab[(size_t)e * 3u + j] = W + e * w_stride;
        stab[(size_t)e * 3u + j] = S + e * s_stride;
    }
}

int launch_flat_tables(uint64_t* wtab, uint64_t* stab, const void* W, const void* S, uint32_t E, size_t w_stride,
                       size_t s_stride, hipStream_t st) {
    if (E == 0) return PLOW_MOE_EINVAL;
    k_flat_tables<<<(E + 255u) / 256u, 256, 0, st>>>(wtab, stab, (uint64_t)(uintptr_t)W, (uint64_t)(uintptr_t)S, E,
                                                     (uint64_t)w_stride, (uint64_t)s_stride);
    return 0;
}

/* Slot-major ops: zero part[s][*] of every slot that no expert serves (sentinel id or a null weight
 * base), which the reference's decode DOWN bodies do (plow runtime/cpu/dev/golden/moe.c:76-80). */
__global__ __launch_bounds__(256) void k_zero_skipped(float* part, const PlowMoeRoute* table,
                                                      const uint64_t* wtab, const uint64_t* stab,
                                                      uint32_t wcols, uint32_t wsel, uint32_t nslot,
                                                      uint32_t E, uint32_t H) {
    const uint32_t s = blockIdx.x;
    if (s >= nslot) return;
    const uint32_t e = table[s].eid;
    if (e < E && wtab[(size_t)e * wcols + wsel] != 0ull && (!stab || stab[(size_t)e * wcols + wsel] != 0ull)) return;
    for (uint32_t h = threadIdx.x; h < H; h += 256u) part[(size_t)s * H + h] = 0.0f;
}

int launch_zero_skipped(float* part, const void* table, const uint64_t* wtab, const uint64_t* stab,
                        uint32_t wcols, uint32_t wsel, uint32_t nslot, uint32_t E, uint32_t H, hipStream_t st) {
    if (nslot == 0) return 0;
    k_zero_skipped<<<nslot, 256, 0, st>>>(part, (const PlowMoeRoute*)table, wtab, stab, wcols, wsel, nslot, E, H);
    return 0;
}
