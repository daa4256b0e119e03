/* oracle.c — CPU restatement of plow's MoE expert-FFN path, one function per device op.
 *
 * TEST INFRASTRUCTURE ONLY. This file is the checker the HIP operator is compared against (and the
 * "port" CPU baseline a benchmark may time). The shipped library never includes, links or calls it.
 *
 * Every op takes the same descriptor and handle table as the operator (include/plow_moe.h) with
 * HOST pointers in the table, in the reference's worker form fn(inst, slice, nblk, tensors):
 * slice s of nblk owns a share of the op's outputs, so nblk threads can run one op concurrently.
 *
 * What each function follows (paths relative to the plow tree):
 *   op 180 router score        runtime/cpu/dev/golden/f32_primitives.c:235-252
 *   op 83/56 router top-k      runtime/cpu/dev/golden/moe_route.c:27-86 (flat arm);
 *                              group-limited arm runtime/common/moe_route_key.h:61-80 +
 *                              runtime/amd/op_moe.h:377-420; shared tail slot op_moe.h:2417-2434;
 *                              logit scale op_moe.h:444-446; sqrt-softplus scores op_moe.h:485-494
 *   op 84 align                runtime/cpu/dev/golden/moe_route.c:91-127
 *   op 87/43 combine           runtime/cpu/dev/golden/moe_route.c:130-147; t_row0 / part16
 *                              runtime/amd/interp.hip:6605-6635
 *   op 1 RMSNorm (+ quant)     runtime/cpu/dev/golden/norm.c:6-43; 1x128 form runtime/amd/op_norm.h:486-551
 *   op 184 1x128 quant         runtime/amd/op_gemm_common.h:2582-2621
 *   op 32 per-row quant        runtime/cpu/dev/golden/fp8.c:9-30
 *   op 85/86 enc 0 (bf16)      runtime/cpu/dev/golden/moe_gemma.c:244-302 through the wtab[E][3]
 *                              table of runtime/amd/op_moe.h:1242-1249
 *   op 85/86 enc 1 arm 0       runtime/amd/op_moe.h:3299-3310 (per-128-K promotion), :3799-3823,
 *                              :3906-3927 (epilogues); decode twin op_moe.h:674-702
 *   op 85/86 enc 1 arm 2/3     runtime/amd/moe_pf_w8a8.h:1-19, :368-379, :401-473
 *   op 85/86 enc 2 arm 8, and
 *   op 48/49 (all enc)         runtime/cpu/dev/golden/moe.c:21-174 with runtime/cpu/dev/
 *                              mxfp4_common.h:30-40 as the row dot; op_moe.h:1234-1399
 *   op 85 enc 1 arm 6          runtime/amd/moe_pf_w8a8.h:118-121, :255-283 (quantizer + arm 2)
 *   op 85 enc 1 arm 4, and
 *   op 86 enc 1 arm 4/5        runtime/amd/moe_pf_w8a8.h:81-92 (the split), :251-283 (on the way in), :375-384
 *                              (both terms through a block's sum), :434-452 (on the way out)
 *   op 188/189/190             runtime/amd/op_moe_fp8_block128.h:7-88, op_gemm_common.h:1845-2010,
 *                              :2582-2621 (SCATTER), interp.hip:5282-5310; op 190 adds in aligned-row
 *                              order where the device adds atomically in no fixed order
 *   op 65/66                   runtime/cpu/dev/golden/fp8.c:33-41, :173-214
 *   op 81/82                   runtime/amd/op_moe.h:6655-6700 (per-row x per-channel epilogue)
 *   op 20 / op 8               runtime/cpu/dev/golden/gemm.c:45-96
 *   GLU activations            runtime/cpu/dev/golden/golden.h:101-133
 *
 * Parity pins are listed per function in tests/test_oracle_*.py. Unpinned at bit level (tolerance
 * level only): the f32 summation order INSIDE one 128-K block of the fp8 x fp8 arms, which the
 * reference leaves to its MFMA; this file sums a block with eight interleaved f32 partials. The
 * sqrt-softplus scores use the C library's expf / log1pf / sqrtf where the reference, device code only, uses
 * its device library's: parity with those bits is unpinned (the expression itself is pinned against f64 and
 * its closed-form ends).
 */
#define _GNU_SOURCE /* sched_getaffinity, pthread_setaffinity_np */
#include "oracle.h"
#include "codec.h"

#include <pthread.h>
#include <sched.h>
#include <stdlib.h>

#define TEN(in, T, k) ((in)->t[(k)] == PLOW_TENSOR_NONE ? (void*)0 : (T)[(in)->t[(k)]])

static void own_range(uint32_t n, uint32_t slice, uint32_t nblk, uint32_t* lo, uint32_t* hi) {
    const uint32_t per = (n + nblk - 1u) / nblk;
    const uint64_t a = (uint64_t)slice * per, b = a + per;
    *lo = a > n ? n : (uint32_t)a;
    *hi = b > n ? n : (uint32_t)b;
}

/* ---- GLU epilogue ------------------------------------------------------------------------------ */

static float act_gelu_tanh(float x) {
    const float c = 0.7978845608028654f * (x + 0.044715f * x * x * x);
    return 0.5f * x * (1.0f + tanhf(c));
}
static float act_silu(float x) { return x / (1.0f + expf(-x)); }
/* act 0 gelu_tanh, 1 silu; gate-only epilogues poison on the pair forms, as the reference's do
 * (plow runtime/cpu/dev/golden/golden.h:110-115). */
static float glu(float g, float u, uint32_t act) {
    if (act == 1u) return act_silu(g) * u;
    if (act == 0u) return act_gelu_tanh(g) * u;
    return NAN;
}
/* Every epilogue that takes the activation's immediates f0 / f1 (plow runtime/cpu/dev/golden/
 * golden.h:116-133): 2 situ (beta, linear beta), 3 swiglu_oai (alpha, limit; limit <= 0 poisons);
 * 4 the clamped SwiGLU of plow's AMD path only (runtime/amd/op_moe.h:236-239, limit in f1). */
static float act_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
static float glu_pair(float g, float u, uint32_t act, float f0, float f1) {
    if (act == 2u) return (f0 * tanhf(g / f0) * act_sigmoid(g)) * (f1 > 0.0f ? f1 * tanhf(u / f1) : u);
    if (act == 3u) {
        if (!(f1 > 0.0f)) return NAN;
        g = g < f1 ? g : f1;
        u = u < -f1 ? -f1 : (u > f1 ? f1 : u);
        return g * act_sigmoid(f0 * g) * (u + 1.0f);
    }
    if (act == 4u) {
        const float gc = fminf(g, f1);
        return (gc / (1.0f + expf(-gc))) * fminf(fmaxf(u, -f1), f1);
    }
    return glu(g, u, act);
}

/* ---- op 180: router score ---------------------------------------------------------------------- */

static void op_gemm_f32(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    float* out = TEN(in, T, 0);
    const orc_bf16* x = TEN(in, T, 1);
    const orc_bf16* w = TEN(in, T, 2);
    const uint32_t M = in->i[0], N = in->i[1], K = in->i[2];
    uint32_t lo, hi;
    own_range(N, slice, nblk, &lo, &hi);
    for (uint32_t m = 0; m < M; m++)
        for (uint32_t n = lo; n < hi; n++) {
            float s = 0.0f; /* one accumulator, ascending k; a bf16 product is exact in f32 */
            for (uint32_t k = 0; k < K; k++) {
                s += orc_bf2f(x[(size_t)m * K + k]) * orc_bf2f(w[(size_t)n * K + k]);
            }
            out[(size_t)m * N + n] = s;
        }
}

/* ---- ops 83 / 56: router top-k ----------------------------------------------------------------- */

static int group_active(uint32_t n_exp, uint32_t n_group, uint32_t topk_group) {
    return n_group > 1u && topk_group > 0u && topk_group < n_group &&
           n_group <= PLOW_ROUTE_MAX_GROUPS && n_exp % n_group == 0u;
}

static void route_one(PlowMoeRoute* tab, const void* logit, const float* bias, uint32_t n_exp,
                      uint32_t k, uint32_t flags, float route_scale, float logit_scale,
                      uint32_t n_group, uint32_t topk_group, float* score, uint64_t* key) {
    const int sigmoid = (flags & PLOW_ROUTE_SIGMOID) != 0, norm = (flags & PLOW_ROUTE_NORM_TOPK) != 0;
    const int f32l = (flags & PLOW_ROUTE_F32_LOGIT) != 0;
    const float ls = logit_scale != 0.0f ? logit_scale : 1.0f;
    for (uint32_t j = PLOW_ROUTE_MAX_TOPK; j < k; j++) { tab[j].eid = PLOW_EXPERT_UNUSED; tab[j].gate = 0.0f; }
    if (k > PLOW_ROUTE_MAX_TOPK) k = PLOW_ROUTE_MAX_TOPK;
#define LOGIT(e) ((f32l ? ((const float*)logit)[e] : orc_bf2f(((const orc_bf16*)logit)[e])) * ls)
    if (flags & PLOW_ROUTE_SQRT_SOFTPLUS) { /* runtime/amd/op_moe.h:485-494: log1p(exp(-|l|)) + max(l, 0) cannot overflow */
        for (uint32_t e = 0; e < n_exp; e++) {
            const float l = LOGIT(e);
            score[e] = sqrtf(log1pf(expf(-fabsf(l))) + fmaxf(l, 0.0f));
        }
    } else if (sigmoid) {
        for (uint32_t e = 0; e < n_exp; e++) score[e] = 1.0f / (1.0f + expf(-LOGIT(e)));
    } else {
        float m = -1e30f, s = 0.0f;
        for (uint32_t e = 0; e < n_exp; e++) { score[e] = LOGIT(e); if (score[e] > m) m = score[e]; }
        for (uint32_t e = 0; e < n_exp; e++) { score[e] = expf(score[e] - m); s += score[e]; }
        for (uint32_t e = 0; e < n_exp; e++) score[e] /= s;
    }
#undef LOGIT
    /* packed selection key: ord(score + bias) above the inverted id, so ties go to the lowest id */
    for (uint32_t e = 0; e < n_exp; e++)
        key[e] = ((uint64_t)orc_ord(score[e] + (bias ? bias[e] : 0.0f)) << 20) |
                 (uint64_t)((n_exp - 1u - e) & 0xFFFFFu);
    if (group_active(n_exp, n_group, topk_group)) {
        const uint32_t gsz = n_exp / n_group;
        uint64_t gk[PLOW_ROUTE_MAX_GROUPS];
        for (uint32_t g = 0; g < n_group; g++) {
            float m1 = -3.0e38f, m2 = -3.0e38f; /* top-2 of the group's BIASED scores, index order */
            for (uint32_t i = 0; i < gsz; i++) {
                const uint32_t e = g * gsz + i;
                const float s = score[e] + (bias ? bias[e] : 0.0f);
                if (s > m1) { m2 = m1; m1 = s; } else if (s > m2) m2 = s;
            }
            gk[g] = ((uint64_t)orc_ord(m1 + m2) << 8) | (uint64_t)((n_group - 1u - g) & 0xFFu);
        }
        for (uint32_t g = 0; g < n_group; g++) {
            uint32_t rank = 0;
            for (uint32_t f = 0; f < n_group; f++) rank += gk[f] > gk[g];
            if (rank >= topk_group) /* dropped group: its experts keep only their id bits */
                for (uint32_t i = 0; i < gsz; i++) {
                    const uint32_t e = g * gsz + i;
                    key[e] = (uint64_t)((n_exp - 1u - e) & 0xFFFFFu);
                }
        }
    }
    uint32_t win[PLOW_ROUTE_MAX_TOPK];
    for (uint32_t j = 0; j < k; j++) win[j] = n_exp - 1u;
    for (uint32_t e = 0; e < n_exp; e++) {
        uint32_t rank = 0;
        for (uint32_t f = 0; f < n_exp; f++) rank += key[f] > key[e];
        if (rank < k) win[rank] = e;
    }
    float gate[PLOW_ROUTE_MAX_TOPK], sum = 0.0f;
    for (uint32_t j = 0; j < k; j++) { gate[j] = score[win[j]]; sum += gate[j]; }
    for (uint32_t j = 0; j < k; j++) {
        if (norm && sum != 0.0f) gate[j] /= sum;
        gate[j] *= route_scale;
        tab[j].eid = win[j];
        tab[j].gate = gate[j];
    }
}

/* t0=table t1=logit t3=bias? i1=n_exp i2=k i3=flags i4=T(0=1) i5=shared_tail i6=n_group
 * i7=topk_group f0=route_scale f1=logit_scale. Token t is owned by slice t % nblk. */
static void op_router_topk(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    PlowMoeRoute* table = TEN(in, T, 0);
    const uint8_t* logit = TEN(in, T, 1);
    const float* bias = TEN(in, T, 3);
    const uint32_t n_exp = in->i[1], k = in->i[2], flags = in->i[3], nt = in->i[4] ? in->i[4] : 1u;
    const uint32_t tail = (in->op == PLOW_DOP_MOE_ROUTER_TOPK_PF && in->i[5]) ? 1u : 0u;
    const size_t esz = (flags & PLOW_ROUTE_F32_LOGIT) ? 4u : 2u;
    float* score = malloc((size_t)n_exp * 4u);
    uint64_t* key = malloc((size_t)n_exp * 8u);
    /* op 83 with t2 bound: the [T][i0] f64 accumulator of the deterministic fused combine is zeroed here
     * (plow runtime/amd/op_moe.h:2329-2340, runtime/amd/interp.hip:6479-6483) */
    double* det_acc = in->op == PLOW_DOP_MOE_ROUTER_TOPK_PF ? TEN(in, T, 2) : NULL;
    if (det_acc) {
        uint32_t lo, hi;
        own_range(nt, slice, nblk, &lo, &hi);
        for (size_t q = (size_t)lo * in->i[0]; q < (size_t)hi * in->i[0]; q++) det_acc[q] = 0.0;
    }
    for (uint32_t tok = slice; tok < nt; tok += nblk) {
        PlowMoeRoute* row = table + (size_t)tok * (k + tail);
        route_one(row, logit + (size_t)tok * n_exp * esz, bias, n_exp, k, flags, in->fj[0].f,
                  in->fj[1].f, in->i[6], in->i[7], score, key);
        if (tail) { row[k].eid = n_exp; row[k].gate = 1.0f; }
    }
    free(score);
    free(key);
}

/* ---- op 84: align ------------------------------------------------------------------------------ */

static void op_align(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    if (slice != 0u || nblk == 0u) return;
    int32_t* meta = TEN(in, T, 0);
    const PlowMoeRoute* table = TEN(in, T, 1);
    uint32_t* row_token = TEN(in, T, 2);
    uint32_t* row_partidx = TEN(in, T, 3);
    float* row_gate = TEN(in, T, 4);
    const uint32_t nt = in->i[0], E = in->i[1], k = in->i[2], nslot = nt * k;
    int32_t *rowoff = meta, *cnt = meta + E, *tilep = meta + 2u * E;
    for (uint32_t e = 0; e < E; e++) cnt[e] = 0;
    for (uint32_t s = 0; s < nslot; s++) if (table[s].eid < E) cnt[table[s].eid]++;
    uint32_t off = 0, tiles = 0;
    for (uint32_t e = 0; e < E; e++) {
        const uint32_t t = ((uint32_t)cnt[e] + PLOW_MPF_BM - 1u) / PLOW_MPF_BM;
        rowoff[e] = (int32_t)off;
        tilep[e] = (int32_t)tiles;
        tiles += t;
        off += t * PLOW_MPF_BM;
    }
    tilep[E] = (int32_t)tiles;
    for (uint32_t r = 0; r < off; r++) {
        row_token[r] = PLOW_EXPERT_UNUSED;
        row_partidx[r] = PLOW_EXPERT_UNUSED;
        row_gate[r] = 0.0f;
    }
    uint32_t* cur = calloc(E ? E : 1u, 4u);
    for (uint32_t s = 0; s < nslot; s++) { /* ascending slot => stable within an expert */
        const uint32_t e = table[s].eid;
        if (e >= E) continue;
        const uint32_t pos = (uint32_t)rowoff[e] + cur[e]++;
        row_token[pos] = s / k;
        row_partidx[pos] = s;
        row_gate[pos] = table[s].gate;
    }
    free(cur);
}

/* ---- ops 87 / 43: combine ---------------------------------------------------------------------- */

static void op_combine(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    const int pf = in->op == PLOW_DOP_MOE_COMBINE_PF;
    const uint32_t H = in->i[0], k = in->i[1], nt = pf ? (in->i[2] ? in->i[2] : 1u) : 1u;
    const size_t r0 = pf ? in->i[3] : 0u;
    const int part16 = pf && in->i[7];
    orc_bf16* out = (orc_bf16*)TEN(in, T, 0) + r0 * H;
    const orc_bf16* residual = TEN(in, T, 1);
    const orc_bf16* shared = TEN(in, T, 2);
    const uint8_t* part = TEN(in, T, 3);
    if (residual) residual += r0 * H;
    if (shared) shared += r0 * H;
    part += r0 * k * H * (part16 ? 2u : 4u);
    uint32_t lo, hi;
    own_range(nt * H, slice, nblk, &lo, &hi);
    /* i4: `part` is the f64 [T][H] fixed-point accumulator op 86 summed in place (k == 1): one stream,
     * scaled by 2^-32 on the way out (plow runtime/amd/op_moe.h:5510-5520) */
    const int det = pf && in->i[4];
    for (uint32_t i = lo; i < hi; i++) {
        const uint32_t tok = i / H, h = i - tok * H;
        float acc = residual ? orc_bf2f(residual[i]) : 0.0f;
        if (shared) acc += orc_bf2f(shared[i]);
        if (det) {
            acc += (float)(((const double*)TEN(in, T, 3) + r0 * H)[i] * 2.3283064365386962890625e-10);
            out[i] = orc_f2bf(acc);
            continue;
        }
        for (uint32_t j = 0; j < k; j++) {
            const size_t at = ((size_t)tok * k + j) * H + h;
            acc += part16 ? orc_bf2f(((const orc_bf16*)part)[at]) : ((const float*)part)[at];
        }
        out[i] = orc_f2bf(acc);
    }
}

/* ---- ops 184 / 32: activation quant ------------------------------------------------------------ */

/* t0=xq t1=x t2=scale(f32 [K/128][pitch]) i0=M i1=K i2=pitch(0 = M). */
static void op_quant_block128(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    uint8_t* xq = TEN(in, T, 0);
    const orc_bf16* x = TEN(in, T, 1);
    float* scale = TEN(in, T, 2);
    const uint32_t M = in->i[0], K = in->i[1], pitch = in->i[2] ? in->i[2] : M, G = K / 128u;
    uint32_t lo, hi;
    own_range(M, slice, nblk, &lo, &hi);
    for (uint32_t m = lo; m < hi; m++)
        for (uint32_t g = 0; g < G; g++) {
            const orc_bf16* src = x + (size_t)m * K + g * 128u;
            float amax = 1e-10f; /* the amax is floored, not the scale */
            for (uint32_t j = 0; j < 128u; j++) amax = fmaxf(amax, fabsf(orc_bf2f(src[j])));
            const float s = amax * (1.0f / 448.0f), inv = 1.0f / s;
            scale[(size_t)g * pitch + m] = s;
            for (uint32_t j = 0; j < 128u; j++)
                xq[(size_t)m * K + g * 128u + j] = orc_f32_to_e4m3(orc_bf2f(src[j]) * inv);
        }
}

/* t0=xq t1=x t2=a_scale(f32 [M]) i0=M i1=K; with t3=gate t4=up bound the row is first produced,
 * x = bf16(act(gate) * up) with act = i2 (0 gelu_tanh, 1 silu, else poison), stored, then quantized
 * (plow runtime/cpu/dev/golden/fp8.c:9-30). */
static void op_quant_row(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    uint8_t* xq = TEN(in, T, 0);
    orc_bf16* x = TEN(in, T, 1);
    float* scale = TEN(in, T, 2);
    const orc_bf16* gate = TEN(in, T, 3);
    const orc_bf16* up = TEN(in, T, 4);
    const uint32_t M = in->i[0], K = in->i[1];
    uint32_t lo, hi;
    own_range(M, slice, nblk, &lo, &hi);
    for (uint32_t m = lo; m < hi; m++) {
        orc_bf16* xr = x + (size_t)m * K;
        float amax = 0.0f;
        for (uint32_t k = 0; k < K; k++) {
            if (gate) xr[k] = orc_f2bf(glu(orc_bf2f(gate[(size_t)m * K + k]), orc_bf2f(up[(size_t)m * K + k]), in->i[2]));
            amax = fmaxf(amax, fabsf(orc_bf2f(xr[k])));
        }
        scale[m] = fmaxf(amax * (1.0f / 448.0f), 1e-12f);
        const float inv = 1.0f / scale[m];
        for (uint32_t k = 0; k < K; k++) xq[(size_t)m * K + k] = orc_f32_to_e4m3(orc_bf2f(xr[k]) * inv);
    }
}

/* ---- row dots, one per weight encoding --------------------------------------------------------- */

/* Every operand of this path (bf16, e4m3, e2m1) is exact in f32 and so is any product of two of
 * them, so a fused and an unfused multiply-add give the same bits; the ORDER of the additions is
 * what each function below fixes. */
static void decode_bf16_row(float* dst, const orc_bf16* src, uint32_t K) {
    for (uint32_t k = 0; k < K; k++) dst[k] = orc_bf2f(src[k]);
}
static float e4m3_lut[256]; /* orc_e4m3_to_f32 of every code, filled once by plow_oracle_exec */
static int e4m3_lut_ready;
static void decode_e4m3_row(float* dst, const uint8_t* src, uint32_t K) {
    for (uint32_t k = 0; k < K; k++) dst[k] = e4m3_lut[src[k]];
}
static void decode_mxfp4_row(float* dst, const uint8_t* src, uint32_t K) {
    for (uint32_t k = 0; k < K; k++) dst[k] = orc_mxfp4_at(src, k);
}

/* Plain ascending-k sum with one accumulator (golden/moe_gemma.c gm_dot_bf16, golden/fp8.c
 * dot_a_w8). */
static float dot_seq(const float* wf, const float* a, uint32_t K) {
    float acc = 0.0f;
    for (uint32_t k = 0; k < K; k++) acc += a[k] * wf[k];
    return acc;
}

/* Sum of one <=128-long block with eight interleaved f32 partials (the order inside a block is the
 * reference MFMA's and is not pinned). */
static float block_dot(const float* w, const float* a, uint32_t n) {
    float p[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    uint32_t k = 0;
    for (; k + 8u <= n; k += 8u)
        for (uint32_t j = 0; j < 8u; j++) p[j] += w[k + j] * a[k + j];
    for (; k < n; k++) p[k & 7u] += w[k] * a[k];
    return ((p[0] + p[4]) + (p[2] + p[6])) + ((p[1] + p[5]) + (p[3] + p[7]));
}

/* Block-fp8 weights, bf16 activations: per 128-K block, dot then `acc += dot * block_scale`.
 * srow = this channel's scale row [ceil(K/128)]. */
static float dot_fp8blk_a16(const float* wf, const float* srow, const float* a, uint32_t K) {
    float acc = 0.0f;
    for (uint32_t k0 = 0, kb = 0; k0 < K; k0 += 128u, kb++) {
        const uint32_t n = K - k0 < 128u ? K - k0 : 128u;
        acc += block_dot(wf + k0, a + k0, n) * srow[kb];
    }
    return acc;
}

/* Block-fp8 weights, 1x128-scaled e4m3 activations: acc = fmaf(t, as[kb] * ws[kb], acc),
 * ascending kb. */
static float dot_fp8blk_a8(const float* wf, const float* srow, const float* a, const float* as,
                           size_t as_stride, uint32_t K) {
    float acc = 0.0f;
    for (uint32_t k0 = 0, kb = 0; k0 < K; k0 += 128u, kb++)
        acc = fmaf(block_dot(wf + k0, a + k0, 128u), as[(size_t)kb * as_stride] * srow[kb], acc);
    return acc;
}

/* The same with two-term activations a ~= as * (hi + lo / 16) (plow runtime/amd/moe_pf_w8a8.h:375-384): the block's
 * lo products join its hi products at 2^-4 before the scales multiply. */
static float dot_fp8blk_a8_split(const float* wf, const float* srow, const float* ahi, const float* alo, const float* as,
                                 uint32_t K) {
    float acc = 0.0f;
    for (uint32_t k0 = 0, kb = 0; k0 < K; k0 += 128u, kb++) {
        const float t = block_dot(wf + k0, ahi + k0, 128u) + 0.0625f * block_dot(wf + k0, alo + k0, 128u);
        acc = fmaf(t, as[kb] * srow[kb], acc);
    }
    return acc;
}

/* One value into its two e4m3 terms (moe_pf_w8a8.h:84-92): hi = e4m3(t), lo = e4m3((t - hi) * 16) */
static void split_e4m3(float t, uint8_t* hi, uint8_t* lo) {
    *hi = orc_f32_to_e4m3(t);
    *lo = orc_f32_to_e4m3((t - e4m3_lut[*hi]) * 16.0f);
}

/* mxfp4 weights, bf16 activations (mxfp4_common.h plow_mxfp4_row_dot): sequential f32 per 32-block,
 * the E8M0 scale multiplied once per block. */
static float dot_mxfp4(const float* wf, const uint8_t* s, const float* a, uint32_t K) {
    float acc = 0.0f;
    for (uint32_t k0 = 0; k0 < K; k0 += 32u) {
        const uint32_t k1 = k0 + 32u < K ? k0 + 32u : K;
        float blk = 0.0f;
        for (uint32_t k = k0; k < k1; k++) blk += wf[k] * a[k];
        acc += blk * orc_e8m0(s[k0 / 32u]);
    }
    return acc;
}

/* ---- the activation quantizer of the fp4 x fp4 arm (A4W4) ------------------------------------------
 * E8M0 byte of a 32-block from its amax, mapping the amax onto e2m1's top code 6 (plow
 * runtime/amd/amd_common.h:1073-1111): 127 for amax not above zero, for +inf / NaN and for the three
 * smallest subnormals; else E - 1 - (M < 2^22) of the float's exponent and mantissa fields, clamped to
 * 1..254. */
static uint8_t mx_act_e8m0(float amax) {
    if (!(amax > 0.0f)) return 127u;
    uint32_t bits;
    memcpy(&bits, &amax, 4);
    const uint32_t E = bits >> 23;
    if (E == 0xFFu || bits < 4u) return 127u;
    int e = (int)E - 1 - (int)((bits & 0x7FFFFFu) < 0x400000u);
    if (e < 1) e = 1;
    if (e > 254) e = 254;
    return (uint8_t)e;
}
/* 1 / 2^(b - 127) (amd_common.h:731-741): exact; b = 254 gives the subnormal 2^-127 */
static float mx_act_inv(uint8_t b) {
    if (b == 254u) return orc_from_bits(0x00400000u);
    return orc_from_bits((uint32_t)(254u - b) << 23);
}
/* f32 -> e2m1 code on the ladder 0, .5, 1, 1.5, 2, 3, 4, 6: nearest, an exact midpoint goes AWAY from
 * zero, saturating at 6; NaN gives 7 with a clear sign, -0 a clear sign (amd_common.h:1031-1068) */
static uint8_t mx_act_fp4(float v) {
    const uint8_t sign = (v < 0.0f) ? 8u : 0u;
    const float a = fabsf(v);
    const uint8_t n = (uint8_t)(!(a < 0.25f) + !(a < 0.75f) + !(a < 1.25f) + !(a < 1.75f) + !(a < 2.5f) + !(a < 3.5f) +
                                !(a < 5.0f));
    return sign | n;
}
/* one 32-block: 16 bytes (element 2i in the low nibble of byte i) and its E8M0 byte
 * (plow runtime/amd/op_moe.h:4132-4179: amax over the block, then every value times the inverse scale) */
static void mx_act_quant32(const float* v, uint8_t* out16, uint8_t* sb_out) {
    float amax = 0.0f;
    for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(v[i]));
    const uint8_t sb = mx_act_e8m0(amax);
    const float inv = mx_act_inv(sb);
    for (int i = 0; i < 16; i++)
        out16[i] = (uint8_t)(mx_act_fp4(v[2 * i] * inv) | (mx_act_fp4(v[2 * i + 1] * inv) << 4));
    *sb_out = sb;
}
/* fp4 x fp4 dot of two decoded rows (raw e2m1 values) with their E8M0 rows: every 32-block's sum of
 * products is exact (multiples of 1/4 below 2^11), scaled by the exact power of two 2^(sa + sw - 254);
 * the order in which the matrix instruction adds the blocks is not specified, so the blocks are added
 * in f64 and rounded once */
static float dot_a4w4(const float* wf, const uint8_t* sw, const float* af, const uint8_t* sa, uint32_t K) {
    double acc = 0.0;
    for (uint32_t k0 = 0; k0 < K; k0 += 32u) {
        float blk = 0.0f;
        for (uint32_t k = k0; k < k0 + 32u; k++) blk += wf[k] * af[k];
        acc += (double)blk * (double)orc_e8m0(sw[k0 / 32u]) * (double)orc_e8m0(sa[k0 / 32u]);
    }
    return (float)acc;
}

/* One weight row of an expert matrix under `enc`, decoded to f32 without its scales. */
typedef struct {
    const float* sf;   /* enc 1: scale row [ceil(K/128)] */
    const uint8_t* sb; /* enc 2: E8M0 row [K/32] */
} RowScale;

static RowScale enc_row(uint32_t enc, const void* W, const void* S, uint32_t n, uint32_t K, float* wf) {
    RowScale rs = {NULL, NULL};
    if (enc == PLOW_MOE_ENC_BF16) {
        decode_bf16_row(wf, (const orc_bf16*)W + (size_t)n * K, K);
    } else if (enc == PLOW_MOE_ENC_MXFP4) {
        decode_mxfp4_row(wf, (const uint8_t*)W + (size_t)n * (K / 2u), K);
        rs.sb = (const uint8_t*)S + (size_t)n * (K / 32u);
    } else {
        decode_e4m3_row(wf, (const uint8_t*)W + (size_t)n * K, K);
        rs.sf = (const float*)S + (size_t)(n >> 7) * ((K + 127u) >> 7);
    }
    return rs;
}

/* bf16-activation dot of a decoded weight row. */
static float enc_dot(uint32_t enc, const float* wf, RowScale rs, const float* a, uint32_t K) {
    if (enc == PLOW_MOE_ENC_BF16) return dot_seq(wf, a, K);
    if (enc == PLOW_MOE_ENC_MXFP4) return dot_mxfp4(wf, rs.sb, a, K);
    return dot_fp8blk_a16(wf, rs.sf, a, K);
}

/* ---- ops 85 / 86: grouped experts over aligned rows -------------------------------------------- */

/* Decoded activation rows of one expert's live segment (pad rows flagged dead). */
typedef struct {
    float* a;        /* [cap][K] */
    uint8_t* live;   /* [cap] */
    uint32_t cap, K;
    uint32_t expert; /* which expert is cached, ~0 = none */
} RowCache;

static void cache_init(RowCache* c, uint32_t K) { c->a = NULL; c->live = NULL; c->cap = 0; c->K = K; c->expert = ~0u; }
static void cache_free(RowCache* c) { free(c->a); free(c->live); }
static void cache_fit(RowCache* c, uint32_t rows) {
    if (rows <= c->cap) return;
    free(c->a); free(c->live);
    c->cap = rows;
    c->a = malloc((size_t)rows * c->K * 4u);
    c->live = malloc(rows);
}

/* 85: t0=fu_g|fq t1=xn2|xq t2=wtab t3=stab t4=meta t5=row_token t6=xs t7=fs  i0=I i1=H i2=E i3=enc
 * i4=xs pitch i5=act i7=arm. Work item = (expert, 128-channel group); slices split E*(I/128)
 * (I rounded up). */
static void op_group_glu(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    const uint64_t* wtab = TEN(in, T, 2);
    const uint64_t* stab = TEN(in, T, 3);
    const int32_t* meta = TEN(in, T, 4);
    const uint32_t* row_token = TEN(in, T, 5);
    const uint32_t I = in->i[0], H = in->i[1], E = in->i[2], enc = in->i[3], act = in->i[5];
    const uint32_t arm = in->i[7], pitch = in->i[4];
    /* arm 6: t1 holds the bf16 rows; each 1x128 group is quantized with op 184's arithmetic and the
     * rest is arm 2 (plow runtime/amd/moe_pf_w8a8.h:118-121, :255-283) */
    /* arm 4: as arm 6 with two e4m3 terms per value, on the way in and on the way out: t0 = fq rows [hi I | lo I]
     * (plow runtime/amd/moe_pf_w8a8.h:115-117, :251-283, :434-452) */
    const int split = enc == PLOW_MOE_ENC_FP8BLK && arm == PLOW_MOE_ARM_W8A8_SPLIT;
    const int xq_inline = (enc == PLOW_MOE_ENC_FP8BLK && arm == PLOW_MOE_ARM_W8A8_XQ) || split;
    const int w8a8 = (enc == PLOW_MOE_ENC_FP8BLK && arm == PLOW_MOE_ARM_W8A8) || xq_inline;
    float* rowlo = NULL; /* arm 4: [cached row][H] the lo terms of the rows split here */
    uint32_t rowlo_cap = 0;
    /* enc 2, arm 0 (the reference's default for mxfp4): fp4 on both operands. t1 = bf16 rows, quantized per
     * 32 with mx_act_quant32; t0 = fu as mxfp4 [R][I/2]; t6 = row_partidx (pad rows are skipped);
     * t7 = the E8M0 rows [R][I/32] it writes (plow runtime/amd/interp.hip:6496-6499, op_moe.h:4183-4632) */
    const int a4w4 = enc == PLOW_MOE_ENC_MXFP4 && arm == PLOW_MOE_ARM_A16;
    uint8_t* rowsa = NULL; /* a4w4: [cached row][H/32] E8M0 bytes of the rows quantized here */
    uint32_t rowsa_cap = 0;
    const float* xs = TEN(in, T, 6);
    const uint32_t G = (I + 127u) / 128u, KB = (H + 127u) / 128u;
    float* rowxs = NULL; /* arm 6: [cached row][KB] scales of the rows quantized here */
    uint32_t rowxs_cap = 0;
    float* wg = malloc((size_t)H * 4u);
    float* wu = malloc((size_t)H * 4u);
    float* v = NULL;
    uint32_t vcap = 0;
    RowCache rc;
    cache_init(&rc, H);
    uint32_t lo, hi;
    own_range(E * G, slice, nblk, &lo, &hi);
    for (uint32_t it = lo; it < hi; it++) {
        const uint32_t e = it / G, g0 = it % G;
        const uint32_t r0 = (uint32_t)meta[e], cnt = (uint32_t)meta[E + e];
        const void* Wg = (const void*)(uintptr_t)wtab[(size_t)e * 3u + 0u];
        const void* Wu = (const void*)(uintptr_t)wtab[(size_t)e * 3u + 1u];
        if (cnt == 0u || !Wg) continue;
        const void* Sg = stab ? (const void*)(uintptr_t)stab[(size_t)e * 3u + 0u] : NULL;
        const void* Su = stab ? (const void*)(uintptr_t)stab[(size_t)e * 3u + 1u] : NULL;
        if (rc.expert != e) {
            cache_fit(&rc, cnt);
            if (xq_inline && rowxs_cap < cnt) { free(rowxs); rowxs = malloc((size_t)cnt * KB * 4u); rowxs_cap = cnt; }
            if (split && rowlo_cap < cnt) { free(rowlo); rowlo = malloc((size_t)cnt * H * 4u); rowlo_cap = cnt; }
            if (a4w4 && rowsa_cap < cnt) { free(rowsa); rowsa = malloc((size_t)cnt * (H / 32u)); rowsa_cap = cnt; }
            for (uint32_t q = 0; q < cnt; q++) {
                const uint32_t tok = row_token[r0 + q];
                rc.live[q] = tok != PLOW_EXPERT_UNUSED;
                if (!rc.live[q]) continue;
                if (xq_inline) {
                    const orc_bf16* src = (const orc_bf16*)TEN(in, T, 1) + (size_t)tok * H;
                    for (uint32_t kb = 0; kb < KB; kb++) {
                        float amax = 1e-10f; /* the amax is floored, not the scale */
                        for (uint32_t j = 0; j < 128u; j++) amax = fmaxf(amax, fabsf(orc_bf2f(src[kb * 128u + j])));
                        const float sc = amax * (1.0f / 448.0f), inv = 1.0f / sc;
                        rowxs[(size_t)q * KB + kb] = sc;
                        for (uint32_t j = 0; j < 128u; j++) {
                            const float t = orc_bf2f(src[kb * 128u + j]) * inv;
                            if (split) {
                                uint8_t bh, bl;
                                split_e4m3(t, &bh, &bl);
                                rc.a[(size_t)q * H + kb * 128u + j] = e4m3_lut[bh];
                                rowlo[(size_t)q * H + kb * 128u + j] = e4m3_lut[bl];
                            } else rc.a[(size_t)q * H + kb * 128u + j] = e4m3_lut[orc_f32_to_e4m3(t)];
                        }
                    }
                } else if (a4w4) { /* the row as raw e2m1 values plus its E8M0 bytes */
                    const orc_bf16* src = (const orc_bf16*)TEN(in, T, 1) + (size_t)tok * H;
                    for (uint32_t b = 0; b < H / 32u; b++) {
                        float v32[32];
                        uint8_t q16[16];
                        for (uint32_t j = 0; j < 32u; j++) v32[j] = orc_bf2f(src[b * 32u + j]);
                        mx_act_quant32(v32, q16, &rowsa[(size_t)q * (H / 32u) + b]);
                        for (uint32_t j = 0; j < 32u; j++)
                            rc.a[(size_t)q * H + b * 32u + j] = orc_e2m1((j & 1u) ? (uint8_t)(q16[j >> 1] >> 4) : (uint8_t)(q16[j >> 1] & 15u));
                    }
                } else if (w8a8) decode_e4m3_row(rc.a + (size_t)q * H, (const uint8_t*)TEN(in, T, 1) + (size_t)tok * H, H);
                else decode_bf16_row(rc.a + (size_t)q * H, (const orc_bf16*)TEN(in, T, 1) + (size_t)tok * H, H);
            }
            rc.expert = e;
        }
        const uint32_t n0 = g0 * 128u, n1 = n0 + 128u < I ? n0 + 128u : I;
        if (a4w4) {
            /* SwiGLU in f32, then every (row, 32 channels) block quantized to mxfp4 with its E8M0 byte */
            uint8_t* fq = TEN(in, T, 0);
            uint8_t* cs = TEN(in, T, 7);
            const uint32_t* rpi = TEN(in, T, 6);
            if (vcap < cnt) { free(v); v = malloc((size_t)cnt * 128u * 4u); vcap = cnt; }
            for (uint32_t n = n0; n < n1; n++) {
                const RowScale sg = enc_row(enc, Wg, Sg, n, H, wg);
                const RowScale su = enc_row(enc, Wu, Su, n, H, wu);
                for (uint32_t q = 0; q < cnt; q++) {
                    if (!rc.live[q]) continue;
                    const float* a = rc.a + (size_t)q * H;
                    const uint8_t* sa = rowsa + (size_t)q * (H / 32u);
                    v[(size_t)q * 128u + (n - n0)] =
                        glu_pair(dot_a4w4(wg, sg.sb, a, sa, H), dot_a4w4(wu, su.sb, a, sa, H), act, in->fj[0].f, in->fj[1].f);
                }
            }
            for (uint32_t q = 0; q < cnt; q++) {
                if (!rc.live[q] || (rpi && rpi[r0 + q] == PLOW_EXPERT_UNUSED)) continue;
                for (uint32_t c0 = 0; c0 < n1 - n0; c0 += 32u)
                    mx_act_quant32(v + (size_t)q * 128u + c0, fq + (size_t)(r0 + q) * (I / 2u) + (n0 + c0) / 2u,
                                   cs + (size_t)(r0 + q) * (I / 32u) + (n0 + c0) / 32u);
            }
        } else if (!w8a8) {
            orc_bf16* fu = TEN(in, T, 0);
            for (uint32_t n = n0; n < n1; n++) {
                const RowScale sg = enc_row(enc, Wg, Sg, n, H, wg);
                const RowScale su = enc_row(enc, Wu, Su, n, H, wu);
                for (uint32_t q = 0; q < cnt; q++) {
                    if (!rc.live[q]) continue;
                    const float* a = rc.a + (size_t)q * H;
                    fu[(size_t)(r0 + q) * I + n] =
                        orc_f2bf(glu_pair(enc_dot(enc, wg, sg, a, H), enc_dot(enc, wu, su, a, H), act, in->fj[0].f, in->fj[1].f));
                }
            }
        } else {
            /* fp8 x fp8: SwiGLU in f32, then the 1x128 output quant (amax floored at 1e-10) */
            uint8_t* fq = TEN(in, T, 0);
            float* fs = TEN(in, T, 7);
            if (vcap < cnt) { free(v); v = malloc((size_t)cnt * 128u * 4u); vcap = cnt; }
            for (uint32_t n = n0; n < n1; n++) {
                decode_e4m3_row(wg, (const uint8_t*)Wg + (size_t)n * H, H);
                decode_e4m3_row(wu, (const uint8_t*)Wu + (size_t)n * H, H);
                for (uint32_t q = 0; q < cnt; q++) {
                    if (!rc.live[q]) continue;
                    const uint32_t tok = row_token[r0 + q];
                    const float* a = rc.a + (size_t)q * H;
                    const float* as = xq_inline ? rowxs + (size_t)q * KB : xs + tok;
                    const uint32_t as_step = xq_inline ? 1u : pitch;
                    const float* al = split ? rowlo + (size_t)q * H : NULL;
                    const float g = split ? dot_fp8blk_a8_split(wg, (const float*)Sg + (size_t)g0 * KB, a, al, as, H)
                                          : dot_fp8blk_a8(wg, (const float*)Sg + (size_t)g0 * KB, a, as, as_step, H);
                    const float u = split ? dot_fp8blk_a8_split(wu, (const float*)Su + (size_t)g0 * KB, a, al, as, H)
                                          : dot_fp8blk_a8(wu, (const float*)Su + (size_t)g0 * KB, a, as, as_step, H);
                    v[(size_t)q * 128u + (n - n0)] = glu_pair(g, u, act, in->fj[0].f, in->fj[1].f);
                }
            }
            for (uint32_t q = 0; q < cnt; q++) {
                if (!rc.live[q]) continue;
                float amax = 1e-10f;
                for (uint32_t j = 0; j < n1 - n0; j++) amax = fmaxf(amax, fabsf(v[(size_t)q * 128u + j]));
                const float s = amax * (1.0f / 448.0f), inv = 1.0f / s;
                fs[(size_t)(r0 + q) * G + g0] = s;
                for (uint32_t j = 0; j < n1 - n0; j++) {
                    if (split) split_e4m3(v[(size_t)q * 128u + j] * inv, &fq[(size_t)(r0 + q) * 2u * I + n0 + j], &fq[(size_t)(r0 + q) * 2u * I + I + n0 + j]);
                    else fq[(size_t)(r0 + q) * I + n0 + j] = orc_f32_to_e4m3(v[(size_t)q * 128u + j] * inv);
                }
            }
        }
    }
    free(wg); free(wu); free(v); free(rowxs); free(rowsa); free(rowlo);
    cache_free(&rc);
}

/* 86: t0=part t1=fu_g|fq t2=wtab t3=stab t4=meta t5=fs t6=row_partidx t7=row_gate  i0=H i1=I i2=E
 * i3=enc i7=arm (2: f32 part, 3: bf16 part; enc 0/1 arm 0 and enc 2 arm 8: f32 part). */
/* One contribution of the deterministic fused combine in the fixed-point domain and its order-independent
 * add (plow runtime/amd/op_moe.h:2153-2163, :3855-3880): rint(clamp(v, +-2^17) * 2^32) is an integer below
 * 2^49, sums of up to 16 of them are exact in f64, so the slices may add in any order (a compare-and-swap
 * loop here; a device-scope f64 atomic on the GPU). */
static double det_q(float v) { return rint((double)fminf(fmaxf(v, -131072.0f), 131072.0f) * 4294967296.0); }
static void det_add(double* p, double q) {
    uint64_t* u = (uint64_t*)p;
    uint64_t old = __atomic_load_n(u, __ATOMIC_RELAXED);
    for (;;) {
        double d;
        memcpy(&d, &old, 8);
        d += q;
        uint64_t nw;
        memcpy(&nw, &d, 8);
        if (__atomic_compare_exchange_n(u, &old, nw, 0, __ATOMIC_RELAXED, __ATOMIC_RELAXED)) return;
    }
}

static void op_group_down(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    const uint64_t* wtab = TEN(in, T, 2);
    const uint64_t* stab = TEN(in, T, 3);
    const int32_t* meta = TEN(in, T, 4);
    const uint32_t* row_partidx = TEN(in, T, 6);
    const float* row_gate = TEN(in, T, 7);
    const uint32_t H = in->i[0], I = in->i[1], E = in->i[2], enc = in->i[3], arm = in->i[7];
    /* arms 4 / 5: t1 = fq rows [hi I | lo I], both terms through the block sums (plow runtime/amd/interp.hip:6560-6571) */
    const int split = enc == PLOW_MOE_ENC_FP8BLK && (arm == PLOW_MOE_ARM_W8A8_SPLIT || arm == PLOW_MOE_ARM_W8A8_SPLIT_P16);
    float* rowlo = NULL;
    uint32_t rowlo_cap = 0;
    const int w8a8 = (enc == PLOW_MOE_ENC_FP8BLK && (arm == PLOW_MOE_ARM_W8A8 || arm == PLOW_MOE_ARM_W8A8_P16)) || split;
    /* enc 2, arm 0 / 1: fp4 on both operands; t1 = fu as mxfp4 [R][I/2], t5 = its E8M0 rows [R][I/32];
     * arm 1 = bf16 part (plow runtime/amd/interp.hip:6581-6589: i7 = part16 on the generic body) */
    const int a4w4 = enc == PLOW_MOE_ENC_MXFP4 && (arm == PLOW_MOE_ARM_A16 || arm == 1u);
    const int part16 = (w8a8 && (arm == PLOW_MOE_ARM_W8A8_P16 || arm == PLOW_MOE_ARM_W8A8_SPLIT_P16)) || (a4w4 && arm == 1u);
    /* i5: t0 is the f64 [T][H] accumulator of the deterministic fused combine; log2(k) + 1, or 256 + k */
    const uint32_t det_k = !in->i[5] ? 0u : in->i[5] > 256u ? in->i[5] - 256u : 1u << (in->i[5] - 1u);
    const float* fs = TEN(in, T, 5);
    const uint32_t G = (H + 127u) / 128u, KB = (I + 127u) / 128u;
    float* wd = malloc((size_t)I * 4u);
    RowCache rc;
    cache_init(&rc, I);
    uint32_t lo, hi;
    own_range(E * G, slice, nblk, &lo, &hi);
    for (uint32_t it = lo; it < hi; it++) {
        const uint32_t e = it / G, g0 = it % G;
        const uint32_t r0 = (uint32_t)meta[e], cnt = (uint32_t)meta[E + e];
        const void* Wd = (const void*)(uintptr_t)wtab[(size_t)e * 3u + 2u];
        if (cnt == 0u || !Wd) continue;
        const void* Sd = stab ? (const void*)(uintptr_t)stab[(size_t)e * 3u + 2u] : NULL;
        if (rc.expert != e) {
            cache_fit(&rc, cnt);
            if (split && rowlo_cap < cnt) { free(rowlo); rowlo = malloc((size_t)cnt * I * 4u); rowlo_cap = cnt; }
            for (uint32_t q = 0; q < cnt; q++) {
                rc.live[q] = row_partidx[r0 + q] != PLOW_EXPERT_UNUSED;
                if (!rc.live[q]) continue;
                if (split) {
                    decode_e4m3_row(rc.a + (size_t)q * I, (const uint8_t*)TEN(in, T, 1) + (size_t)(r0 + q) * 2u * I, I);
                    decode_e4m3_row(rowlo + (size_t)q * I, (const uint8_t*)TEN(in, T, 1) + (size_t)(r0 + q) * 2u * I + I, I);
                } else if (w8a8) decode_e4m3_row(rc.a + (size_t)q * I, (const uint8_t*)TEN(in, T, 1) + (size_t)(r0 + q) * I, I);
                else if (a4w4) decode_mxfp4_row(rc.a + (size_t)q * I, (const uint8_t*)TEN(in, T, 1) + (size_t)(r0 + q) * (I / 2u), I);
                else decode_bf16_row(rc.a + (size_t)q * I, (const orc_bf16*)TEN(in, T, 1) + (size_t)(r0 + q) * I, I);
            }
            rc.expert = e;
        }
        const uint32_t h0 = g0 * 128u, h1 = h0 + 128u < H ? h0 + 128u : H;
        for (uint32_t h = h0; h < h1; h++) {
            RowScale rs = {NULL, NULL};
            if (w8a8) decode_e4m3_row(wd, (const uint8_t*)Wd + (size_t)h * I, I);
            else rs = enc_row(enc, Wd, Sd, h, I, wd);
            for (uint32_t q = 0; q < cnt; q++) {
                if (!rc.live[q]) continue;
                const uint32_t r = r0 + q, pidx = row_partidx[r];
                const float* a = rc.a + (size_t)q * I;
                const float acc = split ? dot_fp8blk_a8_split(wd, (const float*)Sd + (size_t)g0 * KB, a, rowlo + (size_t)q * I,
                                                              fs + (size_t)r * KB, I)
                                  : w8a8 ? dot_fp8blk_a8(wd, (const float*)Sd + (size_t)g0 * KB, a,
                                                       fs + (size_t)r * KB, 1u, I)
                                  : a4w4 ? dot_a4w4(wd, rs.sb, a, (const uint8_t*)TEN(in, T, 5) + (size_t)r * (I / 32u), I)
                                         : enc_dot(enc, wd, rs, a, I);
                const float val = row_gate[r] * acc;
                if (det_k) det_add((double*)TEN(in, T, 0) + (size_t)(pidx / det_k) * H + h, det_q(val));
                else if (part16) ((orc_bf16*)TEN(in, T, 0))[(size_t)pidx * H + h] = orc_f2bf(val);
                else ((float*)TEN(in, T, 0))[(size_t)pidx * H + h] = val;
            }
        }
    }
    free(wd); free(rowlo);
    cache_free(&rc);
}

/* ---- ops 48 / 49: table-driven decode experts (slot-major) ------------------------------------- */

/* 48: t0=fu[B*k][I] t1=x t2=table t3=wtab t4=stab  i0=slots i1=I i2=H i3=n_exp i4=slots per x row
 * (0 = one shared row) i5=act i6=enc. Slot s reads x row s / i4. Sentinel or null base: nothing
 * written. Slices split slots*I. */
static void op_dec_glu(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    orc_bf16* fu = TEN(in, T, 0);
    const orc_bf16* x = TEN(in, T, 1);
    const PlowMoeRoute* tab = TEN(in, T, 2);
    const uint64_t* wtab = TEN(in, T, 3);
    const uint64_t* stab = TEN(in, T, 4);
    const uint32_t nslot = in->i[0], I = in->i[1], H = in->i[2], E = in->i[3], kx = in->i[4];
    const uint32_t act = in->i[5], enc = in->i[6];
    float* a = malloc((size_t)H * 4u);
    float* wg = malloc((size_t)H * 4u);
    float* wu = malloc((size_t)H * 4u);
    uint32_t lo, hi, cur = ~0u;
    own_range(nslot * I, slice, nblk, &lo, &hi);
    for (uint32_t it = lo; it < hi; it++) {
        const uint32_t s = it / I, n = it % I, e = tab[s].eid;
        if (e >= E || !wtab[(size_t)e * 3u]) continue;
        const void* Wg = (const void*)(uintptr_t)wtab[(size_t)e * 3u + 0u];
        const void* Wu = (const void*)(uintptr_t)wtab[(size_t)e * 3u + 1u];
        const void* Sg = stab ? (const void*)(uintptr_t)stab[(size_t)e * 3u + 0u] : NULL;
        const void* Su = stab ? (const void*)(uintptr_t)stab[(size_t)e * 3u + 1u] : NULL;
        if (cur != s) { decode_bf16_row(a, x + (size_t)(kx ? s / kx : 0u) * H, H); cur = s; }
        const RowScale sg = enc_row(enc, Wg, Sg, n, H, wg);
        const RowScale su = enc_row(enc, Wu, Su, n, H, wu);
        fu[(size_t)s * I + n] = orc_f2bf(glu(enc_dot(enc, wg, sg, a, H), enc_dot(enc, wu, su, a, H), act));
    }
    free(a); free(wg); free(wu);
}

/* 49: t0=part[B*k][H] t1=fu t2=table t3=wtab t4=stab  i0=slots i1=H i2=I i3=n_exp i6=enc.
 * part[s] = gate_s * (Wd_e . fu[s]); sentinel or null base writes zeros. */
static void op_dec_down(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    float* part = TEN(in, T, 0);
    const orc_bf16* fu = TEN(in, T, 1);
    const PlowMoeRoute* tab = TEN(in, T, 2);
    const uint64_t* wtab = TEN(in, T, 3);
    const uint64_t* stab = TEN(in, T, 4);
    const uint32_t nslot = in->i[0], H = in->i[1], I = in->i[2], E = in->i[3], enc = in->i[6];
    float* a = malloc((size_t)I * 4u);
    float* wd = malloc((size_t)I * 4u);
    uint32_t lo, hi, cur = ~0u;
    own_range(nslot * H, slice, nblk, &lo, &hi);
    for (uint32_t it = lo; it < hi; it++) {
        const uint32_t s = it / H, h = it % H, e = tab[s].eid;
        const void* Wd = e < E ? (const void*)(uintptr_t)wtab[(size_t)e * 3u + 2u] : NULL;
        if (!Wd) { part[(size_t)s * H + h] = 0.0f; continue; }
        const void* Sd = stab ? (const void*)(uintptr_t)stab[(size_t)e * 3u + 2u] : NULL;
        if (cur != s) { decode_bf16_row(a, fu + (size_t)s * I, I); cur = s; }
        const RowScale rs = enc_row(enc, Wd, Sd, h, I, wd);
        part[(size_t)s * H + h] = tab[s].gate * enc_dot(enc, wd, rs, a, I);
    }
    free(a); free(wd);
}

/* ---- ops 65 / 66: per-output-channel fp8 decode experts ---------------------------------------- */

/* 65: t0=fu t1=x t2=table t3=ewt[E][2] t4=est[E][2]  i0=k i1=I i2=H i3=E i5=B(0 = 1)
 * i6 = activation (0 gelu_tanh, the only one the reference has; 1 silu).
 * ewt[e][0] = fused gate_up rows [2I][H] (gate rows first); est[e][0] = f32 [2I]. */
static void op_pc_glu(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    orc_bf16* fu = TEN(in, T, 0);
    const orc_bf16* x = TEN(in, T, 1);
    const PlowMoeRoute* tab = TEN(in, T, 2);
    const uint64_t* ewt = TEN(in, T, 3);
    const uint64_t* est = TEN(in, T, 4);
    const uint32_t k = in->i[0], I = in->i[1], H = in->i[2], E = in->i[3];
    const uint32_t rows = in->i[5] ? in->i[5] : 1u, act = in->i[6];
    float* a = malloc((size_t)H * 4u);
    float* wt = malloc((size_t)H * 4u);
    uint32_t lo, hi;
    own_range(rows * k, slice, nblk, &lo, &hi);
    for (uint32_t s = lo; s < hi; s++) {
        const uint32_t e = tab[s].eid;
        if (e >= E || !ewt[2u * e] || !est[2u * e]) continue;
        const uint8_t* w = (const uint8_t*)(uintptr_t)ewt[2u * e];
        const float* sc = (const float*)(uintptr_t)est[2u * e];
        decode_bf16_row(a, x + (size_t)(s / k) * H, H);
        for (uint32_t n = 0; n < I; n++) {
            decode_e4m3_row(wt, w + (size_t)n * H, H);
            const float g = dot_seq(wt, a, H) * sc[n];
            decode_e4m3_row(wt, w + (size_t)(I + n) * H, H);
            const float u = dot_seq(wt, a, H) * sc[I + n];
            fu[(size_t)s * I + n] = orc_f2bf(glu(g, u, act));
        }
    }
    free(a); free(wt);
}

/* 66: t0=part t1=fu t2=table t3=ewt t4=est  i0=k i1=H i2=I i3=E i5=B. */
static void op_pc_down(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    float* part = TEN(in, T, 0);
    const orc_bf16* fu = TEN(in, T, 1);
    const PlowMoeRoute* tab = TEN(in, T, 2);
    const uint64_t* ewt = TEN(in, T, 3);
    const uint64_t* est = TEN(in, T, 4);
    const uint32_t k = in->i[0], H = in->i[1], I = in->i[2], E = in->i[3];
    const uint32_t rows = in->i[5] ? in->i[5] : 1u;
    float* a = malloc((size_t)I * 4u);
    float* wt = malloc((size_t)I * 4u);
    uint32_t lo, hi;
    own_range(rows * k, slice, nblk, &lo, &hi);
    for (uint32_t s = lo; s < hi; s++) {
        const uint32_t e = tab[s].eid;
        float* pr = part + (size_t)s * H;
        if (e >= E || !ewt[2u * e + 1u] || !est[2u * e + 1u]) {
            for (uint32_t h = 0; h < H; h++) pr[h] = 0.0f;
            continue;
        }
        const uint8_t* w = (const uint8_t*)(uintptr_t)ewt[2u * e + 1u];
        const float* sc = (const float*)(uintptr_t)est[2u * e + 1u];
        decode_bf16_row(a, fu + (size_t)s * I, I);
        for (uint32_t h = 0; h < H; h++) {
            decode_e4m3_row(wt, w + (size_t)h * I, I);
            pr[h] = tab[s].gate * (dot_seq(wt, a, I) * sc[h]);
        }
    }
    free(a); free(wt);
}

/* ---- ops 81 / 82: grouped per-channel fp8 x per-row fp8 ---------------------------------------- */

/* 81: t0=fu(bf16 [R][I]) t1=xq8([T][H]) t2=ewt t3=meta t4=row_token t5=ascale(f32 [T]) t6=est
 *     i0=I i1=H i2=E i5=act. g = (sum_k xq.w) * (ascale[tok] * wsc[n]). */
static void op_pc_group_glu(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    orc_bf16* fu = TEN(in, T, 0);
    const uint8_t* xq = TEN(in, T, 1);
    const uint64_t* ewt = TEN(in, T, 2);
    const int32_t* meta = TEN(in, T, 3);
    const uint32_t* row_token = TEN(in, T, 4);
    const float* ascale = TEN(in, T, 5);
    const uint64_t* est = TEN(in, T, 6);
    const uint32_t I = in->i[0], H = in->i[1], E = in->i[2], act = in->i[5];
    float* a = malloc((size_t)H * 4u);
    float* wt = malloc((size_t)H * 4u);
    uint32_t lo, hi;
    own_range(E, slice, nblk, &lo, &hi);
    for (uint32_t e = lo; e < hi; e++) {
        const uint32_t r0 = (uint32_t)meta[e], cnt = (uint32_t)meta[E + e];
        if (cnt == 0u || !ewt[2u * e]) continue;
        const uint8_t* w = (const uint8_t*)(uintptr_t)ewt[2u * e];
        const float* sc = (const float*)(uintptr_t)est[2u * e];
        for (uint32_t r = r0; r < r0 + cnt; r++) {
            const uint32_t tok = row_token[r];
            if (tok == PLOW_EXPERT_UNUSED) continue;
            decode_e4m3_row(a, xq + (size_t)tok * H, H);
            const float as = ascale[tok];
            for (uint32_t n = 0; n < I; n++) {
                decode_e4m3_row(wt, w + (size_t)n * H, H);
                const float g = dot_seq(wt, a, H) * (as * sc[n]);
                decode_e4m3_row(wt, w + (size_t)(I + n) * H, H);
                const float u = dot_seq(wt, a, H) * (as * sc[I + n]);
                fu[(size_t)r * I + n] = orc_f2bf(glu(g, u, act));
            }
        }
    }
    free(a); free(wt);
}

/* 82: t0=part t1=fu8([R][I]) t2=ewt t3=meta t4=row_partidx t5=row_gate t6=est t7=fscale(f32 [R])
 *     i0=H i1=I i2=E. part = gate * acc * (fscale[r] * wsc[h]). */
static void op_pc_group_down(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    float* part = TEN(in, T, 0);
    const uint8_t* fu8 = TEN(in, T, 1);
    const uint64_t* ewt = TEN(in, T, 2);
    const int32_t* meta = TEN(in, T, 3);
    const uint32_t* row_partidx = TEN(in, T, 4);
    const float* row_gate = TEN(in, T, 5);
    const uint64_t* est = TEN(in, T, 6);
    const float* fscale = TEN(in, T, 7);
    const uint32_t H = in->i[0], I = in->i[1], E = in->i[2];
    float* a = malloc((size_t)I * 4u);
    float* wt = malloc((size_t)I * 4u);
    uint32_t lo, hi;
    own_range(E, slice, nblk, &lo, &hi);
    for (uint32_t e = lo; e < hi; e++) {
        const uint32_t r0 = (uint32_t)meta[e], cnt = (uint32_t)meta[E + e];
        if (cnt == 0u || !ewt[2u * e + 1u]) continue;
        const uint8_t* w = (const uint8_t*)(uintptr_t)ewt[2u * e + 1u];
        const float* sc = (const float*)(uintptr_t)est[2u * e + 1u];
        for (uint32_t r = r0; r < r0 + cnt; r++) {
            const uint32_t pidx = row_partidx[r];
            if (pidx == PLOW_EXPERT_UNUSED) continue;
            decode_e4m3_row(a, fu8 + (size_t)r * I, I);
            for (uint32_t h = 0; h < H; h++) {
                decode_e4m3_row(wt, w + (size_t)h * I, I);
                float y = row_gate[r] * dot_seq(wt, a, I);
                y *= fscale[r] * sc[h];
                part[(size_t)pidx * H + h] = y;
            }
        }
    }
    free(a); free(wt);
}

/* ---- ops 20 / 8: dense bf16 shared expert ------------------------------------------------------ */

static float dot_bf16_seq(const orc_bf16* a, const orc_bf16* b, uint32_t K) {
    float acc = 0.0f;
    for (uint32_t k = 0; k < K; k++) acc = fmaf(orc_bf2f(a[k]), orc_bf2f(b[k]), acc);
    return acc;
}

/* 20: t0=fu t1=x t2=W_gate t5=W_up  i0=M i1=N i2=K i5=act (biases t6/t7 are not on this path). */
static void op_gemm_glu(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    orc_bf16* C = TEN(in, T, 0);
    const orc_bf16* A = TEN(in, T, 1);
    const orc_bf16* Wg = TEN(in, T, 2);
    const orc_bf16* Wu = TEN(in, T, 5);
    const uint32_t M = in->i[0], N = in->i[1], K = in->i[2], act = in->i[5];
    uint32_t lo, hi;
    own_range(N, slice, nblk, &lo, &hi);
    for (uint32_t m = 0; m < M; m++)
        for (uint32_t n = lo; n < hi; n++) {
            const float g = dot_bf16_seq(A + (size_t)m * K, Wg + (size_t)n * K, K);
            const float u = dot_bf16_seq(A + (size_t)m * K, Wu + (size_t)n * K, K);
            C[(size_t)m * N + n] = orc_f2bf(glu(g, u, act));
        }
}

/* 8: t0=C t1=A t2=B  i0=M i1=N i2=K i4=a_row0 i5=c_row0. */
static void op_gemm(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    const uint32_t M = in->i[0], N = in->i[1], K = in->i[2];
    orc_bf16* C = (orc_bf16*)TEN(in, T, 0) + (size_t)in->i[5] * N;
    const orc_bf16* A = (const orc_bf16*)TEN(in, T, 1) + (size_t)in->i[4] * K;
    const orc_bf16* B = TEN(in, T, 2);
    uint32_t lo, hi;
    own_range(N, slice, nblk, &lo, &hi);
    for (uint32_t m = 0; m < M; m++)
        for (uint32_t n = lo; n < hi; n++)
            C[(size_t)m * N + n] = orc_f2bf(dot_bf16_seq(A + (size_t)m * K, B + (size_t)n * K, K));
}

/* ---- ops 75 / 76: bf16 grouped experts over the fused table ewt[E][2] = {gate_up [2I][H], down [H][I]}
 * (plow runtime/cpu/dev/golden/moe_gemma.c:244-302). 75: t0=fu_g t1=xn2 t2=ewt t3=meta t4=row_token
 * i0=I i1=H i2=n_exp i5=act; 76: t0=part t1=fu_g t2=ewt t3=meta t4=row_partidx t5=row_gate i0=H i1=I
 * i2=n_exp. Pad rows are skipped; a null table entry skips the expert. f32 accumulation in k order. */
static void op_group_glu_gemma(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    orc_bf16* fu = TEN(in, T, 0);
    const orc_bf16* x = TEN(in, T, 1);
    const uint64_t* ewt = TEN(in, T, 2);
    const int32_t* meta = TEN(in, T, 3);
    const uint32_t* row_token = TEN(in, T, 4);
    const uint32_t I = in->i[0], H = in->i[1], E = in->i[2], act = in->i[5];
    float* a = malloc((size_t)H * 4u);
    float* wg = malloc((size_t)H * 4u);
    float* wu = malloc((size_t)H * 4u);
    uint32_t lo, hi;
    own_range(E, slice, nblk, &lo, &hi);
    for (uint32_t e = lo; e < hi; e++) {
        const orc_bf16* W = (const orc_bf16*)(uintptr_t)ewt[(size_t)e * 2u];
        const uint32_t r0 = (uint32_t)meta[e], cnt = (uint32_t)meta[E + e];
        if (!W) continue;
        for (uint32_t n = 0; n < I; n++) {
            decode_bf16_row(wg, W + (size_t)n * H, H);
            decode_bf16_row(wu, W + (size_t)(I + n) * H, H);
            for (uint32_t r = r0; r < r0 + cnt; r++) {
                const uint32_t tok = row_token[r];
                if (tok == PLOW_EXPERT_UNUSED) continue;
                decode_bf16_row(a, x + (size_t)tok * H, H);
                fu[(size_t)r * I + n] = orc_f2bf(glu(dot_seq(wg, a, H), dot_seq(wu, a, H), act));
            }
        }
    }
    free(a); free(wg); free(wu);
}

static void op_group_down_gemma(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    float* part = TEN(in, T, 0);
    const orc_bf16* fu = TEN(in, T, 1);
    const uint64_t* ewt = TEN(in, T, 2);
    const int32_t* meta = TEN(in, T, 3);
    const uint32_t* row_partidx = TEN(in, T, 4);
    const float* row_gate = TEN(in, T, 5);
    const uint32_t H = in->i[0], I = in->i[1], E = in->i[2];
    float* a = malloc((size_t)I * 4u);
    float* wd = malloc((size_t)I * 4u);
    uint32_t lo, hi;
    own_range(E, slice, nblk, &lo, &hi);
    for (uint32_t e = lo; e < hi; e++) {
        const orc_bf16* W = (const orc_bf16*)(uintptr_t)ewt[(size_t)e * 2u + 1u];
        const uint32_t r0 = (uint32_t)meta[e], cnt = (uint32_t)meta[E + e];
        if (!W) continue;
        for (uint32_t h = 0; h < H; h++) {
            decode_bf16_row(wd, W + (size_t)h * I, I);
            for (uint32_t r = r0; r < r0 + cnt; r++) {
                const uint32_t pidx = row_partidx[r];
                if (pidx == PLOW_EXPERT_UNUSED) continue;
                decode_bf16_row(a, fu + (size_t)r * I, I);
                part[(size_t)pidx * H + h] = row_gate[r] * dot_seq(wd, a, I);
            }
        }
    }
    free(a); free(wd);
}

/* ---- ops 150 - 153: flat mxfp4 experts (plow runtime/cpu/dev/golden/moe.c) ------------------------
 * Expert e of a [E][N][K/2] fp4 tensor starts at W + e*N*(K/2), its E8M0 bytes at S + e*N*(K/32), its
 * bf16 bias at b + e*N. Gate / up rows of output n: layout 0 interleaved (2n, 2n + 1), layout 1 blocked
 * (n, I + n) (moe.c:12-16). The bias is added in f32 before the activation (GLU) and before the gate
 * multiply (DOWN). The GLU takes the pair-form activations with fj[0] / fj[1] as their immediates
 * (moe.c:32, 50). */
static float mx_flat_dot(const uint8_t* We, const uint8_t* Se, uint32_t row, const float* a, uint32_t K, float* wf) {
    decode_mxfp4_row(wf, We + (size_t)row * (K / 2u), K);
    return dot_mxfp4(wf, Se + (size_t)row * (K / 32u), a, K);
}

/* 150: t0=fu[B*k][I] t1=x[B][K] t2=table t3=W_gu t4=S_gu t5=bias? i0=k i1=I i2=K i3=n_exp i4=layout
 * i5=act i6=n_batch (0 = 1). Sentinel slot: nothing written (moe.c:21-60). */
static void op_glu_mx(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    orc_bf16* fu = TEN(in, T, 0);
    const orc_bf16* x = TEN(in, T, 1);
    const PlowMoeRoute* tab = TEN(in, T, 2);
    const uint8_t* W = TEN(in, T, 3);
    const uint8_t* S = TEN(in, T, 4);
    const orc_bf16* bias = TEN(in, T, 5);
    const uint32_t k = in->i[0], I = in->i[1], K = in->i[2], E = in->i[3], layout = in->i[4], act = in->i[5];
    const uint32_t B = in->i[6] ? in->i[6] : 1u;
    float* a = malloc((size_t)K * 4u);
    float* wf = malloc((size_t)K * 4u);
    uint32_t lo, hi, cur = ~0u;
    own_range(B * k * I, slice, nblk, &lo, &hi);
    for (uint32_t it = lo; it < hi; it++) {
        const uint32_t s = it / I, n = it % I, e = tab[s].eid;
        if (e >= E) continue;
        if (cur != s) { decode_bf16_row(a, x + (size_t)(s / k) * K, K); cur = s; }
        const uint8_t* We = W + (size_t)e * 2u * I * (K / 2u);
        const uint8_t* Se = S + (size_t)e * 2u * I * (K / 32u);
        const uint32_t rg = layout ? n : 2u * n, ru = layout ? I + n : 2u * n + 1u;
        float g = mx_flat_dot(We, Se, rg, a, K, wf), u = mx_flat_dot(We, Se, ru, a, K, wf);
        if (bias) { g += orc_bf2f(bias[(size_t)e * 2u * I + rg]); u += orc_bf2f(bias[(size_t)e * 2u * I + ru]); }
        fu[(size_t)s * I + n] = orc_f2bf(glu_pair(g, u, act, in->fj[0].f, in->fj[1].f));
    }
    free(a); free(wf);
}

/* 151: t0=part[B*k][H] t1=fu t2=table t3=W_d t4=S_d t5=bias? i0=k i1=H i2=I i3=n_exp i6=n_batch.
 * part[s][h] = gate_s * (W_e[h] . fu[s] + b_e[h]); sentinel slot: zeros (moe.c:65-92). */
static void op_down_mx(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    float* part = TEN(in, T, 0);
    const orc_bf16* fu = TEN(in, T, 1);
    const PlowMoeRoute* tab = TEN(in, T, 2);
    const uint8_t* W = TEN(in, T, 3);
    const uint8_t* S = TEN(in, T, 4);
    const orc_bf16* bias = TEN(in, T, 5);
    const uint32_t k = in->i[0], H = in->i[1], I = in->i[2], E = in->i[3], B = in->i[6] ? in->i[6] : 1u;
    float* a = malloc((size_t)I * 4u);
    float* wf = malloc((size_t)I * 4u);
    uint32_t lo, hi, cur = ~0u;
    own_range(B * k * H, slice, nblk, &lo, &hi);
    for (uint32_t it = lo; it < hi; it++) {
        const uint32_t s = it / H, h = it % H, e = tab[s].eid;
        if (e >= E) { part[(size_t)s * H + h] = 0.0f; continue; }
        if (cur != s) { decode_bf16_row(a, fu + (size_t)s * I, I); cur = s; }
        float acc = mx_flat_dot(W + (size_t)e * H * (I / 2u), S + (size_t)e * H * (I / 32u), h, a, I, wf);
        if (bias) acc += orc_bf2f(bias[(size_t)e * H + h]);
        part[(size_t)s * H + h] = tab[s].gate * acc;
    }
    free(a); free(wf);
}

/* 152: t0=fu_g[rows][I] t1=xn2[T][K] t2=W_gu t3=S_gu t4=meta t5=row_token t6=bias? i0=I i1=K i2=n_exp
 * i3=layout i5=act. Pad rows (token UNUSED) are skipped (moe.c:98-135). */
static void op_glu_mx_pf(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    orc_bf16* fu = TEN(in, T, 0);
    const orc_bf16* x = TEN(in, T, 1);
    const uint8_t* W = TEN(in, T, 2);
    const uint8_t* S = TEN(in, T, 3);
    const int32_t* meta = TEN(in, T, 4);
    const uint32_t* row_token = TEN(in, T, 5);
    const orc_bf16* bias = TEN(in, T, 6);
    const uint32_t I = in->i[0], K = in->i[1], E = in->i[2], layout = in->i[3], act = in->i[5];
    float* a = malloc((size_t)K * 4u);
    float* wf = malloc((size_t)K * 4u);
    uint32_t lo, hi;
    own_range(E, slice, nblk, &lo, &hi);
    for (uint32_t e = lo; e < hi; e++) {
        const uint32_t r0 = (uint32_t)meta[e], cnt = (uint32_t)meta[E + e];
        const uint8_t* We = W + (size_t)e * 2u * I * (K / 2u);
        const uint8_t* Se = S + (size_t)e * 2u * I * (K / 32u);
        for (uint32_t r = r0; r < r0 + cnt; r++) {
            const uint32_t tok = row_token[r];
            if (tok == PLOW_EXPERT_UNUSED) continue;
            decode_bf16_row(a, x + (size_t)tok * K, K);
            for (uint32_t n = 0; n < I; n++) {
                const uint32_t rg = layout ? n : 2u * n, ru = layout ? I + n : 2u * n + 1u;
                float g = mx_flat_dot(We, Se, rg, a, K, wf), u = mx_flat_dot(We, Se, ru, a, K, wf);
                if (bias) { g += orc_bf2f(bias[(size_t)e * 2u * I + rg]); u += orc_bf2f(bias[(size_t)e * 2u * I + ru]); }
                fu[(size_t)r * I + n] = orc_f2bf(glu_pair(g, u, act, in->fj[0].f, in->fj[1].f));
            }
        }
    }
    free(a); free(wf);
}

/* 153: t0=part[T*k][H] t1=fu_g t2=W_d t3=S_d t4=meta t5=bias? t6=row_partidx t7=row_gate i0=H i1=I
 * i2=n_exp. part[row_partidx[r]][h] = row_gate[r] * (W_e[h] . fu_g[r] + b_e[h]); pad rows dropped
 * (moe.c:140-174). */
static void op_down_mx_pf(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    float* part = TEN(in, T, 0);
    const orc_bf16* fu = TEN(in, T, 1);
    const uint8_t* W = TEN(in, T, 2);
    const uint8_t* S = TEN(in, T, 3);
    const int32_t* meta = TEN(in, T, 4);
    const orc_bf16* bias = TEN(in, T, 5);
    const uint32_t* row_partidx = TEN(in, T, 6);
    const float* row_gate = TEN(in, T, 7);
    const uint32_t H = in->i[0], I = in->i[1], E = in->i[2];
    float* a = malloc((size_t)I * 4u);
    float* wf = malloc((size_t)I * 4u);
    uint32_t lo, hi;
    own_range(E, slice, nblk, &lo, &hi);
    for (uint32_t e = lo; e < hi; e++) {
        const uint32_t r0 = (uint32_t)meta[e], cnt = (uint32_t)meta[E + e];
        for (uint32_t r = r0; r < r0 + cnt; r++) {
            const uint32_t pidx = row_partidx[r];
            if (pidx == PLOW_EXPERT_UNUSED) continue;
            decode_bf16_row(a, fu + (size_t)r * I, I);
            for (uint32_t h = 0; h < H; h++) {
                float acc = mx_flat_dot(W + (size_t)e * H * (I / 2u), S + (size_t)e * H * (I / 32u), h, a, I, wf);
                if (bias) acc += orc_bf2f(bias[(size_t)e * H + h]);
                part[(size_t)pidx * H + h] = row_gate[r] * acc;
            }
        }
    }
    free(a); free(wf);
}

/* ---- op 1: RMSNorm with its fused quantizers ------------------------------------------------------ */

/* t0=out t1=x t2=gamma? t3=xq? t4=scale? i0=rows i1=feat i2=out_row0 i4=128: 1x128 groups  f0=eps
 * (plow runtime/cpu/dev/golden/norm.c:6-43: sum of squares in index order, inv = 1 / sqrtf, out =
 * bf16(x * inv * gamma), per-row quant of the ROUNDED row with scale = max(amax / 448, 1e-12); the
 * 1x128 form of runtime/amd/op_norm.h:486-551 quantizes the rounded row like op 184). */
static void op_rmsnorm(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    orc_bf16* out = TEN(in, T, 0);
    const orc_bf16* x = TEN(in, T, 1);
    const orc_bf16* gamma = TEN(in, T, 2);
    uint8_t* q = TEN(in, T, 3);
    float* scale = TEN(in, T, 4);
    const uint32_t rows = in->i[0], feat = in->i[1], out_row0 = in->i[2], blk = in->i[4] == 128u;
    const float eps = in->fj[0].f;
    uint32_t lo, hi;
    own_range(rows, slice, nblk, &lo, &hi);
    for (uint32_t row = lo; row < hi; row++) {
        const orc_bf16* xr = x + (size_t)row * feat;
        orc_bf16* o = out + (size_t)(out_row0 + row) * feat;
        float ss = 0.0f;
        for (uint32_t i = 0; i < feat; i++) { const float v = orc_bf2f(xr[i]); ss += v * v; }
        const float inv = 1.0f / sqrtf(ss / (float)feat + eps);
        for (uint32_t i = 0; i < feat; i++) o[i] = orc_f2bf(orc_bf2f(xr[i]) * inv * (gamma ? orc_bf2f(gamma[i]) : 1.0f));
        if (!q) continue;
        if (blk) {
            for (uint32_t g = 0; g < feat / 128u; g++) {
                float amax = 1e-10f;
                for (uint32_t j = 0; j < 128u; j++) amax = fmaxf(amax, fabsf(orc_bf2f(o[g * 128u + j])));
                const float sc = amax * (1.0f / 448.0f), qi = 1.0f / sc;
                scale[(size_t)g * rows + row] = sc;
                for (uint32_t j = 0; j < 128u; j++) q[(size_t)row * feat + g * 128u + j] = orc_f32_to_e4m3(orc_bf2f(o[g * 128u + j]) * qi);
            }
        } else {
            float amax = 0.0f;
            for (uint32_t i = 0; i < feat; i++) amax = fmaxf(amax, fabsf(orc_bf2f(o[i])));
            scale[row] = fmaxf(amax * (1.0f / 448.0f), 1e-12f);
            const float qi = 1.0f / scale[row];
            for (uint32_t i = 0; i < feat; i++) q[(size_t)row * feat + i] = orc_f32_to_e4m3(orc_bf2f(o[i]) * qi);
        }
    }
}

/* ---- ops 188 / 189 / 190: block-fp8 chain with a bf16 intermediate and atomic reduction ---------- */

/* 188 (plow runtime/amd/op_moe_fp8_block128.h:7-47, op_gemm_common.h:1845-2010 with GLU, GATHER):
 * t0=fu t1=xq t2=xscale[H/128][T] t3=wtab t4=stab t5=meta t6=row_token  i0=I i1=H i2=E i3=T, fj[1] =
 * clamp limit (> 0: gate min, up both sides). fu[r][n] = bf16((g * (1 / (1 + expf(-g)))) * u) for the
 * rows r0 .. r0 + cnt of every expert (a row whose token is out of range computes on zeros), zeros
 * for the pad rows up to the next multiple of 64; an expert without gate or up weights zeroes all of
 * its rows. */
static void op_glu_fp8_block128(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    orc_bf16* fu = TEN(in, T, 0);
    const uint8_t* xq = TEN(in, T, 1);
    const float* xs = TEN(in, T, 2);
    const uint64_t* wtab = TEN(in, T, 3);
    const uint64_t* stab = TEN(in, T, 4);
    const int32_t* meta = TEN(in, T, 5);
    const uint32_t* row_token = TEN(in, T, 6);
    const uint32_t I = in->i[0], H = in->i[1], E = in->i[2], Tn = in->i[3];
    const float limit = in->fj[1].f;
    const uint32_t G = (I + 127u) / 128u, KB = (H + 127u) / 128u;
    float* wg = malloc((size_t)H * 4u);
    float* wu = malloc((size_t)H * 4u);
    float* zero_scale = calloc(KB, 4u);
    RowCache rc;
    cache_init(&rc, H);
    uint32_t lo, hi;
    own_range(E * G, slice, nblk, &lo, &hi);
    for (uint32_t it = lo; it < hi; it++) {
        const uint32_t e = it / G, g0 = it % G;
        const uint32_t r0 = (uint32_t)meta[e], cnt = (uint32_t)meta[E + e];
        if (cnt == 0u) continue;
        const uint32_t padded = (cnt + PLOW_MPF_BM - 1u) / PLOW_MPF_BM * PLOW_MPF_BM;
        const uint32_t n0 = g0 * 128u, n1 = n0 + 128u < I ? n0 + 128u : I;
        const void* Wg = (const void*)(uintptr_t)wtab[(size_t)e * 3u + 0u];
        const void* Wu = (const void*)(uintptr_t)wtab[(size_t)e * 3u + 1u];
        const uint32_t live_rows = (Wg && Wu) ? cnt : 0u;
        for (uint32_t q = live_rows; q < padded; q++)
            for (uint32_t n = n0; n < n1; n++) fu[(size_t)(r0 + q) * I + n] = 0;
        if (!live_rows) continue;
        const float* Sg = (const float*)(uintptr_t)stab[(size_t)e * 3u + 0u];
        const float* Su = (const float*)(uintptr_t)stab[(size_t)e * 3u + 1u];
        if (rc.expert != e) {
            cache_fit(&rc, cnt);
            for (uint32_t q = 0; q < cnt; q++) {
                const uint32_t tok = row_token[r0 + q];
                rc.live[q] = tok < Tn;
                if (rc.live[q]) decode_e4m3_row(rc.a + (size_t)q * H, xq + (size_t)tok * H, H);
                else memset(rc.a + (size_t)q * H, 0, (size_t)H * 4u);
            }
            rc.expert = e;
        }
        for (uint32_t n = n0; n < n1; n++) {
            decode_e4m3_row(wg, (const uint8_t*)Wg + (size_t)n * H, H);
            decode_e4m3_row(wu, (const uint8_t*)Wu + (size_t)n * H, H);
            for (uint32_t q = 0; q < cnt; q++) {
                const float* a = rc.a + (size_t)q * H;
                const float* as = rc.live[q] ? xs + row_token[r0 + q] : zero_scale;
                const size_t step = rc.live[q] ? Tn : 1u;
                float g = dot_fp8blk_a8(wg, Sg + (size_t)g0 * KB, a, as, step, H);
                float u = dot_fp8blk_a8(wu, Su + (size_t)g0 * KB, a, as, step, H);
                if (limit > 0.0f) {
                    g = fminf(g, limit);
                    u = fminf(fmaxf(u, -limit), limit);
                }
                fu[(size_t)(r0 + q) * I + n] = orc_f2bf((g * (1.0f / (1.0f + expf(-g)))) * u);
            }
        }
    }
    free(wg); free(wu); free(zero_scale);
    cache_free(&rc);
}

/* 189 (op_moe_fp8_block128.h:49-55, op_gemm_common.h:2582-2621 with SCATTER; interp.hip:5291-5300):
 * t0=hq[T*topk][I] t1=fu t2=hscale[I/128][T*topk] t3=meta t4=row_partidx t5=out bf16[T][H]
 * i0=I i1=E i2=topk i3=T i4=H. Every aligned row of the tilep[E] * 64 whose slot is in range is
 * quantized 1x128 into its slot's row; out is zeroed. */
static void op_moe_quant_block128(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    uint8_t* hq = TEN(in, T, 0);
    const orc_bf16* fu = TEN(in, T, 1);
    float* hscale = TEN(in, T, 2);
    const int32_t* meta = TEN(in, T, 3);
    const uint32_t* row_partidx = TEN(in, T, 4);
    orc_bf16* out = TEN(in, T, 5);
    const uint32_t I = in->i[0], E = in->i[1], topk = in->i[2], Tn = in->i[3], H = in->i[4];
    const uint32_t rows = (uint32_t)meta[3u * E] * PLOW_MPF_BM, slots = Tn * topk, G = I / 128u;
    uint32_t lo, hi;
    own_range(rows, slice, nblk, &lo, &hi);
    for (uint32_t r = lo; r < hi; r++) {
        const uint32_t dst = row_partidx[r];
        if (dst >= slots) continue;
        for (uint32_t g = 0; g < G; g++) {
            const orc_bf16* src = fu + (size_t)r * I + g * 128u;
            float amax = 1e-10f;
            for (uint32_t j = 0; j < 128u; j++) amax = fmaxf(amax, fabsf(orc_bf2f(src[j])));
            const float sc = amax * (1.0f / 448.0f), inv = 1.0f / sc;
            hscale[(size_t)g * slots + dst] = sc;
            for (uint32_t j = 0; j < 128u; j++)
                hq[(size_t)dst * I + g * 128u + j] = orc_f32_to_e4m3(orc_bf2f(src[j]) * inv);
        }
    }
    own_range(Tn, slice, nblk, &lo, &hi);
    if (hi > lo) memset(out + (size_t)lo * H, 0, (size_t)(hi - lo) * H * 2u);
}

/* 190 (op_moe_fp8_block128.h:57-88 with ATOMIC, op_gemm_common.h:1845-2010 with GATHER, WEIGHTED,
 * SCATTER, ATOMIC): t0=out t1=hq t2=hscale t3=wtab t4=stab t5=meta t6=row_partidx t7=row_gate
 * i0=I i1=H i2=E i3=topk i4=T. out[slot / topk][h] += bf16(gate * (Wd[h] . hq[slot])), each addition
 * rounded to bf16. The device adds with atomics in no fixed order; this restatement adds in aligned-row
 * order (one of the orders the device may take), on slice 0 alone. */
static void op_moe_down_block128(const PlowDevInst* in, uint32_t slice, uint32_t nblk, void* const* T) {
    (void)nblk;
    if (slice != 0u) return;
    orc_bf16* out = TEN(in, T, 0);
    const uint8_t* hq = TEN(in, T, 1);
    const float* hscale = TEN(in, T, 2);
    const uint64_t* wtab = TEN(in, T, 3);
    const uint64_t* stab = TEN(in, T, 4);
    const int32_t* meta = TEN(in, T, 5);
    const uint32_t* row_partidx = TEN(in, T, 6);
    const float* row_gate = TEN(in, T, 7);
    const uint32_t I = in->i[0], H = in->i[1], E = in->i[2], topk = in->i[3], Tn = in->i[4];
    const uint32_t slots = Tn * topk, KB = (I + 127u) / 128u;
    float* wd = malloc((size_t)I * 4u);
    RowCache rc;
    cache_init(&rc, I);
    for (uint32_t e = 0; e < E; e++) {
        const uint32_t r0 = (uint32_t)meta[e], cnt = (uint32_t)meta[E + e];
        const void* Wd = (const void*)(uintptr_t)wtab[(size_t)e * 3u + 2u];
        if (cnt == 0u || !Wd) continue;
        const float* Sd = (const float*)(uintptr_t)stab[(size_t)e * 3u + 2u];
        cache_fit(&rc, cnt);
        for (uint32_t q = 0; q < cnt; q++) {
            const uint32_t dst = row_partidx[r0 + q];
            rc.live[q] = dst < slots;
            if (rc.live[q]) decode_e4m3_row(rc.a + (size_t)q * I, hq + (size_t)dst * I, I);
        }
        for (uint32_t h = 0; h < H; h++) {
            decode_e4m3_row(wd, (const uint8_t*)Wd + (size_t)h * I, I);
            for (uint32_t q = 0; q < cnt; q++) {
                if (!rc.live[q]) continue;
                const uint32_t dst = row_partidx[r0 + q];
                const float acc = dot_fp8blk_a8(wd, Sd + (size_t)(h / 128u) * KB, rc.a + (size_t)q * I, hscale + dst, slots, I);
                orc_bf16* o = out + (size_t)(dst / topk) * H + h;
                *o = orc_f2bf(orc_bf2f(*o) + orc_bf2f(orc_f2bf(acc * row_gate[r0 + q])));
            }
        }
    }
    free(wd);
    cache_free(&rc);
}

/* ---- dispatch ---------------------------------------------------------------------------------- */

typedef void (*op_fn)(const PlowDevInst*, uint32_t, uint32_t, void* const*);

static op_fn resolve(uint16_t op) {
    switch (op) {
    case PLOW_DOP_GEMM_F32: return op_gemm_f32;
    case PLOW_DOP_MOE_ROUTER_TOPK:
    case PLOW_DOP_MOE_ROUTER_TOPK_PF: return op_router_topk;
    case PLOW_DOP_MOE_ALIGN_PF: return op_align;
    case PLOW_DOP_MOE_COMBINE:
    case PLOW_DOP_MOE_COMBINE_PF: return op_combine;
    case PLOW_DOP_QUANT_FP8_BLOCK128: return op_quant_block128;
    case PLOW_DOP_QUANT_FP8: return op_quant_row;
    case PLOW_DOP_MOE_GROUP_GLU_PF: return op_group_glu;
    case PLOW_DOP_MOE_GROUP_DOWN_PF: return op_group_down;
    case PLOW_DOP_MOE_GROUP_GLU_FP8_BLK: return op_dec_glu;
    case PLOW_DOP_MOE_GROUP_DOWN_FP8_BLK: return op_dec_down;
    case PLOW_DOP_MOE_EXPERT_GLU_GEMMA_FP8: return op_pc_glu;
    case PLOW_DOP_MOE_EXPERT_DOWN_GEMMA_FP8: return op_pc_down;
    case PLOW_DOP_MOE_GROUP_GLU_GEMMA_PF_W8A8: return op_pc_group_glu;
    case PLOW_DOP_MOE_GROUP_DOWN_GEMMA_PF_W8A8: return op_pc_group_down;
    case PLOW_DOP_GEMM_GLU: return op_gemm_glu;
    case PLOW_DOP_GEMM: return op_gemm;
    case PLOW_DOP_MOE_GROUP_GLU_GEMMA_PF: return op_group_glu_gemma;
    case PLOW_DOP_MOE_GROUP_DOWN_GEMMA_PF: return op_group_down_gemma;
    case PLOW_DOP_MOE_GLU_MX: return op_glu_mx;
    case PLOW_DOP_MOE_DOWN_MX: return op_down_mx;
    case PLOW_DOP_MOE_GLU_MX_PF: return op_glu_mx_pf;
    case PLOW_DOP_MOE_DOWN_MX_PF: return op_down_mx_pf;
    case PLOW_DOP_RMSNORM: return op_rmsnorm;
    case PLOW_DOP_MOE_GLU_FP8_BLOCK128: return op_glu_fp8_block128;
    case PLOW_DOP_MOE_QUANT_FP8_BLOCK128: return op_moe_quant_block128;
    case PLOW_DOP_MOE_DOWN_FP8_BLOCK128: return op_moe_down_block128;
    default: return NULL;
    }
}

typedef struct {
    op_fn fn;
    const PlowDevInst* in;
    void* const* T;
    uint32_t slice, nblk;
} Job;

/* Timing runs pin worker s to the s-th CPU the process may run on, as plow's CPU benches do with their
 * worker pool (runtime/tests/cpu_dev_moe_gemma_test.c:109-155); off by default (tests do not care). */
static int g_pin_workers = 0;
void plow_oracle_pin_workers(int on) { g_pin_workers = on; }

static void* job_main(void* p) {
    Job* j = p;
    if (g_pin_workers) {
        cpu_set_t allowed, one;
        if (sched_getaffinity(0, sizeof allowed, &allowed) == 0) {
            const int n = CPU_COUNT(&allowed);
            int want = n > 0 ? (int)(j->slice % (uint32_t)n) : -1;
            for (int c = 0; c < CPU_SETSIZE && want >= 0; c++) {
                if (!CPU_ISSET(c, &allowed)) continue;
                if (want-- == 0) {
                    CPU_ZERO(&one);
                    CPU_SET(c, &one);
                    (void)pthread_setaffinity_np(pthread_self(), sizeof one, &one);
                    break;
                }
            }
        }
    }
    j->fn(j->in, j->slice, j->nblk, j->T);
    return NULL;
}

/* plow's CPU workers run with flush-to-zero and denormals-are-zero set (MXCSR bits 15 and 6, plow
 * runtime/cpu/dev/isa_detect.c:158-164): f32 results and operands below 2^-126 read as zero. The
 * restatement runs the same way (threads inherit the mode) and puts the caller's mode back. */
#if defined(__x86_64__)
static unsigned fp_mode_enter(void) {
    const unsigned old = __builtin_ia32_stmxcsr();
    __builtin_ia32_ldmxcsr(old | 0x8040u);
    return old;
}
static void fp_mode_leave(unsigned old) { __builtin_ia32_ldmxcsr((__builtin_ia32_stmxcsr() & ~0x8040u) | (old & 0x8040u)); }
#else
static unsigned fp_mode_enter(void) { return 0; }
static void fp_mode_leave(unsigned old) { (void)old; }
#endif

static int exec_one(op_fn fn, const PlowDevInst* inst, void* const* tensors, uint32_t nthreads) {
    if (nthreads <= 1u) { fn(inst, 0u, 1u, tensors); return 0; }
    if (nthreads > 256u) nthreads = 256u;
    pthread_t th[256];
    Job jobs[256];
    for (uint32_t s = 0; s < nthreads; s++) {
        jobs[s] = (Job){fn, inst, tensors, s, nthreads};
        if (pthread_create(&th[s], NULL, job_main, &jobs[s]) != 0) {
            for (uint32_t q = 0; q < s; q++) pthread_join(th[q], NULL);
            return PLOW_MOE_ENOMEM;
        }
    }
    for (uint32_t s = 0; s < nthreads; s++) pthread_join(th[s], NULL);
    return 0;
}

int plow_oracle_exec(const PlowDevInst* inst, void* const* tensors, uint32_t nthreads) {
    op_fn fn = resolve(inst->op);
    if (!fn) return PLOW_MOE_EUNSUPPORTED;
    if (!e4m3_lut_ready) {
        for (int b = 0; b < 256; b++) e4m3_lut[b] = orc_e4m3_to_f32((uint8_t)b);
        e4m3_lut_ready = 1;
    }
    const unsigned mode = fp_mode_enter();
    int rc = exec_one(fn, inst, tensors, nthreads);
    if (!rc && inst->op == PLOW_DOP_GEMM_F32 && inst->i[7] == PLOW_ROUTER_RAW_MARK) {
        /* the score op that carries its top-k (plow crates/packet/src/dev.rs:90-94,
         * runtime/amd/router_decode.hip:1-63): the table bytes are those of the op pair, so the top-k is
         * op 83 over the logits just written: t3 table, t4 bias, i3 k, i4 flags, i5 bit 0 shared tail,
         * i6 = n_group | topk_group << 16, f0 route scale; the counters (t5) are left as they were */
        PlowDevInst tk;
        memset(&tk, 0, sizeof tk);
        tk.op = PLOW_DOP_MOE_ROUTER_TOPK_PF;
        tk.t[0] = inst->t[3], tk.t[1] = inst->t[0], tk.t[2] = PLOW_TENSOR_NONE, tk.t[3] = inst->t[4];
        for (int q = 4; q < 8; q++) tk.t[q] = PLOW_TENSOR_NONE;
        tk.i[1] = inst->i[1], tk.i[2] = inst->i[3], tk.i[3] = inst->i[4], tk.i[4] = inst->i[0];
        tk.i[5] = inst->i[5] & 1u, tk.i[6] = inst->i[6] & 0xFFFFu, tk.i[7] = inst->i[6] >> 16;
        tk.fj[0].f = inst->fj[0].f;
        rc = exec_one(op_router_topk, &tk, tensors, nthreads);
    }
    fp_mode_leave(mode);
    return rc;
}

int plow_oracle_exec_many(const PlowDevInst* insts, uint32_t n, void* const* tensors, uint32_t nthreads) {
    for (uint32_t i = 0; i < n; i++) {
        const int rc = plow_oracle_exec(&insts[i], tensors, nthreads);
        if (rc) return rc;
    }
    return 0;
}

/* ---- codec exports for the tests --------------------------------------------------------------- */

/* the fp4 x fp4 arm's activation quantizer over n_blocks 32-blocks of f32 values */
void plow_oracle_mx_act_quant(uint8_t* out, uint8_t* scales, const float* v, size_t n_blocks) {
    for (size_t b = 0; b < n_blocks; b++) mx_act_quant32(v + b * 32u, out + b * 16u, scales + b);
}
uint8_t plow_oracle_mx_act_e8m0(float amax) { return mx_act_e8m0(amax); }
uint8_t plow_oracle_mx_act_fp4(float v) { return mx_act_fp4(v); }
uint16_t plow_oracle_f2bf(float f) { return orc_f2bf(f); }
float plow_oracle_bf2f(uint16_t h) { return orc_bf2f(h); }
uint8_t plow_oracle_f32_to_e4m3(float f) { return orc_f32_to_e4m3(f); }
float plow_oracle_e4m3_to_f32(uint8_t b) { return orc_e4m3_to_f32(b); }
float plow_oracle_e2m1(uint8_t nib) { return orc_e2m1(nib); }
float plow_oracle_e8m0(uint8_t s) { return orc_e8m0(s); }
void plow_oracle_f2bf_n(uint16_t* dst, const float* src, size_t n) { for (size_t i = 0; i < n; i++) dst[i] = orc_f2bf(src[i]); }
void plow_oracle_split_e4m3_n(uint8_t* hi, uint8_t* lo, const float* src, size_t n) {
    if (!e4m3_lut_ready) { for (uint32_t b = 0; b < 256u; b++) e4m3_lut[b] = orc_e4m3_to_f32((uint8_t)b); e4m3_lut_ready = 1; }
    for (size_t i = 0; i < n; i++) split_e4m3(src[i], &hi[i], &lo[i]);
}
void plow_oracle_e4m3_encode_n(uint8_t* dst, const float* src, size_t n) { for (size_t i = 0; i < n; i++) dst[i] = orc_f32_to_e4m3(src[i]); }
