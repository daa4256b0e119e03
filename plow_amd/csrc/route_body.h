/* route_body.h — device bodies of the decode router (few-token score, per-token top-k, arrival counter)
 * shared by the library's kernels (route.hip) and by the code object plowrt loads for its raw router
 * segment (plowrt_router_obj.hip). Compile with -ffp-contract=off: no multiply-add is fused unless written
 * as fmaf. */
#ifndef PLOW_MOE_ROUTE_BODY_H
#define PLOW_MOE_ROUTE_BODY_H

#include "common.h"
#include "pm_expf.h"
#include "pm_log1pf.h"

/* Few outputs (decode): TOK tokens x 64 experts per workgroup, one consumer wave per token. Every output
 * is a chain of K dependent multiply-adds (9.3 cycles, 3.9 ns, a step on this chip whatever the operands:
 * register, scalar or DPP), so the kernel's time is the chain's
 * and the job is to keep everything else off the consumer waves' instruction streams:
 *  - four stager waves (16 weight rows each) own every global load. They widen the weight rows to f32
 *    into a double-buffered LDS tile shared by the consumers and copy the tokens' bf16 rows beside it.
 *    Their loads are written by hand (uniform chunk base + a per-lane byte offset that never changes)
 *    and waited for by count, RSR_PF - 1 chunks (about 100 KB a workgroup) in flight: at the chain's pace
 *    a chunk lasts half a microsecond, less than one trip to memory, and loads the compiler issues in a
 *    loop like this one end up waited for in full at every chunk;
 *  - a consumer lane (one expert) reads 4 k of its weight row per 16-byte LDS read, and its token's x
 *    sixteen steps at a time: lane l holds x[16 g + l % 16] and the multiply-add takes its x operand
 *    from lane i of the lane's row of 16 (row broadcast), so one register serves 16 steps and the chain
 *    is one instruction a step.
 * K must be a multiple of RSR_KC and the weight tensor smaller than 2 GiB (32-bit lane offsets). */
#define RSR_KC 256
#define RSR_LD (RSR_KC + 4) /* floats per LDS row: consecutive rows start 4 banks apart */
#define RSR_PF 4
#define RSR_STAGERS 4u
#define RSR_WS_BYTES (2u * 64u * RSR_LD * 4u)
/* The body takes its workgroup coordinates (expert tile bx, token group by) and its LDS as arguments, so
 * that the fused decode router below can run it and carry on. Every wave returns from it (the stagers
 * early), after the same number of barriers. */
template <uint32_t TOK>
__device__ __forceinline__ void router_score_row_body(float* __restrict__ out, const bf16_t* __restrict__ x,
                                                      const bf16_t* __restrict__ w, uint32_t M, uint32_t N, uint32_t K,
                                                      uint32_t bx, uint32_t by, uint8_t* rsr_raw) {
    float* const rsr_ws = (float*)rsr_raw;                        /* [2][64][RSR_LD] f32 weights */
    bf16_t* const rsr_xs = (bf16_t*)(rsr_raw + RSR_WS_BYTES);     /* [2][TOK][RSR_KC] bf16 tokens */
    constexpr int KC = RSR_KC, LD = RSR_LD;
    constexpr int NL = 8 + (int)TOK; /* loads per stager and chunk */
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wv = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint32_t n0 = bx * 64u, m0 = by * TOK;
    const uint32_t NC = K / KC;
    if (wv >= TOK) {
        /* a row of a chunk is 32 16-byte pieces; lane l loads piece l % 32 of rows base + l / 32, + 2, ...
         * (8 rows of this stager's 16) and of every token's row (only the first stager stores those) */
        const uint32_t pc = lane & 31u, sidx = wv - TOK, rbase = sidx * 16u + (lane >> 5);
        v4i wr[RSR_PF][8], xr[RSR_PF][TOK];
        uint32_t voff[8], xoff[TOK];
#pragma unroll
        for (int i = 0; i < 8; i++) { /* a row past N repeats the last row (never stored) */
            const uint32_t r = n0 + rbase + 2u * i;
            voff[i] = ((r < N ? r : N - 1u) * K + pc * 8u) * 2u;
        }
#pragma unroll
        for (uint32_t t = 0; t < TOK; t++) xoff[t] = ((m0 + t < M ? m0 + t : M - 1u) * K + pc * 8u) * 2u;
        auto fetch = [&](int st, uint32_t c) { /* a chunk past the end repeats the last chunk (never read) */
            const size_t off = (size_t)(c < NC ? c : NC - 1u) * (KC * 2u);
            const char* wb = (const char*)w + off;
            const char* xb = (const char*)x + off;
#pragma unroll
            for (int i = 0; i < 8; i++)
                asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(wr[st][i]) : "v"(voff[i]), "s"(wb) : "memory");
#pragma unroll
            for (uint32_t t = 0; t < TOK; t++)
                asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(xr[st][t]) : "v"(xoff[t]), "s"(xb) : "memory");
        };
        auto commit = [&](int st, uint32_t buf) {
            /* loads return in order: this stage's have landed once at most those of the RSR_PF - 1
             * younger stages are outstanding */
            asm volatile("s_waitcnt vmcnt(%8)"
                         : "+v"(wr[st][0]), "+v"(wr[st][1]), "+v"(wr[st][2]), "+v"(wr[st][3]), "+v"(wr[st][4]),
                           "+v"(wr[st][5]), "+v"(wr[st][6]), "+v"(wr[st][7])
                         : "n"((RSR_PF - 1) * NL)
                         : "memory");
#pragma unroll
            for (uint32_t t = 0; t < TOK; t++) asm volatile("" : "+v"(xr[st][t]));
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const uint32_t r = rbase + 2u * i;
                float* d = rsr_ws + ((size_t)buf * 64u + r) * LD + pc * 8u;
                const v4i a = wr[st][i];
                *(float4*)d = make_float4(__uint_as_float((uint32_t)a[0] << 16), __uint_as_float((uint32_t)a[0] & 0xFFFF0000u),
                                          __uint_as_float((uint32_t)a[1] << 16), __uint_as_float((uint32_t)a[1] & 0xFFFF0000u));
                *(float4*)(d + 4) = make_float4(__uint_as_float((uint32_t)a[2] << 16), __uint_as_float((uint32_t)a[2] & 0xFFFF0000u),
                                                __uint_as_float((uint32_t)a[3] << 16), __uint_as_float((uint32_t)a[3] & 0xFFFF0000u));
            }
            if (sidx == 0u && lane < 32u) {
#pragma unroll
                for (uint32_t t = 0; t < TOK; t++) *(v4i*)(rsr_xs + ((size_t)buf * TOK + t) * KC + pc * 8u) = xr[st][t];
            }
        };
#pragma unroll
        for (int st = 0; st < RSR_PF; st++) fetch(st, (uint32_t)st);
        commit(0, 0);
        for (uint32_t c0 = 0; c0 < NC; c0 += RSR_PF) {
#pragma unroll
            for (int st = 0; st < RSR_PF; st++) {
                const uint32_t c = c0 + (uint32_t)st;
                if (c < NC) {
                    lds_barrier(); /* chunk c is published; the consumers are done with chunk c - 1 */
                    fetch(st, c + RSR_PF); /* register stage st held chunk c, already in LDS */
                    if (c + 1u < NC) commit((st + 1) % RSR_PF, (c + 1u) & 1u);
                }
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); /* nothing in flight into dead registers at the end */
        return;
    }
    const uint32_t m = m0 + wv, l16 = lane & 15u;
    float acc = 0.0f;
/* four steps in one statement (no filler between them): x from lanes I .. I + 3 of the row, w = one float4 */
#define RSR_FMAC4(I0, I1, I2, I3, W)                                                                       \
    asm volatile("v_fmac_f32_dpp %0, %1, %2 row_newbcast:" #I0 " row_mask:0xf bank_mask:0xf\n\t"            \
                 "v_fmac_f32_dpp %0, %1, %3 row_newbcast:" #I1 " row_mask:0xf bank_mask:0xf\n\t"            \
                 "v_fmac_f32_dpp %0, %1, %4 row_newbcast:" #I2 " row_mask:0xf bank_mask:0xf\n\t"            \
                 "v_fmac_f32_dpp %0, %1, %5 row_newbcast:" #I3 " row_mask:0xf bank_mask:0xf"                 \
                 : "+v"(acc)                                                                               \
                 : "v"(xv), "v"((W).x), "v"((W).y), "v"((W).z), "v"((W).w))
    for (uint32_t c = 0; c < NC; c++) {
        const uint32_t buf = c & 1u;
        lds_barrier(); /* chunk c is in buffer c & 1 */
        const float* wp = rsr_ws + ((size_t)buf * 64u + lane) * LD;
        const bf16_t* xp = rsr_xs + ((size_t)buf * TOK + wv) * KC + l16;
        float xf[KC / 16];
#pragma unroll
        for (int g = 0; g < KC / 16; g++) xf[g] = __uint_as_float((uint32_t)xp[16 * g] << 16);
        /* operand reads run one 16-k group ahead of the multiply-adds */
        float4 b[2][4];
#pragma unroll
        for (int u = 0; u < 4; u++) b[0][u] = *(const float4*)(wp + 4 * u);
        asm volatile("s_nop 1" ::: "memory"); /* the row-broadcast operand was written by vector instructions */
#pragma unroll
        for (int gq = 0; gq < KC / 16; gq++) {
            const int cur = gq & 1, nxt = cur ^ 1;
            if (gq + 1 < KC / 16) {
#pragma unroll
                for (int u = 0; u < 4; u++) b[nxt][u] = *(const float4*)(wp + 16 * (gq + 1) + 4 * u);
            }
            const float xv = xf[gq];
            RSR_FMAC4(0, 1, 2, 3, b[cur][0]);
            RSR_FMAC4(4, 5, 6, 7, b[cur][1]);
            RSR_FMAC4(8, 9, 10, 11, b[cur][2]);
            RSR_FMAC4(12, 13, 14, 15, b[cur][3]);
        }
    }
#undef RSR_FMAC4
    const uint32_t n = n0 + lane;
    if (m < M && n < N) out[(size_t)m * N + n] = acc;
}

/* One wave per token; lane l holds experts l, l + 64, ... in registers. Selection is k rounds of a
 * wave-wide maximum over the packed key (ord(score + bias), lowest id wins ties). Keys are unique,
 * so round j returns the expert with exactly j keys above it: the reference's rank rule
 * (plow runtime/common/moe_route_key.h) with the same winners in the same order. A wave-wide max is
 * four DPP steps inside each row of 16 lanes plus a scalar max over the four rows. */
#define RT_MAX_E 1024u
#define RT_WAVES 4u

struct RouterArgs {
    PlowMoeRoute* table;
    const void* logit;
    const float* bias;
    uint32_t n_exp, k, flags, T, tail, n_group, topk_group;
    float route_scale, logit_scale;
};

__device__ __forceinline__ uint32_t wave_umax(uint32_t v) {
    uint32_t t;
    t = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, false); v = v > t ? v : t; /* quad_perm 1,0,3,2 */
    t = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, false); v = v > t ? v : t; /* quad_perm 2,3,0,1 */
    t = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xF, 0xF, false); v = v > t ? v : t; /* row_half_mirror */
    t = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xF, 0xF, false); v = v > t ? v : t; /* row_mirror */
    const uint32_t a = (uint32_t)__builtin_amdgcn_readlane((int)v, 0), b = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
    const uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)v, 32), d = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
    const uint32_t ab = a > b ? a : b, cd = c > d ? c : d;
    return ab > cd ? ab : cd;
}

/* one token by one wave; `score` is the wave's own 64 * RT_EPL floats of LDS */
template <uint32_t RT_EPL> /* experts per lane: n_exp <= 64 * RT_EPL */
__device__ __forceinline__ void router_topk_token(const RouterArgs& a, uint32_t tok, float* score) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t E = a.n_exp;
    const bool sigmoid = a.flags & PLOW_ROUTE_SIGMOID, norm = a.flags & PLOW_ROUTE_NORM_TOPK;
    const bool f32l = a.flags & PLOW_ROUTE_F32_LOGIT;
    const float ls = a.logit_scale != 0.0f ? a.logit_scale : 1.0f;
    uint32_t k = a.k;
    PlowMoeRoute* row = a.table + (size_t)tok * (a.k + a.tail);
    for (uint32_t j = PLOW_ROUTE_MAX_TOPK + lane; j < k; j += WAVE) {
        row[j].eid = PLOW_EXPERT_UNUSED;
        row[j].gate = 0.0f;
    }
    if (k > PLOW_ROUTE_MAX_TOPK) k = PLOW_ROUTE_MAX_TOPK;

    /* --- score transform (the whole wave is here: the exponential takes its table entries from the lanes) --- */
    const PmExpLanes tab = pm_exp_lanes();
    float sc[RT_EPL];
#pragma unroll
    for (uint32_t j = 0; j < RT_EPL; j++) {
        const uint32_t e = lane + WAVE * j;
        sc[j] = 0.0f;
        if (e < E)
            sc[j] = (f32l ? ((const float*)a.logit)[(size_t)tok * E + e]
                          : bf2f(((const bf16_t*)a.logit)[(size_t)tok * E + e])) * ls;
    }
    if (a.flags & PLOW_ROUTE_SQRT_SOFTPLUS) { /* sqrt(softplus(l)), softplus as log1p(exp(-|l|)) + max(l, 0) */
#pragma unroll
        for (uint32_t j = 0; j < RT_EPL; j++) {
            const float ex = pm_expf_lanes(-fabsf(sc[j]), tab); /* in [0, 1], or NaN from a NaN logit */
            const float sp = (ex == ex ? pm_log1pf_unit(ex) : ex) + fmaxf(sc[j], 0.0f);
            /* the correctly rounded root: the binary64 root of a binary32 number, rounded once more, is the
             * binary32 root (a root never lies within 2^-49 of a rounding boundary of binary32) */
            sc[j] = (float)__builtin_sqrt((double)sp);
        }
    } else if (sigmoid) {
#pragma unroll
        for (uint32_t j = 0; j < RT_EPL; j++) sc[j] = 1.0f / (1.0f + pm_expf_lanes(-sc[j], tab));
    } else {
        float m = -1e30f; /* the maximum is the same value in any visiting order */
#pragma unroll
        for (uint32_t j = 0; j < RT_EPL; j++)
            if (lane + WAVE * j < E && sc[j] > m) m = sc[j];
        m = wave_max(m);
#pragma unroll
        for (uint32_t j = 0; j < RT_EPL; j++) {
            const uint32_t e = lane + WAVE * j;
            const float ex = pm_expf_lanes(sc[j] - m, tab); /* every lane, also those past the last expert */
            if (e < E) score[e] = ex;
        }
        __builtin_amdgcn_wave_barrier();
        float s = 0.0f; /* the sum IS order dependent: ascending expert id, one accumulator */
#pragma unroll 8
        for (uint32_t e = 0; e < E; e++) s += score[e];
#pragma unroll
        for (uint32_t j = 0; j < RT_EPL; j++) {
            const uint32_t e = lane + WAVE * j;
            if (e < E) sc[j] = score[e] / s;
        }
        __builtin_amdgcn_wave_barrier();
    }

    /* --- selection keys: ord(score + bias); a dropped group's experts fall to ord 0 --- */
    uint32_t ordv[RT_EPL];
    float sel[RT_EPL];
#pragma unroll
    for (uint32_t j = 0; j < RT_EPL; j++) {
        const uint32_t e = lane + WAVE * j;
        sel[j] = sc[j] + ((a.bias && e < E) ? a.bias[e] : 0.0f);
        ordv[j] = route_ord(sel[j]);
    }
    const bool grouped = a.n_group > 1u && a.topk_group > 0u && a.topk_group < a.n_group &&
                         a.n_group <= PLOW_ROUTE_MAX_GROUPS && E % a.n_group == 0u;
    if (grouped) {
        /* group score = sum of the top-2 biased scores of the group (a multiset, so any visiting
         * order gives the same pair); groups ranked by (ord(sum), lowest id) */
        const uint32_t ng = a.n_group, gsz = E / ng;
#pragma unroll
        for (uint32_t j = 0; j < RT_EPL; j++) {
            const uint32_t e = lane + WAVE * j;
            if (e < E) score[e] = sel[j];
        }
        __builtin_amdgcn_wave_barrier();
        const uint32_t lpg = WAVE / ng; /* lanes per group on the fast path */
        const bool fast = (ng & (ng - 1u)) == 0u && gsz % lpg == 0u;
        float m1 = -3.0e38f, m2 = -3.0e38f;
        uint32_t g_of_lane, leader;
        if (fast) {
            g_of_lane = lane / lpg;
            leader = (lane % lpg) == 0u;
            for (uint32_t i = lane % lpg; i < gsz; i += lpg) {
                const float s = score[g_of_lane * gsz + i];
                if (s > m1) { m2 = m1; m1 = s; } else if (s > m2) m2 = s;
            }
            for (uint32_t o = 1; o < lpg; o <<= 1) {
                const float b1 = __shfl_xor(m1, (int)o, 64), b2 = __shfl_xor(m2, (int)o, 64);
                const float hi = fmaxf(m1, b1), lo = fminf(m1, b1);
                m2 = fmaxf(lo, fmaxf(m2, b2));
                m1 = hi;
            }
        } else {
            g_of_lane = lane;
            leader = lane < ng;
            if (leader)
                for (uint32_t i = 0; i < gsz; i++) {
                    const float s = score[lane * gsz + i];
                    if (s > m1) { m2 = m1; m1 = s; } else if (s > m2) m2 = s;
                }
        }
        const uint32_t gord = route_ord(m1 + m2);
        const uint32_t step = fast ? lpg : 1u;
        uint32_t grank = 0;
        for (uint32_t f = 0; f < ng; f++) {
            const uint32_t o = (uint32_t)__shfl((int)gord, (int)(f * step), 64);
            grank += (o > gord) || (o == gord && f < g_of_lane); /* lower id outranks on a tie */
        }
        const unsigned long long keep = __ballot(leader && grank < a.topk_group);
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (uint32_t j = 0; j < RT_EPL; j++) {
            const uint32_t e = lane + WAVE * j;
            if (e < E && !((keep >> ((e / gsz) * step)) & 1ull)) ordv[j] = 0u;
        }
    }

    /* --- k rounds of wave-wide max; inv = E - e (1..E) so that 0 means "no candidate" --- */
    uint32_t picked = 0u; /* bit j: this lane's expert j is already a winner */
    float sum = 0.0f, my_g = 0.0f;
    uint32_t my_e = E - 1u;
    for (uint32_t r = 0; r < k; r++) {
        uint32_t bo = 0u, bi = 0u;
#pragma unroll
        for (uint32_t j = 0; j < RT_EPL; j++) {
            const uint32_t e = lane + WAVE * j, inv = E - e;
            const bool cand = e < E && !((picked >> j) & 1u);
            if (cand && (bi == 0u || ordv[j] > bo || (ordv[j] == bo && inv > bi))) { bo = ordv[j]; bi = inv; }
        }
        const uint32_t mo = wave_umax(bi ? bo : 0u);
        /* the lanes whose best candidate has the winning key: almost always one, whose id is then read
         * straight from it; several (equal keys in different lanes) take the second maximum, over ids */
        const bool top = bi != 0u && bo == mo;
        const unsigned long long tops = __ballot(top);
        uint32_t mi;
        if (__builtin_popcountll(tops) == 1) mi = (uint32_t)__builtin_amdgcn_readlane((int)bi, (int)__builtin_ctzll(tops));
        else mi = tops ? wave_umax(top ? bi : 0u) : 0u;
        const uint32_t ew = mi ? E - mi : E - 1u; /* nothing left: the reference's pre-filled E - 1 */
        const uint32_t wl = ew & 63u, ws = ew >> 6;
        float cand_score = sc[0];
#pragma unroll
        for (uint32_t j = 1; j < RT_EPL; j++)
            if (ws == j) cand_score = sc[j];
        const float g = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(cand_score), (int)wl));
        if (mi && lane == wl) picked |= 1u << ws;
        sum += g; /* slot order, one accumulator, identical in every lane */
        if (lane == r) { my_e = ew; my_g = g; }
    }
    if (lane < k) {
        float g = my_g;
        if (norm && sum != 0.0f) g /= sum;
        g *= a.route_scale;
        row[lane].eid = my_e;
        row[lane].gate = g;
    }
    if (a.tail && lane == 0) {
        row[a.k].eid = E;
        row[a.k].gate = 1.0f;
    }
}

/* the same with the form picked inside the kernel (the fused decode routers) */
__device__ __forceinline__ void router_topk_token_any(const RouterArgs& a, uint32_t tok, float* score) {
    if (a.n_exp <= 64u) router_topk_token<1>(a, tok, score);
    else if (a.n_exp <= 128u) router_topk_token<2>(a, tok, score);
    else if (a.n_exp <= 256u) router_topk_token<4>(a, tok, score);
    else if (a.n_exp <= 384u) router_topk_token<6>(a, tok, score);
    else if (a.n_exp <= 512u) router_topk_token<8>(a, tok, score);
    else router_topk_token<16>(a, tok, score);
}

/* this workgroup was the last of `n` to add itself to *ctr (every thread gets the answer); what the
 * workgroup wrote before is visible to whoever comes last, and the last sees everyone's writes */
__device__ __forceinline__ bool rf_last_arrival(uint32_t* ctr, uint32_t n, uint32_t* s_flag) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t old = __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const uint32_t last = old == n - 1u ? 1u : 0u;
        if (last) __hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *s_flag = last;
    }
    __syncthreads();
    const bool last = *s_flag != 0u;
    if (last) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    return last;
}

#define RSR_LDS (RSR_WS_BYTES + 2u * 4u * RSR_KC * 2u)

#endif
