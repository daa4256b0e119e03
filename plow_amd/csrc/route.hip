/* route.hip — the routing half of the MoE path on gfx950: router score (op 180), router top-k
 * (ops 83 / 56), align / sort / offset scan (op 84) and combine (ops 87 / 43).
 *
 * Everything integer here (selected experts, their order, counts, offsets, the row permutation) is
 * bit-identical to plow's CPU reference (runtime/cpu/dev/golden/moe_route.c), and so are the f32
 * logits and gates, because every floating-point step is done in the reference's own order with
 * correctly rounded IEEE operations and the exponential of pm_expf.h.
 * This file is compiled with -ffp-contract=off: no multiply-add is fused unless written as fmaf.
 */
#include <stdlib.h>
#include <string.h>
#include <type_traits>
#include "common.h"
#include "kernels.h"
#include "pm_expf.h"
#include "tuning.h"
#include "route_body.h"

/* ============================ op 180: router score ============================================= */
/* logit[m][n] = sum_k bf(x[m][k]) * bf(w[n][k]) with ONE f32 accumulator per output walking k in
 * ascending order (plow runtime/cpu/dev/golden/f32_primitives.c:235-252). The product of two bf16
 * values is exact in f32, so fmaf(a, b, acc) rounds exactly like the reference's `acc += a * b`. */
/* Large problems (prefill): (16 * TM) x 64 outputs per workgroup, TM x 4 per thread (independent chains
 * per lane keep the FMA pipe full), operands double buffered in LDS as f32 [k][row] and read as float4
 * (float2 for TM = 2), one LDS-only barrier per 32-k chunk, the next chunk's global loads already in
 * flight.
 * TM = 4 moves the fewest LDS bytes per multiply-add. Per chunk its four waves still pull 256 KB through
 * the LDS while each SIMD issues 512 multiply-adds, about the same number of cycles, and a lone wave per
 * SIMD overlaps the two poorly (measured: it issues 53 % of the cycles). With fewer than two such
 * workgroups per CU, TM = 2 gives every SIMD a second wave to run in the gaps, which more than pays for
 * its extra LDS reads. */
#define RST_KC 32
#define RST_LD 68 /* floats per LDS row of 64: + 4 keeps float4 reads aligned */
template <int TM>
__global__ __launch_bounds__(256) void k_router_score_tile(float* __restrict__ out,
                                                           const bf16_t* __restrict__ x,
                                                           const bf16_t* __restrict__ w, uint32_t M,
                                                           uint32_t N, uint32_t K) {
    constexpr uint32_t BM = 16u * TM;
    __shared__ __attribute__((aligned(16))) float xs[2][RST_KC][BM + 4];
    __shared__ __attribute__((aligned(16))) float ws[2][RST_KC][RST_LD];
    const uint32_t tid = threadIdx.x, tx = tid & 15u, ty = tid >> 4;
    const uint32_t m0 = blockIdx.y * BM, n0 = blockIdx.x * 64u;
    /* staging: rows x 32 k bf16 in 16-byte pieces, one per thread (the x tile has 4 * BM of them) */
    const uint32_t srow = tid >> 2, skc = tid & 3u;
    uint4 xr, wr;
    auto fetch = [&](uint32_t k0) {
        const uint32_t k = k0 + skc * 8u;
        xr = make_uint4(0, 0, 0, 0);
        wr = make_uint4(0, 0, 0, 0);
        if (srow < BM && m0 + srow < M && k < K) xr = *(const uint4*)(x + (size_t)(m0 + srow) * K + k);
        if (n0 + srow < N && k < K) wr = *(const uint4*)(w + (size_t)(n0 + srow) * K + k);
    };
    auto commit = [&](uint32_t buf) {
        const uint32_t a[4] = {xr.x, xr.y, xr.z, xr.w}, b[4] = {wr.x, wr.y, wr.z, wr.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (srow < BM) {
                xs[buf][skc * 8 + 2 * j][srow] = __uint_as_float(a[j] << 16);
                xs[buf][skc * 8 + 2 * j + 1][srow] = __uint_as_float(a[j] & 0xFFFF0000u);
            }
            ws[buf][skc * 8 + 2 * j][srow] = __uint_as_float(b[j] << 16);
            ws[buf][skc * 8 + 2 * j + 1][srow] = __uint_as_float(b[j] & 0xFFFF0000u);
        }
    };
    float acc[TM][4];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = 0.0f;
    fetch(0);
    commit(0);
    lds_barrier();
    uint32_t buf = 0;
    for (uint32_t k0 = 0; k0 < K; k0 += RST_KC, buf ^= 1u) {
        const bool more = k0 + RST_KC < K;
        if (more) fetch(k0 + RST_KC);
        const uint32_t kn = K - k0 < (uint32_t)RST_KC ? K - k0 : (uint32_t)RST_KC;
        if (kn == (uint32_t)RST_KC) {
#pragma unroll
            for (int kk = 0; kk < RST_KC; kk++) {
                float av[TM];
                if (TM == 4) {
                    const float4 a = *(const float4*)&xs[buf][kk][ty * 4u];
                    av[0] = a.x, av[1] = a.y, av[TM - 2] = a.z, av[TM - 1] = a.w;
                } else {
                    const float2 a = *(const float2*)&xs[buf][kk][ty * 2u];
                    av[0] = a.x, av[1] = a.y;
                }
                const float4 b = *(const float4*)&ws[buf][kk][tx * 4u];
                const float bv[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < 4; j++) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
            }
        } else {
            for (uint32_t kk = 0; kk < kn; kk++)
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        acc[i][j] = fmaf(xs[buf][kk][ty * TM + i], ws[buf][kk][tx * 4u + j], acc[i][j]);
        }
        if (more) commit(buf ^ 1u);
        lds_barrier();
    }
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t m = m0 + ty * TM + i, n = n0 + tx * 4u + j;
            if (m < M && n < N) out[(size_t)m * N + n] = acc[i][j];
        }
}

typedef __attribute__((address_space(3))) void rsm_lds_void;

/* Small problems (decode). Two things bound this shape: the dependent chain of K multiply-adds per
 * output, and LDS bandwidth (every multiply-add of every lane reads a fresh operand pair). Both say
 * "spread thin": one wave per workgroup (so one wave per CU's LDS), an 8 x 8 block of outputs per
 * wave, one output per lane. Operands sit in LDS as f32 [row][k] (double buffered) and are read four
 * k at a time; global loads run RSW_PF chunks ahead in a ring of register stages, and the barriers
 * order LDS only so those loads stay in flight. */
#define RSW_KC 256
#define RSW_PF 3
/* Two waves per workgroup: wave 1 stages (global loads RSW_PF chunks ahead, bf16 -> f32, LDS writes),
 * wave 0 only reads operands from LDS and runs the chain of multiply-adds, which is the critical
 * path (K dependent operations per output). One LDS-scoped barrier per chunk hands a buffer over:
 * after barrier i chunk i is in buffer i % 2, and the stager fills the other buffer with chunk i + 1
 * while chunk i is being consumed. */
__global__ __launch_bounds__(128) void k_router_score_wave(float* __restrict__ out,
                                                           const bf16_t* __restrict__ x,
                                                           const bf16_t* __restrict__ w, uint32_t M,
                                                           uint32_t N, uint32_t K) {
    constexpr int KC = RSW_KC, LD = KC + 4; /* +4 floats: the 8 rows start 4 banks apart */
    __shared__ __attribute__((aligned(16))) float xs[2][8][LD];
    __shared__ __attribute__((aligned(16))) float ws[2][8][LD];
    const uint32_t lane = threadIdx.x & 63u;
    const bool stager = threadIdx.x >= 64u;
    const uint32_t m0 = blockIdx.y * 8u, n0 = blockIdx.x * 8u;
    const uint32_t NC = (K + KC - 1u) / KC;
    if (stager) {
        /* a row of a chunk is KC / 8 = 32 16-byte pieces; lane l loads piece l % 32 of rows
         * l / 32, l / 32 + 2, ... (4 rows of each operand) */
        const uint32_t pc = lane & 31u, rsel = lane >> 5;
        uint4 xr[RSW_PF][4], wr[RSW_PF][4];
        auto fetch = [&](int s, uint32_t k0) {
            const uint32_t k = k0 + pc * 8u;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t r = rsel + 2u * i;
                xr[s][i] = make_uint4(0, 0, 0, 0);
                wr[s][i] = make_uint4(0, 0, 0, 0);
                if (m0 + r < M && k < K) xr[s][i] = *(const uint4*)(x + (size_t)(m0 + r) * K + k);
                if (n0 + r < N && k < K) wr[s][i] = *(const uint4*)(w + (size_t)(n0 + r) * K + k);
            }
        };
        auto put = [&](float* d, uint4 a) {
            *(float4*)d = make_float4(__uint_as_float(a.x << 16), __uint_as_float(a.x & 0xFFFF0000u),
                                      __uint_as_float(a.y << 16), __uint_as_float(a.y & 0xFFFF0000u));
            *(float4*)(d + 4) = make_float4(__uint_as_float(a.z << 16), __uint_as_float(a.z & 0xFFFF0000u),
                                            __uint_as_float(a.w << 16), __uint_as_float(a.w & 0xFFFF0000u));
        };
        auto commit = [&](int s, uint32_t buf) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t r = rsel + 2u * i;
                put(&xs[buf][r][pc * 8u], xr[s][i]);
                put(&ws[buf][r][pc * 8u], wr[s][i]);
            }
        };
#pragma unroll
        for (int s = 0; s < RSW_PF; s++) fetch(s, (uint32_t)s * KC);
        commit(0, 0);
        for (uint32_t c0 = 0; c0 < NC; c0 += RSW_PF) {
#pragma unroll
            for (int s = 0; s < RSW_PF; s++) {
                const uint32_t c = c0 + (uint32_t)s;
                if (c < NC) {
                    lds_barrier(); /* chunk c is published; the consumer is done with chunk c - 1 */
                    fetch(s, (c + RSW_PF) * KC); /* register stage s held chunk c, already in LDS */
                    if (c + 1u < NC) commit((s + 1) % RSW_PF, (c + 1u) & 1u);
                }
            }
        }
        return;
    }
    const uint32_t my = lane >> 3, nx = lane & 7u;
    float acc = 0.0f;
    for (uint32_t c = 0; c < NC; c++) {
        lds_barrier(); /* chunk c is in buffer c & 1 */
        const uint32_t k0 = c * KC, buf = c & 1u;
        const uint32_t kn = K - k0 < (uint32_t)KC ? K - k0 : (uint32_t)KC;
        const float* xp = xs[buf][my];
        const float* wp = ws[buf][nx];
        uint32_t kk = 0;
        if (kn == (uint32_t)KC) {
            /* full chunk: operand reads run one 16-k group ahead of the multiply-adds */
            float4 a[2][4], b[2][4];
#pragma unroll
            for (int u = 0; u < 4; u++) { a[0][u] = *(const float4*)(xp + 4 * u); b[0][u] = *(const float4*)(wp + 4 * u); }
#pragma unroll
            for (int gq = 0; gq < KC / 16; gq++) {
                const int cur = gq & 1, nxt = cur ^ 1;
                if (gq + 1 < KC / 16) {
#pragma unroll
                    for (int u = 0; u < 4; u++) {
                        a[nxt][u] = *(const float4*)(xp + 16 * (gq + 1) + 4 * u);
                        b[nxt][u] = *(const float4*)(wp + 16 * (gq + 1) + 4 * u);
                    }
                }
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    acc = fmaf(a[cur][u].x, b[cur][u].x, acc);
                    acc = fmaf(a[cur][u].y, b[cur][u].y, acc);
                    acc = fmaf(a[cur][u].z, b[cur][u].z, acc);
                    acc = fmaf(a[cur][u].w, b[cur][u].w, acc);
                }
            }
            kk = KC;
        }
        for (; kk < kn; kk++) acc = fmaf(xp[kk], wp[kk], acc);
    }
    const uint32_t m = m0 + my, n = n0 + nx;
    if (m < M && n < N) out[(size_t)m * N + n] = acc;
}

template <uint32_t TOK>
__global__ __launch_bounds__((TOK + RSR_STAGERS) * 64u) void k_router_score_row(float* __restrict__ out,
                                                                                const bf16_t* __restrict__ x,
                                                                                const bf16_t* __restrict__ w,
                                                                                uint32_t M, uint32_t N, uint32_t K) {
    extern __shared__ __attribute__((aligned(16))) uint8_t rsr_raw[];
    router_score_row_body<TOK>(out, x, w, M, N, K, blockIdx.x, blockIdx.y, rsr_raw);
}

/* Large problems with K a multiple of 64: the same sums on the matrix unit. v_mfma_f32_16x16x4_f32 adds
 * a[i][k] * b[k][j] for four consecutive k to its f32 accumulator one after the other, each step rounded to
 * nearest even and denormals kept (measured against the fmaf chain, bit for bit, normal and denormal ranges;
 * v_mfma_f32_32x32x2_f32 does the same with two k), so a chain of K / 4 of them IS the reference's sum in the
 * reference's order. A wave computes 16 tokens x 32 experts as two independent chains that share the token
 * operand; lane = (row lane & 15, k lane >> 4).
 * Two facts of the part shape the kernel. (1) The f32 matrix instructions execute on the vector unit's own
 * multiply-add lanes (the f32 matrix peak equals the vector f32 peak): a vector instruction between two of
 * them does not hide behind them, it adds its full time (measured on a 32 x 32 form of this kernel: the eight
 * byte permutes that widened a piece's bf16 operands cost 9 cycles each, 29 of 173 us at T = 4096, E = 256,
 * K = 7168). So an operand is widened by its LDS read: ds_read_u16_d16_hi puts a bf16 into the high half of a
 * register whose low half is zero, which is the f32. The per-lane addresses of the eight 16-byte pieces of a
 * row are computed once (LDS piece p of row r holds global piece p ^ ((r >> 1) & 7), so that the 16 rows of a
 * read fall on distinct banks; that makes them lane-dependent) and stage, block and k half are immediate
 * offsets: the loop issues no vector instruction next to its matrix instructions.
 * (2) A CU's vector-memory path delivers about 38 KB/us whatever level answers, and wave-private operand rings
 * (every token row loaded by each of the waves that use it) ask for more than that at the matrix unit's full
 * rate. So the four waves of a workgroup, stacked over 64 tokens, share one block of 32 experts and one ring:
 * a stage holds 64 + 32 rows (12 KB, direct global -> LDS loads, 8 lanes per 128-byte line), a wave loads a
 * quarter of it (16 token rows, 8 expert rows). A piece (8 k) is only four short matrix instructions, so the
 * reads run two pieces ahead into four sets of operand registers (set = piece % 4: the same in every chunk).
 * The barrier of chunk c sits in its seventh piece, before the first read of chunk c + 1: every wave has then
 * landed its loads of chunk c + 1 and its reads of chunk c - 1, whose stage takes chunk c + 3 (four stages,
 * 48 KB: a CU takes three workgroups). Measured against the earlier forms (private rings, operands widened by
 * permutes; 32 x 32 tiles where they filled the SIMDs evenly): DeepSeek-V3 router at 4096 tokens 176 -> 141 us
 * (a shared-ring 32 x 32 form with the same reads: 147), GLM slice (E = 288, K = 4096) at 8192 tokens 243 -> 166,
 * Qwen3 at 2048 tokens 60 -> 41. */
#define RSM_STAGES 4u
struct RsmStage {
    uint8_t x[64u * 128u];
    uint8_t w[32u * 128u];
};
static_assert(sizeof(RsmStage) == 12288u, "the stage size is an immediate of the LDS reads below");
/* six 2-byte reads of a piece: k = ks and 4 + ks (the lane's address holds 2 ks) of the lane's token row and of
 * its expert row in both 16-row blocks */
template <uint32_t STG>
__device__ __forceinline__ void rsm_read(float (&a)[2], float (&b)[2][2], uint32_t ax, uint32_t aw) {
    asm volatile("ds_read_u16_d16_hi %0, %6 offset:%8\n\t"
                 "ds_read_u16_d16_hi %2, %7 offset:%8\n\t"
                 "ds_read_u16_d16_hi %4, %7 offset:%10\n\t"
                 "ds_read_u16_d16_hi %1, %6 offset:%9\n\t"
                 "ds_read_u16_d16_hi %3, %7 offset:%9\n\t"
                 "ds_read_u16_d16_hi %5, %7 offset:%11"
                 : "+v"(a[0]), "+v"(a[1]), "+v"(b[0][0]), "+v"(b[0][1]), "+v"(b[1][0]), "+v"(b[1][1])
                 : "v"(ax), "v"(aw), "n"(STG * 12288u), "n"(STG * 12288u + 8u), "n"(STG * 12288u + 2048u), "n"(STG * 12288u + 2056u)
                 : "memory");
}
/* all but the newest piece's six reads have landed (LDS answers in order) */
__device__ __forceinline__ void rsm_wait_older(float (&a)[2], float (&b)[2][2]) {
    asm volatile("s_waitcnt lgkmcnt(6)" : "+v"(a[0]), "+v"(a[1]), "+v"(b[0][0]), "+v"(b[0][1]), "+v"(b[1][0]), "+v"(b[1][1]));
}
__global__ __launch_bounds__(256) void k_router_score_mfma(float* __restrict__ out, const bf16_t* __restrict__ x,
                                                                    const bf16_t* __restrict__ w, uint32_t M, uint32_t N,
                                                                    uint32_t K) {
    extern __shared__ __attribute__((aligned(16))) uint8_t rsm_raw[];
    constexpr uint32_t ST = RSM_STAGES, NLD = 3u; /* direct loads per wave and chunk */
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wv = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    RsmStage* const ring = (RsmStage*)rsm_raw;
    const uint32_t G = gridDim.x, gx = (N + 31u) / 32u;
    const uint32_t wg = (G % 8u == 0u) ? (blockIdx.x % 8u) * (G / 8u) + blockIdx.x / 8u : blockIdx.x;
    const uint32_t M0 = (wg / gx) * 64u, N0 = (wg % gx) * 32u; /* the workgroup's block */
    const uint32_t m0 = M0 + 16u * wv, n0 = N0;                /* this wave's tile */
    const uint32_t NC = K / 64u;
    /* this wave's share of a stage: token rows 16 wv .. 16 wv + 15 (two loads) and expert rows 8 wv .. 8 wv + 7;
     * rows past the end of a matrix read its last row and are never stored; no wave leaves early */
    const uint32_t lr = lane >> 3, lp = lane & 7u;
    const uint8_t* const xblk = (const uint8_t*)(x + (size_t)M0 * K);
    const uint8_t* const wblk = (const uint8_t*)(w + (size_t)N0 * K);
    uint32_t xoff[2], woff;
#pragma unroll
    for (uint32_t j = 0; j < 2u; j++) {
        const uint32_t row = 16u * wv + 8u * j + lr;
        const uint32_t mr = M0 + row < M ? row : M - 1u - M0;
        xoff[j] = mr * K * 2u + ((lp ^ ((row >> 1) & 7u)) << 4);
    }
    {
        const uint32_t row = 8u * wv + lr;
        const uint32_t nr = N0 + row < N ? row : N - 1u - N0;
        woff = nr * K * 2u + ((lp ^ ((row >> 1) & 7u)) << 4);
    }
    auto issue = [&](uint32_t c, uint32_t stage) {
        RsmStage* s = &ring[stage];
        /* opaque scalar bases and lane offsets: an address stays "scalar base + 32-bit lane offset" */
        uint64_t xcb = (uint64_t)(uintptr_t)(xblk + (size_t)c * 128u), wcb = (uint64_t)(uintptr_t)(wblk + (size_t)c * 128u);
        asm volatile("" : "+s"(xcb), "+s"(wcb));
#pragma unroll
        for (uint32_t j = 0; j < 2u; j++) {
            uint32_t o = xoff[j];
            asm volatile("" : "+v"(o));
            __builtin_amdgcn_global_load_lds((const void*)((const uint8_t*)(uintptr_t)xcb + o), (rsm_lds_void*)&s->x[(16u * wv + 8u * j) * 128u], 16, 0, 0);
        }
        uint32_t o = woff;
        asm volatile("" : "+v"(o));
        __builtin_amdgcn_global_load_lds((const void*)((const uint8_t*)(uintptr_t)wcb + o), (rsm_lds_void*)&s->w[(8u * wv) * 128u], 16, 0, 0);
    };
    /* operand reads: lane = (row lane & 15, k lane >> 4); 16 is a multiple of 16: the swizzle of row 16 h + r is that of r */
    const uint32_t orow = lane & 15u, ks = lane >> 4, osw = (orow >> 1) & 7u;
    const uint32_t ring0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)&ring[0];
    const uint32_t xrow = ring0 + (16u * wv + orow) * 128u + 2u * ks;
    const uint32_t wrow = ring0 + 64u * 128u + orow * 128u + 2u * ks;
    uint32_t ax[8], aw[8];
#pragma unroll
    for (uint32_t pc = 0; pc < 8u; pc++) ax[pc] = xrow + ((pc ^ osw) << 4), aw[pc] = wrow + ((pc ^ osw) << 4);
    v4f acc[2];
    acc[0] = (v4f){0.0f, 0.0f, 0.0f, 0.0f}, acc[1] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
    float af[4][2], bf[4][2][2]; /* [set][k half] and [set][block][k half]; the low halves stay zero */
#pragma unroll
    for (int q = 0; q < 4; q++)
#pragma unroll
        for (int h = 0; h < 2; h++) af[q][h] = 0.0f, bf[q][0][h] = 0.0f, bf[q][1][h] = 0.0f;
    issue(0u, 0u);
    if (NC > 1u) issue(1u, 1u);
    if (NC > 2u) issue(2u, 2u);
    if (NC > 2u) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NLD) : "memory");
    else if (NC > 1u) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NLD) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    asm volatile("s_barrier" ::: "memory"); /* chunk 0 is complete */
    rsm_read<0u>(af[0], bf[0], ax[0], aw[0]);
    rsm_read<0u>(af[1], bf[1], ax[1], aw[1]);
    rsm_wait_older(af[0], bf[0]);
#define RSM_FENCE() __builtin_amdgcn_sched_barrier(0)
    auto chunk = [&](auto stg_, uint32_t c) {
        constexpr uint32_t STG = decltype(stg_)::value, STN = (STG + 1u) % ST, STF = (STG + 3u) % ST;
#pragma unroll
        for (uint32_t pc = 0; pc < 8u; pc++) {
            const uint32_t cur = pc & 3u, n1 = (pc + 1u) & 3u, n2 = (pc + 2u) & 3u;
            RSM_FENCE();
            acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[cur][0], bf[cur][0][0], acc[0], 0, 0, 0);
            RSM_FENCE();
            if (pc == 6u) {
                /* this wave's loads of chunk c + 1 have landed and so have its reads of chunk c - 1 (its last piece was
                 * waited for seven pieces ago): behind the barrier that holds for every wave */
                if (c + 2u < NC) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NLD) : "memory");
                else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                asm volatile("s_barrier" ::: "memory");
            }
            /* piece p + 2 into the set piece p - 2 used; past the last chunk: stale bytes, never used */
            if (pc < 6u) rsm_read<STG>(af[n2], bf[n2], ax[(pc + 2u) & 7u], aw[(pc + 2u) & 7u]);
            else rsm_read<STN>(af[n2], bf[n2], ax[(pc + 2u) & 7u], aw[(pc + 2u) & 7u]);
            RSM_FENCE();
            acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[cur][0], bf[cur][1][0], acc[1], 0, 0, 0);
            RSM_FENCE();
            if (pc == 6u && c + 3u < NC) issue(c + 3u, STF); /* into the stage chunk c - 1 has left */
            RSM_FENCE();
            acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[cur][1], bf[cur][0][1], acc[0], 0, 0, 0);
            RSM_FENCE();
            acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[cur][1], bf[cur][1][1], acc[1], 0, 0, 0);
            RSM_FENCE();
            rsm_wait_older(af[n1], bf[n1]); /* piece p + 1 */
        }
    };
    for (uint32_t c = 0; c < NC; c += 4u) {
        chunk(std::integral_constant<uint32_t, 0u>{}, c);
        if (c + 1u < NC) chunk(std::integral_constant<uint32_t, 1u>{}, c + 1u);
        if (c + 2u < NC) chunk(std::integral_constant<uint32_t, 2u>{}, c + 2u);
        if (c + 3u < NC) chunk(std::integral_constant<uint32_t, 3u>{}, c + 3u);
    }
#undef RSM_FENCE
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); /* the stale reads of the last two pieces */
    /* acc[b][r] = out[m0 + 4 * (lane / 16) + r][n0 + 16 b + lane % 16] */
#pragma unroll
    for (int b = 0; b < 2; b++) {
        const uint32_t n = n0 + 16u * (uint32_t)b + (lane & 15u);
#pragma unroll
        for (uint32_t r = 0; r < 4u; r++) {
            const uint32_t m = m0 + 4u * (lane >> 4) + r;
            if (m < M && n < N) out[(size_t)m * N + n] = acc[b][r];
        }
    }
}

#define RSM_LDS (RSM_STAGES * (uint32_t)sizeof(RsmStage))

/* dynamic-LDS limits of the score kernels, once per device (plow_moe_device_setup) */
static bool rf_setup();
int plow_moe_route_setup() {
    const bool ok = rf_setup() &&
        hipFuncSetAttribute((const void*)k_router_score_mfma, hipFuncAttributeMaxDynamicSharedMemorySize, (int)RSM_LDS) == hipSuccess &&
        hipFuncSetAttribute((const void*)k_router_score_row<1>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)RSR_LDS) == hipSuccess &&
        hipFuncSetAttribute((const void*)k_router_score_row<2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)RSR_LDS) == hipSuccess &&
        hipFuncSetAttribute((const void*)k_router_score_row<4>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)RSR_LDS) == hipSuccess;
    return ok ? 0 : PLOW_MOE_EDEVICE;
}

int launch_router_score(float* out, const void* x, const void* w, uint32_t M, uint32_t N, uint32_t K,
                        hipStream_t st) {
    if (K % 8u) return PLOW_MOE_EINVAL;
    /* the matrix-unit form from 2^17 outputs on (below that the vector-unit forms, whose chains are shorter still,
     * win: 256 x 256 x 7168 takes 54 us there, 512 x 256 x 7168 takes 67 here and 128 there) */
    const PlowMoeTuning& tune = plow_moe_tuning();
    const uint64_t n_cu = plow_moe_n_cu();
    if (!n_cu) return PLOW_MOE_EDEVICE;
    /* (a load's lane offset is 32 bits and spans 64 rows of a matrix) */
    if (K % 64u == 0u && (uint64_t)K * 2u * 64u < (1ull << 32) && !tune.score_valu && (uint64_t)M * N >= (1u << 17)) {
        const uint32_t g = ((N + 31) / 32) * ((M + 63) / 64);
        k_router_score_mfma<<<g, 256, RSM_LDS, st>>>(out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
    } else if ((uint64_t)M * N >= (1u << 19)) {
        if ((uint64_t)((N + 63) / 64) * ((M + 63) / 64) < 2u * n_cu) { /* fewer than two 64-row workgroups per CU */
            dim3 g((N + 63) / 64, (M + 31) / 32);
            k_router_score_tile<2><<<g, 256, 0, st>>>(out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
        } else {
            dim3 g((N + 63) / 64, (M + 63) / 64);
            k_router_score_tile<4><<<g, 256, 0, st>>>(out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
        }
    } else if (!tune.score_tile8 && K % RSR_KC == 0u && (uint64_t)N * K * 2u < (1ull << 31) && (uint64_t)M * K * 2u < (1ull << 31) &&
               (M < 16u || (uint64_t)M * N <= 2048u || (!tune.score_row_narrow && (uint64_t)((N + 63) / 64) * ((M + 1u) / 2u) <= n_cu))) {
        /* measured against the 8 x 8 tile kernel below: ahead with one or two tokens per workgroup (6 of
         * 38 us at 1 x 384 x 7168) and with four on small score matrices (16 x 64 x 2048: 17 against
         * 25 us); with four tokens on a large one the shared LDS tile is the limit and the two are level */
        /* tokens per workgroup: as many as keep the weight rows' re-reads (once per workgroup row) low */
        const uint32_t lds = RSR_LDS;
        const uint32_t nx = (N + 63) / 64;
        /* a batch whose (token, 64 experts) chains fit the chip one or two to a workgroup keeps that shape beyond 16
         * tokens: every output is one chain of K dependent multiply-adds whatever the tile, and the 8 x 8 tile kernel
         * below runs 64 of them per wave where this one runs 64 per wave with the weight tile to itself */
        if (!tune.score_row_narrow && M >= 16u && (uint64_t)nx * M <= n_cu)
            k_router_score_row<1><<<dim3(nx, M), (1u + RSR_STAGERS) * 64u, lds, st>>>(out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
        else if (!tune.score_row_narrow && M >= 16u && (uint64_t)nx * ((M + 1u) / 2u) <= n_cu)
            k_router_score_row<2><<<dim3(nx, (M + 1u) / 2u), (2u + RSR_STAGERS) * 64u, lds, st>>>(out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
        else if (M >= 16u) k_router_score_row<4><<<dim3(nx, (M + 3u) / 4u), (4u + RSR_STAGERS) * 64u, lds, st>>>(out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
        else if (M >= 4u) k_router_score_row<2><<<dim3(nx, (M + 1u) / 2u), (2u + RSR_STAGERS) * 64u, lds, st>>>(out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
        else k_router_score_row<1><<<dim3(nx, M), (1u + RSR_STAGERS) * 64u, lds, st>>>(out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
    } else {
        dim3 g((N + 7) / 8, (M + 7) / 8);
        k_router_score_wave<<<g, 128, 0, st>>>(out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
    }
    return 0;
}

/* ============================ ops 83 / 56: router top-k ======================================== */
template <uint32_t RT_EPL>
__global__ __launch_bounds__(RT_WAVES* WAVE) void k_router_topk(RouterArgs a) {
    __shared__ float s_score[RT_WAVES][64u * RT_EPL];
    const uint32_t wv = threadIdx.x >> 6;
    const uint32_t tok = blockIdx.x * RT_WAVES + wv;
    if (tok >= a.T) return; /* whole wave leaves together; no block-level barrier below */
    router_topk_token<RT_EPL>(a, tok, s_score[wv]);
}

int launch_router_topk(void* table, const void* logit, const float* bias, uint32_t n_exp, uint32_t k,
                       uint32_t flags, uint32_t T, uint32_t tail, uint32_t n_group, uint32_t topk_group,
                       float route_scale, float logit_scale, hipStream_t st) {
    if (n_exp == 0 || n_exp > RT_MAX_E || k == 0 || T == 0) return PLOW_MOE_EINVAL;
    RouterArgs a = {(PlowMoeRoute*)table, logit, bias, n_exp, k, flags, T, tail, n_group, topk_group,
                    route_scale, logit_scale};
    const dim3 g((T + RT_WAVES - 1) / RT_WAVES), b(RT_WAVES * WAVE);
    /* the smallest instance that holds the experts: a lane's idle candidates cost every selection round */
    if (n_exp <= 64u) k_router_topk<1><<<g, b, 0, st>>>(a);
    else if (n_exp <= 128u) k_router_topk<2><<<g, b, 0, st>>>(a);
    else if (n_exp <= 192u) k_router_topk<3><<<g, b, 0, st>>>(a);
    else if (n_exp <= 256u) k_router_topk<4><<<g, b, 0, st>>>(a);
    else if (n_exp <= 320u) k_router_topk<5><<<g, b, 0, st>>>(a);
    else if (n_exp <= 384u) k_router_topk<6><<<g, b, 0, st>>>(a);
    else if (n_exp <= 512u) k_router_topk<8><<<g, b, 0, st>>>(a);
    else if (n_exp <= 768u) k_router_topk<12><<<g, b, 0, st>>>(a);
    else k_router_topk<16><<<g, b, 0, st>>>(a);
    return 0;
}

/* ============================ op 84: align ===================================================== */
/* One workgroup of 16 waves; a counting sort with one chunk per wave, so the scatter needs no
 * atomics and the result is the reference's order (ascending slot inside each expert,
 * plow runtime/cpu/dev/golden/moe_route.c:118-125):
 *   A  wave w histograms its contiguous range of slots into hist[w][*]          (LDS atomics: a
 *      count does not depend on arrival order)
 *   B  per expert: exclusive prefix over the 16 waves -> base[w][e]; padded prefix over experts ->
 *      rowoff / tilep; pad rows marked
 *   C  wave w walks its range in order, 64 slots a step; lanes with the same expert get consecutive
 *      positions by lane order (ballot + popcount), and the wave's cursor base[w][e] advances. */
#define AL_WAVES 16u
#define AL_MAX_E 1056u

struct AlignArgs {
    int32_t* meta;
    const PlowMoeRoute* table;
    uint32_t* row_token;
    uint32_t* row_partidx;
    float* row_gate;
    uint32_t T, E, k;
};

/* LDS words the single-workgroup align needs with nw waves */
#define AL_LDS_WORDS(nw) (((nw) + 2u) * AL_MAX_E + 64u)
#define AL_MAX_CHUNKS ((AL_MAX_E + WAVE - 1u) / WAVE) /* 64-expert chunks of the padded prefix: 17 */

/* How many lower lanes of the wave hold the same expert as this lane: the lane's position among its
 * expert's slots in this step (slots are in lane order). nl: lanes of the step that hold a slot (they are
 * the first nl). One permute and compare per distance, none of them waiting for another, instead of one
 * round of ballots per distinct expert of the step (some fifty rounds for 64 slots over 256 experts). */
__device__ __forceinline__ uint32_t al_rank_below(uint32_t e, uint32_t lane, uint32_t nl) {
    uint32_t rank = 0;
    for (uint32_t d = 1; d < nl; d++) {
        const uint32_t o = (uint32_t)__shfl_up((int)e, d, 64);
        rank += (lane >= d && o == e) ? 1u : 0u;
    }
    return rank;
}

/* Padded exclusive prefix over the experts' row counts, by all the waves of the workgroup: every wave scans
 * 64-expert chunks of tile counts, one wave scans the chunk totals, every thread finishes its experts.
 * In: s_cnt[e]. Out: s_rowoff[e], meta (rowoff | cnt | tilep | total tiles). s_chunk: 2 * AL_MAX_CHUNKS words.
 * Every thread of the workgroup calls this (three barriers inside; s_cnt must be complete before). */
__device__ __forceinline__ void al_padded_prefix(const AlignArgs& a, uint32_t* s_rowoff, const uint32_t* s_cnt,
                                                 uint32_t* s_chunk, uint32_t nthr) {
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wv = tid >> 6, nw = nthr >> 6, E = a.E;
    const uint32_t chunks = (E + WAVE - 1u) / WAVE;
    for (uint32_t ch = wv; ch < chunks; ch += nw) {
        const uint32_t e = ch * WAVE + lane;
        const uint32_t tiles = e < E ? (s_cnt[e] + PLOW_MPF_BM - 1u) / PLOW_MPF_BM : 0u;
        uint32_t inc = tiles;
#pragma unroll
        for (uint32_t o = 1; o < WAVE; o <<= 1) {
            const uint32_t v = __shfl_up(inc, o, 64);
            if (lane >= o) inc += v;
        }
        if (e < E) s_rowoff[e] = inc - tiles; /* tiles before this expert inside its chunk */
        if (lane == WAVE - 1u) s_chunk[ch] = inc;
    }
    __syncthreads();
    if (wv == 0) {
        const uint32_t v = lane < chunks ? s_chunk[lane] : 0u;
        uint32_t inc = v;
#pragma unroll
        for (uint32_t o = 1; o < WAVE; o <<= 1) {
            const uint32_t u = __shfl_up(inc, o, 64);
            if (lane >= o) inc += u;
        }
        if (lane < chunks) s_chunk[AL_MAX_CHUNKS + lane] = inc - v; /* tiles before the chunk */
        if (lane == WAVE - 1u) a.meta[3u * E] = (int32_t)inc;
    }
    __syncthreads();
    for (uint32_t e = tid; e < E; e += nthr) {
        const uint32_t excl = s_rowoff[e] + s_chunk[AL_MAX_CHUNKS + e / WAVE];
        s_rowoff[e] = excl * PLOW_MPF_BM;
        a.meta[e] = (int32_t)(excl * PLOW_MPF_BM);
        a.meta[E + e] = (int32_t)s_cnt[e];
        a.meta[2u * E + e] = (int32_t)excl;
    }
    __syncthreads();
}
/* The whole workgroup (nw waves) calls this; lds: AL_LDS_WORDS(nw) words. */
__device__ __forceinline__ void align_body(const AlignArgs& a, uint32_t* lds, uint32_t nw) {
    uint32_t(*hist)[AL_MAX_E] = (uint32_t(*)[AL_MAX_E])lds;
    uint32_t* const s_rowoff = lds + nw * AL_MAX_E;
    uint32_t* const s_cnt = s_rowoff + AL_MAX_E;
    uint32_t* const s_chunk = s_cnt + AL_MAX_E;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wv = tid >> 6, nthr = nw * WAVE;
    const uint32_t E = a.E, nslot = a.T * a.k;
    /* slots per wave, a multiple of 64 so that every step of phase C is a whole wave */
    const uint32_t per = ((nslot + nthr - 1u) / nthr) * WAVE;
    const uint32_t lo = wv * per < nslot ? wv * per : nslot, hi = lo + per < nslot ? lo + per : nslot;

    /* the wave's first 64 slots are asked for before anything else and kept: the trip to memory runs under the
     * clearing of the histograms, and the scatter's first step (the only one up to 1024 slots) needs no second */
    const uint32_t e_first = lo + lane < hi ? a.table[lo + lane].eid : PLOW_EXPERT_UNUSED;
    const float g_first = lo + lane < hi ? a.table[lo + lane].gate : 0.0f;
    /* the histograms of all waves sit in one run of words (rows of AL_MAX_E, a multiple of four): 16 bytes a store */
    {
        uint4* const z = (uint4*)lds;
        const uint32_t n4 = ((nw - 1u) * AL_MAX_E + E + 3u) / 4u;
        for (uint32_t i = tid; i < n4; i += nthr) z[i] = make_uint4(0u, 0u, 0u, 0u);
    }
    __syncthreads();
    for (uint32_t s = lo + lane; s < hi; s += WAVE) {
        const uint32_t e = s < lo + WAVE ? e_first : a.table[s].eid;
        if (e < E) atomicAdd(&hist[wv][e], 1u);
    }
    __syncthreads();
    for (uint32_t e = tid; e < E; e += nthr) {
        uint32_t run = 0;
        for (uint32_t w = 0; w < nw; w++) {
            const uint32_t c = hist[w][e];
            hist[w][e] = run;
            run += c;
        }
        s_cnt[e] = run;
    }
    __syncthreads();
    al_padded_prefix(a, s_rowoff, s_cnt, s_chunk, nthr);
    /* pad rows: [rowoff + cnt, rowoff + 64 * ceil(cnt / 64)) */
#pragma unroll 4
    for (uint32_t i = tid; i < E * PLOW_MPF_BM; i += nthr) {
        const uint32_t e = i / PLOW_MPF_BM, j = i % PLOW_MPF_BM;
        const uint32_t c = s_cnt[e], r = s_rowoff[e] + c + j;
        if (c + j < ((c + PLOW_MPF_BM - 1u) / PLOW_MPF_BM) * PLOW_MPF_BM) {
            a.row_token[r] = PLOW_EXPERT_UNUSED;
            a.row_partidx[r] = PLOW_EXPERT_UNUSED;
            a.row_gate[r] = 0.0f;
        }
    }
    /* stable scatter, each wave on its own range and its own cursors (no block barrier needed): a slot goes
     * to its expert's first row + the wave's cursor + its position among the step's slots of that expert;
     * the cursors advance after every lane has read its own (a wave's LDS operations run in order) */
    for (uint32_t s0 = lo; s0 < hi; s0 += WAVE) {
        const uint32_t s = s0 + lane;
        const bool in = s < hi;
        const uint32_t e = s0 == lo ? e_first : (in ? a.table[s].eid : PLOW_EXPERT_UNUSED);
        const float g = s0 == lo ? g_first : (in ? a.table[s].gate : 0.0f);
        const bool live = e < E;
        const uint32_t nl = hi - s0 < WAVE ? hi - s0 : WAVE;
        const uint32_t rank = al_rank_below(e, lane, nl);
        if (live) {
            const uint32_t pos = s_rowoff[e] + hist[wv][e] + rank;
            atomicAdd(&hist[wv][e], 1u);
            a.row_token[pos] = s / a.k;
            a.row_partidx[pos] = s;
            a.row_gate[pos] = g;
        }
    }
}
__global__ __launch_bounds__(AL_WAVES* WAVE) void k_align(AlignArgs a) {
    __shared__ __attribute__((aligned(16))) uint32_t al_lds[AL_LDS_WORDS(AL_WAVES)];
    align_body(a, al_lds, AL_WAVES);
}

/* ============================ the decode router's score with its top-k in one launch ============ */
/* Op 180 marked as carrying its top-k (plow crates/packet/src/dev.rs:90-94, runtime/amd/
 * router_decode.hip:1-63). The score workgroups of a token group count themselves off on the group's
 * arrival counter; the last to arrive runs the top-k of the group's tokens, one wave per token. The
 * bodies are those of the separate kernels: same logits, same table. A counter is zero between launches
 * (the last arrival puts it back); launches that share counters must not overlap. */
struct RouterFuse {
    uint32_t* ctr;       /* token group g counts itself off on ctr[g * stride] */
    uint32_t stride;
    RouterArgs topk;
};
template <uint32_t TOK>
__global__ __launch_bounds__((TOK + RSR_STAGERS) * 64u) void k_router_decode(float* __restrict__ out,
                                                                             const bf16_t* __restrict__ x,
                                                                             const bf16_t* __restrict__ w,
                                                                             uint32_t M, uint32_t N, uint32_t K, RouterFuse f) {
    extern __shared__ __attribute__((aligned(16))) uint8_t rsr_raw[];
    __shared__ uint32_t s_flag;
    router_score_row_body<TOK>(out, x, w, M, N, K, blockIdx.x, blockIdx.y, rsr_raw);
    if (!rf_last_arrival(f.ctr + (size_t)blockIdx.y * f.stride, gridDim.x, &s_flag)) return;
    const uint32_t wv = threadIdx.x >> 6, tok = blockIdx.y * TOK + wv;
    if (wv < TOK && tok < M) router_topk_token_any(f.topk, tok, (float*)rsr_raw + wv * RT_MAX_E);
}
static_assert(RSR_LDS >= 4u * RT_MAX_E * 4u, "the top-k borrows the score kernel's LDS");

static bool rf_setup() {
    return hipFuncSetAttribute((const void*)k_router_decode<1>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)RSR_LDS) == hipSuccess &&
           hipFuncSetAttribute((const void*)k_router_decode<2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)RSR_LDS) == hipSuccess;
}

/* The one-launch form serves the shapes the few-token score kernel above serves (below 16 tokens, K a
 * multiple of its chunk, 32-bit lane offsets). */
bool router_decode_serves(const RouterRun& r) {
    return r.row_ctr && r.table && r.logit && r.x && r.w && r.M >= 1u && r.M < 16u && r.N >= 1u && r.N <= RT_MAX_E &&
           r.k >= 1u && !plow_moe_tuning().score_tile8 && r.K % RSR_KC == 0u && (uint64_t)r.N * r.K * 2u < (1ull << 31) &&
           (uint64_t)r.M * r.K * 2u < (1ull << 31);
}
int launch_router_decode(const RouterRun& r, hipStream_t st) {
    if (!router_decode_serves(r)) return PLOW_MOE_EINVAL;
    RouterFuse f = {};
    const uint32_t tok = r.M >= 4u ? 2u : 1u;
    f.ctr = r.row_ctr, f.stride = tok * 32u; /* one counter per row, 32 words apart: a group takes its first row's */
    f.topk = {(PlowMoeRoute*)r.table, r.logit, r.bias, r.N, r.k, r.flags, r.M, r.tail, r.n_group, r.topk_group,
              r.route_scale, r.logit_scale};
    const uint32_t nx = (r.N + 63u) / 64u;
    if (tok == 2u)
        k_router_decode<2><<<dim3(nx, (r.M + 1u) / 2u), (2u + RSR_STAGERS) * 64u, RSR_LDS, st>>>(
            (float*)r.logit, (const bf16_t*)r.x, (const bf16_t*)r.w, r.M, r.N, r.K, f);
    else
        k_router_decode<1><<<dim3(nx, r.M), (1u + RSR_STAGERS) * 64u, RSR_LDS, st>>>(
            (float*)r.logit, (const bf16_t*)r.x, (const bf16_t*)r.w, r.M, r.N, r.K, f);
    return 0;
}

/* Many slots (prefill): the same counting sort spread over the chip in three launches.
 *   hist     one workgroup per chunk of 1024 slots: per-expert counts of the chunk -> chunk_hist
 *   scan     one workgroup: per expert, exclusive prefix over the chunks (in place); counts, padded
 *            offsets and tile prefix -> meta; pad rows marked
 *   scatter  one workgroup per chunk: the single-workgroup algorithm above on the chunk's 16 waves,
 *            starting from rowoff[e] + chunk prefix
 * chunk_hist is u32 [chunks][E] in the context workspace. */
#define AL_CHUNK (AL_WAVES * WAVE)

__global__ __launch_bounds__(AL_CHUNK) void k_align_hist(const PlowMoeRoute* __restrict__ table,
                                                         uint32_t* __restrict__ chunk_hist,
                                                         uint32_t nslot, uint32_t E) {
    __shared__ uint32_t h[AL_MAX_E];
    const uint32_t tid = threadIdx.x, s = blockIdx.x * AL_CHUNK + tid;
    for (uint32_t e = tid; e < E; e += AL_CHUNK) h[e] = 0u;
    __syncthreads();
    if (s < nslot) {
        const uint32_t e = table[s].eid;
        if (e < E) atomicAdd(&h[e], 1u);
    }
    __syncthreads();
    for (uint32_t e = tid; e < E; e += AL_CHUNK) chunk_hist[(size_t)blockIdx.x * E + e] = h[e];
}

__global__ __launch_bounds__(AL_CHUNK) void k_align_scan(AlignArgs a, uint32_t* __restrict__ chunk_hist,
                                                         uint32_t nchunk) {
    __shared__ uint32_t s_rowoff[AL_MAX_E];
    __shared__ uint32_t s_cnt[AL_MAX_E];
    __shared__ uint32_t s_chunk[2u * AL_MAX_CHUNKS];
    const uint32_t tid = threadIdx.x, E = a.E;
    for (uint32_t e = tid; e < E; e += AL_CHUNK) {
        uint32_t run = 0;
        /* eight chunks' counts are asked for together: one trip to memory per eight, not one per chunk */
        for (uint32_t c0 = 0; c0 < nchunk; c0 += 8u) {
            uint32_t v[8];
#pragma unroll
            for (uint32_t j = 0; j < 8u; j++) v[j] = c0 + j < nchunk ? chunk_hist[(size_t)(c0 + j) * E + e] : 0u;
#pragma unroll
            for (uint32_t j = 0; j < 8u; j++) {
                if (c0 + j < nchunk) chunk_hist[(size_t)(c0 + j) * E + e] = run;
                run += v[j];
            }
        }
        s_cnt[e] = run;
    }
    __syncthreads();
    al_padded_prefix(a, s_rowoff, s_cnt, s_chunk, AL_CHUNK);
#pragma unroll 4
    for (uint32_t i = tid; i < E * PLOW_MPF_BM; i += AL_CHUNK) {
        const uint32_t e = i / PLOW_MPF_BM, j = i % PLOW_MPF_BM;
        const uint32_t c = s_cnt[e], r = s_rowoff[e] + c + j;
        if (c + j < ((c + PLOW_MPF_BM - 1u) / PLOW_MPF_BM) * PLOW_MPF_BM) {
            a.row_token[r] = PLOW_EXPERT_UNUSED;
            a.row_partidx[r] = PLOW_EXPERT_UNUSED;
            a.row_gate[r] = 0.0f;
        }
    }
}

__global__ __launch_bounds__(AL_CHUNK) void k_align_scatter(AlignArgs a, const uint32_t* __restrict__ chunk_hist) {
    __shared__ __attribute__((aligned(16))) uint32_t hist[AL_WAVES][AL_MAX_E];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wv = tid >> 6;
    const uint32_t E = a.E, nslot = a.T * a.k;
    const uint32_t s = blockIdx.x * AL_CHUNK + tid;
    {
        uint4* const z = (uint4*)&hist[0][0];
        const uint32_t n4 = ((AL_WAVES - 1u) * AL_MAX_E + E + 3u) / 4u;
        for (uint32_t i = tid; i < n4; i += AL_CHUNK) z[i] = make_uint4(0u, 0u, 0u, 0u);
    }
    __syncthreads();
    const bool in = s < nslot;
    const uint32_t e = in ? a.table[s].eid : PLOW_EXPERT_UNUSED;
    const float g = in ? a.table[s].gate : 0.0f;
    const bool live = e < E;
    if (live) atomicAdd(&hist[wv][e], 1u);
    __syncthreads();
    /* exclusive prefix over the waves, started at this chunk's global position in the expert */
    for (uint32_t x = tid; x < E; x += AL_CHUNK) {
        uint32_t run = (uint32_t)a.meta[x] + chunk_hist[(size_t)blockIdx.x * E + x];
#pragma unroll
        for (uint32_t w = 0; w < AL_WAVES; w++) {
            const uint32_t c = hist[w][x];
            hist[w][x] = run;
            run += c;
        }
    }
    __syncthreads();
    const uint32_t s0 = blockIdx.x * AL_CHUNK + wv * WAVE; /* the wave's first slot */
    const uint32_t nl = s0 >= nslot ? 0u : (nslot - s0 < WAVE ? nslot - s0 : WAVE);
    const uint32_t rank = al_rank_below(e, lane, nl);
    if (live) {
        const uint32_t pos = hist[wv][e] + rank;
        a.row_token[pos] = s / a.k;
        a.row_partidx[pos] = s;
        a.row_gate[pos] = g;
    }
}

int launch_align(int32_t* meta, const void* table, uint32_t* row_token, uint32_t* row_partidx,
                 float* row_gate, uint32_t T, uint32_t E, uint32_t k, uint32_t* chunk_hist,
                 uint32_t chunk_cap, hipStream_t st) {
    if (E == 0 || E > AL_MAX_E || k == 0) return PLOW_MOE_EINVAL;
    AlignArgs a = {meta, (const PlowMoeRoute*)table, row_token, row_partidx, row_gate, T, E, k};
    const uint32_t nslot = T * k, nchunk = (nslot + AL_CHUNK - 1u) / AL_CHUNK;
    /* one workgroup up to 2048 slots (12 us at 768 slots, 18.5 at 2048, 29.5 at 4096; the three-kernel form
     * takes 20 - 22 us at any of these sizes) */
    if (nslot <= 2u * AL_CHUNK || !chunk_hist || nchunk > chunk_cap) {
        k_align<<<1, AL_WAVES * WAVE, 0, st>>>(a);
        return 0;
    }
    k_align_hist<<<nchunk, AL_CHUNK, 0, st>>>((const PlowMoeRoute*)table, chunk_hist, nslot, E);
    k_align_scan<<<1, AL_CHUNK, 0, st>>>(a, chunk_hist, nchunk);
    k_align_scatter<<<nchunk, AL_CHUNK, 0, st>>>(a, chunk_hist);
    return 0;
}

/* ============================ ops 87 / 43: combine ============================================= */
#include "combine_body.h"

template <uint32_t KT>
__global__ __launch_bounds__(256) void k_combine(CombineArgs a) {
    combine_body<KT>(a);
}

/* The deterministic fused combine (plow runtime/amd/op_moe.h:5380-5520): the DOWN op has summed the k
 * contributions of every token in place as integer-valued doubles (fixed point, 2^-32), so this reads one
 * contiguous f64 stream: out = bf16(residual? + shared? + (float)(acc * 2^-32)), four h per thread. */
__global__ __launch_bounds__(256) void k_combine_det(bf16_t* __restrict__ out, const bf16_t* __restrict__ residual,
                                                     const bf16_t* __restrict__ shared, const double* __restrict__ acc64,
                                                     uint32_t H, uint32_t T) {
    const size_t total = (size_t)T * (H / 4u);
    for (size_t i = (size_t)blockIdx.x * 256u + threadIdx.x; i < total; i += (size_t)gridDim.x * 256u) {
        const size_t o = i * 4u;
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        const double4 v = *(const double4*)(acc64 + o);
        if (residual) {
            const uint2 r = *(const uint2*)(residual + o);
            acc[0] = __uint_as_float(r.x << 16); acc[1] = __uint_as_float(r.x & 0xFFFF0000u);
            acc[2] = __uint_as_float(r.y << 16); acc[3] = __uint_as_float(r.y & 0xFFFF0000u);
        }
        if (shared) {
            const uint2 r = *(const uint2*)(shared + o);
            acc[0] += __uint_as_float(r.x << 16); acc[1] += __uint_as_float(r.x & 0xFFFF0000u);
            acc[2] += __uint_as_float(r.y << 16); acc[3] += __uint_as_float(r.y & 0xFFFF0000u);
        }
        acc[0] += (float)(v.x * PLOW_DET_UNSCALE); acc[1] += (float)(v.y * PLOW_DET_UNSCALE);
        acc[2] += (float)(v.z * PLOW_DET_UNSCALE); acc[3] += (float)(v.w * PLOW_DET_UNSCALE);
        uint2 w;
        w.x = (uint32_t)f2bf(acc[0]) | ((uint32_t)f2bf(acc[1]) << 16);
        w.y = (uint32_t)f2bf(acc[2]) | ((uint32_t)f2bf(acc[3]) << 16);
        *(uint2*)(out + o) = w;
    }
}

int launch_combine_det(void* out, const void* residual, const void* shared, const double* acc, uint32_t H, uint32_t T,
                       hipStream_t st) {
    if (H % 4u || T == 0) return PLOW_MOE_EINVAL;
    const size_t total = (size_t)T * (H / 4u);
    uint32_t blocks = (uint32_t)((total + 255u) / 256u);
    if (blocks > 4096u) blocks = 4096u;
    k_combine_det<<<blocks, 256, 0, st>>>((bf16_t*)out, (const bf16_t*)residual, (const bf16_t*)shared, acc, H, T);
    return 0;
}

/* zero-fill of the f64 accumulator (a kernel, not a memset: the call may be captured into a graph) */
__global__ __launch_bounds__(256) void k_zero_f64(double2* __restrict__ p, size_t n2, double* __restrict__ tail, uint32_t ntail) {
    for (size_t i = (size_t)blockIdx.x * 256u + threadIdx.x; i < n2; i += (size_t)gridDim.x * 256u) p[i] = make_double2(0.0, 0.0);
    if (blockIdx.x == 0 && threadIdx.x < ntail) tail[threadIdx.x] = 0.0;
}

int launch_zero_f64(double* p, size_t n, hipStream_t st) {
    if (n == 0) return 0;
    if ((uintptr_t)p % 16u) return PLOW_MOE_EINVAL;
    const size_t n2 = n / 2u;
    uint32_t blocks = (uint32_t)((n2 + 255u) / 256u);
    if (blocks > 4096u) blocks = 4096u;
    if (blocks == 0u) blocks = 1u;
    k_zero_f64<<<blocks, 256, 0, st>>>((double2*)p, n2, p + 2u * n2, (uint32_t)(n & 1u));
    return 0;
}

int launch_combine(void* out, const void* residual, const void* shared, const void* part, uint32_t H,
                   uint32_t k, uint32_t T, uint32_t part16, hipStream_t st) {
    if (H % 4u || T == 0) return PLOW_MOE_EINVAL;
    CombineArgs a = {(bf16_t*)out, (const bf16_t*)residual, (const bf16_t*)shared, part, H, k, T, part16};
    const size_t total = (size_t)T * (H / 4u);
    uint32_t blocks = (uint32_t)((total + 255u) / 256u);
    if (blocks > 4096u) blocks = 4096u;
    switch (part16 ? 0u : k) {
    case 4: k_combine<4><<<blocks, 256, 0, st>>>(a); break;
    case 6: k_combine<6><<<blocks, 256, 0, st>>>(a); break;
    case 8: k_combine<8><<<blocks, 256, 0, st>>>(a); break;
    case 9: k_combine<9><<<blocks, 256, 0, st>>>(a); break;
    default: k_combine<0><<<blocks, 256, 0, st>>>(a); break;
    }
    return 0;
}
