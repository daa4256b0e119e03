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

/* Large problems with K a multiple of 64: the same sums on the matrix unit. v_mfma_f32_32x32x2_f32
 * adds a[i][k] * b[k][j], then a[i][k + 1] * b[k + 1][j], to its f32 accumulator, each step rounded
 * to nearest even and denormals kept (measured against the fmaf chain, bit for bit, normal and
 * denormal ranges), so a chain of K / 2 of them IS the reference's sum in the reference's order, at
 * twice the rate of the vector unit and without an operand broadcast through LDS.
 * One wave per workgroup computes 32 tokens x 32 experts. Operand rows (bf16, 64 k = one 128-byte line
 * per row and chunk) come in by direct global -> LDS loads in the coalesced shape into a wave-private
 * ring of three chunks, two chunks ahead; no barrier anywhere. A lane reads 16 bytes (8 k) of its
 * token row and of its expert row per piece; lanes 0..31 feed the even k of a pair to the instruction
 * and lanes 32..63 the odd k (one byte permute each widens bf16 to f32). The next piece's LDS reads
 * are issued before the four matrix instructions of this piece and waited for after them. LDS piece p
 * of row r holds global piece p ^ ((r >> 1) & 7): 16 consecutive rows of a piece cover all 64 banks. */
#define RSM_STAGES 3
struct RsmStage {
    uint8_t x[32u * 128u];
    uint8_t w[32u * 128u];
};
typedef __attribute__((address_space(3))) void rsm_lds_void;
/* NWV waves per workgroup, rings of ST chunks: 4 x 3 (one wave per SIMD, two chunks ahead), or 8 x 2 (two waves
 * per SIMD, one chunk ahead: a wave's matrix instructions fill the other's issue gaps) when there are tiles
 * enough for two per SIMD. */
template <uint32_t NWV, uint32_t ST>
__global__ __launch_bounds__(NWV * 64u) void k_router_score_mfma(float* __restrict__ out, const bf16_t* __restrict__ x,
                                                                 const bf16_t* __restrict__ w, uint32_t M, uint32_t N,
                                                                 uint32_t K) {
    static_assert((NWV == 4u && ST == 3u) || (NWV == 8u && ST == 2u), "4 waves x 3 chunks or 8 waves x 2 chunks");
    /* independent waves (a 2 x 2 or 4 x 2 block of tiles): 96 / 128 KB of LDS makes it one workgroup per CU,
     * which puts exactly one (two) waves on every SIMD */
    extern __shared__ __attribute__((aligned(16))) uint8_t rsm_raw[];
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wv = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    RsmStage* const ring = (RsmStage*)rsm_raw + wv * ST;
    /* Workgroup b runs on XCD b % 8 and each XCD has its own L2: the logical index gives one XCD
     * consecutive workgroups, which share their token rows (the expert-tile index runs fastest) */
    const uint32_t G = gridDim.x, gx = (N + 63u) / 64u;
    const uint32_t wg = (G % 8u == 0u) ? (blockIdx.x % 8u) * (G / 8u) + blockIdx.x / 8u : blockIdx.x;
    const uint32_t m0 = ((wg / gx) * (NWV / 2u) + (wv >> 1)) * 32u, n0 = ((wg % gx) * 2u + (wv & 1u)) * 32u;
    if (m0 >= M || n0 >= N) return; /* whole wave; there is no barrier below */
    const uint32_t NC = K / 64u;
    /* load j covers rows 8j .. 8j + 7: lane -> (row lane >> 3, LDS piece lane & 7); rows past the end
     * of the matrix read its last row and are never stored */
    const uint32_t lr = lane >> 3, lp = lane & 7u;
    const uint8_t *xsrc[4], *wsrc[4];
#pragma unroll
    for (uint32_t j = 0; j < 4u; j++) {
        const uint32_t row = 8u * j + lr;
        const uint32_t mr = m0 + row < M ? m0 + row : M - 1u, nr = n0 + row < N ? n0 + row : N - 1u;
        xsrc[j] = (const uint8_t*)(x + (size_t)mr * K) + ((lp ^ ((row >> 1) & 7u)) << 4);
        wsrc[j] = (const uint8_t*)(w + (size_t)nr * K) + ((lp ^ ((row >> 1) & 7u)) << 4);
    }
    auto issue = [&](uint32_t c) {
        RsmStage* s = &ring[c % ST];
#pragma unroll
        for (uint32_t j = 0; j < 4u; j++)
            __builtin_amdgcn_global_load_lds((const void*)(xsrc[j] + (size_t)c * 128u), (rsm_lds_void*)&s->x[8u * j * 128u], 16, 0, 0);
#pragma unroll
        for (uint32_t j = 0; j < 4u; j++)
            __builtin_amdgcn_global_load_lds((const void*)(wsrc[j] + (size_t)c * 128u), (rsm_lds_void*)&s->w[8u * j * 128u], 16, 0, 0);
    };
    /* operand reads: row lane & 31 of the token rows (A) and of the expert rows (B) */
    const uint32_t orow = lane & 31u, osw = (orow >> 1) & 7u;
    const uint32_t ring0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)&ring[0];
    const uint32_t obase = ring0 + orow * 128u;
    const uint32_t sel = lane < 32u ? 0x01000c0cu : 0x03020c0cu; /* low / high bf16 of a dword -> f32 bits */
    v16f acc;
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.0f;
    /* Per piece: issue the next piece's LDS reads, run this piece's four matrix instructions, wait for
     * the reads, widen them into the other half of the operand registers. An instruction's operands
     * are never overwritten while it may still be reading them (the vector unit would wait for it), and
     * the widening runs under the last matrix instruction of the piece. */
    v4i xa, wb;
    float af[2][4], bf[2][4];
    auto read_piece = [&](uint32_t stage, uint32_t pc) {
        const uint32_t addr = obase + stage * (uint32_t)sizeof(RsmStage) + ((pc ^ osw) << 4);
        /* early-clobber outputs: the first read's destination must not be the register the second takes its
         * address from (the data may land before the second instruction issues) */
        asm volatile("ds_read_b128 %0, %2\n\tds_read_b128 %1, %2 offset:4096" : "=&v"(xa), "=&v"(wb) : "v"(addr) : "memory");
    };
    auto widen = [&](uint32_t h, int d0, int d1) {
        if (d0 == 0) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(xa), "+v"(wb));
#pragma unroll
        for (int d = d0; d < d1; d++) {
            af[h][d] = __uint_as_float(__builtin_amdgcn_perm((uint32_t)xa[d], (uint32_t)xa[d], sel));
            bf[h][d] = __uint_as_float(__builtin_amdgcn_perm((uint32_t)wb[d], (uint32_t)wb[d], sel));
        }
    };
    issue(0u);
    if (NC > 1u) issue(1u);
    if (ST > 2u && NC > 2u) issue(2u);
    if (ST > 2u && NC > 2u) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    else if (NC > 1u) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    read_piece(0u, 0u);
    widen(0u, 0, 4);
    uint32_t st = 0;
#define RSM_MFMA(d) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[cur][d], bf[cur][d], acc, 0, 0, 0)
#define RSM_FENCE() __builtin_amdgcn_sched_barrier(0)
    for (uint32_t c = 0; c < NC; c++) {
        const uint32_t stn = st == ST - 1u ? 0u : st + 1u;
#pragma unroll
        for (uint32_t pc = 0; pc < 8u; pc++) {
            const uint32_t cur = pc & 1u, nxt = cur ^ 1u;
            /* everything that is not a matrix instruction is issued behind one, so that the matrix unit
             * is busy while the wave issues it */
            RSM_FENCE();
            RSM_MFMA(0);
            RSM_FENCE();
            if (pc == 7u) {
                /* every piece of chunk c has been read: chunk c + 1 must have landed before its first
                 * piece is read (with three stages chunk c + 2's loads may stay outstanding), and chunk c's
                 * stage takes chunk c + ST */
                if (ST > 2u && c + 2u < NC) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
                else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                read_piece(stn, 0u); /* past the last chunk: stale bytes, never used */
            } else {
                read_piece(st, pc + 1u);
            }
            RSM_FENCE();
            RSM_MFMA(1);
            RSM_FENCE();
            if (pc == 7u && c + ST < NC) {
                RsmStage* s = &ring[(c + ST) % ST];
#pragma unroll
                for (uint32_t j = 0; j < 4u; j++)
                    __builtin_amdgcn_global_load_lds((const void*)(xsrc[j] + (size_t)(c + ST) * 128u), (rsm_lds_void*)&s->x[8u * j * 128u], 16, 0, 0);
            }
            RSM_FENCE();
            RSM_MFMA(2);
            RSM_FENCE();
            if (pc == 7u && c + ST < NC) {
                RsmStage* s = &ring[(c + ST) % ST];
#pragma unroll
                for (uint32_t j = 0; j < 4u; j++)
                    __builtin_amdgcn_global_load_lds((const void*)(wsrc[j] + (size_t)(c + ST) * 128u), (rsm_lds_void*)&s->w[8u * j * 128u], 16, 0, 0);
            }
            RSM_FENCE();
            widen(nxt, 0, 2);
            RSM_FENCE();
            RSM_MFMA(3);
            RSM_FENCE();
            widen(nxt, 2, 4);
        }
        st = stn;
    }
#undef RSM_MFMA
#undef RSM_FENCE
    /* acc[r] = out[m0 + 8 * (r / 4) + 4 * (lane / 32) + r % 4][n0 + lane % 32] */
    const uint32_t n = n0 + (lane & 31u);
#pragma unroll
    for (uint32_t r = 0; r < 16u; r++) {
        const uint32_t m = m0 + 8u * (r >> 2) + 4u * (lane >> 5) + (r & 3u);
        if (m < M && n < N) out[(size_t)m * N + n] = acc[r];
    }
}

/* The 32 x 32 form as it runs by default. Two facts of the part shape it. (1) The f32 matrix instructions
 * execute on the vector unit's own multiply-add lanes (the f32 matrix peak equals the vector f32 peak): vector
 * instructions between two of them do not hide behind them, they add (measured: the eight byte permutes that
 * widened a piece's bf16 operands cost 9 cycles each, 29 of 173 us at T = 4096, E = 256, K = 7168). So operands
 * are widened by the LDS read itself: ds_read_u16_d16_hi puts a bf16 into the high half of a register whose
 * low half is zero, which is the f32; the per-lane addresses of the eight pieces are computed once (the XOR
 * swizzle makes them lane-dependent) and the stage and element are immediate offsets, so the loop issues no
 * vector instruction at all next to its matrix instructions except a chunk's four load addresses.
 * (2) The operand rows of a workgroup's four tiles (64 tokens x 64 experts) are loaded once: a stage holds
 * 64 + 64 rows (16 KB), each wave loads a quarter of it and the four waves meet at one barrier per chunk,
 * after a wave's last LDS read of chunk c has landed and its own loads of chunk c + 1 have: behind the barrier
 * chunk c + 1 is complete and chunk c's stage is free for chunk c + 3. 48 KB of LDS: a CU takes up to three
 * workgroups when the grid has them. */
struct RssStage {
    uint8_t x[64u * 128u];
    uint8_t w[64u * 128u];
};
static_assert(sizeof(RssStage) == 16384u, "the stage size is an immediate of the LDS reads below");
/* eight 2-byte reads: elements 0, 2, 4, 6 of the lane's half of a 16-byte piece (the lane's address already
 * holds its even / odd byte), of its token row and of its expert row; stage STG of the ring */
template <uint32_t STG>
__device__ __forceinline__ void rss_read(float (&a)[4], float (&b)[4], uint32_t ax, uint32_t aw) {
    asm volatile("ds_read_u16_d16_hi %0, %8 offset:%10\n\t"
                 "ds_read_u16_d16_hi %4, %9 offset:%10\n\t"
                 "ds_read_u16_d16_hi %1, %8 offset:%11\n\t"
                 "ds_read_u16_d16_hi %5, %9 offset:%11\n\t"
                 "ds_read_u16_d16_hi %2, %8 offset:%12\n\t"
                 "ds_read_u16_d16_hi %6, %9 offset:%12\n\t"
                 "ds_read_u16_d16_hi %3, %8 offset:%13\n\t"
                 "ds_read_u16_d16_hi %7, %9 offset:%13"
                 : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3])
                 : "v"(ax), "v"(aw), "n"(STG * 16384u), "n"(STG * 16384u + 4u), "n"(STG * 16384u + 8u), "n"(STG * 16384u + 12u)
                 : "memory");
}
__device__ __forceinline__ void rss_wait_reads(float (&a)[4], float (&b)[4]) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]));
}
__global__ __launch_bounds__(256) void k_router_score_mfma_shared(float* __restrict__ out, const bf16_t* __restrict__ x,
                                                                  const bf16_t* __restrict__ w, uint32_t M, uint32_t N,
                                                                  uint32_t K) {
    extern __shared__ __attribute__((aligned(16))) uint8_t rss_raw[];
    constexpr uint32_t ST = RSM_STAGES;
    static_assert(ST == 3u, "the chunk loop below is written out for three stages");
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wv = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    RssStage* const ring = (RssStage*)rss_raw;
    const uint32_t G = gridDim.x, gx = (N + 63u) / 64u;
    const uint32_t wg = (G % 8u == 0u) ? (blockIdx.x % 8u) * (G / 8u) + blockIdx.x / 8u : blockIdx.x;
    const uint32_t M0 = (wg / gx) * 64u, N0 = (wg % gx) * 64u;          /* the workgroup's block */
    const uint32_t m0 = M0 + (wv >> 1) * 32u, n0 = N0 + (wv & 1u) * 32u; /* this wave's tile */
    const uint32_t NC = K / 64u;
    /* this wave's share of a stage: rows 16 wv .. 16 wv + 15 of both operands, two loads of eight rows each;
     * rows past the end of a matrix read its last row and are never stored. No wave leaves early: every wave
     * loads for the others and takes part in the barriers. A load's address is a base the whole wave shares
     * (the block's first row, advanced by the chunk) plus a 32-bit lane offset. */
    const uint32_t lr = lane >> 3, lp = lane & 7u;
    const uint8_t* const xblk = (const uint8_t*)(x + (size_t)M0 * K);
    const uint8_t* const wblk = (const uint8_t*)(w + (size_t)N0 * K);
    uint32_t xoff[2], woff[2];
#pragma unroll
    for (uint32_t j = 0; j < 2u; j++) {
        const uint32_t row = 16u * wv + 8u * j + lr;
        const uint32_t mr = M0 + row < M ? row : M - 1u - M0, nr = N0 + row < N ? row : N - 1u - N0;
        xoff[j] = mr * K * 2u + ((lp ^ ((row >> 1) & 7u)) << 4);
        woff[j] = nr * K * 2u + ((lp ^ ((row >> 1) & 7u)) << 4);
    }
    auto issue = [&](uint32_t c, uint32_t stage) {
        RssStage* s = &ring[stage];
        uint64_t xcb = (uint64_t)(uintptr_t)(xblk + (size_t)c * 128u), wcb = (uint64_t)(uintptr_t)(wblk + (size_t)c * 128u);
        asm volatile("" : "+s"(xcb), "+s"(wcb));
        const uint8_t* const xc = (const uint8_t*)(uintptr_t)xcb;
        const uint8_t* const wc = (const uint8_t*)(uintptr_t)wcb;
        /* the chunk's base addresses and the lane offsets are made opaque here so that an address stays "scalar
         * base + 32-bit lane offset" (two scalar additions per chunk) instead of four 64-bit per-lane pointers
         * advanced on the vector unit */
#pragma unroll
        for (uint32_t j = 0; j < 2u; j++) {
            uint32_t o = xoff[j];
            asm volatile("" : "+v"(o));
            __builtin_amdgcn_global_load_lds((const void*)(xc + o), (rsm_lds_void*)&s->x[(16u * wv + 8u * j) * 128u], 16, 0, 0);
        }
#pragma unroll
        for (uint32_t j = 0; j < 2u; j++) {
            uint32_t o = woff[j];
            asm volatile("" : "+v"(o));
            __builtin_amdgcn_global_load_lds((const void*)(wc + o), (rsm_lds_void*)&s->w[(16u * wv + 8u * j) * 128u], 16, 0, 0);
        }
    };
    /* operand reads: lanes 0..31 take the even k of a pair, lanes 32..63 the odd k; row lane & 31 of the wave's
     * token rows and of its expert rows (32 is a multiple of 16: the swizzle of row 32 h + r is that of r) */
    const uint32_t orow = lane & 31u, osw = (orow >> 1) & 7u;
    const uint32_t ring0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)&ring[0];
    const uint32_t xrow = ring0 + ((wv >> 1) * 32u + orow) * 128u + (lane >> 5) * 2u;
    const uint32_t wrow = ring0 + 64u * 128u + ((wv & 1u) * 32u + orow) * 128u + (lane >> 5) * 2u;
    uint32_t ax[8], aw[8];
#pragma unroll
    for (uint32_t pc = 0; pc < 8u; pc++) ax[pc] = xrow + ((pc ^ osw) << 4), aw[pc] = wrow + ((pc ^ osw) << 4);
    v16f acc;
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.0f;
    float af[2][4], bf[2][4]; /* the low halves stay zero: the reads write high halves only */
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int d = 0; d < 4; d++) af[h][d] = 0.0f, bf[h][d] = 0.0f;
    issue(0u, 0u);
    if (NC > 1u) issue(1u, 1u);
    if (NC > 2u) issue(2u, 2u);
    if (NC > 2u) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else if (NC > 1u) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    asm volatile("s_barrier" ::: "memory"); /* chunk 0 is complete */
    rss_read<0u>(af[0], bf[0], ax[0], aw[0]);
    rss_wait_reads(af[0], bf[0]);
#define RSM_MFMA(d) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[cur][d], bf[cur][d], acc, 0, 0, 0)
#define RSM_FENCE() __builtin_amdgcn_sched_barrier(0)
    /* one chunk in stage STG (a constant: the reads' offsets are immediates) */
    auto chunk = [&](auto stg_, uint32_t c) {
        constexpr uint32_t STG = decltype(stg_)::value, STN = (STG + 1u) % ST;
#pragma unroll
        for (uint32_t pc = 0; pc < 8u; pc++) {
            const uint32_t cur = pc & 1u, nxt = cur ^ 1u;
            RSM_FENCE();
            RSM_MFMA(0);
            RSM_FENCE();
            if (pc == 7u) {
                /* this wave's reads of chunk c have all landed (piece 7 was waited for a piece ago); once its loads
                 * of chunk c + 1 have landed too, the barrier says both of every wave */
                if (c + 2u < NC) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
                else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                asm volatile("s_barrier" ::: "memory");
                rss_read<STN>(af[nxt], bf[nxt], ax[0], aw[0]); /* past the last chunk: stale bytes, never used */
            } else {
                rss_read<STG>(af[nxt], bf[nxt], ax[(pc + 1u) & 7u], aw[(pc + 1u) & 7u]);
            }
            RSM_FENCE();
            RSM_MFMA(1);
            RSM_FENCE();
            if (pc == 7u && c + ST < NC) issue(c + ST, STG); /* into the stage chunk c has left */
            RSM_FENCE();
            RSM_MFMA(2);
            RSM_FENCE();
            RSM_MFMA(3);
            RSM_FENCE();
            rss_wait_reads(af[nxt], bf[nxt]);
        }
    };
    for (uint32_t c = 0; c < NC; c += 3u) {
        chunk(std::integral_constant<uint32_t, 0u>{}, c);
        if (c + 1u < NC) chunk(std::integral_constant<uint32_t, 1u>{}, c + 1u);
        if (c + 2u < NC) chunk(std::integral_constant<uint32_t, 2u>{}, c + 2u);
    }
#undef RSM_MFMA
#undef RSM_FENCE
    /* acc[r] = out[m0 + 8 * (r / 4) + 4 * (lane / 32) + r % 4][n0 + lane % 32] */
    const uint32_t n = n0 + (lane & 31u);
#pragma unroll
    for (uint32_t r = 0; r < 16u; r++) {
        const uint32_t m = m0 + 8u * (r >> 2) + 4u * (lane >> 5) + (r & 3u);
        if (m < M && n < N) out[(size_t)m * N + n] = acc[r];
    }
}

/* The same on v_mfma_f32_16x16x4_f32 (four k per instruction, a quarter of the chain latency per k of
 * the 32x32x2 form, also bit-identical to the sequential sum): a wave computes 16 tokens x 32 experts as
 * two independent chains that share the token operand. Half the outputs per operand byte, but twice as
 * many, shorter-lived waves: this is the form for problems too small to fill the chip with 32 x 32
 * tiles, where the chain latency is the time (from 2^17 outputs; below that the vector-unit form, whose
 * chain is shorter still, wins). Lane = (row lane & 15, k lane >> 4): a lane reads the two
 * dwords of its row's 16-byte piece that hold k = 4 h + (lane >> 4), h = 0, 1, with one ds_read2_b32. */
#define RS16_NB 2
struct Rs16Stage {
    uint8_t x[16u * 128u];
    uint8_t w[RS16_NB * 16u * 128u];
};
__global__ __launch_bounds__(256) void k_router_score_mfma16(float* __restrict__ out, const bf16_t* __restrict__ x,
                                                             const bf16_t* __restrict__ w, uint32_t M, uint32_t N,
                                                             uint32_t K) {
    extern __shared__ __attribute__((aligned(16))) uint8_t rs16_raw[];
    constexpr int NB = RS16_NB, NLD = 2 + 2 * NB; /* direct loads per chunk */
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wv = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    Rs16Stage* const ring = (Rs16Stage*)rs16_raw + wv * RSM_STAGES;
    const uint32_t G = gridDim.x, tn_count = (N + 16u * NB - 1u) / (16u * NB), tm_count = (M + 15u) / 16u;
    const uint32_t wg = (G % 8u == 0u) ? (blockIdx.x % 8u) * (G / 8u) + blockIdx.x / 8u : blockIdx.x;
    const uint32_t wid = wg * 4u + wv;
    if (wid >= tn_count * tm_count) return; /* whole wave; there is no barrier below */
    const uint32_t m0 = (wid / tn_count) * 16u, n0 = (wid % tn_count) * (16u * NB);
    const uint32_t NC = K / 64u;
    const uint32_t lr = lane >> 3, lp = lane & 7u;
    const uint8_t *xsrc[2], *wsrc[2 * NB];
#pragma unroll
    for (uint32_t j = 0; j < 2u * NB; j++) {
        const uint32_t row = 8u * j + lr, sw = ((row & 15u) >> 1) & 7u;
        const uint32_t nr = n0 + row < N ? n0 + row : N - 1u;
        wsrc[j] = (const uint8_t*)(w + (size_t)nr * K) + ((lp ^ sw) << 4);
        if (j < 2u) {
            const uint32_t mr = m0 + row < M ? m0 + row : M - 1u;
            xsrc[j] = (const uint8_t*)(x + (size_t)mr * K) + ((lp ^ sw) << 4);
        }
    }
    auto issue = [&](uint32_t c) {
        Rs16Stage* s = &ring[c % RSM_STAGES];
#pragma unroll
        for (uint32_t j = 0; j < 2u; j++)
            __builtin_amdgcn_global_load_lds((const void*)(xsrc[j] + (size_t)c * 128u), (rsm_lds_void*)&s->x[8u * j * 128u], 16, 0, 0);
#pragma unroll
        for (uint32_t j = 0; j < 2u * NB; j++)
            __builtin_amdgcn_global_load_lds((const void*)(wsrc[j] + (size_t)c * 128u), (rsm_lds_void*)&s->w[8u * j * 128u], 16, 0, 0);
    };
    const uint32_t orow = lane & 15u, ks = lane >> 4, osw = (orow >> 1) & 7u;
    const uint32_t ring0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)&ring[0];
    const uint32_t obase = ring0 + orow * 128u + (ks >> 1) * 4u;
    const uint32_t sel = (ks & 1u) ? 0x03020c0cu : 0x01000c0cu;
    v4f acc[NB];
#pragma unroll
    for (int b = 0; b < NB; b++) acc[b] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
    /* Software pipeline over the 8-k pieces: while piece p multiplies, the reads of piece p + 1 (issued
     * during piece p - 1) are waited for and widened into the other half of the operand registers, and
     * the reads of piece p + 2 are issued. Everything but matrix instructions is issued behind one. */
    uint2 xa[2], wb[2][NB];
    float af[2][2], bf[2][NB][2];
    auto read_piece = [&](uint32_t stage, uint32_t pc, uint32_t buf) {
        const uint32_t addr = obase + stage * (uint32_t)sizeof(Rs16Stage) + ((pc ^ osw) << 4);
        asm volatile("ds_read2_b32 %0, %1 offset1:2" : "=v"(xa[buf]) : "v"(addr) : "memory");
#pragma unroll
        for (int b = 0; b < NB; b++)
            asm volatile("ds_read2_b32 %0, %1 offset1:2" : "=v"(wb[buf][b]) : "v"(addr + 2048u + (uint32_t)b * 2048u) : "memory");
    };
    auto wait_reads = [&](uint32_t buf) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(xa[buf]), "+v"(wb[buf][0]), "+v"(wb[buf][NB - 1])); };
    auto widen_x = [&](uint32_t buf) {
        af[buf][0] = __uint_as_float(__builtin_amdgcn_perm(xa[buf].x, xa[buf].x, sel));
        af[buf][1] = __uint_as_float(__builtin_amdgcn_perm(xa[buf].y, xa[buf].y, sel));
    };
    auto widen_w = [&](uint32_t buf, int b) {
        bf[buf][b][0] = __uint_as_float(__builtin_amdgcn_perm(wb[buf][b].x, wb[buf][b].x, sel));
        bf[buf][b][1] = __uint_as_float(__builtin_amdgcn_perm(wb[buf][b].y, wb[buf][b].y, sel));
    };
    issue(0u);
    if (NC > 1u) issue(1u);
    if (NC > 2u) issue(2u);
    if (NC > 2u) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NLD) : "memory");
    else if (NC > 1u) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NLD) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    read_piece(0u, 0u, 0u);
    wait_reads(0u);
    widen_x(0u);
#pragma unroll
    for (int b = 0; b < NB; b++) widen_w(0u, b);
    read_piece(0u, 1u, 1u);
    wait_reads(1u); /* nothing is in flight across the loop's back edge */
    uint32_t st = 0;
#define RS16_FENCE() __builtin_amdgcn_sched_barrier(0)
    for (uint32_t c = 0; c < NC; c++) {
        const uint32_t stn = st == RSM_STAGES - 1u ? 0u : st + 1u;
#pragma unroll
        for (uint32_t pc = 0; pc < 8u; pc++) {
            const uint32_t cur = pc & 1u, nxt = cur ^ 1u;
            /* four matrix instructions per piece; the other work is spread over the gaps between them */
            RS16_FENCE();
            acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[cur][0], bf[cur][0][0], acc[0], 0, 0, 0);
            RS16_FENCE();
            wait_reads(nxt); /* piece p + 1, requested a piece ago */
            /* piece p + 2 into the raw registers piece p came from (widened a piece ago) */
            if (pc == 6u) {
                /* every piece of chunk c has been read (piece 7 was waited for above): chunk c + 1 must have
                 * landed before its first piece is read, and chunk c's stage takes chunk c + 3 */
                if (c + 2u < NC) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NLD) : "memory");
                else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                read_piece(stn, 0u, cur); /* past the last chunk: stale bytes, never used */
            } else if (pc == 7u) {
                read_piece(stn, 1u, cur);
            } else {
                read_piece(st, pc + 2u, cur);
            }
            RS16_FENCE();
#pragma unroll
            for (int b = 1; b < NB; b++) acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[cur][0], bf[cur][b][0], acc[b], 0, 0, 0);
            RS16_FENCE();
            widen_x(nxt);
            widen_w(nxt, 0);
            RS16_FENCE();
            acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[cur][1], bf[cur][0][1], acc[0], 0, 0, 0);
            RS16_FENCE();
#pragma unroll
            for (int b = 1; b < NB; b++) widen_w(nxt, b);
            RS16_FENCE();
#pragma unroll
            for (int b = 1; b < NB; b++) acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[cur][1], bf[cur][b][1], acc[b], 0, 0, 0);
            RS16_FENCE();
            if (pc == 6u && c + 3u < NC) issue(c + 3u);
            if (pc == 7u) wait_reads(cur); /* nothing in flight across the back edge */
        }
        st = stn;
    }
#undef RS16_FENCE
    /* acc[b][r] = out[m0 + 4 * (lane / 16) + r][n0 + 16 b + lane % 16] */
#pragma unroll
    for (int b = 0; b < NB; b++) {
        const uint32_t n = n0 + 16u * (uint32_t)b + (lane & 15u);
#pragma unroll
        for (uint32_t r = 0; r < 4u; r++) {
            const uint32_t m = m0 + 4u * (lane >> 4) + r;
            if (m < M && n < N) out[(size_t)m * N + n] = acc[b][r];
        }
    }
}

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

/* The 16 x 32 form as it runs by default: like k_router_score_mfma_shared, operands widened by the LDS read
 * (no vector instruction next to the matrix instructions) and operand rows shared by the workgroup. Four waves
 * stacked over 64 tokens share one block of 32 experts: a stage holds 64 + 32 rows (12 KB), a wave loads a
 * quarter of it (16 token rows, 8 expert rows). A piece is only four short matrix instructions, so the reads run
 * two pieces ahead into four sets of operand registers (set = piece % 4: the same in every chunk). The barrier of
 * chunk c sits in its seventh piece, before the first read of chunk c + 1: every wave has then landed its loads
 * of chunk c + 1 and its reads of chunk c - 1, whose stage takes chunk c + 3 (four stages, 48 KB). */
#define RS16S_STAGES 4u
struct Rs16sStage {
    uint8_t x[64u * 128u];
    uint8_t w[32u * 128u];
};
static_assert(sizeof(Rs16sStage) == 12288u, "the stage size is an immediate of the LDS reads below");
/* six 2-byte reads of a piece: k = ks and 4 + ks (the lane's address holds 2 ks) of the lane's token row and of
 * its expert row in both 16-row blocks */
template <uint32_t STG>
__device__ __forceinline__ void rs16s_read(float (&a)[2], float (&b)[2][2], uint32_t ax, uint32_t aw) {
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
__device__ __forceinline__ void rs16s_wait_older(float (&a)[2], float (&b)[2][2]) {
    asm volatile("s_waitcnt lgkmcnt(6)" : "+v"(a[0]), "+v"(a[1]), "+v"(b[0][0]), "+v"(b[0][1]), "+v"(b[1][0]), "+v"(b[1][1]));
}
__global__ __launch_bounds__(256) void k_router_score_mfma16_shared(float* __restrict__ out, const bf16_t* __restrict__ x,
                                                                    const bf16_t* __restrict__ w, uint32_t M, uint32_t N,
                                                                    uint32_t K) {
    extern __shared__ __attribute__((aligned(16))) uint8_t rs16s_raw[];
    constexpr uint32_t ST = RS16S_STAGES, NLD = 3u; /* direct loads per wave and chunk */
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wv = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    Rs16sStage* const ring = (Rs16sStage*)rs16s_raw;
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
        Rs16sStage* s = &ring[stage];
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
    rs16s_read<0u>(af[0], bf[0], ax[0], aw[0]);
    rs16s_read<0u>(af[1], bf[1], ax[1], aw[1]);
    rs16s_wait_older(af[0], bf[0]);
#define RS16_FENCE() __builtin_amdgcn_sched_barrier(0)
    auto chunk = [&](auto stg_, uint32_t c) {
        constexpr uint32_t STG = decltype(stg_)::value, STN = (STG + 1u) % ST, STF = (STG + 3u) % ST;
#pragma unroll
        for (uint32_t pc = 0; pc < 8u; pc++) {
            const uint32_t cur = pc & 3u, n1 = (pc + 1u) & 3u, n2 = (pc + 2u) & 3u;
            RS16_FENCE();
            acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[cur][0], bf[cur][0][0], acc[0], 0, 0, 0);
            RS16_FENCE();
            if (pc == 6u) {
                /* this wave's loads of chunk c + 1 have landed and so have its reads of chunk c - 1 (its last piece was
                 * waited for seven pieces ago): behind the barrier that holds for every wave */
                if (c + 2u < NC) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NLD) : "memory");
                else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                asm volatile("s_barrier" ::: "memory");
            }
            /* piece p + 2 into the set piece p - 2 used; past the last chunk: stale bytes, never used */
            if (pc < 6u) rs16s_read<STG>(af[n2], bf[n2], ax[(pc + 2u) & 7u], aw[(pc + 2u) & 7u]);
            else rs16s_read<STN>(af[n2], bf[n2], ax[(pc + 2u) & 7u], aw[(pc + 2u) & 7u]);
            RS16_FENCE();
            acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[cur][0], bf[cur][1][0], acc[1], 0, 0, 0);
            RS16_FENCE();
            if (pc == 6u && c + 3u < NC) issue(c + 3u, STF); /* into the stage chunk c - 1 has left */
            RS16_FENCE();
            acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[cur][1], bf[cur][0][1], acc[0], 0, 0, 0);
            RS16_FENCE();
            acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[cur][1], bf[cur][1][1], acc[1], 0, 0, 0);
            RS16_FENCE();
            rs16s_wait_older(af[n1], bf[n1]); /* piece p + 1 */
        }
    };
    for (uint32_t c = 0; c < NC; c += 4u) {
        chunk(std::integral_constant<uint32_t, 0u>{}, c);
        if (c + 1u < NC) chunk(std::integral_constant<uint32_t, 1u>{}, c + 1u);
        if (c + 2u < NC) chunk(std::integral_constant<uint32_t, 2u>{}, c + 2u);
        if (c + 3u < NC) chunk(std::integral_constant<uint32_t, 3u>{}, c + 3u);
    }
#undef RS16_FENCE
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

#define RS16_LDS (4u * RSM_STAGES * (uint32_t)sizeof(Rs16Stage))
#define RSM_LDS (4u * RSM_STAGES * (uint32_t)sizeof(RsmStage))
#define RSM_LDS8 (8u * 2u * (uint32_t)sizeof(RsmStage))
#define RSS_LDS (RSM_STAGES * (uint32_t)sizeof(RssStage))
#define RS16S_LDS (RS16S_STAGES * (uint32_t)sizeof(Rs16sStage))

/* dynamic-LDS limits of the score kernels, once per device (plow_moe_device_setup) */
static bool rf_setup();
int plow_moe_route_setup() {
    const bool ok = rf_setup() &&
        hipFuncSetAttribute((const void*)k_router_score_mfma16, hipFuncAttributeMaxDynamicSharedMemorySize, (int)RS16_LDS) == hipSuccess &&
        hipFuncSetAttribute((const void*)k_router_score_mfma<4u, 3u>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)RSM_LDS) == hipSuccess &&
        hipFuncSetAttribute((const void*)k_router_score_mfma<8u, 2u>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)RSM_LDS8) == hipSuccess &&
        hipFuncSetAttribute((const void*)k_router_score_row<1>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)RSR_LDS) == hipSuccess &&
        hipFuncSetAttribute((const void*)k_router_score_row<2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)RSR_LDS) == hipSuccess &&
        hipFuncSetAttribute((const void*)k_router_score_row<4>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)RSR_LDS) == hipSuccess;
    return ok ? 0 : PLOW_MOE_EDEVICE;
}

int launch_router_score(float* out, const void* x, const void* w, uint32_t M, uint32_t N, uint32_t K,
                        hipStream_t st) {
    if (K % 8u) return PLOW_MOE_EINVAL;
    /* 32 x 32 tiles (fewer operand bytes per output) when they fill the SIMDs evenly: a whole number of
     * tiles per SIMD, or at least four; otherwise, from 2^17 outputs, the 16 x 32 tiles */
    const uint64_t t32 = (uint64_t)((N + 31) / 32) * ((M + 31) / 32);
    const PlowMoeTuning& tune = plow_moe_tuning();
    const uint64_t n_cu = plow_moe_n_cu();
    if (!n_cu) return PLOW_MOE_EDEVICE;
    const uint64_t n_simd = 4u * n_cu;
    const uint64_t outputs = (uint64_t)M * N, force32 = tune.score_mfma32_from;
    const bool mfma_ok = K % 64u == 0u && !tune.score_valu;
    const bool use32 = mfma_ok && outputs >= (1u << 18) && (force32 ? outputs >= force32 : (t32 % n_simd == 0u || t32 >= 4u * n_simd));
    const bool use16 = mfma_ok && !use32 && outputs >= (1u << 17);
    if (use16 && !tune.score_private) {
        const uint32_t g = ((N + 31) / 32) * ((M + 63) / 64);
        k_router_score_mfma16_shared<<<g, 256, RS16S_LDS, st>>>(out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
    } else if (use16) {
        const uint32_t lds = RS16_LDS;
        const uint32_t waves = ((N + 16u * RS16_NB - 1u) / (16u * RS16_NB)) * ((M + 15u) / 16u);
        k_router_score_mfma16<<<(waves + 3u) / 4u, 256, lds, st>>>(out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
    } else if (use32) {
        /* two waves per SIMD when the tiles fill both slots of every SIMD a whole number of times (DeepSeek-V3
         * router at 8192 tokens 360 -> 330 us, at 16384 655 -> 591; at 4096, one tile per SIMD, it would leave half
         * the SIMDs idle: 174 -> 298) */
        if (!tune.score_private) {
            const uint32_t g = ((N + 63) / 64) * ((M + 63) / 64);
            k_router_score_mfma_shared<<<g, 256, RSS_LDS, st>>>(out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
            return 0;
        }
        if (t32 % (2u * n_simd) == 0u) {
            const uint32_t g = ((N + 63) / 64) * ((M + 127) / 128);
            k_router_score_mfma<8u, 2u><<<g, 512, RSM_LDS8, st>>>(out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
            return 0;
        }
        const uint32_t lds = RSM_LDS;
        const uint32_t g = ((N + 63) / 64) * ((M + 63) / 64);
        k_router_score_mfma<4u, 3u><<<g, 256, lds, st>>>(out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
    } else if ((uint64_t)M * N >= (1u << 19)) {
        if ((uint64_t)((N + 63) / 64) * ((M + 63) / 64) < 2u * n_cu) { /* fewer than two 64-row workgroups per CU */
            dim3 g((N + 63) / 64, (M + 31) / 32);
            k_router_score_tile<2><<<g, 256, 0, st>>>(out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
        } else {
            dim3 g((N + 63) / 64, (M + 63) / 64);
            k_router_score_tile<4><<<g, 256, 0, st>>>(out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
        }
    } else if (!tune.score_tile8 && K % RSR_KC == 0u && (uint64_t)N * K * 2u < (1ull << 31) && (uint64_t)M * K * 2u < (1ull << 31) &&
               (M < 16u || (uint64_t)M * N <= 2048u)) {
        /* measured against the 8 x 8 tile kernel below: ahead with one or two tokens per workgroup (6 of
         * 38 us at 1 x 384 x 7168) and with four on small score matrices (16 x 64 x 2048: 17 against
         * 25 us); with four tokens on a large one the shared LDS tile is the limit and the two are level */
        /* tokens per workgroup: as many as keep the weight rows' re-reads (once per workgroup row) low */
        const uint32_t lds = RSR_LDS;
        const uint32_t nx = (N + 63) / 64;
        if (M >= 16u) k_router_score_row<4><<<dim3(nx, (M + 3u) / 4u), (4u + RSR_STAGERS) * 64u, lds, st>>>(out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
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
    if (n_exp <= 128u) k_router_topk<2><<<g, b, 0, st>>>(a);
    else if (n_exp <= 256u) k_router_topk<4><<<g, b, 0, st>>>(a);
    else if (n_exp <= 512u) k_router_topk<8><<<g, b, 0, st>>>(a);
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
