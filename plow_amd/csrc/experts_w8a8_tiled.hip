/* experts_w8a8_tiled.hip — the many-rows-per-expert (prefill) form of the block-fp8 x fp8 grouped
 * GEMMs (ops 85 / 86, arm 2 / 3). Same arithmetic as experts_w8a8.hip; different data flow.
 *
 * With hundreds of rows per expert the weights must be reused across rows from on-chip memory, so
 * this is a tiled GEMM: workgroup tile = 128 aligned rows x 128 output channels (GLU: 128 gate + 128
 * up weight rows), 8 waves as 2 (rows) x 4 (channels), each wave 64 rows x 32 channels on
 * v_mfma_f32_32x32x64_f8f6f4 with the weights as the A operand and the rows as the B operand, so
 * that a lane's accumulators belong to ONE row (token): its 1x128 activation scale is one value per
 * lane, and the GLU epilogue's per-row amax is an in-lane reduction plus one shuffle and one LDS hop.
 *
 * The layer is bound by the weight stream, so the loop is built to keep global loads in flight at
 * all times: both operands go global -> LDS directly (global_load_lds_dwordx4, no staging
 * registers) into a ring of three 128-k stages; while stage s is multiplied, stages s+1 and s+2 are
 * in flight. Each wave waits for its own loads of a stage with s_waitcnt vmcnt(n), then an LDS-only
 * barrier publishes the stage. A direct load writes the 64 lanes' 16-byte pieces to consecutive LDS
 * addresses, so rows sit unpadded (128 B) and bank conflicts are avoided by swizzling on the GLOBAL
 * side: LDS piece p of row r holds global piece p ^ ((r >> 1) & 7); the operand reads of 16
 * consecutive rows then cover all 64 banks.
 * Rows of the tile beyond the expert's live rows read some valid row and carry a zero activation
 * scale, so they contribute nothing and are never stored.
 * Per 128-k block: t = two chained matrix instructions (k 0..63, 64..127), then
 * acc = fmaf(t, a_scale[row][kb] * w_scale[nb][kb], acc).
 * Tiles are walked by persistent workgroups (one per CU) in an order that puts the tiles sharing
 * activation rows and weight rows on one XCD at the same time (see the tile loop). */
#include "common.h"
#include "kernels.h"

#define T2_BM 128u
#define T2_BN 128u
#define T2_THREADS 512u
#define T2_STAGES 3u

struct T2Lds {
    uint8_t a[T2_STAGES][T2_BM * 128u]; /* activations, swizzled */
    uint8_t w[T2_STAGES][256u * 128u];  /* weights, swizzled (GLU: rows 0..127 gate, 128..255 up) */
    float as[T2_STAGES][T2_BM];         /* activation scales of the stage's 128-k block */
    float wsc[2][128];                  /* this tile's weight block scales, all of K (gate|down, up) */
    float red[4][T2_BM];                /* GLU: per-row amax of each 32-channel wave column */
    uint32_t scan[T2_THREADS];
    uint32_t prefix[1056];
};

typedef __attribute__((address_space(3))) void lds_void;

/* vmcnt(n) with lgkmcnt / expcnt left open (gfx9 encoding: vmcnt = [3:0] | [15:14]) */
#define WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | (((n) >> 4) << 14))

/* The stage buffers are written by direct global -> LDS loads that the compiler would otherwise
 * fence conservatively (a full s_waitcnt vmcnt(0) before every LDS read and barrier, which would
 * serialise the ring). So the ring is read with explicit ds_read instructions and synchronised with
 * explicit waits: the code below, not the compiler, decides which loads must have landed. */
__device__ __forceinline__ uint32_t lds_off(const void* p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}
__device__ __forceinline__ v4i ds_read16(uint32_t addr) {
    v4i r;
    asm volatile("ds_read_b128 %0, %1" : "=v"(r) : "v"(addr) : "memory");
    return r;
}
__device__ __forceinline__ float ds_read4(uint32_t addr) {
    float r;
    asm volatile("ds_read_b32 %0, %1" : "=v"(r) : "v"(addr) : "memory");
    return r;
}
/* logical 16-byte pieces j, j + 1 of `row` (j even); piece p lives at p ^ ((row >> 1) & 7) */
__device__ __forceinline__ void lds_operand(uint32_t base, uint32_t row, uint32_t j, v4i& lo, v4i& hi) {
    const uint32_t sw = (row >> 1) & 7u;
    lo = ds_read16(base + row * 128u + ((j ^ sw) << 4));
    hi = ds_read16(base + row * 128u + (((j + 1u) ^ sw) << 4));
}
/* all ds_reads issued so far have returned; the operands are tied so nothing is hoisted above */
#define LDS_WAIT4(a, b, c, d) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d))
#define LDS_WAIT2F(a, b) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b))
/* wait until at most n of this wave's loads are outstanding, then the workgroup barrier */
#define STAGE_BARRIER(n) asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(n) : "memory")

#ifdef T2_PROF
__device__ unsigned long long t2_prof[2][256][8];
#define PROF_STAMP(v) const unsigned long long v = __builtin_readcyclecounter()
#else
#define PROF_STAMP(v)
#endif
template <bool GLU>
__global__ __launch_bounds__(T2_THREADS) void k_group_w8a8_tiled(GroupW8A8 g) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    T2Lds& L = *(T2Lds*)lds_raw;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wv = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t NT = g.N / T2_BN;
    constexpr uint32_t WG_PER_WAVE = GLU ? 4u : 2u; /* 8-row weight groups each wave loads per stage */
    constexpr uint32_t NLOAD = 3u + WG_PER_WAVE;    /* direct loads per wave and stage: 2 row groups of
                                                     * activations, the weight groups, 64 scales */

    /* ---- tile directory: inclusive prefix of ceil(cnt / 128) over experts, in LDS ---- */
    {
        uint32_t carry = 0;
        for (uint32_t e0 = 0; e0 < g.E; e0 += T2_THREADS) {
            const uint32_t e = e0 + tid;
            const uint32_t t = e < g.E ? ((uint32_t)g.meta[g.E + e] + T2_BM - 1u) / T2_BM : 0u;
            L.scan[tid] = t;
            __syncthreads();
            for (uint32_t o = 1; o < T2_THREADS; o <<= 1) {
                const uint32_t v = tid >= o ? L.scan[tid - o] : 0u;
                __syncthreads();
                L.scan[tid] += v;
                __syncthreads();
            }
            if (e < g.E) L.prefix[e] = carry + L.scan[tid];
            carry += L.scan[T2_THREADS - 1u];
            __syncthreads();
        }
    }
#ifdef T2_PROF
    unsigned long long pf_setup = 0, pf_ramp = 0, pf_loop = 0, pf_epi = 0, pf_tiles = 0;
    const unsigned long long pf_begin = __builtin_readcyclecounter();
#endif
    const uint32_t total = L.prefix[g.E - 1u] * NT;
    const uint32_t K = g.K, KB = K / 128u;
    const uint32_t wr = wv & 1u, wc = wv >> 1, l32 = lane & 31u, lh = lane >> 5;

    /* Workgroup w runs on XCD w % 8 (round-robin dispatch), and each XCD has its own L2. The logical
     * index below makes the 32 workgroups of one XCD take 32 consecutive tiles of every sweep, and the
     * tile order inside an expert is (16-channel-tile chunk, row tile, channel tile in the chunk): those
     * 32 tiles are then two row tiles x 16 channel tiles of one expert, which read the same activation
     * rows and the same weight rows at about the same time and meet in that L2. */
    const uint32_t G = gridDim.x;
    const uint32_t wg = (G % 8u == 0u) ? (blockIdx.x % 8u) * (G / 8u) + blockIdx.x / 8u : blockIdx.x;
    const uint32_t FC = NT / 16u, RC = NT % 16u;
    for (uint32_t tile = wg; tile < total; tile += G) {
        PROF_STAMP(ts0);
        const uint32_t mt_global = tile / NT;
        uint32_t lo = 0, hi = g.E - 1u; /* first expert whose inclusive prefix exceeds mt_global */
        while (lo < hi) {
            const uint32_t mid = (lo + hi) >> 1;
            if (L.prefix[mid] > mt_global) hi = mid; else lo = mid + 1u;
        }
        /* the same value in every lane; made explicit so that everything indexed by the expert (pointer
         * tables, block scales) is read with scalar loads and never waits on the vector-load counter */
        const uint32_t e = (uint32_t)__builtin_amdgcn_readfirstlane((int)lo);
        const uint32_t pbase = e ? L.prefix[e - 1u] : 0u, Me = L.prefix[e] - pbase;
        const uint32_t idx = tile - pbase * NT;
        uint32_t mt_v, nt_v;
        if (idx < FC * Me * 16u) {
            const uint32_t chunk = idx / (Me * 16u), rem = idx % (Me * 16u);
            mt_v = rem / 16u, nt_v = chunk * 16u + rem % 16u;
        } else {
            const uint32_t rem = idx - FC * Me * 16u;
            mt_v = rem / RC, nt_v = FC * 16u + rem % RC;
        }
        const uint32_t mt = (uint32_t)__builtin_amdgcn_readfirstlane((int)mt_v);
        const uint32_t nt = (uint32_t)__builtin_amdgcn_readfirstlane((int)nt_v);
        const uint32_t cnt = (uint32_t)g.meta[g.E + e], r0 = (uint32_t)g.meta[e] + mt * T2_BM;
        const uint32_t rows = cnt - mt * T2_BM < T2_BM ? cnt - mt * T2_BM : T2_BM; /* live rows here */
        const uint64_t wp0 = g.wtab[(size_t)e * 3u + (GLU ? 0u : 2u)];
        if (wp0 == 0ull) continue; /* expert not resident */
        const uint8_t* W0 = (const uint8_t*)(uintptr_t)wp0;
        const uint8_t* W1 = GLU ? (const uint8_t*)(uintptr_t)g.wtab[(size_t)e * 3u + 1u] : nullptr;
        const float* S0 = (const float*)(uintptr_t)g.stab[(size_t)e * 3u + (GLU ? 0u : 2u)] + (size_t)nt * KB;
        const float* S1 = GLU ? (const float*)(uintptr_t)g.stab[(size_t)e * 3u + 1u] + (size_t)nt * KB : nullptr;

        /* ---- loader: a direct load covers 8 rows x 128 B; lane -> (row l>>3, LDS piece l&7) ---- */
        const uint8_t* asrc[2];
        const uint8_t* wsrc[WG_PER_WAVE];
#pragma unroll
        for (uint32_t i = 0; i < 2u; i++) { /* activation rows 16*wv + 8*i + (lane >> 3) */
            const uint32_t row = 16u * wv + 8u * i + (lane >> 3), p = lane & 7u;
            uint32_t src; /* a pad row reads the tile's first row; its scale is zero */
            if (GLU) {
                const uint32_t tok = row < rows ? g.row_token[r0 + row] : PLOW_EXPERT_UNUSED;
                src = tok != PLOW_EXPERT_UNUSED ? tok : g.row_token[r0];
            } else {
                src = r0 + (row < rows ? row : 0u);
            }
            asrc[i] = (const uint8_t*)g.a + (size_t)src * K + ((p ^ ((row >> 1) & 7u)) << 4);
        }
#pragma unroll
        for (uint32_t i = 0; i < WG_PER_WAVE; i++) { /* weight rows 8*(WG_PER_WAVE*wv + i) + (lane >> 3) */
            const uint32_t row = 8u * (WG_PER_WAVE * wv + i) + (lane >> 3), p = lane & 7u;
            const uint8_t* base = (GLU && row >= 128u) ? W1 : W0;
            wsrc[i] = base + (size_t)(nt * T2_BN + (row & 127u)) * K + ((p ^ ((row >> 1) & 7u)) << 4);
        }
        /* activation scale of row (wv & 1) * 64 + lane (every wave pair loads the same 64 values);
         * a pad row reads tilep[0], which is always 0 */
        const float* ssrc;
        uint32_t sstep;
        {
            const uint32_t row = (wv & 1u) * 64u + lane;
            bool ok = row < rows;
            if (GLU) {
                const uint32_t tok = ok ? g.row_token[r0 + row] : PLOW_EXPERT_UNUSED;
                ok = tok != PLOW_EXPERT_UNUSED;
                ssrc = ok ? g.a_scale + tok : (const float*)(g.meta + 2u * g.E);
                sstep = ok ? g.pitch : 0u;
            } else {
                ok = ok && g.row_partidx[r0 + row] != PLOW_EXPERT_UNUSED;
                ssrc = ok ? g.a_scale + (size_t)(r0 + row) * KB : (const float*)(g.meta + 2u * g.E);
                sstep = ok ? 1u : 0u;
            }
        }
        auto issue = [&](uint32_t kb) {
            const uint32_t st = kb % T2_STAGES;
#ifdef T2_NOSTREAM
            kb &= 1u;
#endif
            __builtin_amdgcn_global_load_lds((const void*)(ssrc + (size_t)kb * sstep),
                                             (lds_void*)&L.as[st][(wv & 1u) * 64u], 4, 0, 0);
#pragma unroll
            for (uint32_t i = 0; i < 2u; i++)
                __builtin_amdgcn_global_load_lds((const void*)(asrc[i] + (size_t)kb * 128u),
                                                 (lds_void*)&L.a[st][(16u * wv + 8u * i) * 128u], 16, 0, 0);
#pragma unroll
            for (uint32_t i = 0; i < WG_PER_WAVE; i++)
                __builtin_amdgcn_global_load_lds((const void*)(wsrc[i] + (size_t)kb * 128u),
                                                 (lds_void*)&L.w[st][8u * (WG_PER_WAVE * wv + i) * 128u], 16, 0, 0);
        };

        /* ---- this lane's two B-operand rows ---- */
        bool rvalid[2];
#pragma unroll
        for (int rt = 0; rt < 2; rt++) {
            const uint32_t row = wr * 64u + (uint32_t)rt * 32u + l32;
            rvalid[rt] = row < rows;
            if (GLU) rvalid[rt] = rvalid[rt] && g.row_token[r0 + row] != PLOW_EXPERT_UNUSED;
            else rvalid[rt] = rvalid[rt] && g.row_partidx[r0 + row] != PLOW_EXPERT_UNUSED;
        }
        const bool wave_live = wr * 64u < rows; /* a wave whose rows are all pad does no matrix work */

        v16f acc[2][GLU ? 2 : 1];
#pragma unroll
        for (int rt = 0; rt < 2; rt++)
#pragma unroll
            for (int gu = 0; gu < (GLU ? 2 : 1); gu++)
#pragma unroll
                for (int i = 0; i < 16; i++) acc[rt][gu][i] = 0.0f;

        /* the tile's weight block scales go to LDS once, so that the loop below has no ordinary
         * vector load whose wait would also wait for the ring */
        for (uint32_t i = tid; i < KB; i += T2_THREADS) {
            L.wsc[0][i] = S0[i];
            if (GLU) L.wsc[1][i] = S1[i];
        }
        __syncthreads();
        issue(0);
        if (KB > 1u) issue(1);
        const uint32_t a_base = lds_off(&L.a[0][0]), w_base = lds_off(&L.w[0][0]), s_base = lds_off(&L.as[0][0]);
        const uint32_t c_base = lds_off(&L.wsc[0][0]);
        PROF_STAMP(ts1);
#ifdef T2_PROF
        unsigned long long ts2 = 0;
#endif
        for (uint32_t kb = 0; kb < KB; kb++) {
            const uint32_t st = kb % T2_STAGES;
            /* this wave's loads of stage kb have landed once at most the next stage's are outstanding;
             * after the barrier stage kb is complete and the buffer of stage kb-1 is free */
            if (kb + 1u < KB) STAGE_BARRIER(NLOAD); else STAGE_BARRIER(0);
#ifdef T2_PROF
            if (kb == 0) ts2 = __builtin_readcyclecounter();
#endif
            if (kb + 2u < KB) issue(kb + 2u);
            if (wave_live) {
                float ws0 = ds_read4(c_base + kb * 4u);
                float ws1 = ds_read4(c_base + ((GLU ? 128u : 0u) + kb) * 4u);
                const uint32_t ab = a_base + st * (T2_BM * 128u), wb = w_base + st * (256u * 128u);
                v4i bl[2][2], bh[2][2];
#pragma unroll
                for (int rt = 0; rt < 2; rt++)
#pragma unroll
                    for (int kk = 0; kk < 2; kk++)
                        lds_operand(ab, wr * 64u + (uint32_t)rt * 32u + l32, 4u * kk + 2u * lh, bl[rt][kk], bh[rt][kk]);
                float asv0 = ds_read4(s_base + (st * T2_BM + wr * 64u + l32) * 4u);
                float asv1 = ds_read4(s_base + (st * T2_BM + wr * 64u + 32u + l32) * 4u);
                LDS_WAIT4(bl[0][0], bh[0][0], bl[0][1], bh[0][1]);
                LDS_WAIT4(bl[1][0], bh[1][0], bl[1][1], bh[1][1]);
                LDS_WAIT2F(asv0, asv1);
                LDS_WAIT2F(ws0, ws1);
                const float asv[2] = {asv0, asv1};
                v8i bf[2][2];
#pragma unroll
                for (int rt = 0; rt < 2; rt++)
#pragma unroll
                    for (int kk = 0; kk < 2; kk++)
                        bf[rt][kk] = __builtin_shufflevector(bl[rt][kk], bh[rt][kk], 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
                for (int gu = 0; gu < (GLU ? 2 : 1); gu++) {
                    const uint32_t wrow = (uint32_t)gu * 128u + wc * 32u + l32;
                    v4i a0l, a0h, a1l, a1h;
                    lds_operand(wb, wrow, 2u * lh, a0l, a0h);
                    lds_operand(wb, wrow, 4u + 2u * lh, a1l, a1h);
                    LDS_WAIT4(a0l, a0h, a1l, a1h);
                    const v8i af0 = __builtin_shufflevector(a0l, a0h, 0, 1, 2, 3, 4, 5, 6, 7);
                    const v8i af1 = __builtin_shufflevector(a1l, a1h, 0, 1, 2, 3, 4, 5, 6, 7);
                    const float wsc = gu ? ws1 : ws0;
#pragma unroll
                    for (int rt = 0; rt < 2; rt++) {
                        v16f t;
#pragma unroll
                        for (int i = 0; i < 16; i++) t[i] = 0.0f;
                        t = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af0, bf[rt][0], t, 0, 0, 0, 0, 0, 0);
                        t = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af1, bf[rt][1], t, 0, 0, 0, 0, 0, 0);
                        const float sc = asv[rt] * wsc;
#pragma unroll
                        for (int i = 0; i < 16; i++) acc[rt][gu][i] = fmaf(t[i], sc, acc[rt][gu][i]);
                    }
                }
            }
        }
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory"); /* ring drained */
        PROF_STAMP(ts3);

        /* ---- epilogue. Lane: row = wr*64 + rt*32 + l32; channels wc*32 + 8*(i/4) + 4*lh + (i%4) ---- */
        if (GLU) {
            float v[2][16];
#pragma unroll
            for (int rt = 0; rt < 2; rt++) {
                float m = 0.0f;
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    v[rt][i] = moe_glu(acc[rt][0][i], acc[rt][GLU ? 1 : 0][i], g.act);
                    m = fmaxf(m, fabsf(v[rt][i]));
                }
                m = fmaxf(m, __shfl_xor(m, 32, 64));
                if (lh == 0) L.red[wc][wr * 64u + (uint32_t)rt * 32u + l32] = m;
            }
            lds_barrier();
#pragma unroll
            for (int rt = 0; rt < 2; rt++) {
                const uint32_t row = wr * 64u + (uint32_t)rt * 32u + l32;
                if (!rvalid[rt]) continue;
                const float amax = fmaxf(fmaxf(1e-10f, L.red[0][row]), fmaxf(fmaxf(L.red[1][row], L.red[2][row]), L.red[3][row]));
                const float s = amax * (1.0f / 448.0f), inv = 1.0f / s;
                uint8_t* orow = (uint8_t*)g.out + (size_t)(r0 + row) * g.N + nt * T2_BN + wc * 32u + 4u * lh;
#pragma unroll
                for (int i4 = 0; i4 < 4; i4++)
                    *(uint32_t*)(orow + i4 * 8) = cvt4_e4m3(v[rt][4 * i4] * inv, v[rt][4 * i4 + 1] * inv,
                                                            v[rt][4 * i4 + 2] * inv, v[rt][4 * i4 + 3] * inv);
                if (wc == 0 && lh == 0) g.out_scale[(size_t)(r0 + row) * NT + nt] = s;
            }
        } else {
#pragma unroll
            for (int rt = 0; rt < 2; rt++) {
                const uint32_t row = wr * 64u + (uint32_t)rt * 32u + l32;
                if (!rvalid[rt]) continue;
                const uint32_t pidx = g.row_partidx[r0 + row];
                const float gate = g.row_gate[r0 + row];
                const size_t ocol = (size_t)pidx * g.N + nt * T2_BN + wc * 32u + 4u * lh;
#pragma unroll
                for (int i4 = 0; i4 < 4; i4++) {
                    const float y0 = gate * acc[rt][0][4 * i4], y1 = gate * acc[rt][0][4 * i4 + 1];
                    const float y2 = gate * acc[rt][0][4 * i4 + 2], y3 = gate * acc[rt][0][4 * i4 + 3];
                    if (g.part16) {
                        uint2 o;
                        o.x = (uint32_t)f2bf(y0) | ((uint32_t)f2bf(y1) << 16);
                        o.y = (uint32_t)f2bf(y2) | ((uint32_t)f2bf(y3) << 16);
                        *(uint2*)((bf16_t*)g.out + ocol + i4 * 8) = o;
                    } else {
                        *(float4*)((float*)g.out + ocol + i4 * 8) = make_float4(y0, y1, y2, y3);
                    }
                }
            }
        }
        lds_barrier(); /* every wave is done with the ring and with L.red before the next tile refills them */
#ifdef T2_PROF
        {
            const unsigned long long ts4 = __builtin_readcyclecounter();
            pf_setup += ts1 - ts0, pf_ramp += ts2 - ts1, pf_loop += ts3 - ts2, pf_epi += ts4 - ts3, pf_tiles++;
        }
#endif
    }
#ifdef T2_PROF
    if (tid == 0 && blockIdx.x < 256u) {
        unsigned long long* o = t2_prof[GLU][blockIdx.x];
        o[0] = pf_setup, o[1] = pf_ramp, o[2] = pf_loop, o[3] = pf_epi, o[4] = pf_tiles;
        o[5] = __builtin_readcyclecounter() - pf_begin;
    }
#endif
}
#ifdef T2_PROF
extern "C" int plow_moe_debug_prof(unsigned long long* out) {
    return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(t2_prof), sizeof(t2_prof));
}
#endif

/* Persistent launch: one workgroup per CU; the tile count is computed on the device from meta. */
template <bool GLU>
static int launch_tiled(const GroupW8A8& g, hipStream_t st) {
    if (g.N == 0 || g.K == 0 || g.E == 0 || g.E > 1056u || g.N % T2_BN || g.K % 128u) return PLOW_MOE_EINVAL;
    if (g.K > 128u * 128u) return PLOW_MOE_EINVAL; /* the tile keeps K / 128 block scales in LDS */
    static bool attr_set[2] = {false, false};
    static int n_cu = 0;
    if (!attr_set[GLU]) {
        if (hipFuncSetAttribute((const void*)k_group_w8a8_tiled<GLU>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)sizeof(T2Lds)) != hipSuccess)
            return PLOW_MOE_EDEVICE;
        attr_set[GLU] = true;
    }
    if (!n_cu) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return PLOW_MOE_EDEVICE;
        n_cu = prop.multiProcessorCount;
    }
    k_group_w8a8_tiled<GLU><<<(uint32_t)n_cu, T2_THREADS, sizeof(T2Lds), st>>>(g);
    return 0;
}

int launch_group_glu_w8a8_tiled(const GroupW8A8& g, hipStream_t st) { return launch_tiled<true>(g, st); }
int launch_group_down_w8a8_tiled(const GroupW8A8& g, hipStream_t st) { return launch_tiled<false>(g, st); }
