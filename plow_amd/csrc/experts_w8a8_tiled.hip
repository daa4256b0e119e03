/* experts_w8a8_tiled.hip — the many-rows-per-expert (prefill) form of the block-fp8 x fp8 grouped
 * GEMMs (ops 85 / 86, arm 2 / 3). Same arithmetic as experts_w8a8.hip; different data flow.
 *
 * With hundreds of rows per expert the weights must be reused across rows from on-chip memory, so
 * this is a classic tiled GEMM: workgroup tile = 256 aligned rows x 128 output channels (GLU: 128
 * gate + 128 up weight rows), 8 waves as 4 (rows) x 2 (channels), each wave 64 rows x 64 channels
 * on v_mfma_f32_32x32x64_f8f6f4 with the weights as the A operand and the rows as the B operand, so
 * that a lane's accumulators belong to ONE row (token): its 1x128 activation scale is one value per
 * lane, and the GLU epilogue's per-row amax is an in-lane reduction plus one shuffle and one LDS hop.
 * Both operands go through LDS, one 128-k block per step, double buffered: the global loads of step
 * s + 1 are issued before the matrix work of step s and stored to the other buffer after it, with
 * one LDS-only barrier per step. LDS rows are padded to 144 bytes so that the 16-byte operand reads
 * of 16 consecutive rows fall on 64 distinct banks.
 * Per 128-k block: t = two chained matrix instructions (k 0..63, 64..127), then
 * acc = fmaf(t, a_scale[row][kb] * w_scale[nb][kb], acc).
 * Tiles are enumerated (expert, 256-row tile, channel tile) with the channel tile fastest: the
 * tiles that share an expert's weight rows are a multiple of 8 workgroups apart, which the hardware
 * dispatch order places on the same XCD (same L2). */
#include "common.h"
#include "kernels.h"

#define TL_BM 256u
#define TL_BN 128u
#define TL_THREADS 512u
#define TL_LD 144u /* bytes per LDS row (128 payload + 16 pad) */

template <bool GLU> struct TileCfg {
    static constexpr uint32_t WROWS = GLU ? 256u : 128u; /* weight rows per step */
    static constexpr uint32_t WPT = WROWS * 8u / TL_THREADS; /* 16-byte weight pieces per thread */
};

struct TileLds {
    uint8_t a[2][TL_BM * TL_LD];  /* activations */
    uint8_t w[2][256u * TL_LD];   /* weights */
    float as[2][TL_BM];           /* activation scales of the step */
    float red[2][TL_BM];          /* GLU: per-row amax of each channel half */
    uint32_t scan[TL_THREADS];
    uint32_t prefix[1056];
};

template <bool GLU>
__global__ __launch_bounds__(TL_THREADS) void k_group_w8a8_tiled(GroupW8A8 g) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    TileLds& L = *(TileLds*)lds_raw;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wv = tid >> 6;
    const uint32_t NT = g.N / TL_BN;

    /* ---- tile directory: inclusive prefix of ceil(cnt / 256) over experts, in LDS ---- */
    {
        uint32_t carry = 0;
        for (uint32_t e0 = 0; e0 < g.E; e0 += TL_THREADS) {
            const uint32_t e = e0 + tid;
            const uint32_t t = e < g.E ? ((uint32_t)g.meta[g.E + e] + TL_BM - 1u) / TL_BM : 0u;
            L.scan[tid] = t;
            __syncthreads();
            for (uint32_t o = 1; o < TL_THREADS; o <<= 1) {
                const uint32_t v = tid >= o ? L.scan[tid - o] : 0u;
                __syncthreads();
                L.scan[tid] += v;
                __syncthreads();
            }
            if (e < g.E) L.prefix[e] = carry + L.scan[tid];
            carry += L.scan[TL_THREADS - 1u];
            __syncthreads();
        }
    }
    const uint32_t total = L.prefix[g.E - 1u] * NT;
    /* persistent workgroups: tile t = (256-row tile, channel tile), channel tile fastest */
    for (uint32_t tile = blockIdx.x; tile < total; tile += gridDim.x) {
    const uint32_t nt = tile % NT, mt_global = tile / NT;
    uint32_t lo = 0, hi = g.E - 1u; /* first expert whose inclusive prefix exceeds mt_global */
    while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (L.prefix[mid] > mt_global) hi = mid; else lo = mid + 1u;
    }
    const uint32_t e = lo;
    const uint32_t mt = mt_global - (e ? L.prefix[e - 1u] : 0u);
    const uint32_t cnt = (uint32_t)g.meta[g.E + e], r0 = (uint32_t)g.meta[e] + mt * TL_BM;
    const uint32_t rows = cnt - mt * TL_BM < TL_BM ? cnt - mt * TL_BM : TL_BM; /* live rows of this tile */
    const uint64_t wp0 = g.wtab[(size_t)e * 3u + (GLU ? 0u : 2u)];
    if (wp0 == 0ull) continue; /* expert not resident */
    const uint32_t K = g.K, KB = K / 128u;
    const uint8_t* W0 = (const uint8_t*)(uintptr_t)wp0;
    const uint8_t* W1 = GLU ? (const uint8_t*)(uintptr_t)g.wtab[(size_t)e * 3u + 1u] : nullptr;
    const float* S0 = (const float*)(uintptr_t)g.stab[(size_t)e * 3u + (GLU ? 0u : 2u)] + (size_t)nt * KB;
    const float* S1 = GLU ? (const float*)(uintptr_t)g.stab[(size_t)e * 3u + 1u] + (size_t)nt * KB : nullptr;

    /* ---- staging assignment: piece p = tid + 512 i -> (row p >> 3, 16-byte piece p & 7) ---- */
    constexpr uint32_t WPT = TileCfg<GLU>::WPT;
    const uint32_t pc = tid & 7u;
    const uint8_t* arow[4];
    bool aval[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t row = (tid >> 3) + 64u * i;
        aval[i] = row < rows;
        uint32_t src = 0;
        if (GLU) {
            src = aval[i] ? g.row_token[r0 + row] : PLOW_EXPERT_UNUSED;
            aval[i] = src != PLOW_EXPERT_UNUSED;
        } else {
            aval[i] = aval[i] && g.row_partidx[r0 + row] != PLOW_EXPERT_UNUSED;
            src = r0 + row;
        }
        arow[i] = (const uint8_t*)g.a + (size_t)(aval[i] ? src : 0u) * K + pc * 16u;
    }
    const uint8_t* wrow[WPT];
#pragma unroll
    for (uint32_t i = 0; i < WPT; i++) {
        const uint32_t row = (tid >> 3) + 64u * i; /* GLU: 0..127 gate, 128..255 up */
        const uint8_t* base = (GLU && row >= 128u) ? W1 : W0;
        wrow[i] = base + (size_t)(nt * TL_BN + (row & 127u)) * K + pc * 16u;
    }
    /* activation scale of row `tid` (threads 0..255) */
    const float* asrc = nullptr;
    uint32_t as_stride = 0;
    if (tid < TL_BM) {
        bool ok = tid < rows;
        if (GLU) {
            const uint32_t tok = ok ? g.row_token[r0 + tid] : PLOW_EXPERT_UNUSED;
            ok = tok != PLOW_EXPERT_UNUSED;
            asrc = ok ? g.a_scale + tok : nullptr;
            as_stride = g.pitch;
        } else {
            asrc = ok ? g.a_scale + (size_t)(r0 + tid) * KB : nullptr;
            as_stride = 1u;
        }
    }

    v4i sa[4], sw[WPT];
    float sas = 0.0f;
    auto fetch = [&](uint32_t kb) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            sa[i] = (v4i){0, 0, 0, 0};
            if (aval[i]) sa[i] = *(const v4i*)(arow[i] + (size_t)kb * 128u);
        }
#pragma unroll
        for (uint32_t i = 0; i < WPT; i++) sw[i] = *(const v4i*)(wrow[i] + (size_t)kb * 128u);
        sas = asrc ? asrc[(size_t)kb * as_stride] : 0.0f;
    };
    auto commit = [&](uint32_t buf) {
#pragma unroll
        for (int i = 0; i < 4; i++)
            *(v4i*)&L.a[buf][((tid >> 3) + 64u * i) * TL_LD + pc * 16u] = sa[i];
#pragma unroll
        for (uint32_t i = 0; i < WPT; i++)
            *(v4i*)&L.w[buf][((tid >> 3) + 64u * i) * TL_LD + pc * 16u] = sw[i];
        if (tid < TL_BM) L.as[buf][tid] = sas;
    };

    /* ---- wave tile: 64 rows x 64 channels ---- */
    const uint32_t wr = wv & 3u, wc = wv >> 2, l32 = lane & 31u, lh = lane >> 5;
    const bool wave_live = wr * 64u < rows; /* a wave whose rows are all pad does no matrix work */
    v16f acc[2][2][GLU ? 2 : 1];
#pragma unroll
    for (int rt = 0; rt < 2; rt++)
#pragma unroll
        for (int ct = 0; ct < 2; ct++)
#pragma unroll
            for (int gu = 0; gu < (GLU ? 2 : 1); gu++)
#pragma unroll
                for (int i = 0; i < 16; i++) acc[rt][ct][gu][i] = 0.0f;

    fetch(0);
    commit(0);
    lds_barrier();
    for (uint32_t kb = 0; kb < KB; kb++) {
        const uint32_t buf = kb & 1u;
        if (kb + 1u < KB) fetch(kb + 1u);
        if (wave_live) {
            const float ws0 = S0[kb];
            const float ws1 = GLU ? S1[kb] : 0.0f;
            /* B operand fragments (rows), both k halves, both row tiles */
            v8i bf[2][2];
            float asv[2];
#pragma unroll
            for (int rt = 0; rt < 2; rt++) {
                const uint32_t row = wr * 64u + (uint32_t)rt * 32u + l32;
                asv[rt] = L.as[buf][row];
#pragma unroll
                for (int kk = 0; kk < 2; kk++) {
                    const uint8_t* p = &L.a[buf][row * TL_LD + (uint32_t)kk * 64u + lh * 32u];
                    const v4i lo = *(const v4i*)p, hi = *(const v4i*)(p + 16);
                    bf[rt][kk] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                }
            }
#pragma unroll
            for (int ct = 0; ct < 2; ct++)
#pragma unroll
                for (int gu = 0; gu < (GLU ? 2 : 1); gu++) {
                    const uint32_t wrw = (uint32_t)gu * 128u + wc * 64u + (uint32_t)ct * 32u + l32;
                    v8i af[2];
#pragma unroll
                    for (int kk = 0; kk < 2; kk++) {
                        const uint8_t* p = &L.w[buf][wrw * TL_LD + (uint32_t)kk * 64u + lh * 32u];
                        const v4i lo = *(const v4i*)p, hi = *(const v4i*)(p + 16);
                        af[kk] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                    }
                    const float wsc = gu ? ws1 : ws0;
#pragma unroll
                    for (int rt = 0; rt < 2; rt++) {
                        v16f t;
#pragma unroll
                        for (int i = 0; i < 16; i++) t[i] = 0.0f;
                        t = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af[0], bf[rt][0], t, 0, 0, 0, 0, 0, 0);
                        t = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af[1], bf[rt][1], t, 0, 0, 0, 0, 0, 0);
                        const float sc = asv[rt] * wsc;
#pragma unroll
                        for (int i = 0; i < 16; i++) acc[rt][ct][gu][i] = fmaf(t[i], sc, acc[rt][ct][gu][i]);
                    }
                }
        }
        if (kb + 1u < KB) commit(buf ^ 1u);
        lds_barrier();
    }

    /* ---- epilogue. Lane: row (token) = wr*64 + rt*32 + l32; channels wc*64 + ct*32 + 8*(i/4) +
     * 4*lh + (i%4), i = 0..15 ---- */
    if (GLU) {
        float v[2][2][16];
#pragma unroll
        for (int rt = 0; rt < 2; rt++) {
            float m = 0.0f;
#pragma unroll
            for (int ct = 0; ct < 2; ct++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    v[rt][ct][i] = moe_glu(acc[rt][ct][0][i], acc[rt][ct][GLU ? 1 : 0][i], g.act);
                    m = fmaxf(m, fabsf(v[rt][ct][i]));
                }
            m = fmaxf(m, __shfl_xor(m, 32, 64));
            if (lh == 0) L.red[wc][wr * 64u + (uint32_t)rt * 32u + l32] = m;
        }
        lds_barrier();
#pragma unroll
        for (int rt = 0; rt < 2; rt++) {
            const uint32_t row = wr * 64u + (uint32_t)rt * 32u + l32;
            if (row >= rows) continue;
            const float amax = fmaxf(1e-10f, fmaxf(L.red[0][row], L.red[1][row]));
            const float s = amax * (1.0f / 448.0f), inv = 1.0f / s;
            uint8_t* orow = (uint8_t*)g.out + (size_t)(r0 + row) * g.N + nt * TL_BN + wc * 64u + 4u * lh;
#pragma unroll
            for (int ct = 0; ct < 2; ct++)
#pragma unroll
                for (int i4 = 0; i4 < 4; i4++)
                    *(uint32_t*)(orow + ct * 32 + i4 * 8) =
                        cvt4_e4m3(v[rt][ct][4 * i4] * inv, v[rt][ct][4 * i4 + 1] * inv,
                                  v[rt][ct][4 * i4 + 2] * inv, v[rt][ct][4 * i4 + 3] * inv);
            if (wc == 0 && lh == 0) g.out_scale[(size_t)(r0 + row) * NT + nt] = s;
        }
    } else {
#pragma unroll
        for (int rt = 0; rt < 2; rt++) {
            const uint32_t row = wr * 64u + (uint32_t)rt * 32u + l32;
            if (row >= rows) continue;
            const uint32_t pidx = g.row_partidx[r0 + row];
            if (pidx == PLOW_EXPERT_UNUSED) continue;
            const float gate = g.row_gate[r0 + row];
            const size_t ocol = (size_t)pidx * g.N + nt * TL_BN + wc * 64u + 4u * lh;
#pragma unroll
            for (int ct = 0; ct < 2; ct++)
#pragma unroll
                for (int i4 = 0; i4 < 4; i4++) {
                    const float y0 = gate * acc[rt][ct][0][4 * i4], y1 = gate * acc[rt][ct][0][4 * i4 + 1];
                    const float y2 = gate * acc[rt][ct][0][4 * i4 + 2], y3 = gate * acc[rt][ct][0][4 * i4 + 3];
                    if (g.part16) {
                        uint2 o;
                        o.x = (uint32_t)f2bf(y0) | ((uint32_t)f2bf(y1) << 16);
                        o.y = (uint32_t)f2bf(y2) | ((uint32_t)f2bf(y3) << 16);
                        *(uint2*)((bf16_t*)g.out + ocol + ct * 32 + i4 * 8) = o;
                    } else {
                        *(float4*)((float*)g.out + ocol + ct * 32 + i4 * 8) = make_float4(y0, y1, y2, y3);
                    }
                }
        }
    }
    lds_barrier(); /* the next tile reuses the LDS buffers */
    } /* tile loop */
}

/* Persistent launch: one workgroup per CU; the tile count is computed on the device from meta. */
template <bool GLU>
static int launch_tiled(const GroupW8A8& g, hipStream_t st) {
    if (g.N == 0 || g.K == 0 || g.E == 0 || g.E > 1056u || g.N % TL_BN || g.K % 128u) return PLOW_MOE_EINVAL;
    static bool attr_set[2] = {false, false};
    static int n_cu = 0;
    if (!attr_set[GLU]) {
        if (hipFuncSetAttribute((const void*)k_group_w8a8_tiled<GLU>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)sizeof(TileLds)) != hipSuccess)
            return PLOW_MOE_EDEVICE;
        attr_set[GLU] = true;
    }
    if (!n_cu) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return PLOW_MOE_EDEVICE;
        n_cu = prop.multiProcessorCount;
    }
    k_group_w8a8_tiled<GLU><<<(uint32_t)n_cu, TL_THREADS, sizeof(TileLds), st>>>(g);
    return 0;
}

int launch_group_glu_w8a8_tiled(const GroupW8A8& g, hipStream_t st) { return launch_tiled<true>(g, st); }
int launch_group_down_w8a8_tiled(const GroupW8A8& g, hipStream_t st) { return launch_tiled<false>(g, st); }
