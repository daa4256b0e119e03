/* experts_gemv.hip — the bf16-activation expert ops (85 / 86 arms 0 and 8, 48 / 49, 65 / 66, 75 / 76) when
 * the batch routes few rows in all (decode at a few tokens).
 *
 * With one row per expert the matrix unit has nothing to amortise: the op is a set of matrix-vector
 * products, bound by how many weight bytes the chip keeps in flight. The tile kernels give a workgroup
 * 128 channels of one expert and a three-step ring, which at nine experts leaves half the CUs idle and
 * the others latency bound. Here every live row gets an equal share of all the waves on the chip; a wave
 * keeps its row of activations in registers and walks its range of output channels, one weight row (two
 * for the GLU) per step: every lane loads 16 bytes of the row per 1 KB piece, decodes them to bf16 exactly
 * as the tile kernels do and multiplies with v_dot2c_f32_bf16; the next channel's loads are issued before
 * this channel's arithmetic, and the lanes' partial sums meet in a wave reduction. The order of the
 * additions differs from the tile kernels' (results agree to rounding, not to the bit). An expert with
 * several rows streams its weights once per row: the form is chosen only for batches of a few rows. */
#include "common.h"
#include "kernels.h"
#include "pm_expf.h"
#include "tuning.h"

enum { GV_BF16 = 0, GV_FP8BLK = 1, GV_MXFP4 = 2, GV_FP8PC = 3 };
#define GV_WAVES 4u
#define GV_WINDOW 256u /* live rows handled per pass (the form is chosen for fewer) */
#define GV_QUADS_FROM 32u /* rows from which a workgroup's waves take neighbouring rows */
#define GV_MAX_E 1088u
#define GV_ECHUNKS (GV_MAX_E / WAVE)
/* A pointer made from a table word is generic to the compiler, which then emits flat loads (they count on
 * both memory counters); this says what it is: global memory. */
typedef const __attribute__((address_space(1))) uint8_t* gv_gptr;

/* k values a lane's 16 bytes of a weight row hold, and the 16-byte pieces of its activation slice */
template <int ENC> struct GvGeom;
template <> struct GvGeom<GV_BF16> { static constexpr uint32_t KL = 8u, XQ = 1u; };
template <> struct GvGeom<GV_FP8BLK> { static constexpr uint32_t KL = 16u, XQ = 2u; };
template <> struct GvGeom<GV_FP8PC> { static constexpr uint32_t KL = 16u, XQ = 2u; };
template <> struct GvGeom<GV_MXFP4> { static constexpr uint32_t KL = 32u, XQ = 4u; };

__device__ __forceinline__ float gv_dot2(uint32_t w2, uint32_t x2, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2bf, w2), __builtin_bit_cast(v2bf, x2), acc, false);
}
/* sum over the wave, in every lane: four steps inside each row of 16 lanes, then the four rows */
__device__ __forceinline__ float gv_wave_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, false));  /* quad_perm 1,0,3,2 */
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, false));  /* quad_perm 2,3,0,1 */
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, false)); /* row_half_mirror */
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, false)); /* row_mirror */
    const float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    const float b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
    const float c = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    const float d = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
    return (a + b) + (c + d);
}

/* one weight row's share of a lane: ITER pieces of 16 bytes (zero past the row's end) and their scales */
template <int ENC, int ITER>
struct GvRow {
    v4i w[ITER];
    uint32_t sb[ITER]; /* mxfp4: the E8M0 byte of the piece's 32 values */
    float sf[ITER];    /* block-fp8: the block scale of the piece's 16 values */
};

template <int ENC, int ITER>
__device__ __forceinline__ void gv_load(GvRow<ENC, ITER>& r, const uint8_t* wrow, const uint8_t* srow, uint32_t lane,
                                        uint32_t pieces) {
#pragma unroll
    for (int it = 0; it < ITER; it++) {
        const uint32_t p = (uint32_t)it * 64u + lane; /* the lane's 16-byte piece of the row */
        const bool in = p < pieces;
        r.w[it] = in ? __builtin_nontemporal_load((const __attribute__((address_space(1))) v4i*)((gv_gptr)wrow + (size_t)p * 16u)) : (v4i){0, 0, 0, 0}; /* read once */
        if (ENC == GV_MXFP4) r.sb[it] = in ? (uint32_t)((gv_gptr)srow)[p] : 0u;
        if (ENC == GV_FP8BLK) r.sf[it] = in ? ((const __attribute__((address_space(1))) float*)(gv_gptr)srow)[p >> 3] : 0.0f; /* 8 pieces of 16 k per 128-k block */
    }
}

/* the lane's share of <row, x>; xs (block fp8 with quantized activations only): the 1x128 activation scale of
 * each piece's block, multiplied into the weight block scale as the tile kernels do */
template <int ENC, int ITER, bool XF8 = false>
__device__ __forceinline__ float gv_dot(const GvRow<ENC, ITER>& r, const v4i (&x)[ITER][GvGeom<ENC>::XQ],
                                        const float (&xs)[ITER]) {
    float acc = 0.0f;
#pragma unroll
    for (int it = 0; it < ITER; it++) {
        if (ENC == GV_BF16) {
#pragma unroll
            for (int j = 0; j < 4; j++) acc = gv_dot2((uint32_t)r.w[it][j], (uint32_t)x[it][0][j], acc);
        } else if (ENC == GV_MXFP4) {
            const float sc = __uint_as_float(r.sb[it] << 23); /* E8M0: 2^(s - 127), folded into the conversion (exact) */
#pragma unroll
            for (int j = 0; j < 4; j++) { /* dword j: 8 nibbles, low nibble = even k */
                const uint32_t wd = (uint32_t)r.w[it][j];
                acc = gv_dot2(__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(wd, sc, 0)), (uint32_t)x[it][j][0], acc);
                acc = gv_dot2(__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(wd, sc, 1)), (uint32_t)x[it][j][1], acc);
                acc = gv_dot2(__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(wd, sc, 2)), (uint32_t)x[it][j][2], acc);
                acc = gv_dot2(__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(wd, sc, 3)), (uint32_t)x[it][j][3], acc);
            }
        } else {
            float part = 0.0f;
#pragma unroll
            for (int j = 0; j < 4; j++) { /* dword j: 4 e4m3 values */
                const uint32_t wd = (uint32_t)r.w[it][j];
                part = gv_dot2(__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wd, 1.0f, false)),
                               (uint32_t)x[it][j >> 1][(j & 1) * 2], part);
                part = gv_dot2(__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wd, 1.0f, true)),
                               (uint32_t)x[it][j >> 1][(j & 1) * 2 + 1], part);
            }
            acc = ENC == GV_FP8BLK ? fmaf(part, XF8 ? xs[it] * r.sf[it] : r.sf[it], acc) : acc + part;
        }
    }
    return acc;
}

/* XF8 (block-fp8 weights, DOWN): the activations are e4m3 rows [rows][K] with one f32 scale per row and 128 k
 * (g.a_f8scale), the intermediate of the fp8 x fp8 arm; they are widened to bf16 once, exactly. */
template <int ENC, bool GLU, int ITER, bool XF8 = false>
__global__ __launch_bounds__(GV_WAVES* WAVE) void k_group_a16_gemv(GroupA16 g) {
    static_assert(!XF8 || (ENC == GV_FP8BLK && !GLU), "quantized activations: the block-fp8 DOWN only");
    constexpr uint32_t KL = GvGeom<ENC>::KL, XQ = GvGeom<ENC>::XQ;
    constexpr int NS = GLU ? 2 : 1;
    __shared__ uint32_t l_row[GV_WINDOW], l_exp[GV_WINDOW];
    __shared__ uint32_t l_n;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wv = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t n_waves = gridDim.x * GV_WAVES, wave_id = blockIdx.x * GV_WAVES + wv;
    const uint32_t K = g.K, N = g.N, E = g.E;
    const uint32_t pieces = K / KL;                                             /* 16-byte pieces of a weight row */
    const uint32_t wrow_bytes = ENC == GV_BF16 ? K * 2u : (ENC == GV_MXFP4 ? K / 2u : K);
    const uint32_t srow_bytes = ENC == GV_MXFP4 ? K / 32u : (ENC == GV_FP8BLK ? (K / 128u) * 4u : 0u);
    const uint32_t wmul = g.wmul ? g.wmul : 1u;

    /* slot-major DOWN: rows of slots that no expert serves are zeroed here, a slot per wave, while wave 0 of each
     * workgroup lists the live rows */
    if (!GLU && g.zs_table && !(g.out_bf16)) {
        const PlowMoeRoute* const tab = (const PlowMoeRoute*)g.zs_table;
        for (uint32_t sl = wave_id; sl < g.zs_nslot; sl += n_waves) {
            const uint32_t e = tab[sl].eid;
            const bool served = e < E && g.wtab[(size_t)e * g.wcols + g.wsel0] != 0ull &&
                                (!g.stab || g.stab[(size_t)e * g.wcols + g.wsel0] != 0ull);
            if (served) continue;
            for (uint32_t h = lane; h < N; h += WAVE) ((float*)g.out)[(size_t)sl * N + h] = 0.0f;
        }
    }
    /* live rows in windows of GV_WINDOW, by their ordinal among the live rows */
    for (uint32_t base = 0;; base += GV_WINDOW) {
        __syncthreads();
        if (wv == 0 && g.tab_direct) { /* the table's live slots in slot order (all of them fit one window) */
            const PlowMoeRoute* const tab = (const PlowMoeRoute*)g.tab_direct;
            uint32_t eid[GV_WINDOW / WAVE];
#pragma unroll
            for (uint32_t j = 0; j < GV_WINDOW / WAVE; j++) {
                const uint32_t sl = j * WAVE + lane;
                eid[j] = sl < g.tab_nslot ? tab[sl].eid : PLOW_EXPERT_UNUSED;
            }
            uint32_t seen = 0;
#pragma unroll
            for (uint32_t j = 0; j < GV_WINDOW / WAVE; j++) {
                const bool live = eid[j] < E;
                const unsigned long long m = __ballot(live);
                const uint32_t ord = seen + (uint32_t)__popcll(m & ((1ull << lane) - 1ull));
                if (live && base == 0u) l_row[ord] = j * WAVE + lane, l_exp[ord] = eid[j];
                seen += (uint32_t)__popcll(m);
            }
            if (lane == 0) l_n = base == 0u ? seen : 0u;
        } else if (wv == 0) { /* one wave lists the window: experts 64 at a time, rows appended in expert order */
            /* every count and offset is asked for before the first is used: one trip to memory, not one per chunk */
            uint32_t cnt_r[GV_ECHUNKS], off_r[GV_ECHUNKS];
#pragma unroll
            for (uint32_t j = 0; j < GV_ECHUNKS; j++) {
                const uint32_t e = j * WAVE + lane;
                cnt_r[j] = e < E ? (uint32_t)g.meta[E + e] : 0u;
                off_r[j] = e < E ? (uint32_t)g.meta[e] : 0u;
            }
            uint32_t seen = 0; /* live rows of the experts before this chunk */
#pragma unroll
            for (uint32_t j = 0; j < GV_ECHUNKS; j++) {
                if (j * WAVE >= E) continue; /* the same in every lane: chunks past the last expert cost nothing */
                const uint32_t e = j * WAVE + lane;
                const uint32_t c = cnt_r[j];
                uint32_t inc = c;
#pragma unroll
                for (uint32_t o = 1; o < WAVE; o <<= 1) {
                    const uint32_t v = __shfl_up(inc, o, 64);
                    if (lane >= o) inc += v;
                }
                const uint32_t first = seen + inc - c; /* ordinal of this expert's first row */
                if (c && first < base + GV_WINDOW) {
                    const uint32_t r0 = off_r[j];
                    for (uint32_t q = 0; q < c; q++) {
                        const uint32_t ord = first + q;
                        if (ord >= base && ord < base + GV_WINDOW) l_row[ord - base] = r0 + q, l_exp[ord - base] = e;
                    }
                }
                seen += (uint32_t)__shfl((int)inc, 63, 64);
            }
            if (lane == 0) l_n = seen > base ? (seen - base < GV_WINDOW ? seen - base : GV_WINDOW) : 0u;
        }
        __syncthreads();
        const uint32_t n = l_n;
        if (n == 0u) break; /* no live row at or past `base` */

        /* the waves are dealt out evenly over the window's rows; a row's waves split its channels evenly */
        constexpr uint32_t RING = ITER == 1 ? 8u : (ITER == 8 ? 2u : 4u);
        /* From a few dozen rows on, the four waves of a workgroup take four consecutive rows of the list and
         * the same share of their channels: rows of one expert are neighbours in the list, so waves that
         * stream the same weight rows start on one CU at the same time and part of the second stream is
         * served by the caches (Kimi-K2 shape, 24 tokens: 847 -> 821 us per layer; keeping the four in step
         * with a barrier per turn of the ring added nothing). With fewer rows every row is dealt its share
         * of all waves (a list that is not a multiple of four would leave waves idle). */
        const bool by_quads = n >= GV_QUADS_FROM;
        uint32_t wpr, ri, part; /* shares per row; this wave's row and share */
        if (by_quads) {
            const uint32_t quads = (n + GV_WAVES - 1u) / GV_WAVES;
            wpr = gridDim.x / quads;
            if (wpr > N) wpr = N;
            ri = wpr ? (blockIdx.x / wpr) * GV_WAVES + wv : n;
            part = wpr ? blockIdx.x % wpr : 0u;
        } else {
            wpr = n_waves / n; /* the form is launched with many more waves than rows */
            if (wpr > N) wpr = N;
            ri = wpr ? wave_id / wpr : n;
            part = wpr ? wave_id % wpr : 0u;
        }
        if (wpr != 0u && ri < n) {
            const uint32_t row = l_row[ri], e = l_exp[ri];
            const uint32_t c_lo = (uint32_t)(((uint64_t)N * part) / wpr), c_hi = (uint32_t)(((uint64_t)N * (part + 1u)) / wpr);
            const uint64_t* wt = g.wtab + (size_t)e * g.wcols;
            const uint64_t* stt = g.stab ? g.stab + (size_t)e * g.wcols : nullptr;
            const uint8_t* wbase[2] = {(const uint8_t*)(uintptr_t)wt[g.wsel0], (const uint8_t*)(uintptr_t)wt[GLU ? g.wsel1 : g.wsel0]};
            const uint8_t* sbase[2] = {stt ? (const uint8_t*)(uintptr_t)stt[g.wsel0] : nullptr,
                                       stt ? (const uint8_t*)(uintptr_t)stt[GLU ? g.wsel1 : g.wsel0] : nullptr};
            const uint32_t wr[2] = {g.wrow0, GLU ? g.wrow1 : g.wrow0};
            const bool resident = wbase[0] && wbase[1] && (ENC == GV_BF16 || (sbase[0] && sbase[1]));
            const uint32_t orow = g.tab_direct ? row : (g.o_idx ? g.o_idx[row] : row);
            if (resident && orow != PLOW_EXPERT_UNUSED && c_lo < c_hi) {
                /* the row of activations: the lane's slice of every piece */
                const uint32_t arow = g.tab_direct ? row / g.tab_kx : (g.a_idx ? g.a_idx[row] : row);
                const uint8_t* xsrc = (const uint8_t*)g.a + (size_t)arow * K * (XF8 ? 1u : 2u);
                v4i x[ITER][XQ];
                float xs[ITER];
#pragma unroll
                for (int it = 0; it < ITER; it++) {
                    const uint32_t p = (uint32_t)it * 64u + lane;
                    xs[it] = 1.0f;
                    if constexpr (XF8) { /* 16 e4m3 values -> the 16 bf16 values the weight pieces meet, same order */
                        const v4i q8 = p < pieces ? *(const v4i*)(xsrc + (size_t)p * 16u) : (v4i){0, 0, 0, 0};
                        xs[it] = p < pieces ? g.a_f8scale[(size_t)arow * (K / 128u) + (p >> 3)] : 0.0f;
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            x[it][j >> 1][(j & 1) * 2] = (int)__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((uint32_t)q8[j], 1.0f, false));
                            x[it][j >> 1][(j & 1) * 2 + 1] = (int)__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((uint32_t)q8[j], 1.0f, true));
                        }
                    } else {
#pragma unroll
                        for (uint32_t j = 0; j < XQ; j++)
                            x[it][j] = p < pieces ? *(const v4i*)(xsrc + ((size_t)p * XQ + j) * 16u) : (v4i){0, 0, 0, 0};
                    }
                }
                const float gate = GLU ? 1.0f : (g.tab_direct ? ((const PlowMoeRoute*)g.tab_direct)[row].gate : (g.gate ? g.gate[row] : 1.0f));
                /* per-channel scales: lane l applies the scale of channel c0 + l when the 64 results of a group are
                 * stored; those of the wave's first group (usually its only one) are asked for here, with the
                 * activations, and not one by one inside the loop */
                auto pc_scale = [&](uint32_t c0, int s_) -> float {
                    const uint32_t ch = c0 + lane < c_hi ? c0 + lane : c_hi - 1u;
                    return ((const float*)sbase[s_])[(size_t)ch * wmul + wr[s_]];
                };
                float pcs0 = 1.0f, pcs1 = 1.0f;
                if (ENC == GV_FP8PC) {
                    pcs0 = pc_scale(c_lo, 0);
                    if (GLU) pcs1 = pc_scale(c_lo, 1);
                }
                auto row_ptrs = [&](uint32_t ch, int s, const uint8_t*& wp, const uint8_t*& sp) {
                    const size_t wrow = (size_t)ch * wmul + wr[s];
                    wp = wbase[s] + wrow * wrow_bytes;
                    sp = ENC == GV_MXFP4 ? sbase[s] + wrow * srow_bytes
                         : ENC == GV_FP8BLK ? sbase[s] + (wrow >> 7) * srow_bytes : nullptr;
                };
                /* A ring of D weight rows (GLU: gate and up rows of a channel alternate, D is even): the loads of
                 * the next D - 1 rows, 6 to 12 KB per wave, are in flight while one row multiplies. Row i of the
                 * wave's range lives in slot i % D; the loop is unrolled D times so that every slot index is a
                 * constant. Conditions on the row index are the same in every lane. */
                constexpr int D = (int)RING, AHEAD = D - 1;
                GvRow<ENC, ITER> ring[D];
                const uint32_t units = (c_hi - c_lo) * (uint32_t)NS;
                auto fetch = [&](GvRow<ENC, ITER>& slot, uint32_t unit, int s) { /* s = unit % NS, a constant at every call */
                    if (unit >= units) return;
                    const uint8_t *wp, *sp;
                    row_ptrs(c_lo + unit / (uint32_t)NS, s, wp, sp);
                    gv_load<ENC, ITER>(slot, wp, sp, lane, pieces);
                };
#pragma unroll
                for (int u = 0; u < AHEAD; u++) fetch(ring[u], (uint32_t)u, u % NS);
                /* lane l keeps the sums of channel c_lo + 64 j + l until the 64 are finished and stored at once */
                float keep_a = 0.0f, keep_b = 0.0f;
                float v0 = 0.0f;
                for (uint32_t i0 = 0; i0 < units; i0 += (uint32_t)D) {
#pragma unroll
                    for (int u = 0; u < D; u++) {
                        const uint32_t unit = i0 + (uint32_t)u;
                        fetch(ring[(u + AHEAD) % D], unit + (uint32_t)AHEAD, (u + AHEAD) % NS);
                        if (unit >= units) continue;
                        const float v = gv_wave_sum(gv_dot<ENC, ITER, XF8>(ring[u], x, xs));
                        if (GLU && (u % NS) == 0) { /* the gate row: its up row comes next */
                            v0 = v;
                            continue;
                        }
                        const uint32_t ch = c_lo + unit / (uint32_t)NS;
                        const uint32_t rel = ch - c_lo;
                        if ((rel & 63u) == lane) keep_a = GLU ? v0 : v, keep_b = v;
                        if ((rel & 63u) == 63u || ch + 1u == c_hi) { /* 64 sums (or the tail): finished and stored at once */
                            const uint32_t c0 = c_lo + (rel & ~63u);
                            if (ENC == GV_FP8PC && c0 != c_lo) { /* a later group of a wave with many channels */
                                pcs0 = pc_scale(c0, 0);
                                if (GLU) pcs1 = pc_scale(c0, 1);
                            }
                            float va = keep_a, vb = keep_b;
                            if (ENC == GV_FP8PC) {
                                va *= pcs0;
                                if (GLU) vb *= pcs1;
                            }
                            const float res = GLU ? moe_glu(va, vb, g.act, g.f0, g.f1) : gate * va;
                            if (c0 + lane <= ch) {
                                if (GLU || g.out_bf16) ((bf16_t*)g.out)[(size_t)orow * N + c0 + lane] = f2bf(res);
                                else ((float*)g.out)[(size_t)orow * N + c0 + lane] = res;
                            }
                        }
                    }
                }
            }
        }
        if (n < GV_WINDOW) break;
    }
}

/* Every wave must be resident at once (a row's share of the waves is fixed when the kernel starts): the
 * grid is what the kernel's registers let a CU hold, asked of the runtime once per kernel. */
template <int ENC, bool GLU, int ITER, bool XF8 = false>
static int launch_gemv_iter(const GroupA16& g, uint32_t n_cu, hipStream_t st) {
    static int per_cu = 0; /* written once with the same value by whoever comes first */
    int nb = __atomic_load_n(&per_cu, __ATOMIC_RELAXED);
    if (nb == 0) {
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, (const void*)k_group_a16_gemv<ENC, GLU, ITER, XF8>, (int)(GV_WAVES * WAVE), 0) != hipSuccess || nb < 1)
            return PLOW_MOE_EDEVICE;
        if (nb > 3) nb = 3;
        __atomic_store_n(&per_cu, nb, __ATOMIC_RELAXED);
    }
    const uint32_t min_grid = GV_WINDOW / GV_WAVES; /* never fewer waves than a window has rows */
    const uint32_t grid = n_cu * (uint32_t)nb < min_grid ? min_grid : n_cu * (uint32_t)nb;
    k_group_a16_gemv<ENC, GLU, ITER, XF8><<<grid, GV_WAVES * WAVE, 0, st>>>(g);
    return 0;
}
template <int ENC, bool GLU, bool XF8 = false>
static int launch_gemv_enc(const GroupA16& g, uint32_t row_bytes, uint32_t n_cu, hipStream_t st) {
    const uint32_t iters = (row_bytes + 1023u) / 1024u;
    if (iters <= 1u) return launch_gemv_iter<ENC, GLU, 1, XF8>(g, n_cu, st);
    if (iters <= 2u) return launch_gemv_iter<ENC, GLU, 2, XF8>(g, n_cu, st);
    if (iters <= 4u) return launch_gemv_iter<ENC, GLU, 4, XF8>(g, n_cu, st);
    if (ENC != GV_MXFP4 && iters <= 8u) return launch_gemv_iter<ENC, GLU, (ENC != GV_MXFP4 ? 8 : 4), XF8>(g, n_cu, st);
    return PLOW_MOE_EINVAL;
}

/* Rows a batch may route in all for this form to be chosen, measured against the tile kernels per layer (a
 * routed row streams its expert's weights by itself here, an expert's rows share them there):
 *   mxfp4 (Kimi-K2 shape)             ahead up to about 28 tokens of 9 slots: 1 token 139 -> 106 us, 4 tokens 305 -> 220,
 *                                     16 tokens 725 -> 637, 24 tokens 938 -> 858, 32 tokens 1006 -> 1037
 *   block fp8 (DeepSeek-V3 shape)     ahead up to 4 tokens: 2 tokens 233 -> 202, 4 tokens 346 -> 328, 5 tokens 361 -> 384
 *   per-channel fp8 (Qwen3 shape)     1 token 87 -> 80, 2 tokens 95 -> 90, mixed from 3 tokens on (skewed routing)
 *   bf16 weights                      level at 1 token, behind at 2 (90 -> 98): twice the bytes per row */
static uint32_t gv_max_slots(uint32_t enc) {
    /* mxfp4: level with the streaming form at 144 rows (Kimi-K2 shape, 16 tokens: 503 against 494 us for the two
     * expert ops), behind at 216 (730 against 649), ahead at 72 (268 against 288) */
    return enc == GV_MXFP4 ? 128u : enc == GV_FP8BLK ? 36u : enc == GV_FP8PC ? 18u : 9u;
}

bool group_a16_gemv_serves(const GroupA16& g) {
    if (!plow_moe_tuning().a16_gemv || (!g.meta && !g.tab_direct) || !g.wtab || g.bias || g.slots_hint == 0u || g.enc > GV_FP8PC ||
        g.slots_hint > gv_max_slots(g.enc))
        return false;
    if (g.tab_direct && (g.tab_nslot > GV_WINDOW || !g.tab_kx || g.a_f8scale)) return false;
    if (g.enc != GV_BF16 && !g.stab) return false;
    if (g.a_f8scale && (g.enc != GV_FP8BLK || g.a_idx)) return false; /* quantized activations: block-fp8 DOWN on aligned rows */
    const uint32_t row_bytes = g.enc == GV_BF16 ? g.K * 2u : (g.enc == GV_MXFP4 ? g.K / 2u : g.K);
    const uint32_t max_bytes = g.enc == GV_MXFP4 ? 4096u : 8192u;
    /* against the streaming fp8 x fp8 DOWN the form wins from rows of a kilobyte on (DeepSeek-V3 shape, one token
     * 44.7 -> 33.0 us); with 256-byte rows a quarter of a wave's lanes have a piece to load (11.3 -> 14.9 us) */
    if (g.a_f8scale && row_bytes < 1024u) return false;
    return g.N != 0u && g.K != 0u && g.K % 128u == 0u && row_bytes <= max_bytes && g.enc <= GV_FP8PC && g.E <= GV_MAX_E;
}

int launch_group_a16_gemv(const GroupA16& g, bool glu, hipStream_t st) {
    if (!group_a16_gemv_serves(g)) return PLOW_MOE_EINVAL;
    const uint32_t n_cu = plow_moe_n_cu();
    if (!n_cu) return PLOW_MOE_EDEVICE;
    const uint32_t row_bytes = g.enc == GV_BF16 ? g.K * 2u : (g.enc == GV_MXFP4 ? g.K / 2u : g.K);
    switch (g.enc) {
    case GV_BF16: return glu ? launch_gemv_enc<GV_BF16, true>(g, row_bytes, n_cu, st) : launch_gemv_enc<GV_BF16, false>(g, row_bytes, n_cu, st);
    case GV_FP8BLK:
        if (g.a_f8scale) return glu ? PLOW_MOE_EINVAL : launch_gemv_enc<GV_FP8BLK, false, true>(g, row_bytes, n_cu, st);
        return glu ? launch_gemv_enc<GV_FP8BLK, true>(g, row_bytes, n_cu, st) : launch_gemv_enc<GV_FP8BLK, false>(g, row_bytes, n_cu, st);
    case GV_MXFP4: return glu ? launch_gemv_enc<GV_MXFP4, true>(g, row_bytes, n_cu, st) : launch_gemv_enc<GV_MXFP4, false>(g, row_bytes, n_cu, st);
    case GV_FP8PC: return glu ? launch_gemv_enc<GV_FP8PC, true>(g, row_bytes, n_cu, st) : launch_gemv_enc<GV_FP8PC, false>(g, row_bytes, n_cu, st);
    default: return PLOW_MOE_EUNSUPPORTED;
    }
}
