/* experts_w8a8_tiled.hip — the many-rows-per-expert (prefill) form of the block-fp8 x fp8 grouped
 * GEMMs (ops 85 / 86, arm 2 / 3). Same arithmetic as experts_w8a8.hip; different data flow.
 *
 * Workgroup tile = 128 aligned rows x 256 weight rows (GLU: 128 gate + 128 up rows of one
 * 128-channel block; DOWN: 256 output channels), K walked in 128-k blocks through a ring of three
 * LDS stages. The twelve waves are specialised:
 *
 *   waves 8..11, loaders   issue every global load of the tile, all of them direct global -> LDS
 *                          (global_load_lds_dwordx4), with 8 consecutive lanes on one 128-byte line,
 *                          the only lane -> address shape the vector memory pipeline takes at full
 *                          rate (a "lane = matrix row" load runs at a quarter of it). A loader that
 *                          finds the load queue full stalls only itself.
 *   waves 0..7, consumers  two per SIMD; read operands from LDS and multiply. Consumer c owns 32 of
 *                          the 256 weight rows (two 16-row groups; GLU: gate and up of channels
 *                          16c..16c+15) and all 128 token rows, on
 *                          v_mfma_f32_16x16x128_f8f6f4 with weights as the A operand and token rows
 *                          as the B operand: a lane's accumulators belong to ONE token row (lane & 15
 *                          of each 16-row group) and four consecutive channels, so the 1x128
 *                          activation scale is one value per lane and row group, and gate / up of a
 *                          channel sit in the same lane and register index.
 *
 * Per 128-k block: a loader waits for its own loads of the block (s_waitcnt vmcnt(n)), then all
 * waves meet at one barrier; after it the consumers multiply the block while the loaders refill the
 * stage the consumers have just left, two blocks ahead. Per 16-row group a consumer issues two
 * matrix instructions (one per weight group) and acc = fmaf(t, a_scale[row][kb] * w_scale, acc); the
 * next group's B operand is read from LDS meanwhile.
 *
 * A direct load writes the 64 lanes' 16-byte pieces to consecutive LDS addresses, so rows sit
 * unpadded (128 B); bank conflicts are avoided by swizzling on the GLOBAL side: LDS piece p of row r
 * holds global piece p ^ lds_swz8(r), and the lanes an operand read serves in one clock then cover all
 * 64 banks. Rows of the tile beyond the expert's live rows read the tile's first row and carry a
 * zero activation scale; 16-row groups with no live row are skipped by the consumers.
 * Tiles are walked by persistent workgroups (one per CU) in an order that puts the tiles sharing
 * token rows and weight rows on one XCD at the same time (see the tile loop). */
#include <stdlib.h>
#include <string.h>
#include <type_traits>
#include "common.h"
#include "kernels.h"
#include "tuning.h"

/* SiLU(g) * u for the tile epilogue, where 128 x 128 of them per tile run on the waves that should be
 * multiplying: hardware exp2 and reciprocal (about 1 ulp each) instead of the library's expf and an
 * IEEE division, a third of the instructions. The result is rounded to fp8 (block mode) or bf16 (op 188,
 * per-channel mode) right after, far above this error: against the expf form over the same accumulators
 * the bf16 result differs in about one element in 10^5, by one bf16 step (measured by the GPU test that
 * runs op 188 on both forms). Limits: +inf gives +inf and NaN stays NaN as with g / (1 + expf(-g));
 * g = -inf gives NaN here (-inf * rcp(inf)) where the library form gives -0, which only an accumulator
 * that has already overflowed can reach. */
__device__ __forceinline__ float t5_glu(float gt, float up, uint32_t act, float f0, float f1) {
    if (act == PLOW_MOE_ACT_SILU) {
        const float e = __builtin_amdgcn_exp2f(gt * -1.4426950408889634f);
        return (gt * __builtin_amdgcn_rcpf(1.0f + e)) * up;
    }
    return moe_glu(gt, up, act, f0, f1);
}

#define T5_BM 144u /* rows the LDS plan holds per tile: nine 16-row groups (kernels built for eight use 128) */
#define T5_AS 192u /* row slots of a stage's scale array (three loaders x 64 lanes) */
#define T5_STAGES 3u
#define T5_MAX_ROW_TILES 65535u /* what the 16-bit tile directory counts */
/* Row tiles of an expert that take their channel tiles together (see the tile loop): eight on the block-scaled
 * fp8 x fp8 and fp4 x fp4 arms (DeepSeek-V3 shape, 4096 tokens: what the L2s fetch drops from x1.30 to x1.10 of the
 * GLU's algorithmic bytes and the layer takes 2.8 % less, 4.5 % at 8192 tokens), one (row-tile-major order) on the
 * others: per-channel fp8 and bf16 rows measured level at 2, 4 and 8, mxfp4 weights under bf16 rows 14 % behind. */
#define T5_RB_BLOCK 8u
#define T5_NLOAD 13 /* direct loads per loader and block: 1 scale, 4 token-row, 8 weight-row; loaders 0 and 1 one more
                     * token-row load (the ninth group) */

struct T5Lds {
    uint8_t a[T5_STAGES][T5_BM * 128u]; /* token rows of a 128-k block, swizzled */
    uint8_t w[T5_STAGES][256u * 128u];  /* weight rows, swizzled; row = 32 * consumer + 16 * group + r */
    float as[T5_STAGES][T5_AS];         /* activation scales of the block */
    float wsc[2][2][128];               /* [tile parity][gate|down, up] weight block scales, all of K */
    uint32_t epi_idx[2][T5_AS];         /* [tile parity] GLU: row_token, DOWN: row_partidx of the tile's rows */
    float epi_gate[2][T5_AS];           /* [tile parity] DOWN: row_gate */
    uint16_t prefix[1056];              /* inclusive tile count over experts: at most 2^18 slots / 144 + 1056 */
};
static_assert(sizeof(T5Lds) <= 160u * 1024u, "the tile's LDS plan must fit one CU");
/* the plan of the fp4 x fp4 arm: 128-row tiles, a block is 256 k (128 bytes of nibbles per row, so the
 * ring has the geometry of the fp8 one), and every row of a stage brings its eight E8M0 bytes */
struct T5LdsA4 {
    uint8_t a[T5_STAGES][128u * 128u];
    uint8_t w[T5_STAGES][256u * 128u];
    uint8_t ts[T5_STAGES][128u][8]; /* token-row scales of the block */
    uint8_t ws[T5_STAGES][256u][8]; /* weight-row scales of the block */
    uint32_t epi_idx[2][T5_AS];
    float epi_gate[2][T5_AS];
    uint16_t prefix[1056];
};
static_assert(sizeof(T5LdsA4) <= 160u * 1024u, "the tile's LDS plan must fit one CU");

/* the plan of the mxfp4-weight form under bf16 rows: a block is 128 k, a token row 256 bytes of bf16 (16-byte pieces
 * swizzled by lds_swz16), a weight row 64 bytes of e2m1 with its four E8M0 bytes beside it; 128-row tiles */
struct T5LdsW4 {
    uint8_t a[T5_STAGES][128u * 256u];
    uint8_t w[T5_STAGES][256u * 64u];
    uint8_t ws[T5_STAGES][256u][4];
    uint32_t epi_idx[2][T5_AS];
    float epi_gate[2][T5_AS];
    uint16_t prefix[1056];
};
static_assert(sizeof(T5LdsW4) <= 160u * 1024u, "the tile's LDS plan must fit one CU");

typedef __attribute__((address_space(3))) void lds_void;

/* The ring is written by direct global -> LDS loads that the compiler would otherwise fence
 * conservatively (a full s_waitcnt vmcnt(0) before every LDS read and barrier). So the ring is read
 * with explicit ds_read instructions and synchronised with explicit waits. */
__device__ __forceinline__ uint32_t lds_off(const void* p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}
template <uint32_t OFF>
__device__ __forceinline__ v4i ds_read16(uint32_t addr) {
    v4i r;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF) : "memory");
    return r;
}
template <uint32_t OFF>
__device__ __forceinline__ float ds_read4(uint32_t addr) {
    float r;
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF) : "memory");
    return r;
}
template <uint32_t OFF>
__device__ __forceinline__ int ds_read1(uint32_t addr) {
    int r;
    asm volatile("ds_read_u8 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF) : "memory");
    return r;
}
template <uint32_t OFF>
__device__ __forceinline__ v2i ds_read8(uint32_t addr) {
    v2i r;
    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF) : "memory");
    return r;
}
/* all ds_reads issued so far have returned */
#define LDS_WAIT_ALL() asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory")
#define WG_BARRIER() asm volatile("s_barrier" ::: "memory")
/* wait until at most n of this wave's loads are outstanding, then the workgroup barrier */
#define LOADER_BARRIER(n) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(n) : "memory")


/* ---- one 128-k block of a consumer wave (names are those of the kernel body) -------------------- */
#define T5_BLOCK_HEAD()                                                                                      \
    const uint32_t ab = a_base + st * (uint32_t)sizeof(L.a[0]), wb = w_base + st * (256u * 128u) + cw * (32u * 128u);  \
    const uint32_t blo = ab + op_lo, bhi = ab + op_hi;                                                       \
    const uint32_t alo = wb + op_lo, ahi = wb + op_hi;                                                       \
    const uint32_t sl = s_base + st * (T5_AS * 4u) + r16 * 4u;                                               \
    const uint32_t cl = c_base + par * 1024u + kb * 4u;
#define T5_ADVANCE() st = st == 2u ? 0u : st + 1u
/* A block of a consumer with N live row groups (N a constant, 1..9): straight-line code without a
 * condition in it, so no value is ever copied between registers. Per-channel mode: the scales are outside
 * the K reduction, so the matrix unit accumulates straight through; block mode: one scaled add per 128-k
 * block, and the scaled adds of group RG follow the matrix instructions of group RG + 1, never wait for
 * a result and overlap with the matrix unit.
 * LDS reads return in issue order: with the reads of group RG + 1 (two operand halves, and the scale in
 * block mode) issued behind those of group RG, "at most that many outstanding" means group RG has
 * arrived. Three operand buffers rotate, so a group's reads are issued two groups before its multiply. */
#define T5_GROUP_N(RG, N)                                                                                    \
    if ((RG) < (N)) {                                                                                        \
        asm volatile("s_waitcnt lgkmcnt(%2)"                                                                 \
                     : "+v"(bl[(RG) % 3]), "+v"(bh[(RG) % 3])                                                \
                     : "n"((RG) + 1 < (N) ? (PC ? 2 : 3) : 0));                                              \
        if (!PC) {                                                                                           \
            asm volatile("" : "+v"(as_[(RG) % 3]));                                                          \
            sc[(RG) & 1][0] = as_[(RG) % 3] * ws0;                                                           \
            sc[(RG) & 1][1] = as_[(RG) % 3] * ws1;                                                           \
        }                                                                                                    \
        if ((RG) + 2 < (N)) {                                                                                \
            bl[((RG) + 2) % 3] = ds_read16<((RG) + 2) * 2048u>(blo);                                         \
            bh[((RG) + 2) % 3] = ds_read16<((RG) + 2) * 2048u>(bhi);                                         \
            if (!PC) as_[((RG) + 2) % 3] = ds_read4<((RG) + 2) * 64u>(sl);                                   \
        }                                                                                                    \
        const v8i b = __builtin_shufflevector(bl[(RG) % 3], bh[(RG) % 3], 0, 1, 2, 3, 4, 5, 6, 7);           \
        if (PC) {                                                                                            \
            acc[RG][0] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(aop[0], b, acc[RG][0], 0, 0, 0, 0, 0, 0); \
            acc[RG][1] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(aop[1], b, acc[RG][1], 0, 0, 0, 0, 0, 0); \
        } else {                                                                                             \
            const v4f z = {0.0f, 0.0f, 0.0f, 0.0f};                                                          \
            t[(RG) & 1][0] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(aop[0], b, z, 0, 0, 0, 0, 0, 0); \
            t[(RG) & 1][1] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(aop[1], b, z, 0, 0, 0, 0, 0, 0); \
        }                                                                                                    \
    }
#define T5_SCALE_N(RG, N)                                                                                    \
    if (!PC && (RG) < (N)) {                                                                                 \
        _Pragma("unroll") for (int i = 0; i < 4; i++) {                                                      \
            acc[RG][0][i] = fmaf(t[(RG) & 1][0][i], sc[(RG) & 1][0], acc[RG][0][i]);                         \
            acc[RG][1][i] = fmaf(t[(RG) & 1][1][i], sc[(RG) & 1][1], acc[RG][1][i]);                         \
        }                                                                                                    \
    }
/* the operands of the block: weight scales, the two weight operands, then the token operands of groups 0
 * and 1; the weight operands are waited for with those groups still in flight */
#define T5_BLOCK_OPERANDS_N(N)                                                                               \
    float ws0 = 0.0f, ws1 = 0.0f;                                                                            \
    if (!PC) {                                                                                               \
        ws0 = ds_read4<0>(cl);                                                                               \
        ws1 = ds_read4<512>(cl);                                                                             \
    }                                                                                                        \
    v4i al[2], ah[2];                                                                                        \
    al[0] = ds_read16<0>(alo), ah[0] = ds_read16<0>(ahi);                                                    \
    al[1] = ds_read16<2048>(alo), ah[1] = ds_read16<2048>(ahi);                                              \
    v4i bl[3], bh[3];                                                                                        \
    float as_[3];                                                                                            \
    as_[0] = as_[1] = as_[2] = 0.0f;                                                                         \
    bl[0] = ds_read16<0>(blo), bh[0] = ds_read16<0>(bhi);                                                    \
    if (!PC) as_[0] = ds_read4<0>(sl);                                                                       \
    if ((N) > 1) {                                                                                           \
        bl[1] = ds_read16<2048u>(blo), bh[1] = ds_read16<2048u>(bhi);                                        \
        if (!PC) as_[1] = ds_read4<64u>(sl);                                                                 \
    }                                                                                                        \
    asm volatile("s_waitcnt lgkmcnt(%6)"                                                                     \
                 : "+v"(al[0]), "+v"(ah[0]), "+v"(al[1]), "+v"(ah[1]), "+v"(ws0), "+v"(ws1)                  \
                 : "n"((PC ? 2 : 3) * ((N) > 1 ? 2 : 1)));                                                   \
    if (!GLU && !PC) ws0 = ws1 = ((cw & 4u) ? ws1 : ws0);                                                    \
    v8i aop[2];                                                                                              \
    _Pragma("unroll") for (int x = 0; x < 2; x++) aop[x] = __builtin_shufflevector(al[x], ah[x], 0, 1, 2, 3, 4, 5, 6, 7);
#define T5_BLOCK_N(N)                                                                                        \
    T5_BLOCK_HEAD()                                                                                          \
    T5_BLOCK_OPERANDS_N(N)                                                                                   \
    v4f t[2][2];                                                                                             \
    float sc[2][2];                                                                                          \
    T5_GROUP_N(0, N)                                                                                         \
    T5_GROUP_N(1, N) T5_SCALE_N(0, N)                                                                        \
    T5_GROUP_N(2, N) T5_SCALE_N(1, N)                                                                        \
    T5_GROUP_N(3, N) T5_SCALE_N(2, N)                                                                        \
    T5_GROUP_N(4, N) T5_SCALE_N(3, N)                                                                        \
    T5_GROUP_N(5, N) T5_SCALE_N(4, N)                                                                        \
    T5_GROUP_N(6, N) T5_SCALE_N(5, N)                                                                        \
    T5_GROUP_N(7, N) T5_SCALE_N(6, N)                                                                        \
    T5_GROUP_N((N) > 8 ? 8 : 0, (N) > 8 ? (N) : 0) T5_SCALE_N(7, N)                                          \
    T5_SCALE_N((N) > 8 ? 8 : 0, (N) > 8 ? (N) : 0)
/* ---- the same block with bf16 activations (A16): a block is 64 k. Token rows are 128 bytes of bf16
 *      (same stage geometry and swizzle as the fp8 rows), weight rows 64 bytes of e4m3 decoded to bf16 in
 *      registers (exact: e4m3 fits bf16), v_mfma_f32_16x16x32_bf16 twice per operand pair. No activation
 *      scales; block mode scales the block's product by the weight block scale (one per two blocks),
 *      per-channel mode accumulates straight through. Weight row r16 of an operand holds its 8-byte piece
 *      j at (j ^ 2 * ((r16 >> 2) & 3)): a ds_read_b64 serves 32 consecutive lanes per clock (16 rows x two
 *      k-chunks), and rows 4 apart start on the same bank. ---- */
#define T5A_BLOCK_HEAD()                                                                                     \
    const uint32_t ab = a_base + st * (uint32_t)sizeof(L.a[0]), wb = w_base + st * (256u * 128u) + cw * (32u * 64u);   \
    const uint32_t b0 = ab + opb0, b1 = ab + opb1;                                                           \
    const uint32_t cl = c_base + par * 1024u + (kb >> 1) * 4u;
#define T5A_DECODE(R) t5a_decode(R)
#define T5A_GROUP_N(RG, N)                                                                                   \
    if ((RG) < (N)) {                                                                                        \
        asm volatile("s_waitcnt lgkmcnt(%2)"                                                                 \
                     : "+v"(bx[(RG) % 3][0]), "+v"(bx[(RG) % 3][1])                                          \
                     : "n"((RG) + 1 < (N) ? 2 : 0));                                                         \
        if ((RG) + 2 < (N)) {                                                                                \
            bx[((RG) + 2) % 3][0] = ds_read16<((RG) + 2) * 2048u>(b0);                                       \
            bx[((RG) + 2) % 3][1] = ds_read16<((RG) + 2) * 2048u>(b1);                                       \
        }                                                                                                    \
        const v8bf B0 = __builtin_bit_cast(v8bf, bx[(RG) % 3][0]), B1 = __builtin_bit_cast(v8bf, bx[(RG) % 3][1]); \
        if (PC) {                                                                                            \
            acc[RG][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aop[0][0], B0, acc[RG][0], 0, 0, 0);        \
            acc[RG][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aop[1][0], B0, acc[RG][1], 0, 0, 0);        \
            acc[RG][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aop[0][1], B1, acc[RG][0], 0, 0, 0);        \
            acc[RG][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aop[1][1], B1, acc[RG][1], 0, 0, 0);        \
        } else {                                                                                             \
            const v4f z = {0.0f, 0.0f, 0.0f, 0.0f};                                                          \
            t[(RG) & 1][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aop[0][0], B0, z, 0, 0, 0);             \
            t[(RG) & 1][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aop[1][0], B0, z, 0, 0, 0);             \
            t[(RG) & 1][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aop[0][1], B1, t[(RG) & 1][0], 0, 0, 0); \
            t[(RG) & 1][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aop[1][1], B1, t[(RG) & 1][1], 0, 0, 0); \
        }                                                                                                    \
    }
#define T5A_SCALE_N(RG, N)                                                                                   \
    if (!PC && (RG) < (N)) {                                                                                 \
        _Pragma("unroll") for (int i = 0; i < 4; i++) {                                                      \
            acc[RG][0][i] = fmaf(t[(RG) & 1][0][i], ws0, acc[RG][0][i]);                                     \
            acc[RG][1][i] = fmaf(t[(RG) & 1][1][i], ws1, acc[RG][1][i]);                                     \
        }                                                                                                    \
    }
#define T5A_BLOCK_N(N)                                                                                       \
    T5A_BLOCK_HEAD()                                                                                         \
    float ws0 = 0.0f, ws1 = 0.0f;                                                                            \
    if (!PC) {                                                                                               \
        ws0 = ds_read4<0>(cl);                                                                               \
        ws1 = ds_read4<512>(cl);                                                                             \
    }                                                                                                        \
    v2i ar[2][2];                                                                                            \
    ar[0][0] = ds_read8<0>(wb + opa0), ar[0][1] = ds_read8<0>(wb + opa1);                                    \
    ar[1][0] = ds_read8<1024>(wb + opa0), ar[1][1] = ds_read8<1024>(wb + opa1);                              \
    v4i bx[3][2];                                                                                            \
    bx[0][0] = ds_read16<0>(b0), bx[0][1] = ds_read16<0>(b1);                                                \
    if ((N) > 1) bx[1][0] = ds_read16<2048u>(b0), bx[1][1] = ds_read16<2048u>(b1);                           \
    asm volatile("s_waitcnt lgkmcnt(%6)"                                                                     \
                 : "+v"(ar[0][0]), "+v"(ar[0][1]), "+v"(ar[1][0]), "+v"(ar[1][1]), "+v"(ws0), "+v"(ws1)      \
                 : "n"((N) > 1 ? 4 : 2));                                                                    \
    if (!GLU && !PC) ws0 = ws1 = ((cw & 4u) ? ws1 : ws0);                                                    \
    v8bf aop[2][2];                                                                                          \
    _Pragma("unroll") for (int x = 0; x < 2; x++)                                                            \
        _Pragma("unroll") for (int k2 = 0; k2 < 2; k2++) aop[x][k2] = T5A_DECODE(ar[x][k2]);                 \
    v4f t[2][2];                                                                                             \
    T5A_GROUP_N(0, N)                                                                                        \
    T5A_GROUP_N(1, N) T5A_SCALE_N(0, N)                                                                      \
    T5A_GROUP_N(2, N) T5A_SCALE_N(1, N)                                                                      \
    T5A_GROUP_N(3, N) T5A_SCALE_N(2, N)                                                                      \
    T5A_GROUP_N(4, N) T5A_SCALE_N(3, N)                                                                      \
    T5A_GROUP_N(5, N) T5A_SCALE_N(4, N)                                                                      \
    T5A_GROUP_N(6, N) T5A_SCALE_N(5, N)                                                                      \
    T5A_GROUP_N(7, N) T5A_SCALE_N(6, N)                                                                      \
    T5A_GROUP_N((N) > 8 ? 8 : 0, (N) > 8 ? (N) : 0) T5A_SCALE_N(7, N)                                        \
    T5A_SCALE_N((N) > 8 ? 8 : 0, (N) > 8 ? (N) : 0)
/* ---- the same block with bf16 weights (W16): a weight row is 128 bytes of bf16 per 64-k block, in the token
 *      rows' geometry and swizzle, read as the operand it is; no scales anywhere, the accumulators run straight
 *      through K ---- */
#define T5W_BLOCK_HEAD()                                                                                     \
    const uint32_t ab = a_base + st * (uint32_t)sizeof(L.a[0]), wb = w_base + st * (256u * 128u) + cw * (32u * 128u);  \
    const uint32_t b0 = ab + opb0, b1 = ab + opb1;
#define T5W_GROUP_N(RG, N)                                                                                   \
    if ((RG) < (N)) {                                                                                        \
        asm volatile("s_waitcnt lgkmcnt(%2)"                                                                 \
                     : "+v"(bx[(RG) % 3][0]), "+v"(bx[(RG) % 3][1])                                          \
                     : "n"((RG) + 1 < (N) ? 2 : 0));                                                         \
        if ((RG) + 2 < (N)) {                                                                                \
            bx[((RG) + 2) % 3][0] = ds_read16<((RG) + 2) * 2048u>(b0);                                       \
            bx[((RG) + 2) % 3][1] = ds_read16<((RG) + 2) * 2048u>(b1);                                       \
        }                                                                                                    \
        const v8bf B0 = __builtin_bit_cast(v8bf, bx[(RG) % 3][0]), B1 = __builtin_bit_cast(v8bf, bx[(RG) % 3][1]); \
        acc[RG][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aop[0][0], B0, acc[RG][0], 0, 0, 0);            \
        acc[RG][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aop[1][0], B0, acc[RG][1], 0, 0, 0);            \
        acc[RG][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aop[0][1], B1, acc[RG][0], 0, 0, 0);            \
        acc[RG][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aop[1][1], B1, acc[RG][1], 0, 0, 0);            \
    }
#define T5W_BLOCK_N(N)                                                                                       \
    T5W_BLOCK_HEAD()                                                                                         \
    v4i ar[2][2];                                                                                            \
    ar[0][0] = ds_read16<0>(wb + opb0), ar[0][1] = ds_read16<0>(wb + opb1);                                  \
    ar[1][0] = ds_read16<2048>(wb + opb0), ar[1][1] = ds_read16<2048>(wb + opb1);                            \
    v4i bx[3][2];                                                                                            \
    bx[0][0] = ds_read16<0>(b0), bx[0][1] = ds_read16<0>(b1);                                                \
    if ((N) > 1) bx[1][0] = ds_read16<2048u>(b0), bx[1][1] = ds_read16<2048u>(b1);                           \
    asm volatile("s_waitcnt lgkmcnt(%4)"                                                                     \
                 : "+v"(ar[0][0]), "+v"(ar[0][1]), "+v"(ar[1][0]), "+v"(ar[1][1])                            \
                 : "n"((N) > 1 ? 4 : 2));                                                                    \
    v8bf aop[2][2];                                                                                          \
    _Pragma("unroll") for (int x = 0; x < 2; x++)                                                            \
        _Pragma("unroll") for (int k2 = 0; k2 < 2; k2++) aop[x][k2] = __builtin_bit_cast(v8bf, ar[x][k2]);   \
    T5W_GROUP_N(0, N) T5W_GROUP_N(1, N) T5W_GROUP_N(2, N) T5W_GROUP_N(3, N)                                  \
    T5W_GROUP_N(4, N) T5W_GROUP_N(5, N) T5W_GROUP_N(6, N) T5W_GROUP_N(7, N)
/* ---- the block with mxfp4 weights under bf16 rows (W4): 128 k. A lane's weight piece is 16 bytes of its row = the 32 k
 *      of ONE E8M0 block (k 32q .. 32q + 31), decoded to bf16 with the scale folded in (exact, as the streaming
 *      kernels do); matrix instruction j multiplies the lane's dword j (k 32q + 8j ..) with the token piece 4q + j,
 *      so the four instructions of an operand pair cover the block's 128 k, each k once. Token pieces of group
 *      RG + 1 are read while group RG multiplies (two buffers of four pieces). No scales outside the decode: the
 *      accumulators run straight through K. ---- */
#define T5X_BLOCK_HEAD()                                                                                     \
    const uint32_t ab = a_base + st * (uint32_t)sizeof(L.a[0]) + r16 * 256u;                                 \
    const uint32_t wb = w_base + st * (256u * 64u) + cw * (32u * 64u) + r16 * 64u + ((q ^ ((r16 >> 2) & 3u)) << 4); \
    const uint32_t wsl = wsb_base + st * 1024u + (cw * 32u + r16) * 4u + q;
#define T5X_READ_GROUP(BUF, RG)                                                                              \
    bx[BUF][0] = ds_read16<(RG) * 4096u>(ab + xo0), bx[BUF][1] = ds_read16<(RG) * 4096u>(ab + xo1);          \
    bx[BUF][2] = ds_read16<(RG) * 4096u>(ab + xo2), bx[BUF][3] = ds_read16<(RG) * 4096u>(ab + xo3);
#define T5X_GROUP_N(RG, N)                                                                                   \
    if ((RG) < (N)) {                                                                                        \
        if ((RG) + 1 < (N)) { T5X_READ_GROUP(((RG) + 1) & 1, (RG) + 1) }                                      \
        asm volatile("s_waitcnt lgkmcnt(%4)"                                                                 \
                     : "+v"(bx[(RG) & 1][0]), "+v"(bx[(RG) & 1][1]), "+v"(bx[(RG) & 1][2]), "+v"(bx[(RG) & 1][3]) \
                     : "n"((RG) + 1 < (N) ? 4 : 0));                                                         \
        _Pragma("unroll") for (int j = 0; j < 4; j++) {                                                      \
            const v8bf B = __builtin_bit_cast(v8bf, bx[(RG) & 1][j]);                                        \
            acc[RG][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aop[0][j], B, acc[RG][0], 0, 0, 0);         \
            acc[RG][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aop[1][j], B, acc[RG][1], 0, 0, 0);         \
        }                                                                                                    \
    }
#define T5X_BLOCK_N(N)                                                                                       \
    T5X_BLOCK_HEAD()                                                                                         \
    v4i ax[2];                                                                                               \
    int sb[2];                                                                                               \
    ax[0] = ds_read16<0>(wb), ax[1] = ds_read16<1024>(wb);                                                   \
    sb[0] = ds_read1<0>(wsl), sb[1] = ds_read1<64>(wsl);                                                     \
    v4i bx[2][4];                                                                                            \
    T5X_READ_GROUP(0, 0)                                                                                     \
    asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(ax[0]), "+v"(ax[1]), "+v"(sb[0]), "+v"(sb[1]));               \
    v8bf aop[2][4];                                                                                          \
    _Pragma("unroll") for (int x = 0; x < 2; x++)                                                            \
        _Pragma("unroll") for (int j = 0; j < 4; j++) aop[x][j] = t5x_decode((uint32_t)ax[x][j], (uint32_t)sb[x]); \
    T5X_GROUP_N(0, N) T5X_GROUP_N(1, N) T5X_GROUP_N(2, N) T5X_GROUP_N(3, N)                                  \
    T5X_GROUP_N(4, N) T5X_GROUP_N(5, N) T5X_GROUP_N(6, N) T5X_GROUP_N(7, N)
/* ---- the block of the fp4 x fp4 arm: 256 k as two matrix instructions of 128 k, both operands e2m1 with
 *      their E8M0 bytes applied by the instruction itself (a lane's 32 k are one scale block, its byte goes
 *      in as a register: with constant scale arguments the compiler would pick the unscaled instruction).
 *      The accumulator runs straight through K. ---- */
#define T5Q_BLOCK_HEAD()                                                                                     \
    const uint32_t ab = a_base + st * (uint32_t)sizeof(L.a[0]), wb = w_base + st * (256u * 128u) + cw * (32u * 128u); \
    const uint32_t b0 = ab + opb0, b1 = ab + opb1;                                                           \
    const uint32_t tsl = ts_base + st * (128u * 8u) + r16 * 8u + q;                                          \
    const uint32_t wsl = wsb_base + st * (256u * 8u) + (cw * 32u + r16) * 8u + q;
#define T5Q_MFMA(A, B, C, SA, SB)                                                                            \
    __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(__builtin_shufflevector(A, zero4, 0, 1, 2, 3, 4, 5, 6, 7), \
                                                     __builtin_shufflevector(B, zero4, 0, 1, 2, 3, 4, 5, 6, 7), C, 4, 4, 0, SA, 0, SB)
#define T5Q_GROUP_N(RG, N)                                                                                   \
    if ((RG) < (N)) {                                                                                        \
        asm volatile("s_waitcnt lgkmcnt(%4)"                                                                 \
                     : "+v"(bx[(RG) % 3][0]), "+v"(bx[(RG) % 3][1]), "+v"(bs[(RG) % 3][0]), "+v"(bs[(RG) % 3][1]) \
                     : "n"((RG) + 1 < (N) ? 4 : 0));                                                         \
        if ((RG) + 2 < (N)) {                                                                                \
            bx[((RG) + 2) % 3][0] = ds_read16<((RG) + 2) * 2048u>(b0);                                       \
            bx[((RG) + 2) % 3][1] = ds_read16<((RG) + 2) * 2048u>(b1);                                       \
            bs[((RG) + 2) % 3][0] = ds_read1<((RG) + 2) * 128u>(tsl);                                        \
            bs[((RG) + 2) % 3][1] = ds_read1<((RG) + 2) * 128u + 4u>(tsl);                                   \
        }                                                                                                    \
        acc[RG][0] = T5Q_MFMA(ax[0][0], bx[(RG) % 3][0], acc[RG][0], as4[0][0], bs[(RG) % 3][0]);            \
        acc[RG][1] = T5Q_MFMA(ax[1][0], bx[(RG) % 3][0], acc[RG][1], as4[1][0], bs[(RG) % 3][0]);            \
        acc[RG][0] = T5Q_MFMA(ax[0][1], bx[(RG) % 3][1], acc[RG][0], as4[0][1], bs[(RG) % 3][1]);            \
        acc[RG][1] = T5Q_MFMA(ax[1][1], bx[(RG) % 3][1], acc[RG][1], as4[1][1], bs[(RG) % 3][1]);            \
    }
#define T5Q_BLOCK_N(N)                                                                                       \
    T5Q_BLOCK_HEAD()                                                                                         \
    const v4i zero4 = {0, 0, 0, 0};                                                                          \
    v4i ax[2][2];                                                                                            \
    int as4[2][2];                                                                                           \
    ax[0][0] = ds_read16<0>(wb + opb0), ax[0][1] = ds_read16<0>(wb + opb1);                                  \
    ax[1][0] = ds_read16<2048>(wb + opb0), ax[1][1] = ds_read16<2048>(wb + opb1);                            \
    as4[0][0] = ds_read1<0>(wsl), as4[0][1] = ds_read1<4>(wsl);                                              \
    as4[1][0] = ds_read1<128>(wsl), as4[1][1] = ds_read1<132>(wsl);                                          \
    v4i bx[3][2];                                                                                            \
    int bs[3][2];                                                                                            \
    bx[0][0] = ds_read16<0>(b0), bx[0][1] = ds_read16<0>(b1);                                                \
    bs[0][0] = ds_read1<0>(tsl), bs[0][1] = ds_read1<4>(tsl);                                                \
    if ((N) > 1) {                                                                                           \
        bx[1][0] = ds_read16<2048u>(b0), bx[1][1] = ds_read16<2048u>(b1);                                    \
        bs[1][0] = ds_read1<128u>(tsl), bs[1][1] = ds_read1<132u>(tsl);                                      \
    }                                                                                                        \
    asm volatile("s_waitcnt lgkmcnt(%8)"                                                                     \
                 : "+v"(ax[0][0]), "+v"(ax[0][1]), "+v"(ax[1][0]), "+v"(ax[1][1]), "+v"(as4[0][0]),          \
                   "+v"(as4[0][1]), "+v"(as4[1][0]), "+v"(as4[1][1])                                         \
                 : "n"((N) > 1 ? 8 : 4));                                                                    \
    T5Q_GROUP_N(0, N) T5Q_GROUP_N(1, N) T5Q_GROUP_N(2, N) T5Q_GROUP_N(3, N)                                  \
    T5Q_GROUP_N(4, N) T5Q_GROUP_N(5, N) T5Q_GROUP_N(6, N) T5Q_GROUP_N(7, N)
/* eight e4m3 bytes -> eight bf16 (the hardware conversion is exact) */
__device__ __forceinline__ v8bf t5a_decode(v2i r) {
    const v2bf p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((uint32_t)r[0], 1.0f, false);
    const v2bf p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((uint32_t)r[0], 1.0f, true);
    const v2bf p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((uint32_t)r[1], 1.0f, false);
    const v2bf p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((uint32_t)r[1], 1.0f, true);
    return (v8bf){p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
}
/* eight e2m1 values of a dword (low nibble = even k) -> eight bf16, scaled by their block's E8M0 byte (exact) */
__device__ __forceinline__ v8bf t5x_decode(uint32_t wd, uint32_t e8m0) {
    const float sc = __uint_as_float(e8m0 << 23); /* 2^(s - 127) */
    const v2bf p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(wd, sc, 0);
    const v2bf p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(wd, sc, 1);
    const v2bf p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(wd, sc, 2);
    const v2bf p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(wd, sc, 3);
    return (v8bf){p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
}
/* the K loop of a tile for a consumer wave with N live groups (BODY empty: it only keeps the barriers) */
#define T5_RUN_BLOCKS(BODY)                                                                                  \
    for (uint32_t kb = 0; kb < KB; kb++) {                                                                   \
        WG_BARRIER(); /* block kb is in LDS */                                                               \
        _Pragma("unroll") for (uint32_t sub = 0; sub < SUBS; sub++) {                                        \
            const uint32_t cw = cw0 + sub;                                                                   \
            (void)cw;                                                                                        \
            v4f(&acc)[NG][2] = accs[sub];                                                                 \
            (void)acc;                                                                                       \
            BODY                                                                                             \
        }                                                                                                    \
        T5_ADVANCE();                                                                                        \
        LDS_WAIT_ALL(); /* nothing of this block is still being read when the next barrier is passed */      \
    }

/* NCW = consumer waves: 8 (768 threads, the library's own launch) or 4 (512 threads: a wave then runs
 * two of the eight consumers' shares one after the other in every block, for callers whose launch shape
 * is fixed at 512 threads). The body takes its LDS as a pointer so that it can also sit in a kernel
 * with static LDS. */
/* NG: 16-row groups a tile may hold, 8 or 9 (see t5_nine_groups below). */
/* A16: `a` holds bf16 rows [..][K] (no activation scales) and a block is 64 k: the bf16-activation arms
 * (block-fp8 weights: ops 85 / 86 arm 0; per-channel fp8 weights: ops 65 / 66). */
/* AM: what the operands are. 0: e4m3 rows with scales (the W8A8 pairs); 1 (A16): bf16 rows, fp8 weights; 3 (A16 and
 * W16): bf16 rows and bf16 weights, no scales at all (ops 85 / 86 arm 0 at enc 0 over wtab[E][3], ops 75 / 76 over the
 * fused table with PC as the layout switch); 2 (A4): mxfp4 rows
 * [..][K / 2] with E8M0 rows [..][K / 32] against mxfp4 weights, a block is 256 k, scales applied by the
 * matrix instruction (ops 85 / 86 with enc 2, arm 0). */
template <bool GLU, bool PC, uint32_t NCW, int NG = 8, int AM = 0>
__device__ __forceinline__ void t5_body(const GroupW8A8& g, uint8_t* lds_raw) {
    static_assert(NG == 8 || NG == 9, "a tile is eight or nine 16-row groups");
    constexpr bool A16 = AM == 1 || AM == 3 || AM == 4, A4 = AM == 2, W16 = AM == 3, W4 = AM == 4;
    constexpr bool W8 = A16 && !W16 && !W4; /* fp8 weight rows under bf16 rows: 64 bytes per block */
    constexpr bool W64 = W8 || W4;           /* weight rows of 64 bytes per block (16 rows per direct load) */
    constexpr bool NOPAD = W16 || W4;        /* forms whose GLU writes live rows only, as the streaming kernels of those encodings do */
    static_assert(!(W16 || W4) || NG == 8, "the bf16- and mxfp4-weight forms under bf16 rows have 128-row tiles");
    static_assert(!W4 || !PC, "mxfp4 weights come through wtab / stab [E][3]");
    static_assert(!A4 || (NG == 8 && !PC), "the fp4 arm has 128-row tiles and no per-channel mode");
    typedef typename std::conditional<A4, T5LdsA4, typename std::conditional<W4, T5LdsW4, T5Lds>::type>::type Lds;
    Lds& L = *(Lds*)lds_raw;
    constexpr uint32_t BN = GLU ? 128u : 256u; /* output channels per tile */
    constexpr uint32_t NTHR = (NCW + 4u) * 64u, SUBS = 8u / NCW;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wv = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const bool loader = wv >= NCW;
    const uint32_t cw = loader ? wv - NCW : wv; /* loader index 0..3, or consumer wave index */
    const uint32_t NT = (g.N + BN - 1u) / BN;
    const uint32_t r16 = lane & 15u, q = lane >> 4;

    if (!form_is_mine(g)) return; /* the device-side choice named the streaming form: the same in every workgroup */
    /* rows a tile may hold */
    const uint32_t cap = 16u * (uint32_t)NG;
    /* ---- tile directory: inclusive prefix of ceil(cnt / cap) over experts, in LDS (the scan
     *      scratch borrows the ring, which is idle here) ---- */
    {
        uint32_t* scan = (uint32_t*)&L.a[0][0];
        uint32_t carry = 0;
        for (uint32_t e0 = 0; e0 < g.E; e0 += NTHR) {
            const uint32_t e = e0 + tid;
            const uint32_t t = e < g.E ? ((uint32_t)g.meta[g.E + e] + cap - 1u) / cap : 0u;
            scan[tid] = t;
            __syncthreads();
            for (uint32_t o = 1; o < NTHR; o <<= 1) {
                const uint32_t v = tid >= o ? scan[tid - o] : 0u;
                __syncthreads();
                scan[tid] += v;
                __syncthreads();
            }
            if (e < g.E) L.prefix[e] = (uint16_t)(carry + scan[tid]);
            carry += scan[NTHR - 1u];
            __syncthreads();
        }
        /* the directory holds 16-bit counts: a batch with more row tiles than that (some 8 million routed rows)
         * is not served. The launchers refuse it where the host knows the row count; a count only the device
         * knows ends every workgroup here, before anything is written. */
        if (carry > T5_MAX_ROW_TILES) return;
    }
    if (GLU && !PC && g.out_bf16) {
        /* bf16 intermediate: the padded rows of an expert whose gate or up weights are not resident are
         * zero-filled (the tile walk below skips such an expert), as in the streaming form */
        for (uint32_t e = blockIdx.x; e < g.E; e += gridDim.x) {
            if (g.wtab[(size_t)e * 3u] != 0ull && g.wtab[(size_t)e * 3u + 1u] != 0ull) continue;
            const uint32_t cnt = (uint32_t)g.meta[g.E + e], r0 = (uint32_t)g.meta[e];
            const uint32_t padded = ((cnt + PLOW_MPF_BM - 1u) / PLOW_MPF_BM) * PLOW_MPF_BM;
            for (uint32_t i = tid; i < padded * (g.N / 4u); i += NTHR)
                *(uint2*)((bf16_t*)g.out + (size_t)(r0 + i / (g.N / 4u)) * g.N + (i % (g.N / 4u)) * 4u) = make_uint2(0u, 0u);
        }
    }
    const uint32_t total = (uint32_t)L.prefix[g.E - 1u] * NT;
    const uint32_t K = g.K, KB = K / (W4 ? 128u : A16 ? 64u : A4 ? 256u : 128u); /* blocks of the K loop */
    const uint32_t KS = K / 128u;                                    /* weight block scales along K */
    const uint32_t KA = A16 ? 2u * K : A4 ? K / 2u : K;              /* bytes of a token row */
    const uint32_t KW = (A4 || W4) ? K / 2u : W16 ? 2u * K : K;      /* bytes of a weight row */
    const uint32_t K32 = K / 32u;                                    /* A4, W4: E8M0 bytes of a row */
    (void)KS, (void)K32;
    const uint32_t a_base = lds_off(&L.a[0][0]), w_base = lds_off(&L.w[0][0]);
    uint32_t s_base = 0, c_base = 0, ts_base = 0, wsb_base = 0;
    if constexpr (A4) {
        ts_base = lds_off(&L.ts[0][0][0]), wsb_base = lds_off(&L.ws[0][0][0]);
    } else if constexpr (W4) {
        wsb_base = lds_off(&L.ws[0][0][0]);
    } else {
        s_base = lds_off(&L.as[0][0]), c_base = lds_off(&L.wsc[0][0][0]);
    }
    (void)s_base, (void)c_base, (void)ts_base, (void)wsb_base;
    /* consumer: this lane's operand pieces 2q, 2q + 1 of row (16 * group + r16) */
    const uint32_t sw = lds_swz8(r16);
    const uint32_t op_lo = r16 * 128u + (((2u * q) ^ sw) << 4), op_hi = r16 * 128u + (((2u * q + 1u) ^ sw) << 4);
    /* A16: this lane's 16-byte token pieces q and 4 + q (k 8q.. and 32 + 8q.. of the 64-k block), and its
     * 8-byte weight pieces of row r16 */
    const uint32_t opb0 = r16 * 128u + ((q ^ sw) << 4), opb1 = r16 * 128u + (((4u + q) ^ sw) << 4);
    const uint32_t swa = ((r16 >> 2) & 3u) * 2u;
    const uint32_t opa0 = r16 * 64u + ((q ^ swa) << 3), opa1 = r16 * 64u + (((4u + q) ^ swa) << 3);
    /* W4: this lane's token pieces 4q .. 4q + 3 of a 256-byte row */
    const uint32_t sx = lds_swz16(r16);
    const uint32_t xo0 = ((4u * q) ^ sx) << 4, xo1 = ((4u * q + 1u) ^ sx) << 4, xo2 = ((4u * q + 2u) ^ sx) << 4, xo3 = ((4u * q + 3u) ^ sx) << 4;
    (void)op_lo, (void)op_hi, (void)opb0, (void)opb1, (void)opa0, (void)opa1, (void)xo0, (void)xo1, (void)xo2, (void)xo3;

    /* Workgroup w runs on XCD w % 8 (round-robin dispatch), and each XCD has its own L2. The logical
     * index below makes the 32 workgroups of one XCD take 32 consecutive tiles of every sweep. Inside an expert
     * the tiles go by blocks of up to T5_ROW_BLOCK row tiles, and inside a block the row tiles of one channel
     * tile are neighbours: wherever the 32 start, they hold a few channel tiles, each with all the block's row
     * tiles, so that a weight row crosses the fabric once for the block (the row tiles of an expert are equally
     * long and walk K in step) and a token row once per 32 / block tiles of its channel tiles. Row-tile-major
     * order, 16 channel tiles of one row tile after the other, read an expert's weights once per row tile
     * whenever its tiles did not start on a multiple of 32. */
    const uint32_t G = gridDim.x;
    const uint32_t wg = (G % 8u == 0u) ? (blockIdx.x % 8u) * (G / 8u) + blockIdx.x / 8u : blockIdx.x;
    const uint32_t nblk = g.N / 128u;
    struct Tile {
        uint32_t e, nt, r0, rows;
        uint32_t single;   /* the expert's only row tile: its weight rows are read once */
        uint64_t wp0, wp1; /* weight rows (GLU block mode: gate, up) */
        uint64_t sp0, sp1; /* block mode: their scale tables */
    };
    /* every value is the same in all lanes (made explicit with readfirstlane so that what is indexed
     * by them is read with scalar loads) */
    auto locate = [&](uint32_t tile) -> Tile {
        const uint32_t mt_global = tile / NT;
        uint32_t lo = 0, hi = g.E - 1u; /* first expert whose inclusive prefix exceeds mt_global */
        while (lo < hi) {
            const uint32_t mid = (lo + hi) >> 1;
            if ((uint32_t)L.prefix[mid] > mt_global) hi = mid; else lo = mid + 1u;
        }
        Tile t;
        t.e = (uint32_t)__builtin_amdgcn_readfirstlane((int)lo);
        const uint32_t pbase = t.e ? (uint32_t)L.prefix[t.e - 1u] : 0u, Me = (uint32_t)L.prefix[t.e] - pbase;
        const uint32_t idx = tile - pbase * NT;
        uint32_t mt_v, nt_v;
        {
            constexpr uint32_t T5_ROW_BLOCK = (W4 || PC || A16) ? 1u : T5_RB_BLOCK;
            const uint32_t full = (Me / T5_ROW_BLOCK) * T5_ROW_BLOCK; /* row tiles in whole blocks */
            if (idx < full * NT) {
                const uint32_t rb = idx / (T5_ROW_BLOCK * NT), rem = idx % (T5_ROW_BLOCK * NT);
                mt_v = rb * T5_ROW_BLOCK + rem % T5_ROW_BLOCK, nt_v = rem / T5_ROW_BLOCK;
            } else {
                const uint32_t rem = idx - full * NT, mb = Me - full; /* the last, shorter block */
                mt_v = full + rem % mb, nt_v = rem / mb;
            }
        }
        const uint32_t mt = (uint32_t)__builtin_amdgcn_readfirstlane((int)mt_v);
        t.nt = (uint32_t)__builtin_amdgcn_readfirstlane((int)nt_v);
        /* meta and the pointer table were written by earlier kernels and the expert index is the same in every
         * lane: read through the constant address space these are scalar loads, which a loader's direct loads in
         * flight do not have to be waited for (a vector load's result would drain them, once per tile) */
        const auto* const meta_c = (const __attribute__((address_space(4))) int32_t*)g.meta;
        const auto* const wtab_c = (const __attribute__((address_space(4))) uint64_t*)g.wtab;
        const uint32_t cnt = (uint32_t)meta_c[g.E + t.e];
        /* nine-group kernels split the expert's rows evenly over its Me = ceil(cnt / cap) tiles, in whole 16-row
         * groups: a tile takes nine groups only where that saves a tile; eight-group kernels fill 128-row tiles
         * and leave the rest to the last one */
        const uint32_t Mu = (uint32_t)__builtin_amdgcn_readfirstlane((int)Me);
        t.single = Mu == 1u ? 1u : 0u;
        const uint32_t h = NG == 8 ? 128u : (((cnt + Mu - 1u) / Mu + 15u) / 16u) * 16u; /* <= cap since cnt <= cap * Me */
        t.r0 = (uint32_t)meta_c[t.e] + mt * h;
        t.rows = cnt - mt * h < h ? cnt - mt * h : h; /* live rows of the tile */
        /* block mode: {gate, up, down} tables; per-channel mode: {gate_up fused [2N][K], down} */
        t.wp0 = PC ? wtab_c[(size_t)t.e * 2u + (GLU ? 0u : 1u)] : wtab_c[(size_t)t.e * 3u + (GLU ? 0u : 2u)];
        t.wp1 = (GLU && !PC) ? wtab_c[(size_t)t.e * 3u + 1u] : t.wp0;
        if (t.wp1 == 0ull) t.wp0 = 0ull; /* gate without up: not resident */
        t.sp0 = t.sp1 = 0ull;
        if (!PC && !W16) {
            const auto* const stab_c = (const __attribute__((address_space(4))) uint64_t*)g.stab;
            t.sp0 = stab_c[(size_t)t.e * 3u + (GLU ? 0u : 2u)];
            t.sp1 = GLU ? stab_c[(size_t)t.e * 3u + 1u] : t.sp0;
        }
        return t;
    };
    /* this workgroup's next tile at or after `from` whose expert is resident (`total` if none); loaders
     * and consumers walk the same sequence */
    auto next_tile = [&](uint32_t from, Tile& t) -> uint32_t {
        for (uint32_t tile = from; tile < total; tile += G) {
            t = locate(tile);
            if (t.wp0 != 0ull) return tile;
        }
        return total;
    };

    /* Barrier protocol, identical in both roles: per tile, one barrier per 128-k block ("block kb of
     * this tile is in LDS; everyone is done with the block before it") and one after the last block
     * (GLU amax exchange). Ring slots and the L.wsc half alternate over a count that runs across
     * tiles, so the loaders work ahead into the next tile while the consumers finish this one. */
    if (loader) {
        /* ================= loaders ================= */
        /* a direct load covers 8 rows x 128 B: lane -> (row l >> 3, LDS piece l & 7) */
        const uint32_t lr = lane >> 3, p = lane & 7u;
        struct Src {
            /* per-lane 32-bit byte offsets from uniform bases: the loads take (scalar base + k offset,
             * vector offset) */
            uint32_t aoff[8], woff[8], sstep;
            uint32_t nine; /* this loader has a ninth-group load in this tile (loaders 0 and 1, tiles of more than 128 rows) */
            /* A4: this lane's dword of the E8M0 rows: token row 32 * cw + l / 2 and weight rows 64 * cw + 32 * j + l / 2 */
            const uint8_t *tsp, *wsp[2];
            const float* ssrc;
            const uint8_t *W0, *W1;
            uint32_t nt; /* weight rows non-temporal: asked for by the launch and the expert has one row tile */
        };
        const uint8_t* const A0 = (const uint8_t*)g.a;
        const bool w_nt = __builtin_amdgcn_readfirstlane((int)g.w_nt) != 0;
        /* Set-up of a tile's sources in two halves, so that its loads (row -> token, scales) are in
         * flight while the loader keeps feeding the tile before: fetch() only issues loads, finish()
         * uses them a few blocks later. Rows below the live count always hold a token. */
        struct Pre {
            uint32_t tok[8], stok, eidx;
            uint32_t tsrow; /* A4: the row of `a` whose scale dword this lane loads */
            float w0, w1, egate;
        };
        auto fetch = [&](const Tile& t, Pre& P) {
            const uint32_t r0 = t.r0, rows = t.rows, nt = t.nt;
#pragma unroll
            for (uint32_t i = 0; i < 8u; i++) { /* token rows 32 * cw + 8 * i + lr, and for loaders 0 and 1 rows
                                                 * 128 + 8 * cw + lr of the ninth group; a pad row reads the first row.
                                                 * W4 (256-byte rows, four to a load): rows 32 * cw + 4 * i + lane / 16 */
                if (!W4 && i >= 5u) { P.tok[i] = 0u; continue; }
                if (!W4 && i == 4u && cw >= 2u) { P.tok[i] = 0u; continue; }
                const uint32_t row = W4 ? 32u * cw + 4u * i + (lane >> 4) : i < 4u ? 32u * cw + 8u * i + lr : 128u + 8u * cw + lr;
                const uint32_t ar = r0 + (row < rows ? row : 0u);
                if (GLU) {
                    P.tok[i] = g.row_token[ar];
                } else if (g.a_slots && (!PC || A16)) { /* rows stored by routing slot: read the slot's row */
                    const uint32_t slot = g.row_partidx[ar];
                    P.tok[i] = slot < g.a_slots ? slot : 0u;
                } else {
                    P.tok[i] = ar;
                }
            }
            {
                const uint32_t row = (cw < 3u ? cw : 0u) * 64u + lane; /* the row whose activation scale this lane loads */
                /* per-channel mode has one activation scale per row, applied in the epilogue: its ring slot
                 * carries zeros */
                /* the fp4 arm's GLU skips the rows its row_partidx operand marks unused */
                P.eidx = row < rows ? ((GLU && !A4) ? g.row_token[r0 + row] : g.row_partidx[r0 + row]) : PLOW_EXPERT_UNUSED;
                P.stok = (PC || A16 || A4) ? PLOW_EXPERT_UNUSED : P.eidx;
                P.egate = (!GLU && row < rows) ? g.row_gate[r0 + row] : 0.0f;
            }
            /* weight block scales of the tile: GLU gate | up of channel block nt; DOWN blocks 2nt, 2nt + 1 */
            if (A4) { /* the token row 32 * cw + lane / 2 of the tile, as a row of `a` */
                const uint32_t row = 32u * cw + (lane >> 1);
                const uint32_t ar = r0 + (row < rows ? row : 0u);
                if (GLU) {
                    const uint32_t tk = g.row_token[ar];
                    P.tsrow = (tk == PLOW_EXPERT_UNUSED || (g.T != 0u && tk >= g.T)) ? 0u : tk;
                } else {
                    P.tsrow = ar;
                }
            }
            P.w0 = P.w1 = 0.0f;
            if (!PC && !A4 && !W16 && !W4) {
                const float* S0 = (const float*)(uintptr_t)t.sp0;
                const float* S1 = (const float*)(uintptr_t)t.sp1;
                const uint32_t nb0 = GLU ? nt : 2u * nt, nb1 = GLU ? nt : (2u * nt + 1u < nblk ? 2u * nt + 1u : 2u * nt);
                const uint32_t i = tid - NCW * 64u; /* 0..255 over the four loaders; KS <= 128 */
                P.w0 = i < KS ? S0[(size_t)nb0 * KS + i] : 0.0f;
                P.w1 = i < KS ? S1[(size_t)nb1 * KS + i] : 0.0f;
            }
        };
        auto finish = [&](const Tile& t, const Pre& P, uint32_t par, Src& S) {
            const uint32_t r0 = t.r0, rows = t.rows, nt = t.nt;
            S.W0 = (const uint8_t*)(uintptr_t)t.wp0;
            S.nt = (w_nt && t.single) ? 1u : 0u;
            S.nine = (cw < 2u && rows > 128u) ? 1u : 0u;
            S.W1 = !GLU ? S.W0 : PC ? S.W0 + (size_t)g.N * KW /* up rows follow the N gate rows */
                               : (const uint8_t*)(uintptr_t)t.wp1;
#pragma unroll
            for (uint32_t i = 0; i < 8u; i++) {
                if (!W4 && i >= 5u) { S.aoff[i] = 0u; continue; }
                if (W4) { /* 256-byte rows: lane -> (row lane / 16 of the load's four, piece lane % 16) */
                    const uint32_t row4 = 32u * cw + 4u * i + (lane >> 4);
                    const uint32_t src4 = (GLU && (P.tok[i] == PLOW_EXPERT_UNUSED || (g.T != 0u && P.tok[i] >= g.T))) ? 0u : P.tok[i];
                    S.aoff[i] = src4 * KA + (((lane & 15u) ^ lds_swz16(row4)) << 4);
                    continue;
                }
                const uint32_t row = i < 4u ? 32u * cw + 8u * i + lr : 128u + 8u * (cw & 1u) + lr;
                /* a pad row, or (where the launch states the rows of `a` in g.T: staged rows end there) a token past the rows that exist, reads row 0 */
                const uint32_t src = (GLU && (P.tok[i] == PLOW_EXPERT_UNUSED || (g.T != 0u && P.tok[i] >= g.T))) ? 0u : P.tok[i];
                S.aoff[i] = src * KA + ((p ^ lds_swz8(row)) << 4);
            }
#pragma unroll
            for (uint32_t i = 0; i < 8u; i++) { /* LDS weight rows R = 64 * cw + 8 * i + lr: consumer R / 32, group (R / 16) & 1 */
                if (W64 && i >= 4u) { S.woff[i] = 0u; continue; }
                /* 64-byte weight rows (fp8 or mxfp4 under bf16 rows): a load covers 16 rows x 64 B, lane -> (row l >> 2, 16-byte slot l & 3) */
                const uint32_t R = W64 ? 64u * cw + 16u * i + (lane >> 2) : 64u * cw + 8u * i + lr;
                uint32_t ch;
                if (GLU) {
                    ch = nt * 128u + 16u * (R >> 5) + (R & 15u);
                } else {
                    ch = nt * 256u + R;
                    if (ch >= g.N) ch = 0; /* past the last channel: any valid row, never stored */
                }
                S.woff[i] = W64 ? ch * KW + (((lane & 3u) ^ ((R >> 2) & 3u)) << 4) : ch * KW + ((p ^ lds_swz8(R)) << 4);
            }
            /* activation scale of row 64 * cw + lane (loader 3 repeats loader 0's 64 values); a pad row
             * reads tilep[0], which is always 0 */
            {
                const uint32_t row = (cw < 3u ? cw : 0u) * 64u + lane;
                const bool ok = P.stok != PLOW_EXPERT_UNUSED && !(GLU && g.T != 0u && P.stok >= g.T); /* a token past the stated rows: zero scale */
                if (GLU) {
                    S.ssrc = ok ? g.a_scale + P.stok : (const float*)(g.meta + 2u * g.E);
                    S.sstep = ok ? g.pitch : 0u;
                } else if (!PC && !A16 && g.a_slots) { /* scales [KB][a_slots], by slot */
                    const bool in = ok && P.stok < g.a_slots;
                    S.ssrc = in ? g.a_scale + P.stok : (const float*)(g.meta + 2u * g.E);
                    S.sstep = in ? g.a_slots : 0u;
                } else {
                    S.ssrc = ok ? g.a_scale + (size_t)(r0 + row) * KB : (const float*)(g.meta + 2u * g.E);
                    S.sstep = ok ? 1u : 0u;
                }
            }
            if constexpr (W4) { /* the four E8M0 bytes of weight row 64 * cw + lane per block, a dword per lane */
                const uint32_t R = 64u * cw + lane;
                uint32_t ch = GLU ? nt * 128u + 16u * (R >> 5) + (R & 15u) : nt * 256u + R;
                if (ch >= g.N) ch = 0;
                S.wsp[0] = ((GLU && (R & 16u)) ? (const uint8_t*)(uintptr_t)t.sp1 : (const uint8_t*)(uintptr_t)t.sp0) + (size_t)ch * K32;
                S.wsp[1] = S.wsp[0];
                S.tsp = nullptr;
            } else if constexpr (A4) {
                S.tsp = g.a_e8m0 + (size_t)P.tsrow * K32 + (lane & 1u) * 4u;
                const uint8_t* const SW0 = (const uint8_t*)(uintptr_t)t.sp0;
                const uint8_t* const SW1 = (const uint8_t*)(uintptr_t)t.sp1;
#pragma unroll
                for (uint32_t j = 0; j < 2u; j++) {
                    const uint32_t R = 64u * cw + 32u * j + (lane >> 1);
                    uint32_t ch = GLU ? nt * 128u + 16u * (R >> 5) + (R & 15u) : nt * 256u + R;
                    if (ch >= g.N) ch = 0;
                    S.wsp[j] = ((GLU && (R & 16u)) ? SW1 : SW0) + (size_t)ch * K32 + (lane & 1u) * 4u;
                }
            } else if constexpr (!W4) {
                const uint32_t i = tid - NCW * 64u;
                if (i < KS) {
                    L.wsc[par][0][i] = P.w0;
                    L.wsc[par][1][i] = P.w1;
                }
            }
            /* what the consumers' epilogue needs per row, so that it does not start with a round trip to
             * memory: loaders 0, 1 and 2 hold rows 0..63, 64..127 and 128..191 */
            if (cw < 3u) {
                L.epi_idx[par][cw * 64u + lane] = P.eidx;
                if (!GLU) L.epi_gate[par][cw * 64u + lane] = P.egate;
            }
        };
        auto issue = [&](const Src& S, uint32_t kb, uint32_t st) {
            if constexpr (A4) { /* eight E8M0 bytes per row and block, a dword per lane */
                __builtin_amdgcn_global_load_lds((const void*)(S.tsp + (size_t)kb * 8u), (lds_void*)&L.ts[st][32u * cw][0], 4, 0, 0);
                __builtin_amdgcn_global_load_lds((const void*)(S.wsp[0] + (size_t)kb * 8u), (lds_void*)&L.ws[st][64u * cw][0], 4, 0, 0);
                __builtin_amdgcn_global_load_lds((const void*)(S.wsp[1] + (size_t)kb * 8u), (lds_void*)&L.ws[st][64u * cw + 32u][0], 4, 0, 0);
            } else if constexpr (W4) {
                __builtin_amdgcn_global_load_lds((const void*)(S.wsp[0] + (size_t)kb * 4u), (lds_void*)&L.ws[st][64u * cw][0], 4, 0, 0);
            } else if constexpr (!A16) {
                __builtin_amdgcn_global_load_lds((const void*)(S.ssrc + (size_t)kb * S.sstep),
                                                 (lds_void*)&L.as[st][(cw < 3u ? cw : 0u) * 64u], 4, 0, 0);
            }
            const uint8_t* const ak = A0 + (size_t)kb * (W4 ? 256u : 128u);
            const uint8_t* const wk0 = S.W0 + (size_t)kb * (W64 ? 64u : 128u);
            const uint8_t* const wk1 = S.W1 + (size_t)kb * (W64 ? 64u : 128u);
            if constexpr (W4) {
#pragma unroll
                for (uint32_t i = 0; i < 8u; i++) /* four token rows of 256 bytes each */
                    __builtin_amdgcn_global_load_lds((const void*)(ak + S.aoff[i]),
                                                     (lds_void*)&L.a[st][(32u * cw + 4u * i) * 256u], 16, 0, 0);
            } else {
#pragma unroll
                for (uint32_t i = 0; i < 4u; i++)
                    __builtin_amdgcn_global_load_lds((const void*)(ak + S.aoff[i]),
                                                     (lds_void*)&L.a[st][(32u * cw + 8u * i) * 128u], 16, 0, 0);
                if (S.nine) /* the ninth group's rows */
                    __builtin_amdgcn_global_load_lds((const void*)(ak + S.aoff[4]),
                                                     (lds_void*)&L.a[st][(128u + 8u * cw) * 128u], 16, 0, 0);
            }
            if (W64) {
#pragma unroll
                for (uint32_t i = 0; i < 4u; i++) /* 16 weight rows of 64 bytes each */
                    __builtin_amdgcn_global_load_lds((const void*)(((GLU && (i & 1u)) ? wk1 : wk0) + S.woff[i]),
                                                     (lds_void*)&L.w[st][(64u * cw + 16u * i) * 64u], 16, 0, 0);
            } else {
                if (S.nt) { /* the same in every lane; the cache policy is an immediate of the instruction */
#pragma unroll
                    for (uint32_t i = 0; i < 8u; i++)
                        __builtin_amdgcn_global_load_lds((const void*)(((GLU && (i & 2u)) ? wk1 : wk0) + S.woff[i]),
                                                         (lds_void*)&L.w[st][(64u * cw + 8u * i) * 128u], 16, 0, LOAD_NT);
                } else {
#pragma unroll
                    for (uint32_t i = 0; i < 8u; i++)
                        __builtin_amdgcn_global_load_lds((const void*)(((GLU && (i & 2u)) ? wk1 : wk0) + S.woff[i]),
                                                         (lds_void*)&L.w[st][(64u * cw + 8u * i) * 128u], 16, 0, 0);
                }
            }
        };
        Tile tcur, tnxt;
        Src cur, nxt;
        Pre pre;
        uint32_t tile = next_tile(wg, tcur), par = 0, slot = 0; /* slot of the current tile's block 0 */
        if (tile < total) {
            fetch(tcur, pre);
            finish(tcur, pre, 0u, cur);
            issue(cur, 0u, 0u);
            issue(cur, 1u, 1u);
        }
        /* the next tile's sources are needed when block KB - 2 of this tile has been passed: they are
         * fetched during block 0 and finished during block KB - 3 (fetched before the loop and finished
         * right after the first barrier if K has two blocks) */
        const bool early = KB < 3u;
        while (tile < total) {
            const uint32_t ntile = next_tile(tile + G, tnxt);
            const bool more = ntile < total;
            if (more && early) fetch(tnxt, pre);
            uint32_t st = slot; /* slot of block kb */
            for (uint32_t kb = 0; kb < KB; kb++) {
                /* loads return in order: block kb has landed once at most the next block's loads (of this
                 * tile or the next) are outstanding. After the barrier the consumers are done with the
                 * block before kb, whose slot takes the block two ahead. */
                if (kb + 1u < KB || more) { /* the loads that may stay outstanding are those of the block after kb */
                    if (W16) { /* 4 token-row and 8 weight-row loads, no scales */
                        LOADER_BARRIER(12);
                    } else if (W4) { /* 1 scale, 8 token-row, 4 weight-row loads */
                        LOADER_BARRIER(13);
                    } else if (A16) { /* 4 token-row and 4 weight-row loads, no scales */
                        if (kb + 1u < KB ? cur.nine : nxt.nine) LOADER_BARRIER(9); else LOADER_BARRIER(8);
                    } else if (A4) { /* 3 scale, 4 token-row, 8 weight-row loads */
                        LOADER_BARRIER(15);
                    } else {
                        if (kb + 1u < KB ? cur.nine : nxt.nine) LOADER_BARRIER(T5_NLOAD + 1); else LOADER_BARRIER(T5_NLOAD);
                    }
                } else {
                    LOADER_BARRIER(0);
                }
                const uint32_t st2 = st >= 1u ? st - 1u : 2u; /* (st + 2) % 3 */
                /* not before this barrier: until it, the consumers may still be in the epilogue of the tile
                 * before, reading the L.epi_* half that finish() overwrites */
                if (more && early && kb == 0u) finish(tnxt, pre, par ^ 1u, nxt);
                /* the next tile's set-up loads go out before this block's direct loads: behind them they would be
                 * the youngest loads at the next barrier, whose count then makes it wait for as many loads of the
                 * block after (in practice for that block: 1.3 us per tile) */
                if (more && !early && kb == 0u) fetch(tnxt, pre);
                if (kb + 2u < KB) issue(cur, kb + 2u, st2);
                else if (more) issue(nxt, kb + 2u - KB, st2);
                st = st == 2u ? 0u : st + 1u;
                if (more && !early && kb == KB - 3u) finish(tnxt, pre, par ^ 1u, nxt);
            }
            WG_BARRIER(); /* after the last block (the consumers' amax exchange) */
            slot = st;
            cur = nxt, tcur = tnxt, tile = ntile, par ^= 1u;
        }
    } else {
        /* ================= consumers ================= */
        /* Consumer wave w runs the shares of the logical consumers SUBS * w .. SUBS * w + SUBS - 1 (one
         * with eight consumer waves, two with four): `cw` below is the logical consumer. */
        Tile t;
        uint32_t par = 0, st = 0;
        const uint32_t cw0 = SUBS * cw;
        for (uint32_t tile = next_tile(wg, t); tile < total; tile = next_tile(tile + G, t), par ^= 1u) {
            const uint32_t r0 = t.r0, rows = t.rows, nt = t.nt;
            const uint32_t ngrp = (rows + 15u) / 16u; /* live 16-row groups */
            /* DOWN: N may end mid-tile (N is a multiple of 128, so a wave's consumers are in or out together) */
            const bool wave_on = (GLU ? nt * 128u + 16u * cw0 : nt * 256u + 32u * cw0) < g.N;
            const uint32_t ngrp_w = wave_on ? ngrp : 0u;
            v4f accs[SUBS][NG][2];
#pragma unroll
            for (uint32_t sub = 0; sub < SUBS; sub++)
#pragma unroll
                for (int rg = 0; rg < NG; rg++)
#pragma unroll
                    for (int x = 0; x < 2; x++) accs[sub][rg][x] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
            /* One form of the block loop per count of live row groups: each is straight-line code. The
             * wait the compiler can see (everything the LDS was asked for has arrived) keeps it from
             * placing waits of its own inside the loops, whose LDS reads it does not see. */
            __builtin_amdgcn_s_waitcnt(0xc07f); /* lgkmcnt(0) */
            if constexpr (A4) {
                switch (ngrp_w) {
                    case 8u: { T5_RUN_BLOCKS(T5Q_BLOCK_N(8)) } break;
                    case 7u: { T5_RUN_BLOCKS(T5Q_BLOCK_N(7)) } break;
                    case 6u: { T5_RUN_BLOCKS(T5Q_BLOCK_N(6)) } break;
                    case 5u: { T5_RUN_BLOCKS(T5Q_BLOCK_N(5)) } break;
                    case 4u: { T5_RUN_BLOCKS(T5Q_BLOCK_N(4)) } break;
                    case 3u: { T5_RUN_BLOCKS(T5Q_BLOCK_N(3)) } break;
                    case 2u: { T5_RUN_BLOCKS(T5Q_BLOCK_N(2)) } break;
                    case 1u: { T5_RUN_BLOCKS(T5Q_BLOCK_N(1)) } break;
                    default: { T5_RUN_BLOCKS() } break;
                }
            } else if constexpr (W4) {
                switch (ngrp_w) {
                    case 8u: { T5_RUN_BLOCKS(T5X_BLOCK_N(8)) } break;
                    case 7u: { T5_RUN_BLOCKS(T5X_BLOCK_N(7)) } break;
                    case 6u: { T5_RUN_BLOCKS(T5X_BLOCK_N(6)) } break;
                    case 5u: { T5_RUN_BLOCKS(T5X_BLOCK_N(5)) } break;
                    case 4u: { T5_RUN_BLOCKS(T5X_BLOCK_N(4)) } break;
                    case 3u: { T5_RUN_BLOCKS(T5X_BLOCK_N(3)) } break;
                    case 2u: { T5_RUN_BLOCKS(T5X_BLOCK_N(2)) } break;
                    case 1u: { T5_RUN_BLOCKS(T5X_BLOCK_N(1)) } break;
                    default: { T5_RUN_BLOCKS() } break;
                }
            } else if constexpr (W16) {
                switch (ngrp_w) {
                    case 8u: { T5_RUN_BLOCKS(T5W_BLOCK_N(8)) } break;
                    case 7u: { T5_RUN_BLOCKS(T5W_BLOCK_N(7)) } break;
                    case 6u: { T5_RUN_BLOCKS(T5W_BLOCK_N(6)) } break;
                    case 5u: { T5_RUN_BLOCKS(T5W_BLOCK_N(5)) } break;
                    case 4u: { T5_RUN_BLOCKS(T5W_BLOCK_N(4)) } break;
                    case 3u: { T5_RUN_BLOCKS(T5W_BLOCK_N(3)) } break;
                    case 2u: { T5_RUN_BLOCKS(T5W_BLOCK_N(2)) } break;
                    case 1u: { T5_RUN_BLOCKS(T5W_BLOCK_N(1)) } break;
                    default: { T5_RUN_BLOCKS() } break;
                }
            } else if constexpr (A16) {
                switch (ngrp_w) {
                    case 9u: if constexpr (NG == 9) { T5_RUN_BLOCKS(T5A_BLOCK_N(9)) } break;
                    case 8u: { T5_RUN_BLOCKS(T5A_BLOCK_N(8)) } break;
                    case 7u: { T5_RUN_BLOCKS(T5A_BLOCK_N(7)) } break;
                    case 6u: { T5_RUN_BLOCKS(T5A_BLOCK_N(6)) } break;
                    case 5u: { T5_RUN_BLOCKS(T5A_BLOCK_N(5)) } break;
                    case 4u: { T5_RUN_BLOCKS(T5A_BLOCK_N(4)) } break;
                    case 3u: { T5_RUN_BLOCKS(T5A_BLOCK_N(3)) } break;
                    case 2u: { T5_RUN_BLOCKS(T5A_BLOCK_N(2)) } break;
                    case 1u: { T5_RUN_BLOCKS(T5A_BLOCK_N(1)) } break;
                    default: { T5_RUN_BLOCKS() } break;
                }
            } else {
            switch (ngrp_w) {
                    case 9u: if constexpr (NG == 9) { T5_RUN_BLOCKS(T5_BLOCK_N(9)) } break;
                    case 8u: { T5_RUN_BLOCKS(T5_BLOCK_N(8)) } break;
                    case 7u: { T5_RUN_BLOCKS(T5_BLOCK_N(7)) } break;
                    case 6u: { T5_RUN_BLOCKS(T5_BLOCK_N(6)) } break;
                    case 5u: { T5_RUN_BLOCKS(T5_BLOCK_N(5)) } break;
                    case 4u: { T5_RUN_BLOCKS(T5_BLOCK_N(4)) } break;
                    case 3u: { T5_RUN_BLOCKS(T5_BLOCK_N(3)) } break;
                    case 2u: { T5_RUN_BLOCKS(T5_BLOCK_N(2)) } break;
                    case 1u: { T5_RUN_BLOCKS(T5_BLOCK_N(1)) } break;
                    default: { T5_RUN_BLOCKS() } break;
                }

            }

            /* ---- epilogue. Lane: row = 16 * rg + r16; GLU channel = ch0 + 4q + i with gate in weight
             *      group 0 and up in group 1; DOWN channel = ch0 + 16 * x + 4q + i ---- */
            const uint32_t stl = st >= 1u ? st - 1u : 2u; /* the ring stage the tile has just left */
            if constexpr (A4 && GLU) {
                /* SwiGLU in f32, then every (row, 32 channels) block to mxfp4 with its E8M0 byte (plow
                 * runtime/amd/op_moe.h:4595-4632). A block is the 16 channels of consumer 2j and those of
                 * consumer 2j + 1: the row maxima meet as in the fp8 epilogue below. */
                float v[SUBS][NG][4];
                auto red = [&](uint32_t x) -> float* { return (float*)&L.w[stl][x * (32u * 128u)]; };
#pragma unroll
                for (uint32_t sub = 0; sub < SUBS; sub++) {
                    const uint32_t cw = cw0 + sub;
                    v4f(&acc)[NG][2] = accs[sub];
#pragma unroll
                    for (int rg = 0; rg < NG; rg++) {
                        float m = 0.0f;
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            v[sub][rg][i] = moe_glu(acc[rg][0][i], acc[rg][1][i], g.act, g.f0, g.f1);
                            m = fmaxf(m, fabsf(v[sub][rg][i]));
                        }
                        m = fmaxf(m, __shfl_xor(m, 16, 64));
                        m = fmaxf(m, __shfl_xor(m, 32, 64));
                        if (q == 0) red(cw)[16u * (uint32_t)rg + r16] = m;
                    }
                }
                asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); /* pairs with the loaders' */
#pragma unroll
                for (uint32_t sub = 0; sub < SUBS; sub++) {
                    const uint32_t cw = cw0 + sub, ch0 = nt * 128u + 16u * cw;
#pragma unroll
                    for (int rg = 0; rg < NG; rg++) {
                        const uint32_t row = 16u * (uint32_t)rg + r16;
                        if (row >= rows || L.epi_idx[par][row] == PLOW_EXPERT_UNUSED) continue;
                        const float amax = fmaxf(red(cw & ~1u)[row], red(cw | 1u)[row]);
                        const uint32_t sb = mxq_e8m0(amax);
                        const float inv = mxq_inv(sb);
                        const uint32_t code = mxq_fp4(v[sub][rg][0] * inv) | (mxq_fp4(v[sub][rg][1] * inv) << 4) |
                                              (mxq_fp4(v[sub][rg][2] * inv) << 8) | (mxq_fp4(v[sub][rg][3] * inv) << 12);
                        *(uint16_t*)((uint8_t*)g.out + (size_t)(r0 + row) * (g.N / 2u) + (ch0 + 4u * q) / 2u) = (uint16_t)code;
                        if (!(cw & 1u) && q == 0) g.out_e8m0[(size_t)(r0 + row) * (g.N / 32u) + (ch0 >> 5)] = (uint8_t)sb;
                    }
                }
            } else if (!PC && GLU && g.out_bf16) {
                /* bf16 intermediate (op 188): bf16(act(g) * u) for live rows, zeros for the pad rows of the
                 * expert's last 64-row tile */
                asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); /* pairs with the loaders' */
                const uint32_t cnt_e = (uint32_t)g.meta[g.E + t.e], erow0 = r0 - (uint32_t)g.meta[t.e];
                const uint32_t padded = ((cnt_e + PLOW_MPF_BM - 1u) / PLOW_MPF_BM) * PLOW_MPF_BM;
#pragma unroll
                for (uint32_t sub = 0; sub < SUBS; sub++) {
                    const uint32_t cw = cw0 + sub, ch0 = nt * 128u + 16u * cw;
                    v4f(&acc)[NG][2] = accs[sub];
#pragma unroll
                    for (int rg = 0; rg < NG; rg++) {
                        const uint32_t row = 16u * (uint32_t)rg + r16;
                        bf16_t* orow = (bf16_t*)g.out + (size_t)(r0 + row) * g.N + ch0 + 4u * q;
                        /* bf16 weights (the reference's bf16 grouped ops write live rows only): pad rows stay untouched */
                        if (row >= rows) {
                            if (!NOPAD && erow0 + row >= cnt_e && erow0 + row < padded) *(uint2*)orow = make_uint2(0u, 0u); /* beyond the expert's rows: a row below its count is the next tile's */
                            continue;
                        }
                        if (NOPAD && L.epi_idx[par][row] == PLOW_EXPERT_UNUSED) continue;
                        uint2 pk = make_uint2(0u, 0u);
                        if (L.epi_idx[par][row] != PLOW_EXPERT_UNUSED) {
                            float o[4];
#pragma unroll
                            for (int i = 0; i < 4; i++) o[i] = t5_glu(acc[rg][0][i], acc[rg][1][i], g.act, g.f0, g.f1);
                            pk.x = (uint32_t)f2bf(o[0]) | ((uint32_t)f2bf(o[1]) << 16);
                            pk.y = (uint32_t)f2bf(o[2]) | ((uint32_t)f2bf(o[3]) << 16);
                        }
                        *(uint2*)orow = pk;
                    }
                }
            } else if (!PC && GLU) {
                float v[SUBS][NG][4];
                /* The row maxima of the eight consumers meet in the ring stage the tile has just left: consumer
                 * x writes its own into the head of its own weight slice there (nobody else reads that slice,
                 * and it is done with it), everyone reads all eight after the barrier; the loaders refill the
                 * stage only after the next tile's first barrier. */
                auto red = [&](uint32_t x) -> float* { return (float*)&L.w[stl][x * (32u * 128u)]; };
#pragma unroll
                for (uint32_t sub = 0; sub < SUBS; sub++) {
                    const uint32_t cw = cw0 + sub;
                    v4f(&acc)[NG][2] = accs[sub];
#pragma unroll
                    for (int rg = 0; rg < NG; rg++) {
                        float m = 0.0f;
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            v[sub][rg][i] = t5_glu(acc[rg][0][i], acc[rg][1][i], g.act, g.f0, g.f1);
                            m = fmaxf(m, fabsf(v[sub][rg][i]));
                        }
                        m = fmaxf(m, __shfl_xor(m, 16, 64));
                        m = fmaxf(m, __shfl_xor(m, 32, 64));
                        if (q == 0) red(cw)[16u * (uint32_t)rg + r16] = m;
                    }
                }
                asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
                for (uint32_t sub = 0; sub < SUBS; sub++) {
                    const uint32_t cw = cw0 + sub, ch0 = nt * 128u + 16u * cw;
#pragma unroll
                    for (int rg = 0; rg < NG; rg++) {
                        const uint32_t row = 16u * (uint32_t)rg + r16;
                        if (row >= rows || L.epi_idx[par][row] == PLOW_EXPERT_UNUSED) continue;
                        float amax = 1e-10f;
#pragma unroll
                        for (int x = 0; x < 8; x++) amax = fmaxf(amax, red((uint32_t)x)[row]);
                        const float s = amax * (1.0f / 448.0f), inv = 1.0f / s;
                        uint8_t* orow = (uint8_t*)g.out + (size_t)(r0 + row) * g.N + ch0 + 4u * q;
                        *(uint32_t*)orow = cvt4_e4m3(v[sub][rg][0] * inv, v[sub][rg][1] * inv, v[sub][rg][2] * inv, v[sub][rg][3] * inv);
                        if (cw == 0 && q == 0) g.out_scale[(size_t)(r0 + row) * NT + nt] = s;
                    }
                }
            } else {
                WG_BARRIER(); /* after the last block (pairs with the loaders') */
#pragma unroll
                for (uint32_t sub = 0; sub < SUBS; sub++) {
                    const uint32_t cw = cw0 + sub;
                    const uint32_t ch0 = GLU ? nt * 128u + 16u * cw : nt * 256u + 32u * cw; /* first channel */
                    v4f(&acc)[NG][2] = accs[sub];
                    /* DOWN, f32 partials: a row's 32 channels of this consumer are one 128-byte line. A 16-row
                     * group goes through LDS once so that it leaves as two stores of 8 whole lines (8 consecutive
                     * lanes per line) instead of two stores that touch 16 half lines each. The staging area is
                     * the consumer's own weight slice of the ring stage it has just left: nobody else reads it,
                     * and the loaders refill it only after the next barrier. Every lane of the wave must call
                     * this. */
                    /* (W4: its weight stage is 16 KB, so the 4 KB per consumer come from the token-row stage it has left as well) */
                    const uint32_t stg = W4 ? a_base + stl * (uint32_t)sizeof(L.a[0]) + cw * (32u * 128u) : w_base + stl * (256u * 128u) + cw * (32u * 128u);
                    auto down_store_f32 = [&](int rg, v4f y0, v4f y1) {
                        const uint32_t buf = stg + (uint32_t)(rg & 1) * 2048u, wsw = r16 & 7u;
                        const uint32_t wr0 = buf + r16 * 128u + ((q ^ wsw) << 4), wr1 = buf + r16 * 128u + (((4u + q) ^ wsw) << 4);
                        const uint32_t lrow = lane >> 3, lp = lane & 7u; /* store layout: row lrow (+ 8), piece lp */
                        const uint32_t rd = buf + lrow * 128u + ((lp ^ (lrow & 7u)) << 4);
                        const uint32_t rowa = 16u * (uint32_t)rg + lrow, rowb = rowa + 8u;
                        const uint32_t pa = L.epi_idx[par][rowa], pb = L.epi_idx[par][rowb];
                        v4f oa, ob;
                        asm volatile("ds_write_b128 %2, %4\n\tds_write_b128 %3, %5\n\t"
                                     "ds_read_b128 %0, %6\n\tds_read_b128 %1, %6 offset:1024\n\t"
                                     "s_waitcnt lgkmcnt(0)"
                                     : "=&v"(oa), "=&v"(ob)
                                     : "v"(wr0), "v"(wr1), "v"(y0), "v"(y1), "v"(rd)
                                     : "memory");
                        if (g.det_k) {
                            /* deterministic fused combine: fixed-point f64 atomics into the token's accumulator
                             * row; 8 lanes cover 256 consecutive bytes of it */
                            if (rowa < rows && pa != PLOW_EXPERT_UNUSED) {
                                double* o = (double*)g.out + (size_t)(pa / g.det_k) * g.N + ch0 + 4u * lp;
                                det_add(o, oa[0]), det_add(o + 1, oa[1]), det_add(o + 2, oa[2]), det_add(o + 3, oa[3]);
                            }
                            if (rowb < rows && pb != PLOW_EXPERT_UNUSED) {
                                double* o = (double*)g.out + (size_t)(pb / g.det_k) * g.N + ch0 + 4u * lp;
                                det_add(o, ob[0]), det_add(o + 1, ob[1]), det_add(o + 2, ob[2]), det_add(o + 3, ob[3]);
                            }
                            return;
                        }
                        float* const ocol = (float*)g.out + ch0 + 4u * lp;
                        if (rowa < rows && pa != PLOW_EXPERT_UNUSED)
                            *(float4*)(ocol + (size_t)pa * g.N) = make_float4(oa[0], oa[1], oa[2], oa[3]);
                        if (rowb < rows && pb != PLOW_EXPERT_UNUSED)
                            *(float4*)(ocol + (size_t)pb * g.N) = make_float4(ob[0], ob[1], ob[2], ob[3]);
                    };
                    if (PC) {
                        /* per-channel arm (plow runtime/amd/op_moe.h:6655-6700): g = acc * (as * wsc[n]); GLU
                         * stores bf16(act(g) * u) and zeroes the expert's pad rows, DOWN stores gate * acc, then
                         * * (as * wsc[h]) */
                        /* bf16 weights carry no scales: the same epilogues with every scale 1 */
                        const float* es = W16 ? nullptr : (const float*)(uintptr_t)g.stab[(size_t)t.e * 2u + (GLU ? 0u : 1u)];
                        const uint32_t cnt_e = (uint32_t)g.meta[g.E + t.e], erow0 = r0 - (uint32_t)g.meta[t.e];
                        const uint32_t padded = ((cnt_e + PLOW_MPF_BM - 1u) / PLOW_MPF_BM) * PLOW_MPF_BM;
                        if (wave_on && !GLU) {
#pragma unroll
                            for (int rg = 0; rg < NG; rg++) {
                                if (16u * (uint32_t)rg >= rows) break; /* uniform */
                                const uint32_t row = 16u * (uint32_t)rg + r16;
                                const float gate = L.epi_gate[par][row]; /* 0 for pad rows */
                                const float as = row < rows ? (A16 ? 1.0f : g.a_scale[r0 + row]) : 0.0f;
                                v4f y[2];
#pragma unroll
                                for (int x = 0; x < 2; x++) {
                                    const uint32_t col = ch0 + 16u * (uint32_t)x + 4u * q;
#pragma unroll
                                    for (int i = 0; i < 4; i++) {
                                        y[x][i] = gate * acc[rg][x][i];
                                        if (!W16) y[x][i] *= as * es[col + i];
                                    }
                                }
                                down_store_f32(rg, y[0], y[1]);
                            }
                        } else if (wave_on) {
#pragma unroll
                            for (int rg = 0; rg < NG; rg++) {
                                const uint32_t row = 16u * (uint32_t)rg + r16;
                                /* A16 with a row -> output row map (slot-major ops): rows leave by that map and
                                 * nothing else of the output is touched */
                                const bool mapped = A16 && g.row_partidx != nullptr;
                                bf16_t* orow = (bf16_t*)g.out + (size_t)(r0 + row) * g.N + ch0 + 4u * q;
                                if (row >= rows) {
                                    if (!W16 && !mapped && erow0 + row >= cnt_e && erow0 + row < padded) *(uint2*)orow = make_uint2(0u, 0u); /* beyond the expert's rows: a row below its count is the next tile's */
                                    continue;
                                }
                                const uint32_t tok = L.epi_idx[par][row];
                                if (mapped) {
                                    const uint32_t orow_i = g.row_partidx[r0 + row];
                                    if (tok == PLOW_EXPERT_UNUSED || orow_i == PLOW_EXPERT_UNUSED) continue;
                                    orow = (bf16_t*)g.out + (size_t)orow_i * g.N + ch0 + 4u * q;
                                } else if (tok == PLOW_EXPERT_UNUSED) {
                                    if (!W16) *(uint2*)orow = make_uint2(0u, 0u);
                                    continue;
                                }
                                const float as = A16 ? 1.0f : g.a_scale[tok];
                                float o[4];
#pragma unroll
                                for (int i = 0; i < 4; i++)
                                    o[i] = W16 ? t5_glu(acc[rg][0][i], acc[rg][1][i], g.act, g.f0, g.f1)
                                               : t5_glu(acc[rg][0][i] * (as * es[ch0 + 4u * q + i]),
                                                        acc[rg][1][i] * (as * es[g.N + ch0 + 4u * q + i]), g.act, g.f0, g.f1);
                                uint2 pk;
                                pk.x = (uint32_t)f2bf(o[0]) | ((uint32_t)f2bf(o[1]) << 16);
                                pk.y = (uint32_t)f2bf(o[2]) | ((uint32_t)f2bf(o[3]) << 16);
                                *(uint2*)orow = pk;
                            }
                        }
                    } else if (wave_on && g.acc_topk) {
                        /* fused combine: add into the bf16 output row of the slot's token */
                        typedef short bf16x2_t __attribute__((ext_vector_type(2)));
#pragma unroll
                        for (int rg = 0; rg < NG; rg++) {
                            const uint32_t row = 16u * (uint32_t)rg + r16;
                            if (row >= rows) continue;
                            const uint32_t pidx = L.epi_idx[par][row];
                            if (pidx == PLOW_EXPERT_UNUSED) continue;
                            const float gate = L.epi_gate[par][row];
                            bf16_t* orow = (bf16_t*)g.out + (size_t)(pidx / g.acc_topk) * g.N + ch0 + 4u * q;
#pragma unroll
                            for (int x = 0; x < 2; x++)
#pragma unroll
                                for (int h = 0; h < 2; h++) {
                                    const uint32_t pk = (uint32_t)f2bf(gate * acc[rg][x][2 * h]) | ((uint32_t)f2bf(gate * acc[rg][x][2 * h + 1]) << 16);
                                    __builtin_amdgcn_global_atomic_fadd_v2bf16((bf16x2_t*)(orow + 16u * (uint32_t)x + 2u * (uint32_t)h),
                                                                               __builtin_bit_cast(bf16x2_t, pk));
                                }
                        }
                    } else if (wave_on && (g.det_k || !g.part16)) {
#pragma unroll
                        for (int rg = 0; rg < NG; rg++) {
                            if (16u * (uint32_t)rg >= rows) break; /* uniform */
                            const float gate = L.epi_gate[par][16u * (uint32_t)rg + r16]; /* 0 for pad rows */
                            down_store_f32(rg, acc[rg][0] * gate, acc[rg][1] * gate);
                        }
                    } else if (wave_on) {
#pragma unroll
                        for (int rg = 0; rg < NG; rg++) {
                            const uint32_t row = 16u * (uint32_t)rg + r16;
                            if (row >= rows) continue;
                            const uint32_t pidx = L.epi_idx[par][row];
                            if (pidx == PLOW_EXPERT_UNUSED) continue;
                            const float gate = L.epi_gate[par][row];
#pragma unroll
                            for (int x = 0; x < 2; x++) {
                                const size_t ocol = (size_t)pidx * g.N + ch0 + 16u * (uint32_t)x + 4u * q;
                                const float y0 = gate * acc[rg][x][0], y1 = gate * acc[rg][x][1];
                                const float y2 = gate * acc[rg][x][2], y3 = gate * acc[rg][x][3];
                                uint2 o;
                                o.x = (uint32_t)f2bf(y0) | ((uint32_t)f2bf(y1) << 16);
                                o.y = (uint32_t)f2bf(y2) | ((uint32_t)f2bf(y3) << 16);
                                *(uint2*)((bf16_t*)g.out + ocol) = o;
                            }
                        }
                    }
                }
            }
        }
    }
}
template <bool GLU, bool PC, uint32_t NCW, int NG>
__global__ __launch_bounds__((NCW + 4u) * 64u) void k_group_w8a8_tiled(GroupW8A8 g) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    t5_body<GLU, PC, NCW, NG>(g, lds_raw);
}
/* the same tiles with bf16 activations; W16: bf16 weights too (PC then only names the fused table layout) */
template <bool GLU, bool PC, bool W16 = false>
__global__ __launch_bounds__(12u * 64u) void k_group_a16_tiled(GroupW8A8 g) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    t5_body<GLU, PC, 8u, 8, W16 ? 3 : 1>(g, lds_raw);
}


/* mxfp4 weights under bf16 activations (ops 85 / 86 arm 8) */
template <bool GLU>
__global__ __launch_bounds__(12u * 64u) void k_group_a16w4_tiled(GroupW8A8 g) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    t5_body<GLU, false, 8u, 8, 4>(g, lds_raw);
}

/* dynamic-LDS limits, once per device (plow_moe_device_setup) */
template <bool GLU, bool PC, uint32_t NCW, int NG>
static bool t5_set_attr() {
    return hipFuncSetAttribute((const void*)k_group_w8a8_tiled<GLU, PC, NCW, NG>, hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)sizeof(T5Lds)) == hipSuccess;
}
template <uint32_t NCW, int NG>
static bool t5_set_attrs() {
    return t5_set_attr<true, false, NCW, NG>() && t5_set_attr<false, false, NCW, NG>() && t5_set_attr<true, true, NCW, NG>() &&
           t5_set_attr<false, true, NCW, NG>();
}
/* mxfp4 on both operands */
template <bool GLU>
__global__ __launch_bounds__(12u * 64u) void k_group_a4w4_tiled(GroupW8A8 g) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    t5_body<GLU, false, 8u, 8, 2>(g, lds_raw);
}
int plow_moe_w8a8_tiled_setup() {
    auto a16 = [](const void* f) {
        return hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(T5Lds)) == hipSuccess;
    };
    const bool ok = t5_set_attrs<8u, 8>() && t5_set_attrs<8u, 9>() && t5_set_attrs<4u, 8>() &&
                    a16((const void*)k_group_a16_tiled<true, false>) && a16((const void*)k_group_a16_tiled<false, false>) &&
                    a16((const void*)k_group_a16_tiled<true, true>) && a16((const void*)k_group_a16_tiled<false, true>) &&
                    a16((const void*)k_group_a16_tiled<true, false, true>) && a16((const void*)k_group_a16_tiled<false, false, true>) &&
                    a16((const void*)k_group_a16_tiled<true, true, true>) && a16((const void*)k_group_a16_tiled<false, true, true>) &&
                    hipFuncSetAttribute((const void*)k_group_a16w4_tiled<true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                        (int)sizeof(T5LdsW4)) == hipSuccess &&
                    hipFuncSetAttribute((const void*)k_group_a16w4_tiled<false>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                        (int)sizeof(T5LdsW4)) == hipSuccess &&
                    hipFuncSetAttribute((const void*)k_group_a4w4_tiled<true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                        (int)sizeof(T5LdsA4)) == hipSuccess &&
                    hipFuncSetAttribute((const void*)k_group_a4w4_tiled<false>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                        (int)sizeof(T5LdsA4)) == hipSuccess;
    return ok ? 0 : PLOW_MOE_EDEVICE;
}

/* Persistent launch: one workgroup per CU; the tile count is computed on the device from meta. */
template <bool GLU, bool PC, uint32_t NCW, int NG>
static int launch_tiled_t(const GroupW8A8& g, hipStream_t st) {
    const uint32_t n_cu = plow_moe_n_cu();
    if (!n_cu) return PLOW_MOE_EDEVICE;
    k_group_w8a8_tiled<GLU, PC, NCW, NG><<<n_cu, (NCW + 4u) * 64u, sizeof(T5Lds), st>>>(g);
    return 0;
}

/* Row tiles of a batch of `slots_bound` routed rows never exceed slots / 128 + E (every expert's last tile may be
 * partial); 0 = the host does not know the count and the kernel checks the real one. */
static bool t5_row_tiles_fit(const GroupW8A8& g) {
    return (uint64_t)g.slots_bound / 128u + g.E <= T5_MAX_ROW_TILES;
}
/* The shapes the tiled form serves: the tile keeps K / 128 block scales in LDS and the load ring runs
 * two blocks ahead. Callers fall back to the streaming form otherwise. */
bool group_w8a8_tiled_serves(const GroupW8A8& g) {
    return g.N != 0u && g.E != 0u && g.E <= 1056u && g.N % 128u == 0u && g.K % 128u == 0u && g.K >= 256u &&
           g.K <= 128u * 128u && g.N >= 256u && t5_row_tiles_fit(g);
}

/* Tiles of nine 16-row groups (144 rows) instead of eight: the ninth group saves an expert with 129..144
 * rows (257..288, ...) a whole second tile, i.e. a second pass over its weight rows. That pays when the
 * weights are the traffic: an expert's matrix of this op is larger than an XCD's 4 MB L2, so a second row
 * tile fetches it again (DeepSeek-V3 shape at 4096 tokens, 128 rows per expert on average: GLU 2030 ->
 * 1818 us). Where they are not (plow's own prefill bench shape: 1 - 2 MB per expert) the larger
 * accumulator only costs registers (+5 %), so those shapes keep eight groups. */
static bool t5_nine_groups(const GroupW8A8& g, bool glu) {
    return (uint64_t)(glu ? 2u : 1u) * g.N * g.K > (4ull << 20);
}

template <bool GLU>
static int launch_tiled(const GroupW8A8& g, hipStream_t st) {
    if (!group_w8a8_tiled_serves(g)) return PLOW_MOE_EINVAL;
    if (plow_moe_tuning().tile_waves4) return g.per_channel ? launch_tiled_t<GLU, true, 4u, 8>(g, st) : launch_tiled_t<GLU, false, 4u, 8>(g, st);
    if (t5_nine_groups(g, GLU)) return g.per_channel ? launch_tiled_t<GLU, true, 8u, 9>(g, st) : launch_tiled_t<GLU, false, 8u, 9>(g, st);
    return g.per_channel ? launch_tiled_t<GLU, true, 8u, 8>(g, st) : launch_tiled_t<GLU, false, 8u, 8>(g, st);
}

int launch_group_a4w4_tiled(const GroupW8A8& g, bool glu, hipStream_t st) {
    if (!g.N || !g.E || g.E > 1056u || g.N % 128u || g.N < 256u || g.K % 256u || g.K < 512u || g.K > 256u * 128u ||
        !t5_row_tiles_fit(g))
        return PLOW_MOE_EINVAL;
    const uint32_t n_cu = plow_moe_n_cu();
    if (!n_cu) return PLOW_MOE_EDEVICE;
    if (glu) k_group_a4w4_tiled<true><<<n_cu, 768, sizeof(T5LdsA4), st>>>(g);
    else k_group_a4w4_tiled<false><<<n_cu, 768, sizeof(T5LdsA4), st>>>(g);
    return 0;
}

/* bf16 activations: `g.a` bf16 [..][K], no activation scales; g.per_channel picks the weight layout */
int launch_group_a16_tiled(const GroupW8A8& g, bool glu, hipStream_t st) {
    if (!group_w8a8_tiled_serves(g)) return PLOW_MOE_EINVAL;
    const uint32_t n_cu = plow_moe_n_cu();
    if (!n_cu) return PLOW_MOE_EDEVICE;
    if (g.w_mxfp4) { /* mxfp4 weights with E8M0 rows through stab [E][3] */
        if (g.per_channel) return PLOW_MOE_EINVAL;
        if (glu) k_group_a16w4_tiled<true><<<n_cu, 768, sizeof(T5LdsW4), st>>>(g);
        else k_group_a16w4_tiled<false><<<n_cu, 768, sizeof(T5LdsW4), st>>>(g);
        return 0;
    }
    if (g.w_bf16) { /* bf16 weights: per_channel names the fused table layout ewt[E][2], nothing else */
        if (glu) {
            if (g.per_channel) k_group_a16_tiled<true, true, true><<<n_cu, 768, sizeof(T5Lds), st>>>(g);
            else k_group_a16_tiled<true, false, true><<<n_cu, 768, sizeof(T5Lds), st>>>(g);
        } else {
            if (g.per_channel) k_group_a16_tiled<false, true, true><<<n_cu, 768, sizeof(T5Lds), st>>>(g);
            else k_group_a16_tiled<false, false, true><<<n_cu, 768, sizeof(T5Lds), st>>>(g);
        }
        return 0;
    }
    if (glu) {
        if (g.per_channel) k_group_a16_tiled<true, true><<<n_cu, 768, sizeof(T5Lds), st>>>(g);
        else k_group_a16_tiled<true, false><<<n_cu, 768, sizeof(T5Lds), st>>>(g);
    } else {
        if (g.per_channel) k_group_a16_tiled<false, true><<<n_cu, 768, sizeof(T5Lds), st>>>(g);
        else k_group_a16_tiled<false, false><<<n_cu, 768, sizeof(T5Lds), st>>>(g);
    }
    return 0;
}

int launch_group_glu_w8a8_tiled(const GroupW8A8& g, hipStream_t st) { return launch_tiled<true>(g, st); }
int launch_group_down_w8a8_tiled(const GroupW8A8& g, hipStream_t st) { return launch_tiled<false>(g, st); }
