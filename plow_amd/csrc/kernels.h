/* kernels.h — host-callable launchers of the device kernels (one per op family). Every launcher is
 * asynchronous on `st`, allocates nothing and returns 0 or a negative PLOW_MOE_E* code. */
#ifndef PLOW_MOE_KERNELS_H
#define PLOW_MOE_KERNELS_H

#include <hip/hip_runtime.h>
#include <stdint.h>

int launch_router_score(float* out, const void* x, const void* w, uint32_t M, uint32_t N, uint32_t K,
                        hipStream_t st);
int launch_router_topk(void* table, const void* logit, const float* bias, uint32_t n_exp, uint32_t k,
                       uint32_t flags, uint32_t T, uint32_t tail, uint32_t n_group, uint32_t topk_group,
                       float route_scale, float logit_scale, hipStream_t st);
/* chunk_hist: u32 [chunk_cap][E] scratch for the multi-workgroup form (NULL = single workgroup) */
int launch_align(int32_t* meta, const void* table, uint32_t* row_token, uint32_t* row_partidx,
                 float* row_gate, uint32_t T, uint32_t E, uint32_t k, uint32_t* chunk_hist,
                 uint32_t chunk_cap, hipStream_t st);

/* The decode router's score with its top-k in one launch (op 180 with the router mark). Every field has
 * the meaning it has on the separate launchers above; `logit` is f32 [M][N] and PLOW_ROUTE_F32_LOGIT is set
 * in flags. `row_ctr`: the caller's arrival counters, one word per row, 32 words apart, zero between
 * launches (the kernel leaves them zero) and used by one launch at a time. */
struct RouterRun {
    void* logit;
    const void* x;
    const void* w;
    uint32_t M, N, K;
    void* table;
    const float* bias;
    uint32_t k, flags, tail, n_group, topk_group;
    float route_scale, logit_scale;
    uint32_t* row_ctr;
};
bool router_decode_serves(const RouterRun& r);
int launch_router_decode(const RouterRun& r, hipStream_t st);
int launch_combine(void* out, const void* residual, const void* shared, const void* part, uint32_t H,
                   uint32_t k, uint32_t T, uint32_t part16, hipStream_t st);
/* the deterministic fused combine: acc is the f64 [T][H] fixed-point accumulator the DOWN op summed in place */
int launch_combine_det(void* out, const void* residual, const void* shared, const double* acc, uint32_t H, uint32_t T,
                       hipStream_t st);
int launch_zero_f64(double* p, size_t n, hipStream_t st);

/* aligned bf16 rows -> two-term e4m3 rows [hi K | lo K] + scales [row][K / 128], and back (rows_bound: an upper bound
 * of the aligned rows, for the grid; the kernels read the count from meta) */
int launch_split_block128(void* fq, float* fs, const void* fu, const int32_t* meta, const uint32_t* row_token, uint32_t K,
                          uint32_t E, uint32_t rows_bound, hipStream_t st);
int launch_join_block128(void* out, const void* fq, const float* fs, const int32_t* meta, const uint32_t* row_partidx,
                         uint32_t K, uint32_t E, uint32_t rows_bound, hipStream_t st);
int launch_quant_block128(void* xq, const void* x, float* scale, uint32_t M, uint32_t K, uint32_t pitch,
                          hipStream_t st);
int launch_quant_block128_scatter(void* hq, const void* fu, float* scale, const void* meta, const void* row_partidx,
                                  void* out, uint32_t K, uint32_t E, uint32_t topk, uint32_t T, uint32_t H,
                                  hipStream_t st);
int launch_rmsnorm(void* out, const void* x, const void* gamma, void* xq, float* scale, uint32_t rows, uint32_t feat,
                   uint32_t out_row0, float eps, uint32_t mode, hipStream_t st);
int launch_quant_row(void* xq, void* x, float* scale, const void* gate, const void* up, uint32_t act,
                     uint32_t M, uint32_t K, hipStream_t st);

/* Grouped experts over aligned rows, block-fp8 weights x 1x128-scaled e4m3 activations. */
struct GroupW8A8 {
    void* out;            /* GLU: fq u8 [R][N]; DOWN: part f32|bf16 [T*k][N] */
    float* out_scale;     /* GLU: fs f32 [R][N/128] */
    const void* a;        /* GLU: xq u8 [T][K]; DOWN: fq u8 [R][K] */
    const float* a_scale; /* GLU: xs f32 [K/128][pitch]; DOWN: fs f32 [R][K/128] */
    const uint64_t* wtab; /* [E][3] */
    const uint64_t* stab; /* [E][3] */
    const int32_t* meta;
    const uint32_t* row_token;   /* GLU */
    const uint32_t* row_partidx; /* DOWN */
    const float* row_gate;       /* DOWN */
    uint32_t N, K, E, pitch, act, part16, T;
    float f0, f1; /* the activation's immediates */
    /* per-channel mode (ops 81 / 82): weights through ewt[E][2] = {gate_up fused [2N][K], down [N][K]},
     * f32 channel scales through est[E][2], one f32 activation scale per row; GLU writes bf16 */
    uint32_t per_channel;
    /* DOWN, block mode: when non-zero, `out` is the bf16 [T][N] layer output and every live row adds
     * gate * acc into row (row_partidx / acc_topk) with packed bf16 atomics (order-dependent rounding;
     * plow's fused-combine variant, runtime/amd/moe_fp8_pf.hip:1219-1230) */
    uint32_t acc_topk;
    /* DOWN: when non-zero (= routing slots per token), `out` is the f64 [T][N] fixed-point accumulator of
     * the deterministic fused combine: every live row adds rint(clamp(gate * acc) * 2^32) into row
     * (row_partidx / det_k) with f64 atomics (order-independent; plow runtime/amd/op_moe.h:2110-2165) */
    uint32_t det_k;
    /* GLU, block mode: when non-zero, `a` holds the bf16 rows [T][K] themselves and the kernel quantizes
     * every 1x128 group as it loads it (a_scale and pitch unused; plow's arm i7 = 6) */
    uint32_t a_bf16;
    /* GLU, block mode: write bf16(act(g) * u) rows [R][N] instead of quantized ones, zeros in the pad
     * rows of every 64-row tile and in all rows of an expert without weights (op 188) */
    uint32_t out_bf16;
    /* DOWN, block mode: when non-zero, `a` and `a_scale` are stored by routing slot ([a_slots][K] and
     * [K/128][a_slots]) and aligned row r reads slot row_partidx[r]; slots >= a_slots are skipped (op 190) */
    uint32_t a_slots;
    /* fp4 x fp4 arm (launch_group_a4w4_tiled): `a` holds mxfp4 rows [..][K / 2] and a_e8m0 their E8M0 rows
     * [..][K / 32]; the GLU writes its output the same way into out / out_e8m0; stab holds E8M0 rows */
    const uint8_t* a_e8m0;
    uint8_t* out_e8m0;
    /* bf16-activation tiled form (launch_group_a16_tiled): the weights are bf16 too, no scale tables; per_channel then
     * only says that the tables are the fused pair ewt[E][2] = {gate_up [2N][K], down} instead of wtab[E][3] */
    uint32_t w_bf16;
    /* the same form with mxfp4 weights (wtab / stab [E][3], stab = E8M0 rows [N][K / 32]): a block is 128 k */
    uint32_t w_mxfp4;
    /* tiled forms: when non-zero, the weight rows of an expert with a single row tile (read once) are loaded
     * non-temporal. Right while the launch is bound by the weight stream; from about 64 rows per expert on
     * average it is bound by what a CU's load path carries and the bit costs time */
    uint32_t w_nt;
    /* Form chosen on the device: when form_word is set, the launch runs only if *form_word == form_want and
     * every workgroup of it returns at once otherwise. The host then launches both forms of the op behind
     * launch_pick_form, which writes the word from the routed rows in meta (0 streaming, 1 tiled). */
    const uint32_t* form_word;
    uint32_t form_want;
    /* tiled forms: an upper bound of the batch's routed rows when the host knows one (0 = unknown). Their tile
     * directory counts row tiles in 16 bits; a batch that may exceed that is refused by the launcher */
    uint32_t slots_bound;
};
#if defined(__HIPCC__)
/* whether this launch is the form the device-side choice names (always, when the launch carries no choice) */
template <typename G>
__device__ __forceinline__ bool form_is_mine(const G& g) {
    uint32_t form = g.form_want;
    if (g.form_word) form = *(const __attribute__((address_space(4))) uint32_t*)g.form_word; /* written by an earlier kernel: a scalar load */
    return form == g.form_want;
}
#endif
/* *word = 1 when meta counts at least 16 routed rows per expert on average (the tiled forms' side of the
 * measured crossover), else 0 */
int launch_pick_form(uint32_t* word, const int32_t* meta, uint32_t E, hipStream_t st);
int launch_group_glu_w8a8(const GroupW8A8& g, hipStream_t st);
int launch_group_down_w8a8(const GroupW8A8& g, hipStream_t st);
/* the many-rows-per-expert form of the same two ops (block mode only) */
int launch_group_glu_w8a8_tiled(const GroupW8A8& g, hipStream_t st);
int launch_group_down_w8a8_tiled(const GroupW8A8& g, hipStream_t st);
/* whether the tiled form serves this shape (callers take the streaming form otherwise) */
bool group_w8a8_tiled_serves(const GroupW8A8& g);
/* the tiled form with bf16 activations (`a` bf16 [..][K], no activation scales): block-fp8 weights
 * (wtab / stab [E][3]; GLU writes bf16 rows, out_bf16 set), per-channel fp8 weights (per_channel set,
 * tables [E][2]) or bf16 weights (w_bf16 set, either layout); GLU gathers rows by row_token and, in the
 * fused-table layout only, may scatter them by
 * row_partidx; DOWN reads aligned rows, or slot rows when a_slots is set */
int launch_group_a16_tiled(const GroupW8A8& g, bool glu, hipStream_t st);
/* the tiled form with mxfp4 on both operands (K a multiple of 256, at least 512) */
int launch_group_a4w4_tiled(const GroupW8A8& g, bool glu, hipStream_t st);
/* bf16 rows [rows][K] -> mxfp4 rows [rows][K / 2] + E8M0 rows [rows][K / 32], the fp4 x fp4 arm's activation
 * quantizer (K a multiple of 32) */
int launch_quant_mx_act(uint8_t* out, uint8_t* scales, const void* x, uint32_t rows, uint32_t K, hipStream_t st);


/* Grouped experts with bf16 activations (see experts_a16.hip). */
struct GroupA16 {
    void* out;              /* GLU: bf16 [rows][N]; DOWN: f32 (or bf16) [rows][N] */
    const void* a;          /* bf16 [rows][K] */
    const uint64_t* wtab;   /* [E][wcols] device pointers */
    const uint64_t* stab;   /* [E][wcols] or NULL (bf16 weights) */
    const int32_t* meta;    /* rowoff | cnt | tilep, or NULL = one dense expert of dense_rows rows */
    const uint32_t* a_idx;  /* aligned row -> row of `a` (NULL = identity) */
    const uint32_t* o_idx;  /* aligned row -> output row (NULL = identity) */
    const float* gate;      /* DOWN: aligned row -> gate (NULL = 1) */
    uint32_t N, K, E, enc, act;
    float f0, f1; /* the activation's immediates */
    uint32_t wcols, wsel0, wsel1; /* table width, column of the first / second weight stream */
    uint32_t wrow0, wrow1;        /* first weight row of each stream inside its tensor (fused gate_up) */
    uint32_t out_bf16, dense_rows;
    uint32_t slots_hint; /* routed slots of the batch when the host knows them (0 = unknown): picks the kernel form */
    /* weight row of output channel n in stream s: n * wmul + wrow_s (wmul 0 reads as 1). Blocked gate | up
     * rows: wmul 1, wrow1 = N; interleaved (2n, 2n + 1): wmul 2, wrow1 = 1 */
    uint32_t wmul;
    /* per-expert bf16 bias rows laid out like the weight rows ([E][bias_rows]), added in f32 before the
     * activation (GLU) or before the gate multiply (DOWN); NULL = none */
    const void* bias;
    uint32_t bias_rows;
    const void* wdirect[2]; /* used when wtab is NULL: the two weight tensors themselves (dense ops) */
    /* matrix-vector form, DOWN with block-fp8 weights only: when set, `a` holds e4m3 rows [rows][K] and this their
     * f32 scales [rows][K / 128] (the intermediate of the fp8 x fp8 arm) */
    const float* a_f8scale;
    /* Form chosen on the device (see GroupW8A8::form_word). form_ws: a word of workspace the launcher may use for the
     * choice when slots_hint is 0 and the op could run tiled (NULL: unknown row counts take the streaming form);
     * form_word / form_want: set by the launcher on the launches that stand behind the choice. */
    uint32_t* form_ws;
    const uint32_t* form_word;
    uint32_t form_want;
    /* matrix-vector form, slot-major DOWN: when set, the routing table [zs_nslot] whose slots no expert serves
     * (sentinel id, or an expert without resident weights) get their f32 output rows zeroed by this launch, as the
     * reference's decode DOWN bodies do (plow runtime/cpu/dev/golden/moe.c:76-80) */
    const void* zs_table;
    uint32_t zs_nslot;
    /* streaming DOWN: set by the launcher when the workgroups take tiles of 256 channels (32 per wave) */
    uint32_t down_wide;
    /* streaming forms: set by the launcher when experts of a handful of rows run with per-wave copies of their rows */
    uint32_t priv_rows;
    /* matrix-vector form of the slot-major ops: when set, the routing table [tab_nslot] itself lists the rows (row =
     * slot, in slot order; its expert and gate from the table; its input row slot / tab_kx, its output row the slot)
     * and meta, a_idx, o_idx and gate are not read: no sort ahead of the op */
    const void* tab_direct;
    uint32_t tab_nslot, tab_kx;
    /* Dense ops of a few rows (one expert, no meta, bf16 weights): scratch the launcher may use to split K over
     * several workgroups per channel tile (NULL: never split). split_ws holds f32 partial rows. */
    void* split_ws;
    size_t split_ws_bytes;
    /* set by the launcher on a K-split launch: "expert" v of the launch is K slice v % ksplit (K columns starting at
     * (v % ksplit) * K of rows whose pitch is kpitch) of weight tensor wdirect[v / ksplit]; it reads activation rows
     * 0 .. dense_rows - 1 and writes output rows v * dense_rows .. */
    uint32_t ksplit, kpitch;
};
/* the matrix-vector form of the same ops for batches that route a handful of rows in all (slots_hint says so) */
bool group_a16_gemv_serves(const GroupA16& g);
int launch_group_a16_gemv(const GroupA16& g, bool glu, hipStream_t st);
int launch_group_glu_a16(const GroupA16& g, hipStream_t st);
int launch_group_down_a16(const GroupA16& g, hipStream_t st);
/* wtab / stab rows {p, p, p} for the experts of one flat tensor: p = W + e * w_stride, S + e * s_stride */
int launch_flat_tables(uint64_t* wtab, uint64_t* stab, const void* W, const void* S, uint32_t E, size_t w_stride,
                       size_t s_stride, hipStream_t st);
int launch_zero_skipped(float* part, const void* table, const uint64_t* wtab, const uint64_t* stab,
                        uint32_t wcols, uint32_t wsel, uint32_t nslot, uint32_t E, uint32_t H, hipStream_t st);

#endif
