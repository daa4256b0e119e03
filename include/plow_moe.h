/* plow_moe.h — C-ABI of the gfx950 (MI355X) Mixture-of-Experts expert-FFN operator.
 *
 * The library behind this header is a drop-in for plow's MoE op family on one AMD GPU: it takes the
 * same 64-byte op descriptor plow's interpreters execute, with the same operand slots, tensor
 * layouts, sentinels and refusal behaviour, and runs it as dedicated HIP kernels on a caller-owned
 * stream. Nothing here allocates per call, synchronises the host, or reads device routing data on
 * the host, so a caller may record the calls into a HIP graph.
 *
 * Reference interfaces this header replaces (paths relative to the plow tree):
 *   descriptor + sentinels   runtime/common/dev_isa.h:1586-1613, :1575, :2064
 *   CPU kernel entry shape   runtime/cpu/dev/cpu_dev.h:172-181   (fn(inst, slice, nblk, tensors, ctx))
 *   op slot maps             runtime/common/dev_isa.h:363-370, :435-474, :495-508, :565-569,
 *                            :653-661, :682-709, :1429-1439; runtime/amd/interp.hip:6202-6293,
 *                            :6384-6399, :6468-6635
 *   native-segment route     crates/plowrt/src/exec/gpu/moe_lt.rs:24-60, :697-814, :1134-1322
 *                            (the moe_pf_lt / moe_dec_lt variants), knobs
 *                            crates/plowrt/src/config.rs:2023-2060
 *
 * All entry points return 0 on success or a negative PLOW_MOE_E* code; they never throw or abort.
 */
#ifndef PLOW_MOE_H
#define PLOW_MOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- descriptor (byte-identical to PlowDevInst, runtime/common/dev_isa.h:1607-1613) ---------- */

typedef union {
    float    f;
    uint32_t u;
} PlowFJ;

typedef struct {
    uint16_t op;
    uint16_t blocks; /* workgroups the producer sliced the op across; advisory for this library */
    PlowFJ   fj[3];  /* fj[2].u on a grouped expert op (75, 76, 81, 82, 85, 86, 152, 153, 188, 190): the
                      * routed slots T * k of the batch if the producer states them, 0 = not stated. An
                      * extension of this library (no MoE op of the reference uses the third immediate):
                      * these ops carry no row count, and the kernel form that serves them best depends on
                      * it. Without it the count is taken from the align op (84) of the same
                      * plow_moe_exec_many / segment run, then from what the op's own operands imply,
                      * then (ops over a routing meta) from that meta on the device. Nothing is remembered
                      * between calls. The count only selects between kernel forms, which agree within
                      * the layer tolerance but not bit for bit: the tiled GLU takes SiLU from the
                      * hardware exp2 / reciprocal where the streaming form uses expf and an IEEE
                      * division (at most one bf16 step on a bf16 intermediate); the matrix-vector DOWN
                      * (at most 36 slots) adds a row's products in another order than the matrix
                      * instruction forms; the tiled W8A8 GLU leaves the fq / fs rows of an expert
                      * whose weights are not resident unwritten where the streaming form zeroes them
                      * (the bf16 intermediate of op 188 is zero-filled by both). */
    uint16_t t[8];   /* handles into the tensor table; PLOW_TENSOR_NONE = absent => NULL */
    uint32_t i[8];
} PlowDevInst;

#define PLOW_TENSOR_NONE   0xFFFFu      /* dev_isa.h:2064 */
#define PLOW_EXPERT_UNUSED 0xFFFFFFFFu  /* dev_isa.h:1575 */

/* Routing table entry (runtime/cpu/dev/golden/gptoss.h:24-28). */
typedef struct {
    uint32_t eid;
    float    gate;
} PlowMoeRoute;

/* Rows each expert's gathered segment is padded to (runtime/amd/op_moe.h:1921-1923) and the
 * capacity contract of the gathered arrays (op_moe.h:2252-2255). */
#define PLOW_MPF_BM 64u
#define PLOW_MPF_META_INTS(n_exp) (3u * (n_exp) + 1u)
#define PLOW_MPF_MAX_ROWS(T, k, n_exp) ((T) * (k) + (n_exp) * (PLOW_MPF_BM - 1u))
#define PLOW_ROUTE_MAX_TOPK 16u         /* golden/moe_route.c:15 */
#define PLOW_ROUTE_MAX_GROUPS 64u       /* runtime/common/moe_route_key.h:33 */

/* ---- opcodes served (numbers from runtime/common/dev_isa.h) ---------------------------------- */
enum {
    PLOW_DOP_RMSNORM                       = 1,   /* the step before the path: t0=out t1=x t2=gamma?
                                                     t3=xq? t4=scale? i0=rows i1=feat i2=out_row0 f0=eps;
                                                     t3 bound: also quantize the rounded row, per row
                                                     (scale f32[rows], as op 32) or, with i4 = 128, per
                                                     1x128 group (scale f32[feat/128][rows], as op 184)
                                                     (runtime/cpu/dev/golden/norm.c:15-43,
                                                     runtime/amd/op_norm.h:486-551)                 */
    PLOW_DOP_GEMM                          = 8,   /* dense bf16 GEMM (shared-expert down)        */
    PLOW_DOP_GEMM_GLU                      = 20,  /* dense bf16 gate|up + GLU (shared expert)    */
    PLOW_DOP_QUANT_FP8                     = 32,  /* per-row e4m3 activation quant; any K; with
                                                   * t3 gate / t4 up bound the row is produced
                                                   * first, x = bf16(act_i2(gate) * up)          */
    PLOW_DOP_MOE_COMBINE                   = 43,
    PLOW_DOP_MOE_GROUP_GLU_FP8_BLK         = 48,  /* decode, table-driven, i6 = enc              */
    PLOW_DOP_MOE_GROUP_DOWN_FP8_BLK        = 49,
    PLOW_DOP_MOE_ROUTER_TOPK               = 56,
    PLOW_DOP_MOE_EXPERT_GLU_GEMMA_FP8      = 65,  /* decode, per-channel fp8, fused gate_up table */
    PLOW_DOP_MOE_EXPERT_DOWN_GEMMA_FP8     = 66,
    PLOW_DOP_MOE_GROUP_GLU_GEMMA_PF        = 75,  /* grouped, bf16, fused table ewt[E][2]        */
    PLOW_DOP_MOE_GROUP_DOWN_GEMMA_PF       = 76,
    PLOW_DOP_MOE_GROUP_GLU_GEMMA_PF_W8A8   = 81,  /* grouped, per-channel fp8 x per-row fp8      */
    PLOW_DOP_MOE_GROUP_DOWN_GEMMA_PF_W8A8  = 82,
    PLOW_DOP_MOE_ROUTER_TOPK_PF            = 83,
    PLOW_DOP_MOE_ALIGN_PF                  = 84,
    PLOW_DOP_MOE_GROUP_GLU_PF              = 85,
    PLOW_DOP_MOE_GROUP_DOWN_PF             = 86,
    PLOW_DOP_MOE_COMBINE_PF                = 87,
    PLOW_DOP_MOE_GLU_MX                    = 150, /* decode, flat mxfp4 tensors [E][2I][K/2]     */
    PLOW_DOP_MOE_DOWN_MX                   = 151,
    PLOW_DOP_MOE_GLU_MX_PF                 = 152, /* the same on gathered rows (after 83 / 84)   */
    PLOW_DOP_MOE_DOWN_MX_PF                = 153,
    PLOW_DOP_GEMM_F32                      = 180, /* router score: bf16 x bf16 -> f32 logits     */
    PLOW_DOP_QUANT_FP8_BLOCK128            = 184, /* 1x128 e4m3 activation quant                 */
    /* the block-fp8 chain with a bf16 intermediate and a slot-major quantized copy of it, reduced into
     * the layer output with bf16 atomics (crates/packet/src/dev.rs:2171-2180,
     * runtime/amd/op_moe_fp8_block128.h:7-88, runtime/amd/interp.hip:5282-5310):
     * 188 t0=fu bf16[R][I] t1=xq t2=xscale f32[H/128][T] t3=wtab t4=stab t5=meta t6=row_token
     *     i0=I i1=H i2=E i3=T, fj[1] > 0: clamped SwiGLU with that limit; pad rows of every tile zeroed
     * 189 t0=hq u8[T*topk][I] t1=fu t2=hscale f32[I/128][T*topk] t3=meta t4=row_partidx t5=out bf16[T][H]
     *     i0=I i1=E i2=topk i3=T i4=H: aligned rows quantized 1x128 into their slot's row; out zeroed
     * 190 t0=out t1=hq t2=hscale t3=wtab t4=stab t5=meta t6=row_partidx t7=row_gate
     *     i0=I i1=H i2=E i3=topk i4=T: out[slot / topk] += bf16(gate * (Wd . hq[slot])), bf16 atomics
     *     (the order of the additions, and so the rounding, is not fixed) */
    PLOW_DOP_MOE_GLU_FP8_BLOCK128          = 188,
    PLOW_DOP_MOE_QUANT_FP8_BLOCK128        = 189,
    PLOW_DOP_MOE_DOWN_FP8_BLOCK128         = 190
};

/* Op 180 with i7 = PLOW_ROUTER_RAW_MARK: the decode router's score with its top-k in one launch
 * (crates/packet/src/dev.rs:90-94, runtime/amd/router_decode.hip:1-63; plowrt routes such an op to
 * router_decode_gfx950.elf). On top of the score's operands (t0 logits f32 [rows][n_exp], t1 x, t2 W,
 * i0 rows, i1 n_exp, i2 K): t3 = routing table, t4 = selection bias, t5 = arrival counters (u32, one per
 * row, 32 words apart, zero between launches: the kernel leaves them zero), i3 = k, i4 = router flags
 * (PLOW_ROUTE_F32_LOGIT set), i5 bit 0 = shared tail slot, i6 = n_group | topk_group << 16, f0 = route
 * scale. Logits and table are the bytes of op 180 followed by op 83. i5 bit 1 (signal the interpreter's
 * counters) is refused. */
#define PLOW_ROUTER_RAW_MARK 0x52545241u

/* Weight encodings (i3 on ops 85/86, i6 on ops 48/49; dev_isa.h:442-461, :691-702). */
enum { PLOW_MOE_ENC_BF16 = 0, PLOW_MOE_ENC_FP8BLK = 1, PLOW_MOE_ENC_MXFP4 = 2 };

/* Arms of ops 85/86 (i7; runtime/amd/interp.hip:6500-6604). 0, 1 and 2/3 are the reference's; 8 is
 * this library's name for "mxfp4 weights, bf16 activations" on gathered rows (the arithmetic of the
 * reference's decode ops 48/49 at enc 2).
 * At enc 2 arm 0 is the reference's default there, fp4 on both operands (runtime/amd/op_moe.h:3948-4720):
 *   85: t0=fu mxfp4 [R][I/2] (out) t1=x bf16 [T][H] t2=wtab t3=stab (E8M0 rows [N][K/32]) t4=meta
 *       t5=row_token t6=row_partidx (rows it marks unused are skipped) t7=E8M0 rows [R][I/32] (out)
 *       i4 = T, the rows of t1 (an extension of this library, which quantizes every token row once ahead
 *       of the GEMM; needs a context); I and H multiples of 256, at least 512
 *   86: t0=part (arm 0: f32, arm 1: bf16) t1=fu mxfp4 t5=its E8M0 rows, the rest as on the other arms */
enum {
    PLOW_MOE_ARM_A16       = 0, /* bf16 activations (enc 0 bf16 weights, enc 1 W8A16)             */
    PLOW_MOE_ARM_A4W4      = 0, /* enc 2: mxfp4 activations, quantized per 32 values by the GLU op  */
    PLOW_MOE_ARM_A4W4_P16  = 1, /* DOWN only, enc 2: as 0 with a bf16 part                         */
    PLOW_MOE_ARM_W8A8      = 2, /* enc 1: e4m3 activations with 1x128 scales; DOWN writes f32 part */
    PLOW_MOE_ARM_W8A8_P16  = 3, /* DOWN only: as 2 with a bf16 part                                */
    /* enc 1, two-term e4m3 activations x ~= s * (hi + lo / 16) per 1x128 group, about the precision of bf16
     * (runtime/amd/moe_pf_w8a8.h:81-92, :115-117; interp.hip:6509-6518, :6560-6571). 85 arm 4: t1 = bf16 x rows,
     * t0 = fq rows [hi I | lo I] (2 I bytes), t7 = fs f32 [rows][I / 128]. 86 arm 4 (f32 part) / 5 (bf16 part): t1 =
     * those fq rows, t5 = fs. Served on the bf16-activation kernels over the context's staging, which holds the
     * aligned intermediate rows as bf16 (rows * I * 2 bytes; the routed row count must be known: an align op in the
     * same run or fj[2]): the GLU multiplies the bf16 rows themselves where the reference multiplies their two
     * terms, and writes the two-term rows; the DOWN multiplies bf16(s * (hi + lo / 16)) */
    PLOW_MOE_ARM_W8A8_SPLIT     = 4,
    PLOW_MOE_ARM_W8A8_SPLIT_P16 = 5, /* DOWN only */
    PLOW_MOE_ARM_W8A8_XQ   = 6, /* GLU only, enc 1: t1 holds the bf16 rows, quantized 1x128 where they
                                   are loaded; equals op 184 + arm 2 bit for bit, writes arm 2's fq / fs
                                   (runtime/amd/moe_pf_w8a8.h:118-121); t6 unused. i4 is unused by the
                                   reference; here a non-zero i4 states the rows of t1, which lets a batch
                                   of many rows per expert run as quantizer + tiled arm 2 over the
                                   context's staging (see plow_moe_reserve_staging: rows * (H + H / 32)
                                   bytes); 0, or rows that do not fit, keep the streaming form         */
    PLOW_MOE_ARM_W4A16     = 8
};

/* GLU activations (i5; runtime/amd/op_moe.h:216-241, golden/golden.h:107-133). */
enum {
    PLOW_MOE_ACT_GELU_TANH = 0,
    PLOW_MOE_ACT_SILU = 1,
    PLOW_MOE_ACT_SITU = 2,         /* pair form, fj[0] = beta, fj[1] = linear beta */
    PLOW_MOE_ACT_SWIGLU_OAI = 3,   /* pair form, fj[0] = alpha, fj[1] = limit (> 0) */
    PLOW_MOE_ACT_SWIGLU_CLAMP = 4  /* pair form, fj[1] = limit */
};

/* Router flags (i3 of ops 56/83; runtime/amd/op_moe.h:453-467). */
enum {
    PLOW_ROUTE_SIGMOID   = 1u, /* else softmax */
    PLOW_ROUTE_NORM_TOPK = 2u,
    PLOW_ROUTE_BIAS      = 4u, /* t3 is bound */
    PLOW_ROUTE_F32_LOGIT = 8u,
    /* selection by a [vocab][k] lookup table instead of by score. Refused: the reference's dispatch of ops 56 / 83
     * binds no table either (runtime/amd/interp.hip:6485-6488 passes null for it) */
    PLOW_ROUTE_HASH      = 16u,
    /* score = sqrt(softplus(logit)) = sqrtf(log1pf(expf(-|l|)) + max(l, 0)), a third transform beside sigmoid
     * and softmax (runtime/amd/op_moe.h:485-494); takes precedence over bit 0 as there */
    PLOW_ROUTE_SQRT_SOFTPLUS = 32u
};

/* ---- error codes -------------------------------------------------------------------------------- */
enum {
    PLOW_MOE_OK           = 0,
    PLOW_MOE_EINVAL       = -22, /* malformed descriptor / operand wiring / geometry                */
    PLOW_MOE_EUNSUPPORTED = -95, /* opcode, encoding or arm this library refuses                    */
    PLOW_MOE_EDEVICE      = -5,  /* a HIP call failed; plow_moe_last_error has the text             */
    PLOW_MOE_ENOMEM       = -12,
    PLOW_MOE_ROLLBACK     = 1    /* segment entry points only: the knob says "leave it to the
                                  * interpreter" (config.rs:2023-2060, value 0 or rows < min_rows) */
};

typedef struct PlowMoeCtx PlowMoeCtx;

/* ABI marker, the analogue of the `plow_moe_lt_abi` word plowrt reads from a loaded object
 * (crates/plowrt/src/exec/gpu/moe_lt.rs:713-724). */
uint32_t plow_moe_abi(void);

/* Create / destroy an operator context on HIP device `device`. The context owns a fixed workspace
 * (routing scratch of the slot-major ops), PLOW_MOE_STAGE_DEFAULT_BYTES of staging for the fp4 x fp4
 * arm, and a second stream with two events (a run's dense shared-expert ops are launched there beside the
 * routed experts, forked off and joined back to the caller's stream inside the run); no op allocates, frees
 * or waits for the device (the ownership contract of runtime/cpu/dev/cpu_dev.h:5-7). Replaces the per-engine load step of moe_lt.rs:697-814. */
int  plow_moe_create(PlowMoeCtx** out, int device);
void plow_moe_destroy(PlowMoeCtx* ctx);

/* Staging of the fp4 x fp4 arm (op 85 at enc 2, arm 0 quantizes its token rows to mxfp4 once, ahead of the
 * GEMM): rows * (H / 2 + H / 32) bytes, each part rounded up to 256. A context starts with
 * PLOW_MOE_STAGE_DEFAULT_BYTES (8192 rows of width 7168); an op 85 whose i4 rows do not fit is refused with
 * PLOW_MOE_EINVAL before anything of its run is launched. This call makes room for `token_rows` rows of
 * width `hidden`: it allocates (call it at set-up, never under stream capture), keeps every earlier block
 * until plow_moe_destroy (graphs captured before stay valid) and returns PLOW_MOE_ENOMEM after seven
 * growths or when the device is out of memory. No counterpart in the reference, which quantizes every
 * gathered row inside its GEMM kernel (runtime/amd/op_moe.h:3948-4720).
 * The same block is the scratch of three other ops, each of which writes what it keeps there and reads it back
 * before it returns its last launch (ops of one context therefore belong on one stream at a time): op 85 arm 6 at
 * many rows (rows * (H + H / 32) bytes), the two-term arms 4 / 5 of ops 85 / 86 (aligned rows * I * 2 bytes: refused
 * when they do not fit) and the dense ops 20 / 8 (K-slice partial sums of a few rows, or the one-expert tables of
 * many: kept on their plain form when they do not fit). */
#define PLOW_MOE_STAGE_DEFAULT_BYTES (32u << 20)
int plow_moe_reserve_staging(PlowMoeCtx* ctx, size_t token_rows, size_t hidden);

/* Text of the last failure on this context (valid until the next call on it). */
const char* plow_moe_last_error(const PlowMoeCtx* ctx);

/* Execute ONE op descriptor asynchronously on `stream` (a hipStream_t; NULL = the null stream).
 * `tensors` is the handle table: tensors[inst->t[j]] is a device pointer. Replaces the
 * per-instruction dispatch of runtime/amd/interp.hip:6202-6635 and the CPU twin's
 * plow_cpu_kernel(op)(inst, slice, nblk, tensors, ctx) (runtime/cpu/dev/cpu_dev.h:172-176); the
 * (slice, nblk) split is internal here. */
int plow_moe_exec(PlowMoeCtx* ctx, const PlowDevInst* inst, void* const* tensors, void* stream);

/* Execute a run of descriptors in order on `stream`. */
int plow_moe_exec_many(PlowMoeCtx* ctx, const PlowDevInst* insts, uint32_t n_inst,
                       void* const* tensors, void* stream);

/* Segment-level entry points: the moe_pf_lt / moe_dec_lt variants. `insts[0..n_inst)` is one MoE
 * segment as plowrt isolates it: the grouped GLU + DOWN pair (ops 85+86, 81+82 or 48+49), optionally
 * preceded by its router/align/quant prologue and followed by its combine. The run is validated as
 * a whole (operand wiring between the ops, geometry, encodings; moe_lt.rs:159-248) and refused with
 * PLOW_MOE_EINVAL before anything is launched. `rows` is the live token count of this step.
 * Knob semantics follow PLOW_MOE_PF_LT / PLOW_MOE_DEC_LT: see plow_moe_set_min_rows. */
int plow_moe_pf(PlowMoeCtx* ctx, const PlowDevInst* insts, uint32_t n_inst, void* const* tensors,
                uint32_t rows, void* stream);
int plow_moe_dec(PlowMoeCtx* ctx, const PlowDevInst* insts, uint32_t n_inst, void* const* tensors,
                 uint32_t rows, void* stream);

/* variant: 0 = prefill (plow_moe_pf), 1 = decode (plow_moe_dec).
 * min_rows < 0: unset, every segment is served; 0: the variant is switched off and the entry point
 * returns PLOW_MOE_ROLLBACK; N > 0: segments with rows < N return PLOW_MOE_ROLLBACK. */
int plow_moe_set_min_rows(PlowMoeCtx* ctx, int variant, int min_rows);

/* plow_moe_exec for callers that cannot allocate. It has no counterpart in the reference: it is for code
 * under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc, where even creating a
 * context (which allocates its workspace) is not possible. It takes no context and calls no allocating
 * routine. Every op of plow_moe_exec is served except op 85 on the fp4 x fp4 arm (enc 2, arm 0), whose
 * staging block belongs to a context: it is refused with PLOW_MOE_EUNSUPPORTED. The ops that need a workspace (slot-major decode experts 48 /
 * 49 / 65 / 66, flat mxfp4 150 - 153) take it from a static device array inside the library (1 MiB per GPU,
 * held until the process ends), which limits them to PLOW_MOE_NOALLOC_MAX_SLOTS routed slots and
 * PLOW_MOE_NOALLOC_MAX_EXPERTS experts: larger calls are refused with PLOW_MOE_EINVAL and a text in `err`
 * (err may be NULL). The op runs on the CURRENT device. All calls on one GPU share that GPU's array: calls
 * that overlap there (two streams, two threads) race; calls on one stream are safe. Nothing in the array
 * has to start at zero and nothing is kept in it between calls. The first call on a device sets the device
 * up (no stream work); inst == NULL does only that, e.g. before a capture begins. */
#define PLOW_MOE_NOALLOC_MAX_SLOTS 4096u
#define PLOW_MOE_NOALLOC_MAX_EXPERTS 1056u
int plow_moe_exec_noalloc(const PlowDevInst* inst, void* const* tensors, void* stream, char* err, size_t err_len);

/* Validate one descriptor against this library's contract without launching (0 = would run). */
int plow_moe_check(PlowMoeCtx* ctx, const PlowDevInst* inst, void* const* tensors);

#ifdef __cplusplus
}
#endif
#endif /* PLOW_MOE_H */
