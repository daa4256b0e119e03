/* api.hip — the C-ABI of the operator (include/plow_moe.h): context, descriptor validation and the
 * op -> kernel dispatch. Host code only; the kernels live in the other translation units.
 *
 * The validation mirrors what plow's host does before it launches a native MoE segment: typed refusal
 * of wrong wiring or geometry before anything is enqueued (crates/plowrt/src/exec/gpu/moe_lt.rs:
 * 159-248, crates/plowrt/src/exec/amd.rs:3450-3480). */
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <new>

#include "../../include/plow_moe.h"
#include "kernels.h"
#include "tuning.h"

/* Slot-major ops (48 / 49 / 65 / 66, 150 / 151) are served by sorting their slots by expert into a
 * workspace first, so that every hit expert streams its weights once; the flat-tensor ops (150 - 153)
 * build their per-expert pointer tables there. A context owns one sized for WS_MAX_SLOTS slots;
 * plow_moe_exec_noalloc carves a smaller one out of the library's static device array. Nothing in a
 * workspace has to start at zero: every word a kernel reads was written earlier in the same call. */
#define WS_MAX_E 1056u
#define WS_MAX_SLOTS (1u << 20)

struct Workspace {
    uint32_t max_e, max_slots, max_chunks;
    int32_t* meta;        /* [3 * max_e + 1] */
    uint32_t* row_token;  /* [max_slots + max_e * (PLOW_MPF_BM - 1)] */
    uint32_t* row_partidx;
    float* row_gate;
    uint32_t* chunk_hist; /* [max_chunks][max_e] scratch of the multi-workgroup align */
    uint64_t* ftab;       /* [2][max_e][3] pointer tables built for the flat-tensor ops (150 - 153) */
    uint32_t* form_words; /* [WS_FORM_WORDS] device-side form choices of grouped ops issued without a row count */
};
#define WS_FORM_WORDS 64u
static constexpr size_t ws_up(size_t v) { return (v + 255u) & ~(size_t)255u; }
static constexpr size_t ws_rows(uint32_t max_e, uint32_t max_slots) { return (size_t)max_slots + (size_t)max_e * (PLOW_MPF_BM - 1u); }
/* bytes of one workspace laid out in a single 256-byte aligned block */
static constexpr size_t ws_bytes(uint32_t max_e, uint32_t max_slots) {
    return ws_up((3u * (size_t)max_e + 1u) * 4u) + 3u * ws_up(ws_rows(max_e, max_slots) * 4u) +
           ws_up((size_t)((max_slots + 1023u) / 1024u) * max_e * 4u) + ws_up((size_t)2u * max_e * 3u * 8u) +
           ws_up(WS_FORM_WORDS * 4u);
}
static_assert(ws_bytes(PLOW_MOE_NOALLOC_MAX_EXPERTS, PLOW_MOE_NOALLOC_MAX_SLOTS) <= PLOW_MOE_STATIC_BYTES,
              "the static device array must hold the workspace of the largest call plow_moe_exec_noalloc accepts");
static Workspace ws_carve(void* base, uint32_t max_e, uint32_t max_slots) {
    Workspace w = {};
    char* p = (char*)base;
    w.max_e = max_e, w.max_slots = max_slots, w.max_chunks = (max_slots + 1023u) / 1024u;
    w.meta = (int32_t*)p, p += ws_up((3u * (size_t)max_e + 1u) * 4u);
    const size_t rb = ws_up(ws_rows(max_e, max_slots) * 4u);
    w.row_token = (uint32_t*)p, p += rb;
    w.row_partidx = (uint32_t*)p, p += rb;
    w.row_gate = (float*)p, p += rb;
    w.chunk_hist = (uint32_t*)p, p += ws_up((size_t)w.max_chunks * max_e * 4u);
    w.ftab = (uint64_t*)p, p += ws_up((size_t)2u * max_e * 3u * 8u);
    w.form_words = (uint32_t*)p;
    return w;
}

/* Staging of the fp4 x fp4 arm (op 85 at enc 2, arm 0): its token rows, quantized to mxfp4 ahead of the
 * GEMM. A context is created with PLOW_MOE_STAGE_DEFAULT_BYTES of it and plow_moe_reserve_staging grows it
 * outside the op path; an op whose batch does not fit is refused before anything is launched. A block
 * that kernels have been given is never freed before plow_moe_destroy: a graph captured earlier keeps
 * pointing at memory that is still the context's. */
#define STAGE_MAX_BLOCKS 8u
struct PlowMoeCtx {
    int device;
    int min_rows[2]; /* [0] prefill, [1] decode; < 0 unset */
    char err[256];
    void* ws_base;   /* the context's own allocation behind `ws` (NULL when `ws` is borrowed) */
    Workspace ws;
    uint32_t form_seq; /* the next of the workspace's form words to hand out (they rotate) */
    void* stage_blocks[STAGE_MAX_BLOCKS]; /* every block ever allocated; the last one is in use */
    uint32_t n_stage;
    void* stage;
    size_t stage_bytes;
    /* a second stream (default priority) and the two events that fork it off the caller's stream and join it back:
     * the dense shared-expert ops of a run go there while the routed experts run (exec_run) */
    hipStream_t side;
    hipEvent_t ev_fork, ev_join;
};

/* bytes of staging the fp4 x fp4 GLU needs for `rows` token rows of width H */
static size_t stage_need(size_t rows, size_t H) { return ws_up(rows * (H / 2u)) + ws_up(rows * (H / 32u)); }

/* A larger staging block on the context's device. Never called from an op: it allocates. The block in use so
 * far stays allocated (work already queued, or a captured graph, may still read it). */
static int stage_grow(PlowMoeCtx* c, size_t bytes) {
    if (bytes <= c->stage_bytes) return 0;
    if (c->n_stage >= STAGE_MAX_BLOCKS) return PLOW_MOE_ENOMEM;
    int prev = 0;
    (void)hipGetDevice(&prev);
    (void)hipSetDevice(c->device);
    void* p = nullptr;
    const bool ok = hipMalloc(&p, bytes) == hipSuccess;
    (void)hipSetDevice(prev);
    if (!ok) {
        (void)hipGetLastError();
        return PLOW_MOE_ENOMEM;
    }
    c->stage_blocks[c->n_stage++] = p;
    c->stage = p, c->stage_bytes = bytes;
    return 0;
}

static int fail(PlowMoeCtx* c, int code, const char* fmt, ...) {
    if (c) {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(c->err, sizeof c->err, fmt, ap);
        va_end(ap);
    }
    return code;
}

static inline void* ten(const PlowDevInst* in, void* const* T, int k) {
    return in->t[k] == PLOW_TENSOR_NONE ? nullptr : T[in->t[k]];
}

extern "C" uint32_t plow_moe_abi(void) { return 1u; }
extern "C" void plow_moe_destroy(PlowMoeCtx* ctx);

extern "C" int plow_moe_create(PlowMoeCtx** out, int device) {
    if (!out) return PLOW_MOE_EINVAL;
    *out = nullptr;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || device < 0 || device >= n) return PLOW_MOE_EDEVICE;
    PlowMoeCtx* c = new (std::nothrow) PlowMoeCtx();
    if (c) memset(c, 0, sizeof *c);
    if (!c) return PLOW_MOE_ENOMEM;
    c->device = device;
    c->min_rows[0] = c->min_rows[1] = -1;
    c->err[0] = 0;
    const int src = plow_moe_device_setup(device); /* CU count, kernel attributes: once per device */
    if (src) {
        delete c;
        return src;
    }
    int prev = 0;
    (void)hipGetDevice(&prev);
    (void)hipSetDevice(device);
    const bool ok = hipMalloc(&c->ws_base, ws_bytes(WS_MAX_E, WS_MAX_SLOTS)) == hipSuccess;
    (void)hipSetDevice(prev);
    if (!ok) {
        plow_moe_destroy(c);
        return PLOW_MOE_ENOMEM;
    }
    c->ws = ws_carve(c->ws_base, WS_MAX_E, WS_MAX_SLOTS);
    if (stage_grow(c, PLOW_MOE_STAGE_DEFAULT_BYTES)) {
        plow_moe_destroy(c);
        return PLOW_MOE_ENOMEM;
    }
    (void)hipGetDevice(&prev);
    (void)hipSetDevice(device);
    const bool side_ok = hipStreamCreateWithFlags(&c->side, hipStreamNonBlocking) == hipSuccess &&
                         hipEventCreateWithFlags(&c->ev_fork, hipEventDisableTiming) == hipSuccess &&
                         hipEventCreateWithFlags(&c->ev_join, hipEventDisableTiming) == hipSuccess;
    (void)hipSetDevice(prev);
    if (!side_ok) {
        plow_moe_destroy(c);
        return PLOW_MOE_EDEVICE;
    }
    *out = c;
    return 0;
}

extern "C" int plow_moe_reserve_staging(PlowMoeCtx* ctx, size_t token_rows, size_t hidden) {
    if (!ctx || !ctx->ws_base) return PLOW_MOE_EINVAL;
    ctx->err[0] = 0;
    const size_t need = stage_need(token_rows, hidden);
    if (need <= ctx->stage_bytes) return 0;
    const int rc = stage_grow(ctx, need);
    if (rc) return fail(ctx, rc, "plow_moe_reserve_staging: %zu bytes could not be allocated (a context grows its staging at most %u times; "
                                 "allocation is refused while a stream capture is active)", need, STAGE_MAX_BLOCKS - 1u);
    return 0;
}

extern "C" void plow_moe_destroy(PlowMoeCtx* ctx) {
    if (!ctx) return;
    if (ctx->ev_fork) (void)hipEventDestroy(ctx->ev_fork);
    if (ctx->ev_join) (void)hipEventDestroy(ctx->ev_join);
    if (ctx->side) (void)hipStreamDestroy(ctx->side);
    (void)hipFree(ctx->ws_base);
    for (uint32_t n = 0; n < ctx->n_stage; n++) (void)hipFree(ctx->stage_blocks[n]);
    delete ctx;
}

extern "C" const char* plow_moe_last_error(const PlowMoeCtx* ctx) { return ctx ? ctx->err : "no context"; }

extern "C" int plow_moe_set_min_rows(PlowMoeCtx* ctx, int variant, int min_rows) {
    if (!ctx || variant < 0 || variant > 1) return PLOW_MOE_EINVAL;
    ctx->min_rows[variant] = min_rows;
    return 0;
}

/* ---- per-op validation + launch --------------------------------------------------------------- */

#define NEED(c, cond, ...) \
    do { if (!(cond)) return fail(c, PLOW_MOE_EINVAL, __VA_ARGS__); } while (0)

/* What a call knows about the batch beyond the descriptor in hand. Nothing of it outlives the call: the
 * kernel form of an op never depends on what ran on the context before.
 *   form   0 / 1: the segment entry points' variant (decode: weight-streaming kernels, prefill: tiled
 *          kernels), -1: decide per op from its row count
 *   slots  routed slots (T * k) of the align op of the same run, 0 = the run has none */
struct Hint {
    int form;
    uint32_t slots;
    /* The sort of a routing table that a slot-major op (48 / 49 / 65 / 66, 150 / 151) of THIS run left in the
     * workspace: the next op of the run over the same table takes it instead of sorting again (a decode layer's
     * DOWN after its GLU). Forgotten with the run, and within it whenever an op that writes routing tables runs. */
    const void* sorted_table;
    uint32_t sorted_nslot, sorted_E, sorted_kx;
};

/* Routed slots of the batch as far as this op can know them: the descriptor's own statement (fj[2].u,
 * an extension of this library: no MoE op of the reference uses the third immediate), else the align op
 * of the same run, else what the op's own operands imply (`own`, 0 = nothing). */
/* aligned rows of a batch of `slots` routed rows over E experts at most (every expert's last tile of 64 may be
 * partial); 0 when the slot count is unknown or the bound does not fit 32 bits */
static uint32_t split_rows_bound(uint32_t slots, uint32_t E) {
    const uint64_t b = (uint64_t)slots + (uint64_t)E * (PLOW_MPF_BM - 1u);
    return slots && b <= 0xFFFFFFFFull ? (uint32_t)(((b + PLOW_MPF_BM - 1u) / PLOW_MPF_BM) * PLOW_MPF_BM) : 0u;
}

static uint32_t slots_of(const PlowDevInst* in, const Hint& h, uint32_t own) {
    if (in->fj[2].u) return in->fj[2].u;
    if (h.slots) return h.slots;
    return own;
}

/* Tiled or weight-streaming form of the fp8 x fp8 grouped GEMMs: the tiled one from 16 rows per expert on
 * average (the measured crossover), when it serves the shape; unknown row counts take the streaming form,
 * which is right at every size and fast at small ones. */
/* Routed rows up to which the fp8 x fp8 DOWN runs as matrix-vector products (measured against the streaming
 * kernel, DeepSeek-V3 shape) */
#define W8A8_GEMV_MAX_SLOTS 36u
/* Tiled forms: the weight rows of an expert with a single row tile are read once and may be loaded non-temporal
 * (the kernel decides that per expert; this is the launch's permission). DOWN: always (measured better from
 * 16 to 143 rows per expert on average: DeepSeek-V3 shape 512 tokens 750 -> 698 us, 4096: 1069 -> 1052; Qwen3
 * 512: 192 -> 175). GLU: up to 80 rows per expert on average (DeepSeek-V3 shape 512 tokens 1301 -> 1179 us,
 * 2048: 1386 -> 1334, 3072: 1577 -> 1618, not taken; fp4 x fp4 arm, Kimi-K2 shape, 3072: 1404 -> 1356) */
static uint32_t tiled_w_nt(uint32_t slots, uint32_t E, bool glu) {
    const int env = plow_moe_tuning().tiled_nt;
    if (env >= 0) return (uint32_t)env;
    return !glu || (slots != 0u && slots <= 80u * E) ? 1u : 0u;
}
static bool want_tiled(const Hint& h, uint32_t slots, const GroupW8A8& g) {
    const int env = plow_moe_tuning().w8a8_kernel;
    const bool tiled = env >= 0 ? env == 1 : h.form >= 0 ? h.form == 1 : slots >= 16u * g.E;
    return tiled && group_w8a8_tiled_serves(g);
}

/* One fp8 x fp8 grouped op. With a row count (or a form stated by the segment entry points or the
 * environment) the host picks the form. Without one - a caller that issues its ops one at a time and fills
 * no fj[2], as plow's interpreter does (runtime/amd/interp.hip:6556-6604) - the count exists only on the
 * device, in meta: a one-workgroup launch adds it up into a word of the workspace, and both forms are
 * launched behind it; every workgroup of the form the word does not name returns at once (a few microseconds
 * per op, where the wrong form costs up to twenty times the op). */
static uint32_t* next_form_word(PlowMoeCtx* c) { return c->ws.form_words + (c->form_seq++ % WS_FORM_WORDS); }

static int launch_w8a8(PlowMoeCtx* c, const Hint& h, uint32_t slots, GroupW8A8& g, bool glu, hipStream_t st) {
    g.slots_bound = slots;
    g.w_nt = tiled_w_nt(slots, g.E, glu);
    const bool open = slots == 0u && h.form < 0 && plow_moe_tuning().w8a8_kernel < 0 && plow_moe_tuning().form_on_device;
    if (!open || !group_w8a8_tiled_serves(g)) {
        if (want_tiled(h, slots, g)) return glu ? launch_group_glu_w8a8_tiled(g, st) : launch_group_down_w8a8_tiled(g, st);
        return glu ? launch_group_glu_w8a8(g, st) : launch_group_down_w8a8(g, st);
    }
    uint32_t* const word = next_form_word(c);
    int rc = launch_pick_form(word, g.meta, g.E, st);
    if (rc) return rc;
    g.form_word = word;
    g.form_want = 0u;
    rc = glu ? launch_group_glu_w8a8(g, st) : launch_group_down_w8a8(g, st);
    if (rc) return rc;
    g.form_want = 1u;
    return glu ? launch_group_glu_w8a8_tiled(g, st) : launch_group_down_w8a8_tiled(g, st);
}

/* the workspace's sort serves this op: same table, slot count and expert count; the GLU also needs the same slots
 * per input row (its row_token = slot / kx), the DOWN reads no row_token */
static bool sort_reusable(const Hint& h, const void* table, uint32_t nslot, uint32_t E, uint32_t kx, bool glu) {
    return h.sorted_table != nullptr && h.sorted_table == table && h.sorted_nslot == nslot && h.sorted_E == E && (!glu || h.sorted_kx == kx);
}

#define ROUTE_FLAGS_SERVED (PLOW_ROUTE_SIGMOID | PLOW_ROUTE_NORM_TOPK | PLOW_ROUTE_BIAS | PLOW_ROUTE_F32_LOGIT | PLOW_ROUTE_SQRT_SOFTPLUS)
static int run_op(PlowMoeCtx* c, const PlowDevInst* in, void* const* T, hipStream_t st, bool launch, Hint& h) {
    const uint32_t* i = in->i;
    if (launch && (in->op == PLOW_DOP_MOE_ROUTER_TOPK || in->op == PLOW_DOP_MOE_ROUTER_TOPK_PF || in->op == PLOW_DOP_GEMM_F32))
        h.sorted_table = nullptr; /* routing tables may change under the sort the workspace holds */
    switch (in->op) {
    case PLOW_DOP_GEMM_F32: {
        NEED(c, ten(in, T, 0) && ten(in, T, 1) && ten(in, T, 2), "op 180: t0 logits, t1 x, t2 W must be bound");
        NEED(c, i[0] && i[1] && i[2] && i[2] % 8u == 0u, "op 180: M, N, K must be non-zero and K a multiple of 8");
        if (i[7] == PLOW_ROUTER_RAW_MARK) {
            /* the score carries its top-k (plow crates/packet/src/dev.rs:90-94): one launch where the few-token
             * score kernel serves the shape, the two launches otherwise; the same bytes either way */
            const uint32_t E = i[1], k = i[3], flags = i[4], ng = i[6] & 0xFFFFu, tg = i[6] >> 16;
            NEED(c, ten(in, T, 3) && ten(in, T, 5), "op 180 (router): t3 table and t5 counters must be bound");
            NEED(c, E <= 1024u && k >= 1u, "op 180 (router): n_exp %u above 1024 or k = 0", E);
            NEED(c, (flags & PLOW_ROUTE_F32_LOGIT) != 0u, "op 180 (router): the top-k reads the f32 logits, flag bit 3 must be set");
            NEED(c, (flags & ~ROUTE_FLAGS_SERVED) == 0u, "op 180 (router): flags 0x%x ask for hash selection (bit 4, no table operand on this op) or an unknown transform", flags);
            NEED(c, ((flags & PLOW_ROUTE_BIAS) != 0u) == (ten(in, T, 4) != nullptr), "op 180 (router): bias flag (bit 2) and the t4 binding disagree");
            if (ng > 1u && tg > 0u && tg < ng)
                NEED(c, ng <= PLOW_ROUTE_MAX_GROUPS && E % ng == 0u && E / ng >= 2u && (uint64_t)tg * (E / ng) >= (k < 16u ? k : 16u),
                     "op 180 (router): group shape n_group=%u topk_group=%u is not selectable for n_exp=%u k=%u", ng, tg, E, k);
            if (i[5] & ~1u) return fail(c, PLOW_MOE_EUNSUPPORTED, "op 180 (router): i5 = %u asks for a signal to the interpreter's counters", i[5]);
            if (!launch) return 0;
            RouterRun r = {};
            r.logit = ten(in, T, 0), r.x = ten(in, T, 1), r.w = ten(in, T, 2), r.M = i[0], r.N = E, r.K = i[2];
            r.table = ten(in, T, 3), r.bias = (const float*)ten(in, T, 4), r.row_ctr = (uint32_t*)ten(in, T, 5);
            r.k = k, r.flags = flags, r.tail = i[5] & 1u, r.n_group = ng, r.topk_group = tg;
            r.route_scale = in->fj[0].f;
            if (router_decode_serves(r)) return launch_router_decode(r, st);
            const int src = launch_router_score((float*)r.logit, r.x, r.w, r.M, r.N, r.K, st);
            if (src) return src;
            return launch_router_topk(r.table, r.logit, r.bias, E, k, flags, r.M, r.tail, ng, tg, r.route_scale, 0.0f, st);
        }
        if (!launch) return 0;
        return launch_router_score((float*)ten(in, T, 0), ten(in, T, 1), ten(in, T, 2), i[0], i[1], i[2], st);
    }
    case PLOW_DOP_MOE_ROUTER_TOPK:
    case PLOW_DOP_MOE_ROUTER_TOPK_PF: {
        const bool pf = in->op == PLOW_DOP_MOE_ROUTER_TOPK_PF;
        const uint32_t E = i[1], k = i[2], flags = i[3], rows = i[4] ? i[4] : 1u;
        NEED(c, ten(in, T, 0) && ten(in, T, 1), "router top-k: t0 table and t1 logits must be bound");
        NEED(c, E >= 1u && E <= 1024u, "router top-k: n_exp %u outside 1..1024", E);
        NEED(c, k >= 1u, "router top-k: k = 0");
        NEED(c, (flags & ~ROUTE_FLAGS_SERVED) == 0u, "router top-k: flags 0x%x ask for hash selection (bit 4, no table operand on this op) or an unknown transform", flags);
        /* the bias operand is read by the GPU reference only under flag bit 2 and by the CPU reference
         * whenever it is bound: a packet where the two disagree is ambiguous and refused */
        NEED(c, ((flags & PLOW_ROUTE_BIAS) != 0u) == (ten(in, T, 3) != nullptr),
             "router top-k: bias flag (bit 2) and the t3 binding disagree");
        if (i[6] > 1u && i[7] > 0u && i[7] < i[6])
            NEED(c, i[6] <= PLOW_ROUTE_MAX_GROUPS && E % i[6] == 0u && E / i[6] >= 2u &&
                        (uint64_t)i[7] * (E / i[6]) >= (k < 16u ? k : 16u),
                 "router top-k: group shape n_group=%u topk_group=%u is not selectable for n_exp=%u k=%u",
                 i[6], i[7], E, k);
        /* op 83 with t2 bound: the [T][i0] f64 accumulator of the deterministic fused combine, zeroed here
         * ahead of the chain that adds into it (plow runtime/amd/interp.hip:6479-6483) */
        double* const det_acc = pf ? (double*)ten(in, T, 2) : nullptr;
        NEED(c, !det_acc || (i[0] != 0u && (uintptr_t)det_acc % 16u == 0u), "op 83: the accumulator (t2) needs its width in i0 and 16-byte alignment");
        if (!launch) return 0;
        if (det_acc) {
            const int zrc = launch_zero_f64(det_acc, (size_t)rows * i[0], st);
            if (zrc) return zrc;
        }
        return launch_router_topk(ten(in, T, 0), ten(in, T, 1), (const float*)ten(in, T, 3), E, k, flags,
                                  rows, pf && i[5] ? 1u : 0u, i[6], i[7], in->fj[0].f, in->fj[1].f, st);
    }
    case PLOW_DOP_MOE_ALIGN_PF: {
        NEED(c, ten(in, T, 0) && ten(in, T, 1) && ten(in, T, 2) && ten(in, T, 3) && ten(in, T, 4),
             "op 84: t0 meta, t1 table, t2 row_token, t3 row_partidx, t4 row_gate must be bound");
        NEED(c, i[1] >= 1u && i[1] <= 1056u && i[2] >= 1u, "op 84: n_exp %u outside 1..1056 or k = 0", i[1]);
        NEED(c, (uint64_t)i[0] * i[2] < (1ull << 31), "op 84: T * k overflows");
        if (!launch) return 0;
        return launch_align((int32_t*)ten(in, T, 0), ten(in, T, 1), (uint32_t*)ten(in, T, 2),
                            (uint32_t*)ten(in, T, 3), (float*)ten(in, T, 4), i[0], i[1], i[2],
                            c->ws.chunk_hist, c->ws.max_chunks, st);
    }
    case PLOW_DOP_MOE_COMBINE:
    case PLOW_DOP_MOE_COMBINE_PF: {
        const bool pf = in->op == PLOW_DOP_MOE_COMBINE_PF;
        const uint32_t H = i[0], k = i[1], rows = pf ? (i[2] ? i[2] : 1u) : 1u;
        const size_t r0 = pf ? i[3] : 0u;
        const uint32_t p16 = pf && i[7] ? 1u : 0u;
        NEED(c, ten(in, T, 0) && ten(in, T, 3), "combine: t0 out and t3 part must be bound");
        NEED(c, H && H % 4u == 0u, "combine: H %u must be a non-zero multiple of 4", H);
        const bool det = pf && i[4] != 0u; /* part is the f64 [T][H] accumulator of the deterministic fused combine */
        NEED(c, !det || (k == 1u && !p16), "op 87: the f64 accumulator form (i4) takes k = 1 and no bf16 partials");
        if (!launch) return 0;
        const char* res = (const char*)ten(in, T, 1);
        const char* sh = (const char*)ten(in, T, 2);
        if (det)
            return launch_combine_det((char*)ten(in, T, 0) + r0 * H * 2u, res ? res + r0 * H * 2u : nullptr,
                                      sh ? sh + r0 * H * 2u : nullptr, (const double*)ten(in, T, 3) + r0 * H, H, rows, st);
        return launch_combine((char*)ten(in, T, 0) + r0 * H * 2u, res ? res + r0 * H * 2u : nullptr,
                              sh ? sh + r0 * H * 2u : nullptr,
                              (const char*)ten(in, T, 3) + r0 * k * H * (p16 ? 2u : 4u), H, k, rows, p16, st);
    }
    case PLOW_DOP_QUANT_FP8_BLOCK128: {
        NEED(c, ten(in, T, 0) && ten(in, T, 1) && ten(in, T, 2), "op 184: t0 xq, t1 x, t2 scale must be bound");
        NEED(c, i[0] && i[1] && i[1] % 128u == 0u, "op 184: K %u must be a non-zero multiple of 128", i[1]);
        NEED(c, i[2] == 0u || i[2] >= i[0], "op 184: scale pitch %u below M %u", i[2], i[0]);
        if (!launch) return 0;
        return launch_quant_block128(ten(in, T, 0), ten(in, T, 1), (float*)ten(in, T, 2), i[0], i[1], i[2], st);
    }
    case PLOW_DOP_QUANT_FP8: {
        NEED(c, ten(in, T, 0) && ten(in, T, 1) && ten(in, T, 2), "op 32: t0 xq, t1 x, t2 scale must be bound");
        NEED(c, !ten(in, T, 3) == !ten(in, T, 4), "op 32: gate (t3) and up (t4) must be bound together");
        NEED(c, i[0] && i[1], "op 32: M %u and K %u must be non-zero", i[0], i[1]);
        if (!launch) return 0;
        return launch_quant_row(ten(in, T, 0), ten(in, T, 1), (float*)ten(in, T, 2), ten(in, T, 3), ten(in, T, 4),
                                i[2], i[0], i[1], st);
    }
    case PLOW_DOP_RMSNORM: {
        NEED(c, ten(in, T, 0) && ten(in, T, 1), "op 1: t0 out and t1 x must be bound");
        NEED(c, !ten(in, T, 3) == !ten(in, T, 4), "op 1: quantized row (t3) and scale (t4) must be bound together");
        NEED(c, i[0] && i[1] && i[1] % 8u == 0u && i[1] <= 16384u, "op 1: rows %u, feat %u (a multiple of 8, at most 16384)", i[0], i[1]);
        const uint32_t mode = !ten(in, T, 3) ? 0u : (i[4] == 128u ? 2u : 1u);
        NEED(c, mode != 2u || i[1] % 128u == 0u, "op 1: 1x128 quantization needs feat %u to be a multiple of 128", i[1]);
        NEED(c, mode == 0u || i[2] == 0u, "op 1: the quantizing forms take no output row offset");
        NEED(c, i[3] == 0u && i[7] == 0u, "op 1: i3 / i7 variants are not served");
        if (!launch) return 0;
        return launch_rmsnorm(ten(in, T, 0), ten(in, T, 1), ten(in, T, 2), ten(in, T, 3), (float*)ten(in, T, 4), i[0], i[1],
                              i[2], in->fj[0].f, mode, st);
    }
    case PLOW_DOP_MOE_GLU_FP8_BLOCK128: {
        const uint32_t I = i[0], H = i[1], E = i[2], Tn = i[3];
        NEED(c, ten(in, T, 0) && ten(in, T, 1) && ten(in, T, 2) && ten(in, T, 3) && ten(in, T, 4) && ten(in, T, 5) && ten(in, T, 6),
             "op 188: t0 fu, t1 xq, t2 xscale, t3 wtab, t4 stab, t5 meta, t6 row_token must be bound");
        NEED(c, I && H && E && Tn, "op 188: zero geometry");
        NEED(c, I % 128u == 0u && H % 128u == 0u, "op 188: I %u and H %u must be multiples of 128", I, H);
        if (!launch) return 0;
        GroupW8A8 g = {};
        g.out = ten(in, T, 0); g.out_bf16 = 1;
        g.a = ten(in, T, 1); g.a_scale = (const float*)ten(in, T, 2);
        g.wtab = (const uint64_t*)ten(in, T, 3); g.stab = (const uint64_t*)ten(in, T, 4);
        g.meta = (const int32_t*)ten(in, T, 5); g.row_token = (const uint32_t*)ten(in, T, 6);
        g.N = I; g.K = H; g.E = E; g.pitch = Tn; g.T = Tn;
        /* SiLU, or the clamped SwiGLU when a limit is given (plow runtime/amd/op_gemm_common.h:1973-1981) */
        g.f1 = in->fj[1].f; g.act = g.f1 > 0.0f ? PLOW_MOE_ACT_SWIGLU_CLAMP : PLOW_MOE_ACT_SILU;
        return launch_w8a8(c, h, slots_of(in, h, 0u), g, true, st);
    }
    case PLOW_DOP_MOE_QUANT_FP8_BLOCK128: {
        NEED(c, ten(in, T, 0) && ten(in, T, 1) && ten(in, T, 2) && ten(in, T, 3) && ten(in, T, 4) && ten(in, T, 5),
             "op 189: t0 hq, t1 fu, t2 hscale, t3 meta, t4 row_partidx, t5 out must be bound");
        NEED(c, i[0] && i[1] && i[2] && i[3] && i[4], "op 189: zero geometry");
        NEED(c, i[0] % 128u == 0u && i[4] % 4u == 0u, "op 189: I %u must be a multiple of 128 and H %u of 4", i[0], i[4]);
        if (!launch) return 0;
        return launch_quant_block128_scatter(ten(in, T, 0), ten(in, T, 1), (float*)ten(in, T, 2), ten(in, T, 3),
                                             ten(in, T, 4), ten(in, T, 5), i[0], i[1], i[2], i[3], i[4], st);
    }
    case PLOW_DOP_MOE_DOWN_FP8_BLOCK128: {
        const uint32_t I = i[0], H = i[1], E = i[2], topk = i[3], Tn = i[4];
        NEED(c, ten(in, T, 0) && ten(in, T, 1) && ten(in, T, 2) && ten(in, T, 3) && ten(in, T, 4) && ten(in, T, 5) &&
                    ten(in, T, 6) && ten(in, T, 7),
             "op 190: t0 out, t1 hq, t2 hscale, t3 wtab, t4 stab, t5 meta, t6 row_partidx, t7 row_gate must be bound");
        NEED(c, I && H && E && topk && Tn, "op 190: zero geometry");
        NEED(c, I % 128u == 0u && H % 128u == 0u, "op 190: I %u and H %u must be multiples of 128", I, H);
        if (!launch) return 0;
        GroupW8A8 g = {};
        g.out = ten(in, T, 0); g.acc_topk = topk;
        g.a = ten(in, T, 1); g.a_scale = (const float*)ten(in, T, 2); g.a_slots = Tn * topk;
        g.wtab = (const uint64_t*)ten(in, T, 3); g.stab = (const uint64_t*)ten(in, T, 4);
        g.meta = (const int32_t*)ten(in, T, 5);
        g.row_partidx = (const uint32_t*)ten(in, T, 6); g.row_gate = (const float*)ten(in, T, 7);
        g.N = H; g.K = I; g.E = E;
        return launch_w8a8(c, h, slots_of(in, h, Tn * topk), g, false, st);
    }
    case PLOW_DOP_MOE_GROUP_GLU_PF: {
        const uint32_t I = i[0], H = i[1], E = i[2], enc = i[3], arm = i[7];
        NEED(c, ten(in, T, 0) && ten(in, T, 1) && ten(in, T, 2) && ten(in, T, 4) && ten(in, T, 5),
             "op 85: t0 fu, t1 x, t2 wtab, t4 meta, t5 row_token must be bound");
        NEED(c, I && H && E, "op 85: zero geometry");
        if (enc == PLOW_MOE_ENC_FP8BLK && arm == PLOW_MOE_ARM_W8A8) {
            NEED(c, ten(in, T, 3) && ten(in, T, 6) && ten(in, T, 7), "op 85 W8A8: t3 stab, t6 xs, t7 fs must be bound");
            NEED(c, I % 128u == 0u && H % 128u == 0u, "op 85 W8A8: I %u and H %u must be multiples of 128", I, H);
            NEED(c, i[4] != 0u, "op 85 W8A8: i4 (row pitch of the activation scales) is zero");
            NEED(c, i[5] <= 2u || i[5] == PLOW_MOE_ACT_SWIGLU_CLAMP, "op 85: activation %u is not served", i[5]);
            if (!launch) return 0;
            GroupW8A8 g = {};
            g.out = ten(in, T, 0); g.out_scale = (float*)ten(in, T, 7);
            g.a = ten(in, T, 1); g.a_scale = (const float*)ten(in, T, 6);
            g.wtab = (const uint64_t*)ten(in, T, 2); g.stab = (const uint64_t*)ten(in, T, 3);
            g.meta = (const int32_t*)ten(in, T, 4); g.row_token = (const uint32_t*)ten(in, T, 5);
            g.N = I; g.K = H; g.E = E; g.pitch = i[4]; g.act = i[5];
            g.f0 = in->fj[0].f; g.f1 = in->fj[1].f;
            return launch_w8a8(c, h, slots_of(in, h, 0u), g, true, st);
        }
        if (enc == PLOW_MOE_ENC_FP8BLK && arm == PLOW_MOE_ARM_W8A8_XQ) {
            NEED(c, ten(in, T, 3) && ten(in, T, 7), "op 85 W8A8 (bf16 rows): t3 stab, t7 fs must be bound");
            NEED(c, I % 128u == 0u && H % 128u == 0u, "op 85 W8A8: I %u and H %u must be multiples of 128", I, H);
            NEED(c, i[5] <= 2u || i[5] == PLOW_MOE_ACT_SWIGLU_CLAMP, "op 85: activation %u is not served", i[5]);
            if (!launch) return 0;
            GroupW8A8 g = {};
            g.out = ten(in, T, 0); g.out_scale = (float*)ten(in, T, 7);
            g.a = ten(in, T, 1); g.a_bf16 = 1;
            g.wtab = (const uint64_t*)ten(in, T, 2); g.stab = (const uint64_t*)ten(in, T, 3);
            g.meta = (const int32_t*)ten(in, T, 4); g.row_token = (const uint32_t*)ten(in, T, 5);
            g.N = I; g.K = H; g.E = E; g.act = i[5];
            g.f0 = in->fj[0].f; g.f1 = in->fj[1].f;
            /* Many rows per expert, the caller states the rows of t1 in i4 (an extension of this library: the
             * reference leaves i4 unused on this arm) and the context's staging holds them: the rows are
             * quantized once, ahead of the GEMM, into the staging block, and the tiled form of arm 2 runs over
             * them - the arm's definition (quantizer op followed by arm 2, bit for bit), where the streaming
             * form would quantize every gathered row again in each of the expert's channel tiles. */
            const uint32_t Tn = i[4], slots = slots_of(in, h, 0u);
            const size_t qbytes = ws_up((size_t)Tn * H), sbytes = ws_up((size_t)Tn * (H / 128u) * 4u);
            if (Tn && c->ws_base && qbytes + sbytes <= c->stage_bytes) {
                GroupW8A8 t = g;
                t.a = c->stage; t.a_scale = (const float*)((uint8_t*)c->stage + qbytes); t.a_bf16 = 0; t.pitch = Tn; t.T = Tn;
                if (want_tiled(h, slots, t)) {
                    const int qrc = launch_quant_block128(c->stage, ten(in, T, 1), (float*)((uint8_t*)c->stage + qbytes), Tn, H, Tn, st);
                    if (qrc) return qrc;
                    t.slots_bound = slots;
                    t.w_nt = tiled_w_nt(slots, t.E, true);
                    return launch_group_glu_w8a8_tiled(t, st);
                }
            }
            /* the streaming form serves this arm at every row count */
            return launch_group_glu_w8a8(g, st);
        }
        /* two-term arm: the bf16-activation GLU into the staging, then the split of its rows */
        const bool split = enc == PLOW_MOE_ENC_FP8BLK && arm == PLOW_MOE_ARM_W8A8_SPLIT;
        const uint32_t split_rows = split ? split_rows_bound(slots_of(in, h, 0u), E) : 0u;
        if (split) {
            NEED(c, ten(in, T, 7), "op 85 two-term arm: t7 fs must be bound");
            NEED(c, c->ws_base && c->stage, "op 85 two-term arm: needs a context (its staging block)");
            NEED(c, split_rows != 0u, "op 85 two-term arm: the routed row count must be known (an align op in the same run, or fj[2])");
            NEED(c, (uint64_t)split_rows * I * 2u <= c->stage_bytes,
                 "op 85 two-term arm: %u aligned rows of width %u need %llu bytes of staging, the context holds %zu: call plow_moe_reserve_staging first",
                 split_rows, I, (unsigned long long)split_rows * I * 2u, c->stage_bytes);
        }
        const bool a16 = (enc == PLOW_MOE_ENC_BF16 && arm == PLOW_MOE_ARM_A16) ||
                         (enc == PLOW_MOE_ENC_FP8BLK && arm == PLOW_MOE_ARM_A16) || split ||
                         (enc == PLOW_MOE_ENC_MXFP4 && arm == PLOW_MOE_ARM_W4A16);
        if (a16) {
            NEED(c, enc == PLOW_MOE_ENC_BF16 || ten(in, T, 3), "op 85: t3 stab must be bound for encoding %u", enc);
            NEED(c, I % 128u == 0u && H % 128u == 0u, "op 85: I %u and H %u must be multiples of 128", I, H);
            NEED(c, i[5] <= 2u || i[5] == PLOW_MOE_ACT_SWIGLU_CLAMP, "op 85: activation %u is not served", i[5]);
            if (!launch) return 0;
            GroupA16 g = {};
            g.out = split ? c->stage : ten(in, T, 0); g.a = ten(in, T, 1);
            g.wtab = (const uint64_t*)ten(in, T, 2);
            g.stab = enc == PLOW_MOE_ENC_BF16 ? nullptr : (const uint64_t*)ten(in, T, 3);
            g.meta = (const int32_t*)ten(in, T, 4); g.a_idx = (const uint32_t*)ten(in, T, 5);
            g.N = I; g.K = H; g.E = E; g.enc = enc; g.act = i[5];
            g.f0 = in->fj[0].f; g.f1 = in->fj[1].f;
            g.wcols = 3; g.wsel0 = 0; g.wsel1 = 1;
            g.slots_hint = slots_of(in, h, 0u);
            if (!g.slots_hint && h.form != 0) g.form_ws = next_form_word(c); /* unknown rows: the form is chosen on the device */
            if (split) {
                const int grc = launch_group_glu_a16(g, st);
                if (grc) return grc;
                return launch_split_block128(ten(in, T, 0), (float*)ten(in, T, 7), c->stage, g.meta, g.a_idx, I, E, split_rows, st);
            }
            return launch_group_glu_a16(g, st);
        }
        if (enc == PLOW_MOE_ENC_MXFP4 && arm == PLOW_MOE_ARM_A4W4) {
            /* fp4 on both operands (plow runtime/amd/op_moe.h:3948-4720): the token rows are quantized to
             * mxfp4 once each, ahead of the GEMM, into the context's staging block (the reference quantizes
             * every gathered row inside its kernel: the same values, k times); the GLU's output leaves as
             * mxfp4 rows (t0) with their E8M0 rows (t7) */
            NEED(c, ten(in, T, 3) && ten(in, T, 6) && ten(in, T, 7), "op 85 A4W4: t3 stab, t6 row_partidx, t7 E8M0 rows must be bound");
            NEED(c, I % 256u == 0u && H % 256u == 0u && I >= 512u && H >= 512u, "op 85 A4W4: I %u and H %u must be multiples of 256, at least 512", I, H);
            NEED(c, i[4] != 0u, "op 85 A4W4: i4 (the number of token rows in t1) is zero");
            NEED(c, i[5] <= 2u || i[5] == PLOW_MOE_ACT_SWIGLU_CLAMP, "op 85: activation %u is not served", i[5]);
            NEED(c, (uint64_t)slots_of(in, h, 0u) / 128u + E <= 65535u, "op 85 A4W4: %u routed rows over %u experts exceed the 65535 row tiles the tiled kernel's directory counts", slots_of(in, h, 0u), E);
            if (!c->ws_base) return fail(c, PLOW_MOE_EUNSUPPORTED, "op 85 A4W4: needs a context (its staging block)");
            /* nothing is allocated here: the batch fits the context's staging or the op is refused */
            NEED(c, stage_need(i[4], H) <= c->stage_bytes,
                 "op 85 A4W4: %u token rows of width %u need %zu bytes of staging, the context holds %zu: call plow_moe_reserve_staging first",
                 i[4], H, stage_need(i[4], H), c->stage_bytes);
            if (!launch) return 0;
            const size_t qbytes = ws_up((size_t)i[4] * (H / 2u));
            uint8_t* const xq4 = (uint8_t*)c->stage;
            uint8_t* const xs = xq4 + qbytes;
            const int qrc = launch_quant_mx_act(xq4, xs, ten(in, T, 1), i[4], H, st);
            if (qrc) return qrc;
            GroupW8A8 g = {};
            g.out = ten(in, T, 0); g.out_e8m0 = (uint8_t*)ten(in, T, 7);
            g.a = xq4; g.a_e8m0 = xs;
            g.wtab = (const uint64_t*)ten(in, T, 2); g.stab = (const uint64_t*)ten(in, T, 3);
            g.meta = (const int32_t*)ten(in, T, 4); g.row_token = (const uint32_t*)ten(in, T, 5);
            g.row_partidx = (const uint32_t*)ten(in, T, 6);
            g.N = I; g.K = H; g.E = E; g.act = i[5]; g.T = i[4];
            g.f0 = in->fj[0].f; g.f1 = in->fj[1].f;
            g.slots_bound = slots_of(in, h, 0u);
            g.w_nt = tiled_w_nt(g.slots_bound, g.E, true);
            return launch_group_a4w4_tiled(g, true, st);
        }
        return fail(c, PLOW_MOE_EUNSUPPORTED, "op 85: encoding %u arm %u is not served", enc, arm);
    }
    case PLOW_DOP_MOE_GROUP_DOWN_PF: {
        const uint32_t H = i[0], I = i[1], E = i[2], enc = i[3], arm = i[7];
        NEED(c, ten(in, T, 0) && ten(in, T, 1) && ten(in, T, 2) && ten(in, T, 4) && ten(in, T, 6) && ten(in, T, 7),
             "op 86: t0 part, t1 fu, t2 wtab, t4 meta, t6 row_partidx, t7 row_gate must be bound");
        NEED(c, I && H && E, "op 86: zero geometry");
        /* i5: the deterministic fused combine. t0 is then the f64 [T][H] fixed-point accumulator (zeroed by
         * op 83) and every live row adds into row slot / k of it. The reference's encoding is log2(k) + 1
         * for a power-of-two k (plow runtime/amd/interp.hip:6596-6600); 256 + k states any k (an extension of
         * this library: a folded shared expert makes k = 9). */
        uint32_t det_k = 0u;
        if (i[5]) {
            NEED(c, i[5] <= 5u || (i[5] > 256u && i[5] <= 256u + 16u), "op 86: i5 = %u is neither log2(k) + 1 for k <= 16 nor 256 + k", i[5]);
            det_k = i[5] > 256u ? i[5] - 256u : 1u << (i[5] - 1u);
            NEED(c, enc == PLOW_MOE_ENC_FP8BLK && arm == PLOW_MOE_ARM_W8A8, "op 86: the deterministic fused combine (i5) is served on the block-fp8 W8A8 arm only");
        }
        if (enc == PLOW_MOE_ENC_FP8BLK && (arm == PLOW_MOE_ARM_W8A8 || arm == PLOW_MOE_ARM_W8A8_P16)) {
            NEED(c, ten(in, T, 3) && ten(in, T, 5), "op 86 W8A8: t3 stab and t5 fs must be bound");
            NEED(c, I % 128u == 0u && H % 128u == 0u, "op 86 W8A8: I %u and H %u must be multiples of 128", I, H);
            if (!launch) return 0;
            GroupW8A8 g = {};
            g.out = ten(in, T, 0);
            g.a = ten(in, T, 1); g.a_scale = (const float*)ten(in, T, 5);
            g.wtab = (const uint64_t*)ten(in, T, 2); g.stab = (const uint64_t*)ten(in, T, 3);
            g.meta = (const int32_t*)ten(in, T, 4);
            g.row_partidx = (const uint32_t*)ten(in, T, 6); g.row_gate = (const float*)ten(in, T, 7);
            g.N = H; g.K = I; g.E = E; g.part16 = arm == PLOW_MOE_ARM_W8A8_P16;
            g.det_k = det_k;
            if (!det_k) { /* a batch of a few rows: the matrix-vector form, every row spread over the whole chip */
                GroupA16 v = {};
                v.out = g.out; v.a = g.a; v.a_f8scale = g.a_scale; v.wtab = g.wtab; v.stab = g.stab; v.meta = g.meta;
                v.o_idx = g.row_partidx; v.gate = g.row_gate;
                v.N = H; v.K = I; v.E = E; v.enc = 1u /* block fp8 */; v.wcols = 3u; v.wsel0 = v.wsel1 = 2u;
                v.out_bf16 = g.part16; v.slots_hint = slots_of(in, h, 0u);
                if (v.slots_hint <= W8A8_GEMV_MAX_SLOTS && group_a16_gemv_serves(v)) return launch_group_a16_gemv(v, false, st);
            }
            return launch_w8a8(c, h, slots_of(in, h, 0u), g, false, st);
        }
        /* two-term arms: the rows back to bf16 in the staging, then the bf16-activation DOWN */
        const bool split = enc == PLOW_MOE_ENC_FP8BLK && (arm == PLOW_MOE_ARM_W8A8_SPLIT || arm == PLOW_MOE_ARM_W8A8_SPLIT_P16);
        const uint32_t split_rows = split ? split_rows_bound(slots_of(in, h, 0u), E) : 0u;
        if (split) {
            NEED(c, ten(in, T, 5), "op 86 two-term arm: t5 fs must be bound");
            NEED(c, c->ws_base && c->stage, "op 86 two-term arm: needs a context (its staging block)");
            NEED(c, split_rows != 0u, "op 86 two-term arm: the routed row count must be known (an align op in the same run, or fj[2])");
            NEED(c, (uint64_t)split_rows * I * 2u <= c->stage_bytes,
                 "op 86 two-term arm: %u aligned rows of width %u need %llu bytes of staging, the context holds %zu: call plow_moe_reserve_staging first",
                 split_rows, I, (unsigned long long)split_rows * I * 2u, c->stage_bytes);
        }
        const bool a16 = (enc == PLOW_MOE_ENC_BF16 && arm == PLOW_MOE_ARM_A16) ||
                         (enc == PLOW_MOE_ENC_FP8BLK && arm == PLOW_MOE_ARM_A16) || split ||
                         (enc == PLOW_MOE_ENC_MXFP4 && arm == PLOW_MOE_ARM_W4A16);
        if (a16) {
            NEED(c, enc == PLOW_MOE_ENC_BF16 || ten(in, T, 3), "op 86: t3 stab must be bound for encoding %u", enc);
            NEED(c, I % 128u == 0u && H % 128u == 0u, "op 86: I %u and H %u must be multiples of 128", I, H);
            if (!launch) return 0;
            if (split) {
                const int jrc = launch_join_block128(c->stage, ten(in, T, 1), (const float*)ten(in, T, 5), (const int32_t*)ten(in, T, 4),
                                                     (const uint32_t*)ten(in, T, 6), I, E, split_rows, st);
                if (jrc) return jrc;
            }
            GroupA16 g = {};
            g.out = ten(in, T, 0); g.a = split ? c->stage : ten(in, T, 1);
            g.out_bf16 = arm == PLOW_MOE_ARM_W8A8_SPLIT_P16 ? 1u : 0u;
            g.wtab = (const uint64_t*)ten(in, T, 2);
            g.stab = enc == PLOW_MOE_ENC_BF16 ? nullptr : (const uint64_t*)ten(in, T, 3);
            g.meta = (const int32_t*)ten(in, T, 4);
            g.o_idx = (const uint32_t*)ten(in, T, 6); g.gate = (const float*)ten(in, T, 7);
            g.N = H; g.K = I; g.E = E; g.enc = enc;
            g.wcols = 3; g.wsel0 = 2; g.wsel1 = 2;
            g.slots_hint = slots_of(in, h, 0u);
            if (!g.slots_hint && h.form != 0) g.form_ws = next_form_word(c); /* unknown rows: the form is chosen on the device */
            return launch_group_down_a16(g, st);
        }
        if (enc == PLOW_MOE_ENC_MXFP4 && (arm == PLOW_MOE_ARM_A4W4 || arm == PLOW_MOE_ARM_A4W4_P16)) {
            /* fp4 on both operands: t1 the mxfp4 rows and t5 the E8M0 rows that op 85 wrote */
            NEED(c, ten(in, T, 3) && ten(in, T, 5), "op 86 A4W4: t3 stab and t5 E8M0 rows must be bound");
            NEED(c, I % 256u == 0u && H % 256u == 0u && I >= 512u && H >= 512u, "op 86 A4W4: I %u and H %u must be multiples of 256, at least 512", I, H);
            NEED(c, (uint64_t)slots_of(in, h, 0u) / 128u + E <= 65535u, "op 86 A4W4: %u routed rows over %u experts exceed the 65535 row tiles the tiled kernel's directory counts", slots_of(in, h, 0u), E);
            if (!launch) return 0;
            GroupW8A8 g = {};
            g.out = ten(in, T, 0);
            g.a = ten(in, T, 1); g.a_e8m0 = (const uint8_t*)ten(in, T, 5);
            g.wtab = (const uint64_t*)ten(in, T, 2); g.stab = (const uint64_t*)ten(in, T, 3);
            g.meta = (const int32_t*)ten(in, T, 4);
            g.row_partidx = (const uint32_t*)ten(in, T, 6); g.row_gate = (const float*)ten(in, T, 7);
            g.N = H; g.K = I; g.E = E; g.part16 = arm == PLOW_MOE_ARM_A4W4_P16;
            g.slots_bound = slots_of(in, h, 0u);
            g.w_nt = tiled_w_nt(g.slots_bound, g.E, false);
            return launch_group_a4w4_tiled(g, false, st);
        }
        return fail(c, PLOW_MOE_EUNSUPPORTED, "op 86: encoding %u arm %u is not served", enc, arm);
    }
    case PLOW_DOP_MOE_GROUP_GLU_GEMMA_PF_W8A8: {
        const uint32_t I = i[0], H = i[1], E = i[2];
        NEED(c, ten(in, T, 0) && ten(in, T, 1) && ten(in, T, 2) && ten(in, T, 3) && ten(in, T, 4) && ten(in, T, 5) && ten(in, T, 6),
             "op 81: t0 fu, t1 xq8, t2 ewt, t3 meta, t4 row_token, t5 ascale, t6 est must be bound");
        NEED(c, I && H && E && I % 128u == 0u && H % 128u == 0u, "op 81: I %u and H %u must be non-zero multiples of 128", I, H);
        NEED(c, i[5] <= 1u, "op 81: activation %u is not served", i[5]);
        if (!launch) return 0;
        GroupW8A8 g = {};
        g.out = ten(in, T, 0); g.a = ten(in, T, 1); g.a_scale = (const float*)ten(in, T, 5);
        g.wtab = (const uint64_t*)ten(in, T, 2); g.stab = (const uint64_t*)ten(in, T, 6);
        g.meta = (const int32_t*)ten(in, T, 3); g.row_token = (const uint32_t*)ten(in, T, 4);
        g.N = I; g.K = H; g.E = E; g.act = i[5]; g.per_channel = 1;
        return launch_w8a8(c, h, slots_of(in, h, 0u), g, true, st);
    }
    case PLOW_DOP_MOE_GROUP_DOWN_GEMMA_PF_W8A8: {
        const uint32_t H = i[0], I = i[1], E = i[2];
        NEED(c, ten(in, T, 0) && ten(in, T, 1) && ten(in, T, 2) && ten(in, T, 3) && ten(in, T, 4) && ten(in, T, 5) && ten(in, T, 6) && ten(in, T, 7),
             "op 82: t0 part, t1 fu8, t2 ewt, t3 meta, t4 row_partidx, t5 row_gate, t6 est, t7 fscale must be bound");
        NEED(c, I && H && E && I % 128u == 0u && H % 128u == 0u, "op 82: I %u and H %u must be non-zero multiples of 128", I, H);
        if (!launch) return 0;
        GroupW8A8 g = {};
        g.out = ten(in, T, 0); g.a = ten(in, T, 1); g.a_scale = (const float*)ten(in, T, 7);
        g.wtab = (const uint64_t*)ten(in, T, 2); g.stab = (const uint64_t*)ten(in, T, 6);
        g.meta = (const int32_t*)ten(in, T, 3);
        g.row_partidx = (const uint32_t*)ten(in, T, 4); g.row_gate = (const float*)ten(in, T, 5);
        g.N = H; g.K = I; g.E = E; g.per_channel = 1;
        return launch_w8a8(c, h, slots_of(in, h, 0u), g, false, st);
    }
    case PLOW_DOP_MOE_GROUP_GLU_FP8_BLK:
    case PLOW_DOP_MOE_EXPERT_GLU_GEMMA_FP8:
    case PLOW_DOP_MOE_GROUP_DOWN_FP8_BLK:
    case PLOW_DOP_MOE_EXPERT_DOWN_GEMMA_FP8: {
        /* slot-major decode experts: sort the slots by expert into the context workspace, then run
         * the grouped kernel with slot-major input / output rows */
        const bool pc = in->op == PLOW_DOP_MOE_EXPERT_GLU_GEMMA_FP8 || in->op == PLOW_DOP_MOE_EXPERT_DOWN_GEMMA_FP8;
        const bool glu = in->op == PLOW_DOP_MOE_GROUP_GLU_FP8_BLK || in->op == PLOW_DOP_MOE_EXPERT_GLU_GEMMA_FP8;
        uint32_t nslot, kx, N, K, E, enc, act;
        if (pc) { /* i0=k i1=N i2=K i3=E i5=B(0 = 1); act: i6 on the GLU (0 gelu_tanh, 1 silu) */
            nslot = i[0] * (i[5] ? i[5] : 1u); kx = i[0]; N = i[1]; K = i[2]; E = i[3];
            enc = 3u; act = glu ? i[6] : 0u;
        } else {  /* i0=slots i1=N i2=K i3=E i4=slots per x row (GLU; 0 = one shared row) i5=act i6=enc */
            nslot = i[0]; kx = glu ? (i[4] ? i[4] : i[0]) : 1u; N = i[1]; K = i[2]; E = i[3];
            enc = i[6]; act = glu ? i[5] : 0u;
        }
        NEED(c, ten(in, T, 0) && ten(in, T, 1) && ten(in, T, 2) && ten(in, T, 3), "op %u: t0 out, t1 in, t2 table, t3 weight table must be bound", (unsigned)in->op);
        NEED(c, pc || enc <= 2u, "op %u: encoding %u is not one of bf16 / block-fp8 / mxfp4", (unsigned)in->op, enc);
        NEED(c, !pc || i[4] == 0u, "op %u: a non-zero slot offset (i4) is not served", (unsigned)in->op);
        NEED(c, (enc == PLOW_MOE_ENC_BF16 || ten(in, T, 4)), "op %u: scale table t4 must be bound for encoding %u", (unsigned)in->op, enc);
        NEED(c, nslot && kx && N && K && E && N % 128u == 0u && K % 128u == 0u, "op %u: N %u and K %u must be non-zero multiples of 128", (unsigned)in->op, N, K);
        NEED(c, E <= c->ws.max_e && nslot <= c->ws.max_slots, "op %u: %u slots / %u experts exceed the workspace (%u slots, %u experts)", (unsigned)in->op, nslot, E, c->ws.max_slots, c->ws.max_e);
        NEED(c, act <= 1u, "op %u: activation %u is not served", (unsigned)in->op, act);
        if (!launch) return 0;
        if (plow_moe_tuning().gemv_direct) {
            /* a handful of slots on the matrix-vector form: the table itself lists the rows, nothing is sorted */
            GroupA16 d = {};
            d.out = ten(in, T, 0); d.a = ten(in, T, 1);
            d.wtab = (const uint64_t*)ten(in, T, 3);
            d.stab = enc == PLOW_MOE_ENC_BF16 ? nullptr : (const uint64_t*)ten(in, T, 4);
            d.N = N; d.K = K; d.E = E; d.enc = enc; d.act = act;
            d.wcols = pc ? 2u : 3u;
            d.slots_hint = nslot;
            d.tab_direct = ten(in, T, 2), d.tab_nslot = nslot, d.tab_kx = glu ? kx : 1u;
            if (glu) d.wsel0 = 0, d.wsel1 = pc ? 0u : 1u, d.wrow1 = pc ? N : 0u;
            else d.wsel0 = d.wsel1 = pc ? 1u : 2u, d.zs_table = ten(in, T, 2), d.zs_nslot = nslot;
            if (group_a16_gemv_serves(d)) return launch_group_a16_gemv(d, glu, st);
        }
        /* align with k = slots per input row: row_token = slot / kx, row_partidx = slot */
        int rc = 0;
        if (!sort_reusable(h, ten(in, T, 2), nslot, E, kx, glu)) {
            rc = launch_align(c->ws.meta, ten(in, T, 2), c->ws.row_token, c->ws.row_partidx, c->ws.row_gate,
                              (nslot + kx - 1u) / kx, E, kx, c->ws.chunk_hist, c->ws.max_chunks, st);
            if (rc) return rc;
            h.sorted_table = ten(in, T, 2), h.sorted_nslot = nslot, h.sorted_E = E, h.sorted_kx = kx;
        }
        GroupA16 g = {};
        g.out = ten(in, T, 0); g.a = ten(in, T, 1);
        g.wtab = (const uint64_t*)ten(in, T, 3);
        g.stab = enc == PLOW_MOE_ENC_BF16 ? nullptr : (const uint64_t*)ten(in, T, 4);
        g.meta = c->ws.meta;
        g.N = N; g.K = K; g.E = E; g.enc = enc; g.act = act;
        g.wcols = pc ? 2u : 3u;
        g.slots_hint = nslot;
        g.o_idx = c->ws.row_partidx;
        if (glu) {
            g.a_idx = c->ws.row_token;
            g.wsel0 = 0; g.wsel1 = pc ? 0u : 1u; g.wrow1 = pc ? N : 0u;
            return launch_group_glu_a16(g, st);
        }
        g.a_idx = c->ws.row_partidx; g.gate = c->ws.row_gate;
        g.wsel0 = g.wsel1 = pc ? 1u : 2u;
        /* the rows of slots no expert serves are zeroed by the launch itself (the matrix-vector and streaming forms) or
         * by one of its own ahead of it (the others) */
        g.zs_table = ten(in, T, 2), g.zs_nslot = nslot;
        return launch_group_down_a16(g, st);
    }
    case PLOW_DOP_MOE_GROUP_GLU_GEMMA_PF:
    case PLOW_DOP_MOE_GROUP_DOWN_GEMMA_PF: {
        /* bf16 grouped experts over the fused table ewt[E][2] = {gate_up [2I][H], down [H][I]}
         * (plow runtime/common/dev_isa.h:616-628): 75 t0=fu_g t1=xn2 t2=ewt t3=meta t4=row_token i0=I i1=H
         * i2=E i5=act; 76 t0=part t1=fu_g t2=ewt t3=meta t4=row_partidx t5=row_gate i0=H i1=I i2=E */
        const bool glu = in->op == PLOW_DOP_MOE_GROUP_GLU_GEMMA_PF;
        const uint32_t N = i[0], K = i[1], E = i[2];
        NEED(c, ten(in, T, 0) && ten(in, T, 1) && ten(in, T, 2) && ten(in, T, 3) && ten(in, T, 4) && (glu || ten(in, T, 5)),
             "op %u: output, input, ewt, meta and the row maps must be bound", (unsigned)in->op);
        NEED(c, N && K && E && N % 128u == 0u && K % 128u == 0u, "op %u: N %u and K %u must be non-zero multiples of 128", (unsigned)in->op, N, K);
        NEED(c, !glu || i[5] <= 1u, "op 75: activation %u is not served", i[5]);
        if (!launch) return 0;
        GroupA16 g = {};
        g.out = ten(in, T, 0); g.a = ten(in, T, 1);
        g.wtab = (const uint64_t*)ten(in, T, 2); g.wcols = 2;
        g.meta = (const int32_t*)ten(in, T, 3);
        g.N = N; g.K = K; g.E = E; g.enc = PLOW_MOE_ENC_BF16; g.act = glu ? i[5] : 0u;
        g.slots_hint = slots_of(in, h, 0u);
        if (!g.slots_hint && h.form != 0) g.form_ws = next_form_word(c); /* unknown rows: the form is chosen on the device */
        if (glu) {
            g.a_idx = (const uint32_t*)ten(in, T, 4);
            g.wsel0 = g.wsel1 = 0; g.wrow1 = N;
            return launch_group_glu_a16(g, st);
        }
        g.o_idx = (const uint32_t*)ten(in, T, 4); g.gate = (const float*)ten(in, T, 5);
        g.wsel0 = g.wsel1 = 1;
        return launch_group_down_a16(g, st);
    }
    case PLOW_DOP_MOE_GLU_MX:
    case PLOW_DOP_MOE_DOWN_MX:
    case PLOW_DOP_MOE_GLU_MX_PF:
    case PLOW_DOP_MOE_DOWN_MX_PF: {
        /* flat mxfp4 tensors (plow runtime/common/dev_isa.h:1285-1335): expert e of [E][rows][K/2] starts
         * at W + e*rows*(K/2), its E8M0 bytes at S + e*rows*(K/32), its bias at b + e*rows. The per-expert
         * pointer tables the kernels read are built in the context workspace by a small launch. */
        const bool glu = in->op == PLOW_DOP_MOE_GLU_MX || in->op == PLOW_DOP_MOE_GLU_MX_PF;
        const bool pf = in->op == PLOW_DOP_MOE_GLU_MX_PF || in->op == PLOW_DOP_MOE_DOWN_MX_PF;
        /* decode: t0 out t1 in t2 table t3 W t4 S t5 bias? i0=k i1=N i2=K i3=E i4=layout i5=act i6=B(0 = 1)
         * prefill GLU:  t0 fu_g t1 xn2 t2 W t3 S t4 meta t5 row_token t6 bias?  i0=I i1=K i2=E i3=layout i5=act
         * prefill DOWN: t0 part t1 fu_g t2 W t3 S t4 meta t5 bias? t6 row_partidx t7 row_gate  i0=H i1=I i2=E */
        const uint32_t N = pf ? i[0] : i[1], K = pf ? i[1] : i[2], E = pf ? i[2] : i[3];
        const uint32_t layout = glu ? (pf ? i[3] : i[4]) : 1u, act = glu ? i[5] : 0u;
        const uint32_t kx = pf ? 0u : i[0], nslot = pf ? 0u : i[0] * (i[6] ? i[6] : 1u);
        void* W = ten(in, T, pf ? 2 : 3);
        void* S = ten(in, T, pf ? 3 : 4);
        void* bias = ten(in, T, pf ? (glu ? 6 : 5) : 5);
        NEED(c, ten(in, T, 0) && ten(in, T, 1) && W && S, "op %u: output, input, weight and scale tensors must be bound", (unsigned)in->op);
        NEED(c, pf ? ten(in, T, 4) != nullptr : ten(in, T, 2) != nullptr, "op %u: %s must be bound", (unsigned)in->op, pf ? "t4 meta" : "t2 table");
        NEED(c, !pf || (glu ? ten(in, T, 5) != nullptr : (ten(in, T, 6) && ten(in, T, 7))), "op %u: the row maps must be bound", (unsigned)in->op);
        NEED(c, N && K && E && N % 128u == 0u && K % 128u == 0u, "op %u: N %u and K %u must be non-zero multiples of 128", (unsigned)in->op, N, K);
        NEED(c, E <= c->ws.max_e && nslot <= c->ws.max_slots && (pf || nslot), "op %u: %u slots / %u experts exceed the workspace (%u slots, %u experts)", (unsigned)in->op, nslot, E, c->ws.max_slots, c->ws.max_e);
        NEED(c, layout <= 1u, "op %u: layout %u is neither interleaved (0) nor blocked (1)", (unsigned)in->op, layout);
        if (act > PLOW_MOE_ACT_SWIGLU_OAI) return fail(c, PLOW_MOE_EUNSUPPORTED, "op %u: activation %u is not served", (unsigned)in->op, act);
        if (!launch) return 0;
        const uint32_t rows = glu ? 2u * N : N; /* weight rows per expert */
        uint64_t* wtab = c->ws.ftab;
        uint64_t* stab = c->ws.ftab + (size_t)c->ws.max_e * 3u;
        int rc = launch_flat_tables(wtab, stab, W, S, E, (size_t)rows * (K / 2u), (size_t)rows * (K / 32u), st);
        if (rc) return rc;
        GroupA16 g = {};
        g.out = ten(in, T, 0); g.a = ten(in, T, 1);
        g.wtab = wtab; g.stab = stab; g.wcols = 3; g.wsel0 = g.wsel1 = 0;
        g.N = N; g.K = K; g.E = E; g.enc = PLOW_MOE_ENC_MXFP4; g.act = act;
        g.f0 = in->fj[0].f; g.f1 = in->fj[1].f; /* the activation's immediates (act 2: betas, act 3: alpha, limit) */
        g.bias = bias; g.bias_rows = rows;
        if (glu) { g.wmul = layout ? 1u : 2u; g.wrow0 = 0; g.wrow1 = layout ? N : 1u; }
        if (pf) {
            g.meta = (const int32_t*)ten(in, T, 4);
            g.slots_hint = slots_of(in, h, 0u);
            if (glu) { g.a_idx = (const uint32_t*)ten(in, T, 5); return launch_group_glu_a16(g, st); }
            g.o_idx = (const uint32_t*)ten(in, T, 6); g.gate = (const float*)ten(in, T, 7);
            return launch_group_down_a16(g, st);
        }
        if (plow_moe_tuning().gemv_direct) { /* a handful of slots: the table itself lists the rows, nothing is sorted */
            GroupA16 d = g;
            d.slots_hint = nslot;
            d.tab_direct = ten(in, T, 2), d.tab_nslot = nslot, d.tab_kx = glu ? kx : 1u;
            if (!glu) d.zs_table = ten(in, T, 2), d.zs_nslot = nslot;
            if (group_a16_gemv_serves(d)) return launch_group_a16_gemv(d, glu, st);
        }
        /* slot-major: sort the slots by expert into the context workspace (row_token = slot / k) */
        if (!sort_reusable(h, ten(in, T, 2), nslot, E, kx, glu)) {
            rc = launch_align(c->ws.meta, ten(in, T, 2), c->ws.row_token, c->ws.row_partidx, c->ws.row_gate,
                              nslot / kx, E, kx, c->ws.chunk_hist, c->ws.max_chunks, st);
            if (rc) return rc;
            h.sorted_table = ten(in, T, 2), h.sorted_nslot = nslot, h.sorted_E = E, h.sorted_kx = kx;
        }
        g.meta = c->ws.meta; g.slots_hint = nslot; g.o_idx = c->ws.row_partidx;
        if (glu) { g.a_idx = c->ws.row_token; return launch_group_glu_a16(g, st); }
        g.a_idx = c->ws.row_partidx; g.gate = c->ws.row_gate;
        g.zs_table = ten(in, T, 2), g.zs_nslot = nslot;
        return launch_group_down_a16(g, st);
    }
    case PLOW_DOP_GEMM_GLU:
    case PLOW_DOP_GEMM: {
        /* dense bf16 shared expert: one "expert" whose rows are the tokens themselves */
        const bool glu = in->op == PLOW_DOP_GEMM_GLU;
        const uint32_t M = i[0], N = i[1], K = i[2];
        NEED(c, ten(in, T, 0) && ten(in, T, 1) && ten(in, T, 2) && (!glu || ten(in, T, 5)), "op %u: output, input and weight tensors must be bound", (unsigned)in->op);
        NEED(c, !ten(in, T, 6) && !ten(in, T, 7), "op %u: the bias operands are not on this path", (unsigned)in->op);
        NEED(c, glu || (!ten(in, T, 3) && !ten(in, T, 4)), "op 8: the folded-norm operands are not on this path");
        NEED(c, M && N && K && N % 128u == 0u && K % 128u == 0u, "op %u: N %u and K %u must be non-zero multiples of 128", (unsigned)in->op, N, K);
        NEED(c, !glu || i[5] <= 1u, "op 20: activation %u is not served", i[5]);
        if (!launch) return 0;
        GroupA16 g = {};
        g.out = (char*)ten(in, T, 0) + (glu ? 0u : (size_t)i[5] * N * 2u);
        g.a = (const char*)ten(in, T, 1) + (glu ? 0u : (size_t)i[4] * K * 2u);
        g.wdirect[0] = ten(in, T, 2); g.wdirect[1] = glu ? ten(in, T, 5) : ten(in, T, 2);
        g.N = N; g.K = K; g.E = 1; g.enc = 0; g.act = glu ? i[5] : 0u;
        g.wcols = 1; g.out_bf16 = 1; g.dense_rows = M;
        if (c->ws_base && c->stage) g.split_ws = c->stage, g.split_ws_bytes = c->stage_bytes; /* few rows: K split over workgroups */
        return glu ? launch_group_glu_a16(g, st) : launch_group_down_a16(g, st);
    }
    default:
        return fail(c, PLOW_MOE_EUNSUPPORTED, "opcode %u is not served by this library", (unsigned)in->op);
    }
}

static int finish(PlowMoeCtx* c, int rc, const PlowDevInst* in) {
    if (rc) {
        if (rc != PLOW_MOE_EINVAL && rc != PLOW_MOE_EUNSUPPORTED) fail(c, rc, "op %u: launcher refused (%d)", (unsigned)in->op, rc);
        else if (!c->err[0]) fail(c, rc, "op %u: refused (%d)", (unsigned)in->op, rc);
        return rc;
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(c, PLOW_MOE_EDEVICE, "op %u: %s", (unsigned)in->op, hipGetErrorString(e));
    return 0;
}

/* the align op of a run states its routed slots (T * k) for the ops that follow it in the same run */
static Hint hint_of_run(const PlowDevInst* insts, uint32_t n_inst, int form) {
    Hint h = {form, 0u, nullptr, 0u, 0u, 0u};
    for (uint32_t n = 0; n < n_inst; n++)
        if (insts[n].op == PLOW_DOP_MOE_ALIGN_PF) {
            const uint64_t slots = (uint64_t)insts[n].i[0] * insts[n].i[2];
            h.slots = slots < 0xFFFFFFFFull ? (uint32_t)slots : 0xFFFFFFFFu;
        }
    return h;
}

/* Operand slots an op writes (bit j: t[j]); every slot for an op this table does not know */
static uint32_t out_slots(const PlowDevInst* in) {
    switch (in->op) {
    case PLOW_DOP_GEMM_F32: return in->i[7] == PLOW_ROUTER_RAW_MARK ? (1u | 8u | 32u) : 1u;
    case PLOW_DOP_MOE_ROUTER_TOPK:
    case PLOW_DOP_MOE_ROUTER_TOPK_PF: return 1u | 4u;
    case PLOW_DOP_MOE_ALIGN_PF: return 1u | 4u | 8u | 16u;
    case PLOW_DOP_MOE_GROUP_GLU_PF: return 1u | 128u;
    case PLOW_DOP_MOE_GROUP_DOWN_PF:
    case PLOW_DOP_MOE_COMBINE_PF:
    case PLOW_DOP_GEMM_GLU:
    case PLOW_DOP_GEMM: return 1u;
    default: return 0xFFu;
    }
}
/* the op keeps something in the context's staging while it runs */
static bool uses_staging(const PlowDevInst* in) {
    if (in->op == PLOW_DOP_GEMM_GLU || in->op == PLOW_DOP_GEMM) return true;
    if (in->op == PLOW_DOP_MOE_GROUP_GLU_PF)
        return (in->i[3] == PLOW_MOE_ENC_FP8BLK && (in->i[7] == PLOW_MOE_ARM_W8A8_XQ || in->i[7] == PLOW_MOE_ARM_W8A8_SPLIT)) ||
               (in->i[3] == PLOW_MOE_ENC_MXFP4 && in->i[7] == PLOW_MOE_ARM_A4W4);
    if (in->op == PLOW_DOP_MOE_GROUP_DOWN_PF)
        return in->i[3] == PLOW_MOE_ENC_FP8BLK && (in->i[7] == PLOW_MOE_ARM_W8A8_SPLIT || in->i[7] == PLOW_MOE_ARM_W8A8_SPLIT_P16);
    return false;
}
/* `x` (an op of the run) may run beside dense op `d`: x neither touches what d writes nor writes what d reads */
static bool beside(const PlowDevInst* x, const PlowDevInst* d) {
    if (uses_staging(x)) return false;
    const uint32_t xo = out_slots(x);
    for (int j = 0; j < 8; j++) {
        if (x->t[j] == PLOW_TENSOR_NONE) continue;
        if (x->t[j] == d->t[0]) return false;
        if ((xo >> j) & 1u)
            for (int q = 1; q < 8; q++)
                if (d->t[q] != PLOW_TENSOR_NONE && x->t[j] == d->t[q]) return false;
    }
    return true;
}

/* A run's dense shared-expert ops (20 / 8: a few dozen workgroups each at a few tokens) go to the context's second
 * stream, forked off the caller's stream ahead of the ops before them that touch none of their operands (the routed
 * experts, whose final pass of workgroups leaves CUs idle) and joined again before the op that follows them: the run's result is
 * that of its ops in order. [a, b): the block of dense ops; h: the first op that runs beside it. */
static bool dense_overlap_plan(const PlowMoeCtx* ctx, const PlowDevInst* insts, uint32_t n_inst, uint32_t* a, uint32_t* b, uint32_t* h) {
    if (!ctx->side || !plow_moe_tuning().dense_overlap) return false;
    uint32_t lo = n_inst;
    for (uint32_t n = 0; n < n_inst; n++)
        if (insts[n].op == PLOW_DOP_GEMM_GLU || insts[n].op == PLOW_DOP_GEMM) { lo = n; break; }
    if (lo == n_inst || lo == 0u) return false;
    uint32_t hi = lo;
    while (hi < n_inst && (insts[hi].op == PLOW_DOP_GEMM_GLU || insts[hi].op == PLOW_DOP_GEMM)) hi++;
    for (uint32_t n = hi; n < n_inst; n++) /* one block only */
        if (insts[n].op == PLOW_DOP_GEMM_GLU || insts[n].op == PLOW_DOP_GEMM) return false;
    for (uint32_t n = lo; n < hi; n++) /* a few rows each: larger ones fill the chip by themselves */
        if (insts[n].i[0] >= 128u) return false;
    uint32_t first = lo;
    while (first > 0u) {
        bool ok = true;
        for (uint32_t d = lo; d < hi && ok; d++) ok = beside(&insts[first - 1u], &insts[d]);
        if (!ok) break;
        first--;
    }
    if (first == lo) return false;
    *a = lo, *b = hi, *h = first;
    return true;
}

static int exec_run(PlowMoeCtx* ctx, const PlowDevInst* insts, uint32_t n_inst, void* const* tensors, void* stream,
                    int form) {
    Hint h = hint_of_run(insts, n_inst, form);
    for (uint32_t n = 0; n < n_inst; n++) { /* refuse the whole run before launching any of it */
        const int rc = run_op(ctx, &insts[n], tensors, nullptr, false, h);
        if (rc) return rc;
    }
    const hipStream_t st = (hipStream_t)stream;
    uint32_t da = 0, db = 0, dh = 0;
    if (!dense_overlap_plan(ctx, insts, n_inst, &da, &db, &dh)) {
        for (uint32_t n = 0; n < n_inst; n++) {
            const int rc = finish(ctx, run_op(ctx, &insts[n], tensors, st, true, h), &insts[n]);
            if (rc) return rc;
        }
        return 0;
    }
    int rc = 0;
    for (uint32_t n = 0; n < dh && !rc; n++) rc = finish(ctx, run_op(ctx, &insts[n], tensors, st, true, h), &insts[n]);
    if (rc) return rc;
    if (hipEventRecord(ctx->ev_fork, st) != hipSuccess || hipStreamWaitEvent(ctx->side, ctx->ev_fork, 0) != hipSuccess)
        return fail(ctx, PLOW_MOE_EDEVICE, "the run's second stream could not be forked");
    for (uint32_t n = da; n < db && !rc; n++) rc = finish(ctx, run_op(ctx, &insts[n], tensors, ctx->side, true, h), &insts[n]);
    for (uint32_t n = dh; n < da && !rc; n++) rc = finish(ctx, run_op(ctx, &insts[n], tensors, st, true, h), &insts[n]);
    /* joined whatever happened in between: a capture of the caller's stream must not end with the fork open */
    if (hipEventRecord(ctx->ev_join, ctx->side) != hipSuccess || hipStreamWaitEvent(st, ctx->ev_join, 0) != hipSuccess)
        return fail(ctx, PLOW_MOE_EDEVICE, "the run's second stream could not be joined");
    if (rc) return rc;
    for (uint32_t n = db; n < n_inst && !rc; n++) rc = finish(ctx, run_op(ctx, &insts[n], tensors, st, true, h), &insts[n]);
    return rc;
}

extern "C" int plow_moe_check(PlowMoeCtx* ctx, const PlowDevInst* inst, void* const* tensors) {
    if (!ctx || !inst || !tensors) return PLOW_MOE_EINVAL;
    ctx->err[0] = 0;
    Hint h = {-1, 0u, nullptr, 0u, 0u, 0u};
    return run_op(ctx, inst, tensors, nullptr, false, h);
}

extern "C" int plow_moe_exec(PlowMoeCtx* ctx, const PlowDevInst* inst, void* const* tensors, void* stream) {
    if (!ctx || !inst || !tensors) return PLOW_MOE_EINVAL;
    ctx->err[0] = 0;
    Hint h = {-1, 0u, nullptr, 0u, 0u, 0u};
    return finish(ctx, run_op(ctx, inst, tensors, (hipStream_t)stream, true, h), inst);
}

extern "C" int plow_moe_exec_many(PlowMoeCtx* ctx, const PlowDevInst* insts, uint32_t n_inst,
                                  void* const* tensors, void* stream) {
    if (!ctx || !insts || !tensors) return PLOW_MOE_EINVAL;
    ctx->err[0] = 0;
    return exec_run(ctx, insts, n_inst, tensors, stream, -1);
}

/* One op with no allocation anywhere on its path: no context (creating one allocates its workspace), the
 * slot-major and flat-tensor ops take their workspace from the library's static device array instead.
 * The first call on a device sets that device up (kernel attributes, the array's address there); inst ==
 * NULL does only that. */
extern "C" int plow_moe_exec_noalloc(const PlowDevInst* inst, void* const* tensors, void* stream, char* err,
                                     size_t err_len) {
    if (err && err_len) err[0] = 0;
    auto say = [&](const char* text) {
        if (err && err_len) snprintf(err, err_len, "%s", text);
    };
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return PLOW_MOE_EDEVICE;
    void* base = plow_moe_static_scratch();
    if (!base) {
        const int rc = plow_moe_device_setup(dev);
        if (rc) {
            say(rc == PLOW_MOE_EUNSUPPORTED ? "the current device is not gfx950" : "device set-up failed");
            return rc;
        }
        base = plow_moe_static_scratch();
        if (!base) return PLOW_MOE_EDEVICE;
    }
    if (!inst) return 0;
    if (!tensors) return PLOW_MOE_EINVAL;
    PlowMoeCtx c = {};
    c.device = dev;
    c.min_rows[0] = c.min_rows[1] = -1;
    c.ws = ws_carve(base, PLOW_MOE_NOALLOC_MAX_EXPERTS, PLOW_MOE_NOALLOC_MAX_SLOTS); /* borrowed: ws_base stays NULL */
    Hint h = {-1, 0u, nullptr, 0u, 0u, 0u};
    const int rc = finish(&c, run_op(&c, inst, tensors, (hipStream_t)stream, true, h), inst);
    if (rc) say(c.err);
    return rc;
}

/* ---- segment entry points ---------------------------------------------------------------------- */

static bool is_glu(uint16_t op) {
    return op == PLOW_DOP_MOE_GROUP_GLU_PF || op == PLOW_DOP_MOE_GROUP_GLU_GEMMA_PF_W8A8 ||
           op == PLOW_DOP_MOE_GROUP_GLU_FP8_BLK || op == PLOW_DOP_MOE_EXPERT_GLU_GEMMA_FP8;
}
static bool is_down(uint16_t op) {
    return op == PLOW_DOP_MOE_GROUP_DOWN_PF || op == PLOW_DOP_MOE_GROUP_DOWN_GEMMA_PF_W8A8 ||
           op == PLOW_DOP_MOE_GROUP_DOWN_FP8_BLK || op == PLOW_DOP_MOE_EXPERT_DOWN_GEMMA_FP8;
}

/* A segment is a run holding exactly one GLU and one DOWN of the same family, GLU first, whose
 * intermediate, expert table and geometry agree; everything else in the run must be an op of this
 * library. */
static int check_segment(PlowMoeCtx* c, const PlowDevInst* insts, uint32_t n) {
    int glu = -1, down = -1;
    for (uint32_t j = 0; j < n; j++) {
        if (is_glu(insts[j].op)) { NEED(c, glu < 0, "segment: more than one GLU op"); glu = (int)j; }
        if (is_down(insts[j].op)) { NEED(c, down < 0, "segment: more than one DOWN op"); down = (int)j; }
    }
    NEED(c, glu >= 0 && down >= 0 && glu < down, "segment: needs one GLU followed by one DOWN");
    const PlowDevInst &g = insts[glu], &d = insts[down];
    NEED(c, d.op == g.op + 1u, "segment: GLU op %u and DOWN op %u are not a pair", (unsigned)g.op, (unsigned)d.op);
    if (g.op == PLOW_DOP_MOE_GROUP_GLU_PF) {
        NEED(c, g.i[0] == d.i[1] && g.i[1] == d.i[0] && g.i[2] == d.i[2], "segment: GLU (I,H,E) and DOWN (H,I,E) disagree");
        NEED(c, g.i[3] == d.i[3], "segment: GLU and DOWN weight encodings differ");
        NEED(c, g.t[2] == d.t[2] && g.t[3] == d.t[3] && g.t[4] == d.t[4], "segment: wtab / stab / meta handles differ");
        const bool quantized_mid = g.i[7] == PLOW_MOE_ARM_W8A8;
        NEED(c, g.t[0] == d.t[1], "segment: DOWN does not read the GLU's output");
        const bool a4w4 = g.i[3] == PLOW_MOE_ENC_MXFP4 && g.i[7] == PLOW_MOE_ARM_A4W4;
        if (quantized_mid || a4w4) NEED(c, g.t[7] == d.t[5], "segment: DOWN does not read the GLU's output scales");
        if (a4w4) NEED(c, d.i[7] == PLOW_MOE_ARM_A4W4 || d.i[7] == PLOW_MOE_ARM_A4W4_P16, "segment: GLU arm %u and DOWN arm %u disagree", g.i[7], d.i[7]);
        NEED(c, (g.i[7] == PLOW_MOE_ARM_W8A8) == (d.i[7] == PLOW_MOE_ARM_W8A8 || d.i[7] == PLOW_MOE_ARM_W8A8_P16),
             "segment: GLU arm %u and DOWN arm %u disagree", g.i[7], d.i[7]);
    } else if (g.op == PLOW_DOP_MOE_GROUP_GLU_GEMMA_PF_W8A8) {
        NEED(c, g.i[0] == d.i[1] && g.i[1] == d.i[0] && g.i[2] == d.i[2], "segment: GLU (I,H,E) and DOWN (H,I,E) disagree");
        NEED(c, g.t[2] == d.t[2] && g.t[3] == d.t[3] && g.t[6] == d.t[6], "segment: ewt / meta / est handles differ");
    } else {
        NEED(c, g.i[1] == d.i[2] && g.i[2] == d.i[1] && g.i[3] == d.i[3], "segment: GLU (I,H,E) and DOWN (H,I,E) disagree");
        NEED(c, g.t[0] == d.t[1] && g.t[2] == d.t[2] && g.t[3] == d.t[3], "segment: fu / table / weight-table handles differ");
    }
    return 0;
}

static int run_segment(PlowMoeCtx* ctx, int variant, const PlowDevInst* insts, uint32_t n_inst,
                       void* const* tensors, uint32_t rows, void* stream) {
    if (!ctx || !insts || !tensors || n_inst == 0) return PLOW_MOE_EINVAL;
    ctx->err[0] = 0;
    const int mr = ctx->min_rows[variant];
    if (mr == 0 || (mr > 0 && rows < (uint32_t)mr)) return PLOW_MOE_ROLLBACK;
    int rc = check_segment(ctx, insts, n_inst);
    if (rc) return rc;
    /* prefill: tiled kernels (the streaming ones where a shape is outside the tiled form's limits);
     * decode: weight-streaming kernels */
    return exec_run(ctx, insts, n_inst, tensors, stream, variant == 0 ? 1 : 0);
}

extern "C" int plow_moe_pf(PlowMoeCtx* ctx, const PlowDevInst* insts, uint32_t n_inst,
                           void* const* tensors, uint32_t rows, void* stream) {
    return run_segment(ctx, 0, insts, n_inst, tensors, rows, stream);
}

extern "C" int plow_moe_dec(PlowMoeCtx* ctx, const PlowDevInst* insts, uint32_t n_inst,
                            void* const* tensors, uint32_t rows, void* stream) {
    return run_segment(ctx, 1, insts, n_inst, tensors, rows, stream);
}
