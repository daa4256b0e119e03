/* plowrt_dec_obj.hip — the device code object an unmodified plowrt loads for its decode-rung W8A8
 * grouped-MoE pair on gfx950: `moe_w8a8_dec_gfx950.elf`.
 *
 * What plowrt expects of that object (plow crates/plowrt/src/exec/amd.rs):
 *   :10799-10852  the file name, the marker `plow_moe_w8a8_dec_abi_1` in the ELF symbol table, the three
 *                 kernels below with argument segments of 96, 80 and 192 bytes and no private memory;
 *   :3416-3430    MoeW8a8DecPairArgs = the GLU block, the DOWN block, a zeroed u32 counter scratch of
 *                 2 * 2 * tiles words that the kernel must leave zeroed, and the GLU share of the grid;
 *   :3443-3560    what reaches it: op 85 with i7 = 6 (bf16 rows, quantized 1x128 where they are loaded;
 *                 x_scale = 0, x_pitch = 0) and op 86 with i7 = 2 on the same tables, I % 256 == 0,
 *                 H % 1024 == 0; grids 2 * tiles * (I / 128) and 2 * tiles * ceil(H / 256);
 *   :17748-17790  the launch: 256 threads, no dynamic LDS; GLU then DOWN back to back, or both grids
 *                 in one launch of the pair kernel.
 * The kernels are the library's weight-streaming kernel (experts_w8a8.hip) in its four-wave form: a work
 * item is (expert, 128 gate|up channels) or (expert, 256 down channels), every wave streams the weights
 * of two 16- or 32-channel shares one after the other, and the items are walked with the launch's
 * stride, so any grid serves. Same arithmetic as the library's ops 85 (arm 6, or arm 2 when x_scale is
 * bound) and 86 (arm 2). Shapes the kernel cannot serve make it return without writing, as plow's own do
 * (runtime/amd/moe_w8a8_dec.hip:486-487). */
#include "experts_w8a8.hip"
#define DP_FN __device__ __forceinline__
#include "dec_pair_protocol.h"

extern "C" __device__ __attribute__((used)) unsigned plow_moe_w8a8_dec_abi_1 = 1;

struct DecGluArgs { /* amd.rs:1784-1807 */
    void* out;
    const void* x;
    const unsigned long long* wtab;
    const unsigned long long* stab;
    const int* meta;
    const unsigned* row_token;
    const float* x_scale;
    float* out_scale;
    unsigned inter, hidden, experts, act;
    float beta, lbeta;
    unsigned x_pitch, reserved;
};
struct DecDownArgs { /* amd.rs:1809-1828 */
    void* part;
    const void* fu;
    const unsigned long long* wtab;
    const unsigned long long* stab;
    const int* meta;
    const unsigned* row_partidx;
    const float* row_gate;
    const float* fu_scale;
    unsigned hidden, inter, experts, reserved;
};
struct DecPairArgs { /* amd.rs:3420-3430 */
    DecGluArgs g;
    DecDownArgs d;
    unsigned* ctr;
    unsigned grid_glu, reserved;
};
static_assert(sizeof(DecGluArgs) == 96 && sizeof(DecDownArgs) == 80 && sizeof(DecPairArgs) == 192, "plowrt's argument blocks");

__device__ __forceinline__ bool dec_glu_ok(const DecGluArgs& a) {
    return a.experts != 0u && a.inter != 0u && a.inter % 128u == 0u && a.hidden != 0u && a.hidden % 128u == 0u &&
           (a.x_scale == nullptr || a.x_pitch != 0u) && (unsigned long long)a.experts * (a.inter / 128u) <= 0x7FFFFFFFull;
}
__device__ __forceinline__ bool dec_down_ok(const DecDownArgs& a) {
    return a.experts != 0u && a.hidden != 0u && a.hidden % 256u == 0u && a.inter != 0u && a.inter % 128u == 0u &&
           (unsigned long long)a.experts * (a.hidden / 256u) <= 0x7FFFFFFFull;
}

/* The pair kernel's counters and its bounded wait: dec_pair_protocol.h. */
__device__ __forceinline__ void dec_item_done(unsigned* mine, uint32_t glu_items, uint32_t down_items) {
    /* release: this item's earlier accesses to the words (its add to word 0, its polls) are ordered before the
     * add; acquire: the item that sees the full count, and resets, is ordered after every other item's */
    const uint32_t before = __hip_atomic_fetch_add(mine + DP_ITEMS_DONE, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    if (dp_is_last(before, glu_items, down_items)) { /* every other item of the expert has made its last access */
        __hip_atomic_store(mine + DP_GLU_DONE, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(mine + DP_ITEMS_DONE, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

/* GLU work items first, first + stride, ...: (expert, 128 channels), heavy (folded shared) expert first */
template <bool AQ, bool FUSED>
__device__ __forceinline__ void dec_glu_items(const DecGluArgs& a, uint32_t first, uint32_t stride, float* s_red,
                                              unsigned* ctr, uint32_t down_items) {
    GroupW8A8 g = {};
    g.out = a.out; g.out_scale = a.out_scale; g.a = a.x; g.a_scale = a.x_scale;
    g.wtab = (const uint64_t*)a.wtab; g.stab = (const uint64_t*)a.stab; g.meta = a.meta; g.row_token = a.row_token;
    g.N = a.inter; g.K = a.hidden; g.E = a.experts; g.pitch = a.x_pitch; g.act = a.act; g.f0 = a.beta; g.f1 = a.lbeta;
    g.a_bf16 = AQ ? 1u : 0u;
    const uint32_t tiles = g.N / SK_BN, items = g.E * tiles;
    for (uint32_t it = first; it < items; it += stride) {
        const uint32_t e = g.E - 1u - it / tiles, ct = it % tiles;
        const uint32_t cnt = (uint32_t)g.meta[g.E + e];
        if (cnt == 0u || g.wtab[(size_t)e * 3u] == 0ull) continue; /* no rows, or not resident */
        const uint32_t r0 = (uint32_t)g.meta[e];
        for (uint32_t rb = 0; rb < cnt; rb += 16u) sk_body<1, true, 3, false, false, 4u, AQ>(g, e, ct, r0, rb, cnt, s_red);
        if (FUSED) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent"); /* this thread's fq / fs stores, device-wide */
            __syncthreads();
            if (threadIdx.x == 0) {
                unsigned* const mine = ctr + dp_expert_words((uint32_t)g.meta[2u * g.E + e]);
                __hip_atomic_fetch_add(mine + DP_GLU_DONE, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                dec_item_done(mine, tiles, down_items);
            }
        }
    }
}

/* DOWN work items: (expert, 256 channels) */
template <bool FUSED>
__device__ __forceinline__ void dec_down_items(const DecDownArgs& a, uint32_t first, uint32_t stride, float* s_red,
                                               unsigned* ctr, uint32_t* s_go, uint32_t spin_limit) {
    GroupW8A8 g = {};
    g.out = a.part; g.a = a.fu; g.a_scale = a.fu_scale;
    g.wtab = (const uint64_t*)a.wtab; g.stab = (const uint64_t*)a.stab; g.meta = a.meta;
    g.row_partidx = a.row_partidx; g.row_gate = a.row_gate;
    g.N = a.hidden; g.K = a.inter; g.E = a.experts;
    const uint32_t tiles = g.N / 256u, items = g.E * tiles;
    for (uint32_t it = first; it < items; it += stride) {
        const uint32_t e = g.E - 1u - it / tiles, ct = it % tiles;
        const uint32_t cnt = (uint32_t)g.meta[g.E + e];
        /* the GLU's own test: what it skipped is not counted and must not be waited for */
        if (cnt == 0u || g.wtab[(size_t)e * 3u] == 0ull) continue;
        bool go = g.wtab[(size_t)e * 3u + 2u] != 0ull;
        const uint32_t glu_items = g.K / SK_BN; /* GLU items of this expert */
        unsigned* const mine = FUSED ? ctr + dp_expert_words((uint32_t)g.meta[2u * g.E + e]) : nullptr;
        const uint32_t r0 = (uint32_t)g.meta[e];
        if (FUSED) {
            if (threadIdx.x == 0) {
                uint32_t ok = 0u;
                for (uint32_t spin = 0; spin < spin_limit; spin++) {
                    if (dp_down_ready(__hip_atomic_load(mine + DP_GLU_DONE, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), glu_items)) { ok = 1u; break; }
                    __builtin_amdgcn_s_sleep(32);
                }
                *s_go = ok;
            }
            __syncthreads();
            const bool ready = *s_go != 0u;
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent"); /* every wave reads fq / fs fresh */
            if (go && !ready) {
                /* the wait gave up: the rows this item owns say so (NaN), they do not keep stale data */
                const float poison = __builtin_nanf("");
                for (uint32_t i = threadIdx.x; i < cnt * 64u; i += 256u) {
                    const uint32_t pidx = g.row_partidx[r0 + i / 64u];
                    if (pidx != PLOW_EXPERT_UNUSED)
                        *(float4*)((float*)g.out + (size_t)pidx * g.N + ct * 256u + (i % 64u) * 4u) = make_float4(poison, poison, poison, poison);
                }
            }
            go = go && ready;
        }
        if (go)
            for (uint32_t rb = 0; rb < cnt; rb += 16u) sk_body<1, false, 3, false, true, 4u, false>(g, e, ct, r0, rb, cnt, s_red);
        if (FUSED) {
            __syncthreads(); /* s_go is free again; every wave is past its reads of fq / fs */
            if (threadIdx.x == 0) dec_item_done(mine, glu_items, tiles);
        }
    }
}

template <bool FUSED>
__device__ __forceinline__ void dec_glu(const DecGluArgs& a, uint32_t first, uint32_t stride, float* s_red, unsigned* ctr,
                                        uint32_t down_items) {
    if (a.x_scale) dec_glu_items<false, FUSED>(a, first, stride, s_red, ctr, down_items); /* e4m3 rows with their scales (arm 2) */
    else dec_glu_items<true, FUSED>(a, first, stride, s_red, ctr, down_items);            /* bf16 rows (arm 6) */
}

extern "C" __global__ __launch_bounds__(256) void plow_moe_w8a8_dec_glu(
    void* __restrict__ out, const void* __restrict__ x, const unsigned long long* __restrict__ wtab,
    const unsigned long long* __restrict__ stab, const int* __restrict__ meta, const unsigned* __restrict__ row_token,
    const float* __restrict__ x_scale, float* __restrict__ out_scale, unsigned inter, unsigned hidden,
    unsigned experts, unsigned act, float beta, float lbeta, unsigned x_pitch, unsigned reserved) {
    __shared__ float s_red[SK_WAVES * 64u];
    const DecGluArgs a = {out, x, wtab, stab, meta, row_token, x_scale, out_scale, inter, hidden, experts, act,
                          beta, lbeta, x_pitch, reserved};
    if (!dec_glu_ok(a)) return;
    dec_glu<false>(a, blockIdx.x, gridDim.x, s_red, nullptr, 0u);
}

extern "C" __global__ __launch_bounds__(256) void plow_moe_w8a8_dec_down(
    void* __restrict__ part, const void* __restrict__ fu, const unsigned long long* __restrict__ wtab,
    const unsigned long long* __restrict__ stab, const int* __restrict__ meta, const unsigned* __restrict__ row_partidx,
    const float* __restrict__ row_gate, const float* __restrict__ fu_scale, unsigned hidden, unsigned inter,
    unsigned experts, unsigned reserved) {
    __shared__ float s_red[SK_WAVES * 64u];
    const DecDownArgs a = {part, fu, wtab, stab, meta, row_partidx, row_gate, fu_scale, hidden, inter, experts, reserved};
    if (!dec_down_ok(a)) return;
    dec_down_items<false>(a, blockIdx.x, gridDim.x, s_red, nullptr, nullptr, 0u);
}

/* Both grids in one launch: workgroups [0, grid_glu) walk the GLU items, the others the DOWN items, each
 * of which waits for its expert's GLU items (counters above). A GLU workgroup never waits and workgroups
 * are dispatched in index order, so everything a waiting workgroup depends on is running or done. */
extern "C" __global__ __launch_bounds__(256) void plow_moe_w8a8_dec_pair(DecPairArgs a) {
    __shared__ float s_red[SK_WAVES * 64u];
    __shared__ uint32_t s_go;
    const uint32_t ng = a.grid_glu, nb = gridDim.x;
    if (!dec_glu_ok(a.g) || !dec_down_ok(a.d) || a.d.inter != a.g.inter || a.d.experts != a.g.experts ||
        a.d.meta != a.g.meta || a.d.wtab != a.g.wtab || a.ctr == nullptr || ng == 0u || ng >= nb)
        return;
    /* a.reserved: polls before a DOWN item gives up its wait (0 = the default, seconds) */
    if (blockIdx.x < ng) dec_glu<true>(a.g, blockIdx.x, ng, s_red, a.ctr, a.d.hidden / 256u);
    else dec_down_items<true>(a.d, blockIdx.x - ng, nb - ng, s_red, a.ctr, &s_go, dp_spin_limit(a.reserved));
}
