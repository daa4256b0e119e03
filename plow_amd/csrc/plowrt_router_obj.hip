/* plowrt_router_obj.hip — the device code object an unmodified plowrt loads for its raw decode-router
 * segments on gfx950: `router_decode_gfx950.elf`.
 *
 * plowrt (plow crates/plowrt/src/exec/amd.rs:10755-10800) wants the kernel `plow_router_decode`, the marker
 * `plow_router_decode_abi_3`, a 104-byte argument block (RouterDecodeArgs, :955-982) and no private memory;
 * it launches rows * per_row workgroups of 512 threads with no dynamic LDS, per_row = ceil(n_exp / 8)
 * (:1009, :17811-17832), for rows <= 256, n_exp <= 512, k <= 8, sigmoid scoring over f32 logits (:995-1008).
 * Workgroups [r * per_row, (r + 1) * per_row) belong to row r; they count themselves off on the row's
 * arrival counter (32 words apart, zero between launches) and the last one runs the top-k over the row
 * (plow runtime/amd/router_decode.hip:40-63).
 *
 * The bodies are the library's: the few-token score (one f32 accumulator per logit walking k upwards, the
 * order of plow's CPU reference) and the per-token top-k. A workgroup of the score body covers 64 experts,
 * so the first ceil(n_exp / 64) workgroups of a row compute and the rest only count themselves off; five
 * of the eight waves work (ended waves do not take part in a workgroup's barriers). Logits and table are
 * the bytes of the library's op 180 followed by op 83. */
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "route_body.h"

extern "C" __device__ __attribute__((used)) unsigned plow_router_decode_abi_3 = 1;

struct RouterDecodeArgs {
    float* logit;
    const bf16_t* x;
    const bf16_t* w;
    unsigned char* table;
    const float* bias;
    unsigned* ctr; /* [rows] counters, 32 words apart, zero between launches */
    unsigned* signal;
    unsigned rows, n_exp, k_dim, topk, flags, shared_tail, n_group, topk_group;
    float route_scale;
    unsigned per_row, signal_add, pad;
};
static_assert(sizeof(RouterDecodeArgs) == 104, "plowrt copies 104 bytes");

extern "C" __global__ __launch_bounds__(512) void plow_router_decode(RouterDecodeArgs a) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[RSR_LDS];
    __shared__ uint32_t s_flag;
    if (a.per_row == 0u || a.n_exp == 0u || a.n_exp > 512u || a.topk == 0u) return;
    const uint32_t row = blockIdx.x / a.per_row, part = blockIdx.x % a.per_row;
    const uint32_t wv = threadIdx.x >> 6, lane = threadIdx.x & 63u;
    if (row >= a.rows || wv >= 1u + RSR_STAGERS) return;
    if (part < (a.n_exp + 63u) / 64u) {
        if (a.k_dim % RSR_KC == 0u) {
            router_score_row_body<1>(a.logit, a.x, a.w, a.rows, a.n_exp, a.k_dim, part, row, lds);
        } else if (wv == 0u) { /* any other K: the same sum, one logit per lane straight from memory */
            const uint32_t n = part * 64u + lane;
            if (n < a.n_exp) {
                float acc = 0.0f;
                for (uint32_t k = 0; k < a.k_dim; k++)
                    acc = fmaf(bf2f(a.x[(size_t)row * a.k_dim + k]), bf2f(a.w[(size_t)n * a.k_dim + k]), acc);
                a.logit[(size_t)row * a.n_exp + n] = acc;
            }
        }
    }
    if (!rf_last_arrival(a.ctr + (size_t)row * 32u, a.per_row, &s_flag)) return;
    if (wv == 0u) {
        const RouterArgs t = {(PlowMoeRoute*)a.table, a.logit, a.bias, a.n_exp, a.topk, a.flags, a.rows, a.shared_tail ? 1u : 0u,
                              a.n_group, a.topk_group, a.route_scale, 0.0f};
        if (a.n_exp <= 128u) router_topk_token<2>(t, row, (float*)lds);
        else if (a.n_exp <= 256u) router_topk_token<4>(t, row, (float*)lds);
        else if (a.n_exp <= 384u) router_topk_token<6>(t, row, (float*)lds);
        else router_topk_token<8>(t, row, (float*)lds);
        if (a.signal_add) { /* the table is written: tell whoever waits on the counter */
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
            if (lane == 0u) __hip_atomic_fetch_add(a.signal, a.signal_add, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}
