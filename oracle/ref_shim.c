/* ref_shim.c — thin driver over plow's OWN CPU kernel library, compiled from the plow tree where it
 * is mounted (never copied). TEST INFRASTRUCTURE ONLY: it exists to validate oracle.c against the
 * reference and to write golden vectors; it does not exist on a machine without the plow tree.
 *
 * Calls plow_cpu_kernel(op)(inst, slice, nblk, tensors, ctx) exactly as the reference's own tests do
 * (runtime/tests/cpu_dev_route_test.c:16-19). */
#include <stdlib.h>
#include <string.h>
#include "cpu_dev.h"

static PlowCpuCtx g_ctx;
static int g_tier = -100;

/* isa_cap: 0 scalar golden tier, 1 AVX-512, 2 AMX. Returns the active tier. */
int plow_ref_init(int isa_cap) {
    if (g_tier == -100) {
        g_tier = plow_cpu_init(isa_cap);
        memset(&g_ctx, 0, sizeof g_ctx);
        g_ctx.scratch_bytes = plow_cpu_scratch_bytes();
        if (g_ctx.scratch_bytes < (8u << 20)) g_ctx.scratch_bytes = 8u << 20;
        g_ctx.scratch = aligned_alloc(64, g_ctx.scratch_bytes);
        plow_cpu_thread_init(&g_ctx);
    }
    return g_tier;
}

int plow_ref_has(uint16_t op) { return plow_cpu_has(op); }
int plow_ref_tier_of(uint16_t op) { return plow_cpu_tier_of(op); }

/* Runs slices 0..nblk-1 of one op in order on the calling thread. -1: no kernel for this op. */
int plow_ref_exec(const PlowDevInst* inst, void* const* tensors, uint32_t nblk) {
    plow_cpu_kernel_fn fn = plow_cpu_kernel(inst->op);
    if (!fn) return -1;
    PlowDevInst in = *inst;
    if (nblk == 0) nblk = 1;
    in.blocks = (uint16_t)nblk;
    for (uint32_t s = 0; s < nblk; s++) fn(&in, s, nblk, tensors, &g_ctx);
    return 0;
}
