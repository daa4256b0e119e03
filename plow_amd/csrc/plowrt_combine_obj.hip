/* plowrt_combine_obj.hip — the device code object an unmodified plowrt loads for its MoE combine
 * segments on gfx950: `moe_combine_gfx950.elf`.
 *
 * plowrt (plow crates/plowrt/src/exec/amd.rs:11666-11716) wants the kernel
 * `plow_moe_combine_fixed_order_gfx950`, five marker symbols, a 48-byte argument block (MoeCombineArgs,
 * :1771-1782), no LDS and no private memory; it launches min(tokens, 512) workgroups of 256 threads
 * (:4018-4036, :16482-16495). The kernel below is the library's combine (op 87: f32 partial rows added in
 * slot order on top of residual and shared, one bf16 rounding) behind that name. plow's own object serves
 * sixteen slots per token only (runtime/bench/amd/lean_moe_combine_ref/kernel.hip:20-21); this one takes
 * any slot count. */
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "combine_body.h"

extern "C" __device__ __attribute__((used)) unsigned plow_moe_combine_fixed_order_abi_1 = 1;
extern "C" __device__ __attribute__((used)) unsigned plow_moe_combine_fixed_order_slots16_1 = 1;
extern "C" __device__ __attribute__((used)) unsigned plow_moe_combine_materialized_f32_1 = 1;
extern "C" __device__ __attribute__((used)) unsigned plow_moe_combine_wave64_1 = 1;
extern "C" __device__ __attribute__((used)) unsigned plow_moe_combine_no_spill_1 = 1;

extern "C" __global__ __launch_bounds__(256) void plow_moe_combine_fixed_order_gfx950(
    bf16_t* __restrict__ out, const bf16_t* __restrict__ residual, const bf16_t* __restrict__ shared,
    const float* __restrict__ part, unsigned hidden, unsigned topk, unsigned tokens, unsigned reserved) {
    (void)reserved;
    if (hidden % 4u || tokens == 0u) return;
    CombineArgs a = {out, residual, shared, part, hidden, topk, tokens, 0u};
    switch (topk) {
    case 8: combine_body<8>(a); break;
    case 9: combine_body<9>(a); break;
    case 16: combine_body<16>(a); break;
    default: combine_body<0>(a); break;
    }
}
