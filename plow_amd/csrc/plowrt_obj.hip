/* plowrt_obj.hip — the device code object an unmodified plowrt loads for its block-fp8 grouped-MoE
 * prefill segments on gfx950: `moe_fp8_pf_gfx950.elf`.
 *
 * What plowrt expects of that object (plow crates/plowrt/src/exec/amd.rs):
 *   :11718-11760  the file name, the five kernel symbols below, and the marker symbol
 *                 `plow_moe_fp8_pf_abi_2` in the ELF symbol table (runtime/amd/moe_fp8_pf.hip:25-26);
 *   :1784-1828    one by-value argument block per kernel: MoeFp8GluArgs (96 bytes) and MoeFp8DownArgs
 *                 (80 bytes); the parameter lists below lay out exactly those bytes
 *                 (runtime/amd/moe_fp8_pf.hip:1176-1189);
 *   :16069-16100  the launch: a 1-D grid taken from the instruction's `blocks` field (any size), 512
 *                 threads, no dynamic LDS. Every kernel here therefore walks its work with a stride of
 *                 gridDim.x and keeps its LDS in a static array.
 * W8A8 (fp8 activations with 1x128 scales): the tiled kernel of experts_w8a8_tiled.hip in its 512-thread
 * form (four consumer waves + four loader waves). W8A16 (bf16 activations): the direct-load kernel of
 * experts_a16.hip with four 16-row groups per pass over the weights. Same arithmetic as the library's
 * ops 85 / 86; shapes a kernel cannot serve make it return without writing, as plow's own do. */
#include "experts_w8a8_tiled.hip"
#include "experts_a16.hip"

extern "C" __device__ __attribute__((used)) unsigned plow_moe_fp8_pf_abi_2 = 1;
extern "C" __device__ __attribute__((used)) unsigned plow_moe_fp8_pf_w8a8_1 = 1;

#define PLOWRT_GLU_ARGS                                                                                       \
    void *__restrict__ out, const void *__restrict__ x, const unsigned long long *__restrict__ wtab,         \
        const unsigned long long *__restrict__ stab, const int *__restrict__ meta,                           \
        const unsigned *__restrict__ row_token, const float *__restrict__ x_scale, float *__restrict__ out_scale, \
        unsigned inter, unsigned hidden, unsigned experts, unsigned act, float beta, float lbeta,            \
        unsigned x_pitch, unsigned reserved
#define PLOWRT_DOWN_ARGS                                                                                      \
    void *__restrict__ part, const void *__restrict__ fu, const unsigned long long *__restrict__ wtab,       \
        const unsigned long long *__restrict__ stab, const int *__restrict__ meta,                           \
        const unsigned *__restrict__ row_partidx, const float *__restrict__ row_gate,                        \
        const float *__restrict__ fu_scale, unsigned hidden, unsigned inter, unsigned experts, unsigned reserved

/* the tiled kernel's limits: its tile directory holds 1056 experts, a tile keeps K / 128 <= 128 block
 * scales in LDS, and the load ring runs two 128-k blocks ahead */
__device__ __forceinline__ bool tiled_ok(unsigned N, unsigned K, unsigned E) {
    return E != 0u && E <= 1056u && N != 0u && N % 128u == 0u && K % 128u == 0u && K >= 256u && K <= 16384u;
}

extern "C" __global__ __launch_bounds__(512) void plow_moe_w8a8_glu_pf_gfx950(PLOWRT_GLU_ARGS) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[sizeof(T5Lds)];
    (void)reserved;
    if (!tiled_ok(inter, hidden, experts) || x_pitch == 0u) return;
    GroupW8A8 g = {};
    g.out = out; g.out_scale = out_scale; g.a = x; g.a_scale = x_scale;
    g.wtab = (const uint64_t*)wtab; g.stab = (const uint64_t*)stab; g.meta = meta; g.row_token = row_token;
    g.N = inter; g.K = hidden; g.E = experts; g.pitch = x_pitch; g.act = act; g.f0 = beta; g.f1 = lbeta;
    t5_body<true, false, 4u>(g, lds);
}

__device__ __forceinline__ void w8a8_down(PLOWRT_DOWN_ARGS, uint8_t* lds, unsigned acc_topk) {
    (void)reserved;
    if (!tiled_ok(hidden, inter, experts)) return;
    GroupW8A8 g = {};
    g.out = part; g.a = fu; g.a_scale = fu_scale;
    g.wtab = (const uint64_t*)wtab; g.stab = (const uint64_t*)stab; g.meta = meta;
    g.row_partidx = row_partidx; g.row_gate = row_gate;
    g.N = hidden; g.K = inter; g.E = experts; g.acc_topk = acc_topk;
    t5_body<false, false, 4u>(g, lds);
}

extern "C" __global__ __launch_bounds__(512) void plow_moe_w8a8_down_pf_gfx950(PLOWRT_DOWN_ARGS) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[sizeof(T5Lds)];
    w8a8_down(part, fu, wtab, stab, meta, row_partidx, row_gate, fu_scale, hidden, inter, experts, reserved, lds, 0u);
}

/* `part` is the bf16 [T][H] layer output the caller has seeded; reserved = routing slots per token */
extern "C" __global__ __launch_bounds__(512) void plow_moe_w8a8_down_acc_pf_gfx950(PLOWRT_DOWN_ARGS) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[sizeof(T5Lds)];
    if (reserved == 0u) return;
    w8a8_down(part, fu, wtab, stab, meta, row_partidx, row_gate, fu_scale, hidden, inter, experts, reserved, lds, reserved);
}

/* bf16 activations: workgroup index b of the logical grid E * N / 128, walked with the launch's stride */
__device__ __forceinline__ bool a16_ok(unsigned N, unsigned K, unsigned E) {
    return E != 0u && N != 0u && N % 128u == 0u && K != 0u && K % 128u == 0u && K <= 16384u &&
           (unsigned long long)E * (N / 128u) <= 0x7FFFFFFFull;
}

extern "C" __global__ __launch_bounds__(512) void plow_moe_fp8_glu_pf_gfx950(PLOWRT_GLU_ARGS) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[sizeof(DmLds<AENC_FP8BLK, true, 4>)];
    (void)x_scale; (void)out_scale; (void)x_pitch; (void)reserved;
    if (!a16_ok(inter, hidden, experts)) return;
    GroupA16 g = {};
    g.out = out; g.a = x; g.wtab = (const uint64_t*)wtab; g.stab = (const uint64_t*)stab; g.meta = meta;
    g.a_idx = row_token;
    g.N = inter; g.K = hidden; g.E = experts; g.enc = AENC_FP8BLK; g.act = act; g.f0 = beta; g.f1 = lbeta;
    g.wcols = 3; g.wsel0 = 0; g.wsel1 = 1;
    const uint32_t nwg = experts * (inter / 128u);
    for (uint32_t b = blockIdx.x; b < nwg; b += gridDim.x) {
        DmWork w;
        if (a16_dma_work<AENC_FP8BLK>(g, b, w)) a16_dma_body<AENC_FP8BLK, true, 4>(g, lds, w);
        __syncthreads();
    }
}

extern "C" __global__ __launch_bounds__(512) void plow_moe_fp8_down_pf_gfx950(PLOWRT_DOWN_ARGS) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[sizeof(DmLds<AENC_FP8BLK, false, 4>)];
    (void)fu_scale; (void)reserved;
    if (!a16_ok(hidden, inter, experts)) return;
    GroupA16 g = {};
    g.out = part; g.a = fu; g.wtab = (const uint64_t*)wtab; g.stab = (const uint64_t*)stab; g.meta = meta;
    g.o_idx = row_partidx; g.gate = row_gate;
    g.N = hidden; g.K = inter; g.E = experts; g.enc = AENC_FP8BLK;
    g.wcols = 3; g.wsel0 = 2; g.wsel1 = 2;
    const uint32_t nwg = experts * (hidden / 128u);
    for (uint32_t b = blockIdx.x; b < nwg; b += gridDim.x) {
        DmWork w;
        if (a16_dma_work<AENC_FP8BLK>(g, b, w)) a16_dma_body<AENC_FP8BLK, false, 4>(g, lds, w);
        __syncthreads();
    }
}
