/* tuning.h — the registry of the library's environment knobs and the per-device facts its launchers
 * use. Every knob is read exactly once per process (thread-safe), here; nothing else in the library
 * calls getenv. Every knob only selects between kernels that compute the same results: they exist for
 * A/B timing, and the defaults are what the measurements chose.
 *
 *   PLOW_MOE_W8A8_KERNEL      stream | tiled   force one form of the fp8 x fp8 grouped GEMMs
 *                                              (default: chosen per op from its row count)
 *   PLOW_MOE_W8A8_TILE_WAVES  4                512-thread form of the tiled kernel (default 768 threads)
 *   PLOW_MOE_TILED_NT         0 | 1            tiled kernels' weight rows never / always non-temporal (default: by rows per expert)
 *   PLOW_MOE_SK_DEPTH         2..4             k-steps of weight loads in flight, register form (default 3)
 *   PLOW_MOE_SK_GLU           regs             block-mode decode GLU on the register form (default: direct-to-LDS form)
 *   PLOW_MOE_SK_DOWN          regs             block-mode decode DOWN on the register form (default: direct-to-LDS form)
 *   PLOW_MOE_SK_NARROW        (any)            decode DOWN register form with 128-channel workgroups (default 256)
 *   PLOW_MOE_A16_KERNEL       regs             bf16-activation kernels on their register form (default: direct-to-LDS form)
 *   PLOW_MOE_SCORE_KERNEL     tile8 | valu     router score: keep the 8 x 8 tile kernel for few outputs / keep
 *                                              the vector-unit kernels at prefill sizes
 *   PLOW_MOE_A16_TILED        0                keep the bf16-activation arms on the streaming kernels at every row count
 *   PLOW_MOE_A16_TILED_MX     0                keep mxfp4 weights under bf16 activations on the streaming kernels at every row count
 *   PLOW_MOE_A16_GEMV         0                keep the bf16-activation arms off the matrix-vector form at a few tokens
 *   PLOW_MOE_A16_DOWN_WIDE    0                streaming bf16-activation DOWN on tiles of 128 channels (default: 256 while
 *                                              they give every CU two workgroups)
 *   PLOW_MOE_A16_PRIVATE_ROWS 0                streaming bf16-activation kernels: experts of a handful of rows share the
 *                                              workgroup's row ring like the others (default: per-wave copies on fp8 and
 *                                              bf16 weights)
 *   PLOW_MOE_GEMV_DIRECT      0                slot-major ops of a handful of slots sort their slots like the others (default: the
 *                                              matrix-vector form lists its rows from the routing table itself)
 *   PLOW_MOE_DENSE_OVERLAP    0                a run's dense shared-expert ops of a few rows stay on the caller's stream, in
 *                                              their place (default: on the context's second stream beside the routed experts)
 *   PLOW_MOE_A16_DENSE_SPLIT  0                dense bf16 ops of a few rows walk the whole K in one workgroup per channel
 *                                              tile (default: K split over several workgroups while the tiles are
 *                                              fewer than the CUs)
 *   PLOW_MOE_SCORE_ROW        narrow           router score: the one-token-per-wave kernel only below 16 tokens (default: while
 *                                              its workgroups fit the chip)
 *   PLOW_MOE_FORM_ON_DEVICE   0                a grouped fp8 x fp8 op without a row count runs the streaming form
 *                                              (default: both forms are launched behind a choice made on the device)
 */
#ifndef PLOW_MOE_TUNING_H
#define PLOW_MOE_TUNING_H

#include <stdint.h>

struct PlowMoeTuning {
    int w8a8_kernel;      /* -1 auto, 0 stream, 1 tiled */
    bool tile_waves4;
    int tiled_nt;         /* -1 auto, 0, 1 */
    int sk_depth;         /* 2..4 */
    bool sk_glu_regs;
    bool sk_down_regs;
    bool sk_narrow;
    bool a16_regs;
    bool score_tile8;
    bool score_valu;
    bool a16_tiled;
    bool a16_gemv;
    bool form_on_device;
    bool score_row_narrow;
    bool a16_tiled_mx;
    bool a16_down_wide;
    bool a16_private_rows;
    bool a16_dense_split;
    bool gemv_direct;
    bool dense_overlap;
};
const PlowMoeTuning& plow_moe_tuning();

/* Per-device set-up, done once per device by plow_moe_create with that device current: the CU count
 * and the dynamic-LDS attribute of every kernel that needs more than the default. Returns 0 or a
 * negative PLOW_MOE_E* code. Launchers read the CU count of the current device with plow_moe_n_cu()
 * (0 if the device was never set up: the launchers then refuse). */
int plow_moe_device_setup(int device);
uint32_t plow_moe_n_cu();

/* The library's static device array: workspace of plow_moe_exec_noalloc, one copy per GPU at its own
 * address, held from the moment the library's code is loaded on that GPU until the process ends. Its
 * address on the current device (resolved by plow_moe_device_setup), or NULL. */
#define PLOW_MOE_STATIC_BYTES (1u << 20)
void* plow_moe_static_scratch();

/* one per translation unit with kernels that use dynamic LDS beyond the default limit */
int plow_moe_route_setup();
int plow_moe_w8a8_setup();
int plow_moe_w8a8_tiled_setup();
int plow_moe_a16_setup();

#endif
