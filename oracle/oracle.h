/* oracle.h — exports of the CPU oracle (liboracle.so). TEST INFRASTRUCTURE ONLY: loaded by tests/,
 * by the smoke check and by the benchmark's cpu_baseline leg; never by the shipped library. */
#ifndef PLOW_ORACLE_H
#define PLOW_ORACLE_H

#include "../include/plow_moe.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Run one op descriptor on the CPU. `tensors` holds HOST pointers (pointer tables such as wtab hold
 * host pointers too). nthreads <= 1 runs slice 0 of 1 inline; otherwise nthreads workers run slices
 * 0..nthreads-1 concurrently, the reference's (slice, nblk) worker contract
 * (runtime/cpu/dev/cpu_dev.h:172-176). Returns 0 or PLOW_MOE_EUNSUPPORTED. */
int plow_oracle_exec(const PlowDevInst* inst, void* const* tensors, uint32_t nthreads);
int plow_oracle_exec_many(const PlowDevInst* insts, uint32_t n, void* const* tensors, uint32_t nthreads);

/* timing runs: pin worker s to the s-th CPU the process may run on (0 = off, the default) */
void plow_oracle_pin_workers(int on);

uint16_t plow_oracle_f2bf(float f);
float    plow_oracle_bf2f(uint16_t h);
uint8_t  plow_oracle_f32_to_e4m3(float f);
float    plow_oracle_e4m3_to_f32(uint8_t b);
float    plow_oracle_e2m1(uint8_t nib);
float    plow_oracle_e8m0(uint8_t s);
void     plow_oracle_f2bf_n(uint16_t* dst, const float* src, size_t n);
void     plow_oracle_e4m3_encode_n(uint8_t* dst, const float* src, size_t n);
/* the two e4m3 terms of ops 85 / 86 arms 4 / 5: hi = e4m3(v), lo = e4m3((v - hi) * 16) */
void     plow_oracle_split_e4m3_n(uint8_t* hi, uint8_t* lo, const float* src, size_t n);
/* the activation quantizer of the fp4 x fp4 arm (ops 85 / 86, enc 2, arm 0): n_blocks 32-blocks of f32 ->
 * 16 bytes and one E8M0 byte each; its two primitives */
void     plow_oracle_mx_act_quant(uint8_t* out, uint8_t* scales, const float* v, size_t n_blocks);
uint8_t  plow_oracle_mx_act_e8m0(float amax);
uint8_t  plow_oracle_mx_act_fp4(float v);

#ifdef __cplusplus
}
#endif
#endif
