/* Measuring aids of the benchmark (libtfcc_bench.so, built from probe.hip by the Makefile of this directory).
 * Not part of the product library and not of its C ABI: nothing but bench.py calls them. */
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* A measuring aid, no counterpart in the reference: a register-resident loop of matrix-core
 * instructions (no LDS, no memory traffic) on `blocks` workgroups of four wavefronts.
 *   kind 0  int8 32x32x32 (65536 ops an instruction), kind 1  fp32 32x32x2 (4096 flops), kind 2  int8 16x16x64 (32768 ops)
 *   changing_operands 0  every instruction sees the same operand values
 *                     1  four accumulators, both operands differ from one instruction to the next
 *   For both of these a wavefront issues 4 * iters instructions (iters a multiple of 4).
 *                     2  (kinds 0 and 2) the issue order of a GEMM kernel: a wavefront owns 128 x 128 outputs in all
 *                        256 accumulation registers, one operand stays for a row of blocks (4 instructions of
 *                        32x32x32, 8 of 16x16x64), the other changes with every instruction, every other row runs
 *                        backwards; after each k step (16 or 64 instructions) every operand register has half of
 *                        its bits flipped.  iters counts k steps.  The operand that stays is the second source.
 *                     3  the same with the first source as the one that stays
 * The caller times the launch; out receives blocks * 256 words that only keep the loop alive. */
int tfcc_bench_probe_mfma(void* stream, int kind, int changing_operands, unsigned blocks, unsigned iters,
                         int32_t* out);
/* Pattern 2 of kind 0 with the matrix cores busy only part of the time: after every k step (16 instructions, 512
 * cycles) each wavefront sleeps 64 * sleep cycles (sleep in {0, 1, 2, 4, 8}: busy share 1, 0.89, 0.80, 0.67, 0.50).
 * Together with the clock and power read while it runs this says what a kernel gains, under the power limit, from
 * spending fewer cycles outside its matrix ops. */
int tfcc_bench_probe_mfma_duty(void* stream, int sleep, unsigned blocks, unsigned ksteps, int32_t* out);
/* More measuring aids: a launch that only reads `bytes` from src once (blocks workgroups of 512 threads,
 * contiguous shares, 16-byte loads) - the time a read-bound kernel of that size cannot beat - and a
 * launch of 256 workgroups that do nothing - the time from dispatch to completion that every kernel pays. */
int tfcc_bench_probe_read(void* stream, const void* src, uint64_t bytes, unsigned blocks, int32_t* out);
int tfcc_bench_probe_launch(void* stream, int32_t* out);

#ifdef __cplusplus
}
#endif
