/* Measuring aids of the benchmark (libtfcc_bench.so, built from probe.hip by the Makefile of this directory).
 * Not part of the product library and not of its C ABI: nothing but bench.py calls them. */
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* A measuring aid, no counterpart in the reference: a register-resident loop of matrix-core
 * instructions (no LDS, no memory traffic) on `blocks` workgroups of four wavefronts, each wavefront
 * issuing 4 * iters instructions (iters a multiple of 4) of kind 0 (int8 32x32x32, 65536 ops each) or 1 (fp32 32x32x2, 4096
 * flops each).  With changing_operands the operands differ from one instruction to the next, as a
 * product of real matrices presents them; otherwise they are constant.  The caller times the launch;
 * out receives blocks * 256 words that only keep the loop alive. */
int tfcc_bench_probe_mfma(void* stream, int kind, int changing_operands, unsigned blocks, unsigned iters,
                         int32_t* out);
/* More measuring aids: a launch that only reads `bytes` from src once (blocks workgroups of 512 threads,
 * contiguous shares, 16-byte loads) - the time a read-bound kernel of that size cannot beat - and a
 * launch of 256 workgroups that do nothing - the time from dispatch to completion that every kernel pays. */
int tfcc_bench_probe_read(void* stream, const void* src, uint64_t bytes, unsigned blocks, int32_t* out);
int tfcc_bench_probe_launch(void* stream, int32_t* out);

#ifdef __cplusplus
}
#endif
