/*
 * CPU oracle for the TFCC matmul hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of the arithmetic the reference performs on its
 * MKL (CPU) device for tfcc::blas::matmul, the quantized uint8 x int8 -> int32
 * matmul and the range-based quantize / requantize / dequantize steps.  It is
 * the checker the parity tests, the smoke test and the benchmark's CPU-baseline
 * leg compare the HIP kernels against.  Nothing on the product path may link,
 * load or call it.
 *
 * Every function cites the reference file:line (relative to the reference
 * root) whose behaviour it restates.
 *
 * Pinning status:
 *   oracle_qgemm_u8s8s32, oracle_reduce_sum_*   pinned by the reference's own AVX2
 *       kernel (oracle/_ref, built from the reference sources) and by the closed
 *       form (A+oA)(B+oB) the reference's test generator uses.
 *   oracle_quantized_scale_info, oracle_dequantized_scale_info,
 *   oracle_requantize_*, oracle_dequantize_*, oracle_quantize_*
 *       pinned by the known answers in tfcc/test/quantization.cpp:67-101,128-189
 *       and by the reference AVX2 requantize/quantize/dequantize kernels in oracle/_ref.
 *   oracle_sgemm_strided_batched
 *       the reference's fp32 arithmetic is oneDNN v1.8.1's sgemm (not vendored,
 *       not present): exact bit pattern "parity unpinned"; pinned to the
 *       mathematics (fp64 accumulation; identity / one-hot / all-ones /
 *       power-of-two cases; brute force) under the stated tolerance
 *       (relative Frobenius error <= 1e-5).
 *   oracle_lstm_cell, oracle_gru_cell_*, oracle_pytorch_gru_cell
 *       pinned by the reference's own scalar cell kernels (oracle/_ref, built from the reference
 *       header) and by the formulas of the reference's test generators
 *       (tfcc/test/python/testcase/rnn/lstmcell.py:31-44, pytorchgrucell.py) evaluated in float64.
 *   oracle_lstm_sequence
 *       pinned by the recurrence of tfcc/test/python/testcase/rnn/lstmforward.py:33-44,62-69 and
 *       lstmbackward.py evaluated in float64, under the fp32 tolerance of the matrix products.
 */
#ifndef TFCC_ORACLE_H_
#define TFCC_ORACLE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- shape rules of tfcc::blas::matmul ------------------------------------- */

enum {
  ORACLE_OK = 0,
  ORACLE_ERR_RANK = 1,   /* "matmul require tensors with two or more dimensions" */
  ORACLE_ERR_SHAPE = 2,  /* "shape invalid" */
};

/*
 * Validation + stride rules.  tfcc/core/operations/tfcc_blas.cpp:26-58 (two-operand),
 * :61-96 (with bias; pass biasRank = -1 for the two-operand form), and
 * tfcc/mkl/interfaces/tfcc_mklblasinterface.cpp:127-151 (m, n, k, strides, result shape,
 * batch count).  resultShape must have room for max(rankA, rankB) entries.
 * *empty is set when either operand has zero elements (the reference then returns an
 * uninitialised tensor of the result shape and computes nothing).
 */
int oracle_matmul_plan(const unsigned* shapeA, int rankA, const unsigned* shapeB, int rankB,
                       const unsigned* shapeBias, int biasRank, unsigned* resultShape,
                       int* resultRank, unsigned* m, unsigned* n, unsigned* k, unsigned* strideA,
                       unsigned* strideB, unsigned* strideC, unsigned* batch, int* empty);

/* ---- fp32 matmul ------------------------------------------------------------ */

/*
 * C[b] = A[b] * B[b] (+ bias broadcast over rows), row-major, batch strides in elements
 * (0 = operand shared by all batches).  tfcc/mkl/interfaces/tfcc_mklblasinterface.cpp:41-67
 * (plain) and :69-78,87-118 (bias pre-fill, then C += A*B).  Sums are formed in double and
 * rounded once; c64 (optional) receives the unrounded double result.
 */
void oracle_sgemm_strided_batched(const float* a, uint64_t strideA, const float* b,
                                  uint64_t strideB, const float* bias, float* c, double* c64,
                                  uint64_t strideC, unsigned m, unsigned n, unsigned k,
                                  unsigned batch);

/* ---- quantized uint8 x int8 -> int32 matmul ---------------------------------- */

/*
 * Row (last dim reduced, result [batch, rows]) and column (result [batch, cols]) sums in int32.
 * tfcc/mkl/operations/tfcc_mklquantization.cpp:205-237 and :239-282.
 */
void oracle_reduce_sum_row_u8(const uint8_t* a, unsigned batch, unsigned row, unsigned col, int32_t* out);
void oracle_reduce_sum_row_s8(const int8_t* a, unsigned batch, unsigned row, unsigned col, int32_t* out);
void oracle_reduce_sum_col_u8(const uint8_t* a, unsigned batch, unsigned row, unsigned col, int32_t* out);
void oracle_reduce_sum_col_s8(const int8_t* a, unsigned batch, unsigned row, unsigned col, int32_t* out);

/*
 * offsetA / offsetB as the quantized matmul derives them from the float ranges:
 * tfcc/mkl/operations/tfcc_mklquantization.cpp:181-186.
 */
void oracle_qmatmul_offsets(float minA, float maxA, float minB, float maxB, int32_t* offsetA,
                            int32_t* offsetB);

/*
 * C[b][i][j] = K*oA*oB + rowsumA[b][i]*oB + colsumB[b][j]*oA + sum_k A[b][i][k]*B[b][k][j],
 * all in wrap-around int32.  Offset matrix: tfcc/mkl/operations/tfcc_mklquantization.cpp:33-69;
 * accumulation into it: tfcc/mkl/gemm/tfcc_mklmatmulkernel.h:142-260 via
 * tfcc/mkl/kernel/tfcc_mklquantizationmatmul.avx256.cpp:90-165.  Strides in elements,
 * 0 = shared.  The caller passes the sums; they are NOT recomputed (the reference trusts them too).
 */
void oracle_qgemm_u8s8s32(unsigned batch, const uint8_t* a, uint64_t strideA, const int8_t* b,
                          uint64_t strideB, const int32_t* rowsumA, uint64_t strideRA,
                          const int32_t* colsumB, uint64_t strideRB, int32_t offsetA,
                          int32_t offsetB, unsigned m, unsigned n, unsigned k, int32_t* c,
                          uint64_t strideC);

/* [minC, maxC] of the int32 result.  tfcc/core/utils/tfcc_quantizationutils.h:23-43. */
void oracle_qmatmul_range(float minA, float maxA, float minB, float maxB, float* minC, float* maxC);

/* ---- range arithmetic --------------------------------------------------------- */

/* tfcc/core/utils/tfcc_quantizationutils.h:45-56.  bits = 8, 16 or 32. */
void oracle_quantized_scale_info(int bits, float minValue, float maxValue, double* scale,
                                 int64_t* offset);
/* tfcc/core/utils/tfcc_quantizationutils.h:58-70. */
void oracle_dequantized_scale_info(int bits, float minValue, float maxValue, double* scale,
                                   double* minRounded);

/* Rounding / contraction of the kernel being restated. */
enum {
  ORACLE_ROUND_NEAREST_EVEN = 0, /* AVX2 path: tfcc/mkl/vcl/tfcc_mklvcl4d.hpp:193-196 */
  ORACLE_ROUND_HALF_AWAY = 1,    /* scalar path: tfcc/mkl/kernel/tfcc_mklquantizationkernel.hpp:53-62 */
};

/*
 * Integer type descriptor: lowest and highest value of the integer type as int64
 * (uint8: 0,255; int8: -128,127; int32: INT32_MIN, INT32_MAX ...).
 */

/*
 * One requantize step: tfcc/mkl/kernel/tfcc_mklquantizationkernel.hpp:46-64 (scalar),
 * tfcc/mkl/kernel/tfcc_mklquantizationkernel.avx256.cpp:120-145 (AVX2).
 *   real = inMin + (double(x) - inLowest) * inScale        (fused when fma != 0)
 *   q    = (int64) round(real * outScale) - outOffset + outLowest, clamped.
 */
int64_t oracle_requantize_one(int64_t x, int64_t inLowest, double inScale, double inMin,
                              double outScale, int64_t outOffset, int64_t outLowest,
                              int64_t outHighest, int rounding, int fma);

/*
 * Whole-tensor requantize int32 -> uint8 including the degenerate-range branches of
 * tfcc/mkl/interfaces/tfcc_mklquantizationinterface.cpp:72-147.
 */
void oracle_requantize_s32_u8(const int32_t* a, uint64_t total, float minIn, float maxIn,
                              float minOut, float maxOut, int rounding, int fma, uint8_t* out);
/* int8 -> uint16, the shape of the reference's known-answer test (tfcc/test/quantization.cpp:88-101) */
void oracle_requantize_s8_u16(const int8_t* a, uint64_t total, float minIn, float maxIn,
                              float minOut, float maxOut, int rounding, int fma, uint16_t* out);

/*
 * dequantize: tfcc/mkl/interfaces/tfcc_mklquantizationinterface.cpp:284-333,
 * kernels tfcc/mkl/kernel/tfcc_mklquantizationkernel.hpp:35-43, ...avx256.cpp:98-118.
 *   out = (float)(min + (double(x) - lowest) * scale)     (fused when fma != 0)
 */
void oracle_dequantize_s8(const int8_t* a, uint64_t total, float minV, float maxV, int fma, float* out);
void oracle_dequantize_u8(const uint8_t* a, uint64_t total, float minV, float maxV, int fma, float* out);
void oracle_dequantize_s32(const int32_t* a, uint64_t total, float minV, float maxV, int fma, float* out);

/*
 * quantize with a given range: tfcc/mkl/interfaces/tfcc_mklquantizationinterface.cpp:191-240,
 * kernels tfcc/mkl/kernel/tfcc_mklquantizationkernel.hpp:25-33, ...avx256.cpp:55-96.
 */
void oracle_quantize_u8(const float* a, uint64_t total, float minV, float maxV, int rounding, uint8_t* out);
void oracle_quantize_s8(const float* a, uint64_t total, float minV, float maxV, int rounding, int8_t* out);

/*
 * Per-output-channel dequantize of int32 accumulators (no counterpart in the reference, which
 * only has per-tensor scales): out[i][j] = (float)((double)acc[i][j] * ((double)scaleA * (double)scaleB[j])).
 */
void oracle_dequant_per_channel(const int32_t* acc, unsigned m, unsigned n, float scaleA,
                                const float* scaleB, float* out);

/* ---- the element-wise neighbours of matmul in one BERT encoder layer ------------ */

/* softmax over the last axis. tfcc/mkl/kernel/tfcc_mklactivationkernel.hpp:112-155. */
void oracle_softmax_lastaxis(const float* a, uint64_t rows, unsigned cols, float* out);
/* layer normalisation over the last axis: tfcc/mkl/interfaces/tfcc_mklnormalizationinterface.cpp:29-62 */
void oracle_layer_norm(const float* a, const float* gamma, const float* beta, float epsilon,
                       uint64_t rows, unsigned cols, float* out);
/* 0.5*v*(1+erf(v/sqrt 2)): tfcc/mkl/kernel/tfcc_mklactivationkernel.hpp:213-220 */
void oracle_gelu_accurate(const float* a, uint64_t total, float* out);

/* ---- recurrent cells and the LSTM sequence that calls matmul once per time step -- */

/* tfcc/mkl/kernel/tfcc_mklcellkernel.hpp:51-87 (gate order i, c, f, o; sigmoid :45-48) */
void oracle_lstm_cell(unsigned batch, unsigned units, const float* stateC, const float* inputValue,
                      const float* stateHValue, const float* bias, float forget, float* h, float* cs);
/* tfcc/mkl/kernel/tfcc_mklcellkernel.hpp:89-133 */
void oracle_gru_cell_gates(unsigned batch, unsigned units, unsigned inputSize, const float* state,
                           const float* inputs, const float* value, const float* bias, float* result);
/* tfcc/mkl/kernel/tfcc_mklcellkernel.hpp:135-158 */
void oracle_gru_cell_candidate(unsigned batch, unsigned units, const float* state, const float* value,
                               const float* bias, const float* cValue, const float* cBias, float* result);
/* tfcc/mkl/kernel/tfcc_mklcellkernel.hpp:160-189 */
void oracle_pytorch_gru_cell(unsigned batch, unsigned units, const float* state, const float* inputValue,
                             const float* stateValue, const float* gateBias, const float* candidateIBias,
                             const float* candidateHBias, float* result);
/*
 * Timing aids of the benchmark's CPU leg (not part of any parity check): the OpenMP thread count of this process,
 * and C = A * B (+ bias) in fp32 with rows dealt to the threads - what a plain port of the reference's fp32 path
 * (tfcc_mklblasinterface.cpp:41-118) costs without oneDNN.  Checked against oracle_sgemm_strided_batched to fp32
 * tolerance only.
 */
void oracle_set_num_threads(int threads);
int oracle_max_threads(void);
void oracle_sgemm_f32_timing(const float* a, const float* b, const float* bias, float* c, unsigned m, unsigned n,
                             unsigned k);

/*
 * tfcc::rnn::lstm_forward / lstm_backward, tfcc/core/operations/tfcc_rnn.cpp:29-81, 83-135:
 * a [seq, batch, length], inputKernel [length, 4 hidden], stateKernel [hidden, 4 hidden], bias [4 hidden],
 * ih / ic [batch, hidden]; per step matmul(x_t, inputKernel), matmul(h, stateKernel), LSTM cell with forget 0.
 * backward != 0 walks the steps from the last to the first; outputs are stored in the order they are produced
 * (:127-133 concatenates them in that order).  out [seq, batch, hidden], h and c [batch, hidden].
 * The two products accumulate in double (the reference's sgemm is oneDNN's; see oracle_sgemm_strided_batched).
 */
void oracle_lstm_sequence(int backward, unsigned seq, unsigned batch, unsigned length, unsigned hidden,
                          const float* a, const float* inputKernel, const float* stateKernel, const float* bias,
                          const float* ih, const float* ic, float* out, float* h, float* c);

#ifdef __cplusplus
}
#endif
#endif
