/*
 * tfcc_rocm.h -- C ABI of the MI355X (gfx950) matmul backend for TFCC.
 *
 * This is the only boundary between the host side (the C++ TFCC device/interface layer, or any
 * FFI: ctypes, cgo, JNI) and the hand-written HIP kernels in libtfcc_rocm.so.  Plain pointers and
 * sizes only.  All tensor pointers are DEVICE pointers to row-major, contiguous data unless a
 * parameter says "host".  `stream` is a hipStream_t passed as void* (NULL = the default stream);
 * every compute entry point only enqueues work on it and returns.
 *
 * Return value: 0 on success, otherwise a TFCC_ROCM_* code; tfcc_rocm_last_error_string() gives
 * the text of the last failure on the calling thread.
 *
 * Each entry point names the reference function (file:line under the reference root) it replaces.
 */
#ifndef TFCC_ROCM_H_
#define TFCC_ROCM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  TFCC_ROCM_OK = 0,
  TFCC_ROCM_INVALID_ARGUMENT = 1, /* bad pointer / size / type code: nothing was launched */
  TFCC_ROCM_HIP_ERROR = 2,        /* a HIP runtime call failed */
  TFCC_ROCM_OUT_OF_MEMORY = 3,    /* device allocation failed */
  TFCC_ROCM_NO_DEVICE = 4,        /* no usable GPU */
};

/* element type codes for the type-generic quantization entry points */
enum {
  TFCC_ROCM_S8 = 0,
  TFCC_ROCM_U8 = 1,
  TFCC_ROCM_S16 = 2,
  TFCC_ROCM_U16 = 3,
  TFCC_ROCM_S32 = 4,
  TFCC_ROCM_U32 = 5,
  /* index types of gather and the remaining types of cast */
  TFCC_ROCM_S64 = 6,
  TFCC_ROCM_U64 = 7,
  TFCC_ROCM_F32 = 8,
  TFCC_ROCM_F64 = 9,
};

const char* tfcc_rocm_last_error_string(void);
/* "tfcc_rocm <version> gfx950" */
const char* tfcc_rocm_version(void);

/* ---------------------------------------------------------------------------------------------
 * Device, stream and memory plumbing.  Replaces what the reference's GPU device/session do with
 * the CUDA runtime: tfcc/cuda/framework/tfcc_cudadevice.cpp:30-55 (memory limit, allocator
 * hooks), tfcc/cuda/framework/tfcc_cudasession.cpp:36-63 (stream), and the copies of
 * tfcc/cuda/interfaces/tfcc_cudadatainterface.cu:62-97.
 * ------------------------------------------------------------------------------------------- */
int tfcc_rocm_device_count(int* count);
int tfcc_rocm_set_device(int device);
int tfcc_rocm_mem_info(size_t* free_bytes, size_t* total_bytes);
int tfcc_rocm_device_name(char* buf, size_t len);
int tfcc_rocm_malloc(void** ptr, size_t bytes);
int tfcc_rocm_free(void* ptr);
int tfcc_rocm_stream_create(void** stream);
int tfcc_rocm_stream_destroy(void* stream);
/* Gives back what the library keeps for `stream` on the current device: the workspace the skinny quantized product
 * allocates per stream on first use (tfcc_rocm_gemv_u8s8s32; blocks it outgrew included - they stay allocated until
 * here, because launches recorded earlier may still use them).  The stream must be idle and no graph recorded on it
 * may be replayed afterwards.  tfcc_rocm_stream_destroy does this itself; call it for streams the library did not
 * create (a framework's own) before they go away.  No counterpart in the reference (its sessions own no such state). */
int tfcc_rocm_stream_release(void* stream);
int tfcc_rocm_stream_synchronize(void* stream);
/* events on a stream, for timing (cf. tfcc::Coster around Session::sync, tfcc_runtime/framework/model.cpp:191-226) */
int tfcc_rocm_event_create(void** event);
int tfcc_rocm_event_destroy(void* event);
int tfcc_rocm_event_record(void* event, void* stream);
int tfcc_rocm_event_elapsed_ms(void* start_event, void* stop_event, float* ms); /* waits for stop_event */
/* Recording of everything issued on `stream` between begin and end into an executable graph that
 * one launch replays.  Stands where the reference assembles a graph's call sequence once and then
 * calls it per run (tfcc_runtime/framework/graph.cpp:54-59,98-123). */
int tfcc_rocm_stream_begin_capture(void* stream);
int tfcc_rocm_stream_end_capture(void* stream, void** graph_exec);
int tfcc_rocm_graph_launch(void* graph_exec, void* stream);
int tfcc_rocm_graph_destroy(void* graph_exec);
/* host<->device copies: synchronise the stream, then copy synchronously (reference semantics) */
int tfcc_rocm_memcpy_h2d(void* stream, void* dst_device, const void* src_host, size_t bytes);
int tfcc_rocm_memcpy_d2h(void* stream, void* dst_host, const void* src_device, size_t bytes);
int tfcc_rocm_memcpy_d2d_async(void* stream, void* dst, const void* src, size_t bytes);
/* fill `count` elements of `elem_size` (1, 2, 4 or 8) bytes with the bit pattern `value` */
int tfcc_rocm_fill_async(void* stream, void* dst, uint64_t value, int elem_size, size_t count);

/* ---------------------------------------------------------------------------------------------
 * fp32 matmul.
 * Replaces _call_matmul_wrapper / _call_matmul_with_beta_wrapper + _mkl_set_bias_wrapper,
 * tfcc/mkl/interfaces/tfcc_mklblasinterface.cpp:41-67, 69-78, 87-118 (same argument meaning:
 * batch strides in elements, 0 = operand shared by every batch; bias[n] or NULL).
 *   C[b] (m x n) = A[b] (m x k) * B[b] (k x n) (+ bias broadcast over rows)
 * ------------------------------------------------------------------------------------------- */
int tfcc_rocm_sgemm_strided_batched(void* stream, const float* a, uint64_t stride_a,
                                    const float* b, uint64_t stride_b, const float* bias, float* c,
                                    uint64_t stride_c, unsigned m, unsigned n, unsigned k,
                                    unsigned batch);

/* The same product with more of the caller's next steps done in the tile store: after the bias,
 * `residual` (optional; laid out like c, batch stride stride_residual) is added, then `activation`
 * is applied (0 none, 1 erf-form GELU, tfcc/mkl/kernel/tfcc_mklactivationkernel.hpp:213-220).  Each
 * step rounds to fp32 exactly as the separate operations would, so fusing changes no bit.  Stands
 * where the reference's runtime calls matmul, then add / gelu as separate operations
 * (tfcc_runtime/operations/math/matmulwithbias.cpp:29-40, add.cpp:27-37, gelu.cpp:27-36). */
int tfcc_rocm_sgemm_fused(void* stream, const float* a, uint64_t stride_a, const float* b,
                          uint64_t stride_b, const float* bias, const float* residual,
                          uint64_t stride_residual, float* c, uint64_t stride_c, unsigned m,
                          unsigned n, unsigned k, unsigned batch, int activation);

/* The general form: operands with their own row strides, a batch that is a grid of outer x inner
 * entries with a stride each, and B optionally given transposed.  It lets a caller multiply
 * permuted views of its tensors in place - e.g. the per-head matrices of a [batch, seq, heads, size]
 * tensor (outer = batch, inner = heads, row stride heads * size), K^T taken straight from K
 * (trans_b), a result written in [batch, seq, heads, size] order - where the reference materialises
 * each permutation first with base::transpose (tfcc/core/operations/tfcc_base.cpp:124-134) because
 * its matmul has no stride or transpose arguments (tfcc/core/operations/tfcc_blas.cpp:26-58).
 * All strides are in elements.  A residual requires a dense result (ldc == n, batch entries back to back). */
typedef struct tfcc_rocm_sgemm_desc {
  const float* a;        /* [m, k], row stride lda */
  const float* b;        /* [k, n], row stride ldb; with trans_b: [n, k], row stride ldb */
  const float* bias;     /* [n] or NULL */
  const float* residual; /* dense [batch][m, n] or NULL */
  float* c;              /* [m, n], row stride ldc */
  unsigned m, n, k;
  unsigned lda, ldb, ldc;
  int trans_b;
  unsigned batch_outer, batch_inner;
  uint64_t stride_a, stride_b, stride_c;                   /* between outer batch entries; 0 = shared */
  uint64_t inner_stride_a, inner_stride_b, inner_stride_c; /* between inner batch entries */
  uint64_t stride_residual;
  int activation;        /* 0 none, 1 erf-form GELU */
} tfcc_rocm_sgemm_desc;
int tfcc_rocm_sgemm_general(void* stream, const tfcc_rocm_sgemm_desc* desc);


/* Up to four products a * b[g] (+ bias[g]) -> c[g] that share a dense [m, k] operand a and have equal
 * shapes ([k, n] each, dense), in one launch: e.g. the query / key / value projections of an attention
 * block, which the reference issues as three matmul calls on the same input
 * (tfcc_runtime/operations/math/matmulwithbias.cpp:29-40 per node).  b, bias (may be NULL) and c are
 * host arrays of `groups` device pointers.  Every product is computed exactly as by a launch of its own. */
int tfcc_rocm_sgemm_grouped(void* stream, const float* a, const float* const* b, const float* const* bias,
                            float* const* c, unsigned groups, unsigned m, unsigned n, unsigned k);

/* ---------------------------------------------------------------------------------------------
 * Quantized uint8 x int8 -> int32 matmul.
 * Replaces _mkl_create_offset_matrix + _MKLQuantizationMatmulAVX256::quantizedMatmulColMajor,
 * tfcc/mkl/operations/tfcc_mklquantization.cpp:33-69,176-201 and
 * tfcc/mkl/kernel/tfcc_mklquantizationmatmul.avx256.h:27-29:
 *   C[b][i][j] = k*oA*oB + rowsum_a[b][i]*oB + colsum_b[b][j]*oA + sum_p A[b][i][p]*B[b][p][j]
 * in wrap-around int32.  rowsum_a / colsum_b are the caller's tensors (as in the reference they
 * are used as given); strides in elements, 0 = shared by all batches.
 * ------------------------------------------------------------------------------------------- */
typedef struct tfcc_rocm_qgemm_desc {
  const uint8_t* a;        /* [batch] m x k */
  const int8_t* b;         /* [batch] k x n */
  const int32_t* rowsum_a; /* [batch] m */
  const int32_t* colsum_b; /* [batch] n */
  uint64_t stride_a, stride_b, stride_rowsum_a, stride_colsum_b, stride_c;
  unsigned m, n, k, batch;
  /* Offsets: either immediate ... */
  int32_t offset_a, offset_b;
  /* ... or derived on the device from float ranges in device memory (all four non-NULL), exactly
   * as tfcc/mkl/operations/tfcc_mklquantization.cpp:181-186 does; then min_c / max_c (device,
   * may be NULL) receive the int32 result's range (tfcc/core/utils/tfcc_quantizationutils.h:30-43). */
  const float *min_a, *max_a, *min_b, *max_b;
  float *min_c, *max_c;
  /* Optional: b as packed once by tfcc_rocm_gemv_pack_b (weights).  A product of at most 8 rows
   * (batch == 1) then streams the packed copy; every other shape reads b. */
  const void* packed_b;
  /* Optional promise: colsum_b holds the true column sums of b (it came from tfcc_rocm_reduce_sum_cols
   * on this b).  The kernel needs the true sums on top of colsum_b as given (it feeds a - 128 to the
   * signed matrix cores) and otherwise accumulates them itself; with the promise it skips that.  The
   * result is the same whenever the promise holds. */
  int colsum_b_is_exact;
} tfcc_rocm_qgemm_desc;

/* int32 result only */
int tfcc_rocm_gemm_u8s8s32(void* stream, const tfcc_rocm_qgemm_desc* desc, int32_t* c);

/*
 * Same product with the requantize step fused into the tile store: replaces the separate pass
 * _MKLRequantizationKernelAVX256<int32_t, uint8_t>::requantize
 * (tfcc/mkl/kernel/tfcc_mklquantizationkernel.avx256.cpp:120-145; fused multiply-add and
 * round-to-nearest-even as that kernel is built).  acc_out may be NULL (int32 not written).
 * Scalars as _requantize_helper computes them (tfcc/mkl/interfaces/tfcc_mklquantizationinterface.cpp:125-130):
 *   in_scale, in_min = get_dequantized_scale_info<int32_t>(minC, maxC)
 *   out_scale, out_offset = get_quantized_scale_info<uint8_t>(minOut, maxOut)
 * If min_out / max_out (device pointers) are both non-NULL the four scalars are instead derived
 * on the device from the result range and *min_out / *max_out; this form needs the desc's float
 * ranges.  Degenerate ranges follow tfcc_mklquantizationinterface.cpp:121-139.
 */
int tfcc_rocm_gemm_u8s8s32_requant_u8(void* stream, const tfcc_rocm_qgemm_desc* desc,
                                      int32_t* acc_out, uint8_t* q_out, double in_scale,
                                      double in_min, double out_scale, int64_t out_offset,
                                      const float* min_out, const float* max_out);

/*
 * Skinny (m <= 8) product for decode shapes, HBM-bandwidth bound; single B shared by the batch of
 * rows (batch folded into m as tfcc_mklquantization.cpp:140-145 does).  Same int32 arithmetic as
 * above; the reference has no dedicated kernel for this shape (it takes the general path).
 * Optional fused per-output-channel dequantize (no counterpart in the reference, which only has
 * per-tensor ranges): f32_out[i][j] = (float)((double)acc[i][j] * ((double)scale_a * (double)scale_b[j])).
 * acc_out and f32_out may each be NULL, not both.
 */
int tfcc_rocm_gemv_u8s8s32(void* stream, const uint8_t* a, const int8_t* b,
                           const int32_t* rowsum_a, const int32_t* colsum_b, int32_t offset_a,
                           int32_t offset_b, unsigned m, unsigned n, unsigned k, int32_t* acc_out,
                           float scale_a, const float* scale_b, float* f32_out);

/* The same product with the caller's promises about its operands (flags, 0 = none: tfcc_rocm_gemv_u8s8s32).
 * TFCC_ROCM_GEMV_COLSUM_B_IS_EXACT: colsum_b holds the true column sums of b (e.g. it was made by
 * tfcc_rocm_reduce_sum_cols from this b, as a weight matrix prepared once has it).  The reference takes the sums as the
 * caller gives them (tfcc/mkl/operations/tfcc_mklquantization.cpp:33-69) and so does this library; what the promise
 * spares is the kernel's own column sums, which it needs in addition to turn its uint8 operand into int8.  With a
 * colsum_b that does not hold the true sums and this flag set, the result is wrong. */
enum { TFCC_ROCM_GEMV_COLSUM_B_IS_EXACT = 1 };
int tfcc_rocm_gemv_u8s8s32_flags(void* stream, const uint8_t* a, const int8_t* b,
                                 const int32_t* rowsum_a, const int32_t* colsum_b, int32_t offset_a,
                                 int32_t offset_b, unsigned m, unsigned n, unsigned k, int32_t* acc_out,
                                 float scale_a, const float* scale_b, float* f32_out, unsigned flags);

/* The same product through an entry point that allocates nothing.  No counterpart in the reference; it is for
 * callers that cannot allocate device memory at the point of the call: code under HIP graph capture, tight serving
 * loops, harnesses that forbid it.  tfcc_rocm_gemv_u8s8s32 keeps the workspace of its K-split kernel in memory it
 * allocates on first use (one per device and stream); this one uses a fixed array inside the library's image, one per
 * GPU (1 MiB x 2: 32768 columns x 8 rows of 64-bit words), and therefore
 *   - takes n <= 32768 on the K-split kernel where that applies (n % 16 == 0, b aligned to 16 bytes, at least 512 steps
 *     of 64 rows x 256 columns); wider products and smaller ones run on the kernel that owns its columns over the whole
 *     of K and needs no workspace (slower on a decode-sized b); what neither kernel takes fails with
 *     TFCC_ROCM_INVALID_ARGUMENT (n * k beyond 2^31, m > 8, unaligned a: not routed to the general kernel);
 *   - must not overlap with another call of itself on the same GPU (two streams): both would add into the same
 *     workspace.  Calls on one stream are ordered and leave the workspace zeroed for the next one.
 * Same arguments and results as tfcc_rocm_gemv_u8s8s32. */
int tfcc_rocm_gemv_u8s8s32_noalloc(void* stream, const uint8_t* a, const int8_t* b,
                                   const int32_t* rowsum_a, const int32_t* colsum_b, int32_t offset_a,
                                   int32_t offset_b, unsigned m, unsigned n, unsigned k, int32_t* acc_out,
                                   float scale_a, const float* scale_b, float* f32_out);

/* The same product on a B that was packed once (weights): column slabs of 16, each K x 16 bytes
 * contiguous and already in matrix-core operand order, so that a decode step streams B at the rate
 * of a plain contiguous read.  The reference re-packs its B operand on every call
 * (tfcc/mkl/gemm/tfcc_mklinputpackermanager.h:34-47) and keeps constants per device
 * (tfcc/core/framework/tfcc_constant.cpp:69-76); packing once per constant is the GPU counterpart.
 * tfcc_rocm_gemv_packed_size gives the byte size of the packed buffer (device memory, 16-byte aligned). */
size_t tfcc_rocm_gemv_packed_size(unsigned n, unsigned k);
int tfcc_rocm_gemv_pack_b(void* stream, const int8_t* b, unsigned n, unsigned k, void* packed);
int tfcc_rocm_gemv_u8s8s32_packed(void* stream, const uint8_t* a, const void* packed_b,
                                  const int32_t* rowsum_a, const int32_t* colsum_b, int32_t offset_a,
                                  int32_t offset_b, unsigned m, unsigned n, unsigned k, int32_t* acc_out,
                                  float scale_a, const float* scale_b, float* f32_out);

/*
 * Row sums (out [batch][row]) and column sums (out [batch][col]) in int32.
 * Replaces _mkl_reduce_sum_row / _mkl_reduce_sum_column,
 * tfcc/mkl/operations/tfcc_mklquantization.cpp:205-237, 239-282.  type: TFCC_ROCM_S8 / U8 / S16.
 */
int tfcc_rocm_reduce_sum_rows(void* stream, const void* a, int type, unsigned batch, unsigned row,
                              unsigned col, int32_t* out);
int tfcc_rocm_reduce_sum_cols(void* stream, const void* a, int type, unsigned batch, unsigned row,
                              unsigned col, int32_t* out);

/* ---------------------------------------------------------------------------------------------
 * Range-based quantize / requantize / dequantize (per tensor).
 * Replaces _MKLRequantizationKernelAVX256::requantize, _MKLQuantizationKernelAVX256::quantize /
 * dequantize (tfcc/mkl/kernel/tfcc_mklquantizationkernel.avx256.cpp:55-145) and the range logic of
 * tfcc/mkl/interfaces/tfcc_mklquantizationinterface.cpp:47-69, 72-147, 150-240, 284-333.
 * All ranges are float scalars in DEVICE memory (as the reference passes them as tensors); the
 * scale/offset arithmetic (tfcc/core/utils/tfcc_quantizationutils.h:45-70) runs on the device in
 * double, so nothing synchronises with the host.
 * ------------------------------------------------------------------------------------------- */
int tfcc_rocm_requantize(void* stream, const void* in, int in_type, void* out, int out_type,
                         uint64_t total, const float* min_in, const float* max_in,
                         const float* min_out, const float* max_out);
int tfcc_rocm_dequantize(void* stream, const void* in, int in_type, uint64_t total,
                         const float* min_v, const float* max_v, float* out);
int tfcc_rocm_quantize(void* stream, const float* in, uint64_t total, const float* min_v,
                       const float* max_v, void* out, int out_type);
/* quantize with the range taken from the data: writes *min_v / *max_v (device) first */
int tfcc_rocm_quantize_minmax(void* stream, const float* in, uint64_t total, void* out,
                              int out_type, float* min_v, float* max_v);

/* ---------------------------------------------------------------------------------------------
 * The element-wise neighbours of matmul inside one transformer encoder layer (fp32).
 * ------------------------------------------------------------------------------------------- */
/* softmax over the last axis: _MKLActivationKernel::softmaxV2, tfcc/mkl/kernel/tfcc_mklactivationkernel.hpp:137-155 */
int tfcc_rocm_softmax_f32(void* stream, const float* in, uint64_t rows, unsigned cols, float* out);
/* softmax(in / divisor) with the division done in fp32 per element first, i.e. the result of
 * `a / s` (tfcc/core/operations/tfcc_operator.cpp:78-95) followed by softmax, in one pass */
int tfcc_rocm_softmax_div_f32(void* stream, const float* in, uint64_t rows, unsigned cols, float divisor,
                              float* out);
/* out = softmax(q k^T [/ divisor]) v for every entry of an outer x inner batch grid, in one launch:
 * q is [s, d], k and v are [t, d], out is [s, d], each with a row stride and two batch strides of its
 * own (in elements), so that the per-head matrices of [batch, seq, heads, size] tensors are used where
 * they lie.  It stands for the node sequence Transpose x3 -> Matmul -> Div -> Softmax -> Matmul ->
 * Transpose that the reference's runtime runs one operation at a time
 * (tfcc_runtime/operations/math/matmul.cpp:27-41, softmax.cpp, base/transpose.cpp) and returns what
 * tfcc_rocm_sgemm_general (trans_b) + tfcc_rocm_softmax_div_f32 (or division, mask addition and softmax one after
 * the other) + tfcc_rocm_sgemm_general return: bit for bit up to t = 128 keys.  Longer key sequences (the reference's
 * path has no limit: tfcc/mkl/kernel/tfcc_mklactivationkernel.hpp:137-155 between two batched products,
 * tfcc/mkl/interfaces/tfcc_mklblasinterface.cpp:127-151) are walked in blocks of 128 keys with a running row maximum
 * and sum: the same function summed in another order, within a few units in the last place of the separate kernels
 * and inside the fp32 tolerance of the path (relative Frobenius error <= 1e-5 against double precision).
 * Limits: d <= 64 and a multiple of 4, input strides multiples of 4, inputs 16-byte
 * aligned, and not a single head (batch_outer * batch_inner == 1) of s <= 8 rows, whose separate product
 * runs on the streaming kernel for short A and sums in another order;
 * tfcc_rocm_attention_f32_supported() tells (1 / 0) whether a descriptor is within them.
 * out must not overlap the inputs. */
typedef struct tfcc_rocm_attention_desc {
  const float* q;
  const float* k;
  const float* v;
  float* out;
  unsigned s, t, d;
  unsigned ldq, ldk, ldv, ldo;
  unsigned batch_outer, batch_inner;
  uint64_t stride_q, stride_k, stride_v, stride_out;                         /* between outer entries */
  uint64_t inner_stride_q, inner_stride_k, inner_stride_v, inner_stride_out; /* between inner entries */
  float divisor;
  int has_divisor; /* 0: plain softmax(q k^T) */
  /* optional (NULL: none): t values per batch entry added to every row of the divided scores before the softmax, as
   * the Add of an attention mask [batch, 1, 1, t] between Div and Softmax does; batch strides in elements (0 where
   * the mask is shared) */
  const float* mask;
  uint64_t stride_mask, inner_stride_mask;
} tfcc_rocm_attention_desc;
int tfcc_rocm_attention_f32_supported(const tfcc_rocm_attention_desc* desc);
int tfcc_rocm_attention_f32(void* stream, const tfcc_rocm_attention_desc* desc);
/* _mkl_layer_normalize, tfcc/mkl/interfaces/tfcc_mklnormalizationinterface.cpp:29-62 */
int tfcc_rocm_layer_norm_f32(void* stream, const float* in, const float* gamma, const float* beta,
                             float epsilon, uint64_t rows, unsigned cols, float* out);
/* Element-wise functions of one tensor with the expressions of the reference's float kernels
 * (tfcc/mkl/kernel/tfcc_mklactivationkernel.hpp:48-110,222-228,284-291): sigmoid 1/(1+exp(0-x)), tanh, relu,
 * softplus log(exp(x)+1), log, rsqrt 1/sqrt(x), erf, abs, sign; and neg 0-x, reciprocal 1/x, sqrt 1/rsqrt(x) as
 * tfcc_runtime/operations/math/neg.cpp:30, reciprocal.cpp:31, sqrt.cpp:31 compose them. */
enum {
  TFCC_ROCM_UNARY_SIGMOID = 0, TFCC_ROCM_UNARY_TANH = 1, TFCC_ROCM_UNARY_RELU = 2, TFCC_ROCM_UNARY_SOFTPLUS = 3,
  TFCC_ROCM_UNARY_LOG = 4, TFCC_ROCM_UNARY_RSQRT = 5, TFCC_ROCM_UNARY_ERF = 6, TFCC_ROCM_UNARY_ABS = 7,
  TFCC_ROCM_UNARY_SIGN = 8, TFCC_ROCM_UNARY_NEG = 9, TFCC_ROCM_UNARY_RECIPROCAL = 10, TFCC_ROCM_UNARY_SQRT = 11
};
int tfcc_rocm_unary_f32(void* stream, int op, const float* in, uint64_t total, float* out);
/* _MKLActivationKernel::geluAccurate, tfcc/mkl/kernel/tfcc_mklactivationkernel.hpp:213-220: 0.5 x (1 + erf(x / sqrt 2)).
 * erf is evaluated through a polynomial fit of log2 erfc (the reference calls the C library's erff): results differ
 * from the reference's in the last bits, by at most 1e-7 + 1e-6 |x'| of the exact value x'. */
int tfcc_rocm_gelu_accurate_f32(void* stream, const float* in, uint64_t total, float* out);
/* out = a * alpha + beta: TransformationInterface::transform, tfcc/core/operations/tfcc_operator.cpp:78-95 */
int tfcc_rocm_transform_f32(void* stream, const float* in, uint64_t total, float alpha, float beta,
                            float* out);
/* out[i] = a[i] + b[i % period] (period == total: plain add; period < total: trailing-dims
 * broadcast of b).  ArithmeticInterface::add, tfcc/core/interfaces/tfcc_arithmeticinterface.h:34-49 */
int tfcc_rocm_add_f32(void* stream, const float* a, const float* b, uint64_t total,
                      uint64_t period, float* out);
/* out = a / alpha + beta: TransformationInterface::transform2 (a / s in tfcc_operator.cpp:78-95) */
int tfcc_rocm_transform2_f32(void* stream, const float* in, uint64_t total, float alpha, float beta,
                             float* out);
/* op: 0 a + b, 1 a - b, 2 a * b, 3 a / b, 4 pow(a, b), 5 max(a, b), 6 min(a, b) with the same trailing-dims
 * broadcast of b as add: ArithmeticInterface::add/sub/mul/div, tfcc/core/interfaces/tfcc_arithmeticinterface.h:34-79;
 * tfcc::math::pow / max / min */
int tfcc_rocm_binary_f32(void* stream, int op, const float* a, const float* b, uint64_t total,
                         uint64_t period, float* out);
/* Reductions over the trailing dimensions, rows x cols -> rows (ReduceInterface::reduceSum / reduceMean / reduceProd /
 * reduceMax / reduceMin, tfcc/mkl/interfaces/tfcc_mklreduceinterface.cpp:107-230). */
enum {
  TFCC_ROCM_REDUCE_SUM = 0, TFCC_ROCM_REDUCE_MEAN = 1, TFCC_ROCM_REDUCE_PROD = 2, TFCC_ROCM_REDUCE_MAX = 3,
  TFCC_ROCM_REDUCE_MIN = 4
};
int tfcc_rocm_reduce_f32(void* stream, int op, const float* in, uint64_t rows, unsigned cols, float* out);
/* min(max(v, lo), hi) (tfcc::math::clip) and v > 0 ? v : v * alpha (tfcc::math::leaky_relu) */
int tfcc_rocm_clip_f32(void* stream, const float* in, uint64_t total, float lo, float hi, float* out);
int tfcc_rocm_leaky_relu_f32(void* stream, const float* in, uint64_t total, float alpha, float* out);
/* out[i] = condition[i] != 0 ? x[i] : y[i] on elements of element_bytes (1, 2, 4, 8) bytes; a null x (or y) stands
 * for one value, the low element_bytes of x_bits (y_bits) (tfcc/mkl/interfaces/tfcc_mklbasicinterface.cpp:398-422). */
int tfcc_rocm_where(void* stream, const uint8_t* condition, const void* x, uint64_t x_bits, const void* y,
                    uint64_t y_bits, unsigned element_bytes, uint64_t total, void* out);
/* tril (upper == 0: row r keeps columns c < r + k + 1) or triu (c >= r + k) of a [rows, cols] matrix, zeros elsewhere
 * (tfcc/mkl/interfaces/tfcc_mklbasicinterface.cpp:433-466). */
int tfcc_rocm_triangle(void* stream, const void* in, uint64_t rows, uint64_t cols, int64_t k, int upper,
                       unsigned element_bytes, void* out);
/* Comparisons with byte results (1 where the relation holds, else 0) for every element type (TFCC_ROCM_S8 .. F64).
 * compare_value: a[i] OP *value, value a host pointer to one element of the tensor's type
 * (tfcc/core/interfaces/tfcc_comparisoninterface.h:38-83).  compare: (a - b) OP 0 with numpy-style broadcasting given as
 * for tfcc_rocm_binary_broadcast_f32, the difference taken in the element type as tfcc::relation::equal and its
 * siblings do for two tensors (tfcc/core/operations/tfcc_relation.cpp:101-115): unsigned differences wrap. */
enum {
  TFCC_ROCM_COMPARE_EQUAL = 0,
  TFCC_ROCM_COMPARE_UNEQUAL = 1,
  TFCC_ROCM_COMPARE_GREATER = 2,
  TFCC_ROCM_COMPARE_GREATER_EQUAL = 3,
  TFCC_ROCM_COMPARE_LESS = 4,
  TFCC_ROCM_COMPARE_LESS_EQUAL = 5
};
int tfcc_rocm_compare_value(void* stream, int op, const void* a, int type, uint64_t total, const void* value,
                            uint8_t* out);
int tfcc_rocm_compare(void* stream, int op, const void* a, const void* b, int type, int rank, const unsigned* dims,
                      const uint64_t* stride_a, const uint64_t* stride_b, uint8_t* out);
/* out[x, z] = first position y of the largest in[x, y, z], in is [outer, length, inner]
 * (tfcc/mkl/interfaces/tfcc_mklbasicinterface.cpp:469-485, :757-776). */
int tfcc_rocm_argmax_f32(void* stream, const float* in, uint64_t outer, unsigned length, uint64_t inner, int64_t* out);
/* The k largest elements of each row of in [rows, length], descending, and their positions; equal values in ascending
 * position (tfcc/mkl/interfaces/tfcc_mklbasicinterface.cpp:159-260, :779-800 leaves their order open).  A NaN counts
 * as larger than every number (the reference's heap comparison v1.value > v2.value leaves its place undefined).
 * 1 <= k <= min(length, 1024): the selection makes one pass over the row per element, one workgroup per row. */
int tfcc_rocm_topk_f32(void* stream, const float* in, uint64_t rows, unsigned length, unsigned k, float* values,
                       uint32_t* positions);
/* out = a op b with numpy-style broadcasting: dims[rank] is the result's shape, stride_a / stride_b the element strides
 * of each operand per result dimension (0 where the operand's extent is 1).  rank <= 6; callers merge adjacent
 * dimensions of the same kind first, as tfcc::math::add does (tfcc/core/operations/tfcc_math.cpp:38-104). */
int tfcc_rocm_binary_broadcast_f32(void* stream, int op, const float* a, const float* b, int rank,
                                   const unsigned* dims, const uint64_t* stride_a, const uint64_t* stride_b, float* out);
/* rank <= 6 permutation: BasicInterface::transpose, tfcc/core/operations/tfcc_base.cpp:124-134.
 * shape / perm are HOST arrays of length rank. */
int tfcc_rocm_transpose_f32(void* stream, const float* in, const unsigned* shape,
                            const unsigned* perm, int rank, float* out);

/* ---- recurrent cells: the element-wise step after the two matrix products of a time step -------------------
 * All tensors row-major and dense; one launch each.
 *
 * CellInterface::processLSTMCell (tfcc/core/interfaces/tfcc_cellinterface.h:33-47; arithmetic of
 * _MKLCellKernel::processLSTMCell, tfcc/mkl/kernel/tfcc_mklcellkernel.hpp:51-87): state_c [batch, units],
 * input_value and state_h_value [batch, 4 * units] in gate order i, c, f, o, bias [4 * units];
 * cs = tanh(xc) * sigmoid(xi) + state_c * sigmoid(xf + forget), h = tanh(cs) * sigmoid(xo).
 * h and cs are [batch, units]; cs may be state_c itself. */
int tfcc_rocm_lstm_cell_f32(void* stream, unsigned batch, unsigned units, const float* state_c,
                            const float* input_value, const float* state_h_value, const float* bias, float forget,
                            float* h, float* cs);
/* One step of tfcc::rnn::lstm_forward / lstm_backward (tfcc/core/operations/tfcc_rnn.cpp:62-71) in one launch:
 * matmul(h_prev, state kernel) and the LSTM cell above on its sums.  batch <= 8.  The state kernel is passed with its
 * gates interleaved: element [k, 4 * u + g] = state_kernel[k, g * units + u], i.e. the [units, 4, units] view of the
 * reference's [units, 4 * units] kernel transposed with perm (0, 2, 1) (tfcc_rocm_transpose_f32 does it once per
 * sequence).  input_value and bias keep the reference's layout.  h must not be h_prev; cs may be state_c. */
int tfcc_rocm_lstm_step_f32(void* stream, unsigned batch, unsigned units, const float* h_prev,
                            const float* state_kernel_interleaved, const float* input_value, const float* bias,
                            float forget, const float* state_c, float* h, float* cs);
/* CellInterface::processGRUCellGates (tfcc_cellinterface.h:49-59; tfcc_mklcellkernel.hpp:89-133):
 * result [batch, input_size + units] = concat(inputs, sigmoid(value[:, :units] + bias[:units]) * state);
 * value [batch, 2 * units], bias [2 * units]. */
int tfcc_rocm_gru_cell_gates_f32(void* stream, unsigned batch, unsigned units, unsigned input_size,
                                 const float* state, const float* inputs, const float* value, const float* bias,
                                 float* result);
/* CellInterface::processGRUCellCandidate (tfcc_cellinterface.h:61-70; tfcc_mklcellkernel.hpp:135-158):
 * u = sigmoid(value[:, units:] + bias[units:]), c = tanh(c_value + c_bias), result = u * state + (1 - u) * c. */
int tfcc_rocm_gru_cell_candidate_f32(void* stream, unsigned batch, unsigned units, const float* state,
                                     const float* value, const float* bias, const float* c_value,
                                     const float* c_bias, float* result);
/* CellInterface::processPyTorchGRUCell (tfcc_cellinterface.h:72-86; tfcc_mklcellkernel.hpp:160-189):
 * input_value and state_value [batch, 3 * units] (r, z, n), gate_bias [2 * units];
 * n = tanh(ni + r * nh), result = n + z * (state - n). */
int tfcc_rocm_pytorch_gru_cell_f32(void* stream, unsigned batch, unsigned units, const float* state,
                                   const float* input_value, const float* state_value, const float* gate_bias,
                                   const float* candidate_i_bias, const float* candidate_h_bias, float* result);

/* ---- data movement between the products: one pass each ------------------------------------------------------------
 * rows x width bytes from src (rows src_pitch bytes apart) to dst (rows dst_pitch bytes apart).  BasicInterface::slice
 * (tfcc/mkl/interfaces/tfcc_mklbasicinterface.cpp:488-515: a [s1, s2, s3] tensor, rows = s1, src = a + start * s3,
 * width = length * s3) and concat (tfcc/core/operations/tfcc_base.cpp:86-106: one copy per value into its column
 * range of the result) are one call each per operand. */
int tfcc_rocm_copy2d(void* stream, const void* src, uint64_t src_pitch, void* dst, uint64_t dst_pitch, uint64_t rows,
                     uint64_t width);
/* GatherInterface::gather (tfcc/mkl/interfaces/tfcc_mklgatherinterface.cpp:28-66): out row i = params row indices[i]
 * (chunk_bytes each), a row of zeros where the index is outside [0, batch).  index_type: TFCC_ROCM_S32 / U32 / S64 / U64. */
int tfcc_rocm_gather_rows(void* stream, const void* params, unsigned batch, uint64_t chunk_bytes, const void* indices,
                          int index_type, uint64_t length, void* out);
/* tfcc::data::cast: out[i] = static_cast<out type>(in[i]) for any pair of the ten element types above. */
int tfcc_rocm_cast(void* stream, const void* in, int in_type, void* out, int out_type, uint64_t total);

#ifdef __cplusplus
}
#endif
#endif /* TFCC_ROCM_H_ */
