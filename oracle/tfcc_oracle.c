/*
 * CPU oracle for the TFCC matmul hot path.  TEST INFRASTRUCTURE ONLY: see tfcc_oracle.h for
 * what each function restates and how it is pinned.  Build with -ffp-contract=off so that
 * every fused multiply-add below is an explicit fma() call and nothing else is fused.
 */
#include "tfcc_oracle.h"

#include <math.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>

/* ---------------------------------------------------------------------------------------------
 * shape rules
 * ------------------------------------------------------------------------------------------- */

int oracle_matmul_plan(const unsigned* shapeA, int rankA, const unsigned* shapeB, int rankB,
                       const unsigned* shapeBias, int biasRank, unsigned* resultShape,
                       int* resultRank, unsigned* m, unsigned* n, unsigned* k, unsigned* strideA,
                       unsigned* strideB, unsigned* strideC, unsigned* batch, int* empty) {
  /* tfcc/core/operations/tfcc_blas.cpp:27-29 */
  if (rankA < 2 || rankB < 2) return ORACLE_ERR_RANK;
  /* :30-32 ranks equal, or one of them is a plain matrix */
  if (rankA != rankB && rankA != 2 && rankB != 2) return ORACLE_ERR_SHAPE;
  /* :33-35 inner dimensions */
  if (shapeA[rankA - 1] != shapeB[rankB - 2]) return ORACLE_ERR_SHAPE;
  /* :71-73 bias is a vector of length N (checked before the leading dims in the 3-operand form) */
  if (biasRank >= 0) {
    if (biasRank != 1 || shapeBias[0] != shapeB[rankB - 1]) return ORACLE_ERR_SHAPE;
  }
  /* :36-42 equal ranks: every leading dim must match exactly (no size-1 broadcast) */
  if (rankA == rankB) {
    for (int i = 0; i + 2 < rankA; ++i) {
      if (shapeA[i] != shapeB[i]) return ORACLE_ERR_SHAPE;
    }
  }
  unsigned sizeA = 1, sizeB = 1;
  for (int i = 0; i < rankA; ++i) sizeA *= shapeA[i];
  for (int i = 0; i < rankB; ++i) sizeB *= shapeB[i];

  /* result shape: tfcc_blas.cpp:44-51, tfcc_mklblasinterface.cpp:138-141 */
  const unsigned* longer = rankA > rankB ? shapeA : shapeB;
  int rank = rankA > rankB ? rankA : rankB;
  for (int i = 0; i < rank; ++i) resultShape[i] = longer[i];
  *m = shapeA[rankA - 2];
  *n = shapeB[rankB - 1];
  *k = shapeA[rankA - 1];
  resultShape[rank - 2] = *m;
  resultShape[rank - 1] = *n;
  *resultRank = rank;
  *empty = (sizeA == 0 || sizeB == 0);

  /* strides: tfcc_mklblasinterface.cpp:131-137 (unsigned arithmetic on purpose) */
  *strideA = *m * *k;
  *strideB = *n * *k;
  *strideC = *m * *n;
  if (rankA != rankB) {
    if (rankA == 2) *strideA = 0;
    if (rankB == 2) *strideB = 0;
  }
  unsigned total = 1;
  for (int i = 0; i < rank; ++i) total *= resultShape[i];
  /* :144-145 */
  *batch = (*m != 0 && *n != 0) ? total / (*m * *n) : 0;
  return ORACLE_OK;
}

/* ---------------------------------------------------------------------------------------------
 * fp32 matmul, double accumulation
 * ------------------------------------------------------------------------------------------- */

void oracle_sgemm_strided_batched(const float* a, uint64_t strideA, const float* b,
                                  uint64_t strideB, const float* bias, float* c, double* c64,
                                  uint64_t strideC, unsigned m, unsigned n, unsigned k,
                                  unsigned batch) {
  double* row = (double*)malloc(sizeof(double) * (n ? n : 1));
  for (unsigned bi = 0; bi < batch; ++bi) {
    const float* pa = a + (size_t)bi * strideA;
    const float* pb = b + (size_t)bi * strideB;
    for (unsigned i = 0; i < m; ++i) {
      for (unsigned j = 0; j < n; ++j) row[j] = 0.0;
      for (unsigned p = 0; p < k; ++p) {
        double av = (double)pa[(size_t)i * k + p];
        const float* brow = pb + (size_t)p * n;
        for (unsigned j = 0; j < n; ++j) row[j] += av * (double)brow[j];
      }
      for (unsigned j = 0; j < n; ++j) {
        /* bias is the initial content of C and the product is added to it:
         * tfcc_mklblasinterface.cpp:69-78,100-104 */
        double v = bias ? (double)bias[j] + row[j] : row[j];
        size_t idx = (size_t)bi * strideC + (size_t)i * n + j;
        if (c) c[idx] = (float)v;
        if (c64) c64[idx] = v;
      }
    }
  }
  free(row);
}

/* The timing leg of the fp32 path: the same product with fp32 accumulation, rows dealt to OpenMP threads,
 * the inner loop over a row of B left to the compiler's vectoriser (built for AVX2 where the host has it).
 * This is what a straightforward CPU port of tfcc_mklblasinterface.cpp:41-118 costs without oneDNN's
 * JIT kernels; it is measured, never compared bit for bit (its sums run in k order in fp32). */
#include <omp.h>
void oracle_set_num_threads(int threads) { if (threads > 0) omp_set_num_threads(threads); }
int oracle_max_threads(void) { return omp_get_max_threads(); }

__attribute__((target_clones("avx2,fma", "default"), optimize("O3")))
void oracle_sgemm_f32_timing(const float* a, const float* b, const float* bias, float* c, unsigned m, unsigned n,
                             unsigned k) {
#pragma omp parallel for schedule(static)
  for (unsigned i = 0; i < m; ++i) {
    float* row = c + (size_t)i * n;
    for (unsigned j = 0; j < n; ++j) row[j] = bias ? bias[j] : 0.f;
    for (unsigned p = 0; p < k; ++p) {
      const float av = a[(size_t)i * k + p];
      const float* brow = b + (size_t)p * n;
      for (unsigned j = 0; j < n; ++j) row[j] += av * brow[j];
    }
  }
}

/* ---------------------------------------------------------------------------------------------
 * quantized matmul
 * ------------------------------------------------------------------------------------------- */

#define DEFINE_REDUCE_ROW(NAME, T)                                                             \
  void NAME(const T* a, unsigned batch, unsigned row, unsigned col, int32_t* out) {            \
    for (unsigned b = 0; b < batch; ++b)                                                       \
      for (unsigned i = 0; i < row; ++i) {                                                     \
        uint32_t s = 0;                                                                        \
        const T* p = a + ((size_t)b * row + i) * col;                                          \
        for (unsigned j = 0; j < col; ++j) s += (uint32_t)(int32_t)p[j];                       \
        out[(size_t)b * row + i] = (int32_t)s;                                                 \
      }                                                                                        \
  }
#define DEFINE_REDUCE_COL(NAME, T)                                                             \
  void NAME(const T* a, unsigned batch, unsigned row, unsigned col, int32_t* out) {            \
    for (unsigned b = 0; b < batch; ++b) {                                                     \
      uint32_t* o = (uint32_t*)(out + (size_t)b * col);                                        \
      for (unsigned j = 0; j < col; ++j) o[j] = 0;                                             \
      for (unsigned i = 0; i < row; ++i) {                                                     \
        const T* p = a + ((size_t)b * row + i) * col;                                          \
        for (unsigned j = 0; j < col; ++j) o[j] += (uint32_t)(int32_t)p[j];                    \
      }                                                                                        \
    }                                                                                          \
  }
DEFINE_REDUCE_ROW(oracle_reduce_sum_row_u8, uint8_t)
DEFINE_REDUCE_ROW(oracle_reduce_sum_row_s8, int8_t)
DEFINE_REDUCE_COL(oracle_reduce_sum_col_u8, uint8_t)
DEFINE_REDUCE_COL(oracle_reduce_sum_col_s8, int8_t)

void oracle_qmatmul_offsets(float minA, float maxA, float minB, float maxB, int32_t* offsetA,
                            int32_t* offsetB) {
  double scale;
  int64_t oa, ob;
  oracle_quantized_scale_info(8, minA, maxA, &scale, &oa);
  oracle_quantized_scale_info(8, minB, maxB, &scale, &ob);
  /* offset -= lowest(T): uint8 lowest is 0, int8 lowest is -128.
   * tfcc/mkl/operations/tfcc_mklquantization.cpp:185-186 */
  oa -= 0;
  ob -= -128;
  *offsetA = (int32_t)oa;
  *offsetB = (int32_t)ob;
}

void oracle_qgemm_u8s8s32(unsigned batch, const uint8_t* a, uint64_t strideA, const int8_t* b,
                          uint64_t strideB, const int32_t* rowsumA, uint64_t strideRA,
                          const int32_t* colsumB, uint64_t strideRB, int32_t offsetA,
                          int32_t offsetB, unsigned m, unsigned n, unsigned k, int32_t* c,
                          uint64_t strideC) {
  /* all arithmetic modulo 2^32, as int32 wrap-around on the reference's x86 build */
  uint32_t oA = (uint32_t)offsetA, oB = (uint32_t)offsetB;
  uint32_t global = oA * oB * (uint32_t)k; /* tfcc_mklquantization.cpp:37 */
  uint32_t* acc = (uint32_t*)malloc(sizeof(uint32_t) * (n ? n : 1));
  for (unsigned bi = 0; bi < batch; ++bi) {
    const uint8_t* pa = a + (size_t)bi * strideA;
    const int8_t* pb = b + (size_t)bi * strideB;
    const int32_t* ra = rowsumA + (size_t)bi * strideRA;
    const int32_t* rb = colsumB + (size_t)bi * strideRB;
    for (unsigned i = 0; i < m; ++i) {
      uint32_t oa = (uint32_t)ra[i] * oB; /* :44 */
      for (unsigned j = 0; j < n; ++j) acc[j] = global + oa + (uint32_t)rb[j] * oA; /* :46-47 */
      for (unsigned p = 0; p < k; ++p) {
        int32_t av = (int32_t)pa[(size_t)i * k + p];
        const int8_t* brow = pb + (size_t)p * n;
        for (unsigned j = 0; j < n; ++j) acc[j] += (uint32_t)(av * (int32_t)brow[j]);
      }
      memcpy(c + (size_t)bi * strideC + (size_t)i * n, acc, sizeof(uint32_t) * n);
    }
  }
  free(acc);
}

static float level_of(float rangeMin, float rangeMax, int64_t lowest, int64_t highest) {
  /* tfcc_quantizationutils.h:23-28: float / int64 -> float division */
  return (rangeMax - rangeMin) / (float)(highest - lowest);
}

void oracle_qmatmul_range(float minA, float maxA, float minB, float maxB, float* minC,
                          float* maxC) {
  float aLevel = level_of(minA, maxA, 0, 255);
  float bLevel = level_of(minB, maxB, -128, 127);
  float cLevel = aLevel * bLevel;
  /* tfcc_quantizationutils.h:40-41: float * int64 is evaluated in float */
  *minC = cLevel * (float)(int64_t)INT32_MIN;
  *maxC = cLevel * (float)(int64_t)INT32_MAX;
}

/* ---------------------------------------------------------------------------------------------
 * range arithmetic
 * ------------------------------------------------------------------------------------------- */

void oracle_quantized_scale_info(int bits, float minValue, float maxValue, double* scale,
                                 int64_t* offset) {
  int64_t stepCnt = (int64_t)1 << bits;
  double rangeAdjust = (double)stepCnt / ((double)stepCnt - 1.0);
  /* (maxValue - minValue) is a float subtraction, then promoted: tfcc_quantizationutils.h:51 */
  float span = maxValue - minValue;
  double range = (double)span * rangeAdjust;
  double rangeScale = (double)stepCnt / range;
  *scale = rangeScale;
  /* round(): half away from zero, in double: :53 */
  *offset = (int64_t)round((double)minValue * rangeScale);
}

void oracle_dequantized_scale_info(int bits, float minValue, float maxValue, double* scale,
                                   double* minRounded) {
  int64_t stepCnt = (int64_t)1 << bits;
  double rangeAdjust = (double)stepCnt / ((double)stepCnt - 1.0);
  float span = maxValue - minValue;
  double range = (double)span * rangeAdjust;
  *scale = range / (double)stepCnt;
  *minRounded = (double)minValue; /* :66-67: the rounding line is commented out */
}

static double round_mode(double v, int rounding) {
  return rounding == ORACLE_ROUND_HALF_AWAY ? round(v) : nearbyint(v); /* default FE_TONEAREST = ties-to-even */
}

static int64_t clamp64(int64_t v, int64_t lo, int64_t hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* (int64) conversion of a double that may be out of range.  On x86-64 cvttsd2si returns
 * INT64_MIN ("integer indefinite") for NaN and for anything outside int64. */
static int64_t to_int64_x86(double v) {
  if (!(v > -9223372036854775808.0 && v < 9223372036854775808.0)) return INT64_MIN;
  return (int64_t)v;
}

int64_t oracle_requantize_one(int64_t x, int64_t inLowest, double inScale, double inMin,
                              double outScale, int64_t outOffset, int64_t outLowest,
                              int64_t outHighest, int rounding, int use_fma) {
  double off = (double)x - (double)inLowest;
  double real = use_fma ? fma(off, inScale, inMin) : inMin + off * inScale;
  int64_t q = to_int64_x86(round_mode(real * outScale, rounding));
  /* wrap-around like the reference's int64 arithmetic */
  q = (int64_t)((uint64_t)q - (uint64_t)outOffset + (uint64_t)outLowest);
  return clamp64(q, outLowest, outHighest);
}

#define DEFINE_REQUANTIZE(NAME, TI, IN_BITS, IN_LOWEST, TO, OUT_BITS, OUT_LOWEST, OUT_HIGHEST)      \
  void NAME(const TI* a, uint64_t total, float minIn, float maxIn, float minOut, float maxOut,     \
            int rounding, int use_fma, TO* out) {                                                  \
    /* tfcc_mklquantizationinterface.cpp:121-124 */                                                \
    if (minOut >= maxOut) {                                                                        \
      for (uint64_t i = 0; i < total; ++i) out[i] = (TO)(OUT_LOWEST);                              \
      return;                                                                                      \
    }                                                                                              \
    double inScale, inMin, outScale;                                                               \
    int64_t outOffset;                                                                             \
    oracle_dequantized_scale_info(IN_BITS, minIn, maxIn, &inScale, &inMin);                        \
    oracle_quantized_scale_info(OUT_BITS, minOut, maxOut, &outScale, &outOffset);                  \
    /* :132-139 constant input: always C round() here, whatever the kernel's rounding */           \
    if (minIn >= maxIn) {                                                                          \
      int64_t q = to_int64_x86(round((double)minIn * outScale));                                   \
      q = (int64_t)((uint64_t)q - (uint64_t)outOffset + (uint64_t)(int64_t)(OUT_LOWEST));          \
      q = clamp64(q, (OUT_LOWEST), (OUT_HIGHEST));                                                 \
      for (uint64_t i = 0; i < total; ++i) out[i] = (TO)q;                                         \
      return;                                                                                      \
    }                                                                                              \
    for (uint64_t i = 0; i < total; ++i)                                                           \
      out[i] = (TO)oracle_requantize_one((int64_t)a[i], (IN_LOWEST), inScale, inMin, outScale,     \
                                         outOffset, (OUT_LOWEST), (OUT_HIGHEST), rounding,         \
                                         use_fma);                                                 \
  }
DEFINE_REQUANTIZE(oracle_requantize_s32_u8, int32_t, 32, (int64_t)INT32_MIN, uint8_t, 8, 0, 255)
DEFINE_REQUANTIZE(oracle_requantize_s8_u16, int8_t, 8, -128, uint16_t, 16, 0, 65535)

#define DEFINE_DEQUANTIZE(NAME, T, BITS, LOWEST)                                                    \
  void NAME(const T* a, uint64_t total, float minV, float maxV, int use_fma, float* out) {         \
    /* tfcc_mklquantizationinterface.cpp:321-324 */                                                \
    if (minV >= maxV) {                                                                            \
      for (uint64_t i = 0; i < total; ++i) out[i] = minV;                                          \
      return;                                                                                      \
    }                                                                                              \
    double scale, minRounded;                                                                      \
    oracle_dequantized_scale_info(BITS, minV, maxV, &scale, &minRounded);                          \
    for (uint64_t i = 0; i < total; ++i) {                                                         \
      double off = (double)a[i] - (double)(LOWEST);                                                \
      out[i] = (float)(use_fma ? fma(off, scale, minRounded) : minRounded + off * scale);          \
    }                                                                                              \
  }
DEFINE_DEQUANTIZE(oracle_dequantize_s8, int8_t, 8, -128)
DEFINE_DEQUANTIZE(oracle_dequantize_u8, uint8_t, 8, 0)
DEFINE_DEQUANTIZE(oracle_dequantize_s32, int32_t, 32, (int64_t)INT32_MIN)

#define DEFINE_QUANTIZE(NAME, T, LOWEST, HIGHEST)                                                   \
  void NAME(const float* a, uint64_t total, float minV, float maxV, int rounding, T* out) {        \
    /* tfcc_mklquantizationinterface.cpp:229-232 */                                                \
    if (minV >= maxV) {                                                                            \
      for (uint64_t i = 0; i < total; ++i) out[i] = (T)(LOWEST);                                   \
      return;                                                                                      \
    }                                                                                              \
    double scale;                                                                                  \
    int64_t offset;                                                                                \
    oracle_quantized_scale_info(8, minV, maxV, &scale, &offset);                                   \
    for (uint64_t i = 0; i < total; ++i) {                                                         \
      int64_t q = to_int64_x86(round_mode((double)a[i] * scale, rounding));                        \
      q = (int64_t)((uint64_t)q - (uint64_t)offset + (uint64_t)(int64_t)(LOWEST));                 \
      out[i] = (T)clamp64(q, (LOWEST), (HIGHEST));                                                 \
    }                                                                                              \
  }
DEFINE_QUANTIZE(oracle_quantize_u8, uint8_t, 0, 255)
DEFINE_QUANTIZE(oracle_quantize_s8, int8_t, -128, 127)

void oracle_dequant_per_channel(const int32_t* acc, unsigned m, unsigned n, float scaleA,
                                const float* scaleB, float* out) {
  for (unsigned i = 0; i < m; ++i)
    for (unsigned j = 0; j < n; ++j)
      out[(size_t)i * n + j] =
          (float)((double)acc[(size_t)i * n + j] * ((double)scaleA * (double)scaleB[j]));
}

/* ---------------------------------------------------------------------------------------------
 * element-wise neighbours (fp32 like the reference's template instantiation for float)
 * ------------------------------------------------------------------------------------------- */

void oracle_softmax_lastaxis(const float* a, uint64_t rows, unsigned cols, float* out) {
  for (uint64_t r = 0; r < rows; ++r) {
    const float* ra = a + r * cols;
    float* rb = out + r * cols;
    float mx = -3.402823466e+38f;
    for (unsigned y = 0; y < cols; ++y) mx = ra[y] > mx ? ra[y] : mx;
    /* exp() is the double overload applied to a float argument, result narrowed */
    for (unsigned y = 0; y < cols; ++y) rb[y] = (float)exp((double)(ra[y] - mx));
    float s = 0.f;
    for (unsigned y = 0; y < cols; ++y) s += rb[y];
    for (unsigned y = 0; y < cols; ++y) rb[y] /= s;
  }
}

void oracle_layer_norm(const float* a, const float* gamma, const float* beta, float epsilon,
                       uint64_t rows, unsigned cols, float* out) {
  for (uint64_t r = 0; r < rows; ++r) {
    const float* in = a + r * cols;
    float* o = out + r * cols;
    float mean = 0.f;
    for (unsigned j = 0; j < cols; ++j) mean += in[j];
    mean /= (float)cols;
    float var = 0.f;
    for (unsigned j = 0; j < cols; ++j) {
      float t = in[j] - mean;
      var += t * t;
    }
    var /= (float)cols;
    float inv = 1.0f / sqrtf(var + epsilon);
    for (unsigned j = 0; j < cols; ++j) {
      float x = inv * gamma[j];
      o[j] = (in[j] - mean) * x + beta[j];
    }
  }
}

void oracle_gelu_accurate(const float* a, uint64_t total, float* out) {
  for (uint64_t i = 0; i < total; ++i) {
    float v = a[i];
    /* 0.5 and 1 are double/int literals: the product is formed in double, erf in float */
    out[i] = (float)(0.5 * (double)v * (double)(1 + erff(v / 1.4142135623730951f)));
  }
}

/* ---- recurrent cells ------------------------------------------------------------------------- */

static float oracle_sigmoid(float v) { return 1.f / (1.f + expf(0.f - v)); }

void oracle_lstm_cell(unsigned batch, unsigned units, const float* stateC, const float* inputValue,
                      const float* stateHValue, const float* bias, float forget, float* h, float* cs) {
  for (unsigned b = 0; b < batch; ++b) {
    const float* x = inputValue + (size_t)b * 4 * units;
    const float* s = stateHValue + (size_t)b * 4 * units;
    for (unsigned i = 0; i < units; ++i) {
      float xi = x[i] + s[i] + bias[i];
      float xc = x[i + units] + s[i + units] + bias[i + units];
      float xf = x[i + 2 * units] + s[i + 2 * units] + bias[i + 2 * units];
      float xo = x[i + 3 * units] + s[i + 3 * units] + bias[i + 3 * units];
      xi = oracle_sigmoid(xi);
      xc = tanhf(xc);
      xf = oracle_sigmoid(xf + forget);
      xo = oracle_sigmoid(xo);
      float c = xc * xi + stateC[(size_t)b * units + i] * xf;
      h[(size_t)b * units + i] = tanhf(c) * xo;
      cs[(size_t)b * units + i] = c;
    }
  }
}

void oracle_gru_cell_gates(unsigned batch, unsigned units, unsigned inputSize, const float* state,
                           const float* inputs, const float* value, const float* bias, float* result) {
  for (unsigned b = 0; b < batch; ++b) {
    float* r = result + (size_t)b * (inputSize + units);
    memcpy(r, inputs + (size_t)b * inputSize, inputSize * sizeof(float));
    for (unsigned i = 0; i < units; ++i)
      r[inputSize + i] = oracle_sigmoid(value[(size_t)b * 2 * units + i] + bias[i]) * state[(size_t)b * units + i];
  }
}

void oracle_gru_cell_candidate(unsigned batch, unsigned units, const float* state, const float* value,
                               const float* bias, const float* cValue, const float* cBias, float* result) {
  for (unsigned b = 0; b < batch; ++b)
    for (unsigned i = 0; i < units; ++i) {
      float u = oracle_sigmoid(value[(size_t)b * 2 * units + units + i] + bias[units + i]);
      float c = tanhf(cValue[(size_t)b * units + i] + cBias[i]);
      result[(size_t)b * units + i] = u * state[(size_t)b * units + i] + (1.f - u) * c;
    }
}

void oracle_pytorch_gru_cell(unsigned batch, unsigned units, const float* state, const float* inputValue,
                             const float* stateValue, const float* gateBias, const float* candidateIBias,
                             const float* candidateHBias, float* result) {
  for (unsigned b = 0; b < batch; ++b) {
    const float* x = inputValue + (size_t)b * 3 * units;
    const float* s = stateValue + (size_t)b * 3 * units;
    for (unsigned i = 0; i < units; ++i) {
      float r = oracle_sigmoid(x[i] + s[i] + gateBias[i]);
      float z = oracle_sigmoid(x[i + units] + s[i + units] + gateBias[i + units]);
      float ni = x[i + 2 * units] + candidateIBias[i];
      float nh = s[i + 2 * units] + candidateHBias[i];
      float n = tanhf(ni + r * nh);
      result[(size_t)b * units + i] = n + z * (state[(size_t)b * units + i] - n);
    }
  }
}

void oracle_lstm_sequence(int backward, unsigned seq, unsigned batch, unsigned length, unsigned hidden,
                          const float* a, const float* inputKernel, const float* stateKernel, const float* bias,
                          const float* ih, const float* ic, float* out, float* h, float* c) {
  const size_t state = (size_t)batch * hidden;
  float* xv = (float*)malloc(state * 4 * sizeof(float));
  float* hv = (float*)malloc(state * 4 * sizeof(float));
  float* hprev = (float*)malloc(state * sizeof(float));
  memcpy(hprev, ih, state * sizeof(float));
  memcpy(c, ic, state * sizeof(float));
  for (unsigned step = 0; step < seq; ++step) {
    const unsigned t = backward ? seq - 1 - step : step;
    oracle_sgemm_strided_batched(a + (size_t)t * batch * length, 0, inputKernel, 0, NULL, xv, NULL, 0, batch, 4 * hidden,
                                 length, 1);
    oracle_sgemm_strided_batched(hprev, 0, stateKernel, 0, NULL, hv, NULL, 0, batch, 4 * hidden, hidden, 1);
    oracle_lstm_cell(batch, hidden, c, xv, hv, bias, 0.f, h, c);
    memcpy(out + (size_t)step * state, h, state * sizeof(float));
    memcpy(hprev, h, state * sizeof(float));
  }
  free(xv);
  free(hv);
  free(hprev);
}
