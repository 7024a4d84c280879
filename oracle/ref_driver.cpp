// C entry points over the REFERENCE's own quantized-matmul, quantization and recurrent-cell kernels.
// TEST INFRASTRUCTURE ONLY.  This file contains no arithmetic of the hot path: the matmul
// micro-kernel, the AVX2 requantize / quantize / dequantize kernels, the scalar kernels and the
// range helpers are the reference's, compiled from where they lie in the reference tree
// (see the Makefile next to this file).  The only restated piece is the offset-matrix pre-fill,
// which in the reference is a file-static function of a translation unit that needs oneDNN
// (tfcc/mkl/operations/tfcc_mklquantization.cpp:33-69) and therefore cannot be compiled here.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <tuple>
#include <vector>

#include "kernel/tfcc_mklquantizationkernel.avx256.h"
#include "kernel/tfcc_mklquantizationkernel.hpp"
#include "kernel/tfcc_mklquantizationmatmul.avx256.h"
#include "kernel/tfcc_mklcellkernel.hpp"
#include "utils/tfcc_quantizationutils.h"

namespace {

// The AVX2 kernels stride by 4 / 8 / 16 elements with no tail handling
// (tfcc/mkl/kernel/tfcc_mklquantizationkernel.avx256.cpp:66,104,127), so run them on padded copies.
template <class T>
std::vector<T> padded(const T* p, uint64_t total, uint64_t mult) {
  std::vector<T> v((total + mult - 1) / mult * mult + mult, T());
  std::memcpy(v.data(), p, total * sizeof(T));
  return v;
}

}  // namespace

extern "C" {

// offsets exactly as tfcc/mkl/operations/tfcc_mklquantization.cpp:181-186 derives them
void ref_qmatmul_offsets(float minA, float maxA, float minB, float maxB, int32_t* offsetA,
                         int32_t* offsetB) {
  int64_t oa, ob;
  std::tie(std::ignore, oa) = tfcc::get_quantized_scale_info<uint8_t>(minA, maxA);
  std::tie(std::ignore, ob) = tfcc::get_quantized_scale_info<int8_t>(minB, maxB);
  oa -= static_cast<int64_t>(std::numeric_limits<uint8_t>::lowest());
  ob -= static_cast<int64_t>(std::numeric_limits<int8_t>::lowest());
  *offsetA = static_cast<int32_t>(oa);
  *offsetB = static_cast<int32_t>(ob);
}

void ref_qmatmul_range(float minA, float maxA, float minB, float maxB, float* minC, float* maxC) {
  std::tie(*minC, *maxC) =
      tfcc::get_quantization_range_for_multiplication<uint8_t, int8_t, int32_t>(minA, maxA, minB, maxB);
}

// General path: offset matrix, then the reference driver accumulates the product into it
// (tfcc/mkl/operations/tfcc_mklquantization.cpp:176-201).
void ref_qgemm_u8s8s32(unsigned batch, const uint8_t* a, unsigned strideA, const int8_t* b,
                       unsigned strideB, const int32_t* rowsumA, unsigned strideRA,
                       const int32_t* colsumB, unsigned strideRB, int32_t offsetA, int32_t offsetB,
                       unsigned m, unsigned n, unsigned k, int32_t* c) {
  unsigned strideC = m * n;
  uint32_t global = (uint32_t)offsetA * (uint32_t)offsetB * (uint32_t)k;
  for (unsigned bi = 0; bi < batch; ++bi)
    for (unsigned i = 0; i < m; ++i)
      for (unsigned j = 0; j < n; ++j)
        c[(size_t)bi * strideC + (size_t)i * n + j] =
            (int32_t)(global + (uint32_t)rowsumA[(size_t)bi * strideRA + i] * (uint32_t)offsetB +
                      (uint32_t)colsumB[(size_t)bi * strideRB + j] * (uint32_t)offsetA);
  tfcc::_MKLQuantizationMatmulAVX256::quantizedMatmulColMajor(batch, b, strideB, a, strideA, n, m,
                                                               k, c, strideC);
}

// N == 1 path: tfcc/mkl/operations/tfcc_mklquantization.cpp:151-174
void ref_qgemm_n1(const uint8_t* a, const int32_t* rowsumA, int32_t offsetA, const int8_t* b,
                  int32_t colsumB, int32_t offsetB, unsigned m, unsigned k, int32_t* c) {
  tfcc::_MKLQuantizationMatmulAVX256::quantizedMatmulN1(a, rowsumA, offsetA, b, colsumB, offsetB, m,
                                                         k, c);
}

void ref_quantized_scale_info_u8(float mn, float mx, double* scale, int64_t* offset) {
  std::tie(*scale, *offset) = tfcc::get_quantized_scale_info<uint8_t>(mn, mx);
}
void ref_quantized_scale_info_u16(float mn, float mx, double* scale, int64_t* offset) {
  std::tie(*scale, *offset) = tfcc::get_quantized_scale_info<uint16_t>(mn, mx);
}
void ref_dequantized_scale_info_s32(float mn, float mx, double* scale, double* minRounded) {
  std::tie(*scale, *minRounded) = tfcc::get_dequantized_scale_info<int32_t>(mn, mx);
}

// requantize, non-degenerate ranges only (the degenerate branches live in the oneDNN-dependent
// interface file).  avx2 != 0: the AVX2 kernel; else the scalar kernel.
#define REF_REQUANTIZE(NAME, TI, TO)                                                              \
  void NAME(const TI* a, uint64_t total, float minIn, float maxIn, float minOut, float maxOut,   \
            int avx2, TO* out) {                                                                 \
    double inScale, inMin, outScale;                                                             \
    int64_t outOffset;                                                                           \
    std::tie(inScale, inMin) = tfcc::get_dequantized_scale_info<TI>(minIn, maxIn);               \
    std::tie(outScale, outOffset) = tfcc::get_quantized_scale_info<TO>(minOut, maxOut);          \
    if (avx2) {                                                                                  \
      auto in = padded(a, total, 4);                                                             \
      std::vector<TO> res(in.size());                                                            \
      tfcc::_MKLRequantizationKernelAVX256<TI, TO>::requantize(                                  \
          in.data(), (unsigned)((total + 3) / 4 * 4), inScale, inMin, outScale, outOffset,       \
          res.data());                                                                           \
      std::memcpy(out, res.data(), total * sizeof(TO));                                          \
    } else {                                                                                     \
      tfcc::_MKLRequantizationKernel<TI, TO>::requantize(a, (unsigned)total, inScale, inMin,     \
                                                         outScale, outOffset, out);              \
    }                                                                                            \
  }
REF_REQUANTIZE(ref_requantize_s32_u8, int32_t, uint8_t)
REF_REQUANTIZE(ref_requantize_s8_u16, int8_t, uint16_t)

#define REF_DEQUANTIZE(NAME, T)                                                                   \
  void NAME(const T* a, uint64_t total, float mn, float mx, int avx2, float* out) {              \
    double scale, minRounded;                                                                    \
    std::tie(scale, minRounded) = tfcc::get_dequantized_scale_info<T>(mn, mx);                   \
    if (avx2) {                                                                                  \
      auto in = padded(a, total, 8);                                                             \
      std::vector<float> res(in.size());                                                         \
      tfcc::_MKLQuantizationKernelAVX256<T>::dequantize(in.data(), (unsigned)((total + 7) / 8 * 8), \
                                                        scale, minRounded, res.data());          \
      std::memcpy(out, res.data(), total * sizeof(float));                                       \
    } else {                                                                                     \
      tfcc::_MKLQuantizationKernel<T>::dequantize(a, (unsigned)total, scale, minRounded, out);   \
    }                                                                                            \
  }
REF_DEQUANTIZE(ref_dequantize_s8, int8_t)
REF_DEQUANTIZE(ref_dequantize_u8, uint8_t)
REF_DEQUANTIZE(ref_dequantize_s32, int32_t)

#define REF_QUANTIZE(NAME, T)                                                                     \
  void NAME(const float* a, uint64_t total, float mn, float mx, int avx2, T* out) {              \
    double scale;                                                                                \
    int64_t offset;                                                                              \
    std::tie(scale, offset) = tfcc::get_quantized_scale_info<T>(mn, mx);                         \
    if (avx2) {                                                                                  \
      auto in = padded(a, total, 16);                                                            \
      std::vector<T> res(in.size());                                                             \
      tfcc::_MKLQuantizationKernelAVX256<T>::quantize(in.data(), (unsigned)((total + 15) / 16 * 16), \
                                                      scale, offset, res.data());                \
      std::memcpy(out, res.data(), total * sizeof(T));                                           \
    } else {                                                                                     \
      tfcc::_MKLQuantizationKernel<T>::quantize(a, (unsigned)total, scale, offset, out);         \
    }                                                                                            \
  }
REF_QUANTIZE(ref_quantize_u8, uint8_t)
REF_QUANTIZE(ref_quantize_s8, int8_t)

// The scalar recurrent-cell kernels of the reference (tfcc/mkl/kernel/tfcc_mklcellkernel.hpp), as compiled.
void ref_lstm_cell(unsigned batch, unsigned units, const float* stateC, const float* inputValue,
                   const float* stateHValue, const float* bias, float forget, float* h, float* cs) {
  tfcc::_MKLCellKernel<float>::processLSTMCell(batch, units, stateC, inputValue, stateHValue, bias, forget, h, cs);
}
void ref_gru_cell_gates(unsigned batch, unsigned units, unsigned inputSize, const float* state, const float* inputs,
                        const float* value, const float* bias, float* result) {
  tfcc::_MKLCellKernel<float>::processGRUCellGates(batch, units, inputSize, state, inputs, value, bias, result);
}
void ref_gru_cell_candidate(unsigned batch, unsigned units, const float* state, const float* value, const float* bias,
                            const float* cValue, const float* cBias, float* result) {
  tfcc::_MKLCellKernel<float>::processGRUCellCandidate(batch, units, state, value, bias, cValue, cBias, result);
}
void ref_pytorch_gru_cell(unsigned batch, unsigned units, const float* state, const float* inputValue,
                          const float* stateValue, const float* gateBias, const float* candidateIBias,
                          const float* candidateHBias, float* result) {
  tfcc::_MKLCellKernel<float>::processPyTorchGRUCell(batch, units, state, inputValue, stateValue, gateBias,
                                                     candidateIBias, candidateHBias, result);
}

}  // extern "C"
