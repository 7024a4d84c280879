// Kernel argument block of the quantized matmul kernels.
#pragma once
#include <stdint.h>

namespace tfcc_rocm {

struct QGemmParams {
  const unsigned char* A;
  const signed char* B;
  const int* rowsumA;
  const int* colsumB;
  int* C;             // int32 result (may be null when requantizing)
  unsigned char* Q;   // requantized result (requant kernels only)
  unsigned long long strideA, strideB, strideRA, strideRB, strideC;
  unsigned M, N, K, batch;
  int offsetA, offsetB;
  // optional float ranges in device memory (then the offsets above are ignored)
  const float *minA, *maxA, *minB, *maxB;
  float *minC, *maxC;
  // requantize scalars (immediate) or output range in device memory
  double inScale, inMin, outScale;
  long long outOffset;
  const float *minOut, *maxOut;
  int colsumExact;    // colsumB holds the true column sums of B: no need to accumulate them
  // tile bookkeeping filled by the launcher
  unsigned tilesM, tilesN, tilesTotal, chunk;
};

}  // namespace tfcc_rocm
