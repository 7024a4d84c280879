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
  // what the requantize step makes of the four immediate scalars above (RequantScalars' derived fields), worked
  // out by launchers whose kernel reads it instead of deriving it per thread; unused with minOut / maxOut
  double rqInScaleFolded, rqInMinFolded, rqMagicFolded, rqOffsetMinusLowest, rqInMinBiased;
  int rqOffsetMinusLowest32, rqFastOK, rqFast32OK, rqFoldedOK, rqBiasedOK;
  // division by tilesM * tilesN and by 4 * tilesN as multiply-high and shift (filled by launchers whose kernel uses them)
  unsigned perBatchMagic, perBatchShift, bandMagic, bandShift;
};

// x / d for any 32-bit x as (mulhi(x, magic) + x) >> shift, evaluated without overflow; shift 0 stands for d == 1.
struct UDiv { unsigned magic, shift; };
static inline UDiv udiv_prepare(unsigned d) {
  if (d <= 1) return {0u, 0u};
  unsigned s = 0;
  while ((1ull << s) < d) ++s;  // ceil(log2 d), 1..32
  const unsigned long long m = ((1ull << 32) * ((1ull << s) - d)) / d + 1;
  return {(unsigned)m, s};
}
#if defined(__HIPCC__)
__device__ __forceinline__ unsigned udiv_apply(unsigned x, unsigned magic, unsigned shift) {
  if (shift == 0u) return x;
  const unsigned t = __umulhi(x, magic);
  return (t + ((x - t) >> 1)) >> (shift - 1);
}
#endif

}  // namespace tfcc_rocm
