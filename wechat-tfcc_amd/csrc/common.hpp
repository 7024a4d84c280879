// Shared plumbing of the HIP translation units: error reporting behind the C ABI and the
// range arithmetic of the quantization path evaluated on the device in double.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tfcc_rocm.h"

namespace tfcc_rocm {

// Records the text returned by tfcc_rocm_last_error_string() for the calling thread.
int set_error(int code, const char* fmt, ...);

#define TFCC_HIP_CHECK(expr)                                                                  \
  do {                                                                                        \
    hipError_t _e = (expr);                                                                   \
    if (_e != hipSuccess)                                                                     \
      return ::tfcc_rocm::set_error(                                                          \
          _e == hipErrorOutOfMemory ? TFCC_ROCM_OUT_OF_MEMORY : TFCC_ROCM_HIP_ERROR,          \
          "%s failed: %s", #expr, hipGetErrorString(_e));                                     \
  } while (0)

#define TFCC_REQUIRE(cond, ...)                                                               \
  do {                                                                                        \
    if (!(cond)) return ::tfcc_rocm::set_error(TFCC_ROCM_INVALID_ARGUMENT, __VA_ARGS__);      \
  } while (0)

// Checks the launch that has just been enqueued.
static inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error(TFCC_ROCM_HIP_ERROR, "%s launch failed: %s", what, hipGetErrorString(e));
  return TFCC_ROCM_OK;
}

static inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// ---- range arithmetic (tfcc/core/utils/tfcc_quantizationutils.h:23-70), host and device ----

struct IntRange {
  long long lowest, highest;
  int bits;
};

__host__ __device__ static inline IntRange int_range(int type) {
  switch (type) {
    case TFCC_ROCM_S8: return {-128, 127, 8};
    case TFCC_ROCM_U8: return {0, 255, 8};
    case TFCC_ROCM_S16: return {-32768, 32767, 16};
    case TFCC_ROCM_U16: return {0, 65535, 16};
    case TFCC_ROCM_S32: return {-2147483648LL, 2147483647LL, 32};
    default: return {0, 4294967295LL, 32};
  }
}

// get_quantized_scale_info<T>: scale = stepCnt / range, offset = round(min * scale)
__host__ __device__ static inline void quantized_scale_info(int bits, float mn, float mx,
                                                            double* scale, long long* offset) {
  double step = (double)(1LL << bits);
  double adjust = step / (step - 1.0);
  float span = mx - mn;  // float subtraction, as in the reference
  double range = (double)span * adjust;
  double s = step / range;
  *scale = s;
  *offset = (long long)round((double)mn * s);
}

// get_dequantized_scale_info<T>: scale = range / stepCnt, minRounded = min
__host__ __device__ static inline void dequantized_scale_info(int bits, float mn, float mx,
                                                              double* scale, double* minRounded) {
  double step = (double)(1LL << bits);
  double adjust = step / (step - 1.0);
  float span = mx - mn;
  double range = (double)span * adjust;
  *scale = range / step;
  *minRounded = (double)mn;
}

// get_quantization_range_for_multiplication<uint8_t, int8_t, int32_t>
__host__ __device__ static inline void qmatmul_range(float minA, float maxA, float minB, float maxB,
                                                     float* minC, float* maxC) {
  float aLevel = (maxA - minA) / 255.0f;
  float bLevel = (maxB - minB) / 255.0f;
  float cLevel = aLevel * bLevel;
  *minC = cLevel * -2147483648.0f;
  *maxC = cLevel * 2147483648.0f;  // (float)INT32_MAX rounds to 2^31
}

// offsets of the quantized matmul: tfcc/mkl/operations/tfcc_mklquantization.cpp:181-186
__host__ __device__ static inline void qmatmul_offsets(float minA, float maxA, float minB, float maxB,
                                                       int* offsetA, int* offsetB) {
  double s;
  long long oa, ob;
  quantized_scale_info(8, minA, maxA, &s, &oa);
  quantized_scale_info(8, minB, maxB, &s, &ob);
  *offsetA = (int)oa;          // - lowest(uint8) = 0
  *offsetB = (int)(ob + 128);  // - lowest(int8) = -128
}

// double -> int64 the way x86 cvttsd2si does it (out of range and NaN give INT64_MIN)
__host__ __device__ static inline long long to_int64_x86(double v) {
  if (!(v > -9223372036854775808.0 && v < 9223372036854775808.0)) return (long long)0x8000000000000000ULL;
  return (long long)v;
}

// One requantize step, AVX2 flavour of the reference: fused multiply-add, nearest-even.
// tfcc/mkl/kernel/tfcc_mklquantizationkernel.avx256.cpp:128-138
struct RequantScalars {
  double inScale, inMin, outScale;
  long long outOffset;
  long long inLowest, outLowest, outHighest;
  int mode;            // 0: per-element arithmetic, 1: fill with fillValue (degenerate ranges)
  long long fillValue;
  double offsetMinusLowest;  // (double)(outOffset - outLowest), exact when fastOK
  int fastOK;                // the double shortcut is exact for every input
  int fast32OK;              // ... and rint(y), rint(y) - (outOffset - outLowest) stay inside int32
  int offsetMinusLowest32;
  // fast32OK, the output scale a power of two and outOffset - outLowest even: the scale is folded into the
  // first step's constants and the offset into the rounding constant (see requantize_one_folded)
  int foldedOK;
  double inScaleFolded, inMinFolded, magicFolded;
  // foldedOK and inMinFolded - 2^52 * inScaleFolded is a double without rounding: the first step can take
  // 2^52 + off (the bits of off under the exponent word of 2^52, no conversion instruction) instead of off
  // (see requantize_one_biased_unclamped)
  int biasedOK;
  double inMinBiased;
};

// offMax = highest - lowest of the input type (its largest x - inLowest)
__host__ __device__ static inline void finish_requant_scalars(RequantScalars& s, double offMax) {
  const long long d = (long long)((unsigned long long)s.outOffset - (unsigned long long)s.outLowest);
  s.offsetMinusLowest = (double)d;
  // real = inMin + off * inScale is monotone in off, so its extremes are at off = 0 and off = offMax
  const double r0 = fabs(s.inMin), r1 = fabs(fma(offMax, s.inScale, s.inMin));
  const double bound = (r0 > r1 ? r0 : r1) * fabs(s.outScale);
  s.fastOK = (d > -(1LL << 52) && d < (1LL << 52) && bound < 1125899906842624.0) ? 1 : 0;  // NaN compares false
  const double dAbs = d < 0 ? -(double)d : (double)d;
  s.fast32OK = (s.fastOK && bound + dAbs < 2147483000.0) ? 1 : 0;
  s.offsetMinusLowest32 = s.fast32OK ? (int)d : 0;
  // Multiplying by 2^e commutes with rounding (no overflow, no subnormals: real is 0 or at least 2^-60 in size
  // for 32-bit inputs and scales of normal size), so fma(off, inScale * 2^e, inMin * 2^e) is the reference's
  // real * outScale bit for bit.  An even d keeps the parity of the candidates of a tie, so adding
  // 1.5 * 2^52 - d rounds exactly like rint(y) - d.
  int e = 0;
  const double mant = frexp(s.outScale, &e);  // outScale = mant * 2^e, mant = 0.5 for a positive power of two
  const bool pow2 = mant == 0.5 && e > -200 && e < 200 && fabs(s.inScale) > 1e-60 && fabs(s.inScale) < 1e60 &&
                    (s.inMin == 0.0 || (fabs(s.inMin) > 1e-60 && fabs(s.inMin) < 1e60));
  s.foldedOK = (s.fast32OK && pow2 && (d & 1) == 0) ? 1 : 0;
  s.inScaleFolded = s.inScale * s.outScale;
  s.inMinFolded = s.inMin * s.outScale;
  s.magicFolded = 6755399441055744.0 - (double)d;
  // t = inMinFolded - 2^52 * inScaleFolded; the scaling by 2^52 is exact, and the error term of the
  // subtraction (Knuth's two-sum) is zero exactly when t is the true difference
  const double big = s.inScaleFolded * 4503599627370496.0;
  const double t = s.inMinFolded - big;
  const double bv = t - s.inMinFolded;
  const double err = (s.inMinFolded - (t - bv)) + (-big - bv);
  s.biasedOK = (s.foldedOK && err == 0.0 && fabs(big) < 1e300 && fabs(t) < 1e300) ? 1 : 0;
  s.inMinBiased = t;
}

// Valid when RequantScalars::fast32OK.  Adding 1.5 * 2^52 rounds y to the nearest integer (ties to
// even, the default rounding mode) in the low mantissa bits: the low dword of the sum is rint(y) as a
// two's-complement int32.  The subtraction cannot overflow because |rint(y)| + |offset| < 2^31.
__device__ static inline int requantize_one_fast32(double off, const RequantScalars& s) {
  const double y = fma(off, s.inScale, s.inMin) * s.outScale;
  const int r = (int)(unsigned)__double_as_longlong(y + 6755399441055744.0);
  const int q = r - s.offsetMinusLowest32;
  const int lo = (int)s.outLowest, hi = (int)s.outHighest;
  return q < lo ? lo : (q > hi ? hi : q);
}

// Valid when RequantScalars::foldedOK: two double operations instead of four, the same value.
__device__ static inline int requantize_one_folded(double off, const RequantScalars& s) {
  const double y = fma(off, s.inScaleFolded, s.inMinFolded);
  const int q = (int)(unsigned)__double_as_longlong(y + s.magicFolded);
  const int lo = (int)s.outLowest, hi = (int)s.outHighest;
  return q < lo ? lo : (q > hi ? hi : q);
}

// The two shortcuts above before the clamp, for callers that clamp while packing (pack_sat_u8).
__device__ static inline int requantize_one_fast32_unclamped(double off, const RequantScalars& s) {
  const double y = fma(off, s.inScale, s.inMin) * s.outScale;
  return (int)(unsigned)__double_as_longlong(y + 6755399441055744.0) - s.offsetMinusLowest32;
}
__device__ static inline int requantize_one_folded_unclamped(double off, const RequantScalars& s) {
  return (int)(unsigned)__double_as_longlong(fma(off, s.inScaleFolded, s.inMinFolded) + s.magicFolded);
}

// Valid when RequantScalars::biasedOK.  The double whose high word is 0x43300000 and whose low word is off is
// 2^52 + off exactly, so fma(2^52 + off, inScaleFolded, inMinFolded - 2^52 * inScaleFolded) rounds the same real
// number off * inScaleFolded + inMinFolded as requantize_one_folded_unclamped does: one rounding, the same value,
// and no integer-to-double conversion.
__device__ static inline int requantize_one_biased_unclamped(unsigned off, const RequantScalars& s) {
  const double d = __hiloint2double(0x43300000, (int)off);
  return (int)(unsigned)__double_as_longlong(fma(d, s.inScaleFolded, s.inMinBiased) + s.magicFolded);
}

// std::max and std::min as the reference's kernels call them (tfcc/mkl/interfaces/tfcc_mklminmaxinterface.cpp:37-61,
// tfcc_mklbasicinterface.cpp:152-153, tfcc/mkl/kernel/tfcc_mklactivationkernel.hpp:67-83): a comparison that a NaN
// fails, so the first argument comes back whenever either is a NaN (fmaxf / fminf would drop the NaN).
__device__ __forceinline__ float ref_max(float a, float b) { return a < b ? b : a; }
__device__ __forceinline__ float ref_min(float a, float b) { return b < a ? b : a; }

// The value of lane i ^ MASK for the six steps of a butterfly over the 64 lanes, without the LDS crossbar that
// __shfl_xor goes through: the two halves and the rows of 16 lanes are exchanged by the swap instructions (a and b
// come back as the two members of the pair, in lane order of the lower one), the steps inside a row are data-parallel
// moves.  wave_sum / wave_max below pair the same lanes in the same order as a __shfl_xor loop from 32 down to 1, and
// their operations commute, so the results have the same bits.
template <int MASK>
__device__ __forceinline__ void butterfly_pair(float v, float& a, float& b) {
  const unsigned u = __builtin_bit_cast(unsigned, v);
  if constexpr (MASK == 32) {
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    a = __builtin_bit_cast(float, (unsigned)r[0]); b = __builtin_bit_cast(float, (unsigned)r[1]);
  } else if constexpr (MASK == 16) {
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    a = __builtin_bit_cast(float, (unsigned)r[0]); b = __builtin_bit_cast(float, (unsigned)r[1]);
  } else {
    a = v;
    unsigned o;
    if constexpr (MASK == 8) {
      o = (unsigned)__builtin_amdgcn_update_dpp(0, (int)u, 0x128, 0xf, 0xf, false);  // row_ror:8
    } else if constexpr (MASK == 4) {
      o = (unsigned)__builtin_amdgcn_update_dpp(0, (int)u, 0x104, 0xf, 0x5, false);       // row_shl:4, lanes 0-3, 8-11
      o = (unsigned)__builtin_amdgcn_update_dpp((int)o, (int)u, 0x114, 0xf, 0xa, false);  // row_shr:4, lanes 4-7, 12-15
    } else if constexpr (MASK == 2) {
      o = (unsigned)__builtin_amdgcn_update_dpp(0, (int)u, 0x4e, 0xf, 0xf, false);   // quad_perm [2, 3, 0, 1]
    } else {
      static_assert(MASK == 1, "a power of two below 64");
      o = (unsigned)__builtin_amdgcn_update_dpp(0, (int)u, 0xb1, 0xf, 0xf, false);   // quad_perm [1, 0, 3, 2]
    }
    b = __builtin_bit_cast(float, o);
  }
}
__device__ __forceinline__ float wave_sum(float v) {
  float a, b;
  butterfly_pair<32>(v, a, b); v = a + b;
  butterfly_pair<16>(v, a, b); v = a + b;
  butterfly_pair<8>(v, a, b); v = a + b;
  butterfly_pair<4>(v, a, b); v = a + b;
  butterfly_pair<2>(v, a, b); v = a + b;
  butterfly_pair<1>(v, a, b); v = a + b;
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
  float a, b;
  butterfly_pair<32>(v, a, b); v = fmaxf(a, b);
  butterfly_pair<16>(v, a, b); v = fmaxf(a, b);
  butterfly_pair<8>(v, a, b); v = fmaxf(a, b);
  butterfly_pair<4>(v, a, b); v = fmaxf(a, b);
  butterfly_pair<2>(v, a, b); v = fmaxf(a, b);
  butterfly_pair<1>(v, a, b); v = fmaxf(a, b);
  return v;
}

// Eight reductions over the 64 lanes at once (eight rows of a softmax held by one wavefront): instead of eight
// butterflies of six steps, the first three steps halve the number of values a lane carries (lanes 32 apart split
// the eight rows between them, then lanes 16 apart, then lanes 8 apart), the last three run on the one value left,
// and lane 8r hands row r's result to everybody.  Every result is formed by the additions of wave_sum in the same
// pairing and order (a lane simply does not compute the copies it would throw away), so the bits are those of
// wave_sum / wave_max applied to each row.  24 vector instructions and 8 lane reads where eight butterflies take 120.
template <bool MAX>
__device__ __forceinline__ void wave_reduce8(float (&v)[8], int lane) {
  auto join = [](float a, float b) { return MAX ? fmaxf(a, b) : a + b; };
  auto bits = [](float x) { return __builtin_bit_cast(unsigned, x); };
  auto real = [](unsigned x) { return __builtin_bit_cast(float, x); };
  float w[4], z[2];
#pragma unroll
  for (int a = 0; a < 4; ++a) {  // lanes 0-31 go on with rows 0-3, lanes 32-63 with rows 4-7
    const auto r = __builtin_amdgcn_permlane32_swap(bits(v[a]), bits(v[a + 4]), false, false);
    w[a] = join(real((unsigned)r[0]), real((unsigned)r[1]));
  }
#pragma unroll
  for (int c = 0; c < 2; ++c) {  // of those, lanes with bit 4 clear go on with the first two, the others with the last two
    const auto r = __builtin_amdgcn_permlane16_swap(bits(w[c]), bits(w[c + 2]), false, false);
    z[c] = join(real((unsigned)r[0]), real((unsigned)r[1]));
  }
  const bool odd = (lane & 8) != 0;  // lanes with bit 3 clear go on with the even row of their two, the others with the odd one
  const float mine = odd ? z[1] : z[0], theirs = odd ? z[0] : z[1];
  float a, b;
  butterfly_pair<8>(theirs, a, b);
  float y = join(mine, b);
  butterfly_pair<4>(y, a, b); y = join(a, b);
  butterfly_pair<2>(y, a, b); y = join(a, b);
  butterfly_pair<1>(y, a, b); y = join(a, b);
#pragma unroll
  for (int r = 0; r < 8; ++r) v[r] = real((unsigned)__builtin_amdgcn_readlane((int)bits(y), 8 * r));
}

// e^x for the x <= 0 a softmax forms by subtracting the row maximum (the reference calls the C library's exp,
// tfcc/mkl/kernel/tfcc_mklactivationkernel.hpp:137-155).  2^(x log2 e) with the hardware's exp2: the product is
// formed in two parts (rounded product + what the rounding and the rounding of log2 e dropped), and the small part
// enters as 2^t (1 + lo ln 2).  Within 2 units in the last place of the exact value (checked on the GPU for every
// float in [-104, 0] against double precision); below -104 the result is 0 like the library's, NaN stays NaN.
// Eight vector instructions where the library's expf takes thirteen.
__device__ static inline float softmax_exp(float x) {
  x = x < -104.0f ? -104.0f : x;
  const float L = 1.44269504088896341f;
  const float t = x * L;
  float lo = fmaf(x, L, -t);
  lo = fmaf(x, 1.92596303e-8f, lo);
  const float e = __builtin_amdgcn_exp2f(t);
  return fmaf(e, lo * 0.693147180559945f, e);
}

// GELU in its erf form, 0.5 x (1 + erf(x / sqrt 2)), the function of the reference's scalar template
// (tfcc/mkl/kernel/tfcc_mklactivationkernel.hpp:213-220, which calls the C library's erff).  One function for the
// stand-alone kernel and for every fused tile store, so that fusing changes no bit.  1 + erf(q) is erfc(-q), and
// erfc(t) = 2^(t P(t)) for t >= 0 with P a degree-8 fit of log2(erfc(t)) / t (tests/golden/fit_gelu_erfc.py
// makes the coefficients: minimax in the error of erfc, 4e-9): for q < 0 the small factor keeps its relative
// accuracy, for q > 0 it is 2 - erfc(q).  Past t = 5 erfc is below 2e-12 and taken as 0, which also gives the
// reference's values at the infinities (NaN at -inf, +inf at +inf) and for NaN.  Eighteen vector instructions
// where the library's erff takes fifty, and closer to the exact value: over all 2^32 floats the largest
// |result - exact| / (1e-7 + 1e-6 |exact|) is 0.24, against 0.83 with the library's erff (checked on the GPU
// against double precision).
__device__ static inline float gelu_erf_f32(float v) {
  const float q = v * 0.70710678118654752f;
  const float t = __builtin_fabsf(q);
  float p = 1.160490228e-05f;
  p = fmaf(p, t, -1.529651927e-04f);
  p = fmaf(p, t, 8.482374833e-04f);
  p = fmaf(p, t, -2.274791477e-03f);
  p = fmaf(p, t, 8.481170516e-05f);
  p = fmaf(p, t, 2.772447281e-02f);
  p = fmaf(p, t, -1.483079046e-01f);
  p = fmaf(p, t, -9.184429049e-01f);
  p = fmaf(p, t, -1.627907276e+00f);
  float e = __builtin_amdgcn_exp2f(p * t);  // erfc(t)
  e = t > 5.0f ? 0.0f : e;
  const float w = q < 0.0f ? e : 2.0f - e;
  return (v * 0.5f) * w;
}

// Four int32 clamped to 0..255 and packed into one word, first value in the low byte: int32 -> int16 and
// int16 -> uint8, both saturating.
__device__ static inline unsigned pack_sat_u8(int a, int b, int c, int d) {
  typedef short pack_v2s __attribute__((ext_vector_type(2)));
  const pack_v2s lo = __builtin_amdgcn_cvt_pk_i16(a, b), hi = __builtin_amdgcn_cvt_pk_i16(c, d);
  unsigned l, h;
  asm("v_sat_pk_u8_i16 %0, %1" : "=v"(l) : "v"(lo));
  asm("v_sat_pk_u8_i16 %0, %1" : "=v"(h) : "v"(hi));
  return l | (h << 16);
}

__device__ static inline long long requantize_one_exact(long long x, const RequantScalars& s) {
  double off = (double)x - (double)s.inLowest;
  double real = fma(off, s.inScale, s.inMin);
  long long q = to_int64_x86(rint(real * s.outScale));
  q = (long long)((unsigned long long)q - (unsigned long long)s.outOffset + (unsigned long long)s.outLowest);
  q = q < s.outLowest ? s.outLowest : q;
  q = q > s.outHighest ? s.outHighest : q;
  return q;
}

// Same result with the integer tail evaluated in double, valid when RequantScalars::fastOK: then
// |y| < 2^50 for every possible input and |outOffset - outLowest| < 2^52, so rint(y), the
// subtraction and the clamp are exact in double.  `off` = x - inLowest as a double.
__device__ static inline int requantize_one_fast(double off, const RequantScalars& s) {
  const double y = fma(off, s.inScale, s.inMin) * s.outScale;
  double q = rint(y) - s.offsetMinusLowest;
  q = fmax(q, (double)s.outLowest);
  q = fmin(q, (double)s.outHighest);
  return (int)q;
}

// The branches of _requantize_helper (tfcc/mkl/interfaces/tfcc_mklquantizationinterface.cpp:121-141)
__host__ __device__ static inline RequantScalars make_requant_scalars(int inType, int outType, float minIn,
                                                                      float maxIn, float minOut, float maxOut) {
  RequantScalars s;
  IntRange ri = int_range(inType), ro = int_range(outType);
  s.inLowest = ri.lowest;
  s.outLowest = ro.lowest;
  s.outHighest = ro.highest;
  s.mode = 0;
  s.fillValue = 0;
  s.inScale = s.inMin = s.outScale = 0.0;
  s.outOffset = 0;
  s.fastOK = 0;
  s.fast32OK = 0;
  s.foldedOK = 0;
  s.biasedOK = 0;
  s.offsetMinusLowest32 = 0;
  s.offsetMinusLowest = 0.0;
  if (minOut >= maxOut) {
    s.mode = 1;
    s.fillValue = ro.lowest;
    return s;
  }
  dequantized_scale_info(ri.bits, minIn, maxIn, &s.inScale, &s.inMin);
  quantized_scale_info(ro.bits, minOut, maxOut, &s.outScale, &s.outOffset);
  if (minIn >= maxIn) {
    long long q = to_int64_x86(round((double)minIn * s.outScale));
    q = (long long)((unsigned long long)q - (unsigned long long)s.outOffset + (unsigned long long)ro.lowest);
    q = q < ro.lowest ? ro.lowest : q;
    q = q > ro.highest ? ro.highest : q;
    s.mode = 1;
    s.fillValue = q;
  }
  finish_requant_scalars(s, (double)(ri.highest - ri.lowest));
  return s;
}

}  // namespace tfcc_rocm
