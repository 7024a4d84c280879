// Bandwidth-bound companions of the quantized matmul: int32 row / column sums, and the
// range-based quantize / requantize / dequantize steps with their scale arithmetic evaluated on
// the device in double (the ranges are float scalars in device memory, as the reference passes
// them as tensors).
//
// Replaces tfcc/mkl/operations/tfcc_mklquantization.cpp:205-318 (reduce_sum),
// tfcc/mkl/kernel/tfcc_mklquantizationkernel.avx256.cpp:55-145 (the AVX2 kernels: nearest-even
// rounding, fused multiply-add) and the branches of
// tfcc/mkl/interfaces/tfcc_mklquantizationinterface.cpp:47-69,72-147,191-240,284-333.
#include "common.hpp"

namespace tfcc_rocm {
namespace {

template <class T>
__device__ __forceinline__ long long load_as_i64(const void* p, size_t i) {
  return (long long)static_cast<const T*>(p)[i];
}

__device__ __forceinline__ long long load_typed(const void* p, int type, size_t i) {
  switch (type) {
    case TFCC_ROCM_S8: return load_as_i64<int8_t>(p, i);
    case TFCC_ROCM_U8: return load_as_i64<uint8_t>(p, i);
    case TFCC_ROCM_S16: return load_as_i64<int16_t>(p, i);
    case TFCC_ROCM_U16: return load_as_i64<uint16_t>(p, i);
    case TFCC_ROCM_S32: return load_as_i64<int32_t>(p, i);
    default: return load_as_i64<uint32_t>(p, i);
  }
}

__device__ __forceinline__ void store_typed(void* p, int type, size_t i, long long v) {
  switch (type) {
    case TFCC_ROCM_S8: static_cast<int8_t*>(p)[i] = (int8_t)v; break;
    case TFCC_ROCM_U8: static_cast<uint8_t*>(p)[i] = (uint8_t)v; break;
    case TFCC_ROCM_S16: static_cast<int16_t*>(p)[i] = (int16_t)v; break;
    case TFCC_ROCM_U16: static_cast<uint16_t*>(p)[i] = (uint16_t)v; break;
    case TFCC_ROCM_S32: static_cast<int32_t*>(p)[i] = (int32_t)v; break;
    default: static_cast<uint32_t*>(p)[i] = (uint32_t)v; break;
  }
}

// ---- row sums: one wavefront per row, 128-bit loads when the row allows it ------------------
template <class T>
__global__ __launch_bounds__(256) void reduce_rows_kernel(const T* a, unsigned rows, unsigned col, int* out) {
  const unsigned wave = (blockIdx.x * 256 + threadIdx.x) >> 6, lane = threadIdx.x & 63;
  if (wave >= rows) return;
  const T* p = a + (size_t)wave * col;
  unsigned s = 0;
  constexpr unsigned PER = 16 / sizeof(T);
  if (col % PER == 0 && ((uintptr_t)a % 16 == 0)) {
    const uint4* v = reinterpret_cast<const uint4*>(p);
    const unsigned chunks = col / PER;
    // eight loads in flight per lane; bytes are summed four at a time by the dot-product instructions
    for (unsigned i0 = lane; i0 < chunks; i0 += 64 * 8) {
      uint4 q[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        q[u] = make_uint4(0, 0, 0, 0);
        if (i0 + 64 * u < chunks) q[u] = v[i0 + 64 * u];
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const unsigned w[4] = {q[u].x, q[u].y, q[u].z, q[u].w};
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          if (sizeof(T) == 1) {
            if (T(-1) < T(0)) s = (unsigned)__builtin_amdgcn_sdot4((int)w[d], 0x01010101, (int)s, false);
            else s = __builtin_amdgcn_udot4(w[d], 0x01010101u, s, false);
          } else {
#pragma unroll
            for (int b = 0; b < 2; ++b) s += (unsigned)(int)(T)(w[d] >> (16 * b));
          }
        }
      }
    }
  } else {
    for (unsigned i = lane; i < col; i += 64) s += (unsigned)(int)p[i];
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) s += __shfl_down(s, off, 64);
  if (lane == 0) out[wave] = (int)s;
}

// ---- column sums: a workgroup owns 256 x (4 bytes) columns of one batch entry and a slab of rows;
// slabs are combined with integer atomics (exact and order independent) into a zeroed result.
template <class T>
__global__ __launch_bounds__(256) void reduce_cols_kernel(const T* a, unsigned row, unsigned col,
                                                          unsigned rowsPerSlab, int* out) {
  const unsigned b = blockIdx.z;
  const unsigned c = blockIdx.x * 256 + threadIdx.x;
  const unsigned r0 = blockIdx.y * rowsPerSlab;
  const unsigned r1 = min(r0 + rowsPerSlab, row);
  if (c >= col) return;
  const T* p = a + (size_t)b * row * col + c;
  unsigned s = 0;
  for (unsigned r = r0; r < r1; ++r) s += (unsigned)(int)p[(size_t)r * col];
  atomicAdd(reinterpret_cast<unsigned*>(out) + (size_t)b * col + c, s);
}

template <class T>
__global__ __launch_bounds__(256) void reduce_cols_vec_kernel(const T* a, unsigned row, unsigned col,
                                                              unsigned rowsPerSlab, int* out) {
  // col % 4 == 0 and 4-byte aligned rows (1-byte types): one dword = 4 columns per thread
  const unsigned b = blockIdx.z;
  const unsigned c4 = blockIdx.x * 256 + threadIdx.x;
  const unsigned r0 = blockIdx.y * rowsPerSlab;
  const unsigned r1 = min(r0 + rowsPerSlab, row);
  if (c4 * 4 >= col) return;
  const unsigned* p = reinterpret_cast<const unsigned*>(a + (size_t)b * row * col) + c4;
  const unsigned pitch = col / 4;
  unsigned s[4] = {0, 0, 0, 0};
  for (unsigned r = r0; r < r1; ++r) {
    unsigned w = p[(size_t)r * pitch];
#pragma unroll
    for (int e = 0; e < 4; ++e) s[e] += (unsigned)(int)(T)(w >> (8 * e));
  }
  unsigned* o = reinterpret_cast<unsigned*>(out) + (size_t)b * col + c4 * 4;
#pragma unroll
  for (int e = 0; e < 4; ++e) atomicAdd(o + e, s[e]);
}

// 16-byte loads of data that is read once
typedef int nt_v4i __attribute__((ext_vector_type(4)));
typedef float nt_v4f __attribute__((ext_vector_type(4)));
__device__ __forceinline__ int4 load_streamed(const int4* p) {
  const nt_v4i v = __builtin_nontemporal_load(reinterpret_cast<const nt_v4i*>(p));
  return make_int4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ float4 load_streamed(const float4* p) {
  const nt_v4f v = __builtin_nontemporal_load(reinterpret_cast<const nt_v4f*>(p));
  return make_float4(v[0], v[1], v[2], v[3]);
}

// Column sums of a 1-byte type with col % 16 == 0 and 16-byte aligned rows.  A workgroup owns 1024 columns
// (64 threads x 16 bytes: whole 1 KB row segments) and a slab of rows, dealt to four row lanes.  A thread takes its
// rows four at a time, transposes each 4 x 4 byte block in registers so that a word holds one column's four rows,
// and adds those with one dot-product instruction; the four row lanes meet in LDS and the slab's sums go to the
// (zeroed) result with integer atomics, whose order does not matter.
__device__ __forceinline__ void transpose_bytes_4x4(const unsigned r[4], unsigned c[4]) {
  const unsigned t0 = __builtin_amdgcn_perm(r[1], r[0], 0x05010400u), t1 = __builtin_amdgcn_perm(r[1], r[0], 0x07030602u);
  const unsigned t2 = __builtin_amdgcn_perm(r[3], r[2], 0x05010400u), t3 = __builtin_amdgcn_perm(r[3], r[2], 0x07030602u);
  c[0] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
  c[1] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
  c[2] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
  c[3] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
}

template <class T>
__global__ __launch_bounds__(256) void reduce_cols_wide_kernel(const T* a, unsigned row, unsigned col,
                                                               unsigned rowsPerSlab, int* out) {
  constexpr bool kSigned = T(-1) < T(0);
  __shared__ int part[4][64][17];
  const unsigned b = blockIdx.z, cg = threadIdx.x & 63u, rl = threadIdx.x >> 6;
  const unsigned c16 = blockIdx.x * 64 + cg;
  const unsigned r0 = blockIdx.y * rowsPerSlab, r1 = min(r0 + rowsPerSlab, row);
  int s[16];
#pragma unroll
  for (int e = 0; e < 16; ++e) s[e] = 0;
  if (c16 * 16 < col) {
    const size_t pitch = col / 16;
    const int4* p = reinterpret_cast<const int4*>(a + (size_t)b * row * col) + c16;
    unsigned r = r0 + rl;
#pragma unroll 2
    for (; r + 12 < r1; r += 16) {
      const int4 v0 = load_streamed(p + (size_t)r * pitch), v1 = load_streamed(p + (size_t)(r + 4) * pitch),
                 v2 = load_streamed(p + (size_t)(r + 8) * pitch), v3 = load_streamed(p + (size_t)(r + 12) * pitch);
      const unsigned w[4][4] = {{(unsigned)v0.x, (unsigned)v1.x, (unsigned)v2.x, (unsigned)v3.x},
                                {(unsigned)v0.y, (unsigned)v1.y, (unsigned)v2.y, (unsigned)v3.y},
                                {(unsigned)v0.z, (unsigned)v1.z, (unsigned)v2.z, (unsigned)v3.z},
                                {(unsigned)v0.w, (unsigned)v1.w, (unsigned)v2.w, (unsigned)v3.w}};
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        unsigned c[4];
        transpose_bytes_4x4(w[d], c);
#pragma unroll
        for (int e = 0; e < 4; ++e)
          s[4 * d + e] = kSigned ? __builtin_amdgcn_sdot4((int)c[e], 0x01010101, s[4 * d + e], false)
                                 : (int)__builtin_amdgcn_udot4(c[e], 0x01010101u, (unsigned)s[4 * d + e], false);
      }
    }
    for (; r < r1; r += 4) {
      const int4 v = load_streamed(p + (size_t)r * pitch);
      const unsigned w[4] = {(unsigned)v.x, (unsigned)v.y, (unsigned)v.z, (unsigned)v.w};
#pragma unroll
      for (int d = 0; d < 4; ++d)
#pragma unroll
        for (int e = 0; e < 4; ++e) s[4 * d + e] += (int)(T)(w[d] >> (8 * e));
    }
  }
#pragma unroll
  for (int e = 0; e < 16; ++e) part[rl][cg][e] = s[e];
  __syncthreads();
  // 1024 sums per workgroup, four per thread
  unsigned* o = reinterpret_cast<unsigned*>(out) + (size_t)b * col;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const unsigned idx = threadIdx.x + 256u * q, g = idx >> 4, e = idx & 15u;
    const unsigned column = (blockIdx.x * 64 + g) * 16 + e;
    if (column < col) atomicAdd(o + column, (unsigned)(part[0][g][e] + part[1][g][e] + part[2][g][e] + part[3][g][e]));
  }
}

__global__ void zero_kernel(int* p, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

// ---- requantize / dequantize / quantize -----------------------------------------------------
__global__ __launch_bounds__(256) void requantize_kernel(const void* in, int inType, void* out, int outType,
                                                         size_t total, const float* minIn, const float* maxIn,
                                                         const float* minOut, const float* maxOut) {
  const RequantScalars s = make_requant_scalars(inType, outType, *minIn, *maxIn, *minOut, *maxOut);
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (; i < total; i += step) {
    long long q = s.fillValue;
    if (!s.mode) {
      const long long x = load_typed(in, inType, i);
      q = s.fastOK ? (long long)requantize_one_fast((double)(x - s.inLowest), s) : requantize_one_exact(x, s);
    }
    store_typed(out, outType, i, q);
  }
}


// int32 -> uint8, the matmul epilogue's type pair.  Four elements per 16-byte load, four loads in flight per
// thread, few enough threads that the scalar set-up (a few hundred double operations) is not what the launch
// spends its time on.
template <int FLAVOUR>  // 1 double shortcut, 2 exact int64, 3 fill, 4 int32 shortcut, 5 folded
__device__ __forceinline__ unsigned requantize_four(const int4& v, const RequantScalars& s) {
  const int x[4] = {v.x, v.y, v.z, v.w};
  unsigned q[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const double off = (double)((unsigned)x[e] ^ 0x80000000u);
    if (FLAVOUR == 5) q[e] = (unsigned)requantize_one_folded(off, s);
    else if (FLAVOUR == 4) q[e] = (unsigned)requantize_one_fast32(off, s);
    else if (FLAVOUR == 1) q[e] = (unsigned)requantize_one_fast(off, s);
    else if (FLAVOUR == 2) q[e] = (unsigned)requantize_one_exact(x[e], s);
    else q[e] = (unsigned)s.fillValue;
  }
  return (q[0] | (q[1] << 8)) | ((q[2] | (q[3] << 8)) << 16);
}

template <int FLAVOUR>
__device__ __forceinline__ void requantize_s32_u8_loop(const int4* in, unsigned* out, size_t total4, const RequantScalars& s) {
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total4; i += 4 * step) {
    int4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (i + u * step < total4) v[u] = load_streamed(in + i + u * step);
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (i + u * step < total4) out[i + u * step] = requantize_four<FLAVOUR>(v[u], s);
  }
}

__global__ __launch_bounds__(256) void requantize_s32_u8_vec_kernel(const int4* in, unsigned* out, size_t total4,
                                                                    const float* minIn, const float* maxIn,
                                                                    const float* minOut, const float* maxOut) {
  const RequantScalars s = make_requant_scalars(TFCC_ROCM_S32, TFCC_ROCM_U8, *minIn, *maxIn, *minOut, *maxOut);
  if (s.mode) requantize_s32_u8_loop<3>(in, out, total4, s);
  else if (s.foldedOK) requantize_s32_u8_loop<5>(in, out, total4, s);
  else if (s.fast32OK) requantize_s32_u8_loop<4>(in, out, total4, s);
  else if (s.fastOK) requantize_s32_u8_loop<1>(in, out, total4, s);
  else requantize_s32_u8_loop<2>(in, out, total4, s);
}

// int32 -> float, four elements per thread and load (the accumulators of a quantized matmul)
__global__ __launch_bounds__(256) void dequantize_s32_vec_kernel(const int4* in, size_t total4, const float* minV,
                                                                 const float* maxV, float4* out) {
  const float mn = *minV, mx = *maxV;
  double scale = 0, minRounded = 0;
  const bool constant = mn >= mx;  // tfcc_mklquantizationinterface.cpp:321-324
  if (!constant) dequantized_scale_info(32, mn, mx, &scale, &minRounded);
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total4; i += 4 * step) {
    int4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (i + u * step < total4) v[u] = load_streamed(in + i + u * step);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (i + u * step >= total4) continue;
      float4 r = make_float4(mn, mn, mn, mn);
      if (!constant) {
        // (double)x - (double)INT32_MIN, exact in double
        r.x = (float)fma((double)((unsigned)v[u].x ^ 0x80000000u), scale, minRounded);
        r.y = (float)fma((double)((unsigned)v[u].y ^ 0x80000000u), scale, minRounded);
        r.z = (float)fma((double)((unsigned)v[u].z ^ 0x80000000u), scale, minRounded);
        r.w = (float)fma((double)((unsigned)v[u].w ^ 0x80000000u), scale, minRounded);
      }
      out[i + u * step] = r;
    }
  }
}

__global__ __launch_bounds__(256) void dequantize_kernel(const void* in, int inType, size_t total,
                                                         const float* minV, const float* maxV, float* out) {
  const float mn = *minV, mx = *maxV;
  const IntRange r = int_range(inType);
  double scale = 0, minRounded = 0;
  const bool constant = mn >= mx;  // tfcc_mklquantizationinterface.cpp:321-324
  if (!constant) dequantized_scale_info(r.bits, mn, mx, &scale, &minRounded);
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (; i < total; i += step) {
    if (constant) {
      out[i] = mn;
    } else {
      double off = (double)load_typed(in, inType, i) - (double)r.lowest;
      out[i] = (float)fma(off, scale, minRounded);
    }
  }
}

__global__ __launch_bounds__(256) void quantize_kernel(const float* in, size_t total, const float* minV,
                                                       const float* maxV, void* out, int outType, int fromData) {
  const float mn = *minV, mx = *maxV;
  const IntRange r = int_range(outType);
  // given range: min >= max fills with lowest (tfcc_mklquantizationinterface.cpp:229-232);
  // range taken from the data: min == max fills with lowest (:58-61)
  const bool fillLowest = fromData ? (mn == mx) : (mn >= mx);
  double scale = 0;
  long long offset = 0;
  if (!fillLowest) quantized_scale_info(r.bits, mn, mx, &scale, &offset);
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (; i < total; i += step) {
    long long q = r.lowest;
    if (!fillLowest) {
      q = to_int64_x86(rint((double)in[i] * scale));
      q = (long long)((unsigned long long)q - (unsigned long long)offset + (unsigned long long)r.lowest);
      q = q < r.lowest ? r.lowest : q;
      q = q > r.highest ? r.highest : q;
    }
    store_typed(out, outType, i, q);
  }
}

// float -> uint8 / int8, four elements per thread and load, four loads in flight
__global__ __launch_bounds__(256) void quantize_8bit_vec_kernel(const float4* in, size_t total4, const float* minV,
                                                                const float* maxV, unsigned* out, int outType,
                                                                int fromData) {
  const float mn = *minV, mx = *maxV;
  const IntRange r = int_range(outType);
  const bool fillLowest = fromData ? (mn == mx) : (mn >= mx);
  double scale = 0;
  long long offset = 0;
  if (!fillLowest) quantized_scale_info(r.bits, mn, mx, &scale, &offset);
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total4; i += 4 * step) {
    float4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (i + u * step < total4) v[u] = load_streamed(in + i + u * step);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (i + u * step >= total4) continue;
      const float x[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
      unsigned word = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        long long q = r.lowest;
        if (!fillLowest) {
          q = to_int64_x86(rint((double)x[e] * scale));
          q = (long long)((unsigned long long)q - (unsigned long long)offset + (unsigned long long)r.lowest);
          q = q < r.lowest ? r.lowest : q;
          q = q > r.highest ? r.highest : q;
        }
        word |= ((unsigned)q & 0xffu) << (8 * e);
      }
      out[i + u * step] = word;
    }
  }
}

// min / max of a float tensor.  Monotone uint encoding so that unsigned atomics order floats.
__device__ __forceinline__ unsigned enc(float f) {
  unsigned u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float dec(unsigned u) {
  return __uint_as_float((u & 0x80000000u) ? (u & 0x7fffffffu) : ~u);
}

// The running minimum / maximum live, order-encoded as unsigned words, in the caller's own result words
// until the finish kernel decodes them in place: no scratch memory that calls on other streams could share.
__global__ void minmax_init_kernel(unsigned* mnWord, unsigned* mxWord) {
  *mnWord = 0xffffffffu;
  *mxWord = 0u;
}

__global__ __launch_bounds__(256) void minmax_kernel(const float* in, size_t total, unsigned* mnWord,
                                                     unsigned* mxWord) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t step = (size_t)gridDim.x * blockDim.x;
  float mn = 3.402823466e+38f, mx = -3.402823466e+38f;
  for (; i < total; i += step) {
    float v = in[i];
    mn = fminf(mn, v);
    mx = fmaxf(mx, v);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    mn = fminf(mn, __shfl_down(mn, off, 64));
    mx = fmaxf(mx, __shfl_down(mx, off, 64));
  }
  if ((threadIdx.x & 63) == 0) {
    atomicMin(mnWord, enc(mn));
    atomicMax(mxWord, enc(mx));
  }
}

// The same reduction without atomics for tensors large enough to matter: every workgroup leaves its minimum
// and maximum in the (not yet written) output buffer of the quantize call, one more workgroup reduces those.
// 65536 atomics on two words took 380 us for 16.7 M floats; this takes the time of reading them once.
__global__ __launch_bounds__(256) void minmax_partial_kernel(const float* in, size_t total, float* partials) {
  __shared__ float shMn[4], shMx[4];
  const size_t total4 = total / 4, step = (size_t)gridDim.x * blockDim.x;
  const float4* in4 = reinterpret_cast<const float4*>(in);
  float mn = 3.402823466e+38f, mx = -3.402823466e+38f;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total4; i += 4 * step) {
    float4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (i + u * step < total4) v[u] = load_streamed(in4 + i + u * step);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (i + u * step >= total4) continue;
      mn = fminf(fminf(mn, fminf(v[u].x, v[u].y)), fminf(v[u].z, v[u].w));
      mx = fmaxf(fmaxf(mx, fmaxf(v[u].x, v[u].y)), fmaxf(v[u].z, v[u].w));
    }
  }
  if (blockIdx.x == 0 && threadIdx.x < total - total4 * 4) {  // the last 1..3 elements
    const float v = in[total4 * 4 + threadIdx.x];
    mn = fminf(mn, v);
    mx = fmaxf(mx, v);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    mn = fminf(mn, __shfl_down(mn, off, 64));
    mx = fmaxf(mx, __shfl_down(mx, off, 64));
  }
  if ((threadIdx.x & 63) == 0) {
    shMn[threadIdx.x >> 6] = mn;
    shMx[threadIdx.x >> 6] = mx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    partials[2 * blockIdx.x] = fminf(fminf(shMn[0], shMn[1]), fminf(shMn[2], shMn[3]));
    partials[2 * blockIdx.x + 1] = fmaxf(fmaxf(shMx[0], shMx[1]), fmaxf(shMx[2], shMx[3]));
  }
}

__global__ __launch_bounds__(256) void minmax_final_kernel(const float* partials, unsigned blocks, float* mnOut,
                                                           float* mxOut) {
  __shared__ float shMn[4], shMx[4];
  float mn = 3.402823466e+38f, mx = -3.402823466e+38f;
  for (unsigned i = threadIdx.x; i < blocks; i += 256) {
    mn = fminf(mn, partials[2 * i]);
    mx = fmaxf(mx, partials[2 * i + 1]);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    mn = fminf(mn, __shfl_down(mn, off, 64));
    mx = fmaxf(mx, __shfl_down(mx, off, 64));
  }
  if ((threadIdx.x & 63) == 0) {
    shMn[threadIdx.x >> 6] = mn;
    shMx[threadIdx.x >> 6] = mx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    *mnOut = fminf(fminf(shMn[0], shMn[1]), fminf(shMn[2], shMn[3]));
    *mxOut = fmaxf(fmaxf(shMx[0], shMx[1]), fmaxf(shMx[2], shMx[3]));
  }
}

__global__ void minmax_finish_kernel(float* mn, float* mx) {
  *mn = dec(*reinterpret_cast<const unsigned*>(mn));
  *mx = dec(*reinterpret_cast<const unsigned*>(mx));
}

unsigned grid_for(size_t total, unsigned perThread = 1) {
  size_t blocks = (total + 256ull * perThread - 1) / (256ull * perThread);
  if (blocks > 256u * 32u) blocks = 256u * 32u;
  if (blocks < 1) blocks = 1;
  return (unsigned)blocks;
}

// the vector kernels: four 16-byte loads per thread per pass, at most 8 workgroups per CU
unsigned stream_grid(size_t total4) {
  size_t blocks = (total4 + 1023) / 1024;
  if (blocks > 256u * 8u) blocks = 256u * 8u;
  if (blocks < 1) blocks = 1;
  return (unsigned)blocks;
}

bool valid_type(int t) { return t >= TFCC_ROCM_S8 && t <= TFCC_ROCM_U32; }

void launch_quantize(hipStream_t s, const float* in, uint64_t total, const float* minV, const float* maxV, void* out,
                     int outType, int fromData) {
  if ((outType == TFCC_ROCM_U8 || outType == TFCC_ROCM_S8) && total % 4 == 0 && (uintptr_t)in % 16 == 0 &&
      (uintptr_t)out % 4 == 0) {
    hipLaunchKernelGGL(quantize_8bit_vec_kernel, dim3(stream_grid(total / 4)), dim3(256), 0, s,
                       reinterpret_cast<const float4*>(in), (size_t)(total / 4), minV, maxV, static_cast<unsigned*>(out),
                       outType, fromData);
  } else {
    hipLaunchKernelGGL(quantize_kernel, dim3(grid_for(total)), dim3(256), 0, s, in, (size_t)total, minV, maxV, out,
                       outType, fromData);
  }
}

template <class T>
int reduce_rows(hipStream_t s, const void* a, unsigned batch, unsigned row, unsigned col, int* out) {
  unsigned long long rows = (unsigned long long)batch * row;
  if (rows >= (1ull << 31)) return set_error(TFCC_ROCM_INVALID_ARGUMENT, "reduce_sum: too many rows");
  unsigned blocks = (unsigned)((rows + 3) / 4);
  hipLaunchKernelGGL(reduce_rows_kernel<T>, dim3(blocks), dim3(256), 0, s, static_cast<const T*>(a),
                     (unsigned)rows, col, out);
  return check_launch("reduce_sum rows");
}

template <class T>
int reduce_cols(hipStream_t s, const void* a, unsigned batch, unsigned row, unsigned col, int* out) {
  size_t n = (size_t)batch * col;
  hipLaunchKernelGGL(zero_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, out, n);
  if (int e = check_launch("reduce_sum cols (zero)")) return e;
  if (batch > 65535) return set_error(TFCC_ROCM_INVALID_ARGUMENT, "reduce_sum: batch too large");
  if constexpr (sizeof(T) == 1) {
    if (col % 16 == 0 && (uintptr_t)a % 16 == 0 && row >= 64) {
      // slabs of at least 64 rows (sixteen 16-byte loads per thread), about a thousand workgroups where the
      // matrix is large enough
      const unsigned wideBlocks = (col / 16 + 63) / 64;
      unsigned wideSlabs = (1024 + wideBlocks * batch - 1) / (wideBlocks * batch);
      if (wideSlabs > row / 64) wideSlabs = row / 64;
      if (wideSlabs < 1) wideSlabs = 1;
      if (wideSlabs > 65535) wideSlabs = 65535;
      unsigned perSlab = (row + wideSlabs - 1) / wideSlabs;
      perSlab = (perSlab + 15) / 16 * 16;  // whole rounds of the four row lanes' four rows
      wideSlabs = (row + perSlab - 1) / perSlab;
      hipLaunchKernelGGL(reduce_cols_wide_kernel<T>, dim3(wideBlocks, wideSlabs, batch), dim3(256), 0, s,
                         static_cast<const T*>(a), row, col, perSlab, out);
      return check_launch("reduce_sum cols");
    }
  }
  const bool vec = sizeof(T) == 1 && col % 4 == 0 && (uintptr_t)a % 4 == 0;
  const unsigned colBlocks = vec ? (col / 4 + 255) / 256 : (col + 255) / 256;
  // enough row slabs for ~2048 workgroups
  unsigned slabs = (2048 + colBlocks * batch - 1) / (colBlocks * batch);
  if (slabs > (row + 31) / 32) slabs = (row + 31) / 32;
  if (slabs < 1) slabs = 1;
  if (slabs > 65535) slabs = 65535;
  const unsigned rowsPerSlab = (row + slabs - 1) / slabs;
  slabs = (row + rowsPerSlab - 1) / rowsPerSlab;
  if (vec)
    hipLaunchKernelGGL(reduce_cols_vec_kernel<T>, dim3(colBlocks, slabs, batch), dim3(256), 0, s,
                       static_cast<const T*>(a), row, col, rowsPerSlab, out);
  else
    hipLaunchKernelGGL(reduce_cols_kernel<T>, dim3(colBlocks, slabs, batch), dim3(256), 0, s,
                       static_cast<const T*>(a), row, col, rowsPerSlab, out);
  return check_launch("reduce_sum cols");
}

}  // namespace
}  // namespace tfcc_rocm

using namespace tfcc_rocm;

extern "C" {

int tfcc_rocm_reduce_sum_rows(void* stream, const void* a, int type, unsigned batch, unsigned row,
                              unsigned col, int32_t* out) {
  TFCC_REQUIRE(a && out, "reduce_sum: null argument");
  TFCC_REQUIRE(batch > 0 && row > 0 && col > 0, "reduce_sum: empty tensor");
  switch (type) {
    case TFCC_ROCM_S8: return reduce_rows<int8_t>(as_stream(stream), a, batch, row, col, out);
    case TFCC_ROCM_U8: return reduce_rows<uint8_t>(as_stream(stream), a, batch, row, col, out);
    case TFCC_ROCM_S16: return reduce_rows<int16_t>(as_stream(stream), a, batch, row, col, out);
  }
  return set_error(TFCC_ROCM_INVALID_ARGUMENT, "reduce_sum: type %d (int8, uint8 or int16)", type);
}

int tfcc_rocm_reduce_sum_cols(void* stream, const void* a, int type, unsigned batch, unsigned row,
                              unsigned col, int32_t* out) {
  TFCC_REQUIRE(a && out, "reduce_sum: null argument");
  TFCC_REQUIRE(batch > 0 && row > 0 && col > 0, "reduce_sum: empty tensor");
  switch (type) {
    case TFCC_ROCM_S8: return reduce_cols<int8_t>(as_stream(stream), a, batch, row, col, out);
    case TFCC_ROCM_U8: return reduce_cols<uint8_t>(as_stream(stream), a, batch, row, col, out);
    case TFCC_ROCM_S16: return reduce_cols<int16_t>(as_stream(stream), a, batch, row, col, out);
  }
  return set_error(TFCC_ROCM_INVALID_ARGUMENT, "reduce_sum: type %d (int8, uint8 or int16)", type);
}

int tfcc_rocm_requantize(void* stream, const void* in, int in_type, void* out, int out_type,
                         uint64_t total, const float* min_in, const float* max_in,
                         const float* min_out, const float* max_out) {
  TFCC_REQUIRE(in && out && min_in && max_in && min_out && max_out, "requantize: null argument");
  TFCC_REQUIRE(total > 0, "requantize: empty tensor");
  TFCC_REQUIRE(valid_type(in_type) && valid_type(out_type), "requantize: bad type code");
  hipStream_t s = as_stream(stream);
  if (in_type == TFCC_ROCM_S32 && out_type == TFCC_ROCM_U8 && total % 4 == 0 && (uintptr_t)in % 16 == 0 &&
      (uintptr_t)out % 4 == 0) {
    hipLaunchKernelGGL(requantize_s32_u8_vec_kernel, dim3(stream_grid(total / 4)), dim3(256), 0, s,
                       static_cast<const int4*>(in), static_cast<unsigned*>(out), (size_t)(total / 4), min_in,
                       max_in, min_out, max_out);
  } else {
    hipLaunchKernelGGL(requantize_kernel, dim3(grid_for(total)), dim3(256), 0, s, in, in_type, out, out_type,
                       (size_t)total, min_in, max_in, min_out, max_out);
  }
  return check_launch("requantize");
}

int tfcc_rocm_dequantize(void* stream, const void* in, int in_type, uint64_t total,
                         const float* min_v, const float* max_v, float* out) {
  TFCC_REQUIRE(in && out && min_v && max_v, "dequantize: null argument");
  TFCC_REQUIRE(total > 0, "dequantize: empty tensor");
  TFCC_REQUIRE(valid_type(in_type), "dequantize: bad type code");
  if (in_type == TFCC_ROCM_S32 && total % 4 == 0 && (uintptr_t)in % 16 == 0 && (uintptr_t)out % 16 == 0) {
    hipLaunchKernelGGL(dequantize_s32_vec_kernel, dim3(stream_grid(total / 4)), dim3(256), 0, as_stream(stream),
                       static_cast<const int4*>(in), (size_t)(total / 4), min_v, max_v, reinterpret_cast<float4*>(out));
  } else {
    hipLaunchKernelGGL(dequantize_kernel, dim3(grid_for(total)), dim3(256), 0, as_stream(stream), in, in_type,
                       (size_t)total, min_v, max_v, out);
  }
  return check_launch("dequantize");
}

int tfcc_rocm_quantize(void* stream, const float* in, uint64_t total, const float* min_v,
                       const float* max_v, void* out, int out_type) {
  TFCC_REQUIRE(in && out && min_v && max_v, "quantize: null argument");
  TFCC_REQUIRE(total > 0, "quantize: empty tensor");
  TFCC_REQUIRE(valid_type(out_type), "quantize: bad type code");
  launch_quantize(as_stream(stream), in, total, min_v, max_v, out, out_type, 0);
  return check_launch("quantize");
}

int tfcc_rocm_quantize_minmax(void* stream, const float* in, uint64_t total, void* out,
                              int out_type, float* min_v, float* max_v) {
  TFCC_REQUIRE(in && out && min_v && max_v, "quantize: null argument");
  TFCC_REQUIRE(total > 0, "quantize: empty tensor");
  TFCC_REQUIRE(valid_type(out_type), "quantize: bad type code");
  hipStream_t s = as_stream(stream);
  unsigned* mnWord = reinterpret_cast<unsigned*>(min_v);
  unsigned* mxWord = reinterpret_cast<unsigned*>(max_v);
  const IntRange range = int_range(out_type);
  const size_t outBytes = (size_t)total * (range.bits / 8);
  const unsigned blocks = stream_grid(total / 4);
  if ((uintptr_t)in % 16 == 0 && (uintptr_t)out % 4 == 0 && outBytes >= (size_t)blocks * 8 && total >= 4096) {
    // partial results rest in the output buffer until the quantize pass overwrites it
    float* partials = static_cast<float*>(out);
    hipLaunchKernelGGL(minmax_partial_kernel, dim3(blocks), dim3(256), 0, s, in, (size_t)total, partials);
    hipLaunchKernelGGL(minmax_final_kernel, dim3(1), dim3(256), 0, s, partials, blocks, min_v, max_v);
  } else {
    hipLaunchKernelGGL(minmax_init_kernel, dim3(1), dim3(1), 0, s, mnWord, mxWord);
    hipLaunchKernelGGL(minmax_kernel, dim3(grid_for(total, 4)), dim3(256), 0, s, in, (size_t)total, mnWord, mxWord);
    hipLaunchKernelGGL(minmax_finish_kernel, dim3(1), dim3(1), 0, s, min_v, max_v);
  }
  launch_quantize(s, in, total, min_v, max_v, out, out_type, 1);
  return check_launch("quantize");
}

}  // extern "C"
