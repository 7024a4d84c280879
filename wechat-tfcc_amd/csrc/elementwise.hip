// The fp32 element-wise / row-wise neighbours of matmul in one transformer encoder layer, so that
// the layer's tensors stay resident on the GPU between the matrix products.  All are bandwidth
// bound: one pass over the data, a wavefront (or workgroup) per row for the row-wise ones.
//
// Numerics follow the reference's scalar MKL kernels:
//   softmax     tfcc/mkl/kernel/tfcc_mklactivationkernel.hpp:137-155  exp(x - max) / sum
//   layer norm  tfcc/mkl/interfaces/tfcc_mklnormalizationinterface.cpp:29-62  two-pass mean / variance,
//               1/sqrt(var + eps), (x - mean) * (inv * gamma) + beta
//   gelu        tfcc/mkl/kernel/tfcc_mklactivationkernel.hpp:213-220  0.5 x (1 + erf(x / sqrt 2))
//   transform   tfcc/core/operations/tfcc_operator.cpp:78-95  a * alpha + beta
//   add         tfcc/core/operations/tfcc_math.cpp:38-104 (trailing-dims broadcast only)
//   transpose   tfcc/core/operations/tfcc_base.cpp:124-134
#include "common.hpp"

namespace tfcc_rocm {
namespace {


// block-wide reductions for rows handled by a whole workgroup
template <bool MAX>
__device__ __forceinline__ float block_reduce(float v, float* sh) {
  v = MAX ? wave_max(v) : wave_sum(v);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  __syncthreads();
  if (lane == 0) sh[wave] = v;
  __syncthreads();
  float r = sh[0];
  for (int i = 1; i < nw; ++i) r = MAX ? fmaxf(r, sh[i]) : r + sh[i];
  return r;
}

// one workgroup of 256 threads per row
__global__ __launch_bounds__(256) void softmax_kernel(const float* in, unsigned cols, float divisor, bool divide,
                                                      float* out) {
  __shared__ float sh[4];
  const float* a = in + (size_t)blockIdx.x * cols;
  float* o = out + (size_t)blockIdx.x * cols;
  float mx = -3.402823466e+38f;
  for (unsigned i = threadIdx.x; i < cols; i += 256) mx = fmaxf(mx, divide ? a[i] / divisor : a[i]);
  mx = block_reduce<true>(mx, sh);
  float s = 0.f;
  for (unsigned i = threadIdx.x; i < cols; i += 256) {
    float e = softmax_exp((divide ? a[i] / divisor : a[i]) - mx);
    o[i] = e;
    s += e;
  }
  s = block_reduce<false>(s, sh);
  const float inverse = 1.0f / s;  // one division per row, a multiplication per value
  for (unsigned i = threadIdx.x; i < cols; i += 256) o[i] = o[i] * inverse;
}

// rows of at most 256 columns: one wavefront per row, values stay in registers
__global__ __launch_bounds__(256) void softmax_small_kernel(const float* in, size_t rows, unsigned cols, float divisor,
                                                            bool divide, float* out) {
  const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  const float* a = in + row * cols;
  float* o = out + row * cols;
  float v[4];
  float mx = -3.402823466e+38f;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    unsigned i = lane + 64 * q;
    v[q] = i < cols ? (divide ? a[i] / divisor : a[i]) : -3.402823466e+38f;
    mx = fmaxf(mx, v[q]);
  }
  mx = wave_max(mx);
  float s = 0.f;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    unsigned i = lane + 64 * q;
    v[q] = i < cols ? softmax_exp(v[q] - mx) : 0.f;
    s += v[q];
  }
  s = wave_sum(s);
  const float inverse = 1.0f / s;  // one division per row, a multiplication per value
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    unsigned i = lane + 64 * q;
    if (i < cols) o[i] = v[q] * inverse;
  }
}

__global__ __launch_bounds__(256) void layer_norm_kernel(const float* in, const float* gamma, const float* beta,
                                                         float eps, unsigned cols, float* out) {
  __shared__ float sh[4];
  const float* a = in + (size_t)blockIdx.x * cols;
  float* o = out + (size_t)blockIdx.x * cols;
  float s = 0.f;
  for (unsigned i = threadIdx.x; i < cols; i += 256) s += a[i];
  const float mean = block_reduce<false>(s, sh) / (float)cols;
  float v = 0.f;
  for (unsigned i = threadIdx.x; i < cols; i += 256) {
    float t = a[i] - mean;
    v += t * t;
  }
  const float var = block_reduce<false>(v, sh) / (float)cols;
  const float inv = 1.0f / sqrtf(var + eps);
  for (unsigned i = threadIdx.x; i < cols; i += 256) o[i] = (a[i] - mean) * (inv * gamma[i]) + beta[i];
}

// rows of at most 256 * PER columns: the row, gamma and beta are read once and stay in registers (same sums
// in the same order as the kernel above)
template <int PER>
__global__ __launch_bounds__(256) void layer_norm_reg_kernel(const float* in, const float* gamma, const float* beta,
                                                             float eps, unsigned cols, float* out) {
  __shared__ float sh[4];
  const float* a = in + (size_t)blockIdx.x * cols;
  float* o = out + (size_t)blockIdx.x * cols;
  float x[PER], gm[PER], bt[PER];
#pragma unroll
  for (int q = 0; q < PER; ++q) {
    const unsigned i = threadIdx.x + 256 * q;
    x[q] = i < cols ? a[i] : 0.f;
    gm[q] = i < cols ? gamma[i] : 0.f;
    bt[q] = i < cols ? beta[i] : 0.f;
  }
  float s = 0.f;
#pragma unroll
  for (int q = 0; q < PER; ++q)
    if (threadIdx.x + 256 * q < cols) s += x[q];
  const float mean = block_reduce<false>(s, sh) / (float)cols;
  float v = 0.f;
#pragma unroll
  for (int q = 0; q < PER; ++q)
    if (threadIdx.x + 256 * q < cols) {
      float t = x[q] - mean;
      v += t * t;
    }
  const float var = block_reduce<false>(v, sh) / (float)cols;
  const float inv = 1.0f / sqrtf(var + eps);
#pragma unroll
  for (int q = 0; q < PER; ++q) {
    const unsigned i = threadIdx.x + 256 * q;
    if (i < cols) o[i] = (x[q] - mean) * (inv * gm[q]) + bt[q];
  }
}

__global__ __launch_bounds__(256) void gelu_kernel(const float* in, size_t total, float* out) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (; i < total; i += step) {
    float v = in[i];
    out[i] = gelu_erf_f32(v);
  }
}

__global__ __launch_bounds__(256) void transform_kernel(const float* in, size_t total, float alpha, float beta,
                                                        float* out) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (; i < total; i += step) out[i] = in[i] * alpha + beta;
}

__global__ __launch_bounds__(256) void transform2_kernel(const float* in, size_t total, float alpha, float beta,
                                                         float* out) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (; i < total; i += step) out[i] = in[i] / alpha + beta;
}

// OP: 0 a + b, 1 a - b, 2 a * b, 3 a / b; b repeats with `period`
template <int OP>
__global__ __launch_bounds__(256) void binary_kernel(const float* a, const float* b, size_t total, size_t period,
                                                     float* out) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (; i < total; i += step) {
    const float x = a[i], y = b[period == total ? i : i % period];
    out[i] = OP == 0 ? x + y : OP == 1 ? x - y : OP == 2 ? x * y : x / y;
  }
}

// Reductions over the trailing dimensions (rows x cols -> rows): sum, mean, product, maximum, minimum
// (tfcc/mkl/interfaces/tfcc_mklreduceinterface.cpp:107-230).  A wavefront per row up to 4096 columns, a workgroup
// per row beyond; partial results meet through lane shuffles (and LDS), in a fixed order.
template <int OP>
__device__ __forceinline__ float reduce_identity() {
  return OP == TFCC_ROCM_REDUCE_PROD ? 1.f : OP == TFCC_ROCM_REDUCE_MAX ? -INFINITY : OP == TFCC_ROCM_REDUCE_MIN ? INFINITY : 0.f;
}
template <int OP>
__device__ __forceinline__ float reduce_join(float a, float b) {
  return OP == TFCC_ROCM_REDUCE_PROD ? a * b : OP == TFCC_ROCM_REDUCE_MAX ? ref_max(a, b) : OP == TFCC_ROCM_REDUCE_MIN ? ref_min(a, b) : a + b;
}
template <int OP>
__device__ __forceinline__ float wave_join(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = reduce_join<OP>(v, __shfl_xor(v, off, 64));
  return v;
}

template <int OP, bool BLOCK>
__global__ __launch_bounds__(256) void reduce_trailing_kernel(const float* in, size_t rows, unsigned cols, float* out) {
  __shared__ float sh[4];
  const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const size_t row = BLOCK ? blockIdx.x : (size_t)blockIdx.x * 4 + wave;
  if (!BLOCK && row >= rows) return;
  const float* a = in + row * cols;
  float v = reduce_identity<OP>();
  for (unsigned i = BLOCK ? threadIdx.x : lane; i < cols; i += BLOCK ? 256 : 64) v = reduce_join<OP>(v, a[i]);
  v = wave_join<OP>(v);
  if (BLOCK) {
    if (lane == 0) sh[wave] = v;
    __syncthreads();
    v = reduce_join<OP>(reduce_join<OP>(sh[0], sh[1]), reduce_join<OP>(sh[2], sh[3]));
  }
  if (OP == TFCC_ROCM_REDUCE_MEAN) v = v / (float)cols;
  if (BLOCK ? threadIdx.x == 0 : lane == 0) out[row] = v;
}

// More element-wise functions of two tensors of one shape (op 4 pow, 5 max, 6 min) and of one tensor with scalars
// (clip: max(min(v, hi), lo); leaky relu: max(v, alpha * v)): tfcc/mkl/kernel/tfcc_mklactivationkernel.hpp, tfcc_math.h.
template <int OP>
__global__ __launch_bounds__(256) void binary2_kernel(const float* a, const float* b, size_t total, size_t period, float* out) {
  const size_t step = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += step) {
    const float x = a[i], y = b[period == total ? i : i % period];
    out[i] = OP == 4 ? powf(x, y) : OP == 5 ? ref_max(x, y) : ref_min(x, y);
  }
}
template <int OP>
__global__ __launch_bounds__(256) void scalar2_kernel(const float* a, size_t total, float p0, float p1, float* out) {
  const size_t step = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += step) {
    const float v = a[i];
    // clip: min(v, hi) first, then max(., lo), as the reference; leaky relu: max(v, alpha * v)
    out[i] = OP == 0 ? ref_max(ref_min(v, p1), p0) : ref_max(v, p0 * v);
  }
}

// The general numpy-style broadcast: every dimension has the output's extent on one side or both, the other side's
// stride is 0 there.
struct BroadcastParams {
  unsigned dims[6];
  unsigned long long strideA[6], strideB[6];
  int rank;
};

template <int OP>
__global__ __launch_bounds__(256) void binary_broadcast_kernel(const float* a, const float* b, size_t total,
                                                               BroadcastParams p, float* out) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (; i < total; i += step) {
    size_t rem = i, ia = 0, ib = 0;
    for (int d = p.rank - 1; d >= 0; --d) {
      const size_t c = rem % p.dims[d];
      rem /= p.dims[d];
      ia += c * p.strideA[d];
      ib += c * p.strideB[d];
    }
    const float x = a[ia], y = b[ib];
    out[i] = OP == 0   ? x + y
             : OP == 1 ? x - y
             : OP == 2 ? x * y
             : OP == 3 ? x / y
             : OP == 4 ? powf(x, y)
             : OP == 5 ? ref_max(x, y)
                       : ref_min(x, y);
  }
}

struct TransposeParams {
  unsigned outShape[6];
  unsigned long long inStride[6];  // input stride of each OUTPUT dim
  int rank;
};

__global__ __launch_bounds__(256) void transpose_kernel(const float* in, size_t total, TransposeParams p, float* out) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (; i < total; i += step) {
    size_t rem = i, src = 0;
    for (int d = p.rank - 1; d >= 0; --d) {
      size_t c = rem % p.outShape[d];
      rem /= p.outShape[d];
      src += c * p.inStride[d];
    }
    out[i] = in[src];
  }
}

// batched 2-D transpose of the last two dims through LDS (both sides coalesced)
__global__ __launch_bounds__(256) void transpose_last2_kernel(const float* in, unsigned rows, unsigned cols, float* out) {
  __shared__ float tile[32][33];
  const size_t b = blockIdx.z;
  const float* a = in + b * (size_t)rows * cols;
  float* o = out + b * (size_t)rows * cols;
  const unsigned c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
  const unsigned tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
  for (unsigned y = ty; y < 32; y += 8)
    if (r0 + y < rows && c0 + tx < cols) tile[y][tx] = a[(size_t)(r0 + y) * cols + c0 + tx];
  __syncthreads();
  for (unsigned y = ty; y < 32; y += 8)
    if (c0 + y < cols && r0 + tx < rows) o[(size_t)(c0 + y) * rows + r0 + tx] = tile[tx][y];
}

unsigned grid_for(size_t total) {
  size_t blocks = (total + 255) / 256;
  if (blocks > 256u * 32u) blocks = 256u * 32u;
  if (blocks < 1) blocks = 1;
  return (unsigned)blocks;
}

// Element-wise functions of one tensor, each with the expression of the reference's float kernel
// (tfcc/mkl/kernel/tfcc_mklactivationkernel.hpp:48-110,222-228,284-291; neg, reciprocal and sqrt as
// tfcc_runtime/operations/math/neg.cpp:30, reciprocal.cpp:31 and sqrt.cpp:31 compose them).
template <int OP>
__device__ __forceinline__ float unary_value(float v) {
  if (OP == TFCC_ROCM_UNARY_SIGMOID) return 1.f / (1.f + expf(0.f - v));
  if (OP == TFCC_ROCM_UNARY_TANH) return tanhf(v);
  if (OP == TFCC_ROCM_UNARY_RELU) return ref_max(v, 0.f);
  if (OP == TFCC_ROCM_UNARY_SOFTPLUS) return logf(expf(v) + 1.f);
  if (OP == TFCC_ROCM_UNARY_LOG) return logf(v);
  if (OP == TFCC_ROCM_UNARY_RSQRT) return 1.f / sqrtf(v);
  if (OP == TFCC_ROCM_UNARY_ERF) return erff(v);
  if (OP == TFCC_ROCM_UNARY_ABS) return fabsf(v);
  if (OP == TFCC_ROCM_UNARY_SIGN) return v < 0.f ? -1.f : (v > 0.f ? 1.f : 0.f);
  if (OP == TFCC_ROCM_UNARY_NEG) return 0.f - v;
  if (OP == TFCC_ROCM_UNARY_RECIPROCAL) return 1.f / v;
  return 1.f / (1.f / sqrtf(v));  // TFCC_ROCM_UNARY_SQRT: 1 / rsqrt(v), rounded twice like the composition
}

template <int OP>
__global__ __launch_bounds__(256) void unary_kernel(const float* in, size_t total, float* out) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) out[i] = unary_value<OP>(in[i]);
}

}  // namespace
}  // namespace tfcc_rocm

using namespace tfcc_rocm;

extern "C" {

static int softmax_launch(void* stream, const float* in, uint64_t rows, unsigned cols, float divisor, bool divide,
                          float* out) {
  TFCC_REQUIRE(in && out, "softmax: null argument");
  TFCC_REQUIRE(rows > 0 && cols > 0, "softmax: empty tensor");
  TFCC_REQUIRE(rows < (1ull << 31), "softmax: too many rows");
  if (cols <= 256)
    hipLaunchKernelGGL(softmax_small_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, as_stream(stream), in,
                       (size_t)rows, cols, divisor, divide, out);
  else
    hipLaunchKernelGGL(softmax_kernel, dim3((unsigned)rows), dim3(256), 0, as_stream(stream), in, cols, divisor, divide,
                       out);
  return check_launch("softmax");
}

int tfcc_rocm_softmax_f32(void* stream, const float* in, uint64_t rows, unsigned cols, float* out) {
  return softmax_launch(stream, in, rows, cols, 1.f, false, out);
}

int tfcc_rocm_softmax_div_f32(void* stream, const float* in, uint64_t rows, unsigned cols, float divisor, float* out) {
  return softmax_launch(stream, in, rows, cols, divisor, true, out);
}

int tfcc_rocm_layer_norm_f32(void* stream, const float* in, const float* gamma, const float* beta,
                             float epsilon, uint64_t rows, unsigned cols, float* out) {
  TFCC_REQUIRE(in && gamma && beta && out, "layer_norm: null argument");
  TFCC_REQUIRE(rows > 0 && cols > 0, "layer_norm: empty tensor");
  TFCC_REQUIRE(rows < (1ull << 31), "layer_norm: too many rows");
  if (cols <= 256 * 4)
    hipLaunchKernelGGL(layer_norm_reg_kernel<4>, dim3((unsigned)rows), dim3(256), 0, as_stream(stream), in, gamma, beta,
                       epsilon, cols, out);
  else
    hipLaunchKernelGGL(layer_norm_kernel, dim3((unsigned)rows), dim3(256), 0, as_stream(stream), in, gamma, beta,
                       epsilon, cols, out);
  return check_launch("layer_norm");
}

int tfcc_rocm_gelu_accurate_f32(void* stream, const float* in, uint64_t total, float* out) {
  TFCC_REQUIRE(in && out, "gelu: null argument");
  TFCC_REQUIRE(total > 0, "gelu: empty tensor");
  hipLaunchKernelGGL(gelu_kernel, dim3(grid_for(total)), dim3(256), 0, as_stream(stream), in, (size_t)total, out);
  return check_launch("gelu");
}

int tfcc_rocm_transform_f32(void* stream, const float* in, uint64_t total, float alpha, float beta, float* out) {
  TFCC_REQUIRE(in && out, "transform: null argument");
  TFCC_REQUIRE(total > 0, "transform: empty tensor");
  hipLaunchKernelGGL(transform_kernel, dim3(grid_for(total)), dim3(256), 0, as_stream(stream), in, (size_t)total,
                     alpha, beta, out);
  return check_launch("transform");
}

int tfcc_rocm_transform2_f32(void* stream, const float* in, uint64_t total, float alpha, float beta, float* out) {
  TFCC_REQUIRE(in && out, "transform2: null argument");
  TFCC_REQUIRE(total > 0, "transform2: empty tensor");
  hipLaunchKernelGGL(transform2_kernel, dim3(grid_for(total)), dim3(256), 0, as_stream(stream), in, (size_t)total,
                     alpha, beta, out);
  return check_launch("transform2");
}

int tfcc_rocm_binary_f32(void* stream, int op, const float* a, const float* b, uint64_t total, uint64_t period,
                         float* out) {
  TFCC_REQUIRE(a && b && out, "binary: null argument");
  TFCC_REQUIRE(op >= 0 && op <= 6, "binary: unknown op %d", op);
  TFCC_REQUIRE(total > 0 && period > 0 && period <= total && total % period == 0, "binary: bad broadcast period");
  const dim3 grid(grid_for(total)), block(256);
  hipStream_t s = as_stream(stream);
  switch (op) {
    case 0: hipLaunchKernelGGL(binary_kernel<0>, grid, block, 0, s, a, b, (size_t)total, (size_t)period, out); break;
    case 1: hipLaunchKernelGGL(binary_kernel<1>, grid, block, 0, s, a, b, (size_t)total, (size_t)period, out); break;
    case 2: hipLaunchKernelGGL(binary_kernel<2>, grid, block, 0, s, a, b, (size_t)total, (size_t)period, out); break;
    case 3: hipLaunchKernelGGL(binary_kernel<3>, grid, block, 0, s, a, b, (size_t)total, (size_t)period, out); break;
    case 4: hipLaunchKernelGGL(binary2_kernel<4>, grid, block, 0, s, a, b, (size_t)total, (size_t)period, out); break;
    case 5: hipLaunchKernelGGL(binary2_kernel<5>, grid, block, 0, s, a, b, (size_t)total, (size_t)period, out); break;
    default: hipLaunchKernelGGL(binary2_kernel<6>, grid, block, 0, s, a, b, (size_t)total, (size_t)period, out); break;
  }
  return check_launch("binary");
}

int tfcc_rocm_reduce_f32(void* stream, int op, const float* in, uint64_t rows, unsigned cols, float* out) {
  TFCC_REQUIRE(in && out, "reduce: null argument");
  TFCC_REQUIRE(rows > 0 && cols > 0, "reduce: empty tensor");
  TFCC_REQUIRE(rows < (1ull << 31), "reduce: too many rows");
  hipStream_t s = as_stream(stream);
  const bool block = cols > 4096;
  const dim3 grid(block ? (unsigned)rows : (unsigned)((rows + 3) / 4)), threads(256);
#define TFCC_REDUCE_CASE(OP)                                                                                        \
  case OP:                                                                                                          \
    if (block) hipLaunchKernelGGL((reduce_trailing_kernel<OP, true>), grid, threads, 0, s, in, (size_t)rows, cols, out); \
    else hipLaunchKernelGGL((reduce_trailing_kernel<OP, false>), grid, threads, 0, s, in, (size_t)rows, cols, out);  \
    break;
  switch (op) {
    TFCC_REDUCE_CASE(TFCC_ROCM_REDUCE_SUM)
    TFCC_REDUCE_CASE(TFCC_ROCM_REDUCE_MEAN)
    TFCC_REDUCE_CASE(TFCC_ROCM_REDUCE_PROD)
    TFCC_REDUCE_CASE(TFCC_ROCM_REDUCE_MAX)
    TFCC_REDUCE_CASE(TFCC_ROCM_REDUCE_MIN)
    default: return set_error(TFCC_ROCM_INVALID_ARGUMENT, "reduce: unknown operation %d", op);
  }
#undef TFCC_REDUCE_CASE
  return check_launch("reduce");
}

int tfcc_rocm_clip_f32(void* stream, const float* in, uint64_t total, float lo, float hi, float* out) {
  TFCC_REQUIRE(in && out, "clip: null argument");
  TFCC_REQUIRE(total > 0, "clip: empty tensor");
  hipLaunchKernelGGL(scalar2_kernel<0>, dim3(grid_for(total)), dim3(256), 0, as_stream(stream), in, (size_t)total, lo, hi, out);
  return check_launch("clip");
}

int tfcc_rocm_leaky_relu_f32(void* stream, const float* in, uint64_t total, float alpha, float* out) {
  TFCC_REQUIRE(in && out, "leaky_relu: null argument");
  TFCC_REQUIRE(total > 0, "leaky_relu: empty tensor");
  hipLaunchKernelGGL(scalar2_kernel<1>, dim3(grid_for(total)), dim3(256), 0, as_stream(stream), in, (size_t)total, alpha, 0.f,
                     out);
  return check_launch("leaky_relu");
}

int tfcc_rocm_binary_broadcast_f32(void* stream, int op, const float* a, const float* b, int rank,
                                   const unsigned* dims, const uint64_t* stride_a, const uint64_t* stride_b, float* out) {
  TFCC_REQUIRE(a && b && out && dims && stride_a && stride_b, "binary_broadcast: null argument");
  TFCC_REQUIRE(op >= 0 && op <= 6, "binary_broadcast: unknown operation %d", op);
  TFCC_REQUIRE(rank >= 1 && rank <= 6, "binary_broadcast: rank %d (1..6)", rank);
  BroadcastParams p{};
  p.rank = rank;
  size_t total = 1;
  for (int d = 0; d < rank; ++d) {
    TFCC_REQUIRE(dims[d] > 0, "binary_broadcast: empty tensor");
    p.dims[d] = dims[d];
    p.strideA[d] = stride_a[d];
    p.strideB[d] = stride_b[d];
    total *= dims[d];
  }
  const dim3 grid(grid_for(total)), block(256);
  hipStream_t s = as_stream(stream);
  switch (op) {
    case 0: hipLaunchKernelGGL(binary_broadcast_kernel<0>, grid, block, 0, s, a, b, total, p, out); break;
    case 1: hipLaunchKernelGGL(binary_broadcast_kernel<1>, grid, block, 0, s, a, b, total, p, out); break;
    case 2: hipLaunchKernelGGL(binary_broadcast_kernel<2>, grid, block, 0, s, a, b, total, p, out); break;
    case 3: hipLaunchKernelGGL(binary_broadcast_kernel<3>, grid, block, 0, s, a, b, total, p, out); break;
    case 4: hipLaunchKernelGGL(binary_broadcast_kernel<4>, grid, block, 0, s, a, b, total, p, out); break;
    case 5: hipLaunchKernelGGL(binary_broadcast_kernel<5>, grid, block, 0, s, a, b, total, p, out); break;
    default: hipLaunchKernelGGL(binary_broadcast_kernel<6>, grid, block, 0, s, a, b, total, p, out); break;
  }
  return check_launch("binary_broadcast");
}

int tfcc_rocm_add_f32(void* stream, const float* a, const float* b, uint64_t total, uint64_t period, float* out) {
  return tfcc_rocm_binary_f32(stream, 0, a, b, total, period, out);
}

int tfcc_rocm_transpose_f32(void* stream, const float* in, const unsigned* shape, const unsigned* perm,
                            int rank, float* out) {
  TFCC_REQUIRE(in && out && shape && perm, "transpose: null argument");
  TFCC_REQUIRE(rank >= 1 && rank <= 6, "transpose: rank %d (1..6)", rank);
  bool seen[6] = {};
  size_t total = 1;
  for (int d = 0; d < rank; ++d) {
    TFCC_REQUIRE(perm[d] < (unsigned)rank && !seen[perm[d]], "transpose: perm is not a permutation");
    seen[perm[d]] = true;
    total *= shape[d];
  }
  TFCC_REQUIRE(total > 0, "transpose: empty tensor");
  // identity up to the last two dims swapped: tiled kernel
  bool last2 = rank >= 2 && perm[rank - 1] == (unsigned)rank - 2 && perm[rank - 2] == (unsigned)rank - 1;
  for (int d = 0; d + 2 < rank && last2; ++d) last2 = perm[d] == (unsigned)d;
  if (last2) {
    unsigned rows = shape[rank - 2], cols = shape[rank - 1];
    size_t batch = total / ((size_t)rows * cols);
    if (batch <= 65535 && (rows + 31) / 32 <= 65535) {
      hipLaunchKernelGGL(transpose_last2_kernel, dim3((cols + 31) / 32, (rows + 31) / 32, (unsigned)batch), dim3(256),
                         0, as_stream(stream), in, rows, cols, out);
      return check_launch("transpose");
    }
  }
  TransposeParams p{};
  p.rank = rank;
  unsigned long long stride[6];
  unsigned long long s = 1;
  for (int d = rank - 1; d >= 0; --d) {
    stride[d] = s;
    s *= shape[d];
  }
  for (int d = 0; d < rank; ++d) {
    p.outShape[d] = shape[perm[d]];
    p.inStride[d] = stride[perm[d]];
  }
  hipLaunchKernelGGL(transpose_kernel, dim3(grid_for(total)), dim3(256), 0, as_stream(stream), in, total, p, out);
  return check_launch("transpose");
}

int tfcc_rocm_unary_f32(void* stream, int op, const float* in, uint64_t total, float* out) {
  TFCC_REQUIRE(in && out, "unary: null argument");
  TFCC_REQUIRE(total > 0, "unary: empty tensor");
  hipStream_t s = as_stream(stream);
  const unsigned grid = grid_for(total);
#define TFCC_UNARY_CASE(OP) \
  case OP: hipLaunchKernelGGL(unary_kernel<OP>, dim3(grid), dim3(256), 0, s, in, (size_t)total, out); break;
  switch (op) {
    TFCC_UNARY_CASE(TFCC_ROCM_UNARY_SIGMOID)
    TFCC_UNARY_CASE(TFCC_ROCM_UNARY_TANH)
    TFCC_UNARY_CASE(TFCC_ROCM_UNARY_RELU)
    TFCC_UNARY_CASE(TFCC_ROCM_UNARY_SOFTPLUS)
    TFCC_UNARY_CASE(TFCC_ROCM_UNARY_LOG)
    TFCC_UNARY_CASE(TFCC_ROCM_UNARY_RSQRT)
    TFCC_UNARY_CASE(TFCC_ROCM_UNARY_ERF)
    TFCC_UNARY_CASE(TFCC_ROCM_UNARY_ABS)
    TFCC_UNARY_CASE(TFCC_ROCM_UNARY_SIGN)
    TFCC_UNARY_CASE(TFCC_ROCM_UNARY_NEG)
    TFCC_UNARY_CASE(TFCC_ROCM_UNARY_RECIPROCAL)
    TFCC_UNARY_CASE(TFCC_ROCM_UNARY_SQRT)
    default: return set_error(TFCC_ROCM_INVALID_ARGUMENT, "unary: unknown function %d", op);
  }
#undef TFCC_UNARY_CASE
  return check_launch("unary");
}

}  // extern "C"
