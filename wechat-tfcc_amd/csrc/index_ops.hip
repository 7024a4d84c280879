// Data movement between the matrix products of a model: row gather (embedding lookup), slice / concat along an
// axis (one strided 2-D copy each) and element type conversion.  All are one pass over the data, bound by HBM.
//
// Semantics follow the reference's CPU kernels:
//   gather        tfcc/mkl/interfaces/tfcc_mklgatherinterface.cpp:28-66 (rows of params by index; an index outside
//                 [0, batch) gives a row of zeros)
//   slice         tfcc/mkl/interfaces/tfcc_mklbasicinterface.cpp:34-70, 488-515 ([s1, s2, s3] -> [s1, length, s3])
//   concat        tfcc/core/operations/tfcc_base.cpp:86-106 (every value copied behind the previous ones along axis)
//   cast          tfcc::data::cast: static_cast element by element
//   where         tfcc/mkl/interfaces/tfcc_mklbasicinterface.cpp:398-422 (condition[i] != 0 ? x : y, either of x and
//                 y a tensor or one value)
//   tril / triu   tfcc/mkl/interfaces/tfcc_mklbasicinterface.cpp:433-466 (row r keeps columns below r + k + 1, or
//                 from r + k on; the rest is 0)
#include "common.hpp"

namespace tfcc_rocm {
namespace {

unsigned copy_grid(size_t units) {
  size_t blocks = (units + 255) / 256;
  if (blocks > 2048) blocks = 2048;
  if (blocks < 1) blocks = 1;
  return (unsigned)blocks;
}

// rows x width units of W bytes, pitches in units
template <class W>
__global__ __launch_bounds__(256) void copy2d_kernel(const W* src, size_t srcPitch, W* dst, size_t dstPitch, size_t rows,
                                                     size_t width) {
  const size_t total = rows * width, stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
    const size_t r = i / width, c = i - r * width;
    dst[r * dstPitch + c] = src[r * srcPitch + c];
  }
}

template <class W, class IDX>
__global__ __launch_bounds__(256) void gather_kernel(const W* params, unsigned batch, size_t chunk, const IDX* indices,
                                                     size_t length, W* out) {
  const size_t total = length * chunk, stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
    const size_t r = i / chunk, c = i - r * chunk;
    const IDX idx = indices[r];
    W v{};
    if (!(idx < (IDX)0) && (unsigned long long)idx < (unsigned long long)batch) v = params[(size_t)idx * chunk + c];
    out[i] = v;
  }
}

template <class IN, class OUT>
__global__ __launch_bounds__(256) void cast_kernel(const IN* in, size_t total, OUT* out) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) out[i] = static_cast<OUT>(in[i]);
}

// elements of W bytes; x / y null: the value in xBits / yBits instead
template <class W>
__global__ __launch_bounds__(256) void where_kernel(const unsigned char* condition, const W* x, W xValue, const W* y,
                                                    W yValue, size_t total, W* out) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride)
    out[i] = condition[i] != 0 ? (x ? x[i] : xValue) : (y ? y[i] : yValue);
}

template <class W, bool UPPER>
__global__ __launch_bounds__(256) void triangle_kernel(const W* in, size_t rows, size_t cols, long long k, W* out) {
  const size_t total = rows * cols, stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
    const long long r = (long long)(i / cols), c = (long long)(i - (size_t)r * cols);
    const bool keep = UPPER ? c >= r + k : c < r + k + 1;
    out[i] = keep ? in[i] : W(0);
  }
}

struct Word16 { unsigned w[4]; };

template <class W>
int launch_copy2d(hipStream_t s, const void* src, size_t srcPitch, void* dst, size_t dstPitch, size_t rows, size_t width) {
  constexpr size_t B = sizeof(W);
  hipLaunchKernelGGL(copy2d_kernel<W>, dim3(copy_grid(rows * (width / B))), dim3(256), 0, s, static_cast<const W*>(src),
                     srcPitch / B, static_cast<W*>(dst), dstPitch / B, rows, width / B);
  return check_launch("copy2d");
}

template <class W>
int launch_gather(hipStream_t s, const void* params, unsigned batch, size_t chunkBytes, const void* indices, int indexType,
                  size_t length, void* out) {
  const size_t chunk = chunkBytes / sizeof(W);
  const dim3 grid(copy_grid(length * chunk)), block(256);
  const W* p = static_cast<const W*>(params);
  W* o = static_cast<W*>(out);
  switch (indexType) {
    case TFCC_ROCM_S32: hipLaunchKernelGGL((gather_kernel<W, int>), grid, block, 0, s, p, batch, chunk, static_cast<const int*>(indices), length, o); break;
    case TFCC_ROCM_U32: hipLaunchKernelGGL((gather_kernel<W, unsigned>), grid, block, 0, s, p, batch, chunk, static_cast<const unsigned*>(indices), length, o); break;
    case TFCC_ROCM_S64: hipLaunchKernelGGL((gather_kernel<W, long long>), grid, block, 0, s, p, batch, chunk, static_cast<const long long*>(indices), length, o); break;
    case TFCC_ROCM_U64: hipLaunchKernelGGL((gather_kernel<W, unsigned long long>), grid, block, 0, s, p, batch, chunk, static_cast<const unsigned long long*>(indices), length, o); break;
    default: return set_error(TFCC_ROCM_INVALID_ARGUMENT, "gather: index type %d (S32, U32, S64 or U64)", indexType);
  }
  return check_launch("gather");
}

bool aligned_to(size_t bytes, const void* a, const void* b, size_t x, size_t y, size_t z) {
  return (uintptr_t)a % bytes == 0 && (uintptr_t)b % bytes == 0 && x % bytes == 0 && y % bytes == 0 && z % bytes == 0;
}

template <class IN>
int launch_cast_from(hipStream_t s, const void* in, void* out, int outType, size_t total) {
  const dim3 grid(copy_grid(total)), block(256);
  const IN* p = static_cast<const IN*>(in);
#define TFCC_CAST_TO(CODE, OUT) \
  case CODE: hipLaunchKernelGGL((cast_kernel<IN, OUT>), grid, block, 0, s, p, total, static_cast<OUT*>(out)); break;
  switch (outType) {
    TFCC_CAST_TO(TFCC_ROCM_S8, signed char)
    TFCC_CAST_TO(TFCC_ROCM_U8, unsigned char)
    TFCC_CAST_TO(TFCC_ROCM_S16, short)
    TFCC_CAST_TO(TFCC_ROCM_U16, unsigned short)
    TFCC_CAST_TO(TFCC_ROCM_S32, int)
    TFCC_CAST_TO(TFCC_ROCM_U32, unsigned)
    TFCC_CAST_TO(TFCC_ROCM_S64, long long)
    TFCC_CAST_TO(TFCC_ROCM_U64, unsigned long long)
    TFCC_CAST_TO(TFCC_ROCM_F32, float)
    TFCC_CAST_TO(TFCC_ROCM_F64, double)
    default: return set_error(TFCC_ROCM_INVALID_ARGUMENT, "cast: unknown result type %d", outType);
  }
#undef TFCC_CAST_TO
  return check_launch("cast");
}

}  // namespace
}  // namespace tfcc_rocm

using namespace tfcc_rocm;

extern "C" {

int tfcc_rocm_copy2d(void* stream, const void* src, uint64_t src_pitch, void* dst, uint64_t dst_pitch, uint64_t rows,
                     uint64_t width) {
  TFCC_REQUIRE(src && dst, "copy2d: null argument");
  TFCC_REQUIRE(rows > 0 && width > 0, "copy2d: empty region");
  TFCC_REQUIRE(src_pitch >= width && dst_pitch >= width, "copy2d: pitch shorter than a row");
  hipStream_t s = as_stream(stream);
  if (aligned_to(16, src, dst, src_pitch, dst_pitch, width)) return launch_copy2d<Word16>(s, src, src_pitch, dst, dst_pitch, rows, width);
  if (aligned_to(4, src, dst, src_pitch, dst_pitch, width)) return launch_copy2d<unsigned>(s, src, src_pitch, dst, dst_pitch, rows, width);
  return launch_copy2d<unsigned char>(s, src, src_pitch, dst, dst_pitch, rows, width);
}

int tfcc_rocm_gather_rows(void* stream, const void* params, unsigned batch, uint64_t chunk_bytes, const void* indices,
                          int index_type, uint64_t length, void* out) {
  TFCC_REQUIRE(params && indices && out, "gather: null argument");
  TFCC_REQUIRE(batch > 0 && chunk_bytes > 0 && length > 0, "gather: empty tensor");
  hipStream_t s = as_stream(stream);
  if (aligned_to(16, params, out, chunk_bytes, 0, 0)) return launch_gather<Word16>(s, params, batch, chunk_bytes, indices, index_type, length, out);
  if (aligned_to(4, params, out, chunk_bytes, 0, 0)) return launch_gather<unsigned>(s, params, batch, chunk_bytes, indices, index_type, length, out);
  return launch_gather<unsigned char>(s, params, batch, chunk_bytes, indices, index_type, length, out);
}

int tfcc_rocm_cast(void* stream, const void* in, int in_type, void* out, int out_type, uint64_t total) {
  TFCC_REQUIRE(in && out, "cast: null argument");
  TFCC_REQUIRE(total > 0, "cast: empty tensor");
  hipStream_t s = as_stream(stream);
  switch (in_type) {
    case TFCC_ROCM_S8: return launch_cast_from<signed char>(s, in, out, out_type, total);
    case TFCC_ROCM_U8: return launch_cast_from<unsigned char>(s, in, out, out_type, total);
    case TFCC_ROCM_S16: return launch_cast_from<short>(s, in, out, out_type, total);
    case TFCC_ROCM_U16: return launch_cast_from<unsigned short>(s, in, out, out_type, total);
    case TFCC_ROCM_S32: return launch_cast_from<int>(s, in, out, out_type, total);
    case TFCC_ROCM_U32: return launch_cast_from<unsigned>(s, in, out, out_type, total);
    case TFCC_ROCM_S64: return launch_cast_from<long long>(s, in, out, out_type, total);
    case TFCC_ROCM_U64: return launch_cast_from<unsigned long long>(s, in, out, out_type, total);
    case TFCC_ROCM_F32: return launch_cast_from<float>(s, in, out, out_type, total);
    case TFCC_ROCM_F64: return launch_cast_from<double>(s, in, out, out_type, total);
    default: return set_error(TFCC_ROCM_INVALID_ARGUMENT, "cast: unknown source type %d", in_type);
  }
}

int tfcc_rocm_where(void* stream, const uint8_t* condition, const void* x, uint64_t x_bits, const void* y,
                    uint64_t y_bits, unsigned element_bytes, uint64_t total, void* out) {
  TFCC_REQUIRE(condition && out, "where: null argument");
  TFCC_REQUIRE(x || y, "where: x and y are both values");
  TFCC_REQUIRE(total > 0, "where: empty tensor");
  hipStream_t s = as_stream(stream);
  const dim3 grid(copy_grid((size_t)total)), block(256);
#define TFCC_WHERE_CASE(BYTES, W)                                                                                  \
  case BYTES:                                                                                                      \
    hipLaunchKernelGGL(where_kernel<W>, grid, block, 0, s, condition, static_cast<const W*>(x), (W)x_bits,          \
                       static_cast<const W*>(y), (W)y_bits, (size_t)total, static_cast<W*>(out));                  \
    break;
  switch (element_bytes) {
    TFCC_WHERE_CASE(1, unsigned char)
    TFCC_WHERE_CASE(2, unsigned short)
    TFCC_WHERE_CASE(4, unsigned)
    TFCC_WHERE_CASE(8, unsigned long long)
    default: return set_error(TFCC_ROCM_INVALID_ARGUMENT, "where: element size %u (1, 2, 4 or 8)", element_bytes);
  }
#undef TFCC_WHERE_CASE
  return check_launch("where");
}

int tfcc_rocm_triangle(void* stream, const void* in, uint64_t rows, uint64_t cols, int64_t k, int upper,
                       unsigned element_bytes, void* out) {
  TFCC_REQUIRE(in && out, "triangle: null argument");
  TFCC_REQUIRE(rows > 0 && cols > 0, "triangle: empty matrix");
  TFCC_REQUIRE(rows < (1ull << 31) && cols < (1ull << 31), "triangle: matrix too large");
  TFCC_REQUIRE(k > -(1ll << 40) && k < (1ll << 40), "triangle: diagonal out of range");
  hipStream_t s = as_stream(stream);
  const dim3 grid(copy_grid((size_t)(rows * cols))), block(256);
#define TFCC_TRIANGLE_CASE(BYTES, W)                                                                               \
  case BYTES:                                                                                                      \
    if (upper)                                                                                                     \
      hipLaunchKernelGGL((triangle_kernel<W, true>), grid, block, 0, s, static_cast<const W*>(in), (size_t)rows,   \
                         (size_t)cols, (long long)k, static_cast<W*>(out));                                        \
    else                                                                                                           \
      hipLaunchKernelGGL((triangle_kernel<W, false>), grid, block, 0, s, static_cast<const W*>(in), (size_t)rows,  \
                         (size_t)cols, (long long)k, static_cast<W*>(out));                                        \
    break;
  switch (element_bytes) {
    TFCC_TRIANGLE_CASE(1, unsigned char)
    TFCC_TRIANGLE_CASE(2, unsigned short)
    TFCC_TRIANGLE_CASE(4, unsigned)
    TFCC_TRIANGLE_CASE(8, unsigned long long)
    default: return set_error(TFCC_ROCM_INVALID_ARGUMENT, "triangle: element size %u (1, 2, 4 or 8)", element_bytes);
  }
#undef TFCC_TRIANGLE_CASE
  return check_launch("triangle");
}

}  // extern "C"
