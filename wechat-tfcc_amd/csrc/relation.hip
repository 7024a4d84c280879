// Comparisons and argmax: byte-valued (0 / 1) results of comparing a tensor with a value or with another tensor, and
// the position of the largest element along one axis.
//
//   tensor (x) value    tfcc/mkl/interfaces/tfcc_mklcomparisoninterface.cpp: result[i] = a[i] OP b ? 1 : 0
//   tensor (x) tensor   tfcc/core/operations/tfcc_relation.cpp:101-115: the operands are subtracted (with numpy-style
//                       broadcasting) and the difference is compared with 0, in the element type: unsigned
//                       differences wrap, and inf - inf is not equal to 0.  The difference is formed here in the
//                       kernel instead of in memory.
//   argmax              tfcc/mkl/interfaces/tfcc_mklbasicinterface.cpp:469-485: the first position of the largest
//                       element (a later element wins only if it is greater).
//   top k               tfcc/mkl/interfaces/tfcc_mklbasicinterface.cpp:159-260, :779-800: the k largest elements of each
//                       row in descending order with their positions.  The reference's heaps leave the order of equal
//                       values to the standard library and to the number of threads; here equal values come in
//                       ascending position.
#include <type_traits>

#include "common.hpp"

namespace tfcc_rocm {
namespace {

struct CompareShape {
  unsigned dims[6];
  unsigned long long strideA[6], strideB[6];
  int rank;
};

template <class T>
__device__ __forceinline__ unsigned char compare_value(int op, T x, T y) {
  switch (op) {
    case TFCC_ROCM_COMPARE_EQUAL: return x == y;
    case TFCC_ROCM_COMPARE_UNEQUAL: return x != y;
    case TFCC_ROCM_COMPARE_GREATER: return x > y;
    case TFCC_ROCM_COMPARE_GREATER_EQUAL: return x >= y;
    case TFCC_ROCM_COMPARE_LESS: return x < y;
    default: return x <= y;
  }
}

// a - b in T: integers wrap (computed unsigned), floating-point types subtract
template <class T>
__device__ __forceinline__ T difference(T x, T y) {
  if constexpr (std::is_floating_point<T>::value) {
    return x - y;
  } else {
    using U = typename std::make_unsigned<T>::type;
    return static_cast<T>(static_cast<U>(static_cast<U>(x) - static_cast<U>(y)));
  }
}

template <class T>
__global__ __launch_bounds__(256) void compare_value_kernel(int op, const T* a, size_t total, T value,
                                                            unsigned char* out) {
  const size_t step = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += step) out[i] = compare_value<T>(op, a[i], value);
}

template <class T>
__global__ __launch_bounds__(256) void compare_tensors_kernel(int op, const T* a, const T* b, size_t total,
                                                              CompareShape p, unsigned char* out) {
  const size_t step = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += step) {
    size_t rem = i, ia = 0, ib = 0;
    for (int d = p.rank - 1; d >= 0; --d) {
      const size_t c = rem % p.dims[d];
      rem /= p.dims[d];
      ia += c * p.strideA[d];
      ib += c * p.strideB[d];
    }
    out[i] = compare_value<T>(op, difference<T>(a[ia], b[ib]), T(0));
  }
}

// 64 neighbouring (outer, inner) positions per workgroup, read coalesced; the axis is cut into four ranges, one per
// wavefront.  Every range starts from the axis' first element as the scalar loop does (a NaN there stays, a NaN
// elsewhere is never taken), and the ranges are joined in ascending order: a later one wins only if it is greater.
__global__ __launch_bounds__(256) void argmax_kernel(const float* a, size_t outer, unsigned length, size_t inner,
                                                     long long* out) {
  __shared__ float sBest[256];
  __shared__ unsigned sIndex[256];
  const size_t total = outer * inner;
  const size_t i = (size_t)blockIdx.x * 64 + (threadIdx.x & 63);
  const unsigned part = threadIdx.x >> 6;
  const bool valid = i < total;
  float best = 0.f;
  unsigned index = 0;
  const float* p = a;
  if (valid) {
    const size_t x = i / inner, z = i - x * inner;
    p = a + x * length * inner + z;
    best = p[0];
    const unsigned begin = (unsigned)((unsigned long long)length * part / 4);
    const unsigned end = (unsigned)((unsigned long long)length * (part + 1) / 4);
    for (unsigned y = begin; y < end; ++y) {
      const float v = p[(size_t)y * inner];
      if (v > best) {
        best = v;
        index = y;
      }
    }
  }
  sBest[threadIdx.x] = best;
  sIndex[threadIdx.x] = index;
  __syncthreads();
  if (valid && part == 0) {
#pragma unroll
    for (int j = 1; j < 4; ++j) {
      const float ob = sBest[threadIdx.x + 64 * j];
      if (ob > best) {
        best = ob;
        index = sIndex[threadIdx.x + 64 * j];
      }
    }
    out[i] = index;
  }
}

// the last axis: one wavefront per row, lanes stride the row, then the lanes' (value, first index) pairs are joined
__global__ __launch_bounds__(256) void argmax_rows_kernel(const float* a, size_t rows, unsigned length, long long* out) {
  const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const unsigned lane = threadIdx.x & 63;
  const float* p = a + row * length;
  // every lane starts from the row's first element, as the scalar loop does: a NaN there stays (nothing is greater),
  // a NaN elsewhere is never taken
  float best = p[0];
  unsigned index = 0;
  for (unsigned y = lane; y < length; y += 64) {
    const float v = p[y];
    if (v > best) {
      best = v;
      index = y;
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ob = __shfl_xor(best, off, 64);
    const unsigned oi = __shfl_xor(index, off, 64);
    // the greater value wins; of equal values the smaller position
    if (ob > best || (!(best > ob) && oi < index)) {
      best = ob;
      index = oi;
    }
  }
  if (lane == 0) out[row] = index;
}

// Floats as unsigned keys of the same order (negative values reversed, the sign bit flipped for the others), joined
// with the complement of the position: the larger composite is the larger value or, of equal values, the earlier one.
__device__ __forceinline__ unsigned long long topk_composite(float v, unsigned position) {
  unsigned bits = __float_as_uint(v);
  if (bits == 0x80000000u) bits = 0;  // -0 and +0 are equal values
  const unsigned key = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
  return ((unsigned long long)key << 32) | (unsigned)(~position);
}

// One workgroup per row, k rounds: each round takes the largest composite below the one taken before.  Every round
// reads the row again (from L2 after the first), four independent loads per thread in flight; this suits the short
// lists of a decoder, where k * length stays small.  The wavefronts' results meet in LDS, two buffers in turn so
// that one barrier per round is enough.
__global__ __launch_bounds__(256) void topk_rows_kernel(const float* a, unsigned length, unsigned k, float* values,
                                                        unsigned* positions) {
  __shared__ unsigned long long sBest[8];
  const size_t row = blockIdx.x;
  const unsigned tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float* p = a + row * length;
  unsigned long long previous = ~0ull;
  for (unsigned round = 0; round < k; ++round) {
    unsigned long long best = 0;  // below the composite of every element: positions stay below 2^32 - 1, so low words are not 0
    unsigned y = tid;
    for (; (unsigned long long)y + 768 < length; y += 1024) {
      const unsigned long long c0 = topk_composite(p[y], y), c1 = topk_composite(p[y + 256], y + 256),
                               c2 = topk_composite(p[y + 512], y + 512), c3 = topk_composite(p[y + 768], y + 768);
      if (c0 < previous && c0 > best) best = c0;
      if (c1 < previous && c1 > best) best = c1;
      if (c2 < previous && c2 > best) best = c2;
      if (c3 < previous && c3 > best) best = c3;
    }
    for (; y < length; y += 256) {
      const unsigned long long c = topk_composite(p[y], y);
      if (c < previous && c > best) best = c;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const unsigned long long other = __shfl_xor(best, off, 64);
      if (other > best) best = other;
    }
    unsigned long long* buffer = sBest + (round & 1) * 4;
    if (lane == 0) buffer[wave] = best;
    __syncthreads();
    best = buffer[0];
#pragma unroll
    for (int w = 1; w < 4; ++w)
      if (buffer[w] > best) best = buffer[w];
    previous = best;
    if (tid == 0 && best != 0) {  // k <= length leaves an element for every round
      const unsigned position = ~(unsigned)(best & 0xffffffffu);
      values[row * k + round] = p[position];
      positions[row * k + round] = position;
    }
  }
}

unsigned grid_of(size_t total) {
  size_t blocks = (total + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  return (unsigned)(blocks ? blocks : 1);
}

template <class T>
int launch_compare_value(hipStream_t s, int op, const void* a, size_t total, const void* value, unsigned char* out) {
  hipLaunchKernelGGL(compare_value_kernel<T>, dim3(grid_of(total)), dim3(256), 0, s, op, static_cast<const T*>(a), total,
                     *static_cast<const T*>(value), out);
  return check_launch("compare_value");
}

template <class T>
int launch_compare_tensors(hipStream_t s, int op, const void* a, const void* b, size_t total, const CompareShape& p,
                           unsigned char* out) {
  hipLaunchKernelGGL(compare_tensors_kernel<T>, dim3(grid_of(total)), dim3(256), 0, s, op, static_cast<const T*>(a),
                     static_cast<const T*>(b), total, p, out);
  return check_launch("compare");
}

}  // namespace
}  // namespace tfcc_rocm

using namespace tfcc_rocm;

#define TFCC_FOR_ELEMENT_TYPES(CALL)          \
  CALL(TFCC_ROCM_S8, signed char)             \
  CALL(TFCC_ROCM_U8, unsigned char)           \
  CALL(TFCC_ROCM_S16, short)                  \
  CALL(TFCC_ROCM_U16, unsigned short)         \
  CALL(TFCC_ROCM_S32, int)                    \
  CALL(TFCC_ROCM_U32, unsigned)               \
  CALL(TFCC_ROCM_S64, long long)              \
  CALL(TFCC_ROCM_U64, unsigned long long)     \
  CALL(TFCC_ROCM_F32, float)                  \
  CALL(TFCC_ROCM_F64, double)

extern "C" {

int tfcc_rocm_compare_value(void* stream, int op, const void* a, int type, uint64_t total, const void* value,
                            uint8_t* out) {
  TFCC_REQUIRE(a && value && out, "compare_value: null argument");
  TFCC_REQUIRE(total > 0, "compare_value: empty tensor");
  TFCC_REQUIRE(op >= TFCC_ROCM_COMPARE_EQUAL && op <= TFCC_ROCM_COMPARE_LESS_EQUAL, "compare_value: unknown operation %d", op);
  hipStream_t s = as_stream(stream);
#define TFCC_COMPARE_CASE(CODE, T) \
  case CODE: return launch_compare_value<T>(s, op, a, (size_t)total, value, out);
  switch (type) {
    TFCC_FOR_ELEMENT_TYPES(TFCC_COMPARE_CASE)
    default: return set_error(TFCC_ROCM_INVALID_ARGUMENT, "compare_value: unknown element type %d", type);
  }
#undef TFCC_COMPARE_CASE
}

int tfcc_rocm_compare(void* stream, int op, const void* a, const void* b, int type, int rank, const unsigned* dims,
                      const uint64_t* stride_a, const uint64_t* stride_b, uint8_t* out) {
  TFCC_REQUIRE(a && b && out && dims && stride_a && stride_b, "compare: null argument");
  TFCC_REQUIRE(op >= TFCC_ROCM_COMPARE_EQUAL && op <= TFCC_ROCM_COMPARE_LESS_EQUAL, "compare: unknown operation %d", op);
  TFCC_REQUIRE(rank >= 1 && rank <= 6, "compare: rank %d (1..6)", rank);
  CompareShape p{};
  p.rank = rank;
  size_t total = 1;
  for (int d = 0; d < rank; ++d) {
    TFCC_REQUIRE(dims[d] > 0, "compare: empty tensor");
    p.dims[d] = dims[d];
    p.strideA[d] = stride_a[d];
    p.strideB[d] = stride_b[d];
    total *= dims[d];
  }
  hipStream_t s = as_stream(stream);
#define TFCC_COMPARE_CASE(CODE, T) \
  case CODE: return launch_compare_tensors<T>(s, op, a, b, total, p, out);
  switch (type) {
    TFCC_FOR_ELEMENT_TYPES(TFCC_COMPARE_CASE)
    default: return set_error(TFCC_ROCM_INVALID_ARGUMENT, "compare: unknown element type %d", type);
  }
#undef TFCC_COMPARE_CASE
}

int tfcc_rocm_argmax_f32(void* stream, const float* in, uint64_t outer, unsigned length, uint64_t inner, int64_t* out) {
  TFCC_REQUIRE(in && out, "argmax: null argument");
  TFCC_REQUIRE(outer > 0 && length > 0 && inner > 0, "argmax: empty tensor");
  TFCC_REQUIRE(outer < (1ull << 36) && inner < (1ull << 36) && outer * inner < (1ull << 36), "argmax: too many positions");
  hipStream_t s = as_stream(stream);
  if (inner == 1 && length >= 64 && outer < (1ull << 31)) {
    hipLaunchKernelGGL(argmax_rows_kernel, dim3((unsigned)((outer + 3) / 4)), dim3(256), 0, s, in, (size_t)outer, length,
                       reinterpret_cast<long long*>(out));
  } else {
    hipLaunchKernelGGL(argmax_kernel, dim3((unsigned)((outer * inner + 63) / 64)), dim3(256), 0, s, in, (size_t)outer,
                       length, (size_t)inner, reinterpret_cast<long long*>(out));
  }
  return check_launch("argmax");
}

int tfcc_rocm_topk_f32(void* stream, const float* in, uint64_t rows, unsigned length, unsigned k, float* values,
                       uint32_t* positions) {
  TFCC_REQUIRE(in && values && positions, "topk: null argument");
  TFCC_REQUIRE(rows > 0 && length > 0, "topk: empty tensor");
  TFCC_REQUIRE(k >= 1 && k <= length, "topk: k = %u of %u elements", k, length);
  // one pass over the row per selected element and one workgroup per row: meant for beam-sized k
  TFCC_REQUIRE(k <= 1024u, "topk: k = %u is beyond the 1024 this selection by repeated passes is meant for", k);
  TFCC_REQUIRE(rows < (1ull << 31) && length < 0x80000000u, "topk: tensor too large");
  hipLaunchKernelGGL(topk_rows_kernel, dim3((unsigned)rows), dim3(256), 0, as_stream(stream), in, length, k, values,
                     positions);
  return check_launch("topk");
}

}  // extern "C"
