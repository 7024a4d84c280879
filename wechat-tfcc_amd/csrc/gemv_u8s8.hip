// Skinny (M <= 8) uint8 x int8 -> int32 product for decode shapes: HBM-bandwidth bound, B [K,N]
// is streamed exactly once.
//
// Same arithmetic as the general quantized matmul (tfcc/mkl/operations/tfcc_mklquantization.cpp:
// 33-69,176-201); the reference has no dedicated kernel for this shape.
//
// Work split: a workgroup of 16 wavefronts owns 64 consecutive columns over the whole of K, so no
// partial sums ever leave the CU.  The wavefronts deal the 64-row steps of K among themselves.
// Per step every lane loads a 16(k) x 4(n) byte block of B as 16 dwords (a wavefront reads four
// 64-byte row segments per instruction; the neighbouring column group, which shares the 128-byte
// lines, is placed on the same XCD), transposes it in registers with v_perm_b32 so that it holds
// 16 consecutive k for each of its four columns, and feeds them to v_mfma_i32_16x16x64_i8 as the
// B operand.  The A operand holds the (up to 8) rows of A, xor 0x80 (a' = a - 128), zero rows, and
// one row of ones in row 15 whose product is the true column sum of B, needed to undo the -128
// shift: sum a*b = sum a'*b + 128*colsum(B).  The 16 partial tiles are added through LDS, the
// offset terms and the optional per-channel dequantize are applied in the store.
#include <stdlib.h>

#include "common.hpp"
#include "gemv.hpp"

namespace tfcc_rocm {

typedef int v4i __attribute__((ext_vector_type(4)));

namespace {

constexpr int kWaves = 16;
constexpr int kThreads = kWaves * 64;
constexpr int kCols = 64;     // columns per workgroup
constexpr int kMaxM = 8;
constexpr int kRows = 16;     // MFMA rows: kMaxM data rows, zeros, ones in row 15
constexpr int kPartRows = 9;  // rows kept per wavefront: 8 data rows + the column-sum row

struct GemvParams {
  const unsigned char* A;
  const signed char* B;
  const int* rowsumA;
  const int* colsumB;
  int* accOut;
  float* f32Out;
  const float* scaleB;
  float scaleA;
  int offsetA, offsetB;
  const float *minA, *maxA, *minB, *maxB;  // optional ranges in device memory (override the offsets)
  float *minC, *maxC;
  unsigned M, N, K;
  unsigned colGroups, groupsPerXcd;
};

__device__ __forceinline__ void transpose4x4(const unsigned r[4], unsigned c[4]) {
  unsigned t0 = __builtin_amdgcn_perm(r[1], r[0], 0x05010400u);
  unsigned t1 = __builtin_amdgcn_perm(r[1], r[0], 0x07030602u);
  unsigned t2 = __builtin_amdgcn_perm(r[3], r[2], 0x05010400u);
  unsigned t3 = __builtin_amdgcn_perm(r[3], r[2], 0x07030602u);
  c[0] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
  c[1] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
  c[2] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
  c[3] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
}

__global__ __launch_bounds__(kThreads) void gemv_kernel(const GemvParams p) {
  __shared__ int red[kWaves][kPartRows][kCols];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: the step loop's bounds stay scalar
  // consecutive workgroup ids go to different XCDs: give each XCD a run of adjacent column groups
  const unsigned cg = (blockIdx.x & 7u) * p.groupsPerXcd + (blockIdx.x >> 3);
  if ((blockIdx.x >> 3) >= p.groupsPerXcd || cg >= p.colGroups) return;
  const unsigned n0 = cg * kCols;
  const unsigned M = p.M, N = p.N, K = p.K;
  const int j = lane & 15, kg = lane >> 4;

  const __amdgpu_buffer_rsrc_t rsrcB =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<signed char*>(p.B), 0, (int)(K * N), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrcA =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(p.A), 0, (int)(M * K), 0x00020000);

  v4i acc[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) acc[e] = v4i{0, 0, 0, 0};

  const unsigned steps = (K + 63) / 64;
  for (unsigned step = wave; step < steps; step += 2 * kWaves) {
    // two steps in flight per wavefront (the second may lie past K: it then reads zeros)
    unsigned braw[2][16];
    v4i a[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const unsigned k0 = (step + u * kWaves) * 64 + kg * 16;  // this lane's 16 rows
#pragma unroll
      for (int q = 0; q < 16; ++q)
        braw[u][q] = __builtin_amdgcn_raw_buffer_load_b32(rsrcB, (k0 + q) * N + n0 + j * 4, 0, 0);
      a[u] = v4i{0, 0, 0, 0};
      if ((unsigned)j < M) {
        a[u] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrcA, (unsigned)j * K + k0, 0, 0));
        a[u] = a[u] ^ (int)0x80808080;
      } else if (j == kRows - 1) {
        a[u] = v4i{0x01010101, 0x01010101, 0x01010101, 0x01010101};
      }
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      unsigned col[4][4];
#pragma unroll
      for (int kq = 0; kq < 4; ++kq) {
        unsigned c4[4];
        transpose4x4(&braw[u][4 * kq], c4);
#pragma unroll
        for (int e = 0; e < 4; ++e) col[e][kq] = c4[e];
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v4i bv = {(int)col[e][0], (int)col[e][1], (int)col[e][2], (int)col[e][3]};
        acc[e] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[u], bv, acc[e], 0, 0, 0);
      }
    }
  }

  // D layout of the 16x16 block: lane (j, kg) holds rows 4*kg + r, column j.
  // Keep rows 0..7 and row 15 (stored as row 8).
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int col = j * 4 + e;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = 4 * kg + r;
      if (row < kMaxM) red[wave][row][col] = acc[e][r];
      else if (row == kRows - 1) red[wave][kMaxM][col] = acc[e][r];
    }
  }
  __syncthreads();

  int oA = p.offsetA, oB = p.offsetB;
  if (p.minA) {
    float mnA = *p.minA, mxA = *p.maxA, mnB = *p.minB, mxB = *p.maxB;
    qmatmul_offsets(mnA, mxA, mnB, mxB, &oA, &oB);
    if (cg == 0 && tid == 0) {
      float mnC, mxC;
      qmatmul_range(mnA, mxA, mnB, mxB, &mnC, &mxC);
      if (p.minC) *p.minC = mnC;
      if (p.maxC) *p.maxC = mxC;
    }
  }
  const unsigned offA = (unsigned)oA, offB = (unsigned)oB;
  const unsigned global = offA * offB * K;
  for (unsigned idx = tid; idx < M * kCols; idx += kThreads) {
    const unsigned r = idx / kCols, c = idx % kCols;
    const unsigned gn = n0 + c;
    if (gn >= N) continue;
    unsigned sum = 0, cs = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      sum += (unsigned)red[w][r][c];
      cs += (unsigned)red[w][kMaxM][c];
    }
    const unsigned v = sum + 128u * cs + global + (unsigned)p.rowsumA[r] * offB + (unsigned)p.colsumB[gn] * offA;
    if (p.accOut) p.accOut[(size_t)r * N + gn] = (int)v;
    if (p.f32Out) p.f32Out[(size_t)r * N + gn] = (float)((double)(int)v * ((double)p.scaleA * (double)p.scaleB[gn]));
  }
}


// ---- pre-packed B (weights that are multiplied many times) --------------------------------------------
// Layout: [N/16 column slabs][K/64 steps][64 lanes][16 bytes], where lane (kg = lane / 16, j = lane % 16)
// of step t holds B[64 t + 16 kg + 0..15][16 slab + j]: exactly the B operand of one
// v_mfma_i32_16x16x64_i8, so a wavefront fetches an operand with one contiguous 1 KiB load and no
// byte shuffling, and a workgroup streams one contiguous slab (K x 16 bytes).  Rows past K and columns
// past N are stored as zeros.
constexpr int kPackWaves = 4;   // wavefronts that share the K steps of one 16-column slab (one slab per workgroup:
                                // two slabs sharing one staged copy of A measured slower, 12.4 against 10.0 us)
constexpr int kStageLoads = 8;  // 16-byte loads per thread in flight while A is staged
constexpr int kPackThreads = kPackWaves * 64;
constexpr int kPackInFlight = 16;  // operand loads in flight per wavefront

__global__ __launch_bounds__(256) void gemv_pack_kernel(const signed char* b, unsigned N, unsigned K, unsigned steps,
                                                        size_t chunks, unsigned char* packed) {
  // one 16-byte chunk per thread (gathered from 16 rows of B: this runs once per weight matrix)
  const size_t c = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (c >= chunks) return;
  const unsigned lane = (unsigned)(c & 63);
  const size_t st = c >> 6;
  const unsigned t = (unsigned)(st % steps), slab = (unsigned)(st / steps);
  const unsigned col = slab * 16 + (lane & 15), k0 = t * 64 + (lane >> 4) * 16;
  unsigned w[4] = {0, 0, 0, 0};
  if (col < N) {
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const unsigned k = k0 + q;
      const unsigned v = k < K ? (unsigned char)b[(size_t)k * N + col] : 0u;
      w[q >> 2] |= v << (8 * (q & 3));
    }
  }
  *reinterpret_cast<v4i*>(packed + c * 16) = v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
}

// STAGE_A: the rows of A (at most 8 x K bytes, the same for every workgroup) are copied to LDS once with
// full-width loads, already xor 0x80, and the operands are read from there.  Fetching them from memory
// per step costs as many load instructions as the B stream itself, mostly empty (M * 4 of 64 lanes):
// 12.7 us against 8.8 us without them for 4096 x 11008.  Without STAGE_A (A too large for LDS) the
// operands are fetched per step.
template <bool STAGE_A>
__global__ __launch_bounds__(kPackThreads) void gemv_packed_kernel(const GemvParams p, const unsigned char* packed,
                                                                  unsigned steps) {
  __shared__ int red[kPackWaves][kPartRows][16];
  extern __shared__ __align__(16) unsigned char aLds[];  // [M][steps * 64 + 16]: the pad spreads the rows over the banks
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: the step loop's bounds stay scalar
  const unsigned slab = blockIdx.x;
  const unsigned M = p.M, N = p.N, K = p.K;
  const int j = lane & 15, kg = lane >> 4;
  const unsigned char* src = packed + (size_t)slab * steps * 1024 + lane * 16;
  const __amdgpu_buffer_rsrc_t rsrcA =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(p.A), 0, (int)(M * K), 0x00020000);
  const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
  v4i acc = {0, 0, 0, 0};
  // what the store needs from memory is fetched first, so that its latency hides behind the B stream
  const unsigned er = tid >> 4, ec = tid & 15, egn = slab * 16 + ec;
  const bool eActive = tid < (int)(M * 16) && egn < N;
  int eRowsum = 0, eColsum = 0;
  float eScale = 0.f;
  if (eActive) {
    eRowsum = p.rowsumA[er];
    eColsum = p.colsumB[egn];
    if (p.f32Out) eScale = p.scaleB[egn];
  }
  float mnA = 0.f, mxA = 0.f, mnB = 0.f, mxB = 0.f;  // ranges in device memory override the immediate offsets
  if (p.minA) { mnA = *p.minA; mxA = *p.maxA; mnB = *p.minB; mxB = *p.maxB; }

  // the wavefronts deal the steps among themselves, kPackInFlight at a time; the first batch of B is
  // requested before A is staged
  v4i bv[kPackInFlight];
  auto loadB = [&](unsigned t0) {
#pragma unroll
    for (int u = 0; u < kPackInFlight; ++u) {
      const unsigned t = t0 + u;
      bv[u] = v4i{0, 0, 0, 0};
      if (t < steps) bv[u] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(src + (size_t)t * 1024));  // streamed once
    }
  };
  loadB(wave * kPackInFlight);
  const unsigned pitch = steps * 64 + 16;
  if constexpr (STAGE_A) {
    const unsigned chunksPerRow = steps * 4, total = M * chunksPerRow;
    for (unsigned c0 = 0; c0 < total; c0 += kPackThreads * kStageLoads) {
      v4i v[kStageLoads];
#pragma unroll
      for (int u = 0; u < kStageLoads; ++u) {
        const unsigned c = c0 + u * kPackThreads + tid, row = c / chunksPerRow, ch = c - row * chunksPerRow;
        // past the end of a row (K not a multiple of 64) and past the last row: zeros from the bounds check
        const unsigned off = (c < total && ch * 16 < K) ? row * K + ch * 16 : 0xfffffff0u;
        v[u] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrcA, off, 0, 0));
      }
#pragma unroll
      for (int u = 0; u < kStageLoads; ++u) {
        const unsigned c = c0 + u * kPackThreads + tid, row = c / chunksPerRow, ch = c - row * chunksPerRow;
        if (c < total) *reinterpret_cast<v4i*>(aLds + row * pitch + ch * 16) = v[u] ^ (int)0x80808080;
      }
    }
    __syncthreads();
  }
  for (unsigned t0 = wave * kPackInFlight; t0 < steps; t0 += kPackWaves * kPackInFlight) {
    if (t0 != (unsigned)wave * kPackInFlight) loadB(t0);
    v4i av[kPackInFlight];
#pragma unroll
    for (int u = 0; u < kPackInFlight; ++u) {
      const unsigned t = t0 + u;
      av[u] = v4i{0, 0, 0, 0};
      if (t < steps) {
        if ((unsigned)j < M) {
          if constexpr (STAGE_A)
            av[u] = *reinterpret_cast<const v4i*>(aLds + (unsigned)j * pitch + t * 64 + kg * 16);
          else
            av[u] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrcA, (unsigned)j * K + t * 64 + kg * 16, 0, 0)) ^
                    (int)0x80808080;
        } else if (j == kRows - 1) {
          av[u] = ones;
        }
      }
    }
#pragma unroll
    for (int u = 0; u < kPackInFlight; ++u) acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(av[u], bv[u], acc, 0, 0, 0);
  }
  // lane (j, kg) holds rows 4 kg + r of column j
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = 4 * kg + r;
    if (row < kMaxM) red[wave][row][j] = acc[r];
    else if (row == kRows - 1) red[wave][kMaxM][j] = acc[r];
  }
  __syncthreads();
  int oA = p.offsetA, oB = p.offsetB;
  if (p.minA) {
    qmatmul_offsets(mnA, mxA, mnB, mxB, &oA, &oB);
    if (blockIdx.x == 0 && tid == 0) {
      float mnC, mxC;
      qmatmul_range(mnA, mxA, mnB, mxB, &mnC, &mxC);
      if (p.minC) *p.minC = mnC;
      if (p.maxC) *p.maxC = mxC;
    }
  }
  const unsigned offA = (unsigned)oA, offB = (unsigned)oB;
  const unsigned global = offA * offB * K;
  // What was asked for at the start is first looked at here: otherwise the compiler widens this column's scale to
  // double right behind its load, and the wait for that load would stand in front of the stream of B.
  asm volatile("" : "+v"(eScale), "+v"(eRowsum), "+v"(eColsum));
  if (eActive) {
    unsigned sum = 0, cs = 0;
#pragma unroll
    for (int w = 0; w < kPackWaves; ++w) {
      sum += (unsigned)red[w][er][ec];
      cs += (unsigned)red[w][kMaxM][ec];
    }
    const unsigned v = sum + 128u * cs + global + (unsigned)eRowsum * offB + (unsigned)eColsum * offA;
    if (p.accOut) p.accOut[(size_t)er * N + egn] = (int)v;
    if (p.f32Out) p.f32Out[(size_t)er * N + egn] = (float)((double)(int)v * ((double)p.scaleA * (double)eScale));
  }
}

}  // namespace

// Whether the skinny kernel can take this shape (else the caller uses the general kernel).
bool gemv_supported(const void* a, const void* b, unsigned m, unsigned n, unsigned k) {
  return m >= 1 && m <= (unsigned)kMaxM && n % 4 == 0 && k % 16 == 0 && (uintptr_t)a % 16 == 0 &&
         (uintptr_t)b % 4 == 0 && ((unsigned long long)k + 2048) * n + 512 < (1ull << 31);
}

int gemv_launch(hipStream_t stream, const unsigned char* a, const signed char* b, const int* rowsumA,
                const int* colsumB, int offsetA, int offsetB, const float* const ranges[4],
                float* const rangeOut[2], unsigned m, unsigned n, unsigned k, int* accOut,
                float scaleA, const float* scaleB, float* f32Out, bool colsumExact) {
  if (gemv_wide_supported(a, b, m, n, k))
    return gemv_wide_launch(stream, false, a, b, rowsumA, colsumB, offsetA, offsetB, ranges, rangeOut, m, n, k, accOut,
                            scaleA, scaleB, f32Out, colsumExact);
  return gemv_onepass_launch(stream, a, b, rowsumA, colsumB, offsetA, offsetB, ranges, rangeOut, m, n, k, accOut, scaleA,
                             scaleB, f32Out);
}

int gemv_onepass_launch(hipStream_t stream, const unsigned char* a, const signed char* b, const int* rowsumA,
                        const int* colsumB, int offsetA, int offsetB, const float* const ranges[4],
                        float* const rangeOut[2], unsigned m, unsigned n, unsigned k, int* accOut,
                        float scaleA, const float* scaleB, float* f32Out) {
  GemvParams p{};
  if (ranges && ranges[0]) {
    p.minA = ranges[0]; p.maxA = ranges[1]; p.minB = ranges[2]; p.maxB = ranges[3];
    if (rangeOut) { p.minC = rangeOut[0]; p.maxC = rangeOut[1]; }
  }
  p.A = a; p.B = b; p.rowsumA = rowsumA; p.colsumB = colsumB;
  p.accOut = accOut; p.f32Out = f32Out; p.scaleA = scaleA; p.scaleB = scaleB;
  p.offsetA = offsetA; p.offsetB = offsetB;
  p.M = m; p.N = n; p.K = k;
  p.colGroups = (n + kCols - 1) / kCols;
  p.groupsPerXcd = (p.colGroups + 7) / 8;
  hipLaunchKernelGGL(gemv_kernel, dim3(p.groupsPerXcd * 8), dim3(kThreads), 0, stream, p);
  return check_launch("skinny quantized matmul");
}

namespace {

__global__ void dequant_per_channel_kernel(const int* acc, unsigned m, unsigned n, float scaleA,
                                           const float* scaleB, float* out) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (size_t)m * n) return;
  out[i] = (float)((double)acc[i] * ((double)scaleA * (double)scaleB[i % n]));
}

}  // namespace
}  // namespace tfcc_rocm

using namespace tfcc_rocm;

extern "C" int tfcc_rocm_gemv_u8s8s32(void* stream, const uint8_t* a, const int8_t* b,
                                      const int32_t* rowsum_a, const int32_t* colsum_b,
                                      int32_t offset_a, int32_t offset_b, unsigned m, unsigned n,
                                      unsigned k, int32_t* acc_out, float scale_a,
                                      const float* scale_b, float* f32_out) {
  return tfcc_rocm_gemv_u8s8s32_flags(stream, a, b, rowsum_a, colsum_b, offset_a, offset_b, m, n, k, acc_out, scale_a,
                                      scale_b, f32_out, 0u);
}

extern "C" int tfcc_rocm_gemv_u8s8s32_flags(void* stream, const uint8_t* a, const int8_t* b,
                                            const int32_t* rowsum_a, const int32_t* colsum_b,
                                            int32_t offset_a, int32_t offset_b, unsigned m, unsigned n,
                                            unsigned k, int32_t* acc_out, float scale_a,
                                            const float* scale_b, float* f32_out, unsigned flags) {
  TFCC_REQUIRE((flags & ~(unsigned)TFCC_ROCM_GEMV_COLSUM_B_IS_EXACT) == 0, "skinny quantized matmul: unknown flags %#x", flags);
  const bool colsumExact = (flags & TFCC_ROCM_GEMV_COLSUM_B_IS_EXACT) != 0;
  TFCC_REQUIRE(a && b && rowsum_a && colsum_b, "skinny quantized matmul: null operand");
  TFCC_REQUIRE(m > 0 && n > 0 && k > 0, "skinny quantized matmul: empty operand");
  TFCC_REQUIRE(acc_out || f32_out, "skinny quantized matmul: no output");
  TFCC_REQUIRE(!f32_out || scale_b, "skinny quantized matmul: dequantize needs scale_b");
  hipStream_t s = as_stream(stream);
  if (gemv_supported(a, b, m, n, k))
    return gemv_launch(s, a, reinterpret_cast<const signed char*>(b), rowsum_a, colsum_b, offset_a,
                       offset_b, nullptr, nullptr, m, n, k, acc_out, scale_a, scale_b, f32_out, colsumExact);
  // shapes the skinny kernel does not take (m > 8, unaligned): general kernel, then dequantize
  TFCC_REQUIRE(acc_out != nullptr, "skinny quantized matmul: this shape needs acc_out (m > 8 or unaligned operands)");
  tfcc_rocm_qgemm_desc d{};
  d.a = a; d.b = b; d.rowsum_a = rowsum_a; d.colsum_b = colsum_b;
  d.m = m; d.n = n; d.k = k; d.batch = 1; d.stride_c = (uint64_t)m * n;
  d.offset_a = offset_a; d.offset_b = offset_b;
  d.colsum_b_is_exact = colsumExact ? 1 : 0;
  if (int e = tfcc_rocm_gemm_u8s8s32(stream, &d, acc_out)) return e;
  if (f32_out) {
    size_t total = (size_t)m * n;
    hipLaunchKernelGGL(dequant_per_channel_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s,
                       acc_out, m, n, scale_a, scale_b, f32_out);
    return check_launch("per-channel dequantize");
  }
  return TFCC_ROCM_OK;
}

// The same product for callers that cannot allocate: the workspace of the kernel that splits K lies inside the
// library's image, one per GPU.
extern "C" int tfcc_rocm_gemv_u8s8s32_noalloc(void* stream, const uint8_t* a, const int8_t* b,
                                              const int32_t* rowsum_a, const int32_t* colsum_b,
                                              int32_t offset_a, int32_t offset_b, unsigned m, unsigned n,
                                              unsigned k, int32_t* acc_out, float scale_a,
                                              const float* scale_b, float* f32_out) {
  TFCC_REQUIRE(a && b && rowsum_a && colsum_b, "skinny quantized matmul: null operand");
  TFCC_REQUIRE(m > 0 && n > 0 && k > 0, "skinny quantized matmul: empty operand");
  TFCC_REQUIRE(acc_out || f32_out, "skinny quantized matmul: no output");
  TFCC_REQUIRE(!f32_out || scale_b, "skinny quantized matmul: dequantize needs scale_b");
  hipStream_t s = as_stream(stream);
  const signed char* bs = reinterpret_cast<const signed char*>(b);
  if (gemv_wide_supported(a, b, m, n, k) && n <= gemv_wide_static_max_n())
    return gemv_wide_launch(s, true, a, bs, rowsum_a, colsum_b, offset_a, offset_b, nullptr, nullptr, m, n, k, acc_out,
                            scale_a, scale_b, f32_out);
  // small or narrow products, and those wider than the workspace inside the library: the kernel that owns its columns
  // over the whole of K uses no workspace at all
  TFCC_REQUIRE(gemv_supported(a, b, m, n, k),
               "skinny quantized matmul without allocation: at most 8 rows, n a multiple of 4, k a multiple of 16, a aligned "
               "to 16 bytes, n * k below 2^31 (beyond the %u columns of the workspace inside the library only the kernel "
               "without a workspace applies)", gemv_wide_static_max_n());
  return gemv_onepass_launch(s, a, bs, rowsum_a, colsum_b, offset_a, offset_b, nullptr, nullptr, m, n, k, acc_out, scale_a,
                             scale_b, f32_out);
}

extern "C" size_t tfcc_rocm_gemv_packed_size(unsigned n, unsigned k) {
  return (size_t)((n + 15) / 16) * ((k + 63) / 64) * 1024;
}

extern "C" int tfcc_rocm_gemv_pack_b(void* stream, const int8_t* b, unsigned n, unsigned k, void* packed) {
  TFCC_REQUIRE(b && packed, "pack: null argument");
  TFCC_REQUIRE(n > 0 && k > 0, "pack: empty operand");
  TFCC_REQUIRE((uintptr_t)packed % 16 == 0, "pack: the packed buffer must be 16-byte aligned");
  const unsigned steps = (k + 63) / 64;
  const size_t chunks = tfcc_rocm_gemv_packed_size(n, k) / 16;
  TFCC_REQUIRE((chunks + 255) / 256 < (1ull << 31), "pack: operand too large");
  hipLaunchKernelGGL(gemv_pack_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, as_stream(stream),
                     reinterpret_cast<const signed char*>(b), n, k, steps, chunks, static_cast<unsigned char*>(packed));
  return check_launch("pack");
}

namespace tfcc_rocm {
bool gemv_packed_supported(const void* a, const void* packed, unsigned m, unsigned k) {
  return m >= 1 && m <= (unsigned)kMaxM && k % 16 == 0 && (uintptr_t)a % 16 == 0 && (uintptr_t)packed % 16 == 0 &&
         (unsigned long long)m * k < (1ull << 31);
}

int gemv_packed_launch(hipStream_t stream, const unsigned char* a, const void* packed, const int* rowsumA,
                       const int* colsumB, int offsetA, int offsetB, const float* const ranges[4],
                       float* const rangeOut[2], unsigned m, unsigned n, unsigned k, int* accOut, float scaleA,
                       const float* scaleB, float* f32Out) {
  GemvParams p{};
  if (ranges && ranges[0]) {
    p.minA = ranges[0]; p.maxA = ranges[1]; p.minB = ranges[2]; p.maxB = ranges[3];
    if (rangeOut) { p.minC = rangeOut[0]; p.maxC = rangeOut[1]; }
  }
  p.A = a; p.rowsumA = rowsumA; p.colsumB = colsumB; p.accOut = accOut; p.f32Out = f32Out;
  p.scaleA = scaleA; p.scaleB = scaleB; p.offsetA = offsetA; p.offsetB = offsetB;
  p.M = m; p.N = n; p.K = k;
  const unsigned steps = (k + 63) / 64;
  const size_t aBytes = (size_t)m * (steps * 64 + 16);
  if (aBytes <= 96 * 1024) {
    auto kern = gemv_packed_kernel<true>;
    if (aBytes > 48 * 1024) {
      static bool attrSet[16] = {};  // per device
      int dev = 0;
      TFCC_HIP_CHECK(hipGetDevice(&dev));
      TFCC_REQUIRE(dev >= 0 && dev < 16, "device index %d", dev);
      if (!attrSet[dev]) {
        TFCC_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           96 * 1024));
        attrSet[dev] = true;
      }
    }
    hipLaunchKernelGGL(kern, dim3((n + 15) / 16), dim3(kPackThreads), aBytes, stream, p,
                       static_cast<const unsigned char*>(packed), steps);
  } else {
    hipLaunchKernelGGL(gemv_packed_kernel<false>, dim3((n + 15) / 16), dim3(kPackThreads), 0, stream, p,
                       static_cast<const unsigned char*>(packed), steps);
  }
  return check_launch("skinny quantized matmul (packed)");
}
}  // namespace tfcc_rocm

extern "C" int tfcc_rocm_gemv_u8s8s32_packed(void* stream, const uint8_t* a, const void* packed_b,
                                             const int32_t* rowsum_a, const int32_t* colsum_b, int32_t offset_a,
                                             int32_t offset_b, unsigned m, unsigned n, unsigned k, int32_t* acc_out,
                                             float scale_a, const float* scale_b, float* f32_out) {
  TFCC_REQUIRE(a && packed_b && rowsum_a && colsum_b, "skinny quantized matmul: null operand");
  TFCC_REQUIRE(m > 0 && n > 0 && k > 0, "skinny quantized matmul: empty operand");
  TFCC_REQUIRE(m <= (unsigned)kMaxM, "skinny quantized matmul on packed weights: at most %d rows", kMaxM);
  TFCC_REQUIRE(k % 16 == 0 && (uintptr_t)a % 16 == 0 && (uintptr_t)packed_b % 16 == 0,
               "skinny quantized matmul on packed weights: k and the operands must be multiples of / aligned to 16");
  TFCC_REQUIRE((unsigned long long)m * k < (1ull << 31), "skinny quantized matmul: operand too large");
  TFCC_REQUIRE(acc_out || f32_out, "skinny quantized matmul: no output");
  TFCC_REQUIRE(!f32_out || scale_b, "skinny quantized matmul: dequantize needs scale_b");
  return gemv_packed_launch(as_stream(stream), a, packed_b, rowsum_a, colsum_b, offset_a, offset_b, nullptr, nullptr, m, n,
                            k, acc_out, scale_a, scale_b, f32_out);
}
