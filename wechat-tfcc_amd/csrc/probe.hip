// Register-resident matrix-core loops: what the matrix cores of this part sustain when nothing else
// limits them (no LDS, no memory), with operands that stay the same from one instruction to the next
// and with operands that change every instruction, as the rows and columns of real matrices do.
// A measuring aid for the benchmark (it says how far a GEMM kernel is from what the hardware delivers
// at the clocks its power limit allows).  Built into the benchmark's own library, not the product's.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "probe.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

__device__ __forceinline__ unsigned hash32(unsigned x) {
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}

// Four accumulators per wavefront (independent instructions back to back), four operand pairs.
template <bool CHANGING>
__global__ __launch_bounds__(256) void probe_i8_kernel(unsigned iters, int* out) {
  const unsigned id = blockIdx.x * 256 + threadIdx.x;
  v4i a[4], b[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const unsigned s = CHANGING ? id * 8 + q : 0x01020304u;  // the same bytes in every lane and register, or noise
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      a[q][e] = (int)(CHANGING ? hash32(s * 4 + e) : s);
      b[q][e] = (int)(CHANGING ? hash32(s * 4 + e + 0x9e3779b9u) : s);
    }
  }
  v16i c[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) c[j][r] = 0;
  for (unsigned i = 0; i < iters; i += 4) {  // iters is a multiple of 4
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int j = 0; j < 4; ++j) c[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[j], b[(j + q) & 3], c[j], 0, 0, 0);
  }
  int s = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += c[j][r];
  out[id] = s;
}

// The same instruction (kind 0) and the 16x16x64 one (kind 2) issued the way a GEMM kernel issues them: a wavefront
// owns 128 x 128 outputs (all 256 accumulation registers), holds the operands of one k step in registers (4 + 4
// quads for 32x32x32, 8 + 8 for 16x16x64) and walks the blocks row by row, every other row backwards, so that one
// operand stays put for a whole row of blocks and the other changes with every instruction.  HOLD_SRC0 says which
// source of the instruction is the one that stays.  After every k step all operand registers are xored with a
// per-lane constant: half of their bits flip, as they do when the next step's data arrives.
// SLEEP > 0: after every k step the wavefront sleeps 64 * SLEEP cycles, which sets the share of time the matrix
// cores are busy (16 instructions of 32 cycles per step): 1 -> 0.89, 2 -> 0.80, 4 -> 0.67, 8 -> 0.50.
template <bool HOLD_SRC0, int SLEEP = 0>
__global__ __launch_bounds__(256) void probe_i8_tile32_kernel(unsigned ksteps, int* out) {
  const unsigned id = blockIdx.x * 256 + threadIdx.x;
  v4i ua[4], ub[4];
#pragma unroll
  for (int q = 0; q < 4; ++q)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      ua[q][e] = (int)hash32(id * 64 + q * 4 + e);
      ub[q][e] = (int)hash32(id * 64 + 32 + q * 4 + e);
    }
  const int flipA = (int)hash32(id + 0x51ed270bu), flipB = (int)hash32(id + 0x2545f491u);
  v16i acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
  for (unsigned s = 0; s < ksteps; ++s) {
#pragma unroll
    for (int m = 0; m < 16; ++m) {
      const int i = m / 4, j = m % 4, js = (i & 1) ? 3 - j : j;
      acc[i][js] = HOLD_SRC0 ? __builtin_amdgcn_mfma_i32_32x32x32_i8(ua[i], ub[js], acc[i][js], 0, 0, 0)
                             : __builtin_amdgcn_mfma_i32_32x32x32_i8(ub[js], ua[i], acc[i][js], 0, 0, 0);
    }
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int e = 0; e < 4; ++e) { ua[q][e] ^= flipA; ub[q][e] ^= flipB; }
    if (SLEEP > 0) __builtin_amdgcn_s_sleep(SLEEP);
  }
  int t = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) t += acc[i][j][r];
  out[id] = t;
}

template <bool HOLD_SRC0>
__global__ __launch_bounds__(256) void probe_i8_tile16_kernel(unsigned ksteps, int* out) {
  const unsigned id = blockIdx.x * 256 + threadIdx.x;
  v4i ua[8], ub[8];
#pragma unroll
  for (int q = 0; q < 8; ++q)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      ua[q][e] = (int)hash32(id * 64 + q * 4 + e);
      ub[q][e] = (int)hash32(id * 64 + 32 + q * 4 + e);
    }
  const int flipA = (int)hash32(id + 0x51ed270bu), flipB = (int)hash32(id + 0x2545f491u);
  v4i acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = v4i{0, 0, 0, 0};
  for (unsigned s = 0; s < ksteps; ++s) {
#pragma unroll
    for (int m = 0; m < 64; ++m) {
      const int i = m / 8, j = m % 8, js = (i & 1) ? 7 - j : j;
      acc[i][js] = HOLD_SRC0 ? __builtin_amdgcn_mfma_i32_16x16x64_i8(ua[i], ub[js], acc[i][js], 0, 0, 0)
                             : __builtin_amdgcn_mfma_i32_16x16x64_i8(ub[js], ua[i], acc[i][js], 0, 0, 0);
    }
#pragma unroll
    for (int q = 0; q < 8; ++q)
#pragma unroll
      for (int e = 0; e < 4; ++e) { ua[q][e] ^= flipA; ub[q][e] ^= flipB; }
  }
  int t = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) t += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
  out[id] = t;
}

// 16x16x64 with the operand pattern of probe_i8_kernel: four accumulators, both operands change every instruction
template <bool CHANGING>
__global__ __launch_bounds__(256) void probe_i8_16_kernel(unsigned iters, int* out) {
  const unsigned id = blockIdx.x * 256 + threadIdx.x;
  v4i a[4], b[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const unsigned s = CHANGING ? id * 8 + q : 0x01020304u;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      a[q][e] = (int)(CHANGING ? hash32(s * 4 + e) : s);
      b[q][e] = (int)(CHANGING ? hash32(s * 4 + e + 0x9e3779b9u) : s);
    }
  }
  v4i c[4] = {v4i{0, 0, 0, 0}, v4i{0, 0, 0, 0}, v4i{0, 0, 0, 0}, v4i{0, 0, 0, 0}};
  for (unsigned i = 0; i < iters; i += 4) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int j = 0; j < 4; ++j) c[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[j], b[(j + q) & 3], c[j], 0, 0, 0);
  }
  int s = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) s += c[j][0] + c[j][1] + c[j][2] + c[j][3];
  out[id] = s;
}

template <bool CHANGING>
__global__ __launch_bounds__(256) void probe_f32_kernel(unsigned iters, int* out) {
  const unsigned id = blockIdx.x * 256 + threadIdx.x;
  float a[4], b[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    a[q] = CHANGING ? (float)(hash32(id * 8 + q) & 0xffff) / 65536.f - 0.5f : 0.5f;
    b[q] = CHANGING ? (float)(hash32(id * 8 + q + 4) & 0xffff) / 65536.f - 0.5f : 0.25f;
  }
  v16f c[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) c[j][r] = 0.f;
  for (unsigned i = 0; i < iters; i += 4) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int j = 0; j < 4; ++j) c[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], b[(j + q) & 3], c[j], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += c[j][r];
  out[id] = (int)s;
}

// Streams `bytes` once: workgroup w reads a contiguous share with 16-byte loads, 16 of them in flight
// per lane.  Nothing is written (one word, never in practice): the time of a launch is what a kernel
// bound by reading that many bytes cannot beat on this part.
__global__ __launch_bounds__(512) void probe_read_kernel(const unsigned char* src, unsigned long long bytes, int* out) {
  const unsigned long long per = ((bytes / gridDim.x) + 15) / 16 * 16;
  const unsigned long long lo = blockIdx.x * per, hi = lo + per < bytes ? lo + per : bytes;
  v4i acc = {0, 0, 0, 0};
  unsigned long long i = lo + threadIdx.x * 16ull;
  for (; i + 15ull * 512 * 16 + 16 <= hi; i += 16ull * 512 * 16) {
    v4i v[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) v[u] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(src + i + u * (512ull * 16)));
#pragma unroll
    for (int u = 0; u < 16; ++u) acc += v[u];
  }
  for (; i + 16 <= hi; i += 512ull * 16) acc += __builtin_nontemporal_load(reinterpret_cast<const v4i*>(src + i));
  const int s = acc[0] + acc[1] + acc[2] + acc[3];
  if (s == 0x12345678) out[0] = s;
}

__global__ void probe_empty_kernel(int* out) {
  if (out == nullptr && threadIdx.x == 1024) __builtin_trap();  // never: keeps the kernel from being dropped
}

// 0 = ok, 1 = bad argument, 2 = launch failed
int launched() { return hipGetLastError() == hipSuccess ? 0 : 2; }

}  // namespace

extern "C" int tfcc_bench_probe_read(void* stream, const void* src, uint64_t bytes, unsigned blocks, int32_t* out) {
  if (!(src && out)) return 1;
  if (!(bytes >= 16 && (uintptr_t)src % 16 == 0 && blocks > 0 && blocks <= 65536)) return 1;
  hipLaunchKernelGGL(probe_read_kernel, dim3(blocks), dim3(512), 0, reinterpret_cast<hipStream_t>(stream),
                     static_cast<const unsigned char*>(src), (unsigned long long)bytes, out);
  return launched();
}

extern "C" int tfcc_bench_probe_launch(void* stream, int32_t* out) {
  if (!(out != nullptr)) return 1;
  hipLaunchKernelGGL(probe_empty_kernel, dim3(256), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), out);
  return launched();
}

extern "C" int tfcc_bench_probe_mfma_duty(void* stream, int sleep, unsigned blocks, unsigned ksteps, int32_t* out) {
  if (!(out != nullptr && blocks > 0 && blocks <= 65536 && ksteps > 0)) return 1;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const dim3 g(blocks), b(256);
  switch (sleep) {
    case 0: hipLaunchKernelGGL((probe_i8_tile32_kernel<false, 0>), g, b, 0, s, ksteps, out); break;
    case 1: hipLaunchKernelGGL((probe_i8_tile32_kernel<false, 1>), g, b, 0, s, ksteps, out); break;
    case 2: hipLaunchKernelGGL((probe_i8_tile32_kernel<false, 2>), g, b, 0, s, ksteps, out); break;
    case 4: hipLaunchKernelGGL((probe_i8_tile32_kernel<false, 4>), g, b, 0, s, ksteps, out); break;
    case 8: hipLaunchKernelGGL((probe_i8_tile32_kernel<false, 8>), g, b, 0, s, ksteps, out); break;
    default: return 1;
  }
  return launched();
}

extern "C" int tfcc_bench_probe_mfma(void* stream, int kind, int changing_operands, unsigned blocks, unsigned iters,
                                    int32_t* out) {
  if (!(out != nullptr)) return 1;
  if (!(blocks > 0 && blocks <= 65536 && iters > 0 && iters % 4 == 0)) return 1;
  if (!(kind == 0 || kind == 1 || kind == 2)) return 1;
  if (!(changing_operands >= 0 && changing_operands <= (kind == 1 ? 1 : 3))) return 1;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const dim3 g(blocks), b(256);
  if (kind == 0) {
    if (changing_operands == 3) hipLaunchKernelGGL(probe_i8_tile32_kernel<true>, g, b, 0, s, iters, out);
    else if (changing_operands == 2) hipLaunchKernelGGL(probe_i8_tile32_kernel<false>, g, b, 0, s, iters, out);
    else if (changing_operands) hipLaunchKernelGGL(probe_i8_kernel<true>, g, b, 0, s, iters, out);
    else hipLaunchKernelGGL(probe_i8_kernel<false>, g, b, 0, s, iters, out);
  } else if (kind == 2) {
    if (changing_operands == 3) hipLaunchKernelGGL(probe_i8_tile16_kernel<true>, g, b, 0, s, iters, out);
    else if (changing_operands == 2) hipLaunchKernelGGL(probe_i8_tile16_kernel<false>, g, b, 0, s, iters, out);
    else if (changing_operands) hipLaunchKernelGGL(probe_i8_16_kernel<true>, g, b, 0, s, iters, out);
    else hipLaunchKernelGGL(probe_i8_16_kernel<false>, g, b, 0, s, iters, out);
  } else {
    if (changing_operands) hipLaunchKernelGGL(probe_f32_kernel<true>, g, b, 0, s, iters, out);
    else hipLaunchKernelGGL(probe_f32_kernel<false>, g, b, 0, s, iters, out);
  }
  return launched();
}
