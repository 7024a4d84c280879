// fp32 matmul for up to eight rows of A (one decode step, one recurrent step): the product is bound by the single
// pass over B, so it runs on the vector ALUs with B streamed straight from memory and no tile staging.
//
// A workgroup of sixteen wavefronts owns 64 (or 32) columns.  Wavefront w walks rows [w * per, (w + 1) * per) of B
// in chunks of 64, one column per lane (a row of B is read as 256 contiguous bytes per wavefront, or two rows as
// 128 bytes each), eight rows in flight per lane, and keeps one accumulator per row of A.  The values of A are the
// same for every lane of a group: they go through a piece of LDS private to the wavefront.  The partial sums of
// an element are then added in a fixed order (wavefronts ascending, lane groups ascending) through LDS, so a
// result does not depend on timing.  Bias, residual and the erf-form GELU follow with the expressions of the tiled
// kernels' epilogue (sgemm.hip), which are those of tfcc::blas::matmul(a, b, bias) on the reference's CPU device
// (tfcc/mkl/interfaces/tfcc_mklblasinterface.cpp:127-190) followed by its element-wise kernels.
#include "sgemm_params.hpp"

namespace tfcc_rocm {
namespace {

using sgemm_detail::SgemmParams;

constexpr int kWaves = 16;  // wavefronts of a workgroup, each with its own range of K
constexpr int kRows = 8;    // rows of B a lane has in flight
constexpr int kChunk = 64;  // rows of K whose values of A a wavefront holds in LDS at a time

// COLS columns per wavefront (64 or 32): the 64 / COLS groups of COLS lanes take consecutive pieces of each
// 64-row chunk, so a narrow B still spreads over many workgroups while every load covers whole 128-byte lines.
//
// The streaming part shared by the kernels below: the partial sums of rows 0 .. MR-1 of A times columns
// colBase .. colBase + COLS - 1 of B, left in smem[wave][row][lane] for all sixteen wavefronts (barrier included).
template <int MR, int COLS>
__device__ __forceinline__ void stream_partial_sums(const float* __restrict__ A, unsigned lda, unsigned M,
                                                    const float* __restrict__ B, unsigned ldb, unsigned N, unsigned K,
                                                    unsigned colBase, float (*smem)[MR][64]) {
  constexpr int SUBS = 64 / COLS;       // lane groups of a wavefront
  constexpr int PIECE = kChunk / SUBS;  // rows of a chunk per lane group
  static_assert(PIECE % kRows == 0, "whole batches of rows per lane group");
  const unsigned lane = threadIdx.x & 63;
  const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const unsigned sub = lane / COLS, lcol = lane % COLS;
  const unsigned col = colBase + lcol;
  const unsigned colRead = col < N ? col : N - 1;  // lanes past the edge read a valid column and drop the sum

  // rows of A beyond M repeat the last one; their sums are never stored
  const float* __restrict__ arow[MR];
#pragma unroll
  for (int m = 0; m < MR; ++m) arow[m] = A + (size_t)((unsigned)m < M ? m : M - 1) * lda;

  const unsigned per = ((K + kWaves * kChunk - 1) / (kWaves * kChunk)) * kChunk;
  const unsigned k0 = min(K, wave * per), k1 = min(K, k0 + per);
  float acc[MR];
#pragma unroll
  for (int m = 0; m < MR; ++m) acc[m] = 0.f;

  // Lane l fetches value l of every row of A for the chunk; each lane group then reads its piece back, four
  // values per instruction.  The piece of LDS is this wavefront's own: no barrier is involved.
  float (*mine)[64] = smem[wave];
  for (unsigned k = k0; k < k1; k += kChunk) {
    const unsigned rows = min((unsigned)kChunk, k1 - k);
#pragma unroll
    for (int m = 0; m < MR; ++m) mine[m][lane] = lane < rows ? arow[m][k + lane] : 0.f;
    const float* __restrict__ bp = B + (size_t)(k + sub * PIECE) * ldb + colRead;
    if (rows == (unsigned)kChunk) {
#pragma unroll
      for (int r = 0; r < PIECE; r += kRows) {
        float b[kRows];
#pragma unroll
        for (int u = 0; u < kRows; ++u) b[u] = bp[(size_t)(r + u) * ldb];
#pragma unroll
        for (int m = 0; m < MR; ++m) {
#pragma unroll
          for (int q = 0; q < kRows; q += 4) {
            const float4 a4 = *reinterpret_cast<const float4*>(&mine[m][sub * PIECE + r + q]);
            acc[m] = fmaf(a4.x, b[q], acc[m]);
            acc[m] = fmaf(a4.y, b[q + 1], acc[m]);
            acc[m] = fmaf(a4.z, b[q + 2], acc[m]);
            acc[m] = fmaf(a4.w, b[q + 3], acc[m]);
          }
        }
      }
    } else {
      for (unsigned r = 0; r < (unsigned)PIECE && sub * PIECE + r < rows; ++r) {
        const float b = bp[(size_t)r * ldb];
#pragma unroll
        for (int m = 0; m < MR; ++m) acc[m] = fmaf(mine[m][sub * PIECE + r], b, acc[m]);
      }
    }
  }

#pragma unroll
  for (int m = 0; m < MR; ++m) smem[wave][m][lane] = acc[m];
  __syncthreads();
}

// element (row, column c of the workgroup's COLS): wavefronts in order, lane groups in order within each
template <int MR, int COLS>
__device__ __forceinline__ float summed(float (*smem)[MR][64], unsigned row, unsigned c) {
  float v = 0.f;
#pragma unroll
  for (int w = 0; w < kWaves; ++w)
#pragma unroll
    for (int g = 0; g < 64 / COLS; ++g) v += smem[w][row][g * COLS + c];
  return v;
}

template <int MR, int COLS>
__global__ __launch_bounds__(kWaves * 64) void sgemv_kernel(SgemmParams p) {
  // [wave][row of A][64]: first each wavefront's current 64 values of every row of A, at the end its partial sums
  __shared__ __attribute__((aligned(16))) float smem[kWaves][MR][64];
  const unsigned lane = threadIdx.x & 63;
  const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const unsigned bi = blockIdx.y;
  const unsigned M = p.M, N = p.N;
  const unsigned bo = bi / p.batchInner, bn = bi - bo * p.batchInner;
  const float* __restrict__ A = p.A + (size_t)bo * p.strideA + (size_t)bn * p.innerA;
  const float* __restrict__ B = p.B + (size_t)bo * p.strideB + (size_t)bn * p.innerB;
  const float* biasPtr = p.bias;
  float* Cbase = p.C + (size_t)bo * p.strideC + (size_t)bn * p.innerC;
  if (p.groups) {
    B = bi == 0 ? p.groupB[0] : bi == 1 ? p.groupB[1] : bi == 2 ? p.groupB[2] : p.groupB[3];
    biasPtr = bi == 0 ? p.groupBias[0] : bi == 1 ? p.groupBias[1] : bi == 2 ? p.groupBias[2] : p.groupBias[3];
    Cbase = bi == 0 ? p.groupC[0] : bi == 1 ? p.groupC[1] : bi == 2 ? p.groupC[2] : p.groupC[3];
  }
  stream_partial_sums<MR, COLS>(A, p.lda, M, B, p.ldb, N, p.K, blockIdx.x * COLS, smem);
  // row m of the result is finished by wavefront m
  const unsigned col = blockIdx.x * COLS + lane;
  if (wave < (unsigned)MR && wave < M && lane < (unsigned)COLS && col < N) {
    float v = summed<MR, COLS>(smem, wave, lane);
    if (biasPtr) v += biasPtr[col];
    if (p.residual) v += p.residual[(size_t)bi * p.strideR + (size_t)wave * N + col];
    if (p.act == 1) v = gelu_erf_f32(v);
    Cbase[(size_t)wave * p.ldc + col] = v;
  }
}

// One LSTM time step in one launch: the product of the previous h with the state kernel, streamed as above, and
// the cell (tfcc/mkl/kernel/tfcc_mklcellkernel.hpp:51-87, the expressions of lstm_cell_kernel in cell.hip) on the
// finished sums.  The state kernel is given with its gates interleaved - column 4 u + g holds gate g (i, c, f, o)
// of unit u - so that the 32 columns of a workgroup are the four gates of 8 units and still contiguous.
struct LstmStepParams {
  const float* hPrev;        // [batch, units]
  const float* kernel;       // [units, units * 4], gates interleaved
  const float* inputValue;   // [batch, 4 * units], gate-major as the reference lays it out
  const float* bias;         // [4 * units], gate-major
  const float* stateC;       // [batch, units]
  float* h;                  // [batch, units]; not hPrev
  float* cs;                 // [batch, units]; may be stateC
  unsigned batch, units;
  float forget;
};

__device__ __forceinline__ float sigmoid_value(float v) { return 1.f / (1.f + expf(0.f - v)); }

template <int MR>
__global__ __launch_bounds__(kWaves * 64) void lstm_step_kernel(LstmStepParams p) {
  constexpr int COLS = 32, UNITS = COLS / 4;
  __shared__ __attribute__((aligned(16))) float smem[kWaves][MR][64];
  const unsigned units = p.units;
  // Thread (row m, column c of the workgroup's 32 = unit j, gate g) finishes one gate: it fetches what that needs
  // besides the sum now, not after the barrier.  The four gates of a (row, unit) pair sit in neighbouring lanes.
  const unsigned tid = threadIdx.x, m = tid / COLS, c = tid % COLS, j = c / 4, g = c % 4, u = blockIdx.x * UNITS + j;
  const bool finisher = m < (unsigned)MR;                  // whole wavefronts (or the lower half of one)
  const bool valid = finisher && m < p.batch && u < units;
  const size_t idx = (size_t)m * units + u;
  float xin = 0.f, bv = 0.f, cPrev = 0.f;
  if (valid) {
    xin = p.inputValue[(size_t)m * 4 * units + (size_t)g * units + u];
    bv = p.bias[(size_t)g * units + u];
    if (g == 0) cPrev = p.stateC[idx];
  }
  stream_partial_sums<MR, COLS>(p.hPrev, units, p.batch, p.kernel, 4 * units, 4 * units, units, blockIdx.x * COLS, smem);
  if (finisher) {
    float pre = xin + summed<MR, COLS>(smem, m, c) + bv;
    if (g == 2) pre += p.forget;
    const float act = g == 1 ? tanhf(pre) : sigmoid_value(pre);
    const int base = (int)(threadIdx.x & 63u) & ~3;
    const float xi = __shfl(act, base, 64), xc = __shfl(act, base + 1, 64), xf = __shfl(act, base + 2, 64),
                xo = __shfl(act, base + 3, 64);
    if (valid && g == 0) {
      const float cs = __fadd_rn(__fmul_rn(xc, xi), __fmul_rn(cPrev, xf));
      p.h[idx] = tanhf(cs) * xo;
      p.cs[idx] = cs;
    }
  }
}

template <int MR, int COLS>
int launch_rows(hipStream_t stream, const SgemmParams& p) {
  hipLaunchKernelGGL((sgemv_kernel<MR, COLS>), dim3((p.N + COLS - 1) / COLS, p.batch), dim3(kWaves * 64), 0, stream, p);
  return check_launch("sgemv");
}

template <int COLS>
int launch_width(hipStream_t stream, const SgemmParams& p) {
  if (p.M == 1) return launch_rows<1, COLS>(stream, p);
  if (p.M == 2) return launch_rows<2, COLS>(stream, p);
  if (p.M <= 4) return launch_rows<4, COLS>(stream, p);
  return launch_rows<8, COLS>(stream, p);
}

}  // namespace

namespace sgemm_detail {

bool sgemv_supported(const SgemmParams& p) { return p.M >= 1 && p.M <= 8 && p.batch <= 65535u && p.N < (1u << 30); }

// 64 columns per wavefront read B in the longest runs (8 x 4096 x 11008: 37 us against 50 with 32 columns); below
// 160 such column blocks too few CUs take part, and 32 columns per wavefront with twice the workgroups are faster
// (8 x 4096 x 8192: 30.8 against 36.2 us, 4096 x 4096: 23.4 against 30.1; 16 columns read B in 64-byte pieces and
// lose: 25.2).  The choice depends on N alone, so that a product is summed the same way alone and in a group.
int sgemv_launch(hipStream_t stream, const SgemmParams& p) {
  return p.N >= 10240 ? launch_width<64>(stream, p) : launch_width<32>(stream, p);
}

}  // namespace sgemm_detail
}  // namespace tfcc_rocm

using namespace tfcc_rocm;

extern "C" int tfcc_rocm_lstm_step_f32(void* stream, unsigned batch, unsigned units, const float* h_prev,
                                       const float* state_kernel_interleaved, const float* input_value,
                                       const float* bias, float forget, const float* state_c, float* h, float* cs) {
  TFCC_REQUIRE(h_prev && state_kernel_interleaved && input_value && bias && state_c && h && cs, "lstm_step: null argument");
  TFCC_REQUIRE(batch >= 1 && batch <= 8, "lstm_step: 1 to 8 rows per step, got %u", batch);
  TFCC_REQUIRE(units >= 1 && units < (1u << 28), "lstm_step: %u units", units);
  TFCC_REQUIRE(h != h_prev, "lstm_step: h must not be the previous h (other workgroups still read it)");
  LstmStepParams p{h_prev, state_kernel_interleaved, input_value, bias, state_c, h, cs, batch, units, forget};
  const dim3 grid((units + 7) / 8), block(kWaves * 64);
  hipStream_t s = as_stream(stream);
  if (batch == 1) hipLaunchKernelGGL(lstm_step_kernel<1>, grid, block, 0, s, p);
  else if (batch == 2) hipLaunchKernelGGL(lstm_step_kernel<2>, grid, block, 0, s, p);
  else if (batch <= 4) hipLaunchKernelGGL(lstm_step_kernel<4>, grid, block, 0, s, p);
  else hipLaunchKernelGGL(lstm_step_kernel<8>, grid, block, 0, s, p);
  return check_launch("lstm_step");
}
