// softmax(Q K^T [/ divisor]) V per batch entry in one launch: key sequences of up to 128 rows with the scores of a
// row block in LDS in one piece (attention_kernel), longer ones in blocks of 128 keys (attention_stream_kernel).
//
// Stands where the reference's runtime runs the attention core of an encoder layer as separate
// operations on tensors in HBM: Matmul (tfcc_runtime/operations/math/matmul.cpp:27-41), Div by a
// value, Softmax (tfcc_runtime/operations/math/softmax.cpp), Matmul again, with base::transpose
// (tfcc/core/operations/tfcc_base.cpp:124-134) before and after.  Here the score matrix of a block of
// 64 query rows never leaves the CU: Q is held in registers, K in LDS, the scores and probabilities in
// LDS, V in registers until the scores are done and then in K's place (70.7 KB, two workgroups per CU).
//
// Every number is computed by the same instruction sequence as in the three separate kernels
// (fp32 32x32x2 matrix ops over ascending k into one accumulator; the softmax of one row by one
// wavefront holding columns l and l + 64), and is rounded to fp32 between the steps, so the result
// equals theirs bit for bit.
#include <float.h>

#include "common.hpp"
#include "qgemm_params.hpp"  // UDiv: division by multiply-high

namespace tfcc_rocm {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kRows = 64;        // query rows per workgroup
constexpr int kThreads = 512;    // eight wavefronts
constexpr int kMaxT = 128;       // key rows
constexpr int kMaxD = 64;        // head width
constexpr int kPitchK = kMaxD + 4;    // floats; 128-bit row reads of 32 consecutive rows hit all banks once
constexpr int kPitchV = kMaxD + 8;    // 32-bit reads of rows r and r + 4 land 32 banks apart
constexpr int kPitchS = kMaxT + 4;
// K and, once the scores are done, V share one region; Q stays in registers.  70.7 KB: two workgroups per CU.
constexpr int kLdsFloats = kMaxT * kPitchV + kRows * kPitchS;

struct AttentionParams {
  const float* Q;
  const float* K;
  const float* V;
  float* O;
  unsigned S, T, D;
  unsigned ldq, ldk, ldv, ldo;
  unsigned long long outerQ, outerK, outerV, outerO;
  unsigned long long innerQ, innerK, innerV, innerO;
  unsigned batchInner, blocksS, total, chunk;
  float divisor;
  int divide;
  const float* mask;  // optional: one value per key column, added to the (divided) scores of every query row
  unsigned long long outerM, innerM;
  unsigned blocksMagic, blocksShift, innerMagic, innerShift;  // division by blocksS and by batchInner as multiply-high
};

// Everything the kernels read of the argument block, named before the first branch: one round trip to memory for it
// instead of one per basic block, at the head of a launch of ten to twenty microseconds.
#define TFCC_ATTENTION_FETCH_ARGUMENTS(p)                                                                              \
  asm volatile("" ::"s"(p.Q), "s"(p.K), "s"(p.V), "s"(p.O), "s"(p.S), "s"(p.T), "s"(p.D), "s"(p.ldq), "s"(p.ldk),      \
               "s"(p.ldv), "s"(p.ldo), "s"(p.outerQ), "s"(p.outerK), "s"(p.outerV), "s"(p.outerO), "s"(p.innerQ),      \
               "s"(p.innerK), "s"(p.innerV), "s"(p.innerO), "s"(p.batchInner), "s"(p.blocksS), "s"(p.total),           \
               "s"(p.chunk), "s"(p.divisor), "s"(p.divide), "s"(p.mask), "s"(p.outerM), "s"(p.innerM),                 \
               "s"(p.blocksMagic), "s"(p.blocksShift), "s"(p.innerMagic), "s"(p.innerShift))


// ROWS query rows per workgroup, a wavefront per eight of them: 64 rows (eight wavefronts, 70.7 KB, two workgroups per
// CU) when every CU gets at most one workgroup that way, 32 rows (four wavefronts, 53.8 KB, three per CU) when the
// 64-row blocks would pile up two on some CUs and one or none on others (16 x 12 heads of 128 rows: 384 blocks of 64
// on 256 CUs against 768 blocks of 32, three on every CU).  The arithmetic per element is the same.
template <int ROWS>
__global__ __launch_bounds__(8 * ROWS, ROWS == 64 ? 4 : 3) void attention_kernel(const AttentionParams p) {
  constexpr int kRows = ROWS, kThreads = 8 * ROWS;
  static_assert(ROWS == 64 || ROWS == 32, "two or one row blocks of 32");
  extern __shared__ __align__(16) float lds[];
  float* KVs = lds;                       // K as [128][kPitchK], later V as [128][kPitchV]
  float* Sc = KVs + kMaxT * kPitchV;      // [64][kPitchS]  scores, then probabilities

  // consecutive workgroup ids land on different XCDs: the blocks of one head stay on one XCD
  const unsigned wg = blockIdx.x;
  TFCC_ATTENTION_FETCH_ARGUMENTS(p);
  const unsigned L = (wg & 7u) * p.chunk + (wg >> 3);
  if ((wg >> 3) >= p.chunk || L >= p.total) return;
  const unsigned bi = udiv_apply(L, p.blocksMagic, p.blocksShift), blk = L - bi * p.blocksS;
  const unsigned bo = udiv_apply(bi, p.innerMagic, p.innerShift), bn = bi - bo * p.batchInner;
  const unsigned s0 = blk * kRows;
  const unsigned S = p.S, T = p.T, D = p.D;
  const float* __restrict__ Q = p.Q + (size_t)bo * p.outerQ + (size_t)bn * p.innerQ;
  const float* __restrict__ K = p.K + (size_t)bo * p.outerK + (size_t)bn * p.innerK;
  const float* __restrict__ V = p.V + (size_t)bo * p.outerV + (size_t)bn * p.innerV;
  float* __restrict__ O = p.O + (size_t)bo * p.outerO + (size_t)bn * p.innerO;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // this lane's two mask values, fetched now: the softmax phase that adds them is far away
  const bool masked = p.mask != nullptr;
  float mk[2] = {0.f, 0.f};
  if (masked) {
    const float* __restrict__ mrow = p.mask + (size_t)bo * p.outerM + (size_t)bn * p.innerM;
#pragma unroll
    for (int q = 0; q < 2; ++q)
      if ((unsigned)lane + 64u * q < T) mk[q] = mrow[lane + 64 * q];
  }
  const int lrow = lane & 31, g = lane >> 5;
  const unsigned Dp = (D + 7u) & ~7u;   // k extent of the score product
  const unsigned Tp = (T + 7u) & ~7u;   // k extent of the second product

  // ---- loads.  K goes to LDS; Q goes through the region the scores will later occupy into the registers
  // the score product takes it from; V waits in registers until K is no longer needed.  A buffer load whose
  // offset lies past the end of its operand returns zero: that is how everything past the operands' extents
  // that a matrix op will read becomes zero.
  const int wmS = wave >> 2, wnS = wave & 3;  // scores: ROWS / 32 x 4 wavefronts, one 32 x 32 block each
  constexpr int CH = kMaxD / 4;               // 16-byte chunks per row
  constexpr int KV_ITEMS = kMaxT * CH / kThreads, Q_ITEMS = kRows * CH / kThreads, KBQ = kMaxD / 8;
  constexpr unsigned kPastEnd = 0xfffffff0u;
  v4f qf[KBQ], vreg[KV_ITEMS];
  {
    const __amdgpu_buffer_rsrc_t rq = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(Q), 0, (int)(((S - 1) * p.ldq + D) * 4u), 0x00020000);
    const __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(K), 0, (int)(((T - 1) * p.ldk + D) * 4u), 0x00020000);
    const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(V), 0, (int)(((T - 1) * p.ldv + D) * 4u), 0x00020000);
    v4f qreg[Q_ITEMS], kreg[KV_ITEMS];
#pragma unroll
    for (int it = 0; it < Q_ITEMS; ++it) {
      const unsigned w = tid + it * kThreads, row = s0 + w / CH, ch = w % CH;
      qreg[it] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(
                                             rq, (row < S && ch * 4 < D) ? (row * p.ldq + ch * 4) * 4u : kPastEnd, 0, 0));
    }
#pragma unroll
    for (int it = 0; it < KV_ITEMS; ++it) {
      const unsigned w = tid + it * kThreads, row = w / CH, ch = w % CH;
      const bool in = row < T && ch * 4 < D;
      kreg[it] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rk, in ? (row * p.ldk + ch * 4) * 4u : kPastEnd, 0, 0));
      vreg[it] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rv, in ? (row * p.ldv + ch * 4) * 4u : kPastEnd, 0, 0));
    }
#pragma unroll
    for (int it = 0; it < KV_ITEMS; ++it) {
      const int w = tid + it * kThreads, row = w / CH, ch = w % CH;
      *reinterpret_cast<v4f*>(KVs + row * kPitchK + ch * 4) = kreg[it];
    }
#pragma unroll
    for (int it = 0; it < Q_ITEMS; ++it) {
      const int w = tid + it * kThreads, row = w / CH, ch = w % CH;
      *reinterpret_cast<v4f*>(Sc + row * kPitchK + ch * 4) = qreg[it];
    }
  }
  __syncthreads();
  {
    const float* qa = Sc + (32 * wmS + lrow) * kPitchK + 4 * g;
#pragma unroll
    for (int kb = 0; kb < KBQ; ++kb) {
      qf[kb] = v4f{0.f, 0.f, 0.f, 0.f};
      if ((unsigned)kb * 8 < Dp) qf[kb] = *reinterpret_cast<const v4f*>(qa + kb * 8);
    }
  }

  // ---- scores.  All K operands are fetched from LDS before the first matrix op, so that their latency
  // is paid once.  A divisor that is a power of two divides exactly like a multiplication by its reciprocal.
  const bool liveS = (unsigned)(32 * wnS) < T;  // wave-uniform: this wavefront's 32 columns exist
  v4f bf[KBQ];
  {
    const float* ka = KVs + (32 * wnS + lrow) * kPitchK + 4 * g;
#pragma unroll
    for (int kb = 0; kb < KBQ; ++kb) {
      bf[kb] = v4f{0.f, 0.f, 0.f, 0.f};
      if (liveS && (unsigned)kb * 8 < Dp) bf[kb] = *reinterpret_cast<const v4f*>(ka + kb * 8);
    }
  }
  __syncthreads();  // every wavefront has taken its Q operands out of the region the scores go to
  if (liveS) {
    v16f acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
    for (int kb = 0; kb < KBQ; ++kb) {
      if ((unsigned)kb * 8 < Dp) {
#pragma unroll
        for (int s = 0; s < 4; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(qf[kb][s], bf[kb][s], acc, 0, 0, 0);
      }
    }
    float* sc = Sc + (32 * wmS + 4 * g) * kPitchS + 32 * wnS + lrow;
    const float divisor = p.divisor;
    const unsigned bits = __builtin_bit_cast(unsigned, divisor), expo = (bits >> 23) & 0xffu;
    if (!p.divide) {
#pragma unroll
      for (int r = 0; r < 16; ++r) sc[(8 * (r / 4) + (r & 3)) * kPitchS] = acc[r];
    } else if ((bits & 0x007fffffu) == 0 && expo >= 2 && expo <= 252) {
      const float inverse = 1.0f / divisor;  // exact: also a power of two
#pragma unroll
      for (int r = 0; r < 16; ++r) sc[(8 * (r / 4) + (r & 3)) * kPitchS] = acc[r] * inverse;
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) sc[(8 * (r / 4) + (r & 3)) * kPitchS] = acc[r] / divisor;
    }
  }
  __syncthreads();

  // ---- K is done with: V takes its place
#pragma unroll
  for (int it = 0; it < KV_ITEMS; ++it) {
    const int w = tid + it * kThreads, row = w / CH, ch = w % CH;
    *reinterpret_cast<v4f*>(KVs + row * kPitchV + ch * 4) = vreg[it];
  }

  // ---- softmax of each row by one wavefront, eight rows in flight; columns T .. Tp-1 become the zeros
  // the next product reads
  {
    const unsigned rows = min((unsigned)kRows, S - s0);
    constexpr int R = 8, W = kThreads / 64;  // R is the eight of wave_reduce8
    for (unsigned base = wave; base < rows; base += W * R) {
      float v[R][2], mx[R], sum[R];
#pragma unroll
      for (int u = 0; u < R; ++u) {
        const unsigned row = min(base + W * u, (unsigned)kRows - 1);  // a row past the block's end is computed and dropped
        const float* sc = Sc + row * kPitchS;
        mx[u] = -FLT_MAX;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          const unsigned i = lane + 64 * q;
          v[u][q] = i < T ? (masked ? sc[i] + mk[q] : sc[i]) : -FLT_MAX;
          mx[u] = fmaxf(mx[u], v[u][q]);
        }
      }
      wave_reduce8<true>(mx, lane);
#pragma unroll
      for (int u = 0; u < R; ++u) {
        sum[u] = 0.f;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          const unsigned i = lane + 64 * q;
          v[u][q] = i < T ? softmax_exp(v[u][q] - mx[u]) : 0.f;
          sum[u] += v[u][q];
        }
      }
      wave_reduce8<false>(sum, lane);
#pragma unroll
      for (int u = 0; u < R; ++u) {
        const unsigned row = base + W * u;
        if (row < rows) {
          float* sc = Sc + row * kPitchS;
          const float inverse = 1.0f / sum[u];  // as the stand-alone softmax: one division per row
#pragma unroll
          for (int q = 0; q < 2; ++q) {
            const unsigned i = lane + 64 * q;
            sc[i] = i < T ? v[u][q] * inverse : 0.f;
          }
        }
      }
    }
  }
  __syncthreads();

  if constexpr (ROWS == 64) {
    // ---- probabilities x V: the first four wavefronts, (wm, wn) owning rows 32*wm.. and columns 32*wn.. of the
    // 64 x D result (one accumulator per element over all of T, as in a product of its own)
    const int wm = wave >> 1, wn = wave & 1;
    if (wave < 4 && (unsigned)(32 * wn) < D) {
      constexpr int KB = kMaxT / 8, HALF = KB / 2;
      v16f acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.f;
      const float* pa = Sc + (32 * wm + lrow) * kPitchS + 4 * g;
      const float* vb = KVs + (4 * g) * kPitchV + 32 * wn + lrow;
#pragma unroll
      for (int h = 0; h < 2; ++h) {  // operands are fetched from LDS for eight steps at a time
        v4f af[HALF], bf[HALF];
#pragma unroll
        for (int q = 0; q < HALF; ++q) {
          const int kb = h * HALF + q;
          af[q] = v4f{0.f, 0.f, 0.f, 0.f};
          bf[q] = v4f{0.f, 0.f, 0.f, 0.f};
          if ((unsigned)kb * 8 < Tp) {
            af[q] = *reinterpret_cast<const v4f*>(pa + kb * 8);
#pragma unroll
            for (int s = 0; s < 4; ++s) bf[q][s] = vb[(kb * 8 + s) * kPitchV];
          }
        }
#pragma unroll
        for (int q = 0; q < HALF; ++q) {
          if ((unsigned)(h * HALF + q) * 8 < Tp) {
#pragma unroll
            for (int s = 0; s < 4; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[q][s], bf[q][s], acc, 0, 0, 0);
          }
        }
      }
      const unsigned col = 32 * wn + lrow;
      if (s0 + 32 * wm + 32 <= S && 32u * wn + 32 <= D && p.ldo < (1u << 24)) {
        // a whole 32 x 32 block: a register per lane (row 4g, column lrow), a scalar per row, no checks
        const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(
            O + (size_t)(s0 + 32 * wm) * p.ldo + 32 * wn, 0, 0x7fffffff, 0x00020000);
        const unsigned voff = ((4 * g) * p.ldo + lrow) * 4u;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float value = acc[r];  // a copy: __builtin_bit_cast applied to a vector element reads element 0
          __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, value), ro, voff,
                                                (8 * (r / 4) + (r & 3)) * p.ldo * 4u, 0);
        }
      } else if (col < D) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const unsigned row = s0 + 32 * wm + 8 * (r / 4) + 4 * g + (r & 3);
          if (row < S) O[(size_t)row * p.ldo + col] = acc[r];
        }
      }
    }
  } else {
    // ---- probabilities x V.  A product of its own sums each element in one accumulator over k in the order
    // 8kb + s, 8kb + 4 + s (s = 0..3) with 32x32x2 matrix ops; the 16x16x4 op adds its four k values to the accumulator
    // one after the other in lane-group order, so feeding lane groups 0..3 the k values 8kb + 2h, 8kb + 4 + 2h,
    // 8kb + 2h + 1, 8kb + 5 + 2h in ops h = 0, 1 gives the same bits - and blocks of 16 x 16 divide the ROWS x D
    // result evenly among all wavefronts: wavefront w owns rows 16 (w / 2).. and the column blocks 2 (w & 1), 2 (w & 1) + 1.
  // With 32 rows this keeps all four SIMDs busy (two 32 x 32 blocks would occupy two); with 64 rows it measured a
  // microsecond slower than the four 32 x 32 blocks above (twice the LDS operand reads, two-way bank conflicts).
    {
      constexpr int KB = kMaxT / 8;
      const int l16 = lane & 15, q = lane >> 4;
      const int rb = wave >> 1, cb0 = 2 * (wave & 1);
      const int kq = (q >> 1) + 4 * (q & 1);  // this lane group's k inside a block of eight, op 0 (op 1: + 2)
      const float* pa = Sc + (16 * rb + l16) * kPitchS + kq;
      const float* vb = KVs + kq * kPitchV + 16 * cb0 + l16;
      const bool live[2] = {(unsigned)(16 * cb0) < D, (unsigned)(16 * cb0 + 16) < D};
      v4f acc[2] = {v4f{0.f, 0.f, 0.f, 0.f}, v4f{0.f, 0.f, 0.f, 0.f}};
      if (live[0]) {
        float af[KB][2], bf[2][KB][2];
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            af[kb][h] = 0.f; bf[0][kb][h] = 0.f; bf[1][kb][h] = 0.f;
          }
          if ((unsigned)kb * 8 < Tp) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
              af[kb][h] = pa[kb * 8 + 2 * h];
              bf[0][kb][h] = vb[(kb * 8 + 2 * h) * kPitchV];
              bf[1][kb][h] = vb[(kb * 8 + 2 * h) * kPitchV + 16];  // columns past D hold zeros
            }
          }
        }
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
          if ((unsigned)kb * 8 < Tp) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
              acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[kb][h], bf[0][kb][h], acc[0], 0, 0, 0);
              acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[kb][h], bf[1][kb][h], acc[1], 0, 0, 0);
            }
          }
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          if (!live[j]) continue;
          const unsigned c0 = 16 * (cb0 + j), r0 = s0 + 16 * rb;
          if (r0 + 16 <= S && c0 + 16 <= D && p.ldo < (1u << 24)) {
            // a whole 16 x 16 block: a register per lane (row 4q, column l16), a scalar per row, no checks
            const __amdgpu_buffer_rsrc_t ro =
                __builtin_amdgcn_make_buffer_rsrc(O + (size_t)r0 * p.ldo + c0, 0, 0x7fffffff, 0x00020000);
            const unsigned voff = ((4 * q) * p.ldo + l16) * 4u;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const float value = acc[j][r];  // a copy: __builtin_bit_cast applied to a vector element reads element 0
              __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, value), ro, voff, r * p.ldo * 4u, 0);
            }
          } else if (c0 + l16 < D) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const unsigned row = r0 + 4 * q + r;
              if (row < S) O[(size_t)row * p.ldo + c0 + l16] = acc[j][r];
            }
          }
        }
      }
    }
  }
}

// ---- the same for key sequences of any length: the keys are walked in blocks of 128 with a running row maximum and
// row sum (m, l).  Per block: scores as above; p = exp(score - m_new) with m_new = max(m, block maximum);
// l = l * exp(m - m_new) + sum(p); the output accumulator of the earlier blocks is scaled by exp(m - m_new) before the
// block's p V is added; at the end every row is divided by its l.  The same real function as the three separate
// kernels, summed in a different order (a row's exponentials are taken against the running maximum and rescaled,
// not against the final one): results agree with them to a few units in the last place, not bit for bit; the
// contract checked is the relative error against double precision.  Blocks of 128 keep the LDS footprint of the
// kernel above (two workgroups per CU) whatever the length.
template <int ROWS>
__global__ __launch_bounds__(8 * ROWS) void attention_stream_kernel(const AttentionParams p) {
  constexpr int kRows = ROWS, kThreads = 8 * ROWS;  // blocks of 64 or 32 query rows, as in attention_kernel
  static_assert(ROWS == 64 || ROWS == 32, "two or one row blocks of 32");
  extern __shared__ __align__(16) float lds[];
  float* KVs = lds;                       // the block's K as [128][kPitchK], then its V as [128][kPitchV]
  float* Sc = KVs + kMaxT * kPitchV;      // [64][kPitchS]  scores, then probabilities of the block
  float* rowScale = Sc + kRows * kPitchS; // [64] what the accumulated rows are multiplied by before the block is added
                                          //      (after the last block: 1 / l)

  const unsigned wg = blockIdx.x;
  TFCC_ATTENTION_FETCH_ARGUMENTS(p);
  const unsigned L = (wg & 7u) * p.chunk + (wg >> 3);
  if ((wg >> 3) >= p.chunk || L >= p.total) return;
  const unsigned bi = udiv_apply(L, p.blocksMagic, p.blocksShift), blk = L - bi * p.blocksS;
  const unsigned bo = udiv_apply(bi, p.innerMagic, p.innerShift), bn = bi - bo * p.batchInner;
  const unsigned s0 = blk * kRows;
  const unsigned S = p.S, T = p.T, D = p.D;
  const float* __restrict__ Q = p.Q + (size_t)bo * p.outerQ + (size_t)bn * p.innerQ;
  const float* __restrict__ K = p.K + (size_t)bo * p.outerK + (size_t)bn * p.innerK;
  const float* __restrict__ V = p.V + (size_t)bo * p.outerV + (size_t)bn * p.innerV;
  float* __restrict__ O = p.O + (size_t)bo * p.outerO + (size_t)bn * p.innerO;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool masked = p.mask != nullptr;
  const float* __restrict__ mrow = masked ? p.mask + (size_t)bo * p.outerM + (size_t)bn * p.innerM : nullptr;
  const int lrow = lane & 31, g = lane >> 5;
  const unsigned Dp = (D + 7u) & ~7u;
  const int wmS = wave >> 2, wnS = wave & 3;  // scores: ROWS / 32 x 4 wavefronts, one 32 x 32 block each
  const int wm = wave >> 1, wn = wave & 1;    // second product: the first half of the wavefronts, ROWS / 32 x 2 blocks of 32 x 32
  constexpr int CH = kMaxD / 4;
  constexpr int KV_ITEMS = kMaxT * CH / kThreads, Q_ITEMS = kRows * CH / kThreads, KBQ = kMaxD / 8;
  constexpr unsigned kPastEnd = 0xfffffff0u;
  const __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(K), 0, (int)(((T - 1) * p.ldk + D) * 4u), 0x00020000);
  const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(V), 0, (int)(((T - 1) * p.ldv + D) * 4u), 0x00020000);

  // ---- Q: through the region of the scores into the registers the score product takes it from, once
  v4f qf[KBQ];
  {
    const __amdgpu_buffer_rsrc_t rq = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(Q), 0, (int)(((S - 1) * p.ldq + D) * 4u), 0x00020000);
#pragma unroll
    for (int it = 0; it < Q_ITEMS; ++it) {
      const unsigned w = tid + it * kThreads, row = w / CH, ch = w % CH;
      const v4f q = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(
                                                rq, (s0 + row < S && ch * 4 < D) ? ((s0 + row) * p.ldq + ch * 4) * 4u : kPastEnd, 0, 0));
      *reinterpret_cast<v4f*>(Sc + row * kPitchK + ch * 4) = q;
    }
    __syncthreads();
    const float* qa = Sc + (32 * wmS + lrow) * kPitchK + 4 * g;
#pragma unroll
    for (int kb = 0; kb < KBQ; ++kb) {
      qf[kb] = v4f{0.f, 0.f, 0.f, 0.f};
      if ((unsigned)kb * 8 < Dp) qf[kb] = *reinterpret_cast<const v4f*>(qa + kb * 8);
    }
  }

  // running maximum and sum of the eight rows this wavefront owns in the softmax step (rows wave + 8 u)
  constexpr int R = 8, W = kThreads / 64;
  static_assert(W * R == kRows, "every row of the block has its wavefront");
  float mrun[R], lrun[R];
#pragma unroll
  for (int u = 0; u < R; ++u) { mrun[u] = -FLT_MAX; lrun[u] = 0.f; }
  // context accumulators: one 32 x 32 block per wavefront of the first half (ROWS = 64), or two 16 x 16 blocks per
  // wavefront of all four (ROWS = 32: rows 16 (wave / 2).., column blocks 2 (wave & 1) and 2 (wave & 1) + 1; see
  // attention_kernel for the order the k values are fed in)
  v16f acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
  v4f acc16[2] = {v4f{0.f, 0.f, 0.f, 0.f}, v4f{0.f, 0.f, 0.f, 0.f}};
  const int l16 = lane & 15, q16 = lane >> 4, rb16 = wave >> 1, cb16 = 2 * (wave & 1);
  const int kq16 = (q16 >> 1) + 4 * (q16 & 1);

  const float divisor = p.divisor;
  const unsigned dbits = __builtin_bit_cast(unsigned, divisor), dexpo = (dbits >> 23) & 0xffu;
  const bool divideByMul = (dbits & 0x007fffffu) == 0 && dexpo >= 2 && dexpo <= 252;  // a power of two: exact
  const float inverseDivisor = 1.0f / divisor;

  // With blocks of 32 rows (every workgroup alone on its CU) K of a block is asked for one block ahead, into the
  // registers that the block before has just emptied into LDS, so that only the first block waits for its keys; with
  // blocks of 64 rows two workgroups per CU cover each other's waits and the registers are worth more (1 % slower).
  constexpr bool kAhead = ROWS == 32;
  v4f kreg[KV_ITEMS];
  auto fetchK = [&](unsigned t0) {
    const unsigned Tb = min((unsigned)kMaxT, T - t0);
#pragma unroll
    for (int it = 0; it < KV_ITEMS; ++it) {
      const unsigned w = tid + it * kThreads, row = w / CH, ch = w % CH;
      const bool in = row < Tb && ch * 4 < D;
      kreg[it] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rk, in ? ((t0 + row) * p.ldk + ch * 4) * 4u : kPastEnd, 0, 0));
    }
  };
  if constexpr (kAhead) fetchK(0);
  for (unsigned t0 = 0; t0 < T; t0 += kMaxT) {
    const unsigned Tb = min((unsigned)kMaxT, T - t0);   // keys of this block
    const unsigned Tbp = (Tb + 7u) & ~7u;                // k extent of the block's second product
    v4f vreg[KV_ITEMS];
    if constexpr (!kAhead) fetchK(t0);
    float mk[2] = {0.f, 0.f};
    if (masked) {
#pragma unroll
      for (int q = 0; q < 2; ++q)
        if ((unsigned)lane + 64u * q < Tb) mk[q] = mrow[t0 + lane + 64 * q];
    }
    __syncthreads();  // the block before is done with K / V and with the probabilities (first block: with Q's staging)
#pragma unroll
    for (int it = 0; it < KV_ITEMS; ++it) {
      const int w = tid + it * kThreads, row = w / CH, ch = w % CH;
      *reinterpret_cast<v4f*>(KVs + row * kPitchK + ch * 4) = kreg[it];
    }
    // (V is asked for once K's registers are free: it travels while the scores are computed)
#pragma unroll
    for (int it = 0; it < KV_ITEMS; ++it) {
      const unsigned w = tid + it * kThreads, row = w / CH, ch = w % CH;
      const bool in = row < Tb && ch * 4 < D;
      vreg[it] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rv, in ? ((t0 + row) * p.ldv + ch * 4) * 4u : kPastEnd, 0, 0));
    }
    if constexpr (kAhead) {
      if (t0 + kMaxT < T) fetchK(t0 + kMaxT);
    }
    __syncthreads();

    // ---- scores of the block
    const bool liveS = (unsigned)(32 * wnS) < Tb;
    if (liveS) {
      v4f bf[KBQ];
      const float* ka = KVs + (32 * wnS + lrow) * kPitchK + 4 * g;
#pragma unroll
      for (int kb = 0; kb < KBQ; ++kb) {
        bf[kb] = v4f{0.f, 0.f, 0.f, 0.f};
        if ((unsigned)kb * 8 < Dp) bf[kb] = *reinterpret_cast<const v4f*>(ka + kb * 8);
      }
      v16f sacc;
#pragma unroll
      for (int r = 0; r < 16; ++r) sacc[r] = 0.f;
#pragma unroll
      for (int kb = 0; kb < KBQ; ++kb) {
        if ((unsigned)kb * 8 < Dp) {
#pragma unroll
          for (int s = 0; s < 4; ++s) sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(qf[kb][s], bf[kb][s], sacc, 0, 0, 0);
        }
      }
      float* sc = Sc + (32 * wmS + 4 * g) * kPitchS + 32 * wnS + lrow;
      if (!p.divide) {
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[(8 * (r / 4) + (r & 3)) * kPitchS] = sacc[r];
      } else if (divideByMul) {
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[(8 * (r / 4) + (r & 3)) * kPitchS] = sacc[r] * inverseDivisor;
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[(8 * (r / 4) + (r & 3)) * kPitchS] = sacc[r] / divisor;
      }
    }
    __syncthreads();

    // ---- K is done with: V takes its place
#pragma unroll
    for (int it = 0; it < KV_ITEMS; ++it) {
      const int w = tid + it * kThreads, row = w / CH, ch = w % CH;
      *reinterpret_cast<v4f*>(KVs + row * kPitchV + ch * 4) = vreg[it];
    }

    // ---- the block's share of the softmax: rows wave + 8 u, columns lane and lane + 64
    {
      float v[R][2], mb[R], sum[R];
#pragma unroll
      for (int u = 0; u < R; ++u) {
        const float* sc = Sc + (wave + W * u) * kPitchS;
        mb[u] = -FLT_MAX;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          const unsigned i = lane + 64 * q;
          v[u][q] = i < Tb ? (masked ? sc[i] + mk[q] : sc[i]) : -FLT_MAX;
          mb[u] = fmaxf(mb[u], v[u][q]);
        }
      }
      wave_reduce8<true>(mb, lane);
      float scale[R];
#pragma unroll
      for (int u = 0; u < R; ++u) {
        const float mnew = fmaxf(mrun[u], mb[u]);
        scale[u] = t0 == 0 ? 0.f : softmax_exp(mrun[u] - mnew);  // nothing is accumulated before the first block
        mrun[u] = mnew;
        sum[u] = 0.f;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          const unsigned i = lane + 64 * q;
          v[u][q] = i < Tb ? softmax_exp(v[u][q] - mnew) : 0.f;
          sum[u] += v[u][q];
        }
      }
      wave_reduce8<false>(sum, lane);
#pragma unroll
      for (int u = 0; u < R; ++u) {
        lrun[u] = lrun[u] * scale[u] + sum[u];
        float* sc = Sc + (wave + W * u) * kPitchS;
#pragma unroll
        for (int q = 0; q < 2; ++q) sc[lane + 64 * q] = v[u][q];  // zeros past the block's keys
        const bool lastBlock = t0 + kMaxT >= T;
        if (lane == 0) rowScale[wave + W * u] = scale[u];
        if (lastBlock && lane == 1) rowScale[kRows + wave + W * u] = 1.0f / lrun[u];
      }
    }
    __syncthreads();

    // ---- accumulated rows scaled, then the block's probabilities x V
    if constexpr (ROWS == 32) {
      if ((unsigned)(16 * cb16) < D) {
        constexpr int KB = kMaxT / 8;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int r = 0; r < 4; ++r) acc16[j][r] *= rowScale[16 * rb16 + 4 * q16 + r];
        const float* pa = Sc + (16 * rb16 + l16) * kPitchS + kq16;
        const float* vb = KVs + kq16 * kPitchV + 16 * cb16 + l16;
        float af[KB][2], bfv[2][KB][2];
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            af[kb][h] = 0.f; bfv[0][kb][h] = 0.f; bfv[1][kb][h] = 0.f;
          }
          if ((unsigned)kb * 8 < Tbp) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
              af[kb][h] = pa[kb * 8 + 2 * h];
              bfv[0][kb][h] = vb[(kb * 8 + 2 * h) * kPitchV];
              bfv[1][kb][h] = vb[(kb * 8 + 2 * h) * kPitchV + 16];  // columns past D hold zeros
            }
          }
        }
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
          if ((unsigned)kb * 8 < Tbp) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
              acc16[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[kb][h], bfv[0][kb][h], acc16[0], 0, 0, 0);
              acc16[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[kb][h], bfv[1][kb][h], acc16[1], 0, 0, 0);
            }
          }
        }
      }
    } else if (wave < ROWS / 16 && (unsigned)(32 * wn) < D) {
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] *= rowScale[32 * wm + 8 * (r / 4) + 4 * g + (r & 3)];
      constexpr int KB = kMaxT / 8, HALF = KB / 2;
      const float* pa = Sc + (32 * wm + lrow) * kPitchS + 4 * g;
      const float* vb = KVs + (4 * g) * kPitchV + 32 * wn + lrow;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        v4f af[HALF], bfv[HALF];
#pragma unroll
        for (int q = 0; q < HALF; ++q) {
          const int kb = h * HALF + q;
          af[q] = v4f{0.f, 0.f, 0.f, 0.f};
          bfv[q] = v4f{0.f, 0.f, 0.f, 0.f};
          if ((unsigned)kb * 8 < Tbp) {
            af[q] = *reinterpret_cast<const v4f*>(pa + kb * 8);
#pragma unroll
            for (int s = 0; s < 4; ++s) bfv[q][s] = vb[(kb * 8 + s) * kPitchV];
          }
        }
#pragma unroll
        for (int q = 0; q < HALF; ++q) {
          if ((unsigned)(h * HALF + q) * 8 < Tbp) {
#pragma unroll
            for (int s = 0; s < 4; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[q][s], bfv[q][s], acc, 0, 0, 0);
          }
        }
      }
    }
  }

  // ---- rows divided by their sums and stored (the reciprocals were left behind the scales by the last block)
  if constexpr (ROWS == 32) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const unsigned col = 16 * (cb16 + j) + l16;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int trow = 16 * rb16 + 4 * q16 + r;
        const unsigned row = s0 + trow;
        if (row < S && col < D) O[(size_t)row * p.ldo + col] = acc16[j][r] * rowScale[kRows + trow];
      }
    }
  } else if (wave < ROWS / 16 && (unsigned)(32 * wn) < D) {
    const unsigned col = 32 * wn + lrow;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int trow = 32 * wm + 8 * (r / 4) + 4 * g + (r & 3);
      const unsigned row = s0 + trow;
      if (row < S && col < D) O[(size_t)row * p.ldo + col] = acc[r] * rowScale[kRows + trow];
    }
  }
}

const char* unsupported(const tfcc_rocm_attention_desc* d) {
  // a lone product of at most eight rows runs on the streaming kernel (sgemv.hip), whose sums are ordered differently
  if (d->s <= 8 && (unsigned long long)d->batch_outer * d->batch_inner == 1) return "a single head of at most eight query rows";
  if (d->d > (unsigned)kMaxD) return "head width above 64";
  if (d->d % 4 != 0) return "head width not a multiple of 4";
  if (d->ldq % 4 || d->ldk % 4 || d->ldv % 4) return "row stride not a multiple of 4 elements";
  if (d->stride_q % 4 || d->stride_k % 4 || d->stride_v % 4 || d->inner_stride_q % 4 || d->inner_stride_k % 4 ||
      d->inner_stride_v % 4)
    return "batch stride not a multiple of 4 elements";
  if ((uintptr_t)d->q % 16 || (uintptr_t)d->k % 16 || (uintptr_t)d->v % 16) return "operand not 16-byte aligned";
  const unsigned long long rows = d->s > d->t ? d->s : d->t, ld = d->ldq > d->ldk ? (d->ldq > d->ldv ? d->ldq : d->ldv)
                                                                                  : (d->ldk > d->ldv ? d->ldk : d->ldv);
  if (rows * ld + d->d >= (1ull << 28)) return "one batch entry spans 2^28 elements or more";
  return nullptr;
}

}  // namespace
}  // namespace tfcc_rocm

using namespace tfcc_rocm;

extern "C" int tfcc_rocm_attention_f32_supported(const tfcc_rocm_attention_desc* d) {
  return d != nullptr && unsupported(d) == nullptr ? 1 : 0;
}

extern "C" int tfcc_rocm_attention_f32(void* stream, const tfcc_rocm_attention_desc* d) {
  TFCC_REQUIRE(d != nullptr, "attention: null descriptor");
  TFCC_REQUIRE(d->q && d->k && d->v && d->out, "attention: null operand");
  TFCC_REQUIRE(d->s > 0 && d->t > 0 && d->d > 0 && d->batch_outer > 0 && d->batch_inner > 0, "attention: empty operand");
  TFCC_REQUIRE(d->ldq >= d->d && d->ldk >= d->d && d->ldv >= d->d && d->ldo >= d->d,
               "attention: row stride shorter than a row");
  const char* why = unsupported(d);
  TFCC_REQUIRE(why == nullptr, "attention: %s (use the separate products and softmax)", why);
  AttentionParams p{};
  p.Q = d->q; p.K = d->k; p.V = d->v; p.O = d->out;
  p.S = d->s; p.T = d->t; p.D = d->d;
  p.ldq = d->ldq; p.ldk = d->ldk; p.ldv = d->ldv; p.ldo = d->ldo;
  p.outerQ = d->stride_q; p.outerK = d->stride_k; p.outerV = d->stride_v; p.outerO = d->stride_out;
  p.innerQ = d->inner_stride_q; p.innerK = d->inner_stride_k; p.innerV = d->inner_stride_v; p.innerO = d->inner_stride_out;
  p.batchInner = d->batch_inner;
  // up to 128 keys: the scores of a row block in one piece; beyond: blocks of 128 keys with a running maximum and sum
  const bool stream128 = d->t > (unsigned)kMaxT;
  int cus = 0;
  {
    int dev = 0;
    TFCC_HIP_CHECK(hipGetDevice(&dev));
    static int cuCount[16] = {};
    TFCC_REQUIRE(dev >= 0 && dev < 16, "device index %d", dev);
    if (!cuCount[dev]) TFCC_HIP_CHECK(hipDeviceGetAttribute(&cuCount[dev], hipDeviceAttributeMultiprocessorCount, dev));
    cus = cuCount[dev];
  }
  // A CU works through its blocks roughly one after the other (two resident workgroups overlap little: 19.1 us for
  // 384 blocks of 64 rows against 12.7 for 192), so what counts is the largest number of rows any CU gets; a block of
  // 32 rows costs about 0.55 of a block of 64 (K and V are loaded per block).  16 x 12 heads of 128 rows: 17.8 against
  // 19.1 us with 32 rows; 32 x 12 heads: 30.5 against 27.7, so those keep 64.
  const unsigned long long heads = (unsigned long long)d->batch_outer * d->batch_inner;
  const unsigned long long blocks64 = (d->s + 63) / 64 * heads, blocks32 = (d->s + 31) / 32 * heads;
  const unsigned long long perCu64 = (blocks64 + cus - 1) / cus, perCu32 = (blocks32 + cus - 1) / cus;
  // (Beyond 128 keys a block of 32 rows walks all the keys again and holds one workgroup per SIMD's registers: it
  // pays only while every block has a CU to itself - 12 heads of 384 rows 25.3 against 28.4 us, 48 heads 70.5 against 54.4.)
  const bool rows32 = stream128 ? blocks32 <= (unsigned long long)cus : perCu32 * 55 < perCu64 * 100;
  const unsigned rowsPerBlock = rows32 ? 32 : kRows;
  p.blocksS = (d->s + rowsPerBlock - 1) / rowsPerBlock;
  const unsigned long long total = (unsigned long long)p.blocksS * d->batch_outer * d->batch_inner;
  TFCC_REQUIRE(total < (1ull << 31) - 8, "attention: too many blocks");
  p.total = (unsigned)total;
  p.chunk = (p.total + 7) / 8;
  const UDiv blocksDiv = udiv_prepare(p.blocksS), innerDiv = udiv_prepare(p.batchInner);
  p.blocksMagic = blocksDiv.magic; p.blocksShift = blocksDiv.shift;
  p.innerMagic = innerDiv.magic; p.innerShift = innerDiv.shift;
  p.divisor = d->divisor;
  p.divide = d->has_divisor ? 1 : 0;
  p.mask = d->mask;
  p.outerM = d->stride_mask;
  p.innerM = d->inner_stride_mask;
  constexpr size_t ldsBytes = (size_t)(kLdsFloats + 2 * kRows) * sizeof(float);
  static_assert(ldsBytes <= 80 * 1024, "two workgroups per CU");
  constexpr size_t ldsBytes32 = (size_t)(kMaxT * kPitchV + 32 * kPitchS) * sizeof(float);
  static_assert(3 * ldsBytes32 <= 160 * 1024, "three workgroups per CU");
  constexpr size_t ldsStream32 = ldsBytes32 + 2 * 32 * sizeof(float);
  static bool attrSet[16] = {};
  int dev = 0;
  TFCC_HIP_CHECK(hipGetDevice(&dev));
  TFCC_REQUIRE(dev >= 0 && dev < 16, "device index %d", dev);
  if (!attrSet[dev]) {
    TFCC_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(attention_kernel<64>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes));
    TFCC_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(attention_kernel<32>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes32));
    TFCC_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(attention_stream_kernel<64>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes));
    TFCC_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(attention_stream_kernel<32>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsStream32));
    attrSet[dev] = true;
  }
  if (stream128 && rows32) hipLaunchKernelGGL(attention_stream_kernel<32>, dim3(p.chunk * 8), dim3(256), ldsStream32, as_stream(stream), p);
  else if (stream128) hipLaunchKernelGGL(attention_stream_kernel<64>, dim3(p.chunk * 8), dim3(kThreads), ldsBytes, as_stream(stream), p);
  else if (rows32) hipLaunchKernelGGL(attention_kernel<32>, dim3(p.chunk * 8), dim3(256), ldsBytes32, as_stream(stream), p);
  else hipLaunchKernelGGL(attention_kernel<64>, dim3(p.chunk * 8), dim3(kThreads), ldsBytes, as_stream(stream), p);
  return check_launch("attention");
}
