// uint8 x int8 -> int32 matrix product for large aligned shapes: the gfx950-specific pipeline.
//
// Same arithmetic as the kernel in gemm_u8s8.hip (which stays the path for unaligned and small
// shapes); replaces tfcc/mkl/operations/tfcc_mklquantization.cpp:33-69,176-201 and the blocked CPU
// GEMM below it (tfcc/mkl/gemm/tfcc_mklsinglethreadgemm.h:93-141, tfcc_mklmatmulkernel.h:142-260).
//
// Data path of one BM x BN tile (WGM x WGN wavefronts; eight for the 256 x 256 tile, so that every
// SIMD holds two: one wavefront's LDS reads, waits and VALU work overlap the other's matrix ops):
//   HBM -> LDS  buffer_load_dwordx4 ... lds (asynchronous, no VGPRs): every K slab of 128 bytes is
//               copied as it lies in memory, A rows as As[row][128] (one whole memory line per row
//               piece) and B rows as Bs[k][BN], into a ring of STAGES LDS buffers, STAGES-1 slabs
//               ahead of the matrix cores.  Out-of-range
//               rows read zero through the buffer descriptor.  The 16-byte chunk a lane copies is
//               chosen so that the LDS image is xor-swizzled (the DMA writes lanes contiguously).
//   LDS -> VGPR A: ds_read_b128 (16 consecutive k of a row), xor 0x80 turns uint8 into int8.
//               B: k is the strided dimension of Bs, and the matrix core wants 16 consecutive k
//               per lane: ds_read_b64_tr_b8 transposes 8(k) x 16(n) byte blocks on the way out of
//               LDS, two of them give a lane its 16 k for one column.
//   MFMA        v_mfma_i32_32x32x32_i8 with the operands swapped (D = B^T A^T), so that a lane owns
//               four consecutive columns of one row of C in each accumulator quad.
//   epilogue    offset terms (see gemm_u8s8.hip), then either 128-bit int32 stores or the fused
//               requantize: four uint8 packed per lane, staged through LDS, written as whole
//               256-byte row segments.
// The true column sums of B (needed because a' = a - 128) are accumulated from the B operands with
// v_dot4_i32_i8 by the two wavefronts of the first tile row.
#include <type_traits>

#include "common.hpp"
#include "lds_dma.hpp"
#include "qgemm_dma.hpp"

namespace tfcc_rocm {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

namespace {

constexpr int BK = 128;      // bytes of k per slab: a row piece of A is one full 128-byte memory line
constexpr int KS = BK / 32;  // 32-deep matrix-op steps per slab

// 16 consecutive rows of one logical chunk fall into 16 different 16-byte slots of the 256-byte bank stripe
__device__ __forceinline__ int swzA(int row) { return (row >> 1) & 7; }

// WRITE_C: the int32 result is stored (always without REQUANT; with it only when the caller wants both).
// OWN_COLSUM: the true column sums of B are accumulated here (the caller's colsum_b is used as given, whatever
// it holds, like the reference does); without it the caller has promised that colsum_b holds them.
template <int BM, int BN, int WGM, int WGN, int STAGES, bool REQUANT, bool WRITE_C, bool OWN_COLSUM>
__global__ __launch_bounds__(WGM * WGN * 64, 2) void qgemm_dma_kernel(const QGemmParams p) {
  constexpr int kThreads = WGM * WGN * 64;
  constexpr int WM = BM / WGM, WN = BN / WGN;
  constexpr int MI = WM / 32, NI = WN / 32;
  static_assert(MI + 2 * NI <= 2 * MI * NI, "operand reads are issued two per matrix op");
  static_assert(NI % WGM == 0, "every 32-column block needs a wavefront row in charge of its column sums");
  static_assert(MI >= 1 && NI >= 1 && (BM * BK / 16) % kThreads == 0 && (BK * BN / 16) % kThreads == 0, "tile shape");
  constexpr int A_BYTES = BM * BK, B_BYTES = BK * BN, STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int A_COPIES = A_BYTES / 16 / kThreads, B_COPIES = B_BYTES / 16 / kThreads;
  constexpr int COPIES = A_COPIES + B_COPIES;  // per thread per slab
  constexpr int BCH = BN / 16;                 // 16-byte chunks per B row
  static_assert(BCH >= 8 && (BCH & (BCH - 1)) == 0, "B swizzle needs at least 8 chunks per row");
  static_assert(COPIES * STAGES < 64, "vmcnt range");

  extern __shared__ __align__(16) unsigned char smem[];
  const unsigned ldsBase = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)smem;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, kept in an SGPR
  const int wm = wave / WGN, wn = wave % WGN;

  // What stands in front of the first copies counts in a launch of ten microseconds: everything they need of the
  // argument block is named before the first branch (one round trip to memory instead of one per basic block), and
  // the divisions of the tile mapping are multiplications by constants the launcher worked out.
  asm volatile("" ::"s"(p.chunk), "s"(p.tilesTotal), "s"(p.tilesM), "s"(p.tilesN), "s"(p.perBatchMagic),
               "s"(p.perBatchShift), "s"(p.bandMagic), "s"(p.bandShift), "s"(p.M), "s"(p.N), "s"(p.K), "s"(p.A), "s"(p.B),
               "s"(p.strideA), "s"(p.strideB));
  unsigned tm, tn, bi;
  {
    // consecutive workgroup ids go to different XCDs: each XCD gets a contiguous run of tiles,
    // ordered in bands of 4 tile rows
    const unsigned wg = blockIdx.x;
    const unsigned xcd = wg & 7u, slot = wg >> 3;
    const unsigned L = xcd * p.chunk + slot;
    if (slot >= p.chunk || L >= p.tilesTotal) return;
    const unsigned perBatch = p.tilesM * p.tilesN;
    bi = udiv_apply(L, p.perBatchMagic, p.perBatchShift);
    unsigned t = L - bi * perBatch;
    const unsigned band = 4u * p.tilesN;
    unsigned g = udiv_apply(t, p.bandMagic, p.bandShift);
    unsigned rowsInBand = min(4u, p.tilesM - g * 4u);
    unsigned r = t - g * band;
    const unsigned rq = rowsInBand == 4u ? r >> 2 : r / rowsInBand;  // a ragged last band is the rare case
    tm = g * 4u + (r - rq * rowsInBand);
    tn = rq;
  }
  const unsigned m0 = tm * BM, n0 = tn * BN;
  const unsigned M = p.M, N = p.N, K = p.K;
  const unsigned char* A = p.A + (size_t)bi * p.strideA;
  const signed char* B = p.B + (size_t)bi * p.strideB;
  // buffer descriptors: base, 0 stride, size in bytes, raw 32-bit format; held in SGPRs
  const v4i rsrcA = make_rsrc(A, M * K);
  const v4i rsrcB = make_rsrc(B, K * N);

  // ---- per-thread copy descriptors: which 16 bytes of the slab this lane moves in each copy.
  // LDS slot s (16 bytes) of the A image holds row s/8, physical chunk s%8 = logical chunk ^ swzA(row).
  unsigned aOff[A_COPIES], bOff[B_COPIES];  // byte offsets into A / B for slab 0
#pragma unroll
  for (int c = 0; c < A_COPIES; ++c) {
    const int s = c * kThreads + tid;
    const int row = s >> 3, phys = s & 7;
    aOff[c] = (m0 + row) * K + ((phys ^ swzA(row)) << 4);
  }
  // LDS slot s of the B image holds k row s/BCH, physical chunk s%BCH = logical chunk ^ (k & 7).
#pragma unroll
  for (int c = 0; c < B_COPIES; ++c) {
    const int s = c * kThreads + tid;
    const int k = s / BCH, phys = s % BCH;
    bOff[c] = k * N + n0 + ((phys ^ (k & 7)) << 4);
  }
  // copy c (0 .. COPIES-1) of a slab: A chunks first, then B
  auto issueCopy = [&](unsigned slab, int c) {
    const unsigned stage = slab % STAGES;
    const unsigned base = __builtin_amdgcn_readfirstlane(ldsBase + stage * STAGE_BYTES + wave * 1024);
    const unsigned k0 = slab * BK;
    if (c < A_COPIES) dma16(rsrcA, base + c * (kThreads * 16), aOff[c] + k0);
    else dma16(rsrcB, base + A_BYTES + (c - A_COPIES) * (kThreads * 16), bOff[c - A_COPIES] + k0 * N);
  };
  auto issueSlab = [&](unsigned slab) {
#pragma unroll
    for (int c = 0; c < COPIES; ++c) issueCopy(slab, c);
  };

  v16i acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
  // Column sums: wavefront row wm owns the blocks j = wm + WGM * t.  Four independent partial sums per block:
  // a single chain would stall on the dot latency.
  constexpr int NT = NI / WGM;
  int colsum[NT][4];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int q = 0; q < 4; ++q) colsum[t][q] = 0;

  // ---- operand addresses inside a stage
  const int l32 = lane & 31, g = lane >> 5;
  // A: row wm*WM + 32*i + l32, logical chunk 2*ks + g
  int aAddr[MI][KS];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int row = wm * WM + 32 * i + l32;
      aAddr[i][ks] = row * BK + (((2 * ks + g) ^ swzA(row)) << 4);
    }
  // B: transposing read.  Within a block of 16 lanes, lane s points at k row (s >> 1) and 8-byte
  // column half (s & 1); the lane then receives, for column 8*(l&8 ? 1 : 0) + (l & 7) of the 16, the
  // bytes of k rows 0..7.  Lane blocks: (lane >> 4) & 1 selects the 16-column half of the 32-column
  // MFMA block, lane >> 5 the k half (g).
  const int s16 = lane & 15, colHalf = (lane >> 4) & 1;
  const int trK = s16 >> 1;           // k row within a group of 8
  const int trByte = (s16 & 1) << 3;  // 0 or 8 within the 16-byte chunk
  int bChunk[NI];                     // logical 16-byte chunk index of this lane's columns
#pragma unroll
  for (int j = 0; j < NI; ++j) bChunk[j] = (wn * WN + 32 * j + 16 * colHalf) >> 4;

  // raw operand loads of one 32-deep k step of a stage (no arithmetic: nothing here waits for LDS);
  // load q of a step: first two transposing reads per B block (the next step needs B first), then
  // the A operand of each row block
  constexpr int NLOAD = MI + 2 * NI, NMFMA = MI * NI;
  auto loadOne = [&](const unsigned char* as, const unsigned char* bs, int ks, int q, v4i (&af)[MI], v4i (&bf)[NI]) {
    if (q >= 2 * NI) {
      af[q - 2 * NI] = *reinterpret_cast<const v4i*>(as + aAddr[q - 2 * NI][ks]);
    } else {
      const int j = q >> 1, half = q & 1;
      const int k = 32 * ks + 16 * g + 8 * half + trK;  // (k & 7) == trK
      const unsigned char* ptr = bs + k * BN + ((bChunk[j] ^ trK) << 4) + trByte;
      v2i t = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
          (__attribute__((address_space(3))) v2i*)(const_cast<unsigned char*>(ptr)));
      bf[j][2 * half] = t[0];
      bf[j][2 * half + 1] = t[1];
    }
  };
  // One k step: the matrix ops on operands (ua, ub) that were read during the previous step, with the
  // LDS reads of the next step's operands (la, lb) issued two at a time between the first half of
  // them: spread out enough not to queue up behind the other wavefronts' reads (all wavefronts run in
  // phase, one barrier per slab), early enough to have returned when the step ends.
  // uint8 -> int8 is the xor on the A operands; block j's column sums belong to wavefront row j % WGM.
  // When `refill` is set the copies of slab `refillSlab` are issued as well, spread over the step for
  // the same reason.
  auto step = [&](v4i (&ua)[MI], v4i (&ub)[NI], v4i (&la)[MI], v4i (&lb)[NI], unsigned stage, int ks,
                  auto refill, unsigned refillSlab) {
    constexpr bool REFILL = decltype(refill)::value;
    constexpr int DMA_EVERY = NMFMA / COPIES > 0 ? NMFMA / COPIES : 1;
    const unsigned char* as = smem + stage * STAGE_BYTES;
    const unsigned char* bs = as + A_BYTES;
#pragma unroll
    for (int t = 0; t < (OWN_COLSUM ? NT : 0); ++t) {
      v4i own = ub[WGM * t];  // the block of this wavefront row: selects on a wave-uniform condition, no branches
#pragma unroll
      for (int w = 1; w < WGM; ++w) own = wm == w ? ub[WGM * t + w] : own;
#pragma unroll
      for (int q = 0; q < 4; ++q) colsum[t][q] = __builtin_amdgcn_sdot4(own[q], 0x01010101, colsum[t][q], false);
    }
    v4i ax = {0, 0, 0, 0};
#pragma unroll
    for (int m = 0; m < NMFMA; ++m) {
      const int i = m / NI, j = m % NI;
#pragma unroll
      for (int q = 2 * m; q < 2 * m + 2 && q < NLOAD; ++q) loadOne(as, bs, ks, q, la, lb);
      if constexpr (REFILL) {
        if (m % DMA_EVERY == 0 && m / DMA_EVERY < COPIES) issueCopy(refillSlab, m / DMA_EVERY);
        if (m == NMFMA - 1) {
#pragma unroll
          for (int c = NMFMA / DMA_EVERY; c < COPIES; ++c) issueCopy(refillSlab, c);  // more copies than matrix ops
        }
      }
      if (j == 0) ax = ua[i] ^ (int)0x80808080;
      acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ub[j], ax, acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // Software pipeline.  The ring holds STAGES slabs.  One barrier per slab, in the middle of it:
  //   before it: this wavefront's copies of slab kt+1 have landed and its reads of slab kt are done
  //   after it : slab kt+1 is complete and visible, slab kt's stage is free and is refilled with
  //              slab kt+STAGES (copies past the end of K read zeros or unused bytes; they are issued
  //              anyway to keep the outstanding-copy count uniform)
  const unsigned KT = (K + BK - 1) / BK;
#pragma unroll
  for (int s = 0; s < STAGES; ++s) issueSlab(s);
  // (everything the tile store needs is worked out and asked for from here on, with the first slabs on their way)
  int offA = p.offsetA, offB = p.offsetB;
  float minC = 0.f, maxC = 0.f;
  if (p.minA) {
    float mnA = *p.minA, mxA = *p.maxA, mnB = *p.minB, mxB = *p.maxB;
    qmatmul_offsets(mnA, mxA, mnB, mxB, &offA, &offB);
    qmatmul_range(mnA, mxA, mnB, mxB, &minC, &maxC);
    if (blockIdx.x == 0 && tid == 0) {
      if (p.minC) *p.minC = minC;
      if (p.maxC) *p.maxC = maxC;
    }
  }

  // The caller's row / column sums this thread turns into offset terms after the main loop are fetched now:
  // at the end their latency would be waited for in full (one tile per CU, nothing to overlap it with).
  static_assert(BM <= kThreads && BN <= kThreads, "one row sum and one column sum per thread");
  unsigned rsPre = 0, csPre = 0;
  {
    const int* rsA = p.rowsumA + (size_t)bi * p.strideRA;
    const int* csB = p.colsumB + (size_t)bi * p.strideRB;
    if (tid < BM && m0 + tid < M) rsPre = (unsigned)rsA[m0 + tid];
    if (tid < BN && n0 + tid < N) csPre = (unsigned)csB[n0 + tid];
  }

  wait_vmcnt<COPIES*(STAGES - 1)>();
  __syncthreads();
  v4i fa[2][MI], fb[2][NI];
#pragma unroll
  for (int q = 0; q < NLOAD; ++q) loadOne(smem, smem + A_BYTES, 0, q, fa[0], fb[0]);
  static_assert(KS % 2 == 0, "the operand registers alternate per step");
  for (unsigned kt = 0; kt < KT; ++kt) {
    const unsigned cur = kt % STAGES, nxt = (kt + 1) % STAGES;
    // k steps 0 .. KS-2 of slab kt, each reading the operands of the step after it
#pragma unroll
    for (int ks = 0; ks < KS - 1; ++ks)
      step(fa[ks & 1], fb[ks & 1], fa[(ks + 1) & 1], fb[(ks + 1) & 1], cur, ks + 1, std::false_type{}, 0u);
    wait_vmcnt<COPIES*(STAGES - 2)>();
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the reads of slab kt have returned
    __syncthreads();
    // last k step of slab kt; reads k step 0 of slab kt+1; refills the stage of slab kt
    step(fa[1], fb[1], fa[0], fb[0], nxt, 0, std::true_type{}, kt + STAGES);
  }
  wait_vmcnt<0>();
  __syncthreads();

  // ---- epilogue.  Accumulator layout (operands swapped): lane (l32, g) holds row l32 of the 32-row
  // block and columns 8*(r/4) + 4*g + r%4 of the 32-column block, r = 0..15.
  int* colTerm = reinterpret_cast<int*>(smem);  // [BN]
  int* rowTerm = colTerm + BN;                  // [BM]
  unsigned char* stageQ = smem + (BM + BN) * 4; // [BM][BN + 4] bytes, requantized tile
  constexpr int QPITCH = BN + 4;
  // lanes l and l+32 hold the two k halves of the same column; the transposing read hands lane
  // (colHalf, s16) column 16*colHalf + s16 of the 32-column block
#pragma unroll
  for (int t = 0; t < (OWN_COLSUM ? NT : 0); ++t) {
    const int j = wm + WGM * t;
    int s = colsum[t][0] + colsum[t][1] + colsum[t][2] + colsum[t][3];
    s += __shfl_xor(s, 32, 64);
    if (g == 0) colTerm[wn * WN + 32 * j + 16 * colHalf + s16] = s;
  }
  __syncthreads();
  const unsigned global = (unsigned)offA * (unsigned)offB * K;
  if (tid < BN) colTerm[tid] = (int)(128u * (OWN_COLSUM ? (unsigned)colTerm[tid] : csPre) + csPre * (unsigned)offA);
  if (tid < BM) rowTerm[tid] = (int)(global + rsPre * (unsigned)offB);
  __syncthreads();

  RequantScalars rq;
  if (REQUANT) {
    if (p.minOut) {
      rq = make_requant_scalars(TFCC_ROCM_S32, TFCC_ROCM_U8, minC, maxC, *p.minOut, *p.maxOut);
    } else {
      rq.inScale = p.inScale; rq.inMin = p.inMin; rq.outScale = p.outScale; rq.outOffset = p.outOffset;
      rq.inLowest = -2147483648LL; rq.outLowest = 0; rq.outHighest = 255; rq.mode = 0; rq.fillValue = 0;
      finish_requant_scalars(rq, 4294967295.0);
    }
  }

  int* C = WRITE_C ? p.C + (size_t)bi * p.strideC : nullptr;
  unsigned char* Q = REQUANT ? p.Q + (size_t)bi * p.strideC : nullptr;

  auto storeTile = [&](auto flavour) {
    constexpr int FLAVOUR = decltype(flavour)::value;  // 0 int32 only, 1 double shortcut, 2 exact int64, 3 fill, 4 int32 shortcut, 5 folded
#pragma unroll
    for (int i = 0; i < MI; ++i) {
      const int trow = wm * WM + 32 * i + l32;
      const unsigned grow = m0 + trow;
      // without an int32 result to store, the 2^31 that turns the accumulator into its offset from INT32_MIN is
      // folded into the row term
      constexpr unsigned kBias = (REQUANT && !WRITE_C) ? 0x80000000u : 0u;
      const int rt = (int)((unsigned)rowTerm[trow] + kBias);
#pragma unroll
      for (int j = 0; j < NI; ++j) {
#pragma unroll
        for (int rq4 = 0; rq4 < 4; ++rq4) {
          const int tcol = wn * WN + 32 * j + 8 * rq4 + 4 * g;  // first of 4 consecutive columns
          const v4i ct = *reinterpret_cast<const v4i*>(colTerm + tcol);
          int v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = (int)((unsigned)acc[i][j][4 * rq4 + e] + (unsigned)rt + (unsigned)ct[e]);
          if constexpr (WRITE_C) {
            if (grow < M && n0 + tcol < N)  // N % 16 == 0: the four columns are in or out together
              *reinterpret_cast<v4i*>(C + (size_t)grow * N + n0 + tcol) = v4i{v[0], v[1], v[2], v[3]};
          }
          if constexpr (FLAVOUR != 0) {
            unsigned q[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const unsigned off = (unsigned)v[e] ^ (0x80000000u ^ kBias);  // v - INT32_MIN
              if constexpr (FLAVOUR == 1) q[e] = (unsigned)requantize_one_fast((double)off, rq);
              else if constexpr (FLAVOUR == 2) q[e] = (unsigned)requantize_one_exact((long long)(int)(off ^ 0x80000000u), rq);
              else if constexpr (FLAVOUR == 4) q[e] = (unsigned)requantize_one_fast32((double)off, rq);
              else if constexpr (FLAVOUR == 5) q[e] = (unsigned)requantize_one_folded((double)off, rq);
              else q[e] = (unsigned)rq.fillValue;
            }
            *reinterpret_cast<unsigned*>(stageQ + trow * QPITCH + tcol) = q[0] | (q[1] << 8) | (q[2] << 16) | (q[3] << 24);
          }
        }
      }
      if constexpr (FLAVOUR != 0) {
        // The rows of block row i (32 per wavefront row) are staged: write them out now, so that the stores are
        // in flight while the next block row is requantized.  16 lanes write one 256-byte row segment.
        __syncthreads();
        constexpr int CHUNKS = BN / 16, PHASE_ROWS = WGM * 32;
        for (int idx = tid; idx < PHASE_ROWS * CHUNKS; idx += kThreads) {
          const int pr = idx / CHUNKS, ch = idx % CHUNKS;
          const int row = (pr >> 5) * WM + 32 * i + (pr & 31);
          const unsigned grow = m0 + row, gcol = n0 + ch * 16;
          if (grow >= M || gcol >= N) continue;
          const unsigned* src = reinterpret_cast<const unsigned*>(stageQ + row * QPITCH + ch * 16);
          v4i v = {(int)src[0], (int)src[1], (int)src[2], (int)src[3]};
          *reinterpret_cast<v4i*>(Q + (size_t)grow * N + gcol) = v;
        }
      }
    }
  };
  if constexpr (!REQUANT) {
    storeTile(std::integral_constant<int, 0>{});
  } else {
    if (rq.mode) storeTile(std::integral_constant<int, 3>{});
    else if (rq.foldedOK) storeTile(std::integral_constant<int, 5>{});
    else if (rq.fast32OK) storeTile(std::integral_constant<int, 4>{});
    else if (rq.fastOK) storeTile(std::integral_constant<int, 1>{});
    else storeTile(std::integral_constant<int, 2>{});
  }
}

template <int BM, int BN, int WGM, int WGN, int STAGES, bool REQUANT, bool WRITE_C, bool OWN_COLSUM>
int launch(hipStream_t stream, QGemmParams p) {
  constexpr int kThreads = WGM * WGN * 64;
  p.tilesM = (p.M + BM - 1) / BM;
  p.tilesN = (p.N + BN - 1) / BN;
  unsigned long long total = (unsigned long long)p.tilesM * p.tilesN * p.batch;
  if (total > 0x7fffffffull) return set_error(TFCC_ROCM_INVALID_ARGUMENT, "quantized matmul: too many tiles");
  p.tilesTotal = (unsigned)total;
  p.chunk = (p.tilesTotal + 7) / 8;
  const UDiv perBatch = udiv_prepare(p.tilesM * p.tilesN), band = udiv_prepare(4u * p.tilesN);
  p.perBatchMagic = perBatch.magic; p.perBatchShift = perBatch.shift;
  p.bandMagic = band.magic; p.bandShift = band.shift;
  constexpr size_t ring = (size_t)STAGES * (BM + BN) * BK;
  constexpr size_t epi = (size_t)(BM + BN) * 4 + (size_t)BM * (BN + 4);
  constexpr size_t lds = ring > epi ? ring : epi;
  static_assert(lds <= 160 * 1024, "LDS budget");
  auto kern = qgemm_dma_kernel<BM, BN, WGM, WGN, STAGES, REQUANT, WRITE_C, OWN_COLSUM>;
  static bool attrSet[16] = {};  // per device: the attribute belongs to the function on one device
  int dev = 0;
  TFCC_HIP_CHECK(hipGetDevice(&dev));
  TFCC_REQUIRE(dev >= 0 && dev < 16, "device index %d", dev);
  if (!attrSet[dev]) {
    TFCC_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attrSet[dev] = true;
  }
  hipLaunchKernelGGL(kern, dim3(p.chunk * 8), dim3(kThreads), lds, stream, p);
  return check_launch("quantized matmul (dma)");
}

}  // namespace

bool qgemm_dma_supported(const QGemmParams& p, bool requant) {
  return (p.K % 16 == 0) && (p.N % 16 == 0) && ((uintptr_t)p.A % 16 == 0) && ((uintptr_t)p.B % 16 == 0) &&
         (p.strideA % 16 == 0) && (p.strideB % 16 == 0) &&
         (p.C == nullptr || ((uintptr_t)p.C % 16 == 0 && p.strideC % 4 == 0)) &&
         (!requant || ((uintptr_t)p.Q % 16 == 0 && p.strideC % 16 == 0)) &&
         ((unsigned long long)p.M + 512) * p.K < (1ull << 32) && ((unsigned long long)p.K + 1024) * p.N + 1024 < (1ull << 32);
}

namespace {
template <int BM, int BN, int WGM, int WGN, int STAGES, bool OWN_COLSUM>
int launch_for_outputs2(hipStream_t stream, const QGemmParams& p, bool requant) {
  if (!requant) return launch<BM, BN, WGM, WGN, STAGES, false, true, OWN_COLSUM>(stream, p);
  return p.C ? launch<BM, BN, WGM, WGN, STAGES, true, true, OWN_COLSUM>(stream, p)
             : launch<BM, BN, WGM, WGN, STAGES, true, false, OWN_COLSUM>(stream, p);
}
template <int BM, int BN, int WGM, int WGN, int STAGES>
int launch_for_outputs(hipStream_t stream, const QGemmParams& p, bool requant) {
  return p.colsumExact ? launch_for_outputs2<BM, BN, WGM, WGN, STAGES, false>(stream, p, requant)
                       : launch_for_outputs2<BM, BN, WGM, WGN, STAGES, true>(stream, p, requant);
}
}  // namespace

int qgemm_dma_launch(hipStream_t stream, const QGemmParams& p, bool requant) {
  const unsigned long long big = (unsigned long long)((p.M + 255) / 256) * ((p.N + 255) / 256) * p.batch;
  if (big >= 192) {
    if (qgemm_w4_supported(p)) return qgemm_w4_launch(stream, p, requant);
    return launch_for_outputs<256, 256, 2, 4, 2>(stream, p, requant);
  }
  // fewer than half a chip of 128x128 tiles: 64x128 tiles (four wavefronts side by side) put twice as many CUs to work
  const unsigned long long mid = (unsigned long long)((p.M + 127) / 128) * ((p.N + 127) / 128) * p.batch;
  if (mid < 128) return launch_for_outputs<64, 128, 1, 4, 2>(stream, p, requant);
  return launch_for_outputs<128, 128, 2, 2, 2>(stream, p, requant);
}

}  // namespace tfcc_rocm
