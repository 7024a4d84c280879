// uint8 x int8 -> int32 matrix product for large aligned shapes: one wavefront per SIMD, 128 x 128 per wavefront.
//
// Same arithmetic as the kernels in gemm_u8s8.hip and gemm_u8s8_dma.hip; replaces
// tfcc/mkl/operations/tfcc_mklquantization.cpp:33-69,176-201 and the blocked CPU GEMM below it
// (tfcc/mkl/gemm/tfcc_mklsinglethreadgemm.h:93-141, tfcc_mklmatmulkernel.h:142-260) for products of at
// least three quarters of a chip of 256 x 256 tiles.
//
// Why a second shape of the same pipeline: with eight wavefronts of 128 x 64 a 32-deep k step moves 6 KiB
// out of LDS per 8 matrix ops; with four wavefronts of 128 x 128 it is 8 KiB per 16, a third less LDS
// traffic per matrix op, and the 256 accumulator registers of a wavefront live in the accumulation half of
// the 512-entry register file a lone wavefront of a SIMD owns.  With one wavefront per SIMD nothing hides a
// stall, so every LDS read and every HBM -> LDS copy is issued a whole k step (reads) or STAGES-1 slabs
// (copies) before its data is needed, between matrix ops that do not depend on it.
//
// Data path of one 256 x 256 tile:
//   HBM -> LDS  buffer_load_dwordx4 ... lds, K slabs of BK bytes as they lie in memory: A rows as As[row][BK],
//               B rows as Bs[k][256], ring of STAGES buffers.  The 16-byte chunk a lane copies is chosen so
//               that the LDS image is swizzled:
//                 A  physical chunk = chunk ^ (row / rows-per-256-bytes): the 16 rows a quarter wavefront
//                    reads with ds_read_b128 fall into 16 different 16-byte bank groups
//                 B  physical chunk = ((chunk >> 1) ^ (k & 7)) | (chunk & 1) << 3: the 8 k rows x 2 column
//                    halves x 2 eight-byte pieces half a wavefront reads with ds_read_b64_tr_b8 cover all 64
//                    banks once
//   LDS -> VGPR A: ds_read_b128 (16 consecutive k of a row), xor 0x80 turns uint8 into int8.
//               B: ds_read_b64_tr_b8 transposes 8(k) x 16(n) byte blocks on the way out of LDS.
//   MFMA        v_mfma_i32_32x32x32_i8 with the operands swapped (D = B^T A^T): a lane owns four consecutive
//               columns of one row of C in each accumulator quad.
//   epilogue    offset terms, then 128-bit int32 stores and / or the fused requantize: four uint8 packed per
//               lane and column quad, words exchanged between the half-wavefronts, 128-bit stores.
#include <type_traits>

#include "common.hpp"
#include "copy_offsets.hpp"
#include "lds_dma.hpp"
#include "qgemm_dma.hpp"

namespace tfcc_rocm {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

namespace {

constexpr int BM = 256, BN = 256, kThreads = 256;
constexpr int MI = 4, NI = 4;  // 32 x 32 blocks per wavefront: 128 x 128

template <int BK>
__device__ __forceinline__ int swz_a(int row) {
  constexpr int CH = BK / 16, RPS = 256 / BK;  // chunks per row, rows per 256-byte bank stripe
  return (row / RPS) & (CH - 1);
}
__device__ __forceinline__ int phys_b(int chunk, int k) { return (((chunk >> 1) ^ k) & 7) | ((chunk & 1) << 3); }

// WRITE_C: the int32 result is stored (always without REQUANT; with it only when the caller wants both).
// OWN_COLSUM: the true column sums of B are accumulated here (the caller's colsum_b is used as given, whatever
// it holds, like the reference does); without it the caller has promised that colsum_b holds them.
template <int BK, int STAGES, bool REQUANT, bool WRITE_C, bool OWN_COLSUM>
__global__ __launch_bounds__(kThreads) void qgemm_w4_kernel(const QGemmParams p) {
  constexpr int KS = BK / 32;  // 32-deep matrix-op steps per slab
  constexpr int CH = BK / 16;  // 16-byte chunks per A row
  constexpr int A_BYTES = BM * BK, B_BYTES = BK * BN, STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int A_COPIES = A_BYTES / 16 / kThreads, B_COPIES = B_BYTES / 16 / kThreads;
  constexpr int COPIES = A_COPIES + B_COPIES;  // per thread per slab
  static_assert(KS >= 2 && KS % 2 == 0, "the operand registers alternate per step");
  static_assert(COPIES * STAGES < 64, "vmcnt range");
  static_assert(COPIES <= 16, "one copy per matrix op of a step");
  static_assert(MI == 4 && NI == 4, "the slot plan of a k step is written for 4 x 4 blocks");

  extern __shared__ __align__(16) unsigned char smem[];
  const unsigned ldsBase = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)smem;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, kept in an SGPR
  const int wm = wave >> 1, wn = wave & 1;

  // Everything this prologue needs of the argument block is read before the first branch (one round trip to
  // memory instead of one per basic block); the divisions of the tile mapping are multiplications by constants
  // the launcher worked out.
  // (every field the prologue and the later blocks read, named before anything is computed from one of them: their
  // loads leave together)
  asm volatile("" ::"s"(p.chunk), "s"(p.tilesTotal), "s"(p.tilesM), "s"(p.tilesN), "s"(p.perBatchMagic),
               "s"(p.perBatchShift), "s"(p.bandMagic), "s"(p.bandShift), "s"(p.M), "s"(p.N), "s"(p.K), "s"(p.A), "s"(p.B),
               "s"(p.strideA), "s"(p.strideB), "s"(p.offsetA), "s"(p.offsetB), "s"(p.minA), "s"(p.maxA), "s"(p.minB),
               "s"(p.maxB), "s"(p.minOut), "s"(p.maxOut), "s"(p.rowsumA), "s"(p.colsumB), "s"(p.strideRA),
               "s"(p.strideRB), "s"(p.strideC), "s"(p.C), "s"(p.Q));
  unsigned tm, tn, bi;
  bool inGrid;
  {
    // consecutive workgroup ids go to different XCDs: each XCD gets a contiguous run of tiles,
    // ordered in bands of 4 tile rows
    const unsigned wg = blockIdx.x;
    const unsigned xcd = wg & 7u, slot = wg >> 3;
    const unsigned L = xcd * p.chunk + slot;
    inGrid = slot < p.chunk && L < p.tilesTotal;
    const unsigned perBatch = p.tilesM * p.tilesN;
    bi = udiv_apply(L, p.perBatchMagic, p.perBatchShift);
    unsigned t = L - bi * perBatch;
    const unsigned band = 4u * p.tilesN;
    unsigned gb = udiv_apply(t, p.bandMagic, p.bandShift);
    unsigned rowsInBand = min(4u, p.tilesM - gb * 4u);
    unsigned r = t - gb * band;
    const unsigned rq = rowsInBand == 4u ? r >> 2 : r / rowsInBand;  // a ragged last band is the rare case
    tm = gb * 4u + (r - rq * rowsInBand);
    tn = rq;
  }
  const unsigned m0 = tm * BM, n0 = tn * BN;
  const unsigned M = p.M, N = p.N, K = p.K;
  const unsigned char* A = p.A + (size_t)bi * p.strideA;
  const signed char* B = p.B + (size_t)bi * p.strideB;
  const v4i rsrcA = make_rsrc(A, M * K);
  const v4i rsrcB = make_rsrc(B, K * N);

  // ---- copies.  Copy c of a slab moves LDS slots c * 256 + tid (16 bytes each); A slot s holds row s / CH,
  // physical chunk s % CH; B slot s holds k row s / 16, physical chunk s % 16.  From one copy to the next the row
  // advances by a multiple of 16, which leaves both swizzles alone.  The lane offsets (one per copy, first slab)
  // go through the range check of the buffer descriptor, so rows past the end of A read zeros; the slab's offset
  // is the same for all lanes and rides in the scalar offset, which is not checked: K is a multiple of BK here,
  // slabs past the end are redirected to the last one (into a stage nobody reads any more), and a lane whose
  // columns of B lie past N carries an offset that fails the check whatever the slab (copy_offsets.hpp).
  unsigned aOff[A_COPIES], bOff[B_COPIES];
#pragma unroll
  for (int c = 0; c < A_COPIES; ++c) aOff[c] = copy_offsets::w4_a_lane_offset(tid, c, m0, K, BK);
#pragma unroll
  for (int c = 0; c < B_COPIES; ++c) bOff[c] = copy_offsets::w4_b_lane_offset(tid, c, n0, N);
  const unsigned KT = K / BK;
  const unsigned ldsWave = __builtin_amdgcn_readfirstlane(ldsBase + wave * 1024);
  // copy c of `slab` into stage `stage` (a compile-time constant wherever this is called)
  // (the scalar offsets of a slab: computed once per step that copies, see slabOffsets)
  auto issueCopy = [&](unsigned soA, unsigned soB, int stage, int c) {
    if (c < A_COPIES) dma16s(rsrcA, ldsWave + (stage * STAGE_BYTES + c * (kThreads * 16)), aOff[c], soA);
    else dma16s(rsrcB, ldsWave + (stage * STAGE_BYTES + A_BYTES + (c - A_COPIES) * (kThreads * 16)), bOff[c - A_COPIES], soB);
  };
  auto slabOffsets = [&](unsigned slab, unsigned& soA, unsigned& soB) {
    const unsigned sl = min(slab, KT - 1);
    soA = __builtin_amdgcn_readfirstlane(sl * BK);
    soB = __builtin_amdgcn_readfirstlane(copy_offsets::w4_b_slab_offset(slab, KT, BK, N));
  };

  if (!inGrid) return;
  // The first slabs are asked for before anything else: everything up to the main loop runs while they travel.
  constexpr int CPS = (STAGES > 2) ? (COPIES / (BK / 32)) : COPIES;  // copies per step that issues copies
  // A CU's path into LDS takes 64 bytes a clock: a whole ring is 2000 clocks of it, and a wavefront that has
  // issued more copies than the path has taken up waits to issue the next.  With four stages of two steps (RAMP)
  // only slabs 0 and 1 are asked for here; slab 2, the rest of slab 3 and the first half of slab 4 follow between
  // the matrix ops of slab 0, on top of the copies every step issues anyway.
  constexpr bool RAMP = STAGES == 4 && (BK / 32) == 2;
#pragma unroll
  for (int s = 0; s < (RAMP ? 2 : STAGES); ++s) {
    unsigned soA, soB;
    slabOffsets(s, soA, soB);
#pragma unroll
    for (int c = 0; c < (s < STAGES - 1 || STAGES == 2 ? COPIES : CPS); ++c) issueCopy(soA, soB, s, c);
  }

  int offA = p.offsetA, offB = p.offsetB;
  float minC = 0.f, maxC = 0.f;
  // The ranges are read through the scalar cache (the constant address space: they are inputs, nothing in this launch
  // writes them).  Read as vector loads they would queue up behind the copies above - memory operations of a
  // wavefront return in the order they were issued - and everything that is worked out from them below would wait
  // until the first two slabs have landed instead of running while they travel.
  typedef const __attribute__((address_space(4))) float* ConstFloats;
  auto uniformLoad = [](const float* ptr) { return *(ConstFloats)(unsigned long long)ptr; };
  if (p.minA) {
    float mnA = uniformLoad(p.minA), mxA = uniformLoad(p.maxA), mnB = uniformLoad(p.minB), mxB = uniformLoad(p.maxB);
    qmatmul_offsets(mnA, mxA, mnB, mxB, &offA, &offB);
    qmatmul_range(mnA, mxA, mnB, mxB, &minC, &maxC);
    if (blockIdx.x == 0 && tid == 0) {
      if (p.minC) *p.minC = minC;
      if (p.maxC) *p.maxC = maxC;
    }
  }

  // The caller's row / column sums this thread turns into offset terms after the main loop are fetched now:
  // at the end their latency would be waited for in full.
  unsigned rsPre = 0, csPre = 0;
  {
    const int* rsA = p.rowsumA + (size_t)bi * p.strideRA;
    const int* csB = p.colsumB + (size_t)bi * p.strideRB;
    if (m0 + tid < M) rsPre = (unsigned)rsA[m0 + tid];
    if (n0 + tid < N) csPre = (unsigned)csB[n0 + tid];
  }

  // the scalars of the requantize step: worked out here, while the first copies are under way
  RequantScalars rq;
  if (REQUANT) {
    if (p.minOut) {
      rq = make_requant_scalars(TFCC_ROCM_S32, TFCC_ROCM_U8, minC, maxC, uniformLoad(p.minOut), uniformLoad(p.maxOut));
    } else {
      rq.inScale = p.inScale; rq.inMin = p.inMin; rq.outScale = p.outScale; rq.outOffset = p.outOffset;
      rq.inLowest = -2147483648LL; rq.outLowest = 0; rq.outHighest = 255; rq.mode = 0; rq.fillValue = 0;
      // finish_requant_scalars, done by the launcher
      rq.inScaleFolded = p.rqInScaleFolded; rq.inMinFolded = p.rqInMinFolded; rq.magicFolded = p.rqMagicFolded;
      rq.offsetMinusLowest = p.rqOffsetMinusLowest; rq.offsetMinusLowest32 = p.rqOffsetMinusLowest32;
      rq.fastOK = p.rqFastOK; rq.fast32OK = p.rqFast32OK; rq.foldedOK = p.rqFoldedOK;
      rq.biasedOK = p.rqBiasedOK; rq.inMinBiased = p.rqInMinBiased;
    }
    // The same in every lane whichever branch made them: kept in scalar registers across the main loop, whose
    // vector registers are all spoken for.
    auto uniformInt = [](int x) { return __builtin_amdgcn_readfirstlane(x); };
    auto uniformDouble = [&](double x) {
      return __hiloint2double(uniformInt(__double2hiint(x)), uniformInt(__double2loint(x)));
    };
    auto uniformLong = [&](long long x) {
      return (long long)(((unsigned long long)(unsigned)uniformInt((int)(x >> 32)) << 32) |
                         (unsigned)uniformInt((int)x));
    };
    rq.inScale = uniformDouble(rq.inScale); rq.inMin = uniformDouble(rq.inMin);
    rq.outScale = uniformDouble(rq.outScale); rq.offsetMinusLowest = uniformDouble(rq.offsetMinusLowest);
    rq.inScaleFolded = uniformDouble(rq.inScaleFolded); rq.inMinFolded = uniformDouble(rq.inMinFolded);
    rq.magicFolded = uniformDouble(rq.magicFolded); rq.inMinBiased = uniformDouble(rq.inMinBiased);
    rq.outOffset = uniformLong(rq.outOffset); rq.fillValue = uniformLong(rq.fillValue);
    rq.offsetMinusLowest32 = uniformInt(rq.offsetMinusLowest32); rq.mode = uniformInt(rq.mode);
    rq.fastOK = uniformInt(rq.fastOK); rq.fast32OK = uniformInt(rq.fast32OK);
    rq.foldedOK = uniformInt(rq.foldedOK); rq.biasedOK = uniformInt(rq.biasedOK);
  }

  // 256 accumulator registers set to zero by 16 matrix ops on zero operands (one instruction per block instead
  // of one per register; the operand is a zero the compiler cannot see through)
  v16i acc[MI][NI];
  {
    const int z = (int)(K >> 31);  // K < 2^31
    const v4i zero4 = {z, z, z, z};
    const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NI; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(zero4, zero4, zero16, 0, 0, 0);
  }
  // Column sums of B: wavefront row w owns the blocks j = w and w + 2 of its wavefront column.  The bytes of an
  // operand word are summed as unsigned values of b + 128 (v_sad_u8 against zero: the dot-product instructions
  // hold up the matrix pipeline, this one does not); the 512 per word too much come off at the end.
  unsigned csum[2][4];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int q = 0; q < 4; ++q) csum[t][q] = 0;

  // ---- operand addresses inside stage 0
  const int l32 = lane & 31, g = lane >> 5;
  // A: row wm*128 + 32*i + l32, logical chunk 2*ks + g; 32 rows further on the swizzle is the same
  int aAddr[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int row = wm * 128 + l32;
    aAddr[ks] = row * BK + (((2 * ks + g) ^ swz_a<BK>(row)) << 4);
  }
  // B: transposing read.  Within a block of 16 lanes, lane s points at k row (s >> 1) and 8-byte column half
  // (s & 1) of a 16-byte chunk; lane blocks: (lane >> 4) & 1 selects the 16-column half of the 32-column block,
  // lane >> 5 the k half (g).  k = 32*ks + 16*g + 8*half + trK, so k & 7 == trK.
  const int s16 = lane & 15, colHalf = (lane >> 4) & 1;
  const int trK = s16 >> 1;
  int bAddr[NI];
#pragma unroll
  for (int j = 0; j < NI; ++j)
    bAddr[j] = A_BYTES + (16 * g + trK) * BN + (phys_b(wn * 8 + 2 * j + colHalf, trK) << 4) + ((s16 & 1) << 3);

  // Operand reads of one k step, in the order they are issued: A of row block 0 first (the xor that makes it int8
  // runs at the end of the same step), the two transposing reads of each B block, the other A row blocks between.
  auto loadOne = [&](int stage, int ks, int q, v4i (&af)[MI], v4i (&bf)[NI]) {
    constexpr int kind[12] = {0, 4, 4, 5, 5, 1, 6, 6, 7, 7, 2, 3};  // 0..3: A row block, 4..7: B block
    constexpr int half[12] = {0, 0, 1, 0, 1, 0, 0, 1, 0, 1, 0, 0};
    const unsigned char* st = smem + stage * STAGE_BYTES;
    if (kind[q] < 4) {
      const int i = kind[q];
      af[i] = *reinterpret_cast<const v4i*>(st + aAddr[ks] + i * 32 * BK);
    } else {
      const int j = kind[q] - 4;
      const unsigned char* ptr = st + bAddr[j] + (32 * ks + 8 * half[q]) * BN;
      v2i t = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
          (__attribute__((address_space(3))) v2i*)(const_cast<unsigned char*>(ptr)));
      bf[j][2 * half[q]] = t[0];
      bf[j][2 * half[q] + 1] = t[1];
    }
  };
  // A lone wavefront of a SIMD issues one instruction every four cycles and a matrix op takes 32: between two
  // matrix ops there is room for seven other instructions of any kind, and what does not fit delays the matrix
  // pipeline.  So the work of a k step is dealt out evenly over its 16 matrix ops (slot m = 0..15):
  //   m < 12      one LDS read of the next step's operands (la, lb), from (ldStage, ldKs)
  //   every m     one xor turning a word of the next uint8 A operand into int8: row block m/4 + 1 of this step,
  //               row block 0 of the next step in the last four slots (ua[0] arrives already converted)
  //   m < 8       one word of this wavefront row's column sums (xor + sad)
  //   some m      one HBM -> LDS copy: copies [copy0, copy0 + ncopy) of dmaSlab into dmaStage
  auto step = [&](auto wrow, v4i (&ua)[MI], v4i (&ub)[NI], v4i (&la)[MI], v4i (&lb)[NI], int ldStage, int ldKs,
                  auto dma, unsigned dmaSlab, int dmaStage, int copy0, bool ramp = false, unsigned rampSlab = 0,
                  int rampStage = 0, int rampCopy0 = 0, int rampCopies = 0) {
    constexpr int WROW = decltype(wrow)::value;
    constexpr bool DMA = decltype(dma)::value;
    unsigned soA = 0, soB = 0, rsoA = 0, rsoB = 0;
    if constexpr (DMA) slabOffsets(dmaSlab, soA, soB);
    if (rampCopies > 0) slabOffsets(rampSlab, rsoA, rsoB);
#pragma unroll
    for (int m = 0; m < 16; ++m) {
      const int i = m / NI, j = m % NI;
      if (m < 12) loadOne(ldStage, ldKs, m, la, lb);
      if (m < 12) ua[i + 1][j] ^= (int)0x80808080;
      else la[0][j] ^= (int)0x80808080;
      if constexpr (OWN_COLSUM) {
        if (m < 8) csum[m >> 2][m & 3] = __builtin_amdgcn_sad_u8((unsigned)ub[WROW + 2 * (m >> 2)][m & 3] ^ 0x80808080u, 0u, csum[m >> 2][m & 3]);
      }
      if (m < rampCopies) {  // the first slab's extra copies, ahead of the step's own in issue order
        if (ramp) issueCopy(rsoA, rsoB, rampStage, rampCopy0 + m);
      }
      if constexpr (DMA) {
        constexpr int FIRST = CPS >= 16 ? 0 : 16 - 2 * CPS;  // 16 copies: every slot; fewer: odd slots at the end
        if (CPS >= 16) issueCopy(soA, soB, dmaStage, copy0 + m);
        else if (m >= FIRST && (m & 1)) issueCopy(soA, soB, dmaStage, copy0 + (m - FIRST) / 2);
      }
      // odd row blocks run their four column blocks backwards: the B operand of a row block's last matrix op is
      // the next row block's first, so one operand out of two stays put across the change of row (fewer operand
      // bits switch; the chip is power-limited on data like this, and the measured gain is half a percent)
      const int js = (i & 1) ? NI - 1 - j : j;
      acc[i][js] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ub[js], ua[i], acc[i][js], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // Software pipeline.  The ring holds STAGES slabs; the loop body is STAGES slabs long, so every stage index is
  // a constant.  One barrier per slab, before its last k step:
  //   before it: this wavefront's copies of slab kt+1 have landed
  //   after it : slab kt+1 is complete and visible; nobody reads slab kt's stage any more (the last step's
  //              operands are in registers), so it is refilled with slab kt+STAGES: all copies during the last
  //              step with two stages, spread over the KS steps up to the next barrier with more
  static_assert(STAGES == 2 || COPIES % KS == 0, "copies per step");
  const unsigned KTR = KT;  // a multiple of STAGES (the launcher checks)
  wait_vmcnt<RAMP ? COPIES : COPIES*(STAGES - 2) + (STAGES > 2 ? CPS : COPIES)>();
  __syncthreads();
  v4i fa[2][MI], fb[2][NI];
#pragma unroll
  for (int q = 0; q < 12; ++q) loadOne(0, 0, q, fa[0], fb[0]);
#pragma unroll
  for (int e = 0; e < 4; ++e) fa[0][0][e] ^= (int)0x80808080;
  auto mainLoop = [&](auto wrow) {
    for (unsigned kt0 = 0; kt0 < KTR; kt0 += STAGES) {
#pragma unroll
      for (int s = 0; s < STAGES; ++s) {
        const unsigned kt = kt0 + s;
#pragma unroll
        for (int ks = 0; ks < KS - 1; ++ks) {
          if (RAMP && s == 0)  // slab 0: slab 2 whole, then the step's own copies 4..7 of slab 3
            step(wrow, fa[0], fb[0], fa[1], fb[1], s, 1, std::true_type{}, kt - 1 + STAGES, STAGES - 1, CPS,
                 kt0 == 0, 2u, 2, 0, COPIES);
          else if constexpr (STAGES > 2)  // copies (ks+1)*CPS.. of the slab that takes the place of slab kt-1
            step(wrow, fa[ks & 1], fb[ks & 1], fa[(ks + 1) & 1], fb[(ks + 1) & 1], s, ks + 1, std::true_type{},
                 kt - 1 + STAGES, (s + STAGES - 1) % STAGES, (ks + 1) * CPS);
          else
            step(wrow, fa[ks & 1], fb[ks & 1], fa[(ks + 1) & 1], fb[(ks + 1) & 1], s, ks + 1, std::false_type{}, 0u, 0, 0);
        }
        if (RAMP && s == 0) {
          // slab 0's barrier: after slab 1's copies came slab 2 (8) and copies 4..7 of slab 3
          if (kt0 == 0) wait_vmcnt<COPIES + CPS>();
          else wait_vmcnt<COPIES*(STAGES - 2)>();
          __syncthreads();
          // copies 0..3 of slab 3, then the step's own
          step(wrow, fa[1], fb[1], fa[0], fb[0], 1, 0, std::true_type{}, kt + STAGES, s, 0, kt0 == 0, 3u, 3, 0, CPS);
        } else {
          wait_vmcnt<COPIES*(STAGES - 2)>();
          __syncthreads();
          step(wrow, fa[1], fb[1], fa[0], fb[0], (s + 1) % STAGES, 0, std::true_type{}, kt + STAGES, s, 0);
        }
      }
    }
  };
  if constexpr (OWN_COLSUM) {
    if (wm == 0) mainLoop(std::integral_constant<int, 0>{});
    else mainLoop(std::integral_constant<int, 1>{});
  } else {
    mainLoop(std::integral_constant<int, 0>{});
  }
  wait_vmcnt<0>();
  __syncthreads();

  // ---- epilogue.  Accumulator layout (operands swapped): lane (l32, g) holds row l32 of the 32-row
  // block and columns 8*(r/4) + 4*g + r%4 of the 32-column block, r = 0..15.
  int* colTerm = reinterpret_cast<int*>(smem);   // [BN]
  int* rowTerm = colTerm + BN;                   // [BM]
  // lanes l and l+32 hold the two k halves of the same column; the transposing read hands lane
  // (colHalf, s16) column 16*colHalf + s16 of the 32-column block
  if constexpr (OWN_COLSUM) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int j = wm + 2 * t;
      // every word summed held four bytes of b + 128: KTR * KS words per partial sum
      int s = (int)(csum[t][0] + csum[t][1] + csum[t][2] + csum[t][3] - 2048u * KTR * KS);
      s += __shfl_xor(s, 32, 64);
      if (g == 0) colTerm[wn * 128 + 32 * j + 16 * colHalf + s16] = s;
    }
    __syncthreads();
  }
  const unsigned global = (unsigned)offA * (unsigned)offB * K;
  colTerm[tid] = (int)(128u * (OWN_COLSUM ? (unsigned)colTerm[tid] : csPre) + csPre * (unsigned)offA);
  rowTerm[tid] = (int)(global + rsPre * (unsigned)offB);
  __syncthreads();

  int* C = WRITE_C ? p.C + (size_t)bi * p.strideC : nullptr;
  unsigned char* Q = REQUANT ? p.Q + (size_t)bi * p.strideC : nullptr;

  // Requantized values leave the registers directly: a lane packs the four uint8 of each of its column quads
  // into a word (two saturating conversions: int32 -> int16 -> uint8, which is the clamp to 0..255), the two
  // half-wavefronts that share a row exchange two of their four words per 32 x 32 block so that each ends up
  // with 16 consecutive columns, and a 128-bit store per block writes 32 bytes of a row per lane pair.
  auto storeTileChecked = [&](auto flavour, auto inside) __attribute__((always_inline)) {
    constexpr int FLAVOUR = decltype(flavour)::value;
    // 0 int32 only, 1 double shortcut, 2 exact int64, 3 fill, 4 int32 shortcut, 5 folded, 6 biased
    constexpr bool INSIDE = decltype(inside)::value;  // the whole tile lies inside the matrix: no bounds tests
#pragma unroll
    for (int i = 0; i < MI; ++i) {
      const int trow = wm * 128 + 32 * i + l32;
      const unsigned grow = m0 + trow;
      // without an int32 result to store, the 2^31 that turns the accumulator into its offset from INT32_MIN is
      // folded into the row term
      constexpr unsigned kBias = (REQUANT && !WRITE_C) ? 0x80000000u : 0u;
      const int rt = (int)((unsigned)rowTerm[trow] + kBias);
#pragma unroll
      for (int j = 0; j < NI; ++j) {
        unsigned packed[4];
#pragma unroll
        for (int rq4 = 0; rq4 < 4; ++rq4) {
          const int tcol = wn * 128 + 32 * j + 8 * rq4 + 4 * g;  // first of 4 consecutive columns
          const v4i ct = *reinterpret_cast<const v4i*>(colTerm + tcol);
          int v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = (int)((unsigned)acc[i][j][4 * rq4 + e] + (unsigned)rt + (unsigned)ct[e]);
          if constexpr (WRITE_C) {
            if (INSIDE || (grow < M && n0 + tcol < N))  // N % 16 == 0: the four columns are in or out together
              *reinterpret_cast<v4i*>(C + (size_t)grow * N + n0 + tcol) = v4i{v[0], v[1], v[2], v[3]};
          }
          if constexpr (FLAVOUR != 0) {
            int q[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const unsigned off = (unsigned)v[e] ^ (0x80000000u ^ kBias);  // v - INT32_MIN
              if constexpr (FLAVOUR == 1) q[e] = requantize_one_fast((double)off, rq);
              else if constexpr (FLAVOUR == 2) q[e] = (int)requantize_one_exact((long long)(int)(off ^ 0x80000000u), rq);
              else if constexpr (FLAVOUR == 4) q[e] = requantize_one_fast32_unclamped((double)off, rq);
              else if constexpr (FLAVOUR == 5) q[e] = requantize_one_folded_unclamped((double)off, rq);
              else if constexpr (FLAVOUR == 6) q[e] = requantize_one_biased_unclamped(off, rq);
              else q[e] = (int)rq.fillValue;
            }
            packed[rq4] = pack_sat_u8(q[0], q[1], q[2], q[3]);
          }
        }
        if constexpr (FLAVOUR != 0) {
          // quads 0, 2 and 1, 3: the upper half-wavefront's first word against the lower one's second
          const auto s02 = __builtin_amdgcn_permlane32_swap(packed[0], packed[2], false, false);
          const auto s13 = __builtin_amdgcn_permlane32_swap(packed[1], packed[3], false, false);
          const unsigned gcol = n0 + wn * 128 + 32 * j + 16 * g;
          if (INSIDE || (grow < M && gcol < N))
            *reinterpret_cast<v4i*>(Q + (size_t)grow * N + gcol) = v4i{(int)s02[0], (int)s02[1], (int)s13[0], (int)s13[1]};
        }
      }
    }
  };
  const bool tileInside = m0 + BM <= M && n0 + BN <= N;  // the same for the whole workgroup
  auto storeTile = [&](auto flavour) __attribute__((always_inline)) {
    if (tileInside) storeTileChecked(flavour, std::true_type{});
    else storeTileChecked(flavour, std::false_type{});
  };
  if constexpr (!REQUANT) {
    storeTile(std::integral_constant<int, 0>{});
  } else {
    if (rq.mode) storeTile(std::integral_constant<int, 3>{});
    else if (rq.biasedOK) storeTile(std::integral_constant<int, 6>{});
    else if (rq.foldedOK) storeTile(std::integral_constant<int, 5>{});
    else if (rq.fast32OK) storeTile(std::integral_constant<int, 4>{});
    else if (rq.fastOK) storeTile(std::integral_constant<int, 1>{});
    else storeTile(std::integral_constant<int, 2>{});
  }
}

template <int BK, int STAGES, bool REQUANT, bool WRITE_C, bool OWN_COLSUM>
int launch_w4(hipStream_t stream, QGemmParams p) {
  p.tilesM = (p.M + BM - 1) / BM;
  p.tilesN = (p.N + BN - 1) / BN;
  unsigned long long total = (unsigned long long)p.tilesM * p.tilesN * p.batch;
  if (total > 0x7fffffffull) return set_error(TFCC_ROCM_INVALID_ARGUMENT, "quantized matmul: too many tiles");
  p.tilesTotal = (unsigned)total;
  p.chunk = (p.tilesTotal + 7) / 8;
  if (REQUANT && !p.minOut) {
    RequantScalars rq;
    rq.inScale = p.inScale; rq.inMin = p.inMin; rq.outScale = p.outScale; rq.outOffset = p.outOffset;
    rq.inLowest = -2147483648LL; rq.outLowest = 0; rq.outHighest = 255; rq.mode = 0; rq.fillValue = 0;
    finish_requant_scalars(rq, 4294967295.0);
    p.rqInScaleFolded = rq.inScaleFolded; p.rqInMinFolded = rq.inMinFolded; p.rqMagicFolded = rq.magicFolded;
    p.rqOffsetMinusLowest = rq.offsetMinusLowest; p.rqOffsetMinusLowest32 = rq.offsetMinusLowest32;
    p.rqFastOK = rq.fastOK; p.rqFast32OK = rq.fast32OK; p.rqFoldedOK = rq.foldedOK;
    p.rqBiasedOK = rq.biasedOK; p.rqInMinBiased = rq.inMinBiased;
  }
  const UDiv perBatch = udiv_prepare(p.tilesM * p.tilesN), band = udiv_prepare(4u * p.tilesN);
  p.perBatchMagic = perBatch.magic; p.perBatchShift = perBatch.shift;
  p.bandMagic = band.magic; p.bandShift = band.shift;
  constexpr size_t ring = (size_t)STAGES * (BM + BN) * BK;
  constexpr size_t epi = (size_t)(BM + BN) * 4;
  constexpr size_t lds = ring > epi ? ring : epi;
  static_assert(lds <= 160 * 1024, "LDS budget");
  auto kern = qgemm_w4_kernel<BK, STAGES, REQUANT, WRITE_C, OWN_COLSUM>;
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
  return check_launch("quantized matmul (four wavefronts)");
}

template <int BK, int STAGES, bool OWN_COLSUM>
int launch_w4_for_outputs(hipStream_t stream, const QGemmParams& p, bool requant) {
  if (!requant) return launch_w4<BK, STAGES, false, true, OWN_COLSUM>(stream, p);
  return p.C ? launch_w4<BK, STAGES, true, true, OWN_COLSUM>(stream, p)
             : launch_w4<BK, STAGES, true, false, OWN_COLSUM>(stream, p);
}

}  // namespace

// On top of what the eight-wavefront kernel asks for: K a multiple of the ring's length in bytes of k.
bool qgemm_w4_supported(const QGemmParams& p) { return p.K % 256 == 0; }

int qgemm_w4_launch(hipStream_t stream, const QGemmParams& p, bool requant) {
  // slabs of 64 bytes of k in a ring of four: copies are asked for two slabs before the barrier that needs them
  return p.colsumExact ? launch_w4_for_outputs<64, 4, false>(stream, p, requant)
                       : launch_w4_for_outputs<64, 4, true>(stream, p, requant);
}

}  // namespace tfcc_rocm
