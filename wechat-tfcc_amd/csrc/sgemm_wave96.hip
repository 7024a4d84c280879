// fp32 matrix product with the instruction order written down: one wavefront per SIMD, 32 rows x NI column blocks of
// 32 per wavefront (NI = 3, 32 x 96 outputs, in the description below).
//
// A product like 1024 x 3072 x 768 has about one tile per CU, so nothing overlaps a workgroup's stalls except its
// own instruction order, and on this hardware nothing overlaps the fp32 matrix ops at all: while one wavefront issues
// them back to back, vector instructions of every wavefront on the SIMD wait (a vector instruction between two
// matrix ops costs about 15 cycles, an LDS read 1.5, a copy 2, scalar instructions nothing).  So the order is
// written down and the loop holds matrix ops, LDS reads, copies and scalar work only: a k step is twelve 32x32x2
// matrix ops (4 k pairs x 3 column blocks, 64 cycles each); the LDS reads of the next step's operands (one 128-bit
// read of A, six two-word reads of B) and the step's share of the HBM -> LDS copies are dealt out over the issue
// slots between them, one step ahead, into a second set of registers; the loop is unrolled over the ring's stages so
// that every LDS address is a register set up before the loop plus an immediate.  Measured in the loop: 64.3-65.5
// cycles per matrix op.
//
// Shapes of workgroup (WGM row blocks of 32 x KSPLIT K groups wavefronts, NI column blocks of 32 per wavefront):
//   groups (WGM = 1, KSPLIT = 4)  a 32 x 32 NI tile, wavefront q sums the 32-k slabs q, q + 4, ... in a ring of its
//                                 own (two half slabs of 16 k, or three of 8 k when three workgroups share a CU, so
//                                 that one's set-up and tile store run under the others' matrix ops; no barrier
//                                 in the loop); the four partial tiles meet in LDS and every wavefront finishes a
//                                 quarter of the tile.  For products the dispatcher sums in four K groups:
//                                 1024 x 768 x 3072 36.3 us against 45.9 for the twelve-wavefront kernel of
//                                 sgemm_dma.hip, three 1024 x 768 x 768 products in one launch 29.5 against 39.9;
//                                 with NI = 2 and NI = 1 the 32 x 64 and 32 x 32 tiles (128 x 768 x 3072: 8.6
//                                 against 11.4 us with the operands in cache).
//          (WGM = 2, KSPLIT = 4)  the same on a 64 x 64 tile: four pairs of wavefronts, a pair sharing its ring.
//          (WGM = 2 or 1, KSPLIT = 2)  two K groups: two pairs of wavefronts on a 64 x 64 tile, or two wavefronts on
//                                 a 32 x 32 tile; a wavefront finishes two quarters of its rows.
//   rows   (WGM = 4, KSPLIT = 1)  a 128 x 32 NI tile, wavefront w owns rows 32w..32w+31, the ring (two slabs of 32 k)
//                                 is shared, one barrier per slab.  For products summed in one pass over K whose
//                                 tiles fill the CUs: 1024 x 3072 x 768 with GELU 39.3 us against 42.4 in 64 x 64
//                                 tiles (NI = 3); 4096^3 150 against 141 TFLOP/s (NI = 4, two workgroups per CU).
// Whole tiles are stored through a buffer descriptor (a lane offset, a scalar per row, an immediate per column
// block: no address arithmetic or bounds checks per value); edge tiles take the checked path.
// The arithmetic is that of sgemm_dma.hip instruction for instruction (k pairs (8kb + s, 8kb + 4 + s) in ascending
// kb, s; groups added in group order), so a product has the same bits whichever kernel the dispatcher picks for its
// number of K groups.  Replaces the same oneDNN calls (tfcc/mkl/interfaces/tfcc_mklblasinterface.cpp:41-67, 69-78,
// 87-118).  Taken for 16-byte aligned operands and strides, K a multiple of 32, B not transposed.
#include "common.hpp"
#include "copy_offsets.hpp"
#include "lds_dma.hpp"
#include "sgemm_params.hpp"

namespace tfcc_rocm {

typedef float w96_v4f __attribute__((ext_vector_type(4)));
typedef float w96_v16f __attribute__((ext_vector_type(16)));
typedef lds_dma_v4i w96_v4i;

namespace {

using sgemm_detail::SgemmParams;

// 16-byte chunk c of A row `row` lies at chunk c ^ swizzle: rows of 128 bytes (32 k), 64 bytes (16 k), 32 bytes (8 k)
template <int BK>
__device__ __forceinline__ int a_row_swizzle(int row) {
  return BK == 32 ? (row >> 1) & 7 : BK == 16 ? (row >> 2) & 3 : (row >> 2) & 1;
}

template <int WGM, int KSPLIT, int BK, int STAGES, bool PLAIN, int NI, bool RAMP>
__global__ __launch_bounds__(64 * WGM * KSPLIT > 256 ? 64 * WGM * KSPLIT : 256) void sgemm_wave96_kernel(
    const float* hotA, const float* hotB, const float* hotB1, const float* hotB2, unsigned hotM, unsigned hotN,
    unsigned hotK, unsigned hotLda, unsigned hotLdb, unsigned hotBatch, const SgemmParams p) {
  // The leading arguments repeat what the first copies need: scalar arguments at the front of the list arrive in
  // registers with the wavefront, the structure has to be fetched from the argument block first, and nothing of it
  // is looked at before the first slabs are on their way when PLAIN (every batch entry's A starts at hotA, and
  // either its B at hotB too or the launch is the grouped form with at most three products: hotB, hotB1, hotB2 are
  // their B).  hotBatch: p.batch, bit 30 set for the grouped form.
  static_assert(WGM * KSPLIT == 4 || WGM * KSPLIT == 2 || WGM * KSPLIT == 8,
                "four wavefronts (one per SIMD), two, or eight");
  static_assert(KSPLIT == 1 || KSPLIT == 2 || KSPLIT == 4, "the quads of a column block divide among the K groups");
  static_assert(NI >= 1 && NI <= 4, "one to four column blocks of 32 per wavefront");
  constexpr int BN = 32 * NI;       // columns of a tile
  static_assert(BK == 32 || BK == 16 || BK == 8, "ring slabs of 32, 16 or 8 k");
  static_assert(STAGES >= 2, "ring depth");
  static_assert(!RAMP || (STAGES >= 3 && BK <= 16 && WGM == 1), "the ramp fills the last stage during slab 0's first step");
  constexpr int BM = 32 * WGM;
  constexpr int KS = BK / 8;        // k steps per ring slab
  constexpr int CH = BK / 4;        // 16-byte chunks per A row
  constexpr int SUB = 32 / BK;      // ring slabs per 32-k slab of the product
  constexpr int A_BYTES = BM * BK * 4, B_BYTES = BK * BN * 4, STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int A_UNITS = A_BYTES / 1024, UNITS = STAGE_BYTES / 1024;  // 1 KB copies per ring slab
  static_assert(UNITS % WGM == 0, "every wavefront of a group issues the same number of copies");
  constexpr int COPIES = UNITS / WGM;
  static_assert(COPIES <= 4 * NI - 1 && COPIES * STAGES < 64, "copies fit the slots of one step and the vmcnt range");
  constexpr int GROUP_BYTES = STAGES * STAGE_BYTES;
  constexpr int BCH = BN / 4;     // 16-byte chunks per B row
  constexpr bool SHARED = WGM > 1;  // the group's wavefronts read each other's copies

  extern __shared__ __align__(16) unsigned char smem[];
  const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int grp = wv / WGM, wm = wv - grp * WGM;  // wave-uniform
  const int lane = threadIdx.x & 63;
  unsigned char* gsm = smem + grp * GROUP_BYTES;
  const unsigned ldsGroup = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)gsm;

  unsigned tm, tn, bi;
  {
    // consecutive workgroup ids land on different XCDs: hand each XCD a contiguous run of tiles
    const unsigned wg = blockIdx.x;
    const unsigned xcd = wg & 7u, slot = wg >> 3;
    const unsigned tilesM = (hotM + BM - 1) / BM, tilesN = (hotN + BN - 1) / BN;
    const unsigned perBatch = tilesM * tilesN;
    const unsigned tilesTotal = perBatch * (hotBatch & 0x3fffffffu);  // the launcher checks that this fits
    const unsigned chunk = (tilesTotal + 7u) / 8u;
    const unsigned L = xcd * chunk + slot;
    if (slot >= chunk || L >= tilesTotal) return;
    // (a division is some thirty instructions in front of the first copies: the common cases - one product, a band
    // of a power of two of tiles, whole bands - go without)
    const bool oneProduct = tilesTotal == perBatch;
    bi = oneProduct ? 0u : L / perBatch;
    unsigned t = L - bi * perBatch;
    const unsigned band = 4u * tilesN;
    unsigned gb = (band & (band - 1u)) == 0u ? t >> (unsigned)__builtin_ctz(band) : t / band;
    unsigned rowsInBand = min(4u, tilesM - gb * 4u);
    unsigned r = t - gb * band;
    const unsigned rq = rowsInBand == 4u ? r >> 2 : r / rowsInBand;
    tm = gb * 4u + (r - rq * rowsInBand);
    tn = rq;
  }
  const unsigned m0 = tm * BM, n0 = tn * BN;
  const unsigned M = hotM, N = hotN, K = hotK;
  const bool grouped = (hotBatch >> 30) & 1u;
  const float* A = hotA;
  const float* B = hotB;
  if (grouped) {
    B = bi == 1 ? hotB1 : bi == 2 ? hotB2 : B;
    if (!PLAIN) B = bi == 3 ? p.groupB[3] : B;
  } else if (!PLAIN) {
    const unsigned bo = bi / p.batchInner, bn = bi - bo * p.batchInner;
    A += (size_t)bo * p.strideA + (size_t)bn * p.innerA;
    B += (size_t)bo * p.strideB + (size_t)bn * p.innerB;
  }
  const unsigned lda = hotLda, ldb = hotLdb;
  const w96_v4i rsrcA = make_rsrc(A, ((M - 1) * lda + K) * 4u);
  const w96_v4i rsrcB = make_rsrc(B, ((K - 1) * ldb + N) * 4u);

  const int lrow = lane & 31, g = lane >> 5;

  // ---- copy descriptors.  Copy c of a ring slab is unit u = c * WGM + wm of the group's stage image; LDS slot s
  // (16 bytes) of the A image holds row s / CH, physical chunk s % CH = logical chunk ^ swizzle(row); slot s of the
  // B image holds k row s / BCH, chunk s % BCH.  The lane offsets are those of k = 0; the slab's k goes into the
  // copy's scalar offset.
  unsigned off[COPIES];
#pragma unroll
  for (int c = 0; c < COPIES; ++c) {
    const int u = c * WGM + wm;
    if (u < A_UNITS) {
      const int s = u * 64 + lane, row = s / CH, phys = s % CH;
      off[c] = ((m0 + row) * lda + ((phys ^ a_row_swizzle<BK>(row)) << 2)) * 4u;
    } else {
      // (columns past N: an offset that fails the range check whatever the slab's scalar offset, copy_offsets.hpp)
      off[c] = copy_offsets::w96_b_lane_offset((u - A_UNITS) * 64 + lane, BCH, n0, N, ldb);
    }
  }
  // ring slab t of this group covers k0(t) .. k0(t) + BK - 1; past the end of K it is all zeros
  const unsigned slabs32 = K / 32;                                      // the launcher checks K % 32 == 0
  const unsigned T = ((slabs32 + KSPLIT - 1) / KSPLIT) * SUB;            // ring slabs per group
  auto k0Of = [&](unsigned t) { return ((t / SUB) * KSPLIT + grp) * 32u + (t % SUB) * BK; };
  // Nothing of a copy's set-up runs on the vector unit (a vector instruction between two matrix ops delays the
  // second by some 15 cycles): the lane offsets never change, the slab's k goes into the scalar offset, and a slab
  // past the end of K is read through a descriptor of size zero, which makes every lane read zeros.
  auto issueCopy = [&](unsigned t, unsigned stage, int c) {
    const unsigned k0 = k0Of(t);
    const bool live = k0 < K;
    const int u = c * WGM + wm;
    const bool isA = u < A_UNITS;
    const unsigned dst = ldsGroup + stage * STAGE_BYTES + u * 1024;
    const unsigned so = isA ? k0 * 4u : k0 * ldb * 4u;
    w96_v4i rsrc = isA ? rsrcA : rsrcB;
    rsrc[2] = live ? rsrc[2] : 0;
    dma16s(rsrc, dst, off[c], live ? so : 0u);
  };

  // the first slabs are on their way before anything else is set up (RAMP: all but the last stage's, which is asked
  // for during the first step of slab 0 - what is asked for at the start delays the first slab, 0.4 us per slab
  // with operands in HBM)
#pragma unroll
  for (int s = 0; s < (RAMP ? STAGES - 1 : STAGES); ++s)
#pragma unroll
    for (int c = 0; c < COPIES; ++c) issueCopy((unsigned)s, (unsigned)s, c);

  // What the tile store needs from the argument block is worked out from here on (the empty statement keeps the
  // compiler from moving it, and the wait for the block, in front of the copies).
  unsigned late = 0;
  asm volatile("" : "+s"(late));
  const unsigned biL = bi + late;
  const unsigned ldc = p.ldc;
  const float* biasPtr = p.bias;
  float* Cbase;
  if (grouped) {  // selects, not indexing: the argument block stays in scalar registers
    biasPtr = biL == 0 ? p.groupBias[0] : biL == 1 ? p.groupBias[1] : biL == 2 ? p.groupBias[2] : p.groupBias[3];
    Cbase = biL == 0 ? p.groupC[0] : biL == 1 ? p.groupC[1] : biL == 2 ? p.groupC[2] : p.groupC[3];
  } else {
    const unsigned bo = biL / p.batchInner, bn = biL - bo * p.batchInner;
    Cbase = p.C + (size_t)bo * p.strideC + (size_t)bn * p.innerC;
  }

  // ---- values needed only in the tile store are fetched now.  Rows: lane (lrow, g) stores, for register r of
  // column block j, row 8*(r/4) + 4*g + r%4 of its wavefront's 32 and column 32*j + lrow.  Groups: after the
  // partial tiles met in LDS, wavefront w finishes registers 4w .. 4w+3 of each column block (rows 8w + 4g + e):
  // value q = 4j + e of its twelve is register 4w + e of block j.
  constexpr int QPW = 4 / KSPLIT;   // quads of four registers of each column block that a wavefront finishes
  constexpr int OWN = 4 * QPW * NI; // values a lane finishes: value q is register 4 (grp QPW + q / 4 % QPW) + q % 4 of
                                    // block q / (4 QPW)
  auto ownBlock = [&](int q) { return q / (4 * QPW); };
  auto ownRegister = [&](int q) { return 4 * ((KSPLIT == 1 ? 0 : grp * QPW) + (q >> 2) % QPW) + (q & 3); };
  const unsigned gcol0 = n0 + lrow;
  float bv[NI];
#pragma unroll
  for (int j = 0; j < NI; ++j) bv[j] = (biasPtr && gcol0 + 32 * j < N) ? biasPtr[gcol0 + 32 * j] : 0.f;
  float rv[OWN];
  const float* Rp = p.residual ? p.residual + (size_t)biL * p.strideR : nullptr;  // dense, flat batch
  if (Rp) {
#pragma unroll
    for (int q = 0; q < OWN; ++q) {
      const int j = ownBlock(q), r = ownRegister(q);
      const unsigned grow = m0 + wm * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
      const unsigned gc = gcol0 + 32 * j;
      rv[q] = (grow < M && gc < N) ? Rp[(size_t)grow * N + gc] : 0.f;
    }
  }

  w96_v16f acc[NI];
#pragma unroll
  for (int j = 0; j < NI; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;

  // ---- operand addresses inside a stage: A row wm*32 + lrow, logical chunk 2*kb + g; B column 32*j + lrow,
  // k rows 8*kb + 4*g + s
  const int arow = wm * 32 + lrow;
  const int aBase = arow * (BK * 4), aSwz = a_row_swizzle<BK>(arow);
  const int bBase = A_BYTES + (4 * g) * (BN * 4) + lrow * 4;
  struct Ops { w96_v4f a; float b[4][NI]; };
  // In the unrolled part of the loop the stage is a constant, and every LDS address is one of a few registers set up
  // here plus an immediate: no address arithmetic between the matrix ops.  The B operands of a step are then read two
  // per instruction (two offsets of up to 255 words from one register: a register per stage, k step and half step).
  typedef const __attribute__((address_space(3))) float* LdsFloats;
  typedef const __attribute__((address_space(3))) w96_v4f* LdsQuads;
  constexpr bool PAIRED = STAGES * KS * 2 <= (NI <= 2 ? 12 : 8);
  unsigned aAddr[KS], bAddr[PAIRED ? STAGES : 1][KS][2];
#pragma unroll
  for (int kb = 0; kb < KS; ++kb) {
    aAddr[kb] = ldsGroup + aBase + (((2 * kb + g) ^ aSwz) << 4);
    asm volatile("" : "+v"(aAddr[kb]));
#pragma unroll
    for (int st = 0; st < (PAIRED ? STAGES : 1); ++st)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        bAddr[st][kb][h] = ldsGroup + st * STAGE_BYTES + bBase + (8 * kb + 2 * h) * (BN * 4);
        asm volatile("" : "+v"(bAddr[st][kb][h]));
      }
  }

  // One k step: twelve matrix ops on `cur`; in the issue slots between them the reads of the operands of step
  // (ldStage, ldKb) into `nxt` and, in a slab's last step, the copies of the slab that takes its stage.  fixedStage:
  // ldStage is a constant where the call is written.
  auto step = [&](const Ops& cur, Ops& nxt, unsigned ldStage, int ldKb, bool fixedStage, bool dma, unsigned dmaSlab,
                  unsigned dmaStage) __attribute__((always_inline)) {
    const unsigned char* st = gsm + ldStage * STAGE_BYTES;
#pragma unroll
    for (int m = 0; m < 4 * NI; ++m) {
      const int s = m / NI, j = m % NI;
      if (fixedStage) {
        if (m == 0) nxt.a = *reinterpret_cast<LdsQuads>(aAddr[ldKb] + ldStage * STAGE_BYTES);
        if (PAIRED) {
          if (m & 1) {  // values 2 * (m / 2) and 2 * (m / 2) + 1 of the step's 4 NI, NI to a k row
#pragma unroll
            for (int e = 0; e < 2; ++e) {
              const int v = (m / 2) * 2 + e, vs = v / NI, vj = v % NI;
              nxt.b[vs][vj] = reinterpret_cast<LdsFloats>(bAddr[PAIRED ? ldStage : 0][ldKb][vs / 2])[(vs & 1) * BN + vj * 32];
            }
          }
        } else {
          nxt.b[s][j] = reinterpret_cast<LdsFloats>(bAddr[0][ldKb][0] + ldStage * STAGE_BYTES)[s * BN + j * 32];
        }
      } else {
        if (m == 0) nxt.a = *reinterpret_cast<const w96_v4f*>(st + aBase + (((2 * ldKb + g) ^ aSwz) << 4));
        nxt.b[s][j] = *reinterpret_cast<const float*>(st + bBase + (8 * ldKb + s) * (BN * 4) + j * 128);
      }
      if (dma && m >= 1 && m <= COPIES) issueCopy(dmaSlab, dmaStage, m - 1);
      acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(cur.a[s], cur.b[s][j], acc[j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // ---- software pipeline.  At the start of slab t's last step: this wavefront's copies of slab t+1 have landed
  // and its reads of slab t have returned; with a shared ring a barrier makes that true of the whole group.  Then
  // slab t+1 is complete and visible, and slab t's stage is free: it is refilled with slab t+STAGES while the last
  // step's matrix ops run on operands already in registers.
  wait_vmcnt<COPIES*((RAMP ? STAGES - 1 : STAGES) - 1)>();
  if constexpr (SHARED) __syncthreads();
  Ops ops[2];
  ops[0].a = *reinterpret_cast<const w96_v4f*>(gsm + aBase + ((g ^ aSwz) << 4));
#pragma unroll
  for (int s = 0; s < 4; ++s)
#pragma unroll
    for (int j = 0; j < NI; ++j) ops[0].b[s][j] = *reinterpret_cast<const float*>(gsm + bBase + s * (BN * 4) + j * 128);
  // one ring slab in stage `stage`: KS steps starting on the operands in `first`; the next slab's first operands end
  // up in `first` again when KS is even, in `other` when it is odd (then the loops below alternate the two)
  auto slab = [&](unsigned t, unsigned stage, bool fixedStage, Ops& first, Ops& other) __attribute__((always_inline)) {
    const unsigned next = stage + 1 == STAGES ? 0 : stage + 1;
#pragma unroll
    for (int kb = 0; kb < KS - 1; ++kb)
      step(kb & 1 ? other : first, kb & 1 ? first : other, stage, kb + 1, fixedStage, RAMP && kb == 0 && t == 0,
           (unsigned)(STAGES - 1), (unsigned)(STAGES - 1));
    wait_vmcnt<COPIES*(STAGES - 2)>();
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the reads of slab t have returned
    if constexpr (SHARED) __syncthreads();
    step((KS - 1) & 1 ? other : first, (KS - 1) & 1 ? first : other, next, 0, fixedStage, true, t + STAGES, stage);
  };
  // U slabs per trip with the stages written out (a multiple of the ring depth, even when the operand sets
  // alternate); what is left of T after whole trips runs with the stage counted.  T is a multiple of 32 / BK.
  constexpr int ALT = (KS & 1) ? 2 : 1;
  constexpr int U = STAGES % ALT == 0 ? STAGES : STAGES * ALT;
  unsigned t = 0;
  for (; t + U <= T; t += U) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const bool odd = (KS & 1) && (u & 1);
      slab(t + u, u % STAGES, true, ops[odd ? 1 : 0], ops[odd ? 0 : 1]);
    }
  }
  unsigned stage = 0;  // U is a multiple of the ring depth
  for (; t < T; t += ALT) {
    slab(t, stage, false, ops[0], ops[1]);
    stage = stage + 1 == STAGES ? 0 : stage + 1;
    if constexpr (KS & 1) {
      slab(t + 1, stage, false, ops[1], ops[0]);
      stage = stage + 1 == STAGES ? 0 : stage + 1;
    }
  }
  wait_vmcnt<0>();
  __syncthreads();

  // ---- tile store: + bias, + residual, GELU
  const int act = p.act;
  auto finish = [&](float v, int q, int j) {
    v += bv[j];
    if (Rp) v += rv[q];
    // same expression as the stand-alone GELU kernel, so that fusing changes no bit
    if (act == 1) v = gelu_erf_f32(v);
    return v;
  };
  if constexpr (KSPLIT == 1) {
    if (m0 + wm * 32 + 32 <= M && n0 + BN <= N && ldc < (1u << 24)) {
      // A whole tile: no bounds to check, and the addresses are a register per lane (row 4g, column lrow), a scalar
      // per row and an immediate per column block.
      const __amdgpu_buffer_rsrc_t rc =
          __builtin_amdgcn_make_buffer_rsrc(Cbase + (size_t)(m0 + wm * 32) * ldc + n0, 0, 0x7fffffff, 0x00020000);
      const unsigned voff = ((4 * g) * ldc + lrow) * 4u;
      auto store = [&](bool gelu) __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < 16; ++r)
#pragma unroll
          for (int j = 0; j < NI; ++j) {
            float out = acc[j][r] + bv[j];
            if (Rp) out += rv[j * 16 + r];
            if (gelu) out = gelu_erf_f32(out);
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, out), rc, voff + j * 128,
                                                  (8 * (r >> 2) + (r & 3)) * ldc * 4u, 0);
          }
      };
      if (act == 1) store(true); else store(false);
      return;
    }
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const unsigned gc = gcol0 + 32 * j;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const unsigned grow = m0 + wm * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
        if (grow < M && gc < N) Cbase[(size_t)grow * ldc + gc] = finish(acc[j][r], j * 16 + r, j);
      }
    }
  } else {
    // the partial tiles of the K groups go through LDS (the rings are idle now), four registers per 128-bit access:
    // registers 4c .. 4c+3 of column block j of the wavefront (group q, rows wm) lie at
    // red4[(((q * WGM + wm) * NI + j) * 4 + c) * 64 + lane]; wavefront (grp, wm) adds the quads c = grp QPW .. of every
    // block in group order
    w96_v4f* red4 = reinterpret_cast<w96_v4f*>(smem);
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int c = 0; c < 4; ++c)
        red4[(((grp * WGM + wm) * NI + j) * 4 + c) * 64 + lane] =
            w96_v4f{acc[j][4 * c], acc[j][4 * c + 1], acc[j][4 * c + 2], acc[j][4 * c + 3]};
    __syncthreads();
    float sums[OWN];
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int cq = 0; cq < QPW; ++cq) {
        const int c = grp * QPW + cq;
        w96_v4f v = red4[((wm * NI + j) * 4 + c) * 64 + lane];
#pragma unroll
        for (int o = 1; o < KSPLIT; ++o) {
          const w96_v4f w = red4[(((o * WGM + wm) * NI + j) * 4 + c) * 64 + lane];
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] += w[e];
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) sums[(j * QPW + cq) * 4 + e] = v[e];
      }
    if (m0 + wm * 32 + 32 <= M && n0 + BN <= N && ldc < (1u << 24)) {
      // A whole tile: no bounds to check, and the addresses are a register per lane (row 4g, column lrow of the
      // wavefront's 8 QPW rows), a scalar per row and an immediate per column block.
      const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc(
          Cbase + (size_t)(m0 + wm * 32 + 8 * grp * QPW) * ldc + n0, 0, 0x7fffffff, 0x00020000);
      const unsigned voff = ((4 * g) * ldc + lrow) * 4u;
      auto store = [&](bool gelu) __attribute__((always_inline)) {
#pragma unroll
        for (int q = 0; q < OWN; ++q) {
          const int j = q / (4 * QPW), cq = (q >> 2) % QPW, e = q & 3;
          float out = sums[q] + bv[j];
          if (Rp) out += rv[q];
          if (gelu) out = gelu_erf_f32(out);
          __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, out), rc, voff + j * 128,
                                                (8 * cq + e) * ldc * 4u, 0);
        }
      };
      if (act == 1) store(true); else store(false);
      return;
    }
#pragma unroll
    for (int q = 0; q < OWN; ++q) {
      const int j = ownBlock(q), r = ownRegister(q);
      const unsigned grow = m0 + wm * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
      const unsigned gc = gcol0 + 32 * j;
      float out = sums[q] + bv[j];
      if (Rp) out += rv[q];
      if (act == 1) out = gelu_erf_f32(out);
      if (grow < M && gc < N) {
        Cbase[(size_t)grow * ldc + gc] = out;
      }
    }
  }
}

template <int WGM, int KSPLIT, int BK, int STAGES, int NI = 3, bool RAMP = false>
int launch_wave96(hipStream_t stream, SgemmParams p) {
  constexpr int BM = 32 * WGM, BN = 32 * NI;
  constexpr size_t ring = (size_t)KSPLIT * STAGES * (BM + BN) * BK * 4;
  constexpr size_t red = KSPLIT > 1 ? (size_t)KSPLIT * WGM * 16 * NI * 64 * 4 : 0;
  constexpr size_t lds = ring > red ? ring : red;
  static_assert(lds <= 160 * 1024, "LDS budget");
  if (!sgemm_detail::set_tiles(p, BM, BN)) return set_error(TFCC_ROCM_INVALID_ARGUMENT, "sgemm: too many tiles");
  const bool sameStart = p.batch == 1 || (p.strideA == 0 && p.innerA == 0 && p.strideB == 0 && p.innerB == 0);
  const bool plain = p.groups ? p.groups <= 3 : sameStart;
  TFCC_REQUIRE(p.batch < (1u << 30), "sgemm: batch of %u", p.batch);
  auto kern = plain ? sgemm_wave96_kernel<WGM, KSPLIT, BK, STAGES, true, NI, RAMP>
                    : sgemm_wave96_kernel<WGM, KSPLIT, BK, STAGES, false, NI, RAMP>;
  static bool attrSet[16][2] = {};  // per device: the attribute belongs to the function on one device
  int dev = 0;
  TFCC_HIP_CHECK(hipGetDevice(&dev));
  TFCC_REQUIRE(dev >= 0 && dev < 16, "device index %d", dev);
  if (!attrSet[dev][plain]) {
    TFCC_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attrSet[dev][plain] = true;
  }
  const unsigned hotBatch = p.batch | (p.groups ? 1u << 30 : 0u);
  hipLaunchKernelGGL(kern, dim3(p.chunk * 8), dim3(64 * WGM * KSPLIT), lds, stream, p.A, p.groups ? p.groupB[0] : p.B,
                     p.groups ? p.groupB[1] : nullptr, p.groups ? p.groupB[2] : nullptr, (unsigned)p.M, (unsigned)p.N,
                     (unsigned)p.K, (unsigned)p.lda, (unsigned)p.ldb, hotBatch, p);
  return check_launch("sgemm");
}

}  // namespace

namespace sgemm_detail {

int sgemm_wave96_launch(hipStream_t stream, SgemmParams p, int ksplit, int blocks, int rowBlocks) {
  if (ksplit == 4 && rowBlocks == 2 && blocks == 2) return launch_wave96<2, 4, 16, 2, 2>(stream, p);  // 64 x 64, eight wavefronts
  if (ksplit == 2) {
    // two K groups: two wavefronts on a 32-row tile, or two pairs of wavefronts on a 64 x 64 tile
    if (rowBlocks == 2 && blocks == 2) return launch_wave96<2, 2, 16, 2, 2>(stream, p);
    if (rowBlocks == 1 && blocks == 1) return launch_wave96<1, 2, 8, 3, 1>(stream, p);
  }
  if (rowBlocks != 0 && rowBlocks != (ksplit == 1 ? 4 : 1))
    return set_error(TFCC_ROCM_INVALID_ARGUMENT, "sgemm: no wavefront kernel for %d K groups and %d row blocks", ksplit, rowBlocks);
  if (ksplit == 4) {
    // Three or more tiles per CU: rings of three slabs of 8 k (12 KB per wavefront with 96 columns) let three
    // workgroups share a CU, so that all of a CU's tiles overlap.  Fewer: two slabs of 16 k, which leave a slab's
    // copies twice the time to land.  (With 32 columns a slab of 16 k would be more copies than a step has slots.)
    const unsigned long long tiles =
        (unsigned long long)((p.M + 31) / 32) * ((p.N + 32 * blocks - 1) / (32 * blocks)) * p.batch;
    if (blocks == 3) return tiles > 512 ? launch_wave96<1, 4, 8, 3, 3>(stream, p) : launch_wave96<1, 4, 16, 2, 3>(stream, p);
    // 64 columns, at most one tile per CU (128 x 768 x 3072): a third slab in the ring.  Two leave a slab's copies
    // one slab of matrix ops (0.4 us) to land, less than a trip to HBM: 11.1 -> 9.8 us with operands that come from
    // HBM, 8.1 -> 8.3 us with operands in cache; four and six slabs ask for so much at once that the first slab
    // lands later (10.2, 11.1 us), and slabs of 8 k read A in 32-byte pieces (12.2 us).  No gain with 96 columns.
    // The third slab is asked for during slab 0's first step, not at the start (RAMP): 8.3 -> 8.1 us in cache, 9.8 ->
    // 9.75 from HBM.  (The same ring on 96 columns: no gain, 11.9 against 11.7 us for 1024 x 768 x 768 in cache.)
    if (blocks == 2)
      return tiles > 512 ? launch_wave96<1, 4, 8, 3, 2>(stream, p)
                         : tiles <= 256 ? launch_wave96<1, 4, 16, 3, 2, true>(stream, p) : launch_wave96<1, 4, 16, 2, 2>(stream, p);
    if (blocks == 1) return launch_wave96<1, 4, 8, 3, 1>(stream, p);
  }
  if (ksplit == 1 && blocks == 3) return launch_wave96<4, 1, 32, 2, 3>(stream, p);
  if (ksplit == 1 && blocks == 4) return launch_wave96<4, 1, 32, 2, 4>(stream, p);
  return set_error(TFCC_ROCM_INVALID_ARGUMENT, "sgemm: no wavefront kernel for %d K groups and %d column blocks", ksplit, blocks);
}

}  // namespace sgemm_detail
}  // namespace tfcc_rocm
