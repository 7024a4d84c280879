// fp32 matrix product for the small-tile configurations with the K slabs copied HBM -> LDS by the
// asynchronous buffer_load ... lds path instead of through registers.
//
// Same arithmetic as sgemm_kernel in sgemm.hip, instruction for instruction: 32x32x2 fp32 matrix ops
// over ascending k into one accumulator per element, K groups added in group order, bias / residual /
// GELU in the tile store - a product gives the same bits whichever of the two kernels runs it.  It
// replaces the same oneDNN calls (tfcc/mkl/interfaces/tfcc_mklblasinterface.cpp:41-67, 69-78, 87-118).
//
// What differs is how a slab of 32 k gets into LDS.  Every wavefront issues whole 1 KB copies (64
// lanes x 16 bytes, written to LDS in lane order): the A image is As[row][32] with its 16-byte chunks
// xor-swizzled (the lane picks the global chunk that belongs at its LDS position), the B image is the
// slab as it lies in memory, Bs[k][BN].  No registers, no LDS store instructions, no transposition:
// a lane reads the four B operands of a step as four 32-bit words of one column.  A ring of STAGES
// slabs per K group is kept in flight; one barrier per slab, placed before the slab's last step so
// that the freed stage is refilled while that step's matrix ops run.
//
// Taken only for 16-byte aligned operands and strides, K a multiple of 32 (a partial slab of A
// cannot be zeroed on its way into LDS) and B not transposed.
#include "common.hpp"
#include "lds_dma.hpp"
#include "sgemm_params.hpp"

namespace tfcc_rocm {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef lds_dma_v4i v4i;

namespace {

using sgemm_detail::SgemmParams;

constexpr int BK = 32;       // floats of k per slab: a row piece of A is one 128-byte memory line
constexpr int KS = BK / 8;   // steps of 8 k (four matrix ops) per slab
constexpr unsigned kPastEnd = 0xfffffff0u;  // a byte offset past the end of any operand: the copy writes zeros

__device__ __forceinline__ int row_swizzle(int row) { return (row >> 1) & 7; }

// WGM x WGN wavefronts, each owning a 32 x (32 * NI) block (a lane owns NI consecutive columns); KSPLIT
// groups of them on the same tile, group q walking the slabs q, q + KSPLIT, ... through a ring of its own.
// VSPLIT > 1 (with KSPLIT == 1): one group does the work of VSPLIT groups one slab after the other, with an
// accumulator per would-be group (slab s goes to accumulator s % VSPLIT) and the same final additions in
// group order - bit for bit the result of KSPLIT = VSPLIT, for launches that fill the chip without
// splitting K across wavefronts (several products in one launch).
template <int WGM, int WGN, int NI, int KSPLIT, int STAGES, int VSPLIT = 1>
__global__ __launch_bounds__(WGM * WGN * 64 * KSPLIT) void sgemm_dma_kernel(const SgemmParams p) {
  static_assert(VSPLIT == 1 || KSPLIT == 1, "accumulators per would-be group only without real groups");
  static_assert(NI == 1 || NI == 3 || NI == 4, "a lane reads its B operands as one word, three words 32 columns apart or four consecutive words");
  constexpr bool STRIDED = NI == 3;  // lane lrow owns columns lrow, lrow + 32, lrow + 64 of the wavefront's block
  constexpr int GW = WGM * WGN;
  constexpr bool PRIVATE_RING = GW == 1;  // one wavefront per group: nobody else reads or fills its ring
  constexpr int WN = 32 * NI;
  constexpr int BM = WGM * 32, BN = WGN * WN;
  constexpr int A_BYTES = BM * BK * 4, B_BYTES = BK * BN * 4, STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int A_UNITS = A_BYTES / 1024, UNITS = STAGE_BYTES / 1024;  // 1 KB copies per slab
  constexpr int COPIES = (UNITS + GW - 1) / GW;                        // per wavefront per slab
  constexpr bool SPARE = COPIES * GW != UNITS;  // some wavefronts issue one copy more than there is to do:
                                                // it reads past the end (zeros) into a spare 1 KB
  constexpr int GROUP_BYTES = STAGES * STAGE_BYTES + (SPARE ? 1024 : 0);
  constexpr int BCH = BN / 4;  // 16-byte chunks per B row
  static_assert(COPIES * STAGES < 64, "vmcnt range");
  static_assert(STAGES >= 2 && KS % 2 == 0, "ring depth; the operand registers alternate per step");

  extern __shared__ __align__(16) unsigned char smem[];
  const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int grp = wv / GW, wave = wv - grp * GW;  // wave-uniform
  const int lane = threadIdx.x & 63;
  const int wm = wave / WGN, wn = wave % WGN;
  unsigned char* gsm = smem + grp * GROUP_BYTES;
  const unsigned ldsGroup = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)gsm;

  // A launch of these kernels is a few microseconds, so what stands in front of its first copies counts: everything
  // they need of the argument block is named before the first branch (one round trip to memory instead of one per
  // basic block), and the divisions of the tile mapping are multiplications by constants the launcher worked out.
  asm volatile("" ::"s"(p.chunk), "s"(p.tilesTotal), "s"(p.tilesM), "s"(p.tilesN), "s"(p.perBatchMagic),
               "s"(p.perBatchShift), "s"(p.bandMagic), "s"(p.bandShift), "s"(p.innerMagic), "s"(p.innerShift),
               "s"(p.batchInner), "s"(p.M), "s"(p.N), "s"(p.K), "s"(p.lda), "s"(p.ldb), "s"(p.groups), "s"(p.A), "s"(p.B),
               "s"(p.strideA), "s"(p.strideB), "s"(p.innerA), "s"(p.innerB), "s"(p.groupB[0]), "s"(p.groupB[1]), "s"(p.groupB[2]),
               "s"(p.groupB[3]));
  unsigned tm, tn, bi;
  {
    // consecutive workgroup ids land on different XCDs: hand each XCD a contiguous run of tiles
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
  const unsigned bo = udiv_apply(bi, p.innerMagic, p.innerShift), bn = bi - bo * p.batchInner;
  const float* A = p.A + (size_t)bo * p.strideA + (size_t)bn * p.innerA;
  const float* B = p.B + (size_t)bo * p.strideB + (size_t)bn * p.innerB;
  if (p.groups)  // selects, not indexing: the argument block stays in scalar registers
    B = bi == 0 ? p.groupB[0] : bi == 1 ? p.groupB[1] : bi == 2 ? p.groupB[2] : p.groupB[3];
  const unsigned lda = p.lda, ldb = p.ldb;
  const v4i rsrcA = make_rsrc(A, ((M - 1) * lda + K) * 4u);
  const v4i rsrcB = make_rsrc(B, ((K - 1) * ldb + N) * 4u);

  const int lrow = lane & 31, g = lane >> 5;

  // ---- copy descriptors.  Copy c of a slab is unit u = c * GW + wave of the stage image; LDS slot s
  // (16 bytes) of the A image holds row s / 8, physical chunk s % 8 = logical chunk ^ row_swizzle(row);
  // slot s of the B image holds k row s / BCH, chunk s % BCH.
  unsigned off[COPIES];  // this lane's byte offset into A or B for k = 0
#pragma unroll
  for (int c = 0; c < COPIES; ++c) {
    const int u = c * GW + wave;
    if (u < A_UNITS) {
      const int s = u * 64 + lane, row = s >> 3, phys = s & 7;
      off[c] = ((m0 + row) * lda + ((phys ^ row_swizzle(row)) << 2)) * 4u;
    } else if (u < UNITS) {
      const int s = (u - A_UNITS) * 64 + lane, k = s / BCH, ch = s % BCH;
      off[c] = (k * ldb + n0 + ch * 4) * 4u;
    } else {
      off[c] = kPastEnd;
    }
  }
  // slab `slab` of this group = slab slab * KSPLIT + grp of the product; one past the end of K copies zeros
  auto issueSlab = [&](unsigned slab) {
    const unsigned stage = slab % STAGES;
    const unsigned k0 = (slab * KSPLIT + grp) * BK;
    const bool live = k0 < K;
#pragma unroll
    for (int c = 0; c < COPIES; ++c) {
      const int u = c * GW + wave;
      const bool isA = u < A_UNITS, spare = u >= UNITS;
      const unsigned dst = __builtin_amdgcn_readfirstlane(
          ldsGroup + (spare ? STAGES * STAGE_BYTES : stage * STAGE_BYTES + u * 1024));
      const unsigned src = (live && !spare) ? off[c] + (isA ? k0 * 4u : k0 * ldb * 4u) : kPastEnd;
      dma16(isA ? rsrcA : rsrcB, dst, src);
    }
  };

  v16f accs[VSPLIT][NI];
#pragma unroll
  for (int v = 0; v < VSPLIT; ++v)
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) accs[v][j][r] = 0.f;

  // ---- operand addresses inside a stage: A row wm*32 + lrow, logical chunk 2*kb + g; B columns
  // wn*WN + NI*lrow .. + NI-1, k rows 8*kb + 4*g + s
  struct BOps { float v[4][NI]; };  // [s][j]
  const int arow = wm * 32 + lrow;
  const int aBase = arow * (BK * 4), aSwz = row_swizzle(arow);
  const int bBase = A_BYTES + (4 * g) * (BN * 4) + (wn * WN + (STRIDED ? lrow : NI * lrow)) * 4;
  auto readOps = [&](unsigned stage, int kb, v4f& a, BOps& b) {
    const unsigned char* st = gsm + stage * STAGE_BYTES;
    a = *reinterpret_cast<const v4f*>(st + aBase + (((2 * kb + g) ^ aSwz) << 4));
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      if constexpr (NI == 4) {
        const v4f w = *reinterpret_cast<const v4f*>(st + bBase + (8 * kb + s) * (BN * 4));
#pragma unroll
        for (int j = 0; j < 4; ++j) b.v[s][j] = w[j];
      } else {
#pragma unroll
        for (int j = 0; j < NI; ++j)
          b.v[s][j] = *reinterpret_cast<const float*>(st + bBase + (8 * kb + s) * (BN * 4) + j * 128);
      }
    }
  };
  auto mma = [&](v16f (&acc)[NI], const v4f& a, const BOps& b) {
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
      for (int j = 0; j < NI; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], b.v[s][j], acc[j], 0, 0, 0);
  };

  // ---- software pipeline.  Before the barrier of slab kt: this wavefront's copies of slab kt+1 have
  // landed and its reads of slab kt are done.  After it: slab kt+1 is complete and visible, the stage of
  // slab kt is free and is refilled with slab kt+STAGES while the last step of slab kt runs on operands
  // already in registers.  Every group makes the same number of steps (the barriers are workgroup-wide).
  const unsigned KT = ((K + BK - 1) / BK + KSPLIT - 1) / KSPLIT;
#pragma unroll
  for (int s = 0; s < STAGES; ++s) issueSlab(s);
  // (what the tile store needs of the argument block is read from here on, not in front of the copies)
  const unsigned ldc = p.ldc;
  const float* biasPtr = p.bias;
  float* Cbase = p.C + (size_t)bo * p.strideC + (size_t)bn * p.innerC;
  if (p.groups) {
    biasPtr = bi == 0 ? p.groupBias[0] : bi == 1 ? p.groupBias[1] : bi == 2 ? p.groupBias[2] : p.groupBias[3];
    Cbase = bi == 0 ? p.groupC[0] : bi == 1 ? p.groupC[1] : bi == 2 ? p.groupC[2] : p.groupC[3];
  }
  // values needed only in the tile store are fetched now, behind the first slabs: at the end their latency would be
  // waited for in full (memory operations return in the order they were issued, so the wait below also covers the
  // part of slab 1 that was asked for before these)
  const unsigned gcol = n0 + wn * WN + (STRIDED ? lrow : NI * lrow);  // first of this lane's NI columns
  constexpr unsigned CSTEP = STRIDED ? 32 : 1;                          // from one of them to the next
  float bv[NI];
#pragma unroll
  for (int j = 0; j < NI; ++j) bv[j] = (biasPtr && gcol + j * CSTEP < N) ? biasPtr[gcol + j * CSTEP] : 0.f;
  constexpr bool EARLY_RESIDUAL = NI != 4;  // short launches on small tiles; a large tile fetches it in the store
  float rv[EARLY_RESIDUAL ? 16 * NI : 1];
  if constexpr (EARLY_RESIDUAL) {
    if (p.residual && grp == 0) {
      const float* Rp = p.residual + (size_t)bi * p.strideR;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const unsigned grow = m0 + wm * 32 + 8 * (r / 4) + 4 * g + (r & 3);
#pragma unroll
        for (int j = 0; j < NI; ++j)
          rv[r * NI + j] = (grow < M && gcol + j * CSTEP < N) ? Rp[(size_t)grow * N + gcol + j * CSTEP] : 0.f;
      }
    }
  }

  wait_vmcnt<COPIES*(STAGES - 1)>();
  if constexpr (!PRIVATE_RING) __syncthreads();
  v4f fa[2];
  BOps fb[2];
  readOps(0, 0, fa[0], fb[0]);
  for (unsigned ko = 0; ko < (KT + VSPLIT - 1) / VSPLIT; ++ko) {
#pragma unroll
    for (int v = 0; v < VSPLIT; ++v) {  // a slab past the end of K is all zeros
      const unsigned kt = ko * VSPLIT + v;
      const unsigned cur = kt % STAGES, nxt = (kt + 1) % STAGES;
#pragma unroll
      for (int kb = 0; kb < KS - 1; ++kb) {
        readOps(cur, kb + 1, fa[(kb + 1) & 1], fb[(kb + 1) & 1]);
        mma(accs[v], fa[kb & 1], fb[kb & 1]);
      }
      wait_vmcnt<COPIES*(STAGES - 2)>();
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the reads of slab kt have returned
      if constexpr (!PRIVATE_RING) __syncthreads();
      readOps(nxt, 0, fa[0], fb[0]);
      issueSlab(kt + STAGES);
      mma(accs[v], fa[(KS - 1) & 1], fb[(KS - 1) & 1]);
    }
  }
  wait_vmcnt<0>();
  __syncthreads();

  v16f acc[NI];
#pragma unroll
  for (int j = 0; j < NI; ++j) {
    acc[j] = accs[0][j];
#pragma unroll
    for (int v = 1; v < VSPLIT; ++v)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[j][r] += accs[v][j][r];
  }
  if constexpr (KSPLIT > 1) {
    // partial tiles of groups 1 .. KSPLIT-1 go through LDS (the rings are idle now) and are added by
    // group 0 in group order
    float* red = reinterpret_cast<float*>(smem);
    if (grp > 0) {
#pragma unroll
      for (int j = 0; j < NI; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) red[(((((grp - 1) * GW + wave) * NI + j) * 16 + r) * 64) + lane] = acc[j][r];
    }
    __syncthreads();
    if (grp > 0) return;
#pragma unroll
    for (int q = 1; q < KSPLIT; ++q)
#pragma unroll
      for (int j = 0; j < NI; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] += red[(((((q - 1) * GW + wave) * NI + j) * 16 + r) * 64) + lane];
  }

  // ---- tile store: + bias, + residual, GELU.  Lane (lrow, g) owns columns NI*lrow .. of the wavefront's
  // block and rows 8*(r/4) + 4*g + r%4.
  const float* R = p.residual ? p.residual + (size_t)bi * p.strideR : nullptr;  // dense, flat batch
  const int act = p.act;
  const bool residualByQuads = EARLY_RESIDUAL || !R || reinterpret_cast<uintptr_t>(R) % 16 == 0;
  if (m0 + wm * 32 + 32 <= M && n0 + wn * WN + WN <= N && ldc < (1u << 24) && residualByQuads) {
    // A whole 32 x WN block: no bounds to check, and the addresses are a register per lane (row 4g, the lane's first
    // column), a scalar per row and an immediate per column - no address arithmetic per value (vector instructions
    // are what a tile store costs: they do not run under another wavefront's fp32 matrix ops).
    const unsigned blockCol = n0 + wn * WN;
    const __amdgpu_buffer_rsrc_t rc =
        __builtin_amdgcn_make_buffer_rsrc(Cbase + (size_t)(m0 + wm * 32) * ldc + blockCol, 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t rr = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(R ? R + (size_t)(m0 + wm * 32) * N + blockCol : Cbase), 0, 0x7fffffff, 0x00020000);
    const unsigned laneCol = STRIDED ? lrow : NI * lrow;
    const unsigned voff = ((4 * g) * ldc + laneCol) * 4u, voffR = ((4 * g) * N + laneCol) * 4u;
    auto store = [&](bool gelu) __attribute__((always_inline)) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const unsigned rowInBlock = 8 * (r / 4) + (r & 3);
        float v[NI];
#pragma unroll
        for (int j = 0; j < NI; ++j) v[j] = acc[j][r] + bv[j];
        if (R) {
          if constexpr (EARLY_RESIDUAL) {
#pragma unroll
            for (int j = 0; j < NI; ++j) v[j] += rv[r * NI + j];
          } else {
            const v4f w = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rr, voffR, rowInBlock * N * 4u, 0));
#pragma unroll
            for (int j = 0; j < NI; ++j) v[j] += w[j];
          }
        }
        if (gelu) {
#pragma unroll
          for (int j = 0; j < NI; ++j) v[j] = gelu_erf_f32(v[j]);
        }
        if constexpr (NI == 4) {
          typedef unsigned v4u __attribute__((ext_vector_type(4)));
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, v4f{v[0], v[1], v[2], v[3]}), rc, voff,
                                                 rowInBlock * ldc * 4u, 0);
        } else {
#pragma unroll
          for (int j = 0; j < NI; ++j)
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v[j]), rc, voff + j * CSTEP * 4u,
                                                  rowInBlock * ldc * 4u, 0);
        }
      }
    };
    if (act == 1) store(true); else store(false);
    return;
  }
  if (gcol >= N) return;
  const bool whole = gcol + (NI - 1) * CSTEP < N;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const unsigned grow = m0 + wm * 32 + 8 * (r / 4) + 4 * g + (r & 3);
    if (grow >= M) continue;
    float v[NI];
#pragma unroll
    for (int j = 0; j < NI; ++j) v[j] = acc[j][r] + bv[j];
    if (R) {
      if constexpr (EARLY_RESIDUAL) {
#pragma unroll
        for (int j = 0; j < NI; ++j) v[j] += rv[r * NI + j];
      } else {
#pragma unroll
        for (int j = 0; j < NI; ++j)
          if (gcol + j * CSTEP < N) v[j] += R[(size_t)grow * N + gcol + j * CSTEP];
      }
    }
    // same expression as the stand-alone GELU kernel, so that fusing changes no bit
    if (act == 1) {
#pragma unroll
      for (int j = 0; j < NI; ++j) v[j] = gelu_erf_f32(v[j]);
    }
    float* dst = Cbase + (size_t)grow * ldc + gcol;
    if constexpr (NI == 4) {
      if (whole) {
        *reinterpret_cast<v4f*>(dst) = v4f{v[0], v[1], v[2], v[3]};
        continue;
      }
    }
#pragma unroll
    for (int j = 0; j < NI; ++j)
      if (gcol + j * CSTEP < N) dst[j * CSTEP] = v[j];
  }
}

template <int WGM, int WGN, int NI, int KSPLIT, int STAGES, int VSPLIT = 1>
int launch(hipStream_t stream, SgemmParams p) {
  constexpr int GW = WGM * WGN, BM = WGM * 32, BN = WGN * 32 * NI;
  constexpr int STAGE_BYTES = (BM + BN) * BK * 4, UNITS = STAGE_BYTES / 1024;
  constexpr int COPIES = (UNITS + GW - 1) / GW;
  constexpr size_t lds = (size_t)KSPLIT * (STAGES * STAGE_BYTES + (COPIES * GW != UNITS ? 1024 : 0));
  static_assert(lds <= 160 * 1024 && (size_t)(KSPLIT - 1) * BM * BN * sizeof(float) <= lds, "LDS budget");
  if (!sgemm_detail::set_tiles(p, BM, BN)) return set_error(TFCC_ROCM_INVALID_ARGUMENT, "sgemm: too many tiles");
  auto kern = sgemm_dma_kernel<WGM, WGN, NI, KSPLIT, STAGES, VSPLIT>;
  static bool attrSet[16] = {};  // per device: the attribute belongs to the function on one device
  int dev = 0;
  TFCC_HIP_CHECK(hipGetDevice(&dev));
  TFCC_REQUIRE(dev >= 0 && dev < 16, "device index %d", dev);
  if (!attrSet[dev]) {
    TFCC_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attrSet[dev] = true;
  }
  hipLaunchKernelGGL(kern, dim3(p.chunk * 8), dim3(GW * 64 * KSPLIT), lds, stream, p);
  return check_launch("sgemm");
}

}  // namespace

namespace sgemm_detail {

bool sgemm_dma_available(int config, int ksplit) {
  return (config >= 0 && config <= 3 && (ksplit == 1 || ksplit == 2)) || (config == 5 && ksplit == 2);
}

// Two stages everywhere: more workgroups per CU beat a deeper ring (measured 42.3 against 43.9 us with
// three stages, 1024 x 3072 x 768 in 64x64 tiles).
int sgemm_dma_launch(hipStream_t stream, SgemmParams p, int config, int ksplit, bool serialGroups) {
#define TFCC_DMA_CASE(C, WGM, WGN)                                                  \
  if (config == C) {                                                                \
    if (ksplit == 1) return launch<WGM, WGN, 1, 1, 2>(stream, p);                      \
    if (ksplit == 2 && serialGroups) return launch<WGM, WGN, 1, 1, 2, 2>(stream, p);   \
    if (ksplit == 2) return launch<WGM, WGN, 1, 2, 2>(stream, p);                      \
  }
  TFCC_DMA_CASE(0, 2, 2)  // 64 x 64
  TFCC_DMA_CASE(1, 1, 3)  // 32 x 96
  TFCC_DMA_CASE(2, 1, 2)  // 32 x 64
  TFCC_DMA_CASE(3, 1, 1)  // 32 x 32
#undef TFCC_DMA_CASE
  // 128 x 96, twelve wavefronts, one group doing the work of `ksplit` groups: four times the rows of A per copy of B
  if (config == 5 && ksplit == 2 && serialGroups) return launch<4, 3, 1, 1, 2, 2>(stream, p);
  return set_error(TFCC_ROCM_INVALID_ARGUMENT, "sgemm: no direct-to-LDS kernel for this configuration");
}

}  // namespace sgemm_detail
}  // namespace tfcc_rocm
