// fp32 matrix product for mid-sized shapes: one wavefront per SIMD, 32 x 96 outputs per wavefront.
//
// A product like 1024 x 3072 x 768 has about one tile per CU, so nothing overlaps a workgroup's stalls except its
// own instruction order.  The kernels of sgemm_dma.hip leave that order to the compiler, which sinks the LDS reads
// next to their matrix ops (fewer registers) and waits for each in turn; with one wavefront per SIMD that costs a
// fifth of the time.  Here the order is written down: a k step is twelve 32x32x2 matrix ops (4 k pairs x 3 column
// blocks, 64 cycles each), and the 13 LDS reads of the next step's operands and the step's share of the HBM -> LDS
// copies are dealt out over the issue slots between them, one step ahead, into a second set of registers.
//
// Two shapes of workgroup, four wavefronts each:
//   groups (WGM = 1, KSPLIT = 4)  a 32 x 96 tile, wavefront q sums the 32-k slabs q, q + 4, ... in a ring of its
//                                 own (two half slabs of 16 k, 16 KB per wavefront, so that two workgroups share a
//                                 CU and one's set-up and tile store run under the other's matrix ops; no barrier
//                                 in the loop); the four partial tiles meet in LDS and every wavefront finishes a
//                                 quarter of the tile.  This is the shape the dispatcher uses: 1024 x 768 x 3072
//                                 39.2 us against 45.9 for the twelve-wavefront kernel of sgemm_dma.hip, three
//                                 1024 x 768 x 768 products in one launch 33.4 against 39.9.
//   rows   (WGM = 4, KSPLIT = 1)  a 128 x 96 tile, wavefront w owns rows 32w..32w+31, the ring (slabs of 32 k:
//                                 A 128 x 32 + B 32 x 96) is shared, one barrier per slab.  Measured no faster than
//                                 the twelve-wavefront kernel on 1024 x 3072 x 768 (the tile store with its GELU is
//                                 not hidden by anything) and not dispatched.
// The arithmetic is that of sgemm_dma.hip instruction for instruction (k pairs (8kb + s, 8kb + 4 + s) in ascending
// kb, s; groups added in group order), so a product has the same bits whichever kernel the dispatcher picks for its
// number of K groups.  Replaces the same oneDNN calls (tfcc/mkl/interfaces/tfcc_mklblasinterface.cpp:41-67, 69-78,
// 87-118).  Taken for 16-byte aligned operands and strides, K a multiple of 32, B not transposed.
#include "common.hpp"
#include "lds_dma.hpp"
#include "sgemm_params.hpp"

namespace tfcc_rocm {

typedef float w96_v4f __attribute__((ext_vector_type(4)));
typedef float w96_v16f __attribute__((ext_vector_type(16)));
typedef lds_dma_v4i w96_v4i;

namespace {

using sgemm_detail::SgemmParams;

constexpr int BN96 = 96;

// 16-byte chunk c of A row `row` lies at chunk c ^ swizzle: rows of 128 bytes (32 k), 64 bytes (16 k), 32 bytes (8 k)
template <int BK>
__device__ __forceinline__ int a_row_swizzle(int row) {
  return BK == 32 ? (row >> 1) & 7 : BK == 16 ? (row >> 2) & 3 : (row >> 2) & 1;
}

template <int WGM, int KSPLIT, int BK, int STAGES>
__global__ __launch_bounds__(256) void sgemm_wave96_kernel(const SgemmParams p) {
  static_assert(WGM * KSPLIT == 4, "four wavefronts");
  static_assert(BK == 32 || BK == 16 || BK == 8, "ring slabs of 32, 16 or 8 k");
  static_assert(STAGES >= 2, "ring depth");
  constexpr int BM = 32 * WGM;
  constexpr int KS = BK / 8;        // k steps per ring slab
  constexpr int CH = BK / 4;        // 16-byte chunks per A row
  constexpr int SUB = 32 / BK;      // ring slabs per 32-k slab of the product
  constexpr int A_BYTES = BM * BK * 4, B_BYTES = BK * BN96 * 4, STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int A_UNITS = A_BYTES / 1024, UNITS = STAGE_BYTES / 1024;  // 1 KB copies per ring slab
  static_assert(UNITS % WGM == 0, "every wavefront of a group issues the same number of copies");
  constexpr int COPIES = UNITS / WGM;
  static_assert(COPIES <= 11 && COPIES * STAGES < 64, "copies fit the slots of one step and the vmcnt range");
  constexpr int GROUP_BYTES = STAGES * STAGE_BYTES;
  constexpr int BCH = BN96 / 4;     // 16-byte chunks per B row
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
    const unsigned L = xcd * p.chunk + slot;
    if (slot >= p.chunk || L >= p.tilesTotal) return;
    const unsigned perBatch = p.tilesM * p.tilesN;
    bi = L / perBatch;
    unsigned t = L - bi * perBatch;
    const unsigned band = 4u * p.tilesN;
    unsigned gb = t / band;
    unsigned rowsInBand = min(4u, p.tilesM - gb * 4u);
    unsigned r = t - gb * band;
    tm = gb * 4u + r % rowsInBand;
    tn = r / rowsInBand;
  }
  const unsigned m0 = tm * BM, n0 = tn * BN96;
  const unsigned M = p.M, N = p.N, K = p.K;
  const unsigned bo = bi / p.batchInner, bn = bi - bo * p.batchInner;
  const float* A = p.A + (size_t)bo * p.strideA + (size_t)bn * p.innerA;
  const float* B = p.B + (size_t)bo * p.strideB + (size_t)bn * p.innerB;
  const float* biasPtr = p.bias;
  float* Cbase = p.C + (size_t)bo * p.strideC + (size_t)bn * p.innerC;
  if (p.groups) {  // selects, not indexing: the argument block stays in scalar registers
    B = bi == 0 ? p.groupB[0] : bi == 1 ? p.groupB[1] : bi == 2 ? p.groupB[2] : p.groupB[3];
    biasPtr = bi == 0 ? p.groupBias[0] : bi == 1 ? p.groupBias[1] : bi == 2 ? p.groupBias[2] : p.groupBias[3];
    Cbase = bi == 0 ? p.groupC[0] : bi == 1 ? p.groupC[1] : bi == 2 ? p.groupC[2] : p.groupC[3];
  }
  const unsigned lda = p.lda, ldb = p.ldb, ldc = p.ldc;
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
      const int s = (u - A_UNITS) * 64 + lane, k = s / BCH, ch = s % BCH;
      off[c] = (k * ldb + n0 + ch * 4) * 4u;
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

  // the first slabs are on their way before anything else is set up
#pragma unroll
  for (int s = 0; s < STAGES; ++s)
#pragma unroll
    for (int c = 0; c < COPIES; ++c) issueCopy((unsigned)s, (unsigned)s, c);

  // ---- values needed only in the tile store are fetched now.  Rows: lane (lrow, g) stores, for register r of
  // column block j, row 8*(r/4) + 4*g + r%4 of its wavefront's 32 and column 32*j + lrow.  Groups: after the
  // partial tiles met in LDS, wavefront w finishes registers 12w .. 12w+11 of the 48 (j = idx / 16, r = idx % 16).
  constexpr int OWN = KSPLIT == 1 ? 48 : 12;
  const int firstIdx = KSPLIT == 1 ? 0 : 12 * grp;
  const unsigned gcol0 = n0 + lrow;
  float bv[3];
#pragma unroll
  for (int j = 0; j < 3; ++j) bv[j] = (biasPtr && gcol0 + 32 * j < N) ? biasPtr[gcol0 + 32 * j] : 0.f;
  float rv[OWN];
  const float* Rp = p.residual ? p.residual + (size_t)bi * p.strideR : nullptr;  // dense, flat batch
  if (Rp) {
#pragma unroll
    for (int q = 0; q < OWN; ++q) {
      const int idx = firstIdx + q, j = idx >> 4, r = idx & 15;
      const unsigned grow = m0 + wm * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
      const unsigned gc = gcol0 + 32 * j;
      rv[q] = (grow < M && gc < N) ? Rp[(size_t)grow * N + gc] : 0.f;
    }
  }

  w96_v16f acc[3];
#pragma unroll
  for (int j = 0; j < 3; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;

  // ---- operand addresses inside a stage: A row wm*32 + lrow, logical chunk 2*kb + g; B column 32*j + lrow,
  // k rows 8*kb + 4*g + s
  const int arow = wm * 32 + lrow;
  const int aBase = arow * (BK * 4), aSwz = a_row_swizzle<BK>(arow);
  const int bBase = A_BYTES + (4 * g) * (BN96 * 4) + lrow * 4;
  struct Ops { w96_v4f a; float b[4][3]; };

  // One k step: twelve matrix ops on `cur`; in the issue slots between them the 13 reads of the operands of step
  // (ldStage, ldKb) into `nxt` and, in a slab's last step, the copies of the slab that takes its stage.
  auto step = [&](const Ops& cur, Ops& nxt, const unsigned char* ldStage, int ldKb, bool dma, unsigned dmaSlab,
                  unsigned dmaStage) {
#pragma unroll
    for (int m = 0; m < 12; ++m) {
      const int s = m / 3, j = m % 3;
      if (m == 0) nxt.a = *reinterpret_cast<const w96_v4f*>(ldStage + aBase + (((2 * ldKb + g) ^ aSwz) << 4));
      nxt.b[s][j] = *reinterpret_cast<const float*>(ldStage + bBase + (8 * ldKb + s) * (BN96 * 4) + j * 128);
      if (dma && m >= 1 && m <= COPIES) issueCopy(dmaSlab, dmaStage, m - 1);
      acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(cur.a[s], cur.b[s][j], acc[j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // ---- software pipeline.  At the start of slab t's last step: this wavefront's copies of slab t+1 have landed
  // and its reads of slab t have returned; with a shared ring a barrier makes that true of the whole group.  Then
  // slab t+1 is complete and visible, and slab t's stage is free: it is refilled with slab t+STAGES while the last
  // step's matrix ops run on operands already in registers.
  wait_vmcnt<COPIES*(STAGES - 1)>();
  if constexpr (SHARED) __syncthreads();
  Ops ops[2];
  ops[0].a = *reinterpret_cast<const w96_v4f*>(gsm + aBase + ((g ^ aSwz) << 4));
#pragma unroll
  for (int s = 0; s < 4; ++s)
#pragma unroll
    for (int j = 0; j < 3; ++j) ops[0].b[s][j] = *reinterpret_cast<const float*>(gsm + bBase + s * (BN96 * 4) + j * 128);
  // one ring slab: KS steps starting on the operands in `first`; the next slab's first operands end up in `first`
  // again when KS is even, in `other` when it is odd (then the loop below alternates the two)
  unsigned stage = 0;  // of slab t
  auto slab = [&](unsigned t, Ops& first, Ops& other) {
    const unsigned next = stage + 1 == STAGES ? 0 : stage + 1;
    const unsigned char* stCur = gsm + stage * STAGE_BYTES;
    const unsigned char* stNext = gsm + next * STAGE_BYTES;
#pragma unroll
    for (int kb = 0; kb < KS - 1; ++kb) step(kb & 1 ? other : first, kb & 1 ? first : other, stCur, kb + 1, false, 0u, 0u);
    wait_vmcnt<COPIES*(STAGES - 2)>();
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the reads of slab t have returned
    if constexpr (SHARED) __syncthreads();
    step((KS - 1) & 1 ? other : first, (KS - 1) & 1 ? first : other, stNext, 0, true, t + STAGES, stage);
    stage = next;
  };
  if constexpr (KS & 1) {
    for (unsigned t = 0; t < T; t += 2) {  // T is a multiple of 32 / BK >= 2
      slab(t, ops[0], ops[1]);
      slab(t + 1, ops[1], ops[0]);
    }
  } else {
    for (unsigned t = 0; t < T; ++t) slab(t, ops[0], ops[1]);
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
#pragma unroll
    for (int j = 0; j < 3; ++j) {
      const unsigned gc = gcol0 + 32 * j;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const unsigned grow = m0 + wm * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
        if (grow < M && gc < N) Cbase[(size_t)grow * ldc + gc] = finish(acc[j][r], j * 16 + r, j);
      }
    }
  } else {
    // the four partial tiles go through LDS (the rings are idle now), four registers per 128-bit access: registers
    // 4c .. 4c+3 of group q lie at red4[(q * 12 + c) * 64 + lane]; wavefront w adds the four of its twelve registers
    // (quads 3w .. 3w+2) in group order
    w96_v4f* red4 = reinterpret_cast<w96_v4f*>(smem);
#pragma unroll
    for (int j = 0; j < 3; ++j)
#pragma unroll
      for (int c = 0; c < 4; ++c)
        red4[(grp * 12 + j * 4 + c) * 64 + lane] = w96_v4f{acc[j][4 * c], acc[j][4 * c + 1], acc[j][4 * c + 2], acc[j][4 * c + 3]};
    __syncthreads();
    float sums[12];
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      w96_v4f v = red4[(3 * grp + c) * 64 + lane];
#pragma unroll
      for (int o = 1; o < KSPLIT; ++o) {
        const w96_v4f w = red4[(o * 12 + 3 * grp + c) * 64 + lane];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += w[e];
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) sums[4 * c + e] = v[e];
    }
#pragma unroll
    for (int q = 0; q < 12; ++q) {
      const int idx = firstIdx + q, j = idx >> 4, r = idx & 15;
      const float v = sums[q];
      const unsigned grow = m0 + 8 * (r >> 2) + 4 * g + (r & 3);
      const unsigned gc = gcol0 + 32 * j;
      // bv is indexed by a wave-uniform j: selects keep it in registers
      const float b = j == 0 ? bv[0] : j == 1 ? bv[1] : bv[2];
      float out = v + b;
      if (Rp) out += rv[q];
      if (act == 1) out = gelu_erf_f32(out);
      if (grow < M && gc < N) {
        if (p.lnGamma) {
          // read back by another workgroup, possibly on another XCD, later in this launch: written through to
          // device scope (the L2 caches of the XCDs do not see each other's plain stores before the launch ends)
          __hip_atomic_store(p.lnSums + (size_t)grow * N + gc, out, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
          Cbase[(size_t)grow * ldc + gc] = out;
        }
      }
    }
    if (p.lnGamma) {
      // ---- layer normalisation of the band's 32 rows by whichever of its workgroups stores its tile last.
      // Every store above has been acknowledged at device scope before this wavefront reaches the barrier, and
      // the band's counter is incremented after the barrier: the workgroup that reads tilesN - 1 from it sees all
      // tiles of the band complete.  It resets the counter, so that the next launch finds zeros.
      wait_vmcnt<0>();
      __syncthreads();
      unsigned* flag = reinterpret_cast<unsigned*>(smem);
      if (threadIdx.x == 0) {
        unsigned* counter = p.lnCounters + tm;
        const unsigned before = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const bool last = before == p.tilesN - 1;
        if (last) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *flag = last ? 1u : 0u;
      }
      __syncthreads();
      if (*flag == 0u) return;
      // One wavefront per row, eight rows each.  The stand-alone kernel (layer_norm_reg_kernel in elementwise.hip)
      // gives a row to 256 threads: thread t holds columns t, t + 256, ..., adds them in that order, the four
      // wavefronts reduce by butterfly and their sums are added in wavefront order.  Lane l plays threads l,
      // l + 64, l + 128, l + 192 of that kernel with the same additions in the same order: the same bits.
      constexpr int PER = (int)(sgemm_detail::kLayerNormMaxColumns / 256);
      float gm[4][PER], bt[4][PER];
#pragma unroll
      for (int w = 0; w < 4; ++w)
#pragma unroll
        for (int q = 0; q < PER; ++q) {
          const unsigned c = lane + 64 * w + 256 * q;
          gm[w][q] = c < N ? p.lnGamma[c] : 0.f;
          bt[w][q] = c < N ? p.lnBeta[c] : 0.f;
        }
      const float eps = p.lnEps;
      // four rows at a time: their 64 loads are all under way before the first is waited for (one row after the
      // other the tail costs a memory round trip per row)
      for (int u0 = 0; u0 < 8; u0 += 4) {
        float x[4][4][PER];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const unsigned row = m0 + 8 * wv + u0 + u;
          const float* src = p.lnSums + (size_t)row * N;
#pragma unroll
          for (int w = 0; w < 4; ++w)
#pragma unroll
            for (int q = 0; q < PER; ++q) {
              const unsigned c = lane + 64 * w + 256 * q;
              x[u][w][q] = (row < M && c < N) ? __hip_atomic_load(src + c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0.f;
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const unsigned row = m0 + 8 * wv + u0 + u;
          if (row >= M) break;  // wave-uniform
          float S[4];
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            float t = 0.f;
#pragma unroll
            for (int q = 0; q < PER; ++q)
              if (lane + 64 * w + 256 * q < N) t += x[u][w][q];
            S[w] = wave_sum(t);
          }
          const float mean = (((S[0] + S[1]) + S[2]) + S[3]) / (float)N;
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            float t = 0.f;
#pragma unroll
            for (int q = 0; q < PER; ++q)
              if (lane + 64 * w + 256 * q < N) {
                const float d = x[u][w][q] - mean;
                t += d * d;
              }
            S[w] = wave_sum(t);
          }
          const float var = (((S[0] + S[1]) + S[2]) + S[3]) / (float)N;
          const float inv = 1.0f / sqrtf(var + eps);
          float* dst = Cbase + (size_t)row * ldc;
#pragma unroll
          for (int w = 0; w < 4; ++w)
#pragma unroll
            for (int q = 0; q < PER; ++q) {
              const unsigned c = lane + 64 * w + 256 * q;
              if (c < N) dst[c] = (x[u][w][q] - mean) * (inv * gm[w][q]) + bt[w][q];
            }
        }
      }
    }
  }
}

template <int WGM, int KSPLIT, int BK, int STAGES>
int launch_wave96(hipStream_t stream, SgemmParams p) {
  constexpr int BM = 32 * WGM;
  constexpr size_t ring = (size_t)KSPLIT * STAGES * (BM + BN96) * BK * 4;
  constexpr size_t red = KSPLIT > 1 ? (size_t)KSPLIT * 48 * 64 * 4 : 0;
  constexpr size_t lds = ring > red ? ring : red;
  static_assert(lds <= 160 * 1024, "LDS budget");
  if (!sgemm_detail::set_tiles(p, BM, BN96)) return set_error(TFCC_ROCM_INVALID_ARGUMENT, "sgemm: too many tiles");
  auto kern = sgemm_wave96_kernel<WGM, KSPLIT, BK, STAGES>;
  static bool attrSet[16] = {};  // per device: the attribute belongs to the function on one device
  int dev = 0;
  TFCC_HIP_CHECK(hipGetDevice(&dev));
  TFCC_REQUIRE(dev >= 0 && dev < 16, "device index %d", dev);
  if (!attrSet[dev]) {
    TFCC_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attrSet[dev] = true;
  }
  hipLaunchKernelGGL(kern, dim3(p.chunk * 8), dim3(256), lds, stream, p);
  return check_launch("sgemm");
}

}  // namespace

namespace sgemm_detail {

int sgemm_wave96_launch(hipStream_t stream, SgemmParams p, int ksplit) {
  if (ksplit == 4) {
    // Three or more tiles per CU: rings of three slabs of 8 k (12 KB per wavefront) let three workgroups share a CU,
    // so that all of a CU's tiles overlap (three 1024 x 768 x 768 products in one launch: 33.9 us -> see below).
    // Fewer: two slabs of 16 k, which leave a slab's copies twice the time to land.
    const unsigned long long tiles = (unsigned long long)((p.M + 31) / 32) * ((p.N + BN96 - 1) / BN96) * p.batch;
    if (tiles > 512) return launch_wave96<1, 4, 8, 3>(stream, p);
    return launch_wave96<1, 4, 16, 2>(stream, p);
  }
  return set_error(TFCC_ROCM_INVALID_ARGUMENT, "sgemm: no 32 x 96 wavefront kernel for %d K groups", ksplit);
}

}  // namespace sgemm_detail
}  // namespace tfcc_rocm
