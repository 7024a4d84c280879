// fp32 strided-batched matrix product on the gfx950 fp32 matrix cores with the bias add fused
// into the tile store.
//
// Replaces the oneDNN calls of tfcc/mkl/interfaces/tfcc_mklblasinterface.cpp:41-67 (matmul) and
// :69-78,87-118 (bias pre-fill + accumulate), with the same argument meaning: row-major operands,
// batch strides in elements, stride 0 = operand shared by every batch.
//
// A workgroup of four wavefronts owns a BM x BN tile of one batch entry and walks K in slabs of
// BK = 32.  Both slabs are kept in LDS with k contiguous (As[row][k], Bs[col][k]) so that a lane
// fetches the operands of four v_mfma_f32_32x32x2_f32 steps with one 128-bit LDS read: lane
// (i, g) holds k = 8*kb + 4*g + s of row/column i for step s, for A and B alike.  B is row-major
// [K,N] in HBM: every thread loads a 4(k) x 4(n) block as four 128-bit rows, transposes it by
// register renaming and writes four 128-bit chunks.  16-byte chunks are xor-swizzled by the row
// index, and tile columns are stored interleaved (LDS row j*32+i holds tile column NI*i+j of the
// wavefront's column range) so that a lane owns NI consecutive output columns.
#include "common.hpp"
#include "sgemm_params.hpp"

namespace tfcc_rocm {

using sgemm_detail::SgemmParams;

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

namespace {

constexpr int BK = 32;
constexpr int CH = BK / 4;  // 16-byte chunks per LDS row

__device__ __forceinline__ int swz(int row, int chunk) { return chunk ^ ((row >> 1) & (CH - 1)); }

// WGM x WGN wavefronts, each owning an (MI*32) x (NI*32) sub-tile.  With KSPLIT > 1 the workgroup
// holds KSPLIT such groups of four wavefronts on the same tile: group q walks the K slabs q,
// q + KSPLIT, ... through LDS buffers of its own and the partial tiles are added up through LDS in
// a fixed order at the end.  That is for products with few tiles and a long K, where one group per
// CU could not hide the memory latency of its own loads.
// TRANSB: B is given as B^T, an [N, K] row-major matrix (k contiguous), and is staged like A.
template <int WGM, int WGN, int MI, int NI, bool VEC, int KSPLIT, bool TRANSB>
__global__ __launch_bounds__(WGM * WGN * 64 * KSPLIT) void sgemm_kernel(const SgemmParams p) {
  constexpr int GW = WGM * WGN;      // wavefronts per group
  constexpr int kThreads = GW * 64;  // threads per group
  static_assert(GW == 4 || GW == 3, "three or four wavefronts per group");
  constexpr int BM = WGM * MI * 32, BN = WGN * NI * 32;
  constexpr int WM = MI * 32, WN = NI * 32;
  constexpr int A_TOTAL = BM * CH;                              // 128-bit chunks of A
  constexpr int B_TOTAL = TRANSB ? BN * CH : (BN / 4) * CH;     // chunks of B^T, or 4x4 blocks of B
  constexpr int A_ITEMS = (A_TOTAL + kThreads - 1) / kThreads;  // per thread
  constexpr int B_ITEMS = (B_TOTAL + kThreads - 1) / kThreads;

  extern __shared__ __align__(16) float smemf[];
  const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int grp = wv / GW;  // K group, wave-uniform
  float* As = smemf + grp * 2 * (BM + BN) * BK;  // [2][BM][BK]
  float* Bs = As + 2 * BM * BK;                  // [2][BN][BK]

  const int tid = threadIdx.x - grp * kThreads, lane = tid & 63, wave = wv - grp * GW;
  const int wm = wave / WGN, wn = wave % WGN;

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
    unsigned g = t / band;
    unsigned rowsInBand = min(4u, p.tilesM - g * 4u);
    unsigned r = t - g * band;
    tm = g * 4u + r % rowsInBand;
    tn = r / rowsInBand;
  }
  const unsigned m0 = tm * BM, n0 = tn * BN;
  const unsigned M = p.M, N = p.N, K = p.K;
  const unsigned bo = bi / p.batchInner, bn = bi - bo * p.batchInner;
  const float* __restrict__ A = p.A + (size_t)bo * p.strideA + (size_t)bn * p.innerA;
  const float* __restrict__ B = p.B + (size_t)bo * p.strideB + (size_t)bn * p.innerB;
  const float* biasPtr = p.bias;
  float* Cbase = p.C + (size_t)bo * p.strideC + (size_t)bn * p.innerC;
  if (p.groups) {  // selects, not indexing: the argument block stays in scalar registers
    B = bi == 0 ? p.groupB[0] : bi == 1 ? p.groupB[1] : bi == 2 ? p.groupB[2] : p.groupB[3];
    biasPtr = bi == 0 ? p.groupBias[0] : bi == 1 ? p.groupBias[1] : bi == 2 ? p.groupBias[2] : p.groupBias[3];
    Cbase = bi == 0 ? p.groupC[0] : bi == 1 ? p.groupC[1] : bi == 2 ? p.groupC[2] : p.groupC[3];
  }
  const unsigned lda = p.lda, ldb = p.ldb, ldc = p.ldc;

  v16f acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // The residual values this lane adds in the store are fetched now, in the small-tile configurations where
  // the launch is short and a load issued at the end would be waited for in full.
  float bv[NI];  // bias of this lane's columns, fetched before the main loop for the same reason
  {
    const unsigned col0 = n0 + wn * WN + NI * (lane & 31);
#pragma unroll
    for (int j = 0; j < NI; ++j) bv[j] = (biasPtr && col0 + j < N) ? biasPtr[col0 + j] : 0.f;
  }
  constexpr bool EARLY_RESIDUAL = MI * NI * 16 <= 32;
  float rv[EARLY_RESIDUAL ? MI : 1][EARLY_RESIDUAL ? NI : 1][16];
  if constexpr (EARLY_RESIDUAL) {
    if (p.residual && grp == 0) {
      const float* Rp = p.residual + (size_t)bi * p.strideR;
      const unsigned col0 = n0 + wn * WN + NI * (lane & 31);
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const unsigned grow = m0 + wm * WM + i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r & 3);
#pragma unroll
          for (int j = 0; j < NI; ++j)
            rv[i][j][r] = (grow < M && col0 + j < N) ? Rp[(size_t)grow * N + col0 + j] : 0.f;
        }
    }
  }

  v4f aReg[A_ITEMS];
  v4f bReg[B_ITEMS][TRANSB ? 1 : 4];

  // Vector path: raw buffer loads, an offset past the end of the operand reads zero (rows >= M of
  // A, rows >= K of B).  The k tail of an A row is zeroed explicitly: it would otherwise meet the
  // zero rows of B as garbage that may be Inf/NaN.
  const __amdgpu_buffer_rsrc_t rsrcA =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(A), 0, VEC ? (int)(((M - 1) * lda + K) * 4u) : 0, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrcB = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(B), 0, VEC ? (int)((TRANSB ? (N - 1) * ldb + K : (K - 1) * ldb + N) * 4u) : 0, 0x00020000);

  auto loadA = [&](unsigned k0) {
#pragma unroll
    for (int it = 0; it < A_ITEMS; ++it) {
      const int w = tid + it * kThreads;
      if (A_TOTAL % kThreads != 0 && w >= A_TOTAL) break;
      const int row = w / CH, ch = w % CH;
      const unsigned gr = m0 + row, gk = k0 + ch * 4;
      v4f v = {0.f, 0.f, 0.f, 0.f};
      if constexpr (VEC) {
        // Only the slab that crosses the end of K masks its values: a select on every loaded value
        // would make the compiler wait for the load right here instead of after the matrix ops.
        v = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rsrcA, (gr * lda + gk) * 4u, 0, 0));
        if (k0 + BK > K) {
          asm volatile("" ::: "memory");  // keeps this a real (wave-uniform) branch
          v = gk < K ? v : v4f{0.f, 0.f, 0.f, 0.f};
        }
      } else {
        if (gr < M) {
#pragma unroll
          for (int q = 0; q < 4; ++q)
            if (gk + q < K) v[q] = A[(size_t)gr * lda + gk + q];
        }
      }
      aReg[it] = v;
    }
  };
  auto loadB = [&](unsigned k0) {
#pragma unroll
    for (int it = 0; it < B_ITEMS; ++it) {
      const int w = tid + it * kThreads;
      if (B_TOTAL % kThreads != 0 && w >= B_TOTAL) break;
      if constexpr (TRANSB) {
        const int row = w / CH, ch = w % CH;
        const unsigned gn = n0 + row, gk = k0 + ch * 4;
        v4f v = {0.f, 0.f, 0.f, 0.f};
        if constexpr (VEC) {
          v = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rsrcB, (gn * ldb + gk) * 4u, 0, 0));
          if (k0 + BK > K) {
            asm volatile("" ::: "memory");  // as for A: a real branch, taken by the last slab only
            v = gk < K ? v : v4f{0.f, 0.f, 0.f, 0.f};
          }
        } else {
          if (gn < N) {
#pragma unroll
            for (int q = 0; q < 4; ++q)
              if (gk + q < K) v[q] = B[(size_t)gn * ldb + gk + q];
          }
        }
        bReg[it][0] = v;
      } else {
        const int nq = w % (BN / 4), kq = w / (BN / 4);
        const unsigned gn = n0 + nq * 4, gk = k0 + kq * 4;
#pragma unroll
        for (int q = 0; q < (TRANSB ? 1 : 4); ++q) {
          v4f v = {0.f, 0.f, 0.f, 0.f};
          if constexpr (VEC) {
            v = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rsrcB, ((gk + q) * ldb + gn) * 4u, 0, 0));
          } else {
            if (gk + q < K) {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (gn + e < N) v[e] = B[(size_t)(gk + q) * ldb + gn + e];
            }
          }
          bReg[it][q] = v;
        }
      }
    }
  };
  auto storeTiles = [&](int buf) {
    float* as = As + buf * BM * BK;
    float* bs = Bs + buf * BN * BK;
#pragma unroll
    for (int it = 0; it < A_ITEMS; ++it) {
      const int w = tid + it * kThreads;
      if (A_TOTAL % kThreads != 0 && w >= A_TOTAL) break;
      const int row = w / CH, ch = w % CH;
      *reinterpret_cast<v4f*>(as + row * BK + swz(row, ch) * 4) = aReg[it];
    }
#pragma unroll
    for (int it = 0; it < B_ITEMS; ++it) {
      const int w = tid + it * kThreads;
      if (B_TOTAL % kThreads != 0 && w >= B_TOTAL) break;
      if constexpr (TRANSB) {
        const int n = w / CH, ch = w % CH;
        const int wnn = n / WN, within = n % WN;
        const int row = wnn * WN + (within % NI) * 32 + within / NI;
        *reinterpret_cast<v4f*>(bs + row * BK + swz(row, ch) * 4) = bReg[it][0];
      } else {
        const int nq = w % (BN / 4), kq = w / (BN / 4);
#pragma unroll
        for (int j = 0; j < (TRANSB ? 1 : 4); ++j) {
          const int n = nq * 4 + j;
          const int wnn = n / WN, within = n % WN;
          const int row = wnn * WN + (within % NI) * 32 + within / NI;
          v4f v = {bReg[it][0][j], bReg[it][TRANSB ? 0 : 1][j], bReg[it][TRANSB ? 0 : 2][j], bReg[it][TRANSB ? 0 : 3][j]};
          *reinterpret_cast<v4f*>(bs + row * BK + swz(row, kq) * 4) = v;
        }
      }
    }
  };

  // every group makes the same number of steps (the barriers are workgroup-wide); a slab past the
  // end of K loads zeros
  const unsigned KT = ((K + BK - 1) / BK + KSPLIT - 1) / KSPLIT;
  loadA(grp * BK);
  loadB(grp * BK);
  storeTiles(0);
  __syncthreads();

  const int lrow = lane & 31, g = lane >> 5;
  for (unsigned kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < KT) {
      loadA(((kt + 1) * KSPLIT + grp) * BK);
      loadB(((kt + 1) * KSPLIT + grp) * BK);
    }
    const float* as = As + buf * BM * BK + (wm * WM) * BK;
    const float* bs = Bs + buf * BN * BK + (wn * WN) * BK;
#pragma unroll
    for (int kb = 0; kb < BK / 8; ++kb) {
      v4f af[MI], bf[NI];
#pragma unroll
      for (int i = 0; i < MI; ++i) {
        const int row = i * 32 + lrow;
        af[i] = *reinterpret_cast<const v4f*>(as + row * BK + swz(row, kb * 2 + g) * 4);
      }
#pragma unroll
      for (int j = 0; j < NI; ++j) {
        const int row = j * 32 + lrow;
        bf[j] = *reinterpret_cast<const v4f*>(bs + row * BK + swz(row, kb * 2 + g) * 4);
      }
#pragma unroll
      for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
          for (int j = 0; j < NI; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i][s], bf[j][s], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < KT) storeTiles(buf ^ 1);
    __syncthreads();
  }

  if constexpr (KSPLIT > 1) {
    // partial tiles of groups 1 .. KSPLIT-1 go through LDS (the slab buffers are free after the last
    // barrier) and are added by group 0 in group order
    float* red = smemf;
    const int slot = ((grp - 1) * GW + wave) * MI * NI;
    if (grp > 0) {
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) red[((slot + i * NI + j) * 16 + r) * 64 + lane] = acc[i][j][r];
    }
    __syncthreads();
    if (grp > 0) return;
#pragma unroll
    for (int q = 1; q < KSPLIT; ++q)
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            acc[i][j][r] += red[((((q - 1) * GW + wave) * MI * NI + i * NI + j) * 16 + r) * 64 + lane];
  }

  // ---- epilogue: + bias, store.  Lane (i, g) owns columns NI*i .. NI*i+NI-1 of the wavefront's
  // column range and rows 8*(r/4) + 4*g + r%4 of each 32-row block.
  float* __restrict__ C = Cbase;
  const float* __restrict__ R = p.residual ? p.residual + (size_t)bi * p.strideR : nullptr;  // dense, flat batch
  const int act = p.act;
  const unsigned gcol = n0 + wn * WN + NI * lrow;
  const bool residualByLanes = EARLY_RESIDUAL || !R || (VEC && reinterpret_cast<uintptr_t>(R) % 16 == 0 && N % 4 == 0);
  if (m0 + wm * WM + WM <= M && n0 + wn * WN + WN <= N && ldc < (1u << 24) && residualByLanes) {
    // A whole WM x WN block: no bounds to check, and the addresses are a register per lane (row 4g, the lane's first
    // column), a scalar per row and an immediate per column - no address arithmetic per value.
    const unsigned blockCol = n0 + wn * WN;
    const __amdgpu_buffer_rsrc_t rc =
        __builtin_amdgcn_make_buffer_rsrc(C + (size_t)(m0 + wm * WM) * ldc + blockCol, 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t rr = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(R ? R + (size_t)(m0 + wm * WM) * N + blockCol : C), 0, 0x7fffffff, 0x00020000);
    const unsigned voff = ((4 * g) * ldc + NI * lrow) * 4u, voffR = ((4 * g) * N + NI * lrow) * 4u;
    auto store = [&](bool gelu) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < MI; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const unsigned rowInBlock = i * 32 + 8 * (r / 4) + (r & 3);
          float v[NI];
#pragma unroll
          for (int j = 0; j < NI; ++j) v[j] = acc[i][j][r] + bv[j];
          if (R) {
            if constexpr (EARLY_RESIDUAL) {
#pragma unroll
              for (int j = 0; j < NI; ++j) v[j] += rv[i][j][r];
            } else if constexpr (NI == 4) {
              const v4f w = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rr, voffR, rowInBlock * N * 4u, 0));
#pragma unroll
              for (int j = 0; j < NI; ++j) v[j] += w[j];
            } else {
#pragma unroll
              for (int j = 0; j < NI; ++j)
                v[j] += __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rr, voffR + j * 4u, rowInBlock * N * 4u, 0));
            }
          }
          if (gelu) {
#pragma unroll
            for (int j = 0; j < NI; ++j) v[j] = gelu_erf_f32(v[j]);
          }
          if constexpr (NI == 4 && VEC) {
            typedef unsigned v4u __attribute__((ext_vector_type(4)));
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, v4f{v[0], v[1], v[2], v[3]}), rc, voff,
                                                   rowInBlock * ldc * 4u, 0);
          } else {
#pragma unroll
            for (int j = 0; j < NI; ++j)
              __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v[j]), rc, voff + j * 4u,
                                                    rowInBlock * ldc * 4u, 0);
          }
        }
      }
    };
    if (act == 1) store(true); else store(false);
    return;
  }
  const bool vecOK = VEC && (gcol + NI <= N);
#pragma unroll
  for (int i = 0; i < MI; ++i) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const unsigned grow = m0 + wm * WM + i * 32 + 8 * (r / 4) + 4 * g + (r & 3);
      if (grow >= M) continue;
      float v[NI];
#pragma unroll
      for (int j = 0; j < NI; ++j) v[j] = acc[i][j][r] + bv[j];
      const size_t off = (size_t)grow * ldc + gcol;
      if (R) {
        if constexpr (EARLY_RESIDUAL) {
#pragma unroll
          for (int j = 0; j < NI; ++j) v[j] += rv[i][j][r];
        } else {
          const size_t roff = (size_t)grow * N + gcol;
#pragma unroll
          for (int j = 0; j < NI; ++j)
            if (gcol + j < N) v[j] += R[roff + j];
        }
      }
      if (act == 1) {
        // same expression as the stand-alone GELU kernel, so that fusing changes no bit
#pragma unroll
        for (int j = 0; j < NI; ++j)
          v[j] = gelu_erf_f32(v[j]);
      }
      if (vecOK) {
        if constexpr (NI == 4) *reinterpret_cast<v4f*>(C + off) = v4f{v[0], v[1], v[2], v[3]};
        else if constexpr (NI == 2) *reinterpret_cast<float2*>(C + off) = make_float2(v[0], v[1]);
        else {
#pragma unroll
          for (int j = 0; j < NI; ++j) C[off + j] = v[j];
        }
      } else {
#pragma unroll
        for (int j = 0; j < NI; ++j)
          if (gcol + j < N) C[off + j] = v[j];
      }
    }
  }
}

template <int WGM, int WGN, int MI, int NI, bool VEC, int KSPLIT = 1, bool TRANSB = false>
int launch(hipStream_t stream, SgemmParams p) {
  constexpr int BM = WGM * MI * 32, BN = WGN * NI * 32;
  if (!sgemm_detail::set_tiles(p, BM, BN)) return set_error(TFCC_ROCM_INVALID_ARGUMENT, "sgemm: too many tiles");
  constexpr size_t lds = KSPLIT * 2 * (size_t)(BM + BN) * BK * sizeof(float);
  static_assert(lds <= 160 * 1024 && (size_t)(KSPLIT - 1) * BM * BN * sizeof(float) <= lds, "LDS budget");
  auto kern = sgemm_kernel<WGM, WGN, MI, NI, VEC, KSPLIT, TRANSB>;
  static bool attrSet[16] = {};  // per device: the attribute belongs to the function on one device
  int dev = 0;
  TFCC_HIP_CHECK(hipGetDevice(&dev));
  TFCC_REQUIRE(dev >= 0 && dev < 16, "device index %d", dev);
  if (!attrSet[dev]) {
    TFCC_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attrSet[dev] = true;
  }
  hipLaunchKernelGGL(kern, dim3(p.chunk * 8), dim3(WGM * WGN * 64 * KSPLIT), lds, stream, p);
  return check_launch("sgemm");
}

// The tile table of the kernels that copy K slabs straight into LDS, ordered by falling tile area.
const struct { int config; unsigned bm, bn, waves; } kTiles[] = {{0, 64, 64, 4}, {1, 32, 96, 3}, {2, 32, 64, 2}, {3, 32, 32, 1}};

// Tile and number of K groups for m x n x k with K a multiple of 32: the tile that covers the 256 CUs in the fewest
// tile-area rounds, the larger one on a tie (less operand traffic); as few K groups as give every CU eight
// wavefronts, each group keeping at least four slabs.
void choose_dma_tiles(unsigned m, unsigned n, unsigned k, unsigned fillBatch, int& best, unsigned long long& bestTiles,
                      int& ksplit) {
  best = 0;
  unsigned long long bestCost = ~0ull;
  bestTiles = 0;
  for (int c = 0; c < 4; ++c) {
    const unsigned long long tiles =
        (unsigned long long)((m + kTiles[c].bm - 1) / kTiles[c].bm) * ((n + kTiles[c].bn - 1) / kTiles[c].bn) * fillBatch;
    const unsigned long long cost = ((tiles + 255) / 256) * (kTiles[c].bm * kTiles[c].bn);
    if (cost < bestCost) {
      best = c;
      bestCost = cost;
      bestTiles = tiles;
    }
  }
  ksplit = 1;
  while (ksplit < 4 && bestTiles * kTiles[best].waves * ksplit < 256ull * 8 && k >= 128u * (ksplit * 2)) ksplit *= 2;
}

// The number of K groups the kernels for B as stored [k, n] would sum this product with (the sums of an element
// are defined by it, not by the tile shape): B given transposed must use the same, so that transposing B first
// and multiplying give the same bits as multiplying the transposed view.
// 128 x 128 tiles: once there are enough of them to fill the 256 CUs twice over, and only when they are mostly
// result (a batch of 768 products of 64 x 64 x 64 counts 768 such tiles, each three quarters empty: 23 us in them
// against 11 in 64 x 64 tiles).
bool takes_128_tiles(unsigned m, unsigned n, unsigned fillBatch) {
  const unsigned long long big = (unsigned long long)((m + 127) / 128) * ((n + 127) / 128) * fillBatch;
  return big >= 512 && (unsigned long long)m * n * fillBatch * 100 >= big * (128 * 128) * 75;
}

int k_groups_of_plain_product(unsigned m, unsigned n, unsigned k, unsigned fillBatch) {
  if (takes_128_tiles(m, n, fillBatch)) return 1;
  if (k % 32 == 0) {
    int best, ksplit;
    unsigned long long tiles;
    choose_dma_tiles(m, n, k, fillBatch, best, tiles, ksplit);
    return ksplit;
  }
  const unsigned long long small = (unsigned long long)((m + 63) / 64) * ((n + 63) / 64) * fillBatch;
  const unsigned long long flat = (unsigned long long)((m + 31) / 32) * ((n + 95) / 96) * fillBatch;
  const bool preferFlat = ((flat + 255) / 256) * (32 * 96) < ((small + 255) / 256) * (64 * 64);
  if (preferFlat && flat <= 320 && k >= 512) return 4;
  if (small <= 320 && k >= 512) return 4;
  if (small <= 640 && k >= 256) return 2;
  return 1;
}

// Picks the tile configuration from the shape of one product and the number of batch entries that
// count towards filling the chip (`fillBatch`), and launches.
int dispatch(hipStream_t s, const SgemmParams& p, bool vec, bool tb, unsigned fillBatch, unsigned lda, unsigned ldb,
             unsigned ldc) {
  const unsigned m = p.M, n = p.N, k = p.K;
  const unsigned long long rowsB = tb ? n : k;
  if (tb) {
    if (vec) {
      const int groups = k_groups_of_plain_product(m, n, k, fillBatch);
      if (groups == 4) return launch<2, 2, 1, 1, true, 4, true>(s, p);
      if (groups == 2) return launch<2, 2, 1, 1, true, 2, true>(s, p);
      return launch<2, 2, 1, 1, true, 1, true>(s, p);
    }
    TFCC_REQUIRE((unsigned long long)m * ldc < (1ull << 32) && (unsigned long long)m * lda < (1ull << 32) &&
                 rowsB * ldb < (1ull << 32), "sgemm: operand larger than 2^32 elements");
    return launch<2, 2, 1, 1, false, 1, true>(s, p);
  }
  // One product (or a few that share A) of at most eight rows: a single pass over B decides the time, and the
  // streaming kernel makes it without tiles.  A true batch keeps the tiled kernels, whose sums the fused attention
  // kernel reproduces bit for bit.
  if (fillBatch == 1 && sgemm_detail::sgemv_supported(p)) return sgemm_detail::sgemv_launch(s, p);
  // 128x128 tiles once there are enough of them to fill the 256 CUs twice over, else 64x64
  if (vec) {
    // (whole slabs of K: four hand-scheduled wavefronts of 32 x 128 on a shared ring, two workgroups per CU -
    // 4096^3: 150 TFLOP/s against 141 for the same tiles scheduled by the compiler)
    if (takes_128_tiles(m, n, fillBatch)) return k % 32 == 0 ? sgemm_detail::sgemm_wave96_launch(s, p, 1, 4) : launch<4, 1, 1, 4, true>(s, p);
    // few 64x64 tiles and a long K: several K groups per workgroup keep the CUs that have a tile busy
    const unsigned long long small = (unsigned long long)((m + 63) / 64) * ((n + 63) / 64) * fillBatch;
    // 32x96 tiles when they cover the 256 CUs in fewer tile-area rounds than 64x64 tiles would
    const unsigned long long flat = (unsigned long long)((m + 31) / 32) * ((n + 95) / 96) * fillBatch;
    const bool preferFlat = ((flat + 255) / 256) * (32 * 96) < ((small + 255) / 256) * (64 * 64);
    if (k % 32 == 0) {
      // whole slabs of K: the kernels that copy the slabs straight into LDS
      int best, ksplit;
      unsigned long long bestTiles;
      choose_dma_tiles(m, n, k, fillBatch, best, bestTiles, ksplit);
      // The hand-scheduled kernel of sgemm_wave96.hip (one wavefront per SIMD, no vector instruction between its
      // matrix ops) takes every product with four K groups - the groups as the four wavefronts of a workgroup on
      // 32 x 96, 32 x 64 and 32 x 32 tiles, four pairs of wavefronts on 64 x 64 tiles (1024 x 768 x 3072: 36.3
      // against 45.9 us for the kernels of sgemm_dma.hip, 128 x 768 x 3072: 8.6 against 11.4 with the operands in
      // cache, 960 x 1024 x 2048: 34.4 against 41.9) ...
      if (ksplit == 4) {
        // (Tiles of 16 x 96 from 16x16x4 matrix ops - the same bits, 256 tiles instead of 192 for 128 x 768 x 3072 and
        // a quarter less matrix time - were built and measured: 7.6 against 8.3 us with the operands in cache, 10.1
        // against 9.8 with them in HBM, where the wait for the first slab and the bytes in flight decide, not the
        // matrix ops.  The table's tiles keep the product.)
        const int c = kTiles[best].config;
        return sgemm_detail::sgemm_wave96_launch(s, p, 4, c == 0 ? 2 : c == 1 ? 3 : c == 2 ? 2 : 1, c == 0 ? 2 : 1);
      }
      // ... with two K groups the 64 x 64 tiles (two pairs of wavefronts) and the 32 x 32 tiles (two wavefronts):
      // 1024^3 20.1 against 24.2 us, 400 x 400 x 256 5.3 against 7.3; on 32 x 96 and 32 x 64 tiles the kernels of
      // sgemm_dma.hip are as fast or faster and keep the product ...
      if (ksplit == 2 && kTiles[best].config == 0) return sgemm_detail::sgemm_wave96_launch(s, p, 2, 2, 2);
      if (ksplit == 2 && kTiles[best].config == 3) return sgemm_detail::sgemm_wave96_launch(s, p, 2, 1, 1);
      // ... and without K groups the products whose 128 x 96 tiles fill at least 70 % of the CUs in each of their
      // rounds (or 128 x 128 tiles 85 %), K >= 512: four wavefronts of 32 x 96 (32 x 128) share each copy of B
      // (1024 x 3072 x 768 with GELU: 39.3 against 42.4 us in 64 x 64 tiles, 1536^3: 69 against 80, 2048^3 in
      // 128 x 128 tiles: 120 against 136; below those fills, or with a short K, the tiles of the table win).  The
      // sums are the same in every case: the K groups of the table, ascending k inside a group.
      if (ksplit == 1 && k >= 512) {
        const unsigned long long wide = (unsigned long long)((m + 127) / 128) * ((n + 95) / 96) * fillBatch;
        const unsigned long long wide4 = (unsigned long long)((m + 127) / 128) * ((n + 127) / 128) * fillBatch;
        const bool ok3 = wide * 100 >= 70 * 256 * ((wide + 255) / 256), ok4 = wide4 * 100 >= 85 * 256 * ((wide4 + 255) / 256);
        const unsigned long long cost3 = ((wide + 255) / 256) * 96, cost4 = ((wide4 + 255) / 256) * 128;
        if (ok4 && (!ok3 || cost4 < cost3)) return sgemm_detail::sgemm_wave96_launch(s, p, 1, 4);
        if (ok3) return sgemm_detail::sgemm_wave96_launch(s, p, 1);
      }
      // What is left runs on the kernels of sgemm_dma.hip.  Several products in one launch (p.batch counts them;
      // fillBatch = 1 chose the configuration of a single one so that each is summed exactly as on its own): when
      // they fill the chip without the K groups, one group per tile plays all of them; and when 128 x 96 tiles over
      // all of them still occupy most of the CUs in one round, twelve wavefronts share each copy of B among four
      // times the rows (the sums are those of the 32 x 96 tiles).
      const bool serial = ksplit > 1 && bestTiles * (p.batch / fillBatch) * kTiles[best].waves >= 256ull * 8;
      if (serial && kTiles[best].config == 1) {
        const unsigned long long wide = (unsigned long long)((m + 127) / 128) * ((n + 95) / 96) * p.batch;
        if (wide <= 256 && wide >= 160) return sgemm_detail::sgemm_dma_launch(s, p, 5, ksplit, true);
      }
      return sgemm_detail::sgemm_dma_launch(s, p, kTiles[best].config, ksplit, serial);
    }
    if (preferFlat && flat <= 320 && k >= 512) return launch<1, 3, 1, 1, true, 4>(s, p);
    if (small <= 320 && k >= 512) return launch<2, 2, 1, 1, true, 4>(s, p);
    if (small <= 640 && k >= 256) return launch<2, 2, 1, 1, true, 2>(s, p);
    return launch<2, 2, 1, 1, true>(s, p);
  }
  TFCC_REQUIRE((unsigned long long)m * ldc < (1ull << 32) && (unsigned long long)m * lda < (1ull << 32) &&
               rowsB * ldb < (1ull << 32), "sgemm: operand larger than 2^32 elements");
  return launch<2, 2, 1, 1, false>(s, p);
}

}  // namespace
}  // namespace tfcc_rocm

using namespace tfcc_rocm;

extern "C" int tfcc_rocm_sgemm_strided_batched(void* stream, const float* a, uint64_t stride_a,
                                               const float* b, uint64_t stride_b, const float* bias,
                                               float* c, uint64_t stride_c, unsigned m, unsigned n,
                                               unsigned k, unsigned batch) {
  return tfcc_rocm_sgemm_fused(stream, a, stride_a, b, stride_b, bias, nullptr, 0, c, stride_c, m, n, k, batch, 0);
}

extern "C" int tfcc_rocm_sgemm_fused(void* stream, const float* a, uint64_t stride_a, const float* b,
                                     uint64_t stride_b, const float* bias, const float* residual,
                                     uint64_t stride_residual, float* c, uint64_t stride_c, unsigned m,
                                     unsigned n, unsigned k, unsigned batch, int activation) {
  tfcc_rocm_sgemm_desc d{};
  d.a = a; d.b = b; d.bias = bias; d.residual = residual; d.c = c;
  d.m = m; d.n = n; d.k = k;
  d.lda = k; d.ldb = n; d.ldc = n;
  d.batch_outer = batch; d.batch_inner = 1;
  d.stride_a = stride_a; d.stride_b = stride_b; d.stride_c = stride_c; d.stride_residual = stride_residual;
  d.activation = activation;
  return tfcc_rocm_sgemm_general(stream, &d);
}

extern "C" int tfcc_rocm_sgemm_general(void* stream, const tfcc_rocm_sgemm_desc* d) {
  TFCC_REQUIRE(d != nullptr, "sgemm: null descriptor");
  TFCC_REQUIRE(d->a && d->b && d->c, "sgemm: null operand");
  TFCC_REQUIRE(d->m > 0 && d->n > 0 && d->k > 0 && d->batch_outer > 0 && d->batch_inner > 0, "sgemm: empty operand");
  TFCC_REQUIRE(d->activation == 0 || d->activation == 1, "sgemm: unknown activation %d", d->activation);
  const unsigned m = d->m, n = d->n, k = d->k;
  TFCC_REQUIRE(d->lda >= k && d->ldc >= n && d->ldb >= (d->trans_b ? k : n), "sgemm: row stride shorter than a row");
  const unsigned long long batch64 = (unsigned long long)d->batch_outer * d->batch_inner;
  TFCC_REQUIRE(batch64 < (1ull << 31), "sgemm: too many batch entries");
  TFCC_REQUIRE(!d->residual || (d->ldc == n && (d->batch_inner == 1 || (d->inner_stride_c == (uint64_t)m * n &&
                                                                          d->stride_c == (uint64_t)d->batch_inner * m * n))),
               "sgemm: a residual needs a dense result");
  SgemmParams p{};
  p.A = d->a; p.B = d->b; p.bias = d->bias; p.C = d->c; p.residual = d->residual; p.strideR = d->stride_residual;
  p.act = d->activation;
  p.strideA = d->stride_a; p.strideB = d->stride_b; p.strideC = d->stride_c;
  p.innerA = d->inner_stride_a; p.innerB = d->inner_stride_b; p.innerC = d->inner_stride_c;
  p.batchInner = d->batch_inner;
  p.lda = d->lda; p.ldb = d->ldb; p.ldc = d->ldc;
  p.M = m; p.N = n; p.K = k; p.batch = (unsigned)batch64;
  const unsigned batch = p.batch;
  const bool tb = d->trans_b != 0;
  const unsigned long long rowsB = tb ? n : k, colsB = tb ? k : n;  // B as stored
  const bool vec = (k % 4 == 0) && (n % 4 == 0) && ((uintptr_t)d->a % 16 == 0) && ((uintptr_t)d->b % 16 == 0) &&
                   ((uintptr_t)d->c % 16 == 0) && (d->lda % 4 == 0) && (d->ldb % 4 == 0) && (d->ldc % 4 == 0) &&
                   (p.strideA % 4 == 0) && (p.strideB % 4 == 0) && (p.strideC % 4 == 0) && (p.innerA % 4 == 0) &&
                   (p.innerB % 4 == 0) && (p.innerC % 4 == 0) &&
                   (((unsigned long long)m + 256) * d->lda + k + 256 < (1ull << 30)) &&
                   ((rowsB + 256) * d->ldb + colsB + 1024 < (1ull << 30));
  hipStream_t s = as_stream(stream);
  return dispatch(s, p, vec, tb, batch, d->lda, d->ldb, d->ldc);
}

extern "C" int tfcc_rocm_sgemm_grouped(void* stream, const float* a, const float* const* b, const float* const* bias,
                                       float* const* c, unsigned groups, unsigned m, unsigned n, unsigned k) {
  TFCC_REQUIRE(a && b && c, "grouped sgemm: null operand");
  TFCC_REQUIRE(groups >= 1 && groups <= 4, "grouped sgemm: 1 to 4 products per launch, got %u", groups);
  TFCC_REQUIRE(m > 0 && n > 0 && k > 0, "grouped sgemm: empty operand");
  SgemmParams p{};
  p.A = a; p.M = m; p.N = n; p.K = k; p.batch = groups; p.batchInner = 1;
  p.lda = k; p.ldb = n; p.ldc = n;
  p.groups = groups;
  bool aligned = (uintptr_t)a % 16 == 0;
  for (unsigned g = 0; g < 4; ++g) {
    const unsigned src = g < groups ? g : 0;
    TFCC_REQUIRE(b[src] && c[src], "grouped sgemm: null operand");
    p.groupB[g] = b[src];
    p.groupBias[g] = bias ? bias[src] : nullptr;
    p.groupC[g] = c[src];
    aligned = aligned && (uintptr_t)b[src] % 16 == 0 && (uintptr_t)c[src] % 16 == 0;
  }
  p.B = p.groupB[0];
  p.C = p.groupC[0];
  const bool vec = aligned && (k % 4 == 0) && (n % 4 == 0) && (((unsigned long long)m + 256) * k + k + 256 < (1ull << 30)) &&
                   (((unsigned long long)k + 256) * n + n + 1024 < (1ull << 30));
  // the tile configuration is the one a single product of this shape gets, so that every product
  // of the group is summed in exactly the order of a launch of its own
  return dispatch(as_stream(stream), p, vec, false, 1, k, n, n);
}

