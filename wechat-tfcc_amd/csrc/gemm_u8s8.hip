// uint8 x int8 -> int32 matrix product on the gfx950 int8 matrix cores, with the offset terms of
// the reference's quantized matmul and (optionally) its requantize step fused into the tile store.
//
// Replaces tfcc/mkl/operations/tfcc_mklquantization.cpp:33-69,176-201 (offset matrix + threaded
// driver), tfcc/mkl/gemm/tfcc_mklsinglethreadgemm.h:93-141 (blocking / packing) and the 24x4x2
// micro-kernel tfcc/mkl/gemm/tfcc_mklmatmulkernel.h:142-260.
//
// Layout.  A is [M,K] uint8 and B is [K,N] int8, both row-major in HBM.  A workgroup of four
// wavefronts owns a BM x BN tile of C and walks K in slabs of BK bytes:
//   * A slab: 128-bit global loads (16 consecutive k of one row), xor 0x80 turns the uint8 into
//     int8 (a' = a - 128), 128-bit LDS stores into As[row][k] with the 16-byte chunks of a row
//     xor-swizzled by the row index so that both the stores and the matrix-core operand reads are
//     bank-conflict free.
//   * B slab: k is the strided dimension in HBM but the matrix-core operand wants 16 consecutive
//     k per lane, so every thread loads a 16(k) x 4(n) byte block as 16 dwords (a wavefront reads
//     whole 256-byte rows), transposes it in registers with v_perm_b32 and stores four 128-bit
//     chunks into Bs[col][k].  Tile columns are stored interleaved (LDS row = j*32 + i for tile
//     column NI*i + j) so that the lane i of a 32-column MFMA block ends up owning NI consecutive
//     output columns: the epilogue then writes 4 packed uint8 (one dword) or 4 int32 (128 bits)
//     per lane and a wavefront writes whole 128-byte / 512-byte row segments.
//   * v_mfma_i32_32x32x32_i8 accumulates a' * b in int32; each wavefront holds a (BM/2)x(BN/2)
//     sub-tile in registers.
// The int8 product is turned into the reference's result with rank-1 terms in the epilogue:
//   sum (a+oA)(b+oB) = sum a'b + 128*colsum(B)[j] + oB*rowsumA[i] + oA*colsumB[j] + K*oA*oB
// where rowsumA / colsumB are the caller's tensors (used as given, like the reference) and
// colsum(B) is the true column sum, accumulated on the fly from the transposed B registers with
// v_dot4_i32_i8 so that no assumption about the caller's tensors is needed.
#include <type_traits>

#include "common.hpp"
#include "gemv.hpp"
#include "qgemm_dma.hpp"
#include "qgemm_params.hpp"

namespace tfcc_rocm {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

namespace {

constexpr int kThreads = 256;

// 4x4 byte transpose: in r[q] = bytes (n0..n3) of k-row q; out c[j] = bytes (k0..k3) of column j
__device__ __forceinline__ void transpose4x4(const unsigned r[4], unsigned c[4]) {
  // v_perm_b32(hi, lo, sel): selector bytes 0-3 pick from lo, 4-7 from hi
  unsigned t0 = __builtin_amdgcn_perm(r[1], r[0], 0x05010400u);  // r0.b0 r1.b0 r0.b1 r1.b1
  unsigned t1 = __builtin_amdgcn_perm(r[1], r[0], 0x07030602u);  // r0.b2 r1.b2 r0.b3 r1.b3
  unsigned t2 = __builtin_amdgcn_perm(r[3], r[2], 0x05010400u);
  unsigned t3 = __builtin_amdgcn_perm(r[3], r[2], 0x07030602u);
  c[0] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);  // t0.lo16 t2.lo16
  c[1] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);  // t0.hi16 t2.hi16
  c[2] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
  c[3] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
}

template <int BK>
__device__ __forceinline__ int swizzled_chunk(int row, int chunk) {
  constexpr int CH = BK / 16;       // 16-byte chunks per LDS row
  constexpr int RP = 16 / CH;       // rows per 256 bytes
  return chunk ^ ((row / RP) & (CH - 1));
}

template <int BM, int BN, int BK, bool ALIGNED, bool REQUANT>
__global__ __launch_bounds__(kThreads) void qgemm_kernel(const QGemmParams p) {
  constexpr int WM = BM / 2, WN = BN / 2;  // wavefront sub-tile
  constexpr int MI = WM / 32, NI = WN / 32;
  constexpr int CH = BK / 16;
  constexpr int A_ITEMS = BM * CH / kThreads;            // 16-byte chunks of A per thread
  constexpr int B_ITEMS = (BN / 4) * CH / kThreads;      // 16(k) x 4(n) blocks of B per thread
  static_assert(A_ITEMS >= 1 && B_ITEMS >= 1, "tile too small for 256 threads");
  static_assert(NI == 4 || NI == 2, "column interleave assumes 2 or 4 blocks per wavefront");

  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* As = smem;                       // [2][BM][BK]
  unsigned char* Bs = smem + 2 * BM * BK;         // [2][BN][BK]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // ---- which tile: consecutive workgroup ids go to different XCDs (round robin over 8), so give
  // each XCD a contiguous run of tiles, ordered in bands of 4 tile rows, to keep the A rows and B
  // columns one L2 sees as few as possible.
  unsigned tm, tn, bi;
  {
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
  const unsigned char* __restrict__ A = p.A + (size_t)bi * p.strideA;
  const signed char* __restrict__ B = p.B + (size_t)bi * p.strideB;

  // offsets: immediate, or from float ranges in device memory
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

  v16i acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  v4i aReg[A_ITEMS];
  unsigned bReg[B_ITEMS][16];
  int colsum[4] = {0, 0, 0, 0};  // true column sums of this thread's 4 columns over its k chunks

  // ---- global -> registers
  // In the aligned path every global read is a raw buffer load: an offset past the end of the
  // operand (rows >= M of A, rows >= K of B) returns zero without a branch.  Bytes of A beyond K
  // inside a row and columns of B beyond N read neighbouring data; they only ever meet zero
  // B rows or columns that are never stored.
  const __amdgpu_buffer_rsrc_t rsrcA =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(A), 0, ALIGNED ? (int)(M * K) : 0, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrcB =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<signed char*>(B), 0, ALIGNED ? (int)(K * N) : 0, 0x00020000);
  auto loadA = [&](unsigned k0) {
#pragma unroll
    for (int it = 0; it < A_ITEMS; ++it) {
      const int w = tid + it * kThreads;
      const int row = w / CH, ch = w % CH;
      const unsigned gr = m0 + row, gk = k0 + ch * 16;
      v4i v = {0, 0, 0, 0};
      if constexpr (ALIGNED) {
        v = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrcA, gr * K + gk, 0, 0));
      } else {
        if (gr < M) {
          unsigned char tmp[16];
#pragma unroll
          for (int q = 0; q < 16; ++q) tmp[q] = (gk + q < K) ? A[(size_t)gr * K + gk + q] : 0;
#pragma unroll
          for (int q = 0; q < 4; ++q)
            v[q] = (int)(tmp[4 * q] | (tmp[4 * q + 1] << 8) | (tmp[4 * q + 2] << 16) | ((unsigned)tmp[4 * q + 3] << 24));
        }
      }
      aReg[it] = v;
    }
  };
  auto loadB = [&](unsigned k0) {
#pragma unroll
    for (int it = 0; it < B_ITEMS; ++it) {
      const int w = tid + it * kThreads;
      const int nd = w % (BN / 4), ch = w / (BN / 4);
      const unsigned gn = n0 + nd * 4, gk = k0 + ch * 16;
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        unsigned v = 0;
        if constexpr (ALIGNED) {
          v = __builtin_amdgcn_raw_buffer_load_b32(rsrcB, (gk + q) * N + gn, 0, 0);
        } else {
          if (gk + q < K) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (gn + e < N) v |= (unsigned)(unsigned char)B[(size_t)(gk + q) * N + gn + e] << (8 * e);
          }
        }
        bReg[it][q] = v;
      }
    }
  };
  // ---- registers -> LDS (A: uint8 -> int8; B: transpose, column interleave, column sums)
  auto storeTiles = [&](int buf) {
    unsigned char* as = As + buf * BM * BK;
    unsigned char* bs = Bs + buf * BN * BK;
#pragma unroll
    for (int it = 0; it < A_ITEMS; ++it) {
      const int w = tid + it * kThreads;
      const int row = w / CH, ch = w % CH;
      v4i v = aReg[it] ^ (int)0x80808080;
      *reinterpret_cast<v4i*>(as + row * BK + swizzled_chunk<BK>(row, ch) * 16) = v;
    }
#pragma unroll
    for (int it = 0; it < B_ITEMS; ++it) {
      const int w = tid + it * kThreads;
      const int nd = w % (BN / 4), ch = w / (BN / 4);
      unsigned col[4][4];  // [column j][k quad]
#pragma unroll
      for (int kq = 0; kq < 4; ++kq) {
        unsigned c4[4];
        transpose4x4(&bReg[it][4 * kq], c4);
#pragma unroll
        for (int j = 0; j < 4; ++j) col[j][kq] = c4[j];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int kq = 0; kq < 4; ++kq)
          colsum[j] = __builtin_amdgcn_sdot4((int)col[j][kq], 0x01010101, colsum[j], false);
        // tile column -> LDS row (interleave NI columns per lane)
        const int n = nd * 4 + j;
        const int wnn = n / WN, within = n % WN;
        const int row = wnn * WN + (within % NI) * 32 + within / NI;
        v4i v = {(int)col[j][0], (int)col[j][1], (int)col[j][2], (int)col[j][3]};
        *reinterpret_cast<v4i*>(bs + row * BK + swizzled_chunk<BK>(row, ch) * 16) = v;
      }
    }
  };

  const unsigned KT = (K + BK - 1) / BK;
  loadA(0);
  loadB(0);
  storeTiles(0);
  __syncthreads();

  const int lrow = lane & 31, khalf = lane >> 5;
  for (unsigned kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < KT) {
      loadA((kt + 1) * BK);
      loadB((kt + 1) * BK);
    }
    const unsigned char* as = As + buf * BM * BK + (wm * WM) * BK;
    const unsigned char* bs = Bs + buf * BN * BK + (wn * WN) * BK;
#pragma unroll
    for (int ks = 0; ks < BK / 32; ++ks) {
      v4i af[MI], bf[NI];
#pragma unroll
      for (int i = 0; i < MI; ++i) {
        const int row = i * 32 + lrow;  // (wm*WM is a multiple of 16: swizzle of the absolute row is the same)
        af[i] = *reinterpret_cast<const v4i*>(as + row * BK + swizzled_chunk<BK>(row, ks * 2 + khalf) * 16);
      }
#pragma unroll
      for (int j = 0; j < NI; ++j) {
        const int row = j * 32 + lrow;
        bf[j] = *reinterpret_cast<const v4i*>(bs + row * BK + swizzled_chunk<BK>(row, ks * 2 + khalf) * 16);
      }
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < KT) storeTiles(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue.  LDS is free now: reuse it for the per-tile row / column terms.
  int* colTerm = reinterpret_cast<int*>(smem);            // [BN]  indexed by tile column
  int* rowTerm = colTerm + BN;                             // [BM]
  for (int i = tid; i < BN; i += kThreads) colTerm[i] = 0;
  __syncthreads();
  {
    // every thread owned the same 4 columns in every slab: nd = tid % (BN/4) (+ it*256 % (BN/4) = 0)
    const int nd = tid % (BN / 4);
#pragma unroll
    for (int j = 0; j < 4; ++j) atomicAdd(&colTerm[nd * 4 + j], colsum[j]);
  }
  __syncthreads();
  const int* __restrict__ rsA = p.rowsumA + (size_t)bi * p.strideRA;
  const int* __restrict__ csB = p.colsumB + (size_t)bi * p.strideRB;
  const unsigned global = (unsigned)offA * (unsigned)offB * K;
  for (int i = tid; i < BN; i += kThreads) {
    unsigned gn = n0 + i;
    unsigned cs = gn < N ? (unsigned)csB[gn] : 0u;
    colTerm[i] = (int)(128u * (unsigned)colTerm[i] + cs * (unsigned)offA);
  }
  for (int i = tid; i < BM; i += kThreads) {
    unsigned gm = m0 + i;
    unsigned rs = gm < M ? (unsigned)rsA[gm] : 0u;
    rowTerm[i] = (int)(global + rs * (unsigned)offB);
  }
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

  int* __restrict__ C = p.C ? p.C + (size_t)bi * p.strideC : nullptr;
  unsigned char* __restrict__ Q = REQUANT ? p.Q + (size_t)bi * p.strideC : nullptr;
  const unsigned colBase = wn * WN + NI * lrow;       // tile column of this lane's first element
  const unsigned gcol = n0 + colBase;
  int ct[NI];
#pragma unroll
  for (int j = 0; j < NI; ++j) ct[j] = colTerm[colBase + j];
  const bool vecOK = ALIGNED && (gcol + NI <= N);     // N % 4 == 0 and base pointers aligned when ALIGNED

  // FLAVOUR 0: int32 only; 1: requantize, double shortcut; 2: exact int64 path; 3: constant fill; 4: int32 shortcut
  auto storeTile = [&](auto flavour) {
    constexpr int FLAVOUR = decltype(flavour)::value;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int trow = wm * WM + i * 32 + 8 * (r / 4) + 4 * khalf + (r & 3);
        const unsigned grow = m0 + trow;
        if (grow >= M) continue;
        const int rt = rowTerm[trow];
        int v[NI];
#pragma unroll
        for (int j = 0; j < NI; ++j) v[j] = (int)((unsigned)acc[i][j][r] + (unsigned)rt + (unsigned)ct[j]);
        const size_t off = (size_t)grow * N + gcol;
        if (C) {
          if (vecOK) {
            if constexpr (NI == 4) *reinterpret_cast<v4i*>(C + off) = v4i{v[0], v[1], v[2], v[3]};
            else *reinterpret_cast<int2*>(C + off) = make_int2(v[0], v[1]);
          } else {
#pragma unroll
            for (int j = 0; j < NI; ++j) if (gcol + j < N) C[off + j] = v[j];
          }
        }
        if constexpr (FLAVOUR != 0) {
          unsigned q[NI];
#pragma unroll
          for (int j = 0; j < NI; ++j) {
            if constexpr (FLAVOUR == 1) {
              // (double)(v - INT32_MIN) without a 64-bit integer: flip the sign bit, convert as unsigned
              q[j] = (unsigned)requantize_one_fast((double)((unsigned)v[j] ^ 0x80000000u), rq);
            } else if constexpr (FLAVOUR == 2) {
              q[j] = (unsigned)requantize_one_exact((long long)v[j], rq);
            } else if constexpr (FLAVOUR == 4) {
              q[j] = (unsigned)requantize_one_fast32((double)((unsigned)v[j] ^ 0x80000000u), rq);
            } else {
              q[j] = (unsigned)rq.fillValue;
            }
          }
          if (vecOK) {
            if constexpr (NI == 4) *reinterpret_cast<unsigned*>(Q + off) = q[0] | (q[1] << 8) | (q[2] << 16) | (q[3] << 24);
            else *reinterpret_cast<unsigned short*>(Q + off) = (unsigned short)(q[0] | (q[1] << 8));
          } else {
#pragma unroll
            for (int j = 0; j < NI; ++j) if (gcol + j < N) Q[off + j] = (unsigned char)q[j];
          }
        }
      }
    }
  };
  if constexpr (!REQUANT) {
    storeTile(std::integral_constant<int, 0>{});
  } else {
    // uniform over the whole launch: every wavefront takes the same branch
    if (rq.mode) storeTile(std::integral_constant<int, 3>{});
    else if (rq.fast32OK) storeTile(std::integral_constant<int, 4>{});
    else if (rq.fastOK) storeTile(std::integral_constant<int, 1>{});
    else storeTile(std::integral_constant<int, 2>{});
  }
}

template <int BM, int BN, int BK, bool ALIGNED, bool REQUANT>
int launch(hipStream_t stream, QGemmParams p) {
  p.tilesM = (p.M + BM - 1) / BM;
  p.tilesN = (p.N + BN - 1) / BN;
  unsigned long long total = (unsigned long long)p.tilesM * p.tilesN * p.batch;
  if (total > 0x7fffffffull) return set_error(TFCC_ROCM_INVALID_ARGUMENT, "quantized matmul: too many tiles");
  p.tilesTotal = (unsigned)total;
  p.chunk = (p.tilesTotal + 7) / 8;
  constexpr size_t lds = 2 * (size_t)(BM + BN) * BK;
  static_assert(lds >= (size_t)(BM + BN) * 4, "epilogue terms must fit in the slab buffers");
  auto kern = qgemm_kernel<BM, BN, BK, ALIGNED, REQUANT>;
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
  return check_launch("quantized matmul");
}

template <bool REQUANT>
int dispatch(hipStream_t stream, const QGemmParams& p) {
  if (qgemm_dma_supported(p, REQUANT)) return qgemm_dma_launch(stream, p, REQUANT);
  const bool aligned = (p.K % 16 == 0) && (p.N % 4 == 0) && ((uintptr_t)p.A % 16 == 0) &&
                       ((uintptr_t)p.B % 4 == 0) && (p.strideA % 16 == 0) && (p.strideB % 4 == 0) &&
                       (p.C == nullptr || ((uintptr_t)p.C % 16 == 0 && p.strideC % 4 == 0)) &&
                       (!REQUANT || ((uintptr_t)p.Q % 4 == 0 && p.strideC % 4 == 0));
  // big tiles once they fill the 256 CUs reasonably; otherwise 128x128
  const unsigned long long big = (unsigned long long)((p.M + 255) / 256) * ((p.N + 255) / 256) * p.batch;
  if (aligned) {
    if (big >= 192) return launch<256, 256, 64, true, REQUANT>(stream, p);
    return launch<128, 128, 128, true, REQUANT>(stream, p);
  }
  return launch<128, 128, 128, false, REQUANT>(stream, p);
}

int fill_params(const tfcc_rocm_qgemm_desc* d, QGemmParams& p) {
  TFCC_REQUIRE(d != nullptr, "quantized matmul: null descriptor");
  TFCC_REQUIRE(d->a && d->b && d->rowsum_a && d->colsum_b, "quantized matmul: null operand");
  TFCC_REQUIRE(d->m > 0 && d->n > 0 && d->k > 0 && d->batch > 0, "quantized matmul: empty operand");
  const bool anyRange = d->min_a || d->max_a || d->min_b || d->max_b;
  const bool allRange = d->min_a && d->max_a && d->min_b && d->max_b;
  TFCC_REQUIRE(!anyRange || allRange, "quantized matmul: give all four range pointers or none");
  TFCC_REQUIRE((unsigned long long)d->m * d->n < (1ull << 32) && (unsigned long long)d->m * d->k < (1ull << 32) &&
               ((unsigned long long)d->k + 256) * d->n + 512 < (1ull << 32),
               "quantized matmul: operand larger than 2^32 elements");
  p = QGemmParams{};
  p.A = d->a; p.B = d->b; p.rowsumA = d->rowsum_a; p.colsumB = d->colsum_b;
  p.strideA = d->stride_a; p.strideB = d->stride_b; p.strideRA = d->stride_rowsum_a;
  p.strideRB = d->stride_colsum_b; p.strideC = d->stride_c;
  p.M = d->m; p.N = d->n; p.K = d->k; p.batch = d->batch;
  p.offsetA = d->offset_a; p.offsetB = d->offset_b;
  p.colsumExact = d->colsum_b_is_exact ? 1 : 0;
  if (allRange) { p.minA = d->min_a; p.maxA = d->max_a; p.minB = d->min_b; p.maxB = d->max_b; p.minC = d->min_c; p.maxC = d->max_c; }
  return TFCC_ROCM_OK;
}

}  // namespace
}  // namespace tfcc_rocm

using namespace tfcc_rocm;

extern "C" int tfcc_rocm_gemm_u8s8s32(void* stream, const tfcc_rocm_qgemm_desc* desc, int32_t* c) {
  QGemmParams p;
  if (int e = fill_params(desc, p)) return e;
  TFCC_REQUIRE(c != nullptr, "quantized matmul: null result");
  p.C = c;
  // decode shapes: a few rows against a large B are bandwidth bound and take the skinny kernel, on the
  // packed copy of B when the caller has one
  if (desc->packed_b && p.batch == 1 && gemv_packed_supported(p.A, desc->packed_b, p.M, p.K)) {
    const float* ranges[4] = {p.minA, p.maxA, p.minB, p.maxB};
    float* rangeOut[2] = {p.minC, p.maxC};
    return gemv_packed_launch(as_stream(stream), p.A, desc->packed_b, p.rowsumA, p.colsumB, p.offsetA, p.offsetB,
                              ranges, rangeOut, p.M, p.N, p.K, c, 0.f, nullptr, nullptr);
  }
  if (p.batch == 1 && p.M <= 8 && (unsigned long long)p.N * p.K >= (1u << 20) && gemv_supported(p.A, p.B, p.M, p.N, p.K)) {
    const float* ranges[4] = {p.minA, p.maxA, p.minB, p.maxB};
    float* rangeOut[2] = {p.minC, p.maxC};
    return gemv_launch(as_stream(stream), p.A, p.B, p.rowsumA, p.colsumB, p.offsetA, p.offsetB, ranges, rangeOut,
                       p.M, p.N, p.K, c, 0.f, nullptr, nullptr, p.colsumExact != 0);
  }
  return dispatch<false>(as_stream(stream), p);
}

extern "C" int tfcc_rocm_gemm_u8s8s32_requant_u8(void* stream, const tfcc_rocm_qgemm_desc* desc,
                                                 int32_t* acc_out, uint8_t* q_out, double in_scale,
                                                 double in_min, double out_scale, int64_t out_offset,
                                                 const float* min_out, const float* max_out) {
  QGemmParams p;
  if (int e = fill_params(desc, p)) return e;
  TFCC_REQUIRE(q_out != nullptr, "quantized matmul: null requantized result");
  TFCC_REQUIRE((min_out == nullptr) == (max_out == nullptr), "quantized matmul: give both output range pointers or none");
  TFCC_REQUIRE(min_out == nullptr || p.minA != nullptr,
               "quantized matmul: an output range in device memory needs the operand ranges in the descriptor");
  p.C = acc_out;
  p.Q = q_out;
  p.inScale = in_scale; p.inMin = in_min; p.outScale = out_scale; p.outOffset = out_offset;
  p.minOut = min_out; p.maxOut = max_out;
  return dispatch<true>(as_stream(stream), p);
}
