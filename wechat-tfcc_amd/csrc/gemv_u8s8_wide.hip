// Skinny (M <= 8) uint8 x int8 -> int32 product on a row-major B, split over K as well as over N.
//
// Same arithmetic as gemv_u8s8.hip (tfcc/mkl/operations/tfcc_mklquantization.cpp:33-69,176-201; the reference
// has no kernel of its own for this shape).  What differs is how B [K, N] is walked.  A kernel that owns a
// column group over the whole of K reads 64-byte pieces of rows that lie N bytes apart and has only N / 64
// workgroups; here a wavefront reads 64 rows x 256 columns in one go, as sixteen 128-bit loads per lane that
// cover four 256-byte row pieces each, and a workgroup of sixteen wavefronts owns 256 columns over one part of
// K.  The parts of K of a column block are added up across workgroups: int32 sums do not depend on the order,
// so this costs no determinism.  Every workgroup folds the correction for the uint8 of A into its partial sums
// (128 x its partial column sums of B: the correction is linear in B too) and adds them to a tile in a workspace
// with one 64-bit atomic per element: the sum in the upper half, a count of one in the lower.  The value the
// atomic returns tells a thread whether its addition was the last one for that element; if so it has the whole
// sum (what came back plus its own), puts the workspace word back to zero for the next launch, applies the
// offset terms and the optional per-channel dequantize and writes the element.  One trip to memory and back,
// no counters, no fences; elements of one tile may be finished by different workgroups.
//
// Per step a lane holds 16 rows x 16 columns of B as bytes and needs, for each of its 16 columns, the 16 rows
// in one register quad (the B operand of v_mfma_i32_16x16x64_i8): sixteen 4 x 4 byte transposes with
// v_perm_b32.  Matrix op c of a step multiplies the c-th column of every lane, i.e. columns 16 j + c.
#include <mutex>
#include <unordered_map>

#include "common.hpp"
#include "gemv.hpp"

namespace tfcc_rocm {

typedef int v4i __attribute__((ext_vector_type(4)));

namespace {

constexpr int kWaves = 16;
constexpr int kThreads = kWaves * 64;
constexpr int kCols = 256;     // columns per workgroup
constexpr int kMaxM = 8;
constexpr int kPartRows = 9;   // rows of a partial tile: 8 rows of A and the column sums of B
// The partial tile in LDS: column 16 j + c of the block lives at word c * 16 + j of its row, so that the 16 lanes
// of one matrix op that hold one row add to 16 neighbouring banks; rows are 260 words apart, which puts rows
// r, r + 4 and 8 (the three rows the lanes of one instruction touch) 16 banks apart: no two lanes of an
// instruction meet in a bank.
constexpr int kRowPitch = kCols + 4;
__device__ __forceinline__ int tile_slot(int row, int col) { return row * kRowPitch + (col & 15) * 16 + (col >> 4); }
constexpr unsigned kMaxStaticN = 32768;  // widest B the workspace inside the library serves
constexpr unsigned kMaxStaticBlocks = kMaxStaticN / kCols;

struct GemvWideParams {
  const unsigned char* A;
  const signed char* B;
  const int* rowsumA;
  const int* colsumB;
  int* accOut;
  float* f32Out;
  const float* scaleB;
  float scaleA;
  int offsetA, offsetB;
  const float *minA, *maxA, *minB, *maxB;  // optional ranges in device memory (override the offsets)
  float *minC, *maxC;
  unsigned M, N, K;
  unsigned colBlocks, kParts, stepsPerWave, chunk;
  unsigned long long* tiles;  // [colBlocks][8][256]: sum << 32 | arrivals, all zero between launches
};

// The workspace of the entry point that must not allocate: one per GPU, inside the library's image.
__device__ __align__(256) unsigned long long scratch[kMaxStaticBlocks * kMaxM * kCols];

__device__ __forceinline__ void transpose4x4(const unsigned r[4], unsigned c[4]) {
  unsigned t0 = __builtin_amdgcn_perm(r[1], r[0], 0x05010400u);
  unsigned t1 = __builtin_amdgcn_perm(r[1], r[0], 0x07030602u);
  unsigned t2 = __builtin_amdgcn_perm(r[3], r[2], 0x05010400u);
  unsigned t3 = __builtin_amdgcn_perm(r[3], r[2], 0x07030602u);
  c[0] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
  c[1] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
  c[2] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
  c[3] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
}

// The arguments a wavefront needs before it can ask for its first bytes come first and one by one: the build
// passes -amdgpu-kernarg-preload-count, which has the first arguments of a kernel (scalars and pointers, up to the
// free user SGPRs) delivered in registers at wavefront start instead of fetched from the argument block, a round trip
// of about 0.6 us at the head of a 12 us kernel.  The argument block still carries everything (hot.* repeats them).
struct GemvWideHot {
  const signed char* B;
  const unsigned char* A;
  unsigned M, N, K, colBlocks, kParts, stepsPerWave, chunk;
};
__global__ __launch_bounds__(kThreads) void gemv_wide_kernel(const signed char* hotB, const unsigned char* hotA,
                                                             unsigned hotM, unsigned hotN, unsigned hotK,
                                                             unsigned hotColBlocks, unsigned hotKParts,
                                                             unsigned hotStepsPerWave, unsigned hotChunk,
                                                             const GemvWideParams p) {
  __shared__ int tile[kPartRows * kRowPitch];
  const GemvWideHot hot = {hotB, hotA, hotM, hotN, hotK, hotColBlocks, hotKParts, hotStepsPerWave, hotChunk};

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Consecutive workgroup ids go to different XCDs: each XCD gets a contiguous run of (column block, part) pairs,
  // so that the parts of a block mostly meet on one XCD and every XCD has the same number of pairs to within one
  // (measured: 1.1 us faster than handing the pairs out in the order of the ids).
  const unsigned L = (blockIdx.x & 7u) * hot.chunk + (blockIdx.x >> 3);
  if ((blockIdx.x >> 3) >= hot.chunk || L >= hot.colBlocks * hot.kParts) return;
  const unsigned cb = L / hot.kParts, part = L - cb * hot.kParts;
  const unsigned n0 = cb * kCols;
  const unsigned M = hot.M, N = hot.N, K = hot.K;
  const int j = lane & 15, kg = lane >> 4;

  const __amdgpu_buffer_rsrc_t rsrcB =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<signed char*>(hot.B), 0, (int)(K * N), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrcA =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(hot.A), 0, (int)(M * K), 0x00020000);

  // What the end of the kernel needs from memory is asked for now: column tid % 256 of every row this thread
  // finishes (rows tid / 256 + kRowsPerPass t), so that the only wait left there is the atomic's own.
  static_assert(kThreads % kCols == 0 && kMaxM % (kThreads / kCols) == 0, "element ownership of the last phase");
  constexpr int kRowsPerPass = kThreads / kCols, kPasses = kMaxM / kRowsPerPass;
  const unsigned ec = tid % kCols, egn = n0 + ec, er0 = tid / kCols;
  int eColsum = 0, eRowsum[kPasses] = {};
  float eScale = 0.f;
  if (egn < N) {
    eColsum = p.colsumB[egn];
    if (p.f32Out) eScale = p.scaleB[egn];
#pragma unroll
    for (int t = 0; t < kPasses; ++t)
      if (er0 + kRowsPerPass * t < M) eRowsum[t] = p.rowsumA[er0 + kRowsPerPass * t];
  }
  float mnA = 0.f, mxA = 0.f, mnB = 0.f, mxB = 0.f;  // ranges in device memory override the immediate offsets
  if (p.minA) { mnA = *p.minA; mxA = *p.maxA; mnB = *p.minB; mxB = *p.maxB; }

  // columns past N: a lane whose 16 columns lie outside reads nothing (N is a multiple of 16)
  const bool colsInside = n0 + 16u * j < N;
  const unsigned steps = (K + 63) / 64;
  const unsigned firstStep = (part * kWaves + wave) * hot.stepsPerWave;
  v4i raw[16], aRaw;
  // the 16 rows x 16 columns of this lane in step `step` (steps and rows past the end read zeros) and its 16
  // bytes of row j of A
  auto issueLoads = [&](unsigned step) {
    const unsigned k0 = step * 64 + kg * 16;
    aRaw = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(
                                       rsrcA, ((unsigned)j < M && k0 < K) ? (unsigned)j * K + k0 : 0xfffffff0u, 0, 0));
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const unsigned off = (colsInside && step < steps) ? (k0 + q) * N + n0 + 16u * j : 0xfffffff0u;
      raw[q] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrcB, off, 0, 0));
    }
  };
  // (the tile is cleared before the loads are issued: a barrier waits for all of a wavefront's outstanding
  // memory operations, and with the loads ahead of it every wavefront would wait for the slowest one's data; a bare
  // s_barrier after a wait for the LDS stores alone, with the loads issued first, measured 0.6 us slower still)
  for (int i = tid; i < kPartRows * kRowPitch; i += kThreads) tile[i] = 0;
  __syncthreads();
  issueLoads(firstStep);
  for (unsigned s = 0; s < hot.stepsPerWave; ++s) {
    const unsigned step = firstStep + s;
    if (step >= steps) break;  // wave-uniform; no barrier inside this loop
    const unsigned k0 = step * 64 + kg * 16;  // this lane's 16 rows
    // A operand: rows 0..M-1 of A (uint8 -> int8 by the xor), zeros, ones in row 15
    v4i a = {0, 0, 0, 0};
    if ((unsigned)j < M) {
      if (k0 < K) a = aRaw ^ (int)0x80808080;  // past K the operand stays zero (the xor would make it -128)
    } else if (j == 15) {
      a = v4i{0x01010101, 0x01010101, 0x01010101, 0x01010101};
    }
#pragma unroll
    for (int w = 0; w < 4; ++w) {  // column quad w of this lane: columns 4w .. 4w+3
      unsigned col[4][4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {  // row quad t
        const unsigned r4[4] = {(unsigned)raw[4 * t][w], (unsigned)raw[4 * t + 1][w], (unsigned)raw[4 * t + 2][w],
                                (unsigned)raw[4 * t + 3][w]};
        unsigned c4[4];
        transpose4x4(r4, c4);
#pragma unroll
        for (int e = 0; e < 4; ++e) col[e][t] = c4[e];
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const v4i bv = {(int)col[e][0], (int)col[e][1], (int)col[e][2], (int)col[e][3]};
        const v4i d = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, bv, v4i{0, 0, 0, 0}, 0, 0, 0);
        // lane (j, kg) holds rows 4 kg + r of output column 16 j + 4 w + e: rows 0..7 in the lanes of kg 0 and 1,
        // the column sums (row 15, kept as row 8) in element 3 of the lanes of kg 3
        const int slot = (4 * w + e) * 16 + j;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if (kg < 2) atomicAdd(&tile[(4 * kg + r) * kRowPitch + slot], d[r]);
          else if (r == 3 && kg == 3) atomicAdd(&tile[kMaxM * kRowPitch + slot], d[3]);
        }
      }
    }
    if (s + 1 < hot.stepsPerWave) issueLoads(step + 1);
  }
  __syncthreads();

  int oA = p.offsetA, oB = p.offsetB;
  if (p.minA) {
    qmatmul_offsets(mnA, mxA, mnB, mxB, &oA, &oB);
    if (cb == 0 && part == 0 && tid == 0) {
      float mnC, mxC;
      qmatmul_range(mnA, mxA, mnB, mxB, &mnC, &mxC);
      if (p.minC) *p.minC = mnC;
      if (p.maxC) *p.maxC = mxC;
    }
  }
  const unsigned offA = (unsigned)oA, offB = (unsigned)oB;
  const unsigned global = offA * offB * K;
  unsigned long long* ws = p.tiles + (size_t)cb * (kMaxM * kCols);
#pragma unroll
  for (int t = 0; t < kPasses; ++t) {
    const unsigned r = er0 + kRowsPerPass * t, idx = r * kCols + ec;
    if (r >= M || egn >= N) continue;
    unsigned sum = (unsigned)tile[tile_slot(r, ec)] + 128u * (unsigned)tile[tile_slot(kMaxM, ec)];
    if (hot.kParts > 1) {
      // Device scope: the parts of a column block may run anywhere on the chip.  One element after the other: with
      // all of a thread's atomics under way at once the kernel measured 0.5 us slower.
      const unsigned long long before =
          __hip_atomic_fetch_add(ws + idx, ((unsigned long long)sum << 32) | 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if ((unsigned)before != hot.kParts - 1) continue;  // others are still to come: one of them finishes the element
      sum += (unsigned)(before >> 32);
      __hip_atomic_store(ws + idx, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const unsigned v = sum + global + (unsigned)eRowsum[t] * offB + (unsigned)eColsum * offA;
    if (p.accOut) p.accOut[(size_t)r * N + egn] = (int)v;
    if (p.f32Out) p.f32Out[(size_t)r * N + egn] = (float)((double)(int)v * ((double)p.scaleA * (double)eScale));
  }
}

// ---- workspaces.  The ordinary entry points use one per (device, stream), allocated on first use and kept:
// launches on one stream run in order, so they can share it; launches on different streams may overlap.
struct Workspace {
  unsigned long long* tiles = nullptr;
  unsigned blocks = 0;
};
std::mutex gWorkspaceMutex;
std::unordered_map<unsigned long long, Workspace> gWorkspaces;  // key: device and stream

int workspace_for(hipStream_t stream, unsigned blocks, Workspace* out) {
  int dev = 0;
  TFCC_HIP_CHECK(hipGetDevice(&dev));
  const unsigned long long key = ((unsigned long long)(unsigned)dev << 56) ^ (unsigned long long)(uintptr_t)stream;
  std::lock_guard<std::mutex> lock(gWorkspaceMutex);
  Workspace& w = gWorkspaces[key];
  if (w.blocks < blocks) {
    // the old one may still be in use by launches of this stream
    if (w.tiles) {
      TFCC_HIP_CHECK(hipStreamSynchronize(stream));
      TFCC_HIP_CHECK(hipFree(w.tiles));
      w = Workspace{};
    }
    const size_t bytes = (size_t)blocks * kMaxM * kCols * sizeof(unsigned long long);
    void* mem = nullptr;
    TFCC_HIP_CHECK(hipMalloc(&mem, bytes));
    TFCC_HIP_CHECK(hipMemset(mem, 0, bytes));
    w.tiles = static_cast<unsigned long long*>(mem);
    w.blocks = blocks;
  }
  *out = w;
  return TFCC_ROCM_OK;
}

// The address of `scratch` on the current device, looked up once per device.
int static_workspace(Workspace* out) {
  static unsigned long long* base[16] = {};
  static std::mutex m;
  int dev = 0;
  TFCC_HIP_CHECK(hipGetDevice(&dev));
  TFCC_REQUIRE(dev >= 0 && dev < 16, "device index %d", dev);
  std::lock_guard<std::mutex> lock(m);
  if (!base[dev]) {
    void* ptr = nullptr;
    TFCC_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    base[dev] = static_cast<unsigned long long*>(ptr);
  }
  out->tiles = base[dev];
  out->blocks = kMaxStaticBlocks;
  return TFCC_ROCM_OK;
}

}  // namespace

bool gemv_wide_supported(const void* a, const void* b, unsigned m, unsigned n, unsigned k) {
  return m >= 1 && m <= (unsigned)kMaxM && n % 16 == 0 && k % 16 == 0 && (uintptr_t)a % 16 == 0 &&
         (uintptr_t)b % 16 == 0 && (unsigned long long)k * n + 4096ull * n < (1ull << 32) &&
         (unsigned long long)m * k < (1ull << 31) &&
         // worth it from a few hundred wavefront steps on; below that the one-pass kernel's launch is all there is
         (unsigned long long)((k + 63) / 64) * ((n + kCols - 1) / kCols) >= 512;
}

unsigned gemv_wide_static_max_n() { return kMaxStaticN; }

int gemv_wide_launch(hipStream_t stream, bool staticWorkspace, const unsigned char* a, const signed char* b,
                     const int* rowsumA, const int* colsumB, int offsetA, int offsetB, const float* const ranges[4],
                     float* const rangeOut[2], unsigned m, unsigned n, unsigned k, int* accOut, float scaleA,
                     const float* scaleB, float* f32Out) {
  GemvWideParams p{};
  if (ranges && ranges[0]) {
    p.minA = ranges[0]; p.maxA = ranges[1]; p.minB = ranges[2]; p.maxB = ranges[3];
    if (rangeOut) { p.minC = rangeOut[0]; p.maxC = rangeOut[1]; }
  }
  p.A = a; p.B = b; p.rowsumA = rowsumA; p.colsumB = colsumB;
  p.accOut = accOut; p.f32Out = f32Out; p.scaleA = scaleA; p.scaleB = scaleB;
  p.offsetA = offsetA; p.offsetB = offsetB;
  p.M = m; p.N = n; p.K = k;
  p.colBlocks = (n + kCols - 1) / kCols;
  const unsigned steps = (k + 63) / 64;
  // one step per wavefront while that gives at most about four workgroups per CU, more steps beyond
  unsigned spw = 1;
  while ((unsigned long long)p.colBlocks * ((steps + kWaves * spw - 1) / (kWaves * spw)) > 1024 && spw < 64) spw *= 2;
  p.stepsPerWave = spw;
  p.kParts = (steps + kWaves * spw - 1) / (kWaves * spw);
  p.chunk = (p.colBlocks * p.kParts + 7) / 8;
  Workspace w;
  if (staticWorkspace) {
    TFCC_REQUIRE(n <= kMaxStaticN, "skinny quantized matmul without allocation: n %u beyond the %u columns its workspace holds", n, kMaxStaticN);
    if (int e = static_workspace(&w)) return e;
  } else if (p.kParts > 1) {
    if (int e = workspace_for(stream, p.colBlocks, &w)) return e;
  }
  p.tiles = w.tiles;
  hipLaunchKernelGGL(gemv_wide_kernel, dim3(p.chunk * 8), dim3(kThreads), 0, stream, p.B, p.A, p.M, p.N, p.K,
                     p.colBlocks, p.kParts, p.stepsPerWave, p.chunk, p);
  return check_launch("skinny quantized matmul (split over K)");
}

}  // namespace tfcc_rocm
