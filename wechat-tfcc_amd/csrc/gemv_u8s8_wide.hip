// Skinny (M <= 8) uint8 x int8 -> int32 product on a row-major B, split over K as well as over N.
//
// Same arithmetic as gemv_u8s8.hip (tfcc/mkl/operations/tfcc_mklquantization.cpp:33-69,176-201; the reference
// has no kernel of its own for this shape).  What differs is how B [K, N] is walked.  A kernel that owns a
// column group over the whole of K reads 64-byte pieces of rows that lie N bytes apart and has only N / 64
// workgroups; here a wavefront reads 64 rows x 256 columns per step, as sixteen 128-bit loads per lane that
// cover four 256-byte row pieces each, and a workgroup owns 256 columns over one part of K.
//
// Per step a lane holds 16 rows x 16 columns of B as bytes and needs, for each of its 16 columns, the 16 rows
// in one register quad (the B operand of v_mfma_i32_16x16x64_i8): sixteen 4 x 4 byte transposes with
// v_perm_b32.  Matrix op c of a step multiplies the c-th column of every lane, i.e. columns 16 j + c.  The A
// operand holds the rows of A (uint8 -> int8 by an xor, corrected with 128 x the column sums of B) padded to MR
// rows (1, 4 or 8: a kernel per padding, so that nothing is done for rows that are not there), and a row of ones
// right after them that yields those column sums, unless the caller has vouched for colsum_b (EXACT): then that
// row, its LDS traffic and its sums are left out.
//
// Two shapes of workgroup:
//   gemv_wide16_kernel  sixteen wavefronts, one step each: every byte of B the launch reads is asked for in the
//                       first microsecond (a decode-sized B is bound by how many bytes are in flight).  The
//                       wavefronts meet in an LDS tile through 64-bit adds that carry two rows each: the matrix op
//                       starts from a bias instead of zero, so every partial sum is non-negative and the low row
//                       never carries into the high one.
//   gemv_wide_kernel    four wavefronts of several steps with the loads of two steps in flight, for products so
//                       large that sixteen-wavefront workgroups of one step would be more than the chip holds at
//                       once: accumulators carry the sums from step to step and the wavefronts meet once, through
//                       a slot each in LDS (plain stores, nothing to clear).
//
// The parts of K of a column block are added up across workgroups: int32 sums do not depend on the order, so this
// costs no determinism.  A thread adds its elements to a tile in a workspace with 64-bit atomics that carry an
// arrival count next to the sums; the value an atomic returns tells the thread whether its addition was the last
// one, and if so it has the whole sum (what came back plus its own), puts the workspace word back to zero for the
// next launch, applies the offset terms and the optional per-channel dequantize and writes the elements.  One trip
// to memory and back, no fences; elements of one tile may be finished by different workgroups.  Two rows share a
// word when the partial sums are small enough to be made non-negative and added without a carry from one field into
// the next: [count 6 | row 2p+1: 29 | row 2p: 29]; otherwise a word holds [sum 32 | count 32].
#include <mutex>

#include "common.hpp"
#include "gemv.hpp"
#include "gemv_workspace.hpp"

namespace tfcc_rocm {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));

namespace {

constexpr int kCols = 256;     // columns per workgroup
constexpr int kMaxM = 8;
constexpr unsigned kMaxStaticN = 32768;  // widest B the workspace inside the library serves
constexpr unsigned kMaxStaticBlocks = kMaxStaticN / kCols;
constexpr unsigned long long kPackMask = (1ull << 29) - 1;
constexpr int kDefaultWaves = 16;               // wavefronts per workgroup
constexpr unsigned kDefaultStepsPerWave = 1;    // 64-row steps per wavefront

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
  unsigned packBias;          // two rows per workspace word, each partial sum made non-negative by this; 0: a word per row
  unsigned long long* tiles;  // [colBlocks][8][256] words, all zero between launches
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

// Rows r0 .. r0 + RPT - 1 of column egn (ec within the block) of this workgroup's partial tile, in sum[]: joins them
// with the other parts of K through the workspace and, for the elements this thread completes, applies the offset
// terms and writes the results.
template <int RPT, bool EXACT>
__device__ __forceinline__ void join_and_store(const GemvWideParams& p, unsigned kParts, unsigned cb, unsigned ec,
                                               unsigned egn, int r0, unsigned (&sum)[RPT], const int (&eRowsum)[RPT],
                                               int eColsum, float eScale, int oA, int oB) {
  const unsigned M = p.M, N = p.N, K = p.K;
  const unsigned offA = (unsigned)oA, offB = (unsigned)oB;
  // with the caller's word for colsum_b the correction for the uint8 of A comes from it, once per element
  const unsigned global = offA * offB * K + (EXACT ? 128u * (unsigned)eColsum : 0u);
  bool done[RPT];
#pragma unroll
  for (int t = 0; t < RPT; ++t) done[t] = true;
  if (kParts > 1) {
    unsigned long long* ws = p.tiles + (size_t)cb * (kMaxM * kCols);
    // Device scope: the parts of a column block may run anywhere on the chip.
    if (p.packBias) {
      const unsigned kPackBias = p.packBias;
      constexpr int PAIRS = (RPT + 1) / 2;
      // word of pair q: rows (r0 + 2q, r0 + 2q + 1); a thread with a single row has the word of that row to itself
      auto word = [&](int q) { return ws + (size_t)(RPT >= 2 ? r0 / 2 + q : r0) * kCols + ec; };
      unsigned long long mine[PAIRS], before[PAIRS];
#pragma unroll
      for (int q = 0; q < PAIRS; ++q) {
        const unsigned lo = sum[2 * q] + kPackBias, hi = (2 * q + 1 < RPT) ? sum[2 * q + 1] + kPackBias : 0u;
        mine[q] = (unsigned long long)lo | ((unsigned long long)hi << 29) | (1ull << 58);
        before[q] = __hip_atomic_fetch_add(word(q), mine[q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
#pragma unroll
      for (int q = 0; q < PAIRS; ++q) {
        const bool last = (unsigned)(before[q] >> 58) == kParts - 1;
        if (last) {
          __hip_atomic_store(word(q), 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          const unsigned long long total = before[q] + mine[q];
          sum[2 * q] = (unsigned)(total & kPackMask) - kParts * kPackBias;
          if (2 * q + 1 < RPT) sum[2 * q + 1] = (unsigned)((total >> 29) & kPackMask) - kParts * kPackBias;
        }
        done[2 * q] = last;
        if (2 * q + 1 < RPT) done[2 * q + 1] = last;
      }
    } else {
      unsigned long long before[RPT];
#pragma unroll
      for (int t = 0; t < RPT; ++t)
        before[t] = __hip_atomic_fetch_add(ws + (size_t)(r0 + t) * kCols + ec, ((unsigned long long)sum[t] << 32) | 1ull,
                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
      for (int t = 0; t < RPT; ++t) {
        done[t] = (unsigned)before[t] == kParts - 1;
        if (done[t]) {
          __hip_atomic_store(ws + (size_t)(r0 + t) * kCols + ec, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          sum[t] += (unsigned)(before[t] >> 32);
        }
      }
    }
  }
#pragma unroll
  for (int t = 0; t < RPT; ++t) {
    const unsigned r = r0 + t;
    if (!done[t] || r >= M) continue;
    const unsigned v = sum[t] + global + (unsigned)eRowsum[t] * offB + (unsigned)eColsum * offA;
    if (p.accOut) p.accOut[(size_t)r * N + egn] = (int)v;
    if (p.f32Out) p.f32Out[(size_t)r * N + egn] = (float)((double)(int)v * ((double)p.scaleA * (double)eScale));
  }
}

// ---- sixteen wavefronts, one step each.
// The LDS tile holds pairs of rows as 64-bit words.  Rows 2q and 2q + 1 of A are rows 4q and 4q + 1 of the matrix
// op's A operand, so that lane group q of the result (lanes 16q .. 16q + 15 hold output rows 4q .. 4q + 3) has pair q in
// its first two registers and ONE 64-bit add per matrix op takes all pairs of rows to the tile; the row of ones sits
// where the first free first-register slot is (output row 4 MR/2 for MR <= 4, output row 2 for MR = 8, which lane group
// 0 adds with a second instruction), as the low half of pair MR/2.  Column 16 j + c of the block lives at word
// c * 16 + j of its pair row, so that the 16 lanes of one matrix op that hold one pair add to 16 neighbouring words;
// pair rows are 2176 bytes apart, which puts neighbouring pairs half the banks apart.
constexpr int kPairPitch = kCols + 16;  // 64-bit words
constexpr unsigned kTileBias = 1u << 21;  // one step of 64 rows sums to less than 2^20 in absolute value
template <int MR, bool EXACT>
struct Tile16 {
  static constexpr int kRows = MR + (EXACT ? 0 : 1);  // rows of the matrix op's output that are kept
  static constexpr int kPairs = (kRows + 1) / 2;
  static constexpr int kWords = kPairs * kPairPitch;
};

// The arguments a wavefront needs before it can ask for its first bytes come first and one by one: the build
// passes -amdgpu-kernarg-preload-count, which has the first arguments of a kernel (scalars and pointers, up to the
// free user SGPRs) delivered in registers at wavefront start instead of fetched from the argument block, a round trip
// of about 0.6 us at the head of a 12 us kernel.  The argument block still carries everything.
template <int MR, bool EXACT>
__global__ __launch_bounds__(1024) void gemv_wide16_kernel(const signed char* hotB, const unsigned char* hotA,
                                                           unsigned hotM, unsigned hotN, unsigned hotK,
                                                           unsigned hotColBlocks, unsigned hotKParts, unsigned hotChunk,
                                                           const GemvWideParams p) {
  static_assert(MR == 1 || MR == 4 || MR == 8, "rows of A are padded to 1, 4 or 8");
  constexpr int kWaves = 16, kThreads = kWaves * 64;
  using Tile = Tile16<MR, EXACT>;
  __shared__ unsigned long long tile[Tile::kWords];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Consecutive workgroup ids go to different XCDs: each XCD gets a contiguous run of (column block, part) pairs,
  // so that the parts of a block mostly meet on one XCD and every XCD has the same number of pairs to within one
  // (measured: 1.1 us faster than handing the pairs out in the order of the ids).
  const unsigned L = (blockIdx.x & 7u) * hotChunk + (blockIdx.x >> 3);
  if ((blockIdx.x >> 3) >= hotChunk || L >= hotColBlocks * hotKParts) return;
  const unsigned cb = L / hotKParts, part = L - cb * hotKParts;
  const unsigned n0 = cb * kCols;
  const unsigned M = hotM, N = hotN, K = hotK;
  const int j = lane & 15, kg = lane >> 4;

  const __amdgpu_buffer_rsrc_t rsrcB =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<signed char*>(hotB), 0, (int)(K * N), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrcA =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(hotA), 0, (int)(M * K), 0x00020000);

  // What the end of the kernel needs from memory is asked for now: column tid % 256 and the rows this thread
  // finishes, so that the only wait left there is the atomic's own.
  constexpr int RPT = MR >= 2 ? 2 : 1;  // rows per thread in the last phase: a pair shares a workspace word
  const unsigned ec = tid % kCols, egn = n0 + ec;
  const int r0 = (tid / kCols) * RPT;   // four threads per column, as many of them as there are pairs of rows
  const bool finisher = r0 < MR && egn < N;
  int eColsum = 0, eRowsum[RPT] = {};
  float eScale = 0.f;
  if (finisher) {
    eColsum = p.colsumB[egn];
    if (p.f32Out) eScale = p.scaleB[egn];
#pragma unroll
    for (int t = 0; t < RPT; ++t)
      if ((unsigned)(r0 + t) < M) eRowsum[t] = p.rowsumA[r0 + t];
  }
  float mnA = 0.f, mxA = 0.f, mnB = 0.f, mxB = 0.f;  // ranges in device memory override the immediate offsets
  if (p.minA) { mnA = *p.minA; mxA = *p.maxA; mnB = *p.minB; mxB = *p.maxB; }

  // columns past N: a lane whose 16 columns lie outside reads nothing (N is a multiple of 16)
  const bool colsInside = n0 + 16u * j < N;
  const unsigned steps = (K + 63) / 64;
  const unsigned step = part * kWaves + wave;
  const unsigned k0 = step * 64 + kg * 16;  // this lane's 16 rows
  // The tile is cleared behind a barrier that waits for this wavefront's LDS stores only (the compiler puts no wait
  // for outstanding loads in front of a barrier on this target), so the loads of B may already be on their way:
  // 0.15-0.3 us faster for M = 1 and 4 when the kernel forms the column sums itself, 0.4 us slower when it does not
  // (measured, M = 1 / 4 / 8: 10.56 / 11.47 / 12.09 against 10.71 / 11.60 / 12.07 us, and with the sums given 11.13 /
  // 12.05 / 12.00 against 10.74 / 11.56 / 11.55).
  constexpr bool kLoadsFirst = !EXACT;
  auto clearTile = [&]() {
    for (int i = tid; i < Tile::kWords; i += kThreads) tile[i] = 0;
    __syncthreads();
  };
  if constexpr (!kLoadsFirst) clearTile();
  // the 16 rows x 16 columns of this lane (a step or rows past the end read zeros) and its 16 bytes of row j of A
  v4i raw[16];
  // lane j supplies row j of the matrix op's A operand: rows 4q and 4q + 1 are rows 2q and 2q + 1 of A
  const unsigned aRow = (j & 3) < 2 ? 2u * (j >> 2) + (j & 3) : 0xffffffffu;
  constexpr int kOnesRow = MR == 8 ? 2 : MR == 4 ? 8 : 1;  // the operand row that holds ones (column sums)
  const v4i aRaw = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(
                                               rsrcA, (aRow < M && k0 < K) ? aRow * K + k0 : 0xfffffff0u, 0, 0));
  {
    const bool live = colsInside && step < steps;
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const unsigned off = live ? (k0 + q) * N + n0 + 16u * j : 0xfffffff0u;
      raw[q] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrcB, off, 0, 0));
    }
  }
  if constexpr (kLoadsFirst) clearTile();
  // A operand: rows 0..M-1 of A (uint8 -> int8 by the xor), zeros, ones in row MR
  v4i a = {0, 0, 0, 0};
  if (aRow < M) {
    if (k0 < K) a = aRaw ^ (int)0x80808080;  // past K the operand stays zero (the xor would make it -128)
  } else if (!EXACT && j == kOnesRow) {
    a = v4i{0x01010101, 0x01010101, 0x01010101, 0x01010101};
  }
  // The offsets that ranges in device memory stand for (two divisions in double precision) are worked out here, with
  // the loads of B under way, not behind the barrier in front of the finish; the ranges were asked for before B, so
  // waiting for them waits for nothing else.
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
  const v4i bias = {(int)kTileBias, (int)kTileBias, (int)kTileBias, (int)kTileBias};
  // what this lane adds to the tile: registers 0, 1 of its result are pair kg of A's rows (for MR = 1 the second one
  // is the column sums, for MR = 4 lane group 2 holds them in register 0); for MR = 8 lane group 0 holds the column
  // sums in register 2 and adds them as pair 4
  const bool addRows = kg < (MR + 1) / 2 || (!EXACT && MR == 4 && kg == 2);
  const bool addSums = !EXACT && MR == 8 && kg == 0;
  // Transposes row quad by row quad, in the order the loads return: every byte of the launch was asked for at its
  // start, so a wavefront's loads come back spread over most of the kernel's life, and all that is left to do when
  // the last four rows arrive is a quarter of the transposes and the matrix ops.  (A row quad's registers are free
  // again once it is transposed, so the transposed copy needs no registers of its own.)
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
      const v4i d = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, bv, bias, 0, 0, 0);
      // lane (j, kg) holds rows 4 kg + r of output column 16 j + 4 w + e, each at least 2^20: two rows per add
      const int slot = (4 * w + e) * 16 + j;
      if (addRows)
        atomicAdd(&tile[kg * kPairPitch + slot], (unsigned long long)(unsigned)d[0] | ((unsigned long long)(unsigned)d[1] << 32));
      if (addSums)
        atomicAdd(&tile[4 * kPairPitch + slot], (unsigned long long)(unsigned)d[2] | ((unsigned long long)(unsigned)d[3] << 32));
    }
  }
  __syncthreads();

  if (!finisher) return;
  // ---- this thread's rows r0 .. r0 + RPT - 1 of column ec: every one of the sixteen wavefronts added its bias
  unsigned sum[RPT];
  {
    const int slot = (ec & 15) * 16 + (ec >> 4);
    constexpr unsigned kAllBias = kWaves * kTileBias;
    auto field = [&](int row) {
      const unsigned long long word = tile[(row >> 1) * kPairPitch + slot];
      return (unsigned)(row & 1 ? word >> 32 : word) - kAllBias;
    };
    const unsigned correction = EXACT ? 0u : 128u * field(MR);
#pragma unroll
    for (int t = 0; t < RPT; ++t) sum[t] = field(r0 + t) + correction;
  }
  // What was asked for at the start is first looked at here: without this the compiler forms the product of the two
  // scales right behind the load of this column's scale, and the wait for that load, the first of the kernel, would
  // stand in front of the loads of B (M = 4 and 8; a microsecond).
  asm volatile("" : "+v"(eScale), "+v"(eColsum));
#pragma unroll
  for (int t = 0; t < RPT; ++t) asm volatile("" : "+v"(eRowsum[t]));
  join_and_store<RPT, EXACT>(p, hotKParts, cb, ec, egn, r0, sum, eRowsum, eColsum, eScale, oA, oB);
}

// ---- four wavefronts of several steps.
// LDS slot of one wavefront: the row quads [quad][j][c ^ j] as 16-byte entries (a matrix op's 16 lanes of one quad
// write 16 different bank groups, and so do the 16 threads that later read neighbouring columns of one j), then the
// column sums as words [j][c ^ j].  MR = 1 keeps its single row as words like the column sums.
template <int MR, bool EXACT>
struct SlotLayout {
  static constexpr int kQuads = MR == 8 ? 2 : 1;
  static constexpr int kRowBytes = MR == 1 ? kCols * 4 : kQuads * kCols * 16;
  static constexpr int kBytes = kRowBytes + (EXACT ? 0 : kCols * 4);
};

template <int MR, bool EXACT>
__global__ __launch_bounds__(256) void gemv_wide_kernel(const signed char* hotB, const unsigned char* hotA,
                                                        unsigned hotM, unsigned hotN, unsigned hotK,
                                                        unsigned hotColBlocks, unsigned hotKParts,
                                                        unsigned hotStepsPerWave, unsigned hotChunk,
                                                        const GemvWideParams p) {
  static_assert(MR == 1 || MR == 4 || MR == 8, "rows of A are padded to 1, 4 or 8");
  constexpr int WAVES = 4, kThreads = WAVES * 64;
  using Slot = SlotLayout<MR, EXACT>;
  __shared__ __align__(16) unsigned char slots[WAVES * Slot::kBytes];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const unsigned L = (blockIdx.x & 7u) * hotChunk + (blockIdx.x >> 3);
  if ((blockIdx.x >> 3) >= hotChunk || L >= hotColBlocks * hotKParts) return;
  const unsigned cb = L / hotKParts, part = L - cb * hotKParts;
  const unsigned n0 = cb * kCols;
  const unsigned M = hotM, N = hotN, K = hotK;
  const int j = lane & 15, kg = lane >> 4;

  const __amdgpu_buffer_rsrc_t rsrcB =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<signed char*>(hotB), 0, (int)(K * N), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrcA =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(hotA), 0, (int)(M * K), 0x00020000);

  const bool colsInside = n0 + 16u * j < N;
  const unsigned steps = (K + 63) / 64;
  const unsigned S = hotStepsPerWave;
  const unsigned firstStep = (part * WAVES + wave) * S;
  v4i raw[2][16], aRaw[2];
  auto issueLoads = [&](unsigned step, int buf) {
    const unsigned k0 = step * 64 + kg * 16;
    aRaw[buf] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(
                                            rsrcA, ((unsigned)j < M && k0 < K) ? (unsigned)j * K + k0 : 0xfffffff0u, 0, 0));
    const bool live = colsInside && step < steps;
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const unsigned off = live ? (k0 + q) * N + n0 + 16u * j : 0xfffffff0u;
      raw[buf][q] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrcB, off, 0, 0));
    }
  };
  issueLoads(firstStep, 0);
  if (S > 1) issueLoads(firstStep + 1, 1);

  // one thread per column finishes the tile: all MR rows of column tid
  constexpr int RPT = MR;
  const unsigned ec = tid, egn = n0 + ec;
  const bool finisher = egn < N;
  int eColsum = 0, eRowsum[RPT] = {};
  float eScale = 0.f;
  if (finisher) {
    eColsum = p.colsumB[egn];
    if (p.f32Out) eScale = p.scaleB[egn];
#pragma unroll
    for (int t = 0; t < RPT; ++t)
      if ((unsigned)t < M) eRowsum[t] = p.rowsumA[t];
  }
  float mnA = 0.f, mxA = 0.f, mnB = 0.f, mxB = 0.f;
  if (p.minA) { mnA = *p.minA; mxA = *p.maxA; mnB = *p.minB; mxB = *p.maxB; }

  v4i acc[16];
#pragma unroll
  for (int c = 0; c < 16; ++c) acc[c] = v4i{0, 0, 0, 0};

  // one step: transposes row quad by row quad (in the order the loads return), then the sixteen matrix ops
  auto compute = [&](unsigned step, int buf) {
    const unsigned k0 = step * 64 + kg * 16;
    v4i a = {0, 0, 0, 0};
    if ((unsigned)j < M) {
      if (k0 < K) a = aRaw[buf] ^ (int)0x80808080;
    } else if (!EXACT && j == MR) {
      a = v4i{0x01010101, 0x01010101, 0x01010101, 0x01010101};
    }
    unsigned col[4][4][4];  // [column quad w][column e of the quad][row quad t]
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const unsigned r4[4] = {(unsigned)raw[buf][4 * t][w], (unsigned)raw[buf][4 * t + 1][w],
                                (unsigned)raw[buf][4 * t + 2][w], (unsigned)raw[buf][4 * t + 3][w]};
        unsigned c4[4];
        transpose4x4(r4, c4);
#pragma unroll
        for (int e = 0; e < 4; ++e) col[w][e][t] = c4[e];
      }
#pragma unroll
    for (int w = 0; w < 4; ++w)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const v4i bv = {(int)col[w][e][0], (int)col[w][e][1], (int)col[w][e][2], (int)col[w][e][3]};
        acc[4 * w + e] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, bv, acc[4 * w + e], 0, 0, 0);
      }
  };
  for (unsigned s = 0; s < S; s += 2) {
    // (steps past the end of K read zeros and add nothing; S is the same for every wavefront)
    compute(firstStep + s, 0);
    if (s + 2 < S) issueLoads(firstStep + s + 2, 0);
    if (s + 1 < S) {
      compute(firstStep + s + 1, 1);
      if (s + 3 < S) issueLoads(firstStep + s + 3, 1);
    }
  }
  // ---- the wavefront's partial tile into its slot.  Lane (j, kg) holds rows 4 kg + r of column 16 j + c in acc[c][r].
  {
    unsigned char* slot = slots + wave * Slot::kBytes;
    constexpr int kgSum = MR / 4, rSum = MR % 4;  // where the row of ones put the column sums
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      const int sw = c ^ j;
      if constexpr (MR == 1) {
        if (kg == 0) reinterpret_cast<int*>(slot)[j * 16 + sw] = acc[c][0];
      } else {
        if (kg < Slot::kQuads) reinterpret_cast<v4i*>(slot)[(kg * 16 + j) * 16 + sw] = acc[c];
      }
      if constexpr (!EXACT) {
        if (kg == kgSum) reinterpret_cast<int*>(slot + Slot::kRowBytes)[j * 16 + sw] = acc[c][rSum];
      }
    }
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
  if (!finisher) return;
  unsigned sum[RPT];
  {
    const int ej = ec >> 4, esw = (ec & 15) ^ ej;
    int rows[RPT] = {};
    int csum = 0;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      const unsigned char* slot = slots + w * Slot::kBytes;
      if constexpr (MR == 1) {
        rows[0] += reinterpret_cast<const int*>(slot)[ej * 16 + esw];
      } else {
#pragma unroll
        for (int q = 0; q < Slot::kQuads; ++q) {
          const v4i v = reinterpret_cast<const v4i*>(slot)[(q * 16 + ej) * 16 + esw];
#pragma unroll
          for (int e = 0; e < 4; ++e) rows[4 * q + e] += v[e];
        }
      }
      if constexpr (!EXACT) csum += reinterpret_cast<const int*>(slot + Slot::kRowBytes)[ej * 16 + esw];
    }
#pragma unroll
    for (int t = 0; t < RPT; ++t) sum[t] = (unsigned)rows[t] + (EXACT ? 0u : 128u * (unsigned)csum);
  }
  // What was asked for at the start is first looked at here: without this the compiler forms the product of the two
  // scales right behind the load of this column's scale, and the wait for that load, the first of the kernel, would
  // stand in front of the loads of B (M = 4 and 8; a microsecond).
  asm volatile("" : "+v"(eScale), "+v"(eColsum));
#pragma unroll
  for (int t = 0; t < RPT; ++t) asm volatile("" : "+v"(eRowsum[t]));
  join_and_store<RPT, EXACT>(p, hotKParts, cb, ec, egn, 0, sum, eRowsum, eColsum, eScale, oA, oB);
}

// ---- workspaces.  The ordinary entry points use one per (device, stream), allocated on first use and kept
// (gemv_workspace.hpp has the rules): launches on one stream run in order, so they can share it; launches on
// different streams may overlap.
gemv_ws::Registry gWorkspaces;

unsigned long long workspace_key(int dev, hipStream_t stream) {
  return ((unsigned long long)(unsigned)dev << 56) ^ (unsigned long long)(uintptr_t)stream;
}
int workspace_alloc(void** mem, size_t bytes) {
  if (hipMalloc(mem, bytes) != hipSuccess) return TFCC_ROCM_OUT_OF_MEMORY;
  if (hipMemset(*mem, 0, bytes) != hipSuccess) {
    (void)hipFree(*mem);
    return TFCC_ROCM_HIP_ERROR;
  }
  return 0;
}
void workspace_free(void* mem) { (void)hipFree(mem); }

__global__ void clear_words_kernel(unsigned long long* words, size_t count) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) words[i] = 0;
}

// The address of `scratch` on the current device, looked up once per device.
int static_workspace(unsigned long long** out) {
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
  *out = base[dev];
  return TFCC_ROCM_OK;
}

template <bool SIXTEEN, int MR, bool EXACT>
int launch_wide(hipStream_t stream, const GemvWideParams& p) {
  if (SIXTEEN) {
    hipLaunchKernelGGL((gemv_wide16_kernel<MR, EXACT>), dim3(p.chunk * 8), dim3(1024), 0, stream, p.B, p.A, p.M, p.N, p.K,
                       p.colBlocks, p.kParts, p.chunk, p);
  } else {
    hipLaunchKernelGGL((gemv_wide_kernel<MR, EXACT>), dim3(p.chunk * 8), dim3(256), 0, stream, p.B, p.A, p.M, p.N, p.K,
                       p.colBlocks, p.kParts, p.stepsPerWave, p.chunk, p);
  }
  return check_launch("skinny quantized matmul (split over K)");
}

template <bool SIXTEEN>
int launch_wide_rows(hipStream_t stream, const GemvWideParams& p, bool exact) {
  if (p.M == 1) return exact ? launch_wide<SIXTEEN, 1, true>(stream, p) : launch_wide<SIXTEEN, 1, false>(stream, p);
  if (p.M <= 4) return exact ? launch_wide<SIXTEEN, 4, true>(stream, p) : launch_wide<SIXTEEN, 4, false>(stream, p);
  return exact ? launch_wide<SIXTEEN, 8, true>(stream, p) : launch_wide<SIXTEEN, 8, false>(stream, p);
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

int gemv_wide_release_stream(hipStream_t stream) {
  int dev = 0;
  TFCC_HIP_CHECK(hipGetDevice(&dev));
  gWorkspaces.release(workspace_key(dev, stream), workspace_free);
  return TFCC_ROCM_OK;
}

int gemv_wide_launch(hipStream_t stream, bool staticWorkspace, const unsigned char* a, const signed char* b,
                     const int* rowsumA, const int* colsumB, int offsetA, int offsetB, const float* const ranges[4],
                     float* const rangeOut[2], unsigned m, unsigned n, unsigned k, int* accOut, float scaleA,
                     const float* scaleB, float* f32Out, bool colsumExact) {
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
  int waves = kDefaultWaves;
  unsigned spw = kDefaultStepsPerWave;
  // more steps per wavefront once the grid would exceed about four workgroups per CU (sixteen wavefronts make
  // one step each: a product that needs more goes to four wavefronts of several steps)
  if (waves == 16 && (spw != 1 || (unsigned long long)p.colBlocks * ((steps + 15) / 16) > 1024)) { waves = 4; spw = 4; }
  while ((unsigned long long)p.colBlocks * ((steps + waves * spw - 1) / (waves * spw)) > 1024 && spw < 64) spw *= 2;
  p.stepsPerWave = spw;
  p.kParts = (steps + waves * spw - 1) / (waves * spw);
  p.chunk = (p.colBlocks * p.kParts + 7) / 8;
  // Two rows per workspace word while the sum of the parts' biased partial sums stays inside a 29-bit field: a part
  // of R rows sums to at most R x 255 x 128 in absolute value, the bias is the next power of two, and a biased sum
  // is below twice the bias.
  {
    const unsigned long long bound = (unsigned long long)waves * spw * 64 * 32640ull;
    unsigned long long bias = 1;
    while (bias <= bound) bias <<= 1;
    p.packBias = (p.kParts < 64 && p.kParts * 2 * bias <= (1ull << 29)) ? (unsigned)bias : 0u;
  }
  unsigned long long key = 0;
  bool leased = false;
  if (staticWorkspace) {
    TFCC_REQUIRE(n <= kMaxStaticN, "skinny quantized matmul without allocation: n %u beyond the %u columns its workspace holds", n, kMaxStaticN);
    if (int e = static_workspace(&p.tiles)) return e;
  } else if (p.kParts > 1) {
    int dev = 0;
    TFCC_HIP_CHECK(hipGetDevice(&dev));
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    TFCC_HIP_CHECK(hipStreamIsCapturing(stream, &capture));
    key = workspace_key(dev, stream);
    gemv_ws::Lease lease;
    const int e = gWorkspaces.acquire(key, p.colBlocks, (size_t)kMaxM * kCols * sizeof(unsigned long long),
                                      capture == hipStreamCaptureStatusNone, workspace_alloc, &lease);
    if (e == gemv_ws::kWouldAllocate)
      // the stream is being recorded and has no workspace of this width yet: nothing may be allocated now, so this
      // launch goes to the kernel that needs none (same sums; slower on a decode-sized B).  A product of the same
      // width issued once before the recording, or the entry point without allocation, avoids this.
      return gemv_onepass_launch(stream, a, b, rowsumA, colsumB, offsetA, offsetB, ranges, rangeOut, m, n, k, accOut,
                                 scaleA, scaleB, f32Out);
    if (e == TFCC_ROCM_OUT_OF_MEMORY) return set_error(e, "skinny quantized matmul: no memory for the workspace");
    if (e) return set_error(e, "skinny quantized matmul: workspace set-up failed");
    p.tiles = static_cast<unsigned long long*>(lease.mem);
    leased = true;
    if (lease.mustClear) {  // a fill kernel, not a memset: this may be inside a recording
      hipLaunchKernelGGL(clear_words_kernel, dim3(256), dim3(256), 0, stream, p.tiles, lease.blocks * kMaxM * kCols);
      if (int ce = check_launch("workspace clear")) { gWorkspaces.mark_dirty(key); return ce; }
    }
  }
  int status;
  status = waves == 16 ? launch_wide_rows<true>(stream, p, colsumExact) : launch_wide_rows<false>(stream, p, colsumExact);
  if (status != TFCC_ROCM_OK && leased) gWorkspaces.mark_dirty(key);
  return status;
}

}  // namespace tfcc_rocm
