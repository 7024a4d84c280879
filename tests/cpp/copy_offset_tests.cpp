// Host-side proof that the HBM -> LDS copies of the kernels that keep a slab's offset in the copy's scalar offset
// never address memory outside their operand: for ragged shapes, every (lane offset, scalar offset) pair the kernels
// can issue is enumerated; a lane offset that passes the descriptor's range check (offset + 16 <= size) must stay
// inside the operand with every scalar offset added, and every element a tile needs must be covered exactly once.
// No GPU: the offset functions are the ones the kernels compile (wechat-tfcc_amd/csrc/copy_offsets.hpp).
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "copy_offsets.hpp"

using namespace tfcc_rocm::copy_offsets;

static int failures = 0;
#define EXPECT(cond, ...)                 \
  do {                                    \
    if (!(cond)) {                        \
      if (++failures < 20) {              \
        std::printf("FAIL %s: ", #cond);  \
        std::printf(__VA_ARGS__);         \
        std::printf("\n");                \
      }                                   \
    }                                     \
  } while (0)

// int8 kernel: 256 x 256 tiles, BK = 64, 256 threads, B copies per slab = 64 * 256 / 16 / 256 = 4, A copies 4
static void check_w4(unsigned M, unsigned N, unsigned K) {
  const unsigned BK = 64, KT = K / BK;
  const unsigned long long bytesA = (unsigned long long)M * K, bytesB = (unsigned long long)K * N;
  for (unsigned m0 = 0; m0 < M; m0 += 256)
    for (unsigned n0 = 0; n0 < N; n0 += 256) {
      std::vector<int> seen(64 * 256, 0);  // [k][column of the tile] of one slab
      for (int tid = 0; tid < 256; ++tid)
        for (int c = 0; c < 4; ++c) {
          const unsigned vb = w4_b_lane_offset(tid, c, n0, N);
          const bool passes = (unsigned long long)vb + 16 <= bytesB;
          for (unsigned slab = 0; slab < KT + 4; ++slab) {  // the ring asks for slabs past the end too
            const unsigned so = w4_b_slab_offset(slab, KT, BK, N);
            if (passes) EXPECT((unsigned long long)vb + so + 16 <= bytesB, "w4 B %ux%ux%u tile (%u,%u) tid %d c %d slab %u", M, N, K, m0, n0, tid, c, slab);
          }
          if (passes) {
            const unsigned k = vb / N, col = vb % N;
            EXPECT(k < 64 && col >= n0 && col < n0 + 256, "w4 B lane outside the tile");
            if (k < 64 && col >= n0 && col < n0 + 256) seen[k * 256 + (col - n0)]++;
          }
          const unsigned va = w4_a_lane_offset(tid, c, m0, K, (int)BK);
          if ((unsigned long long)va + 16 <= bytesA)
            EXPECT((unsigned long long)va + (KT - 1) * BK + 16 <= bytesA, "w4 A %ux%ux%u tile row %u tid %d c %d", M, N, K, m0, tid, c);
        }
      for (unsigned k = 0; k < 64; ++k)
        for (unsigned col = 0; col < 256 && n0 + col < N; col += 16)
          EXPECT(seen[k * 256 + col] == 1, "w4 B element (k %u, col %u) copied %d times", k, n0 + col, seen[k * 256 + col]);
    }
}

// fp32 kernel: tile of BN = 32 NI columns, ring slabs of BK k rows; B image slots of 16 bytes
static void check_w96(unsigned N, unsigned K, unsigned ldb, int NI, int BK) {
  const int BN = 32 * NI, BCH = BN / 4, slots = BK * BCH;
  const unsigned long long bytesB = ((unsigned long long)(K - 1) * ldb + N) * 4ull;
  for (unsigned n0 = 0; n0 < N; n0 += BN)
    for (int s = 0; s < slots; ++s) {
      const unsigned v = w96_b_lane_offset(s, BCH, n0, N, ldb);
      if ((unsigned long long)v + 16 > bytesB) continue;  // fails the range check: reads zeros
      for (unsigned k0 = 0; k0 + BK <= K; k0 += BK) {
        const unsigned long long so = (unsigned long long)k0 * ldb * 4ull;
        EXPECT(v + so + 16 <= bytesB, "w96 B N %u K %u ldb %u NI %d BK %d n0 %u slot %d k0 %u", N, K, ldb, NI, BK, n0, s, k0);
      }
    }
}

int main() {
  // the shapes the advisory named plus a spread of ragged ones (N a multiple of 16 for int8, of 4 for fp32)
  const unsigned shapesQ[][3] = {{4096, 4000, 4096}, {4096, 4096, 4096}, {3840, 3856, 512}, {4096, 16, 256}, {300, 4080, 1024}, {257, 272, 256}};
  for (auto& s : shapesQ) check_w4(s[0], s[1], s[2]);
  const unsigned shapesF[][3] = {{768, 1024, 768}, {100, 1024, 100}, {100, 1024, 132}, {3076, 2048, 3076}, {4, 32, 4}, {92, 64, 4096}, {260, 512, 260}};
  for (auto& s : shapesF)
    for (int NI = 1; NI <= 4; ++NI)
      for (int BK : {8, 16, 32}) check_w96(s[0], s[1], s[2], NI, BK);
  // the marker itself must fail the check of every operand size the kernels accept
  EXPECT((unsigned long long)kCopyOutOfRange + 16 > 0xffffffffull - 1024, "marker below the largest operand");
  EXPECT((unsigned long long)kCopyOutOfRange + 16 <= 0xffffffffull, "marker + 16 wraps");
  if (failures) {
    std::printf("%d failures\n", failures);
    return 1;
  }
  std::printf("copy offsets ok\n");
  return 0;
}
