// Argument block shared by the fp32 GEMM kernels (register-staged in sgemm.hip, direct-to-LDS in
// sgemm_dma.hip) and the entry points that pick between them.
#pragma once

#include "common.hpp"
#include "qgemm_params.hpp"  // UDiv: division by multiply-high

namespace tfcc_rocm {
namespace sgemm_detail {

struct SgemmParams {
  const float* A;
  const float* B;
  const float* bias;
  const float* residual;  // optional, laid out like C (batch stride strideR): added after the bias
  float* C;
  unsigned long long strideA, strideB, strideC, strideR;  // between outer batch entries (elements)
  unsigned long long innerA, innerB, innerC;              // between inner batch entries
  unsigned batchInner;    // batch entry bi = (bi / batchInner, bi % batchInner); 1 for a flat batch
  unsigned lda, ldb, ldc; // row strides of A, of B (of B^T when transposed) and of C, in elements
  int act;                // 0 none, 1 erf-form GELU applied last
  // grouped form (groups > 0): batch entry g multiplies the shared A by groupB[g] into groupC[g]
  unsigned groups;
  const float* groupB[4];
  const float* groupBias[4];
  float* groupC[4];
  unsigned M, N, K, batch;
  unsigned tilesM, tilesN, tilesTotal, chunk;
  // division by tilesM * tilesN, by 4 * tilesN and by batchInner as multiply-high and shift (set_tiles)
  unsigned perBatchMagic, perBatchShift, bandMagic, bandShift, innerMagic, innerShift;
};

// Fills in the tile counts for BM x BN tiles; false when there are too many tiles for one grid.
inline bool set_tiles(SgemmParams& p, unsigned bm, unsigned bn) {
  p.tilesM = (p.M + bm - 1) / bm;
  p.tilesN = (p.N + bn - 1) / bn;
  const unsigned long long total = (unsigned long long)p.tilesM * p.tilesN * p.batch;
  if (total > 0x7fffffffull) return false;
  p.tilesTotal = (unsigned)total;
  p.chunk = (p.tilesTotal + 7) / 8;
  const UDiv perBatch = udiv_prepare(p.tilesM * p.tilesN), band = udiv_prepare(4u * p.tilesN),
             inner = udiv_prepare(p.batchInner);
  p.perBatchMagic = perBatch.magic; p.perBatchShift = perBatch.shift;
  p.bandMagic = band.magic; p.bandShift = band.shift;
  p.innerMagic = inner.magic; p.innerShift = inner.shift;
  return true;
}

// The direct-to-LDS kernels (sgemm_dma.hip).  `config`: 0 = 64x64 tiles, 1 = 32x96, 2 = 32x64, 3 = 32x32,
// 5 = 128x96 (serial groups only); ksplit 1 or 2 groups of wavefronts on one tile (four K groups run on the
// kernels of sgemm_wave96.hip).
// Requires 16-byte aligned operands and strides, K a multiple of 32 and B not transposed.
bool sgemm_dma_available(int config, int ksplit);
// serialGroups: one group of wavefronts per tile does the work of the `ksplit` groups one slab after the other
// (same additions, same result) - for launches that fill the chip anyway.
int sgemm_dma_launch(hipStream_t stream, SgemmParams p, int config, int ksplit, bool serialGroups);

// The hand-scheduled kernels with one wavefront per SIMD (sgemm_wave96.hip), a wavefront owning 32 rows x `blocks`
// column blocks of 32: ksplit = 4 - tiles of 32 x 32 blocks with the four K groups as the four wavefronts of a
// workgroup (blocks 1, 2 or 3), or 64 x 64 tiles with eight wavefronts (blocks 2, rowBlocks 2); ksplit = 2 - 64 x 64 tiles (blocks 2, rowBlocks 2: two pairs of wavefronts) or 32 x 32
// (blocks 1, rowBlocks 1: two wavefronts); ksplit = 1 - tiles of 128 x 32 blocks, four wavefronts on a shared ring
// (blocks 3 or 4).  Same requirements and the same bits as the kernels above for the same number of K groups.
int sgemm_wave96_launch(hipStream_t stream, SgemmParams p, int ksplit, int blocks = 3, int rowBlocks = 0);

// The streaming kernel for up to eight rows of A (sgemv.hip): any K, N, strides and alignment; B not transposed.
bool sgemv_supported(const SgemmParams& p);
int sgemv_launch(hipStream_t stream, const SgemmParams& p);

}  // namespace sgemm_detail
}  // namespace tfcc_rocm
