// Internal interface of the DMA-pipelined quantized matmul kernel (large aligned shapes).
#pragma once
#include <hip/hip_runtime.h>

#include "qgemm_params.hpp"

namespace tfcc_rocm {

// Alignment and size conditions of the kernel: K and N multiples of 16, 16-byte aligned operands.
bool qgemm_dma_supported(const QGemmParams& p, bool requant);
int qgemm_dma_launch(hipStream_t stream, const QGemmParams& p, bool requant);

// The same product with four wavefronts of 128 x 128 per 256 x 256 tile (gemm_u8s8_w4.hip), for launches of at
// least three quarters of a chip of such tiles; asks for K % 256 == 0 on top of qgemm_dma_supported.
bool qgemm_w4_supported(const QGemmParams& p);
int qgemm_w4_launch(hipStream_t stream, const QGemmParams& p, bool requant);

}  // namespace tfcc_rocm
