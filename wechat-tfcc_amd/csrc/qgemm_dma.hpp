// Internal interface of the DMA-pipelined quantized matmul kernel (large aligned shapes).
#pragma once
#include <hip/hip_runtime.h>

#include "qgemm_params.hpp"

namespace tfcc_rocm {

// Alignment and size conditions of the kernel: K and N multiples of 16, 16-byte aligned operands.
bool qgemm_dma_supported(const QGemmParams& p, bool requant);
int qgemm_dma_launch(hipStream_t stream, const QGemmParams& p, bool requant);

}  // namespace tfcc_rocm
