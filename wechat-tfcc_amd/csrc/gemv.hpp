// Internal interface of the skinny (M <= 8) quantized matmul kernel.
#pragma once
#include <hip/hip_runtime.h>

namespace tfcc_rocm {

// Whether the skinny kernel takes this shape / alignment.
bool gemv_supported(const void* a, const void* b, unsigned m, unsigned n, unsigned k);

// ranges: {minA, maxA, minB, maxB} device pointers or null; rangeOut: {minC, maxC} or null.
int gemv_launch(hipStream_t stream, const unsigned char* a, const signed char* b, const int* rowsumA,
                const int* colsumB, int offsetA, int offsetB, const float* const ranges[4],
                float* const rangeOut[2], unsigned m, unsigned n, unsigned k, int* accOut,
                float scaleA, const float* scaleB, float* f32Out);

// The same on weights packed by tfcc_rocm_gemv_pack_b.
bool gemv_packed_supported(const void* a, const void* packed, unsigned m, unsigned k);
int gemv_packed_launch(hipStream_t stream, const unsigned char* a, const void* packed, const int* rowsumA,
                       const int* colsumB, int offsetA, int offsetB, const float* const ranges[4],
                       float* const rangeOut[2], unsigned m, unsigned n, unsigned k, int* accOut, float scaleA,
                       const float* scaleB, float* f32Out);

}  // namespace tfcc_rocm
