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
                float scaleA, const float* scaleB, float* f32Out, bool colsumExact = false);

// The kernel that owns a column group over the whole of K (no workspace), whatever the shape.
int gemv_onepass_launch(hipStream_t stream, const unsigned char* a, const signed char* b, const int* rowsumA,
                        const int* colsumB, int offsetA, int offsetB, const float* const ranges[4],
                        float* const rangeOut[2], unsigned m, unsigned n, unsigned k, int* accOut,
                        float scaleA, const float* scaleB, float* f32Out);

// The same product split over K as well as over N (gemv_u8s8_wide.hip): whole 256-byte row pieces per load and
// several hundred workgroups for a decode-sized B, partial tiles added through a workspace.  Asks for n % 16 == 0
// and a B aligned to 16 bytes; gemv_launch takes it when it applies.  staticWorkspace: use the workspace inside
// the library's image (no allocation; n <= gemv_wide_static_max_n()) instead of one allocated per stream.
// colsumExact: the caller vouches that colsumB holds the true column sums of b (the kernel then does not form them).
bool gemv_wide_supported(const void* a, const void* b, unsigned m, unsigned n, unsigned k);
unsigned gemv_wide_static_max_n();
int gemv_wide_launch(hipStream_t stream, bool staticWorkspace, const unsigned char* a, const signed char* b,
                     const int* rowsumA, const int* colsumB, int offsetA, int offsetB, const float* const ranges[4],
                     float* const rangeOut[2], unsigned m, unsigned n, unsigned k, int* accOut, float scaleA,
                     const float* scaleB, float* f32Out, bool colsumExact = false);
// Gives back the workspaces kept for `stream` on the current device (the stream must be idle).
int gemv_wide_release_stream(hipStream_t stream);

// The same on weights packed by tfcc_rocm_gemv_pack_b.
bool gemv_packed_supported(const void* a, const void* packed, unsigned m, unsigned k);
int gemv_packed_launch(hipStream_t stream, const unsigned char* a, const void* packed, const int* rowsumA,
                       const int* colsumB, int offsetA, int offsetB, const float* const ranges[4],
                       float* const rangeOut[2], unsigned m, unsigned n, unsigned k, int* accOut, float scaleA,
                       const float* scaleB, float* f32Out);

}  // namespace tfcc_rocm
