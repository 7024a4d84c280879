// Device / stream / memory plumbing of the C ABI and the per-thread error text.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "common.hpp"

namespace tfcc_rocm {

static thread_local char g_error[512] = "";

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

namespace {

template <class T>
__global__ void fill_kernel(T* dst, T value, size_t count) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (; i < count; i += step) dst[i] = value;
}

template <class T>
int fill(hipStream_t s, void* dst, uint64_t value, size_t count) {
  if (count == 0) return TFCC_ROCM_OK;
  size_t blocks = (count + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(fill_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, s, static_cast<T*>(dst), (T)value, count);
  return check_launch("fill");
}

}  // namespace
}  // namespace tfcc_rocm

using namespace tfcc_rocm;

extern "C" {

const char* tfcc_rocm_last_error_string(void) { return g_error; }
const char* tfcc_rocm_version(void) { return "tfcc_rocm 0.1 gfx950"; }

int tfcc_rocm_device_count(int* count) {
  TFCC_REQUIRE(count != nullptr, "device_count: null argument");
  hipError_t e = hipGetDeviceCount(count);
  if (e != hipSuccess) {
    *count = 0;
    return set_error(TFCC_ROCM_NO_DEVICE, "hipGetDeviceCount failed: %s", hipGetErrorString(e));
  }
  return TFCC_ROCM_OK;
}

int tfcc_rocm_set_device(int device) {
  TFCC_HIP_CHECK(hipSetDevice(device));
  return TFCC_ROCM_OK;
}

int tfcc_rocm_mem_info(size_t* free_bytes, size_t* total_bytes) {
  TFCC_REQUIRE(free_bytes && total_bytes, "mem_info: null argument");
  TFCC_HIP_CHECK(hipMemGetInfo(free_bytes, total_bytes));
  return TFCC_ROCM_OK;
}

int tfcc_rocm_device_name(char* buf, size_t len) {
  TFCC_REQUIRE(buf && len > 0, "device_name: null argument");
  int dev = 0;
  TFCC_HIP_CHECK(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  TFCC_HIP_CHECK(hipGetDeviceProperties(&prop, dev));
  snprintf(buf, len, "%s (%s, %d CUs)", prop.name, prop.gcnArchName, prop.multiProcessorCount);
  return TFCC_ROCM_OK;
}

int tfcc_rocm_malloc(void** ptr, size_t bytes) {
  TFCC_REQUIRE(ptr != nullptr, "malloc: null argument");
  *ptr = nullptr;
  TFCC_HIP_CHECK(hipMalloc(ptr, bytes));
  return TFCC_ROCM_OK;
}

int tfcc_rocm_free(void* ptr) {
  TFCC_HIP_CHECK(hipFree(ptr));
  return TFCC_ROCM_OK;
}

int tfcc_rocm_stream_create(void** stream) {
  TFCC_REQUIRE(stream != nullptr, "stream_create: null argument");
  hipStream_t s;
  TFCC_HIP_CHECK(hipStreamCreate(&s));  // default priority on purpose
  *stream = s;
  return TFCC_ROCM_OK;
}

int tfcc_rocm_stream_destroy(void* stream) {
  TFCC_HIP_CHECK(hipStreamDestroy(as_stream(stream)));
  return TFCC_ROCM_OK;
}

int tfcc_rocm_stream_synchronize(void* stream) {
  TFCC_HIP_CHECK(hipStreamSynchronize(as_stream(stream)));
  return TFCC_ROCM_OK;
}

int tfcc_rocm_memcpy_h2d(void* stream, void* dst_device, const void* src_host, size_t bytes) {
  if (bytes == 0) return TFCC_ROCM_OK;
  TFCC_REQUIRE(dst_device && src_host, "memcpy_h2d: null argument");
  TFCC_HIP_CHECK(hipStreamSynchronize(as_stream(stream)));
  TFCC_HIP_CHECK(hipMemcpy(dst_device, src_host, bytes, hipMemcpyHostToDevice));
  return TFCC_ROCM_OK;
}

int tfcc_rocm_memcpy_d2h(void* stream, void* dst_host, const void* src_device, size_t bytes) {
  if (bytes == 0) return TFCC_ROCM_OK;
  TFCC_REQUIRE(dst_host && src_device, "memcpy_d2h: null argument");
  TFCC_HIP_CHECK(hipStreamSynchronize(as_stream(stream)));
  TFCC_HIP_CHECK(hipMemcpy(dst_host, src_device, bytes, hipMemcpyDeviceToHost));
  return TFCC_ROCM_OK;
}

int tfcc_rocm_memcpy_d2d_async(void* stream, void* dst, const void* src, size_t bytes) {
  if (bytes == 0) return TFCC_ROCM_OK;
  TFCC_REQUIRE(dst && src, "memcpy_d2d: null argument");
  TFCC_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
  return TFCC_ROCM_OK;
}

int tfcc_rocm_fill_async(void* stream, void* dst, uint64_t value, int elem_size, size_t count) {
  if (count == 0) return TFCC_ROCM_OK;
  TFCC_REQUIRE(dst != nullptr, "fill: null argument");
  switch (elem_size) {
    case 1: return fill<uint8_t>(as_stream(stream), dst, value, count);
    case 2: return fill<uint16_t>(as_stream(stream), dst, value, count);
    case 4: return fill<uint32_t>(as_stream(stream), dst, value, count);
    case 8: return fill<uint64_t>(as_stream(stream), dst, value, count);
  }
  return set_error(TFCC_ROCM_INVALID_ARGUMENT, "fill: element size %d", elem_size);
}

}  // extern "C"
