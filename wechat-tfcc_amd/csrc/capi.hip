// Device / stream / memory plumbing of the C ABI and the per-thread error text.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "common.hpp"
#include "gemv.hpp"

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

int tfcc_rocm_stream_release(void* stream) {
  // the stream's pending work may still use what is given back
  TFCC_HIP_CHECK(hipStreamSynchronize(as_stream(stream)));
  return tfcc_rocm::gemv_wide_release_stream(as_stream(stream));
}

int tfcc_rocm_stream_destroy(void* stream) {
  if (int e = tfcc_rocm_stream_release(stream)) return e;
  TFCC_HIP_CHECK(hipStreamDestroy(as_stream(stream)));
  return TFCC_ROCM_OK;
}

int tfcc_rocm_stream_synchronize(void* stream) {
  TFCC_HIP_CHECK(hipStreamSynchronize(as_stream(stream)));
  return TFCC_ROCM_OK;
}

int tfcc_rocm_event_create(void** event) {
  TFCC_REQUIRE(event != nullptr, "event_create: null argument");
  hipEvent_t e;
  TFCC_HIP_CHECK(hipEventCreate(&e));
  *event = e;
  return TFCC_ROCM_OK;
}

int tfcc_rocm_event_destroy(void* event) {
  TFCC_HIP_CHECK(hipEventDestroy(static_cast<hipEvent_t>(event)));
  return TFCC_ROCM_OK;
}

int tfcc_rocm_event_record(void* event, void* stream) {
  TFCC_REQUIRE(event != nullptr, "event_record: null argument");
  TFCC_HIP_CHECK(hipEventRecord(static_cast<hipEvent_t>(event), as_stream(stream)));
  return TFCC_ROCM_OK;
}

int tfcc_rocm_event_elapsed_ms(void* start, void* stop, float* ms) {
  TFCC_REQUIRE(start && stop && ms, "event_elapsed_ms: null argument");
  TFCC_HIP_CHECK(hipEventSynchronize(static_cast<hipEvent_t>(stop)));
  TFCC_HIP_CHECK(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
  return TFCC_ROCM_OK;
}

int tfcc_rocm_stream_begin_capture(void* stream) {
  TFCC_REQUIRE(stream != nullptr, "begin_capture: the default stream cannot be captured");
  // relaxed: a cache miss in the caller's allocator may still reach hipMalloc while recording
  TFCC_HIP_CHECK(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeRelaxed));
  return TFCC_ROCM_OK;
}

int tfcc_rocm_stream_end_capture(void* stream, void** graph_exec) {
  TFCC_REQUIRE(stream && graph_exec, "end_capture: null argument");
  *graph_exec = nullptr;
  hipGraph_t graph = nullptr;
  TFCC_HIP_CHECK(hipStreamEndCapture(as_stream(stream), &graph));
  TFCC_REQUIRE(graph != nullptr, "end_capture: the capture was invalidated");
  hipGraphExec_t exec = nullptr;
  hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  TFCC_HIP_CHECK(e);
  *graph_exec = exec;
  return TFCC_ROCM_OK;
}

int tfcc_rocm_graph_launch(void* graph_exec, void* stream) {
  TFCC_REQUIRE(graph_exec != nullptr, "graph_launch: null argument");
  TFCC_HIP_CHECK(hipGraphLaunch(static_cast<hipGraphExec_t>(graph_exec), as_stream(stream)));
  return TFCC_ROCM_OK;
}

int tfcc_rocm_graph_destroy(void* graph_exec) {
  if (graph_exec == nullptr) return TFCC_ROCM_OK;
  TFCC_HIP_CHECK(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec)));
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
