// extern "C" face of tfcc::runtime::Model (declared in tfcc_rocm_runtime.h).
#include "tfcc_rocm_runtime.h"

#include <cstdlib>
#include <cstring>
#include <sstream>
#include <string>

#include "runtime.h"
#include "tfcc_rocm.h"
#include "tfcc_rocm_device.h"

namespace {
thread_local std::string g_error;

template <class F>
int guarded(F&& body) {
  try {
    body();
    return 0;
  } catch (const std::exception& e) {
    g_error = e.what();
  } catch (...) {
    g_error = "unknown exception";
  }
  return 1;
}

void* copy_out(const std::string& s) {
  char* p = static_cast<char*>(std::malloc(s.size() + 1));
  if (p == nullptr) throw tfcc::ResourceExhaustedError();
  std::memcpy(p, s.data(), s.size());
  p[s.size()] = 0;
  return p;
}

tfcc::runtime::Model& as_model(void* m) {
  if (m == nullptr) throw tfcc::InvalidArgumentError("null model");
  return *static_cast<tfcc::runtime::Model*>(m);
}

void rocm_check(int status) {
  if (status != TFCC_ROCM_OK) throw tfcc::ROCMRuntimeError(status, tfcc_rocm_last_error_string());
}
}  // namespace

extern "C" {

const char* tfcc_rocm_runtime_last_error(void) { return g_error.c_str(); }

int tfcc_rocm_runtime_initialize(void) {
  return guarded([] {
    if (tfcc::Session::getThreadDefault() == nullptr) tfcc::initialize_rocm();
  });
}

int tfcc_rocm_runtime_initialize_host(void) {
  return guarded([] {
    if (tfcc::Session::getThreadDefault() == nullptr) tfcc::initialize_host();
  });
}

int tfcc_rocm_runtime_model_create(const void* archive, size_t len, void** model) {
  return guarded([&] {
    if (archive == nullptr || model == nullptr) throw tfcc::InvalidArgumentError("null argument");
    *model = new tfcc::runtime::Model(std::string(static_cast<const char*>(archive), len));
  });
}

int tfcc_rocm_runtime_model_destroy(void* model) {
  return guarded([&] { delete static_cast<tfcc::runtime::Model*>(model); });
}

int tfcc_rocm_runtime_model_run(void* model, const void* inputs, size_t len, void** outputs, size_t* outputs_len) {
  return guarded([&] {
    if (outputs == nullptr || outputs_len == nullptr) throw tfcc::InvalidArgumentError("null argument");
    std::string out;
    as_model(model).run(std::string(static_cast<const char*>(inputs), len), out);
    *outputs = copy_out(out);
    *outputs_len = out.size();
  });
}

int tfcc_rocm_runtime_buffer_free(void* buffer) {
  std::free(buffer);
  return 0;
}

int tfcc_rocm_runtime_model_test(void* model, const void* npz, size_t len, int* passed, char** report) {
  return guarded([&] {
    if (passed == nullptr) throw tfcc::InvalidArgumentError("null argument");
    std::ostringstream ss;
    *passed = as_model(model).test(std::string(static_cast<const char*>(npz), len), ss) ? 1 : 0;
    if (report) *report = static_cast<char*>(copy_out(ss.str()));
  });
}

int tfcc_rocm_runtime_set_fusion(int enable) {
  return guarded([&] { tfcc::runtime::Graph::setFusionThreadLocal(enable != 0); });
}

int tfcc_rocm_runtime_model_step_count(void* model, size_t* steps) {
  return guarded([&] {
    if (steps == nullptr) throw tfcc::InvalidArgumentError("null argument");
    *steps = as_model(model).getEntranceGraph().stepCount();
  });
}

int tfcc_rocm_runtime_model_set_replay(void* model, int enable) {
  return guarded([&] { as_model(model).getEntranceGraph().enableReplay(enable != 0); });
}

int tfcc_rocm_runtime_model_time(void* model, const void* inputs, size_t len, int warmup, int iters,
                                 double* microseconds_per_run) {
  return guarded([&] {
    if (microseconds_per_run == nullptr || iters <= 0) throw tfcc::InvalidArgumentError("bad argument");
    tfcc::runtime::Model& m = as_model(model);
    std::vector<tfcc::runtime::proto::DataItem> out;
    m.run(tfcc::runtime::proto::parse_inputs(std::string(static_cast<const char*>(inputs), len)), out);
    tfcc::runtime::Graph& graph = m.getEntranceGraph();
    auto* session = dynamic_cast<tfcc::ROCMSession*>(tfcc::Session::getThreadDefault());
    if (session == nullptr) throw tfcc::RuntimeError("timing needs a ROCm session");
    for (int i = 0; i < warmup; ++i) graph.process();
    void *start = nullptr, *stop = nullptr;
    rocm_check(tfcc_rocm_event_create(&start));
    rocm_check(tfcc_rocm_event_create(&stop));
    rocm_check(tfcc_rocm_event_record(start, session->getStream()));
    for (int i = 0; i < iters; ++i) graph.process();
    rocm_check(tfcc_rocm_event_record(stop, session->getStream()));
    float ms = 0;
    rocm_check(tfcc_rocm_event_elapsed_ms(start, stop, &ms));
    tfcc_rocm_event_destroy(start);
    tfcc_rocm_event_destroy(stop);
    *microseconds_per_run = static_cast<double>(ms) * 1000.0 / iters;
  });
}

}  // extern "C"
