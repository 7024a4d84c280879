/*
 * C ABI of the model runtime on the ROCm device, for callers that cannot include the C++ classes
 * (the Python test and benchmark harness binds it with ctypes).  It stands in front of
 * tfcc::runtime::Model, whose C++ interface follows the reference's
 * tfcc_runtime/framework/model.h:37-103: a model is created from the bytes of a model archive
 * (zip of model.pb + model.npz, model.cpp:57-80) and run on serialized tfcc.runtime.data.Inputs,
 * giving serialized tfcc.runtime.data.Outputs (model.cpp:145-181, tfcc_runtime/proto/data.proto).
 *
 * Every function returns 0 on success; otherwise tfcc_rocm_runtime_last_error() holds the text of
 * the C++ exception (thread local).  All calls for one model must come from the thread that called
 * tfcc_rocm_runtime_initialize(): device and session are per-thread defaults, as in the reference
 * (tfcc/core/framework/tfcc_session.h:29,60-62).
 */
#ifndef TFCC_ROCM_RUNTIME_H_
#define TFCC_ROCM_RUNTIME_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* tfcc::initialize_cuda / initialize_mkl counterpart (tfcc/cuda/utils/tfcc_cudautils.cpp:24-60):
 * gives the calling thread a ROCm device and session.  Idempotent per thread. */
int tfcc_rocm_runtime_initialize(void);
/* Same, with the host-memory device that has no compute interface: archives load and graphs build,
 * value / vector / reshape steps run, any tensor computation raises NotImplementedError as the
 * reference's default interfaces do (tfcc/core/interfaces/tfcc_blasinterface.cpp:23-30).  For
 * machines without a GPU. */
int tfcc_rocm_runtime_initialize_host(void);
const char* tfcc_rocm_runtime_last_error(void);

/* Model::Model(const std::string& data), model.cpp:57-108 */
int tfcc_rocm_runtime_model_create(const void* archive, size_t len, void** model);
int tfcc_rocm_runtime_model_destroy(void* model);

/* Model::run(inputs, outputs), model.cpp:145-181.  *outputs is allocated by the library; release it
 * with tfcc_rocm_runtime_buffer_free. */
int tfcc_rocm_runtime_model_run(void* model, const void* inputs, size_t len, void** outputs,
                                size_t* outputs_len);
int tfcc_rocm_runtime_buffer_free(void* buffer);

/* Model::test(npz, stream), model.cpp:185-280: runs the entrance graph on the arrays of an .npz and
 * compares every output found there; *passed = 1 when all are similar.  The summary text comes
 * back in *report (release with tfcc_rocm_runtime_buffer_free). */
int tfcc_rocm_runtime_model_test(void* model, const void* npz, size_t len, int* passed,
                                 char** report);

/* Graphs built after this call on the calling thread fuse node sequences into single kernels
 * (matmul + gelu, matmul + residual add, div + softmax; the default) or run every node as written.
 * Results are bit-identical either way.  The reference selects a fused variant of the model per
 * device instead (model.cpu.pb, tfcc_runtime/framework/model.cpp:311-322). */
int tfcc_rocm_runtime_set_fusion(int enable);

/* number of bound steps of the entrance graph (builds it if needed); nodes fused together share one */
int tfcc_rocm_runtime_model_step_count(void* model, size_t* steps);

/* Record the entrance graph's kernel sequence once and replay it with one launch per run from
 * then on (no counterpart in the reference, whose graphs are x86 call sequences). */
int tfcc_rocm_runtime_model_set_replay(void* model, int enable);

/* Sets the inputs once, then times `iters` runs of the entrance graph alone (no host copies) with
 * events on the session's stream after `warmup` untimed runs; microseconds per run. */
int tfcc_rocm_runtime_model_time(void* model, const void* inputs, size_t len, int warmup, int iters,
                                 double* microseconds_per_run);

#ifdef __cplusplus
}
#endif
#endif /* TFCC_ROCM_RUNTIME_H_ */
