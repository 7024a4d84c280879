// The ROCm device for TFCC: Device / Session subclasses over the C ABI of libtfcc_rocm.so, the
// interface implementations they install, and the backend-specific quantized matmul operations.
//
// Shape of a GPU backend in the reference: tfcc/cuda/framework/tfcc_cudadevice.cpp:36-109 (allocator
// hooks, 90 % memory limit, interface installation), tfcc/cuda/framework/tfcc_cudasession.cpp:36-63
// (stream ownership, session allocator chained to the device's with a sync before a real free),
// tfcc/cuda/utils/tfcc_cudautils.cpp:24-60 (initialize_cuda).  The quantized matmul is not part of
// Interface<T> in the reference either: it is a public backend header
// (tfcc/mkl/operations/tfcc_mklquantization.h:39-51), mirrored here as tfcc::rocm::quantization.
#pragma once

#include <tuple>

#include "tfcc_interfaces.h"

namespace tfcc {

// a failing call into libtfcc_rocm.so; what() carries the library's error text
class ROCMRuntimeError : public Exception {
  int _status;

 public:
  ROCMRuntimeError(int status, const std::string& text) : Exception(text), _status(status) {}
  int status() const { return _status; }
};

class ROCMDevice : public Device {
  unsigned _index;

 public:
  explicit ROCMDevice(unsigned index);
  ROCMDevice(unsigned index, std::unique_ptr<Allocator> allocator);
  ~ROCMDevice() override;
  void attach() override;
  unsigned index() const { return _index; }
  static unsigned getDeviceCount();
};

class ROCMSession : public Session {
  ROCMDevice& _device;
  void* _stream;  // hipStream_t
  bool _recording = false;  // the stream's launches are being recorded into a graph, not run

 public:
  explicit ROCMSession(ROCMDevice& device);
  ROCMSession(ROCMDevice& device, std::unique_ptr<Allocator> allocator);
  ~ROCMSession() override;
  void sync() const override;
  Device& getDevice() override { return _device; }
  const Device& getDevice() const override { return _device; }
  void* getStream() const { return _stream; }
  // While the stream records (a HIP graph capture), nothing may wait for it or move data between host and device:
  // sync(), data::get and data::set throw RuntimeError before they touch the stream, so that the recording itself
  // stays valid and can be ended in the ordinary way by whoever began it.
  void setRecording(bool recording) { _recording = recording; }
  bool recording() const { return _recording; }
};

// Creates (once per process) one ROCMDevice per GPU and gives the calling thread a device and a
// session of its own as thread defaults.
void initialize_rocm();
void initialize_rocm(unsigned deviceID);

// Plain host memory device whose only interface is Data (memory moves): lets the framework types
// (Variable, View, allocators, shape checks) and the runtime's loading and graph building be
// exercised on machines without a GPU.  Every compute interface keeps the throwing default.
class HostDevice : public Device {
 public:
  HostDevice();
  void attach() override {}
};
class HostSession : public Session {
  HostDevice& _device;

 public:
  explicit HostSession(HostDevice& device);
  ~HostSession() override;
  void sync() const override {}
  Device& getDevice() override { return _device; }
  const Device& getDevice() const override { return _device; }
};

// gives the calling thread the process-wide host device and a host session of its own
void initialize_host();

namespace rocm {

// Fused forms: what a caller would otherwise issue as consecutive operations, done in one kernel
// with the same fp32 rounding after every step (results are bit-identical to the separate calls).
// Backend-specific, like the quantized matmul: they need the ROCm device as the thread default.
namespace blas {
enum class Activation { NONE = 0, GELU = 1 };
// activation(a * b + bias + residual); bias and residual may be null; residual has the result's shape.
// Checks and shape rules of tfcc::blas::matmul.
Variable<float> matmul_fused(const Tensor<float>& a, const Tensor<float>& b, const Tensor<float>* bias,
                             const Tensor<float>* residual, Activation activation);
// transpose(matmul(transpose(a, permA), transpose(b, permB)) [+ bias], permC) for tensors of one rank from 2 to 4
// without materialising any of the three permutations (an empty perm is the identity): the kernel walks the
// operands through their strides.  Needs the k dimension of the permuted a, the k or the n dimension
// of the permuted b and the n dimension of the result to be the contiguous one of their tensors;
// anything else raises NotImplementedError.  Results equal the step-by-step form bit for bit.
Variable<float> matmul_permuted(const Tensor<float>& a, const std::vector<size_t>& permA, const Tensor<float>& b,
                                const std::vector<size_t>& permB, const std::vector<size_t>& permC,
                                const Tensor<float>* bias = nullptr);
// { a * b[g] + bias[g] } for up to four weight matrices of one shape ([k, n], rank 2) in a single launch;
// a: [..., k] of any rank >= 2 (its leading dimensions are the rows).  Each result equals
// tfcc::blas::matmul(a, b[g], bias[g]) bit for bit.  Raises NotImplementedError for anything else.
std::vector<Variable<float>> matmul_grouped(const Tensor<float>& a, const std::vector<const Tensor<float>*>& b,
                                            const std::vector<const Tensor<float>*>& bias);
// transpose(matmul(softmax(matmul(transpose(q, permQ), transpose(k, permK)) [/ *divisor], last axis),
// transpose(v, permV)), permOut) for rank-4 tensors in one launch (an empty perm is the identity;
// divisor may be null).  transpose(k, permK) is the [.., size, keys] operand the first product takes.
// The result equals the step-by-step form bit for bit.  Raises NotImplementedError when the layout or
// the sizes are outside what the kernel takes (more than 128 keys, head size above 64, a head size or
// strides that are not multiples of 4, size not the contiguous dimension of q, k, v and the result).
// mask (optional): added to the divided scores before the softmax; a rank-4 tensor [b0 or 1, b1 or 1, 1, keys]
// against scores [b0, b1, queries, keys], anything else raises NotImplementedError.
Variable<float> attention_permuted(const Tensor<float>& q, const std::vector<size_t>& permQ, const Tensor<float>& k,
                                   const std::vector<size_t>& permK, const Tensor<float>& v,
                                   const std::vector<size_t>& permV, const std::vector<size_t>& permOut,
                                   const float* divisor, const Tensor<float>* mask = nullptr);
}  // namespace blas
namespace math {
// softmax(a / divisor, axis)
Variable<float> softmax_div(const Tensor<float>& a, size_t axis, float divisor);
}  // namespace math

namespace quantization {

// tfcc::mkl::quantization::matmul (tfcc/mkl/operations/tfcc_mklquantization.cpp:71-203): same
// argument meaning, checks, error texts, batch folding and result ranges.
std::tuple<Variable<int32_t>, Variable<float>, Variable<float>> matmul(
    const Tensor<uint8_t>& a, const Tensor<int32_t>& reduceSumA, const Tensor<float>& minA,
    const Tensor<float>& maxA, const Tensor<int8_t>& b, const Tensor<int32_t>& reduceSumB,
    const Tensor<float>& minB, const Tensor<float>& maxB);

// The same product with requantize<uint8_t>(c, minC, maxC, minOutput, maxOutput) fused into the
// kernel's store; `accumulators`, when given, also receives the int32 result.
std::tuple<Variable<uint8_t>, Variable<float>, Variable<float>> matmul_requantize(
    const Tensor<uint8_t>& a, const Tensor<int32_t>& reduceSumA, const Tensor<float>& minA,
    const Tensor<float>& maxA, const Tensor<int8_t>& b, const Tensor<int32_t>& reduceSumB,
    const Tensor<float>& minB, const Tensor<float>& maxB, const Tensor<float>& minOutput,
    const Tensor<float>& maxOutput, Variable<int32_t>* accumulators = nullptr);

// tfcc::mkl::quantization::reduce_sum (tfcc_mklquantization.cpp:284-318); T = int8_t, uint8_t, int16_t
template <class T>
Variable<int32_t> reduce_sum(const Tensor<T>& a, bool row);

// What a constant weight matrix of a quantized matmul needs besides itself, computed once: its column
// sums (the reference recomputes reduce_sum(b) per call, tfcc/test/quantization.cpp:112-118) and a copy
// in the layout the skinny kernel streams at full rate (the reference re-packs b inside every call,
// tfcc/mkl/gemm/tfcc_mklinputpackermanager.h:34-47).  Build it next to the Constant it belongs to; it
// refers to `b`, which must outlive it, and belongs to the device that was current when it was built.
class PreparedWeights {
  const Tensor<int8_t>* _b;
  Variable<int32_t> _reduceSum;
  Variable<uint8_t> _packed;

 public:
  explicit PreparedWeights(const Tensor<int8_t>& b);  // b: [k, n]
  PreparedWeights(PreparedWeights&&) = default;
  PreparedWeights& operator=(PreparedWeights&&) = default;
  const Tensor<int8_t>& weights() const { return *_b; }
  const Tensor<int32_t>& reduceSum() const { return _reduceSum; }  // reduce_sum(b, false)
  const void* packed() const { return _packed.data(); }
};

// matmul(a, reduceSumA, minA, maxA, w.weights(), w.reduceSum(), minB, maxB): the same checks and the
// same result; products of at most 8 rows stream the packed copy, large ones skip the accumulation of the
// true column sums (they are what w.reduceSum() holds).
std::tuple<Variable<int32_t>, Variable<float>, Variable<float>> matmul(
    const Tensor<uint8_t>& a, const Tensor<int32_t>& reduceSumA, const Tensor<float>& minA,
    const Tensor<float>& maxA, const PreparedWeights& w, const Tensor<float>& minB, const Tensor<float>& maxB);

}  // namespace quantization
}  // namespace rocm
}  // namespace tfcc
