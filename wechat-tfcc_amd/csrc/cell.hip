// Recurrent cells: the element-wise step that follows the two matrix products of an LSTM / GRU time step.
// One thread per (batch row, unit); every operand is read once, coalesced along the units.
//
// Arithmetic and operand layout follow the reference's scalar kernels, expression by expression:
//   LSTM cell             tfcc/mkl/kernel/tfcc_mklcellkernel.hpp:51-87   (gate order i, c, f, o)
//   GRU gates             tfcc/mkl/kernel/tfcc_mklcellkernel.hpp:89-133
//   GRU candidate         tfcc/mkl/kernel/tfcc_mklcellkernel.hpp:135-158
//   PyTorch-style GRU     tfcc/mkl/kernel/tfcc_mklcellkernel.hpp:160-189
// with sigmoid(v) = 1 / (1 + exp(0 - v)) (:45-48).
#include "common.hpp"

namespace tfcc_rocm {
namespace {

__device__ __forceinline__ float sigmoid_value(float v) { return 1.f / (1.f + expf(0.f - v)); }

// h and cs may be any two buffers of batch * units floats (h is often a row block of the output sequence);
// they may not overlap the inputs except that cs may be stateC itself (each element is read before it is written
// by the same thread).
__global__ __launch_bounds__(256) void lstm_cell_kernel(unsigned batch, unsigned units, const float* stateC,
                                                        const float* inputValue, const float* stateHValue,
                                                        const float* bias, float forget, float* h, float* cs) {
  const size_t total = (size_t)batch * units;
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += stride) {
    const unsigned b = (unsigned)(idx / units), i = (unsigned)(idx - (size_t)b * units);
    const float* x = inputValue + (size_t)b * 4 * units + i;
    const float* s = stateHValue + (size_t)b * 4 * units + i;
    float xi = x[0] + s[0] + bias[i];
    float xc = x[units] + s[units] + bias[i + units];
    float xf = x[2 * (size_t)units] + s[2 * (size_t)units] + bias[i + 2 * (size_t)units];
    float xo = x[3 * (size_t)units] + s[3 * (size_t)units] + bias[i + 3 * (size_t)units];
    xi = sigmoid_value(xi);
    xc = tanhf(xc);
    xf = sigmoid_value(xf + forget);
    xo = sigmoid_value(xo);
    const float c = __fadd_rn(__fmul_rn(xc, xi), __fmul_rn(stateC[idx], xf));
    h[idx] = tanhf(c) * xo;
    cs[idx] = c;
  }
}

// result[b] = concat(inputs[b], sigmoid(value[b, :units] + bias[:units]) * state[b])
__global__ __launch_bounds__(256) void gru_gates_kernel(unsigned batch, unsigned units, unsigned inputSize,
                                                        const float* state, const float* inputs, const float* value,
                                                        const float* bias, float* result) {
  const unsigned width = inputSize + units;
  const size_t total = (size_t)batch * width;
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += stride) {
    const unsigned b = (unsigned)(idx / width), j = (unsigned)(idx - (size_t)b * width);
    if (j < inputSize) {
      result[idx] = inputs[(size_t)b * inputSize + j];
    } else {
      const unsigned i = j - inputSize;
      const float r = sigmoid_value(value[(size_t)b * 2 * units + i] + bias[i]);
      result[idx] = r * state[(size_t)b * units + i];
    }
  }
}

// u = sigmoid(value[b, units + i] + bias[units + i]); c = tanh(cValue + cBias); result = u * state + (1 - u) * c
__global__ __launch_bounds__(256) void gru_candidate_kernel(unsigned batch, unsigned units, const float* state,
                                                            const float* value, const float* bias,
                                                            const float* cValue, const float* cBias, float* result) {
  const size_t total = (size_t)batch * units;
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += stride) {
    const unsigned b = (unsigned)(idx / units), i = (unsigned)(idx - (size_t)b * units);
    const float u = sigmoid_value(value[(size_t)b * 2 * units + units + i] + bias[units + i]);
    const float c = tanhf(cValue[idx] + cBias[i]);
    result[idx] = __fadd_rn(__fmul_rn(u, state[idx]), __fmul_rn(1.f - u, c));
  }
}

__global__ __launch_bounds__(256) void pytorch_gru_cell_kernel(unsigned batch, unsigned units, const float* state,
                                                               const float* inputValue, const float* stateValue,
                                                               const float* gateBias, const float* candidateIBias,
                                                               const float* candidateHBias, float* result) {
  const size_t total = (size_t)batch * units;
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += stride) {
    const unsigned b = (unsigned)(idx / units), i = (unsigned)(idx - (size_t)b * units);
    const float* x = inputValue + (size_t)b * 3 * units + i;
    const float* s = stateValue + (size_t)b * 3 * units + i;
    const float r = sigmoid_value(x[0] + s[0] + gateBias[i]);
    const float z = sigmoid_value(x[units] + s[units] + gateBias[i + units]);
    const float ni = x[2 * (size_t)units] + candidateIBias[i];
    const float nh = s[2 * (size_t)units] + candidateHBias[i];
    const float n = tanhf(__fadd_rn(ni, __fmul_rn(r, nh)));
    result[idx] = __fadd_rn(n, __fmul_rn(z, state[idx] - n));
  }
}

unsigned cell_grid(size_t total) {
  size_t blocks = (total + 255) / 256;
  if (blocks > 2048) blocks = 2048;
  return (unsigned)blocks;
}

}  // namespace
}  // namespace tfcc_rocm

using namespace tfcc_rocm;

extern "C" {

int tfcc_rocm_lstm_cell_f32(void* stream, unsigned batch, unsigned units, const float* state_c,
                            const float* input_value, const float* state_h_value, const float* bias, float forget,
                            float* h, float* cs) {
  TFCC_REQUIRE(state_c && input_value && state_h_value && bias && h && cs, "lstm_cell: null argument");
  TFCC_REQUIRE(batch > 0 && units > 0, "lstm_cell: empty state");
  TFCC_REQUIRE((unsigned long long)batch * units < (1ull << 30), "lstm_cell: state too large");
  hipLaunchKernelGGL(lstm_cell_kernel, dim3(cell_grid((size_t)batch * units)), dim3(256), 0, as_stream(stream), batch,
                     units, state_c, input_value, state_h_value, bias, forget, h, cs);
  return check_launch("lstm_cell");
}

int tfcc_rocm_gru_cell_gates_f32(void* stream, unsigned batch, unsigned units, unsigned input_size,
                                 const float* state, const float* inputs, const float* value, const float* bias,
                                 float* result) {
  TFCC_REQUIRE(state && inputs && value && bias && result, "gru_cell_gates: null argument");
  TFCC_REQUIRE(batch > 0 && units > 0, "gru_cell_gates: empty state");
  TFCC_REQUIRE((unsigned long long)batch * ((unsigned long long)units + input_size) < (1ull << 30),
               "gru_cell_gates: result too large");
  hipLaunchKernelGGL(gru_gates_kernel, dim3(cell_grid((size_t)batch * ((size_t)units + input_size))), dim3(256), 0,
                     as_stream(stream), batch, units, input_size, state, inputs, value, bias, result);
  return check_launch("gru_cell_gates");
}

int tfcc_rocm_gru_cell_candidate_f32(void* stream, unsigned batch, unsigned units, const float* state,
                                     const float* value, const float* bias, const float* c_value,
                                     const float* c_bias, float* result) {
  TFCC_REQUIRE(state && value && bias && c_value && c_bias && result, "gru_cell_candidate: null argument");
  TFCC_REQUIRE(batch > 0 && units > 0, "gru_cell_candidate: empty state");
  TFCC_REQUIRE((unsigned long long)batch * units < (1ull << 30), "gru_cell_candidate: state too large");
  hipLaunchKernelGGL(gru_candidate_kernel, dim3(cell_grid((size_t)batch * units)), dim3(256), 0, as_stream(stream),
                     batch, units, state, value, bias, c_value, c_bias, result);
  return check_launch("gru_cell_candidate");
}

int tfcc_rocm_pytorch_gru_cell_f32(void* stream, unsigned batch, unsigned units, const float* state,
                                   const float* input_value, const float* state_value, const float* gate_bias,
                                   const float* candidate_i_bias, const float* candidate_h_bias, float* result) {
  TFCC_REQUIRE(state && input_value && state_value && gate_bias && candidate_i_bias && candidate_h_bias && result,
               "pytorch_gru_cell: null argument");
  TFCC_REQUIRE(batch > 0 && units > 0, "pytorch_gru_cell: empty state");
  TFCC_REQUIRE((unsigned long long)batch * units < (1ull << 30), "pytorch_gru_cell: state too large");
  hipLaunchKernelGGL(pytorch_gru_cell_kernel, dim3(cell_grid((size_t)batch * units)), dim3(256), 0,
                     as_stream(stream), batch, units, state, input_value, state_value, gate_bias, candidate_i_bias,
                     candidate_h_bias, result);
  return check_launch("pytorch_gru_cell");
}

}  // extern "C"
