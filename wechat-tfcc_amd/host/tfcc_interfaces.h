// The plug-in surface a device implements, and the operator functions that dispatch to it.
//
// A device owns one Interface<T> per element type; each is a bundle of sub-interfaces whose
// default implementation throws NotImplementedError, exactly as in the reference
// (tfcc/core/interfaces/tfcc_interface.h:76-161, tfcc_blasinterface.cpp:23-30).  A backend
// subclasses the sub-interfaces it supports and installs them with set*Interface from its device
// constructor (tfcc/cuda/interfaces/tfcc_cudainterface.cpp:38-70).
//
// Sub-interfaces present here: the matmul path itself (Blas, Quantization, Data) and the few
// neighbours one transformer encoder layer needs (Activation: softmax / geluAccurate,
// Normalization: layerNormalize, Basic: transpose, Arithmetic: add, Transformation: transform).
//
// Operator functions (same names and checks as tfcc/core/operations/):
//   blas::matmul            tfcc_blas.cpp:26-96
//   data::set/get/...       tfcc_data.cpp
//   quantization::*         tfcc_quantization.cpp:26-98
//   math::softmax, gelu_accurate   tfcc_math.cpp:455-461,585-592
//   nn::layer_normalization tfcc_nn.cpp:755-762
//   base::transpose         tfcc_base.cpp:124-134
#pragma once

#include <algorithm>
#include <tuple>

#include "tfcc_core.h"

namespace tfcc {

// Element type codes shared by the type-generic calls below (the order of the C ABI's TFCC_ROCM_S8 .. F64).
template <class T> struct ElementCode;
#define TFCC_ELEMENT_CODE(T, V) template <> struct ElementCode<T> { static constexpr int value = V; };
TFCC_ELEMENT_CODE(int8_t, 0) TFCC_ELEMENT_CODE(uint8_t, 1) TFCC_ELEMENT_CODE(int16_t, 2) TFCC_ELEMENT_CODE(uint16_t, 3)
TFCC_ELEMENT_CODE(int32_t, 4) TFCC_ELEMENT_CODE(uint32_t, 5) TFCC_ELEMENT_CODE(int64_t, 6) TFCC_ELEMENT_CODE(uint64_t, 7)
TFCC_ELEMENT_CODE(float, 8) TFCC_ELEMENT_CODE(double, 9)
#undef TFCC_ELEMENT_CODE

template <class T>
class BlasInterface {
 public:
  virtual ~BlasInterface() {}
  // a: [..., m, k], b: [..., k, n]; one operand may be a plain matrix shared by the whole batch
  virtual Variable<T> matmul(const Tensor<T>&, const Tensor<T>&) { throw NotImplementedError(); }
  // c = a * b + bias, bias: [n]
  virtual Variable<T> matmul(const Tensor<T>&, const Tensor<T>&, const Tensor<T>&) { throw NotImplementedError(); }
};

template <class T>
class QuantizationInterface {
 public:
  virtual ~QuantizationInterface() {}
  virtual std::tuple<Variable<T>, Variable<float>, Variable<float>> quantize(const Tensor<float>&) {
    throw NotImplementedError();
  }
  virtual Variable<T> quantize(const Tensor<float>&, const Tensor<float>&, const Tensor<float>&) {
    throw NotImplementedError();
  }
#define TFCC_REQUANTIZE_DEFAULT(TI)                                                                        \
  virtual Variable<T> requantize(const Tensor<TI>&, const Tensor<float>&, const Tensor<float>&,            \
                                 const Tensor<float>&, const Tensor<float>&) {                             \
    throw NotImplementedError();                                                                           \
  }
  TFCC_REQUANTIZE_DEFAULT(int8_t)
  TFCC_REQUANTIZE_DEFAULT(uint8_t)
  TFCC_REQUANTIZE_DEFAULT(int16_t)
  TFCC_REQUANTIZE_DEFAULT(uint16_t)
  TFCC_REQUANTIZE_DEFAULT(int32_t)
  TFCC_REQUANTIZE_DEFAULT(uint32_t)
#undef TFCC_REQUANTIZE_DEFAULT
  virtual Variable<float> dequantize(const Tensor<T>&, const Tensor<float>&, const Tensor<float>&) {
    throw NotImplementedError();
  }
};

template <class T>
class DataInterface {
 public:
  virtual ~DataInterface() {}
  virtual void set(T*, const T*, size_t) { throw NotImplementedError(); }  // host -> device, len elements
  virtual void set(Variable<T>&, const T*) { throw NotImplementedError(); }
  virtual void set(Variable<T>&, std::vector<T>&&) { throw NotImplementedError(); }
  virtual void get(const Tensor<T>&, T*) { throw NotImplementedError(); }  // device -> host, synchronises
  virtual void zeros(Variable<T>&) { throw NotImplementedError(); }
  virtual void ones(Variable<T>&) { throw NotImplementedError(); }
  virtual void fill(Variable<T>&, T) { throw NotImplementedError(); }  // every element = the value (an addition)
  virtual Variable<T> copy(const Tensor<T>&) { throw NotImplementedError(); }
  // element-wise static_cast into this interface's type, one virtual per source type, and the conversion to
  // 0 / 1 bytes (tfcc/core/interfaces/tfcc_datainterface.h:40-53)
  virtual Variable<T> cast(const Tensor<float>&) { throw NotImplementedError(); }
  virtual Variable<T> cast(const Tensor<double>&) { throw NotImplementedError(); }
  virtual Variable<T> cast(const Tensor<int8_t>&) { throw NotImplementedError(); }
  virtual Variable<T> cast(const Tensor<uint8_t>&) { throw NotImplementedError(); }
  virtual Variable<T> cast(const Tensor<int16_t>&) { throw NotImplementedError(); }
  virtual Variable<T> cast(const Tensor<uint16_t>&) { throw NotImplementedError(); }
  virtual Variable<T> cast(const Tensor<int32_t>&) { throw NotImplementedError(); }
  virtual Variable<T> cast(const Tensor<uint32_t>&) { throw NotImplementedError(); }
  virtual Variable<T> cast(const Tensor<int64_t>&) { throw NotImplementedError(); }
  virtual Variable<T> cast(const Tensor<uint64_t>&) { throw NotImplementedError(); }
  virtual Variable<uint8_t> cast_to_boolean(const Tensor<T>&) { throw NotImplementedError(); }
};

template <class T>
class ActivationInterface {
 public:
  virtual ~ActivationInterface() {}
  virtual Variable<T> softmax(const Tensor<T>&, size_t) { throw NotImplementedError(); }
  virtual Variable<T> geluAccurate(const Tensor<T>&) { throw NotImplementedError(); }
  // one of the UnaryFunction values below applied to every element
  virtual Variable<T> unary(const Tensor<T>&, int) { throw NotImplementedError(); }
  // tfcc/core/interfaces/tfcc_activationinterface.h:34-43
  virtual Variable<T> leakyRelu(const Tensor<T>&, T) { throw NotImplementedError(); }
  virtual Variable<T> pow(const Tensor<T>&, T) { throw NotImplementedError(); }
  virtual Variable<T> pow(const Tensor<T>&, const Tensor<T>&) { throw NotImplementedError(); }  // equal rank, broadcast
  virtual Variable<T> pow(T, const Tensor<T>&) { throw NotImplementedError(); }
};

// element-wise functions of one tensor (the numbering of the kernel library's TFCC_ROCM_UNARY_* values)
enum class UnaryFunction { SIGMOID = 0, TANH, RELU, SOFTPLUS, LOG, RSQRT, ERF, ABS, SIGN, NEG, RECIPROCAL, SQRT };

template <class T>
class NormalizationInterface {
 public:
  virtual ~NormalizationInterface() {}
  virtual Variable<T> layerNormalize(const Tensor<T>&, const Tensor<T>&, const Tensor<T>&, T, size_t) {
    throw NotImplementedError();
  }
};

template <class T>
class BasicInterface {
 public:
  virtual ~BasicInterface() {}
  virtual Variable<T> transpose(const Tensor<T>&, const std::vector<size_t>&) { throw NotImplementedError(); }
  virtual Variable<T> slice(const Tensor<T>&, size_t, unsigned, unsigned) { throw NotImplementedError(); }
  virtual Variable<T> concat(const std::vector<const Tensor<T>*>&, size_t) { throw NotImplementedError(); }
  virtual void assignTo(const Tensor<T>&, size_t, unsigned, Variable<T>&) { throw NotImplementedError(); }
  // rows of params by index (tfcc/core/interfaces/tfcc_gatherinterface.h): indices of the type with code indexCode
  virtual Variable<T> clip(const Tensor<T>&, T, T) { throw NotImplementedError(); }
  virtual Variable<int64_t> argmax(const Tensor<T>&, size_t) { throw NotImplementedError(); }
  virtual std::tuple<Variable<T>, Variable<uint32_t>> topK(const Tensor<T>&, unsigned) { throw NotImplementedError(); }
  // tfcc/core/interfaces/tfcc_basicinterface.h: where with tensor / value operands (x or y null: the value), tril, triu
  virtual Variable<T> where(const Tensor<uint8_t>&, const Tensor<T>*, T, const Tensor<T>*, T) { throw NotImplementedError(); }
  virtual Variable<T> triangle(const Tensor<T>&, int64_t, bool /*upper*/) { throw NotImplementedError(); }
  virtual Variable<T> gather(const Tensor<T>&, const void* /*indices*/, int /*indexCode*/, const Shape& /*indexShape*/) {
    throw NotImplementedError();
  }
};

template <class T>
class ArithmeticInterface {
 public:
  virtual ~ArithmeticInterface() {}
  virtual Variable<T> add(const Tensor<T>&, const Tensor<T>&) { throw NotImplementedError(); }
  virtual Variable<T> sub(const Tensor<T>&, const Tensor<T>&) { throw NotImplementedError(); }
  virtual Variable<T> mul(const Tensor<T>&, const Tensor<T>&) { throw NotImplementedError(); }
  virtual Variable<T> div(const Tensor<T>&, const Tensor<T>&) { throw NotImplementedError(); }
};

// tfcc/core/interfaces/tfcc_comparisoninterface.h:27-83: tensor against value, byte results (1 where the relation
// holds).  compareDifference is an addition: (a - b) against 0 for two tensors of equal rank with broadcast
// dimensions, which tfcc::relation's tensor-tensor forms otherwise compose from a subtraction in memory and a
// comparison with 0 (tfcc/core/operations/tfcc_relation.cpp:101-115).
enum class Relation { EQUAL = 0, UNEQUAL, GREATER, GREATER_EQUAL, LESS, LESS_EQUAL };

template <class T>
class ComparisonInterface {
 public:
  virtual ~ComparisonInterface() {}
  virtual Variable<uint8_t> compare(const Tensor<T>&, T, Relation) { throw NotImplementedError(); }
  virtual Variable<uint8_t> compareDifference(const Tensor<T>&, const Tensor<T>&, Relation) { throw NotImplementedError(); }
  Variable<uint8_t> equal(const Tensor<T>& a, T b) { return compare(a, b, Relation::EQUAL); }
  Variable<uint8_t> unequal(const Tensor<T>& a, T b) { return compare(a, b, Relation::UNEQUAL); }
  Variable<uint8_t> greater(const Tensor<T>& a, T b) { return compare(a, b, Relation::GREATER); }
  Variable<uint8_t> greaterEqual(const Tensor<T>& a, T b) { return compare(a, b, Relation::GREATER_EQUAL); }
  Variable<uint8_t> less(const Tensor<T>& a, T b) { return compare(a, b, Relation::LESS); }
  Variable<uint8_t> lessEqual(const Tensor<T>& a, T b) { return compare(a, b, Relation::LESS_EQUAL); }
};

// tfcc/core/interfaces/tfcc_minmaxinterface.h:30-68
template <class T>
class MinMaxInterface {
 public:
  virtual ~MinMaxInterface() {}
  virtual Variable<T> min(const Tensor<T>&, const Tensor<T>&) { throw NotImplementedError(); }
  virtual Variable<T> min(const Tensor<T>&, T) { throw NotImplementedError(); }
  virtual Variable<T> max(const Tensor<T>&, const Tensor<T>&) { throw NotImplementedError(); }
  virtual Variable<T> max(const Tensor<T>&, T) { throw NotImplementedError(); }
};

// tfcc/core/interfaces/tfcc_reduceinterface.h:27-41: the dimensions from `keep` on are reduced and stay in the
// result's shape with length 1.
template <class T>
class ReduceInterface {
 public:
  virtual ~ReduceInterface() {}
  virtual Variable<T> reduceSum(const Tensor<T>&, size_t) { throw NotImplementedError(); }
  virtual Variable<T> reduceMean(const Tensor<T>&, size_t) { throw NotImplementedError(); }
  virtual Variable<T> reduceProd(const Tensor<T>&, size_t) { throw NotImplementedError(); }
  virtual Variable<T> reduceMax(const Tensor<T>&, size_t) { throw NotImplementedError(); }
  virtual Variable<T> reduceMin(const Tensor<T>&, size_t) { throw NotImplementedError(); }
};

template <class T>
class TransformationInterface {
 public:
  virtual ~TransformationInterface() {}
  virtual Variable<T> transform(const Tensor<T>&, T, T) { throw NotImplementedError(); }   // a * alpha + beta
  virtual Variable<T> transform2(const Tensor<T>&, T, T) { throw NotImplementedError(); }  // a / alpha + beta
};

// tfcc/core/interfaces/tfcc_cellinterface.h:23-88.  processLSTMCellInto is an addition for callers that own
// the memory of a whole sequence: the same step written into h and cs ([batch, units] each; cs may be
// stateC's own memory), so that a sequence needs neither a copy nor a concat per step.
template <class T>
class CellInterface {
 public:
  virtual ~CellInterface() {}
  virtual std::tuple<Variable<T>, Variable<T>> processLSTMCell(const Tensor<T>&, const Tensor<T>&, const Tensor<T>&,
                                                               const Tensor<T>&, T) {
    throw NotImplementedError();
  }
  virtual void processLSTMCellInto(const Tensor<T>&, const Tensor<T>&, const Tensor<T>&, const Tensor<T>&, T, T*, T*) {
    throw NotImplementedError();
  }
  // A whole time step in one launch, for devices that have one: the state kernel in the layout that launch wants
  // (made once per sequence), then per step matmul(h, stateKernel) and the cell together.  NotImplementedError
  // (the default, or for shapes the device does not take) sends the caller to the two calls above.
  virtual Variable<T> prepareLSTMStateKernel(const Tensor<T>&, unsigned /*batch*/) { throw NotImplementedError(); }
  virtual void processLSTMStepInto(const Tensor<T>& /*stateC*/, const Tensor<T>& /*inputValue*/, const Tensor<T>& /*h*/,
                                   const Tensor<T>& /*preparedStateKernel*/, const Tensor<T>& /*bias*/, T /*forget*/,
                                   T* /*hOut*/, T* /*csOut*/) {
    throw NotImplementedError();
  }
  virtual Variable<T> processGRUCellGates(const Tensor<T>&, const Tensor<T>&, const Tensor<T>&, const Tensor<T>&) {
    throw NotImplementedError();
  }
  virtual Variable<T> processGRUCellCandidate(const Tensor<T>&, const Tensor<T>&, const Tensor<T>&, const Tensor<T>&,
                                              const Tensor<T>&) {
    throw NotImplementedError();
  }
  virtual Variable<T> processPyTorchGRUCell(const Tensor<T>&, const Tensor<T>&, const Tensor<T>&, const Tensor<T>&,
                                            const Tensor<T>&, const Tensor<T>&) {
    throw NotImplementedError();
  }
};

template <class T>
class Interface {
#define TFCC_SUB_INTERFACE(NAME)                                                     \
 private:                                                                            \
  std::unique_ptr<NAME##Interface<T>> _##NAME{new NAME##Interface<T>()};             \
                                                                                     \
 public:                                                                             \
  NAME##Interface<T>& get##NAME##Interface() { return *_##NAME; }                    \
  void set##NAME##Interface(std::unique_ptr<NAME##Interface<T>> p) { _##NAME = std::move(p); }
  TFCC_SUB_INTERFACE(Blas)
  TFCC_SUB_INTERFACE(Quantization)
  TFCC_SUB_INTERFACE(Data)
  TFCC_SUB_INTERFACE(Activation)
  TFCC_SUB_INTERFACE(Normalization)
  TFCC_SUB_INTERFACE(Basic)
  TFCC_SUB_INTERFACE(Arithmetic)
  TFCC_SUB_INTERFACE(Transformation)
  TFCC_SUB_INTERFACE(Cell)
  TFCC_SUB_INTERFACE(MinMax)
  TFCC_SUB_INTERFACE(Reduce)
  TFCC_SUB_INTERFACE(Comparison)
#undef TFCC_SUB_INTERFACE
};

// the element types a device carries an Interface for
struct InterfaceSet {
  Interface<float> f32;
  Interface<double> f64;
  Interface<int8_t> s8;
  Interface<uint8_t> u8;
  Interface<int16_t> s16;
  Interface<uint16_t> u16;
  Interface<int32_t> s32;
  Interface<uint32_t> u32;
  Interface<int64_t> s64;
  Interface<uint64_t> u64;
};

namespace detail {
inline Interface<float>& pick(InterfaceSet& s, float) { return s.f32; }
inline Interface<double>& pick(InterfaceSet& s, double) { return s.f64; }
inline Interface<int8_t>& pick(InterfaceSet& s, int8_t) { return s.s8; }
inline Interface<uint8_t>& pick(InterfaceSet& s, uint8_t) { return s.u8; }
inline Interface<int16_t>& pick(InterfaceSet& s, int16_t) { return s.s16; }
inline Interface<uint16_t>& pick(InterfaceSet& s, uint16_t) { return s.u16; }
inline Interface<int32_t>& pick(InterfaceSet& s, int32_t) { return s.s32; }
inline Interface<uint32_t>& pick(InterfaceSet& s, uint32_t) { return s.u32; }
inline Interface<int64_t>& pick(InterfaceSet& s, int64_t) { return s.s64; }
inline Interface<uint64_t>& pick(InterfaceSet& s, uint64_t) { return s.u64; }
}  // namespace detail

template <class T>
Interface<T>& Device::getInterface(T) {
  return detail::pick(*_interfaces, T());
}

// tfcc/core/operations/tfcc_operation.cpp:22-26
template <class T>
struct Operation {
  static Interface<T>& getCurrentInterface() {
    Device* d = Device::getThreadDefault();
    if (d == nullptr) throw RuntimeError("no default device on this thread: call an initialize function first");
    return d->getInterface(T());
  }
};

// ---------------------------------------------------------------------------------------------
// operator functions
// ---------------------------------------------------------------------------------------------
namespace blas {

namespace detail {
// the checks shared by both forms; returns the result shape for the empty-operand shortcut
template <class T>
std::vector<unsigned> check(const Tensor<T>& a, const Tensor<T>& b, const Tensor<T>* bias) {
  const size_t ra = a.shape().size(), rb = b.shape().size();
  if (ra < 2 || rb < 2) throw InvalidArgumentError("matmul require tensors with two or more dimensions");
  if (ra != rb && ra != 2 && rb != 2) throw InvalidArgumentError("shape invalid");
  if (a.shape(ra - 1) != b.shape(rb - 2)) throw InvalidArgumentError("shape invalid");
  if (bias && (bias->shape().size() != 1 || bias->size() != b.shape(rb - 1))) throw InvalidArgumentError("shape invalid");
  std::vector<unsigned> s = ra > rb ? a.shape().toVector() : b.shape().toVector();
  if (ra == rb) {
    // The reference wants equal leading dimensions (tfcc/core/operations/tfcc_blas.cpp:36-42).  Accepted on
    // top of that: a leading dimension of 1 on one side stands for every index of the other side's.
    for (size_t i = 0; i + 2 < ra; ++i) {
      if (a.shape(i) != b.shape(i) && a.shape(i) != 1 && b.shape(i) != 1) throw InvalidArgumentError("shape invalid");
      s[i] = a.shape(i) == 1 ? b.shape(i) : a.shape(i);
    }
  }
  s[s.size() - 2] = a.shape(ra - 2);
  s[s.size() - 1] = b.shape(rb - 1);
  return s;
}
}  // namespace detail

template <class T>
Variable<T> matmul(const Tensor<T>& a, const Tensor<T>& b) {
  std::vector<unsigned> s = detail::check<T>(a, b, nullptr);
  if (a.size() == 0 || b.size() == 0) return Variable<T>(Shape(std::move(s)));  // nothing to compute
  return Operation<T>::getCurrentInterface().getBlasInterface().matmul(a, b);
}

template <class T>
Variable<T> matmul(const Tensor<T>& a, const Tensor<T>& b, const Tensor<T>& c) {
  std::vector<unsigned> s = detail::check<T>(a, b, &c);
  if (a.size() == 0 || b.size() == 0) return Variable<T>(Shape(std::move(s)));
  return Operation<T>::getCurrentInterface().getBlasInterface().matmul(a, b, c);
}

}  // namespace blas

namespace data {

template <class T>
void set(Variable<T>& a, const T* values) {
  Operation<T>::getCurrentInterface().getDataInterface().set(a, values);
}
template <class T>
void set(Variable<T>& a, std::vector<T> values) {
  if (values.size() != a.size()) throw InvalidArgumentError("the length of vector and variable is unequal");
  Operation<T>::getCurrentInterface().getDataInterface().set(a, std::move(values));
}
template <class T>
Variable<T> set(std::vector<T> values, Shape shape) {
  Variable<T> v(std::move(shape));
  set(v, std::move(values));
  return v;
}
template <class T>
std::vector<T> get(const Tensor<T>& a) {
  std::vector<T> out(a.size());
  if (a.size() > 0) Operation<T>::getCurrentInterface().getDataInterface().get(a, out.data());
  return out;
}
template <class T>
void zeros(Variable<T>& a) {
  Operation<T>::getCurrentInterface().getDataInterface().zeros(a);
}
template <class T>
void ones(Variable<T>& a) {
  Operation<T>::getCurrentInterface().getDataInterface().ones(a);
}
template <class T>
void fill(Variable<T>& a, T value) {
  Operation<T>::getCurrentInterface().getDataInterface().fill(a, value);
}
template <class T>
Variable<T> copy(const Tensor<T>& a) {
  return Operation<T>::getCurrentInterface().getDataInterface().copy(a);
}

}  // namespace data

namespace quantization {

template <class T>
std::tuple<Variable<T>, Variable<float>, Variable<float>> quantize(const Tensor<float>& a) {
  return Operation<T>::getCurrentInterface().getQuantizationInterface().quantize(a);
}
template <class T>
Variable<T> quantize(const Tensor<float>& a, const Tensor<float>& minValue, const Tensor<float>& maxValue) {
  return Operation<T>::getCurrentInterface().getQuantizationInterface().quantize(a, minValue, maxValue);
}
template <class T, class TI>
Variable<T> requantize(const Tensor<TI>& a, const Tensor<float>& minInput, const Tensor<float>& maxInput,
                       const Tensor<float>& minOutput, const Tensor<float>& maxOutput) {
  return Operation<T>::getCurrentInterface().getQuantizationInterface().requantize(a, minInput, maxInput, minOutput,
                                                                                   maxOutput);
}
template <class T>
Variable<float> dequantize(const Tensor<T>& a, const Tensor<float>& minValue, const Tensor<float>& maxValue) {
  return Operation<T>::getCurrentInterface().getQuantizationInterface().dequantize(a, minValue, maxValue);
}

}  // namespace quantization

namespace math {

template <class T>
Variable<T> softmax(const Tensor<T>& a, size_t axis) {
  if (axis >= a.shape().size()) throw InvalidArgumentError("invalid axis");
  return Operation<T>::getCurrentInterface().getActivationInterface().softmax(a, axis);
}
template <class T>
Variable<T> gelu_accurate(const Tensor<T>& a) {
  if (a.size() == 0) throw InvalidArgumentError("invalid tensor");
  return Operation<T>::getCurrentInterface().getActivationInterface().geluAccurate(a);
}
// tfcc::math::sigmoid, tanh, relu, softplus, log, rsqrt, erf, abs, sign (tfcc/core/operations/tfcc_math.h); neg,
// reciprocal and sqrt stand for 0 - a, 1 / a and 1 / rsqrt(a) as the reference's runtime writes them
template <class T>
Variable<T> unary(const Tensor<T>& a, UnaryFunction f) {
  if (a.size() == 0) throw InvalidArgumentError("invalid tensor");
  return Operation<T>::getCurrentInterface().getActivationInterface().unary(a, static_cast<int>(f));
}
#define TFCC_UNARY_FUNCTION(NAME, VALUE) \
  template <class T>                     \
  Variable<T> NAME(const Tensor<T>& a) { return unary(a, UnaryFunction::VALUE); }
TFCC_UNARY_FUNCTION(sigmoid, SIGMOID)
TFCC_UNARY_FUNCTION(tanh, TANH)
TFCC_UNARY_FUNCTION(relu, RELU)
TFCC_UNARY_FUNCTION(softplus, SOFTPLUS)
TFCC_UNARY_FUNCTION(log, LOG)
TFCC_UNARY_FUNCTION(rsqrt, RSQRT)
TFCC_UNARY_FUNCTION(erf, ERF)
TFCC_UNARY_FUNCTION(abs, ABS)
TFCC_UNARY_FUNCTION(sign, SIGN)
#undef TFCC_UNARY_FUNCTION
namespace detail {
// _get_broadcast_shape of tfcc/core/operations/tfcc_math.cpp:38-86: numpy-style right-aligned broadcasting (extents
// equal or 1); runs of dimensions of the same kind (equal / first broadcast / second broadcast) are merged, so the
// interface sees two shapes of equal rank.  Returns (result shape, merged shape of s1, merged shape of s2).
inline std::tuple<Shape, Shape, Shape> broadcast_shapes(const Shape& s1, const Shape& s2) {
  if (s1.size() == 0 || s2.size() == 0) throw InvalidArgumentError("invalid tensor shape");
  std::vector<unsigned> resultS = s1.size() > s2.size() ? s1.toVector() : s2.toVector(), newS1, newS2;
  for (size_t i = 0; i < s1.size() && i < s2.size(); ++i) {
    const unsigned l1 = s1[s1.size() - 1 - i], l2 = s2[s2.size() - 1 - i];
    if (l1 != l2 && l1 != 1 && l2 != 1) throw InvalidArgumentError("broadcast failed");
    // the reference takes max(l1, l2): an empty dimension against 1 would come out as 1 and the empty operand be read
    resultS[resultS.size() - 1 - i] = l1 == 1 ? l2 : l1;
  }
  auto kind = [](unsigned l1, unsigned l2) { return l1 == l2 ? 0 : l1 == 1 ? 1 : 2; };
  const size_t maxLen = std::max(s1.size(), s2.size());
  unsigned len1 = s1[s1.size() - 1], len2 = s2[s2.size() - 1];
  int type = kind(len1, len2);
  for (size_t i = 1; i < maxLen; ++i) {
    const unsigned l1 = i < s1.size() ? s1[s1.size() - 1 - i] : 1, l2 = i < s2.size() ? s2[s2.size() - 1 - i] : 1;
    if (kind(l1, l2) != type) {
      newS1.insert(newS1.begin(), len1);
      newS2.insert(newS2.begin(), len2);
      type = kind(l1, l2);
      len1 = l1;
      len2 = l2;
    } else {
      len1 *= l1;
      len2 *= l2;
    }
  }
  if (len1 != 1 || len2 != 1 || newS1.empty()) {
    newS1.insert(newS1.begin(), len1);
    newS2.insert(newS2.begin(), len2);
  }
  return std::make_tuple(Shape(std::move(resultS)), Shape(std::move(newS1)), Shape(std::move(newS2)));
}

template <class T, class F>
Variable<T> broadcast_binary(const Tensor<T>& a, const Tensor<T>& b, F call) {
  Shape resultS, newAS, newBS;
  std::tie(resultS, newAS, newBS) = broadcast_shapes(a.shape(), b.shape());
  if (resultS.area() == 0) return Variable<T>(resultS);
  View<T> aView(a, newAS), bView(b, newBS);
  Variable<T> result = call(Operation<T>::getCurrentInterface().getArithmeticInterface(), aView, bView);
  result.reshape(std::move(resultS));
  return result;
}
}  // namespace detail

// tfcc::math::add / sub / mul / div (tfcc/core/operations/tfcc_math.cpp:88-150)
template <class T>
Variable<T> add(const Tensor<T>& a, const Tensor<T>& b) {
  return detail::broadcast_binary(a, b, [](ArithmeticInterface<T>& i, const Tensor<T>& x, const Tensor<T>& y) { return i.add(x, y); });
}
template <class T>
Variable<T> sub(const Tensor<T>& a, const Tensor<T>& b) {
  return detail::broadcast_binary(a, b, [](ArithmeticInterface<T>& i, const Tensor<T>& x, const Tensor<T>& y) { return i.sub(x, y); });
}
template <class T>
Variable<T> mul(const Tensor<T>& a, const Tensor<T>& b) {
  return detail::broadcast_binary(a, b, [](ArithmeticInterface<T>& i, const Tensor<T>& x, const Tensor<T>& y) { return i.mul(x, y); });
}
template <class T>
Variable<T> div(const Tensor<T>& a, const Tensor<T>& b) {
  return detail::broadcast_binary(a, b, [](ArithmeticInterface<T>& i, const Tensor<T>& x, const Tensor<T>& y) { return i.div(x, y); });
}
// tfcc::math::min / max of two tensors or a tensor and a value (tfcc/core/operations/tfcc_math.cpp:257-320)
template <class T>
Variable<T> min(const Tensor<T>& a, const Tensor<T>& b) {
  Shape resultS, newAS, newBS;
  std::tie(resultS, newAS, newBS) = detail::broadcast_shapes(a.shape(), b.shape());
  if (resultS.area() == 0) return Variable<T>(resultS);
  View<T> aView(a, newAS), bView(b, newBS);
  Variable<T> result = Operation<T>::getCurrentInterface().getMinMaxInterface().min(aView, bView);
  result.reshape(std::move(resultS));
  return result;
}
template <class T>
Variable<T> max(const Tensor<T>& a, const Tensor<T>& b) {
  Shape resultS, newAS, newBS;
  std::tie(resultS, newAS, newBS) = detail::broadcast_shapes(a.shape(), b.shape());
  if (resultS.area() == 0) return Variable<T>(resultS);
  View<T> aView(a, newAS), bView(b, newBS);
  Variable<T> result = Operation<T>::getCurrentInterface().getMinMaxInterface().max(aView, bView);
  result.reshape(std::move(resultS));
  return result;
}
template <class T>
Variable<T> min(const Tensor<T>& a, T b) {
  if (a.size() == 0) throw InvalidArgumentError("invalid tensor");
  return Operation<T>::getCurrentInterface().getMinMaxInterface().min(a, b);
}
template <class T>
Variable<T> min(T a, const Tensor<T>& b) { return min(b, a); }
template <class T>
Variable<T> max(const Tensor<T>& a, T b) {
  if (a.size() == 0) throw InvalidArgumentError("invalid tensor");
  return Operation<T>::getCurrentInterface().getMinMaxInterface().max(a, b);
}
template <class T>
Variable<T> max(T a, const Tensor<T>& b) { return max(b, a); }
// tfcc::math::leaky_relu, pow, clip (tfcc/core/operations/tfcc_math.cpp:343-350, :423-452, :536-543).  The reference
// expands both operands of pow to the result's shape first; here the kernel reads them through their own strides.
template <class T>
Variable<T> leaky_relu(const Tensor<T>& a, T alpha) {
  if (a.size() == 0) throw InvalidArgumentError("invalid tensor");
  return Operation<T>::getCurrentInterface().getActivationInterface().leakyRelu(a, alpha);
}
template <class T>
Variable<T> pow(const Tensor<T>& a, T exponent) {
  if (a.size() == 0) throw InvalidArgumentError("invalid tensor");
  return Operation<T>::getCurrentInterface().getActivationInterface().pow(a, exponent);
}
template <class T>
Variable<T> pow(const Tensor<T>& a, const Tensor<T>& exponent) {
  if (a.size() == 0 || exponent.size() == 0) throw InvalidArgumentError("invalid tensor");
  Shape resultS, newAS, newBS;
  std::tie(resultS, newAS, newBS) = detail::broadcast_shapes(a.shape(), exponent.shape());
  View<T> aView(a, newAS), bView(exponent, newBS);
  Variable<T> result = Operation<T>::getCurrentInterface().getActivationInterface().pow(aView, bView);
  result.reshape(std::move(resultS));
  return result;
}
template <class T>
Variable<T> pow(T a, const Tensor<T>& exponent) {
  if (exponent.size() == 0) throw InvalidArgumentError("invalid tensor");
  return Operation<T>::getCurrentInterface().getActivationInterface().pow(a, exponent);
}
template <class T>
Variable<T> clip(const Tensor<T>& a, T minValue, T maxValue) {
  if (a.size() == 0) throw InvalidArgumentError("invalid tensor");
  return Operation<T>::getCurrentInterface().getBasicInterface().clip(a, minValue, maxValue);
}
// tfcc::math::argmax (tfcc/core/operations/tfcc_math.cpp:675-684): the axis stays with length 1
template <class T>
Variable<int64_t> argmax(const Tensor<T>& a, size_t axis) {
  if (a.size() == 0) throw InvalidArgumentError("invalid tensor");
  if (axis >= a.shape().size()) throw InvalidArgumentError("invalid axis");
  return Operation<T>::getCurrentInterface().getBasicInterface().argmax(a, axis);
}
// tfcc::math::top_k (tfcc/core/operations/tfcc_math.cpp:546-556): the k largest along the last axis and their positions
template <class T>
std::tuple<Variable<T>, Variable<uint32_t>> top_k(const Tensor<T>& a, unsigned k) {
  if (a.size() == 0) throw InvalidArgumentError("invalid tensor");
  if (a.shape(a.shape().size() - 1) < k) throw InvalidArgumentError("invalid k");
  return Operation<T>::getCurrentInterface().getBasicInterface().topK(a, k);
}
// tfcc::math::reduce_sum / mean / prod / max / min (tfcc/core/operations/tfcc_math.cpp:464-522)
#define TFCC_REDUCE_FUNCTION(NAME, METHOD)                                                   \
  template <class T>                                                                         \
  Variable<T> NAME(const Tensor<T>& a, size_t keep) {                                        \
    if (a.size() == 0) throw InvalidArgumentError("invalid tensor");                         \
    if (keep >= a.shape().size()) throw InvalidArgumentError("invalid keep dims");           \
    return Operation<T>::getCurrentInterface().getReduceInterface().METHOD(a, keep);         \
  }
TFCC_REDUCE_FUNCTION(reduce_sum, reduceSum)
TFCC_REDUCE_FUNCTION(reduce_mean, reduceMean)
TFCC_REDUCE_FUNCTION(reduce_prod, reduceProd)
TFCC_REDUCE_FUNCTION(reduce_max, reduceMax)
TFCC_REDUCE_FUNCTION(reduce_min, reduceMin)
#undef TFCC_REDUCE_FUNCTION
template <class T>
Variable<T> transform(const Tensor<T>& a, T alpha, T beta) {
  return Operation<T>::getCurrentInterface().getTransformationInterface().transform(a, alpha, beta);
}
template <class T>
Variable<T> transform2(const Tensor<T>& a, T alpha, T beta) {
  return Operation<T>::getCurrentInterface().getTransformationInterface().transform2(a, alpha, beta);
}

}  // namespace math

// tfcc::relation (tfcc/core/operations/tfcc_relation.cpp:81-300): tensor against value, value against tensor (the
// mirrored relation on the tensor) and tensor against tensor (the difference against 0, with broadcasting).
namespace relation {
namespace detail {
inline Relation mirrored(Relation r) {
  switch (r) {
    case Relation::GREATER: return Relation::LESS;
    case Relation::GREATER_EQUAL: return Relation::LESS_EQUAL;
    case Relation::LESS: return Relation::GREATER;
    case Relation::LESS_EQUAL: return Relation::GREATER_EQUAL;
    default: return r;
  }
}
}  // namespace detail
template <class T>
Variable<uint8_t> compare(const Tensor<T>& a, T b, Relation r) {
  if (a.size() == 0) throw InvalidArgumentError();
  return Operation<T>::getCurrentInterface().getComparisonInterface().compare(a, b, r);
}
template <class T>
Variable<uint8_t> compare(T a, const Tensor<T>& b, Relation r) {
  return compare(b, a, detail::mirrored(r));
}
template <class T>
Variable<uint8_t> compare(const Tensor<T>& a, const Tensor<T>& b, Relation r) {
  if (a.size() == 0 || b.size() == 0) throw InvalidArgumentError();
  Shape resultS, newAS, newBS;
  std::tie(resultS, newAS, newBS) = math::detail::broadcast_shapes(a.shape(), b.shape());
  View<T> aView(a, newAS), bView(b, newBS);
  Variable<uint8_t> result = Operation<T>::getCurrentInterface().getComparisonInterface().compareDifference(aView, bView, r);
  result.reshape(std::move(resultS));
  return result;
}
#define TFCC_RELATION_FUNCTION(NAME, VALUE)                                                          \
  template <class T>                                                                                 \
  Variable<uint8_t> NAME(const Tensor<T>& a, T b) { return compare(a, b, Relation::VALUE); }         \
  template <class T>                                                                                 \
  Variable<uint8_t> NAME(T a, const Tensor<T>& b) { return compare(a, b, Relation::VALUE); }         \
  template <class T>                                                                                 \
  Variable<uint8_t> NAME(const Tensor<T>& a, const Tensor<T>& b) { return compare(a, b, Relation::VALUE); }
TFCC_RELATION_FUNCTION(equal, EQUAL)
TFCC_RELATION_FUNCTION(unequal, UNEQUAL)
TFCC_RELATION_FUNCTION(greater, GREATER)
TFCC_RELATION_FUNCTION(greater_equal, GREATER_EQUAL)
TFCC_RELATION_FUNCTION(less, LESS)
TFCC_RELATION_FUNCTION(less_equal, LESS_EQUAL)
#undef TFCC_RELATION_FUNCTION
}  // namespace relation

namespace nn {

template <class T>
Variable<T> layer_normalization(const Tensor<T>& a, const Tensor<T>& gamma, const Tensor<T>& beta, T epsilon,
                                size_t beginNormAxis) {
  return Operation<T>::getCurrentInterface().getNormalizationInterface().layerNormalize(a, gamma, beta, epsilon,
                                                                                        beginNormAxis);
}

}  // namespace nn

namespace data {
// tfcc::data::cast<DST>(a): element-wise static_cast (tfcc/core/operations/tfcc_data.h)
template <class DST, class SRC>
Variable<DST> cast(const Tensor<SRC>& a) {
  if (a.size() == 0) return Variable<DST>(a.shape());
  return Operation<DST>::getCurrentInterface().getDataInterface().cast(a);
}
// tfcc::data::cast_to_boolean(a): 1 where the element is not zero, else 0
template <class T>
Variable<uint8_t> cast_to_boolean(const Tensor<T>& a) {
  if (a.size() == 0) return Variable<uint8_t>(a.shape());
  return Operation<T>::getCurrentInterface().getDataInterface().cast_to_boolean(a);
}
}  // namespace data

namespace base {
// tfcc/core/operations/tfcc_base.cpp:28-41
template <class T>
Variable<T> slice(const Tensor<T>& a, size_t axis, unsigned start, unsigned end) {
  if (axis >= a.shape().size()) throw InvalidArgumentError("invalid axis");
  if (start >= end) throw InvalidArgumentError("start large than end");
  if (start >= a.shape(axis)) throw InvalidArgumentError("invalid start");
  return Operation<T>::getCurrentInterface().getBasicInterface().slice(a, axis, start, end);
}
// tfcc/core/operations/tfcc_base.cpp:86-121
template <class T>
Variable<T> concat(const std::vector<const Tensor<T>*>& values, size_t axis) {
  if (values.size() == 0) throw InvalidArgumentError("values.size could not be zero");
  for (const Tensor<T>* tensor : values) {
    if (axis >= tensor->shape().size()) throw InvalidArgumentError("invalid axis");
    if (tensor->shape().size() != values[0]->shape().size()) throw InvalidArgumentError("invalid shape");
    for (size_t i = 0; i < tensor->shape().size(); ++i)
      if (i != axis && tensor->shape(i) != values[0]->shape(i)) throw InvalidArgumentError("invalid shape");
  }
  return Operation<T>::getCurrentInterface().getBasicInterface().concat(values, axis);
}
template <class T>
Variable<T> concat(std::initializer_list<const Tensor<T>*> values, size_t axis) {
  return concat(std::vector<const Tensor<T>*>(values), axis);
}
// tfcc/core/operations/tfcc_base.cpp:162-181: a written into b at position `start` along `axis`
template <class T>
void assign_to(const Tensor<T>& a, size_t axis, unsigned start, Variable<T>& b) {
  if (a.shape().size() != b.shape().size()) throw InvalidArgumentError("dimensions not match");
  if (axis >= a.shape().size()) throw InvalidArgumentError("invalid axis");
  for (size_t i = 0; i < a.shape().size(); ++i)
    if (i != axis && a.shape(i) != b.shape(i)) throw InvalidArgumentError("shape not match");
  if (b.shape(axis) < start + a.shape(axis)) throw InvalidArgumentError("b is too small to assign");
  Operation<T>::getCurrentInterface().getBasicInterface().assignTo(a, axis, start, b);
}
// tfcc/core/operations/tfcc_base.cpp:43-59: num equal parts along axis
template <class T>
std::vector<Variable<T>> split(const Tensor<T>& a, size_t num, size_t axis) {
  if (axis >= a.shape().size()) throw InvalidArgumentError("invalid axis");
  if (num == 0 || a.shape(axis) % num != 0) throw InvalidArgumentError("invalid num");
  const unsigned s = a.shape(axis) / static_cast<unsigned>(num);
  std::vector<Variable<T>> values;
  BasicInterface<T>& basic = Operation<T>::getCurrentInterface().getBasicInterface();
  for (size_t i = 0; i < num; ++i)
    values.emplace_back(basic.slice(a, axis, static_cast<unsigned>(i) * s, static_cast<unsigned>(i + 1) * s));
  return values;
}
// tfcc/core/operations/tfcc_base.cpp:184-210: values of one shape joined along a new dimension at axis
template <class T>
Variable<T> stack(const std::vector<const Tensor<T>*>& values, size_t axis) {
  if (values.size() == 0) throw InvalidArgumentError("values's size should be greater than zero");
  if (axis > values[0]->shape().size()) throw InvalidArgumentError("invalid axis");
  std::vector<unsigned> s = values[0]->shape().toVector();
  s.insert(s.begin() + axis, 1);
  std::vector<View<T>> views;
  for (const Tensor<T>* tensor : values) {
    if (tensor->shape() != values[0]->shape()) throw InvalidArgumentError("the shape of values are unequal");
    views.emplace_back(*tensor, Shape(s));
  }
  std::vector<const Tensor<T>*> tensors;
  for (View<T>& view : views) tensors.push_back(&view);
  return concat(tensors, axis);
}
// tfcc/core/operations/tfcc_base.cpp:136-160: zeros in front of and behind a along axis
template <class T>
Variable<T> pad(const Tensor<T>& a, size_t axis, unsigned paddingHead, unsigned paddingEnd) {
  if (axis >= a.shape().size()) throw InvalidArgumentError("invalid axis");
  std::vector<unsigned> s = a.shape().toVector();
  Variable<T> head, tail;
  std::vector<const Tensor<T>*> parts;
  DataInterface<T>& dataInterface = Operation<T>::getCurrentInterface().getDataInterface();
  if (paddingHead > 0) {
    s[axis] = paddingHead;
    head = Variable<T>(Shape(s));
    dataInterface.zeros(head);
    parts.push_back(&head);
  }
  parts.push_back(&a);
  if (paddingEnd > 0) {
    s[axis] = paddingEnd;
    tail = Variable<T>(Shape(s));
    dataInterface.zeros(tail);
    parts.push_back(&tail);
  }
  return concat(parts, axis);
}
}  // namespace base

namespace base {
// tfcc::base::tril / triu (tfcc/core/operations/tfcc_base.cpp:249-266)
template <class T>
Variable<T> tril(const Tensor<T>& a, int64_t k) {
  if (a.shape().size() != 2) throw InvalidArgumentError("invalid shape");
  return Operation<T>::getCurrentInterface().getBasicInterface().triangle(a, k, false);
}
template <class T>
Variable<T> triu(const Tensor<T>& a, int64_t k) {
  if (a.shape().size() != 2) throw InvalidArgumentError("invalid shape");
  return Operation<T>::getCurrentInterface().getBasicInterface().triangle(a, k, true);
}
}  // namespace base

namespace nn {
// tfcc::nn::where (tfcc/core/operations/tfcc_nn.cpp:496-523)
template <class T>
Variable<T> where(const Tensor<uint8_t>& condition, const Tensor<T>& x, const Tensor<T>& y) {
  if (condition.shape() != x.shape() || x.shape() != y.shape()) throw InvalidArgumentError("condition x and y has different shape");
  return Operation<T>::getCurrentInterface().getBasicInterface().where(condition, &x, T(), &y, T());
}
template <class T>
Variable<T> where(const Tensor<uint8_t>& condition, T x, const Tensor<T>& y) {
  if (condition.shape() != y.shape()) throw InvalidArgumentError("condition x and y has different shape");
  return Operation<T>::getCurrentInterface().getBasicInterface().where(condition, nullptr, x, &y, T());
}
template <class T>
Variable<T> where(const Tensor<uint8_t>& condition, const Tensor<T>& x, T y) {
  if (condition.shape() != x.shape()) throw InvalidArgumentError("condition x and y has different shape");
  return Operation<T>::getCurrentInterface().getBasicInterface().where(condition, &x, T(), nullptr, y);
}
// tfcc::nn::gather (tfcc/core/operations/tfcc_nn.cpp:345-385) for int32 / uint32 / int64 / uint64 indices
template <class T, class IDX>
Variable<T> gather(const Tensor<T>& params, const Tensor<IDX>& indices) {
  static_assert(ElementCode<IDX>::value >= 4 && ElementCode<IDX>::value <= 7, "indices of 32 or 64 bits");
  if (params.size() == 0) throw InvalidArgumentError("invalid tensor");
  std::vector<unsigned> shape = indices.shape().toVector();
  for (size_t i = 1; i < params.shape().size(); ++i) shape.push_back(params.shape(i));
  if (indices.size() == 0) return Variable<T>(Shape(std::move(shape)));
  return Operation<T>::getCurrentInterface().getBasicInterface().gather(params, indices.data(), ElementCode<IDX>::value,
                                                                      indices.shape());
}
}  // namespace nn

namespace rnn {

namespace detail {
// tfcc::rnn::lstm_forward / lstm_backward (tfcc/core/operations/tfcc_rnn.cpp:29-81, 83-135): the same checks,
// gate layout, forget bias 0 and output order (outputs in the order the steps are taken).  The products of the
// inputs with inputKernel do not depend on the recurrence, so all steps share one matmul of [seq * batch, length];
// each step then costs one launch (the product with stateKernel and the cell together, where the device offers
// that) or two (matmul, then a cell launch), and writes h straight into its row block of the result.
template <class T>
std::tuple<Variable<T>, Variable<T>, Variable<T>> lstm_sequence(bool backward, const Tensor<T>& a,
                                                                const Tensor<T>& inputKernel,
                                                                const Tensor<T>& stateKernel, const Tensor<T>& bias,
                                                                const Tensor<T>& ih, const Tensor<T>& ic) {
  if (a.shape().size() != 3) throw InvalidArgumentError("invalid input");
  const unsigned seq = a.shape(0), batch = a.shape(1), length = a.shape(2);
  if (ih.shape() != ic.shape() || ih.shape().size() != 2 || ih.shape(0) != batch)
    throw InvalidArgumentError("invalid ih or ic");
  const unsigned hidden = ih.shape(1);
  if (inputKernel.shape().size() != 2 || inputKernel.shape(0) != length || inputKernel.shape(1) != hidden * 4)
    throw InvalidArgumentError("invalid input kernel");
  if (stateKernel.shape().size() != 2 || stateKernel.shape(0) != hidden || stateKernel.shape(1) != hidden * 4)
    throw InvalidArgumentError("invalid state kernel");
  if (bias.shape().size() != 1 || bias.shape(0) != 4 * hidden) throw InvalidArgumentError("invalid bias");
  if (a.size() == 0 || hidden == 0) throw InvalidArgumentError("invalid input");

  Interface<T>& interface = Operation<T>::getCurrentInterface();
  View<T> flat(a, Shape({seq * batch, length}));
  Variable<T> inputValues = interface.getBlasInterface().matmul(flat, inputKernel);  // [seq * batch, 4 hidden]
  Variable<T> result({seq, batch, hidden});
  Variable<T> c = interface.getDataInterface().copy(ic);
  const size_t state = static_cast<size_t>(batch) * hidden;
  View<T> h(ih);
  Variable<T> prepared;  // the state kernel as the one-launch step wants it, where the device has such a step
  bool oneLaunch = false;
  try {
    prepared = interface.getCellInterface().prepareLSTMStateKernel(stateKernel, batch);
    oneLaunch = true;
  } catch (const NotImplementedError&) {
  }
  for (unsigned step = 0; step < seq; ++step) {
    const unsigned t = backward ? seq - 1 - step : step;
    View<T> x(inputValues, inputValues.shape(), t * batch, (t + 1) * batch);
    if (oneLaunch) {
      interface.getCellInterface().processLSTMStepInto(c, x, h, prepared, bias, static_cast<T>(0),
                                                       result.data() + step * state, c.data());
    } else {
      Variable<T> stateValues = interface.getBlasInterface().matmul(h, stateKernel);
      interface.getCellInterface().processLSTMCellInto(c, x, stateValues, bias, static_cast<T>(0),
                                                       result.data() + step * state, c.data());
    }
    h = View<T>(result, result.shape(), step, step + 1);
    h.reshape(Shape({batch, hidden}));
  }
  Variable<T> lastH = interface.getDataInterface().copy(h);
  return std::make_tuple(std::move(result), std::move(lastH), std::move(c));
}
}  // namespace detail

template <class T>
std::tuple<Variable<T>, Variable<T>, Variable<T>> lstm_forward(const Tensor<T>& a, const Tensor<T>& inputKernel,
                                                               const Tensor<T>& stateKernel, const Tensor<T>& bias,
                                                               const Tensor<T>& ih, const Tensor<T>& ic) {
  return detail::lstm_sequence(false, a, inputKernel, stateKernel, bias, ih, ic);
}

template <class T>
std::tuple<Variable<T>, Variable<T>, Variable<T>> lstm_backward(const Tensor<T>& a, const Tensor<T>& inputKernel,
                                                                const Tensor<T>& stateKernel, const Tensor<T>& bias,
                                                                const Tensor<T>& ih, const Tensor<T>& ic) {
  return detail::lstm_sequence(true, a, inputKernel, stateKernel, bias, ih, ic);
}

}  // namespace rnn

namespace base {

template <class T>
Variable<T> transpose(const Tensor<T>& a, const std::vector<size_t>& perm) {
  if (perm.size() != a.shape().size()) throw InvalidArgumentError("perm and tensor don't match");
  std::set<size_t> seen(perm.begin(), perm.end());
  if (seen.size() != perm.size() || (!perm.empty() && *seen.rbegin() >= perm.size()))
    throw InvalidArgumentError("invalid perm");
  return Operation<T>::getCurrentInterface().getBasicInterface().transpose(a, perm);
}

}  // namespace base

// a + b, a * s, a + s  (tfcc/core/operations/tfcc_operator.cpp:34-95)
template <class T>
Variable<T> operator+(const Tensor<T>& a, const Tensor<T>& b) {
  return math::add(a, b);
}
template <class T>
Variable<T> operator*(const Tensor<T>& a, T s) {
  return math::transform(a, s, static_cast<T>(0));
}
template <class T>
Variable<T> operator+(const Tensor<T>& a, T s) {
  return math::transform(a, static_cast<T>(1), s);
}
template <class T>
Variable<T> operator-(const Tensor<T>& a, T s) {
  return math::transform(a, static_cast<T>(1), static_cast<T>(-s));
}
template <class T>
Variable<T> operator/(const Tensor<T>& a, T s) {
  return math::transform2(a, s, static_cast<T>(0));
}
template <class T>
Variable<T> operator+(T s, const Tensor<T>& a) {
  return math::transform(a, static_cast<T>(1), s);
}
template <class T>
Variable<T> operator*(T s, const Tensor<T>& a) {
  return math::transform(a, s, static_cast<T>(0));
}
template <class T>
Variable<T> operator-(T s, const Tensor<T>& a) {
  return math::transform(a, static_cast<T>(-1), s);
}
template <class T>
Variable<T> operator-(const Tensor<T>& a, const Tensor<T>& b) {
  return math::sub(a, b);
}
template <class T>
Variable<T> operator*(const Tensor<T>& a, const Tensor<T>& b) {
  return math::mul(a, b);
}
template <class T>
Variable<T> operator/(const Tensor<T>& a, const Tensor<T>& b) {
  return math::div(a, b);
}

}  // namespace tfcc
