// The operations this runtime knows.  Each follows the accept/reject rules of the reference's
// operation of the same name (tfcc_runtime/operations/<package>/<name>.cpp): input and output
// counts, the Any's message type, and the element types of the symbols involved; a rejected node
// is offered to the next registered operation and ends as UnknowNodeError when nobody takes it.
//
//   math.Matmul, math.MatmulWithBias    operations/math/matmul.cpp:52-81, matmulwithbias.cpp:52-88
//   math.Add / Sub / Mul / Div          operations/math/add.cpp:80-126 (tensor and value operand forms)
//   math.Gelu, math.Softmax             operations/math/gelu.cpp, softmax.cpp
//   math.Abs / Erf / Log / Neg / Reciprocal / Relu / Rsqrt / Sigmoid / Sign / Softplus / Sqrt / Tanh
//                                       operations/math/<name>.cpp
//   nn.LayerNormalization               operations/nn/layernormalization.cpp:52-88
//   rnn.BidirectionalLSTM               operations/rnn/bidirectionallstm.cpp:27-128
//   base.Squeeze / Unsqueeze / Flatten  operations/base/squeeze.cpp, unsqueeze.cpp, flatten.cpp (Views of the input)
//   base.GetShape, base.GetDimension    operations/base/getshape.cpp, getdimension.cpp
//   base.At / At1 / ToTensor / ToValue / ToVector
//                                       operations/base/at.cpp, at1.cpp, totensor.cpp, tovalue.cpp, tovector.cpp
//   base.Split / Stack / SliceV2 / Pad  operations/base/split.cpp, stack.cpp, slicev2.cpp, pad.cpp
//   nn.Gather, base.Cast, base.SliceV1, base.Concat
//                                       operations/nn/gather.cpp, base/cast.cpp, slicev1.cpp, concat.cpp
//   base.Transpose, base.Reshape, base.Identity, base.CreateVector
//                                       operations/base/transpose.cpp, reshape.cpp:27-59,74-104,
//                                       identity.cpp, createvector.cpp:63-121
#include <algorithm>
#include <array>
#include <cmath>
#include <functional>
#include <map>
#include <type_traits>

#include "runtime.h"

namespace tfcc {
namespace runtime {

namespace {

bool same_dtype(Graph& g, const std::vector<std::string>& names, DataType dtype) {
  for (const std::string& n : names)
    if (g.getSymbolManager().getSymbolInfo(n).dtype != dtype) return false;
  return true;
}

SymbolType stype_of(Graph& g, const std::string& name) { return g.getSymbolManager().getSymbolInfo(name).stype; }

template <class T>
class TypedOperation : public Operation {
 protected:
  static constexpr DataType DTYPE = DataTypeOf<T>::value;
  std::string _url;

 public:
  explicit TypedOperation(const std::string& message) : _url(type_url(message)) {}
  std::string getOperationTypeUrl() const override { return _url; }
};

// ---- math.Matmul / math.MatmulWithBias ------------------------------------------------------------------
template <class T>
class Matmul : public TypedOperation<T> {
 public:
  Matmul() : TypedOperation<T>("math.Matmul") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 2 || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, this->DTYPE) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    auto& sm = graph.getSymbolManager();
    const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
    const Tensor<T>* b = sm.getTensor(node.inputs[1], T());
    Variable<T>* out = sm.getVariable(node.outputs[0], T());
    graph.addStep([a, b, out] { *out = blas::matmul(*a, *b); });
    return true;
  }
};

template <class T>
class MatmulWithBias : public TypedOperation<T> {
 public:
  MatmulWithBias() : TypedOperation<T>("math.MatmulWithBias") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 3 || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, this->DTYPE) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    auto& sm = graph.getSymbolManager();
    const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
    const Tensor<T>* b = sm.getTensor(node.inputs[1], T());
    const Tensor<T>* bias = sm.getTensor(node.inputs[2], T());
    Variable<T>* out = sm.getVariable(node.outputs[0], T());
    graph.addStep([a, b, bias, out] { *out = blas::matmul(*a, *b, *bias); });
    return true;
  }
};

// ---- math.Add / Sub / Mul / Div / Pow / Max / Min --------------------------------------------------------
// tensor (x) tensor, tensor (x) value, value (x) tensor and value (x) value forms, as
// tfcc_runtime/operations/math/{add,sub,mul,div,pow,max,min}.cpp register them.
enum class Arith { ADD, SUB, MUL, DIV, POW, MAX, MIN };

template <Arith OP, class T>
class Arithmetic : public TypedOperation<T> {
  static const char* message() {
    switch (OP) {
      case Arith::ADD: return "math.Add";
      case Arith::SUB: return "math.Sub";
      case Arith::MUL: return "math.Mul";
      case Arith::DIV: return "math.Div";
      case Arith::POW: return "math.Pow";
      case Arith::MAX: return "math.Max";
      default: return "math.Min";
    }
  }
  static Variable<T> tt(const Tensor<T>& a, const Tensor<T>& b) {
    switch (OP) {
      case Arith::ADD: return a + b;
      case Arith::SUB: return a - b;
      case Arith::MUL: return a * b;
      case Arith::DIV: return a / b;
      case Arith::POW: return math::pow(a, b);
      case Arith::MAX: return math::max(a, b);
      default: return math::min(a, b);
    }
  }
  static Variable<T> tv(const Tensor<T>& a, T b) {
    switch (OP) {
      case Arith::ADD: return a + b;
      case Arith::SUB: return a - b;
      case Arith::MUL: return a * b;
      case Arith::DIV: return a / b;
      case Arith::POW: return math::pow(a, b);
      case Arith::MAX: return math::max(a, b);
      default: return math::min(a, b);
    }
  }
  static Variable<T> vt(T a, const Tensor<T>& b) {
    switch (OP) {
      case Arith::ADD: return a + b;
      case Arith::SUB: return a - b;
      case Arith::MUL: return a * b;
      case Arith::DIV: throw NotImplementedError("value / tensor");
      case Arith::POW: return math::pow(a, b);
      case Arith::MAX: return math::max(a, b);
      default: return math::min(a, b);
    }
  }
  static T vv(T a, T b) {
    switch (OP) {
      case Arith::ADD: return a + b;
      case Arith::SUB: return a - b;
      case Arith::MUL: return a * b;
      case Arith::DIV: return a / b;
      case Arith::POW: return static_cast<T>(std::pow(a, b));
      case Arith::MAX: return std::max(a, b);
      default: return std::min(a, b);
    }
  }

 public:
  Arithmetic() : TypedOperation<T>(message()) {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 2 || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, this->DTYPE) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    auto& sm = graph.getSymbolManager();
    const SymbolType s0 = stype_of(graph, node.inputs[0]), s1 = stype_of(graph, node.inputs[1]);
    if (is_tensor(s0) && is_tensor(s1)) {
      const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
      const Tensor<T>* b = sm.getTensor(node.inputs[1], T());
      Variable<T>* out = sm.getVariable(node.outputs[0], T());
      graph.addStep([a, b, out] { *out = tt(*a, *b); });
    } else if (is_tensor(s0) && is_value(s1)) {
      const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
      const T* b = sm.getValue(node.inputs[1], T());
      Variable<T>* out = sm.getVariable(node.outputs[0], T());
      graph.addStep([a, b, out] { *out = tv(*a, *b); });
    } else if (is_value(s0) && is_tensor(s1)) {
      const T* a = sm.getValue(node.inputs[0], T());
      const Tensor<T>* b = sm.getTensor(node.inputs[1], T());
      Variable<T>* out = sm.getVariable(node.outputs[0], T());
      graph.addStep([a, b, out] { *out = vt(*a, *b); });
    } else if (is_value(s0) && is_value(s1)) {
      const T* a = sm.getValue(node.inputs[0], T());
      const T* b = sm.getValue(node.inputs[1], T());
      T* out = sm.getValue(node.outputs[0], T());
      graph.addStep([a, b, out] { *out = vv(*a, *b); });
    } else {
      return false;
    }
    return true;
  }
};

// ---- element-wise functions of one symbol ---------------------------------------------------------------
// tensor -> tensor and value -> value forms, as tfcc_runtime/operations/math/{abs,erf,log,neg,reciprocal,relu,
// rsqrt,sigmoid,sign,softplus,sqrt,tanh}.cpp register them (the value forms exist there for neg, reciprocal,
// rsqrt and sqrt: neg.cpp:41, reciprocal.cpp:42, rsqrt.cpp:41, sqrt.cpp:41)
template <UnaryFunction F, class T>
class Unary : public TypedOperation<T> {
  static const char* message() {
    switch (F) {
      case UnaryFunction::SIGMOID: return "math.Sigmoid";
      case UnaryFunction::TANH: return "math.Tanh";
      case UnaryFunction::RELU: return "math.Relu";
      case UnaryFunction::SOFTPLUS: return "math.Softplus";
      case UnaryFunction::LOG: return "math.Log";
      case UnaryFunction::RSQRT: return "math.Rsqrt";
      case UnaryFunction::ERF: return "math.Erf";
      case UnaryFunction::ABS: return "math.Abs";
      case UnaryFunction::SIGN: return "math.Sign";
      case UnaryFunction::NEG: return "math.Neg";
      case UnaryFunction::RECIPROCAL: return "math.Reciprocal";
      default: return "math.Sqrt";
    }
  }
  static constexpr bool kValueForm = F == UnaryFunction::NEG || F == UnaryFunction::RECIPROCAL ||
                                     F == UnaryFunction::RSQRT || F == UnaryFunction::SQRT;
  static T value(T a) {
    if (F == UnaryFunction::NEG) return static_cast<T>(0) - a;
    if (F == UnaryFunction::RECIPROCAL) return static_cast<T>(1) / a;
    if (F == UnaryFunction::RSQRT) return static_cast<T>(1) / static_cast<T>(std::sqrt(a));
    return static_cast<T>(std::sqrt(a));
  }

 public:
  Unary() : TypedOperation<T>(message()) {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 1 || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, this->DTYPE) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    auto& sm = graph.getSymbolManager();
    const SymbolType si = stype_of(graph, node.inputs[0]), so = stype_of(graph, node.outputs[0]);
    if (is_tensor(si) && is_tensor(so)) {
      const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
      Variable<T>* out = sm.getVariable(node.outputs[0], T());
      graph.addStep([a, out] { *out = math::unary(*a, F); });
      return true;
    }
    if (kValueForm && is_value(si) && is_value(so)) {
      const T* a = sm.getValue(node.inputs[0], T());
      T* out = sm.getValue(node.outputs[0], T());
      graph.addStep([a, out] { *out = value(*a); });
      return true;
    }
    return false;
  }
};

// ---- math.Gelu / math.Softmax -----------------------------------------------------------------------------
template <class T>
class Gelu : public TypedOperation<T> {
 public:
  Gelu() : TypedOperation<T>("math.Gelu") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 1 || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, this->DTYPE) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    auto& sm = graph.getSymbolManager();
    const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
    Variable<T>* out = sm.getVariable(node.outputs[0], T());
    graph.addStep([a, out] { *out = math::gelu_accurate(*a); });
    return true;
  }
};

template <class T>
class Softmax : public TypedOperation<T> {
 public:
  Softmax() : TypedOperation<T>("math.Softmax") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 1 || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, this->DTYPE) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    size_t axis = 0;
    wire::Reader r(node.operation);
    uint32_t f, t;
    while (r.next(f, t)) {
      if (f == 1 && t == 0) axis = static_cast<size_t>(r.varint());
      else r.skip(t);
    }
    auto& sm = graph.getSymbolManager();
    const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
    Variable<T>* out = sm.getVariable(node.outputs[0], T());
    graph.addStep([a, out, axis] { *out = math::softmax(*a, axis); });
    return true;
  }
};

// ---- math.ReduceSum / ReduceMean / ReduceProd / ReduceMax / ReduceMin --------------------------------------
// The axes are sorted and moved behind the others with a transpose when they are not the trailing ones already; the
// result keeps them with length 1 (tfcc_runtime/operations/math/reducemean.cpp:27-45, utils/reduceutils.h:25-50).
enum class Reduction { SUM, MEAN, PROD, MAX, MIN };

template <Reduction R, class T>
class Reduce : public TypedOperation<T> {
  static const char* message() {
    switch (R) {
      case Reduction::SUM: return "math.ReduceSum";
      case Reduction::MEAN: return "math.ReduceMean";
      case Reduction::PROD: return "math.ReduceProd";
      case Reduction::MAX: return "math.ReduceMax";
      default: return "math.ReduceMin";
    }
  }
  static Variable<T> trailing(const Tensor<T>& a, size_t keep) {
    switch (R) {
      case Reduction::SUM: return math::reduce_sum(a, keep);
      case Reduction::MEAN: return math::reduce_mean(a, keep);
      case Reduction::PROD: return math::reduce_prod(a, keep);
      case Reduction::MAX: return math::reduce_max(a, keep);
      default: return math::reduce_min(a, keep);
    }
  }

 public:
  Reduce() : TypedOperation<T>(message()) {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 1 || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, this->DTYPE) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    std::vector<size_t> axes;
    wire::Reader r(node.operation);
    uint32_t f, t;
    while (r.next(f, t)) {
      if (f == 1) r.repeatedVarint(t, axes);
      else r.skip(t);
    }
    std::sort(axes.begin(), axes.end());
    auto& sm = graph.getSymbolManager();
    const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
    Variable<T>* out = sm.getVariable(node.outputs[0], T());
    graph.addStep([a, out, axes] {
      const size_t rank = a->shape().size();
      std::vector<unsigned> target = a->shape().toVector();
      std::vector<bool> reduced(rank, false);
      for (size_t axis : axes) {
        if (axis >= rank) throw InvalidArgumentError("invalid axis");
        target[axis] = 1;
        reduced[axis] = true;
      }
      std::vector<size_t> perm;
      for (size_t i = 0; i < rank; ++i)
        if (!reduced[i]) perm.push_back(i);
      for (size_t axis : axes) perm.push_back(axis);
      bool inPlace = true;
      for (size_t i = 0; i < perm.size(); ++i) inPlace = inPlace && perm[i] == i;
      if (inPlace) {
        *out = trailing(*a, rank - axes.size());
      } else {
        Variable<T> moved = base::transpose(*a, perm);
        *out = trailing(moved, rank - axes.size());
        out->reshape(Shape(target));
      }
    });
    return true;
  }
};

// ---- math.Clip (tensor, minimum value, maximum value), math.LeakyRelu (alpha in the node) --------------------
// tfcc_runtime/operations/math/clip.cpp:52-87, leakyrelu.cpp:52-86
template <class T>
class Clip : public TypedOperation<T> {
 public:
  Clip() : TypedOperation<T>("math.Clip") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 3 || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, this->DTYPE) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    if (!is_value(stype_of(graph, node.inputs[1])) || !is_value(stype_of(graph, node.inputs[2]))) return false;
    auto& sm = graph.getSymbolManager();
    const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
    const T* lo = sm.getValue(node.inputs[1], T());
    const T* hi = sm.getValue(node.inputs[2], T());
    Variable<T>* out = sm.getVariable(node.outputs[0], T());
    graph.addStep([a, lo, hi, out] { *out = math::clip(*a, *lo, *hi); });
    return true;
  }
};

template <class T>
class LeakyRelu : public TypedOperation<T> {
 public:
  LeakyRelu() : TypedOperation<T>("math.LeakyRelu") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 1 || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, this->DTYPE) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    proto::Value v;
    wire::Reader r(node.operation);
    uint32_t f, t;
    while (r.next(f, t)) {
      if (f == 1 && t == 2) v = proto::parse_value(r.sub());
      else r.skip(t);
    }
    T alpha = static_cast<T>(0);
    if (!v.get(alpha)) return false;
    auto& sm = graph.getSymbolManager();
    const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
    Variable<T>* out = sm.getVariable(node.outputs[0], T());
    graph.addStep([a, alpha, out] { *out = math::leaky_relu(*a, alpha); });
    return true;
  }
};

// ---- relation.Equal / UnEqual / Greater / GreaterOrEqual / Less / LessOrEqual / Not --------------------------
// Inputs of one element type, a BOOL result; tensor and value operands in the four combinations
// (tfcc_runtime/operations/relation/equal.cpp:83-133 and its siblings).  Not: BOOL -> BOOL, a tensor or a value
// (relation/not_.cpp:53-88).
template <Relation R, class T>
class Compare : public TypedOperation<T> {
  static const char* message() {
    switch (R) {
      case Relation::EQUAL: return "relation.Equal";
      case Relation::UNEQUAL: return "relation.UnEqual";
      case Relation::GREATER: return "relation.Greater";
      case Relation::GREATER_EQUAL: return "relation.GreaterOrEqual";
      case Relation::LESS: return "relation.Less";
      default: return "relation.LessOrEqual";
    }
  }
  static uint8_t vv(T a, T b) {
    switch (R) {
      case Relation::EQUAL: return a == b;
      case Relation::UNEQUAL: return a != b;
      case Relation::GREATER: return a > b;
      case Relation::GREATER_EQUAL: return a >= b;
      case Relation::LESS: return a < b;
      default: return a <= b;
    }
  }

 public:
  Compare() : TypedOperation<T>(message()) {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 2 || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, BOOL) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    auto& sm = graph.getSymbolManager();
    const SymbolType s0 = stype_of(graph, node.inputs[0]), s1 = stype_of(graph, node.inputs[1]);
    if (is_tensor(s0) && is_tensor(s1)) {
      const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
      const Tensor<T>* b = sm.getTensor(node.inputs[1], T());
      Variable<uint8_t>* out = sm.getVariable(node.outputs[0], uint8_t());
      graph.addStep([a, b, out] { *out = relation::compare(*a, *b, R); });
    } else if (is_tensor(s0) && is_value(s1)) {
      const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
      const T* b = sm.getValue(node.inputs[1], T());
      Variable<uint8_t>* out = sm.getVariable(node.outputs[0], uint8_t());
      graph.addStep([a, b, out] { *out = relation::compare(*a, *b, R); });
    } else if (is_value(s0) && is_tensor(s1)) {
      const T* a = sm.getValue(node.inputs[0], T());
      const Tensor<T>* b = sm.getTensor(node.inputs[1], T());
      Variable<uint8_t>* out = sm.getVariable(node.outputs[0], uint8_t());
      graph.addStep([a, b, out] { *out = relation::compare(*a, *b, R); });
    } else if (is_value(s0) && is_value(s1)) {
      const T* a = sm.getValue(node.inputs[0], T());
      const T* b = sm.getValue(node.inputs[1], T());
      uint8_t* out = sm.getValue(node.outputs[0], uint8_t());
      graph.addStep([a, b, out] { *out = vv(*a, *b); });
    } else {
      return false;
    }
    return true;
  }
};

class Not : public Operation {
 public:
  std::string getOperationTypeUrl() const override { return type_url("relation.Not"); }
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 1 || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, BOOL) || !same_dtype(graph, node.inputs, BOOL)) return false;
    auto& sm = graph.getSymbolManager();
    const SymbolType si = stype_of(graph, node.inputs[0]);
    if (is_tensor(si)) {
      const Tensor<uint8_t>* a = sm.getTensor(node.inputs[0], uint8_t());
      Variable<uint8_t>* out = sm.getVariable(node.outputs[0], uint8_t());
      graph.addStep([a, out] { *out = relation::equal(*a, static_cast<uint8_t>(0)); });
      return true;
    }
    if (is_value(si)) {
      const uint8_t* a = sm.getValue(node.inputs[0], uint8_t());
      uint8_t* out = sm.getValue(node.outputs[0], uint8_t());
      graph.addStep([a, out] { *out = *a == 0; });
      return true;
    }
    return false;
  }
};

// ---- math.ArgMax: int64 positions along `axis`, which stays with length 1 (math/argmax.cpp:27-38) ----------
template <class T>
class ArgMax : public TypedOperation<T> {
 public:
  ArgMax() : TypedOperation<T>("math.ArgMax") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 1 || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, DataTypeOf<int64_t>::value) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    size_t axis = 0;
    wire::Reader r(node.operation);
    uint32_t f, t;
    while (r.next(f, t)) {
      if (f == 1 && t == 0) axis = static_cast<size_t>(r.varint());
      else r.skip(t);
    }
    auto& sm = graph.getSymbolManager();
    const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
    Variable<int64_t>* out = sm.getVariable(node.outputs[0], int64_t());
    graph.addStep([a, out, axis] { *out = math::argmax(*a, axis); });
    return true;
  }
};

// ---- base.Expand (tensor, shape vector) and base.Tile (tensor, repeats vector) ------------------------------
// Broadcasting does the work: Expand adds zeros of the wanted shape to the input (base/expand.cpp:28-47); Tile views
// the input as [1, s0, 1, s1, ...], multiplies it by ones of [r0, s0, r1, s1, ...] and views the product as
// [r0 * s0, r1 * s1, ...] (base/tile.cpp:28-62).
template <class T, class IDX>
class Expand : public TypedOperation<T> {
 public:
  Expand() : TypedOperation<T>("base.Expand") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if constexpr (!std::is_integral<IDX>::value || sizeof(IDX) < 4) {
      return false;
    } else {
      if (node.inputs.size() != 2 || node.outputs.size() != 1) return false;
      auto& sm = graph.getSymbolManager();
      if (sm.getSymbolInfo(node.outputs[0]).dtype != this->DTYPE || sm.getSymbolInfo(node.inputs[0]).dtype != this->DTYPE)
        return false;
      if (sm.getSymbolInfo(node.inputs[1]).dtype != DataTypeOf<IDX>::value) return false;
      const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
      const std::vector<IDX>* shape = sm.getVector(node.inputs[1], IDX());
      Variable<T>* out = sm.getVariable(node.outputs[0], T());
      graph.addStep([a, shape, out] {
        std::vector<unsigned> real(shape->size());
        for (size_t i = 0; i < shape->size(); ++i) {
          if ((*shape)[i] <= 0) throw RuntimeError("Expand: invalid shape");
          real[i] = static_cast<unsigned>((*shape)[i]);
        }
        Variable<T> zeros{Shape(real)};
        data::zeros(zeros);
        *out = *a + zeros;
      });
      return true;
    }
  }
};

template <class T, class IDX>
class Tile : public TypedOperation<T> {
 public:
  Tile() : TypedOperation<T>("base.Tile") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if constexpr (!std::is_integral<IDX>::value || sizeof(IDX) < 4) {
      return false;
    } else {
      if (node.inputs.size() != 2 || node.outputs.size() != 1) return false;
      auto& sm = graph.getSymbolManager();
      if (sm.getSymbolInfo(node.outputs[0]).dtype != this->DTYPE || sm.getSymbolInfo(node.inputs[0]).dtype != this->DTYPE)
        return false;
      if (sm.getSymbolInfo(node.inputs[1]).dtype != DataTypeOf<IDX>::value) return false;
      const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
      const std::vector<IDX>* repeats = sm.getVector(node.inputs[1], IDX());
      Variable<T>* out = sm.getVariable(node.outputs[0], T());
      graph.addStep([a, repeats, out] {
        if (repeats->size() != a->shape().size()) throw RuntimeError("Tile: repeated error");
        std::vector<unsigned> target = a->shape().toVector(), viewed, onesShape;
        for (size_t i = 0; i < repeats->size(); ++i) {
          if ((*repeats)[i] <= 0) throw RuntimeError("Tile: repeated error");
          const unsigned r = static_cast<unsigned>((*repeats)[i]);
          viewed.push_back(1);
          viewed.push_back(target[i]);
          onesShape.push_back(r);
          onesShape.push_back(target[i]);
          target[i] *= r;
        }
        View<T> spread(*a, Shape(viewed));
        Variable<T> ones{Shape(onesShape)};
        data::ones(ones);
        *out = spread * ones;
        out->reshape(Shape(target));
      });
      return true;
    }
  }
};

// ---- nn.Where (condition, x, y), base.Tril / Triu (k in the node), base.CreateTensor, base.Range -----------
// Where: a BOOL tensor and two operands of the node's type of which one may be a value (nn/where.cpp:100-125).
// CreateTensor: zeros of the shape vector plus the value of the node (base/createtensor.cpp:28-45); the sum is formed
// on the host and written with one fill.  Range: start, limit, delta values -> a vector (base/range.cpp:28-36).
template <class T>
class Where : public TypedOperation<T> {
 public:
  Where() : TypedOperation<T>("nn.Where") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 3 || node.outputs.size() != 1) return false;
    auto& sm = graph.getSymbolManager();
    if (sm.getSymbolInfo(node.inputs[0]).dtype != BOOL || !is_tensor(stype_of(graph, node.inputs[0]))) return false;
    if (sm.getSymbolInfo(node.inputs[1]).dtype != this->DTYPE || sm.getSymbolInfo(node.inputs[2]).dtype != this->DTYPE ||
        sm.getSymbolInfo(node.outputs[0]).dtype != this->DTYPE)
      return false;
    const SymbolType sx = stype_of(graph, node.inputs[1]), sy = stype_of(graph, node.inputs[2]);
    const Tensor<uint8_t>* c = sm.getTensor(node.inputs[0], uint8_t());
    if (is_tensor(sx) && is_tensor(sy)) {
      const Tensor<T>* x = sm.getTensor(node.inputs[1], T());
      const Tensor<T>* y = sm.getTensor(node.inputs[2], T());
      Variable<T>* out = sm.getVariable(node.outputs[0], T());
      graph.addStep([c, x, y, out] { *out = nn::where(*c, *x, *y); });
    } else if (is_value(sx) && is_tensor(sy)) {
      const T* x = sm.getValue(node.inputs[1], T());
      const Tensor<T>* y = sm.getTensor(node.inputs[2], T());
      Variable<T>* out = sm.getVariable(node.outputs[0], T());
      graph.addStep([c, x, y, out] { *out = nn::where(*c, *x, *y); });
    } else if (is_tensor(sx) && is_value(sy)) {
      const Tensor<T>* x = sm.getTensor(node.inputs[1], T());
      const T* y = sm.getValue(node.inputs[2], T());
      Variable<T>* out = sm.getVariable(node.outputs[0], T());
      graph.addStep([c, x, y, out] { *out = nn::where(*c, *x, *y); });
    } else {
      return false;
    }
    return true;
  }
};

template <class T, bool UPPER>
class Triangle : public TypedOperation<T> {
 public:
  Triangle() : TypedOperation<T>(UPPER ? "base.Triu" : "base.Tril") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 1 || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, this->DTYPE) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    int64_t k = 0;
    wire::Reader r(node.operation);
    uint32_t f, t;
    while (r.next(f, t)) {
      if (f == 1 && t == 0) k = static_cast<int64_t>(r.varint());
      else r.skip(t);
    }
    auto& sm = graph.getSymbolManager();
    const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
    Variable<T>* out = sm.getVariable(node.outputs[0], T());
    graph.addStep([a, out, k] { *out = UPPER ? base::triu(*a, k) : base::tril(*a, k); });
    return true;
  }
};

template <class T, class IDX>
class CreateTensor : public TypedOperation<T> {
 public:
  CreateTensor() : TypedOperation<T>("base.CreateTensor") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if constexpr (!std::is_integral<IDX>::value || sizeof(IDX) < 4) {
      return false;
    } else {
      if (node.inputs.size() != 1 || node.outputs.size() != 1) return false;
      auto& sm = graph.getSymbolManager();
      if (sm.getSymbolInfo(node.outputs[0]).dtype != this->DTYPE) return false;
      if (sm.getSymbolInfo(node.inputs[0]).dtype != DataTypeOf<IDX>::value) return false;
      proto::Value v;
      uint64_t wanted = 0;
      wire::Reader r(node.operation);
      uint32_t f, t;
      while (r.next(f, t)) {
        if (f == 1 && t == 2) v = proto::parse_value(r.sub());
        else if (f == 2 && t == 0) wanted = r.varint();
        else r.skip(t);
      }
      if (wanted != static_cast<uint64_t>(this->DTYPE)) return false;
      T value = static_cast<T>(0);
      if (!v.get(value)) return false;
      value = static_cast<T>(static_cast<T>(0) + value);
      const std::vector<IDX>* shape = sm.getVector(node.inputs[0], IDX());
      Variable<T>* out = sm.getVariable(node.outputs[0], T());
      graph.addStep([shape, value, out] {
        std::vector<unsigned> real;
        for (IDX d : *shape) real.push_back(static_cast<unsigned>(d));
        *out = Variable<T>{Shape(real)};
        if (out->size() > 0) data::fill(*out, value);
      });
      return true;
    }
  }
};

template <class T>
class Range : public TypedOperation<T> {
 public:
  Range() : TypedOperation<T>("base.Range") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 3 || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, this->DTYPE) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    auto& sm = graph.getSymbolManager();
    for (const std::string& name : node.inputs)
      if (!is_value(stype_of(graph, name))) return false;
    const T* start = sm.getValue(node.inputs[0], T());
    const T* limit = sm.getValue(node.inputs[1], T());
    const T* delta = sm.getValue(node.inputs[2], T());
    std::vector<T>* out = sm.getVector(node.outputs[0], T());
    graph.addStep([start, limit, delta, out] {
      out->clear();
      // the reference's loop does not end for a step that does not move towards the limit
      if (*start < *limit && !(*delta > static_cast<T>(0))) throw RuntimeError("Range: delta must be positive");
      for (T x = *start; x < *limit; x += *delta) out->push_back(x);
    });
    return true;
  }
};

// ---- math.TopK (tensor, k value) -> values, int64 positions; k is clipped to the last dimension ---------------
// tfcc_runtime/operations/math/topk.cpp:28-135 sorts on the host after a read-back; here the rows are searched on the
// device and the positions converted to int64 there.  Equal values come in ascending position.
template <class T, class LEN>
class TopK : public TypedOperation<T> {
 public:
  TopK() : TypedOperation<T>("math.TopK") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 2 || node.outputs.size() != 2) return false;
    auto& sm = graph.getSymbolManager();
    if (sm.getSymbolInfo(node.outputs[0]).dtype != this->DTYPE || sm.getSymbolInfo(node.inputs[0]).dtype != this->DTYPE)
      return false;
    if (sm.getSymbolInfo(node.inputs[1]).dtype != DataTypeOf<LEN>::value || !is_value(stype_of(graph, node.inputs[1])))
      return false;
    if (sm.getSymbolInfo(node.outputs[1]).dtype != DataTypeOf<int64_t>::value) return false;
    const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
    const LEN* k = sm.getValue(node.inputs[1], LEN());
    Variable<T>* values = sm.getVariable(node.outputs[0], T());
    Variable<int64_t>* positions = sm.getVariable(node.outputs[1], int64_t());
    graph.addStep([a, k, values, positions] {
      if (a->size() == 0) throw InvalidArgumentError("invalid tensor");
      if (*k <= 0) throw InvalidArgumentError("invalid k");
      const unsigned length = a->shape(a->shape().size() - 1);
      const unsigned count = static_cast<unsigned>(std::min<uint64_t>(static_cast<uint64_t>(*k), length));
      Variable<uint32_t> found;
      std::tie(*values, found) = math::top_k(*a, count);
      *positions = data::cast<int64_t>(found);
    });
    return true;
  }
};

// ---- nn.LayerNormalization --------------------------------------------------------------------------------
template <class T>
class LayerNormalization : public TypedOperation<T> {
 public:
  LayerNormalization() : TypedOperation<T>("nn.LayerNormalization") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 3 || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, this->DTYPE) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    proto::Value eps;
    wire::Reader r(node.operation);
    uint32_t f, t;
    while (r.next(f, t)) {
      if (f == 1 && t == 2) eps = proto::parse_value(r.sub());
      else r.skip(t);
    }
    T epsilon = static_cast<T>(0);
    if (!eps.get(epsilon)) return false;
    auto& sm = graph.getSymbolManager();
    const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
    const Tensor<T>* gamma = sm.getTensor(node.inputs[1], T());
    const Tensor<T>* beta = sm.getTensor(node.inputs[2], T());
    Variable<T>* out = sm.getVariable(node.outputs[0], T());
    graph.addStep([a, gamma, beta, epsilon, out] {
      *out = nn::layer_normalization(*a, *gamma, *beta, epsilon, a->shape().size() - 1);
    });
    return true;
  }
};

// ---- base.Transpose ------------------------------------------------------------------------------------------
template <class T>
class Transpose : public TypedOperation<T> {
 public:
  Transpose() : TypedOperation<T>("base.Transpose") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 1 || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, this->DTYPE) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    std::vector<size_t> perm;
    wire::Reader r(node.operation);
    uint32_t f, t;
    while (r.next(f, t)) {
      if (f == 1) r.repeatedVarint(t, perm);
      else r.skip(t);
    }
    auto& sm = graph.getSymbolManager();
    const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
    Variable<T>* out = sm.getVariable(node.outputs[0], T());
    graph.addStep([a, out, perm] { *out = base::transpose(*a, perm); });
    return true;
  }
};

// ---- base.Reshape: output is a View of the input; 0 keeps a dimension, one negative entry is inferred ----------
template <class T, class SHAPE>
class Reshape : public TypedOperation<T> {
 public:
  Reshape() : TypedOperation<T>("base.Reshape") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 2 || node.outputs.size() != 1) return false;
    auto& sm = graph.getSymbolManager();
    if (sm.getSymbolInfo(node.outputs[0]).dtype != this->DTYPE || sm.getSymbolInfo(node.inputs[0]).dtype != this->DTYPE)
      return false;
    if (sm.getSymbolInfo(node.inputs[1]).dtype != DataTypeOf<SHAPE>::value) return false;
    const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
    const std::vector<SHAPE>* shape = sm.getVector(node.inputs[1], SHAPE());
    View<T>* out = sm.getView(node.outputs[0], T());
    graph.addStep([a, shape, out] {
      int inferred = -1;
      unsigned area = 1;
      std::vector<unsigned> real(shape->size());
      for (size_t i = 0; i < shape->size(); ++i) {
        const SHAPE d = (*shape)[i];
        if (d == 0) {
          if (i >= a->shape().size()) throw RuntimeError("Reshape: invalid shape");
          real[i] = a->shape(i);
          area *= real[i];
        } else if (d < 0) {
          if (inferred >= 0) throw RuntimeError("Reshape: invalid shape");
          inferred = static_cast<int>(i);
        } else {
          real[i] = static_cast<unsigned>(d);
          area *= real[i];
        }
      }
      if (inferred >= 0) {
        if (area == 0) throw RuntimeError("Reshape: invalid shape");
        real[inferred] = a->size() / area;
      }
      *out = View<T>(*a, Shape(std::move(real)));
    });
    return true;
  }
};

// ---- base.Squeeze / base.Unsqueeze / base.Flatten: the output is a View of the input under another shape ---------
// tfcc_runtime/operations/base/squeeze.cpp:27-52,78-113, unsqueeze.cpp:27-52,78-113, flatten.cpp:27-90
enum class Reshaping { SQUEEZE, UNSQUEEZE, FLATTEN };

template <Reshaping KIND, class T>
class ShapeView : public TypedOperation<T> {
  static const char* message() {
    return KIND == Reshaping::SQUEEZE ? "base.Squeeze" : KIND == Reshaping::UNSQUEEZE ? "base.Unsqueeze" : "base.Flatten";
  }

 public:
  ShapeView() : TypedOperation<T>(message()) {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 1 || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, this->DTYPE) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    std::vector<size_t> axes;  // Flatten: its one axis
    wire::Reader r(node.operation);
    uint32_t f, t;
    while (r.next(f, t)) {
      if (f == 1 && KIND == Reshaping::FLATTEN && t == 0) axes.assign(1, static_cast<size_t>(r.varint()));
      else if (f == 1 && KIND != Reshaping::FLATTEN) r.repeatedVarint(t, axes);
      else r.skip(t);
    }
    if (KIND == Reshaping::FLATTEN && axes.empty()) axes.assign(1, 0);  // proto3: a zero field is not written
    std::sort(axes.begin(), axes.end());
    auto& sm = graph.getSymbolManager();
    const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
    View<T>* out = sm.getView(node.outputs[0], T());
    graph.addStep([a, out, axes] {
      std::vector<unsigned> shape;
      const size_t rank = a->shape().size();
      if (KIND == Reshaping::FLATTEN) {
        if (axes[0] >= rank) throw RuntimeError("Flatten: axis error");
        unsigned s1 = 1, s2 = 1;
        for (size_t i = 0; i < rank; ++i) (i < axes[0] ? s1 : s2) *= a->shape(i);
        shape = {s1, s2};
      } else if (axes.empty()) {
        shape = a->shape().toVector();
      } else if (KIND == Reshaping::SQUEEZE) {
        size_t pos = 0;
        for (size_t i = 0; i < rank; ++i) {
          if (pos < axes.size() && i == axes[pos]) {
            if (a->shape(i) != 1) throw RuntimeError("Squeeze: invalid axes");
            ++pos;
          } else {
            shape.push_back(a->shape(i));
          }
        }
        if (pos != axes.size()) throw RuntimeError("Squeeze: invalid axes");
      } else {
        shape.resize(rank + axes.size());
        size_t pos0 = 0, pos1 = 0;
        for (size_t i = 0; i < shape.size(); ++i) {
          if (pos1 < axes.size() && i == axes[pos1]) {
            shape[i] = 1;
            ++pos1;
          } else {
            if (pos0 >= rank) throw RuntimeError("Unsqueeze: invalid axes");
            shape[i] = a->shape(pos0++);
          }
        }
      }
      *out = View<T>(*a, Shape(std::move(shape)));
    });
    return true;
  }
};

// ---- base.GetShape (a uint32 vector) / base.GetDimension (a value of any type) -----------------------------------
// tfcc_runtime/operations/base/getshape.cpp:27-78, getdimension.cpp:27-76
template <class T>
class GetShape : public TypedOperation<T> {
 public:
  GetShape() : TypedOperation<T>("base.GetShape") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 1 || node.outputs.size() != 1) return false;
    auto& sm = graph.getSymbolManager();
    if (sm.getSymbolInfo(node.outputs[0]).dtype != DataTypeOf<uint32_t>::value ||
        sm.getSymbolInfo(node.inputs[0]).dtype != this->DTYPE)
      return false;
    const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
    std::vector<uint32_t>* out = sm.getVector(node.outputs[0], uint32_t());
    graph.addStep([a, out] { *out = a->shape().toVector(); });
    return true;
  }
};

template <class SRC, class DST>
class GetDimension : public TypedOperation<SRC> {
 public:
  GetDimension() : TypedOperation<SRC>("base.GetDimension") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 1 || node.outputs.size() != 1) return false;
    auto& sm = graph.getSymbolManager();
    if (sm.getSymbolInfo(node.outputs[0]).dtype != DataTypeOf<DST>::value || sm.getSymbolInfo(node.inputs[0]).dtype != this->DTYPE)
      return false;
    size_t axis = 0;
    wire::Reader r(node.operation);
    uint32_t f, t;
    while (r.next(f, t)) {
      if (f == 1 && t == 0) axis = static_cast<size_t>(r.varint());
      else r.skip(t);
    }
    const Tensor<SRC>* a = sm.getTensor(node.inputs[0], SRC());
    DST* out = sm.getValue(node.outputs[0], DST());
    graph.addStep([a, out, axis] {
      if (axis >= a->shape().size()) throw RuntimeError("GetDimension: axis error");
      *out = static_cast<DST>(a->shape(axis));
    });
    return true;
  }
};

// ---- nn.Gather, base.Cast, base.SliceV1, base.Concat: data movement between the products -------------------------
// tfcc_runtime/operations/nn/gather.cpp:27-92 (axis 0 only), base/cast.cpp:30-129 (tensor and value forms),
// base/slicev1.cpp:27-92 (start from a value symbol, length from the message), base/concat.cpp:27-90
template <class T, class IDX>
class Gather : public TypedOperation<T> {
 public:
  Gather() : TypedOperation<T>("nn.Gather") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 2 || node.outputs.size() != 1) return false;
    auto& sm = graph.getSymbolManager();
    if (sm.getSymbolInfo(node.outputs[0]).dtype != this->DTYPE || sm.getSymbolInfo(node.inputs[0]).dtype != this->DTYPE)
      return false;
    if (sm.getSymbolInfo(node.inputs[1]).dtype != DataTypeOf<IDX>::value) return false;
    uint64_t axis = 0;
    wire::Reader r(node.operation);
    uint32_t f, t;
    while (r.next(f, t)) {
      if (f == 1 && t == 0) axis = r.varint();
      else r.skip(t);
    }
    const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
    const Tensor<IDX>* indices = sm.getTensor(node.inputs[1], IDX());
    Variable<T>* out = sm.getVariable(node.outputs[0], T());
    graph.addStep([a, indices, axis, out] {
      if (axis != 0) throw RuntimeError("Gather: invalid axis");
      *out = nn::gather(*a, *indices);
    });
    return true;
  }
};

template <class SRC, class DST>
class Cast : public TypedOperation<SRC> {
 public:
  Cast() : TypedOperation<SRC>("base.Cast") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 1 || node.outputs.size() != 1) return false;
    auto& sm = graph.getSymbolManager();
    const SymbolInfo& in = sm.getSymbolInfo(node.inputs[0]);
    const SymbolInfo& outInfo = sm.getSymbolInfo(node.outputs[0]);
    // BOOL symbols live in bytes: a BOOL source converts like uint8, a BOOL result is 1 where the source is not 0
    // (tfcc_runtime/operations/base/cast.cpp:58-79)
    const bool fromBool = std::is_same<SRC, uint8_t>::value && in.dtype == BOOL;
    const bool toBool = std::is_same<DST, uint8_t>::value && outInfo.dtype == BOOL;
    if (in.dtype != this->DTYPE && !fromBool) return false;
    if (outInfo.dtype != DataTypeOf<DST>::value && !toBool) return false;
    uint64_t wanted = 0;
    wire::Reader r(node.operation);
    uint32_t f, t;
    while (r.next(f, t)) {
      if (f == 1 && t == 0) wanted = r.varint();
      else r.skip(t);
    }
    if (wanted != static_cast<uint64_t>(outInfo.dtype)) return false;
    if (toBool) {
      if (is_tensor(in.stype) && is_tensor(outInfo.stype)) {
        const Tensor<SRC>* a = sm.getTensor(node.inputs[0], SRC());
        Variable<uint8_t>* out = sm.getVariable(node.outputs[0], uint8_t());
        graph.addStep([a, out] { *out = relation::unequal(*a, static_cast<SRC>(0)); });
      } else if (is_value(in.stype) && is_value(outInfo.stype)) {
        const SRC* a = sm.getValue(node.inputs[0], SRC());
        uint8_t* out = sm.getValue(node.outputs[0], uint8_t());
        graph.addStep([a, out] { *out = *a ? 1 : 0; });
      } else {
        return false;
      }
      return true;
    }
    if (is_tensor(in.stype) && is_tensor(outInfo.stype)) {
      const Tensor<SRC>* a = sm.getTensor(node.inputs[0], SRC());
      Variable<DST>* out = sm.getVariable(node.outputs[0], DST());
      graph.addStep([a, out] { *out = data::cast<DST>(*a); });
    } else if (is_value(in.stype) && is_value(outInfo.stype)) {
      const SRC* a = sm.getValue(node.inputs[0], SRC());
      DST* out = sm.getValue(node.outputs[0], DST());
      graph.addStep([a, out] { *out = static_cast<DST>(*a); });
    } else {
      return false;
    }
    return true;
  }
};

template <class T, class POS>
class SliceV1 : public TypedOperation<T> {
 public:
  SliceV1() : TypedOperation<T>("base.SliceV1") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (!std::is_integral<POS>::value) return false;  // the position is a value of one of the eight integer types
    if (node.inputs.size() != 2 || node.outputs.size() != 1) return false;
    auto& sm = graph.getSymbolManager();
    if (sm.getSymbolInfo(node.outputs[0]).dtype != this->DTYPE || sm.getSymbolInfo(node.inputs[0]).dtype != this->DTYPE)
      return false;
    if (sm.getSymbolInfo(node.inputs[1]).dtype != DataTypeOf<POS>::value) return false;
    uint64_t axis = 0, length = 0;
    wire::Reader r(node.operation);
    uint32_t f, t;
    while (r.next(f, t)) {
      if (f == 1 && t == 0) axis = r.varint();
      else if (f == 2 && t == 0) length = r.varint();
      else r.skip(t);
    }
    const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
    const POS* pos = sm.getValue(node.inputs[1], POS());
    Variable<T>* out = sm.getVariable(node.outputs[0], T());
    graph.addStep([a, pos, axis, length, out] {
      if (*pos < POS(0)) throw RuntimeError("SliceV1: invalid pos");
      const unsigned start = static_cast<unsigned>(*pos);
      *out = base::slice(*a, static_cast<size_t>(axis), start, start + static_cast<unsigned>(length));
    });
    return true;
  }
};

template <class T>
class Concat : public TypedOperation<T> {
 public:
  Concat() : TypedOperation<T>("base.Concat") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.empty() || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, this->DTYPE) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    uint64_t axis = 0;
    wire::Reader r(node.operation);
    uint32_t f, t;
    while (r.next(f, t)) {
      if (f == 1 && t == 0) axis = r.varint();
      else r.skip(t);
    }
    auto& sm = graph.getSymbolManager();
    std::vector<const Tensor<T>*> values;
    for (const std::string& name : node.inputs) values.push_back(sm.getTensor(name, T()));
    Variable<T>* out = sm.getVariable(node.outputs[0], T());
    graph.addStep([values, axis, out] { *out = base::concat(values, static_cast<size_t>(axis)); });
    return true;
  }
};

// ---- base.Split / Stack / SliceV2 / Pad ------------------------------------------------------------------------------
// tfcc_runtime/operations/base/split.cpp:27-87 (as many equal parts as the node has outputs), stack.cpp:27-87,
// slicev2.cpp:27-121 (start and end from value symbols, negative ones count from the end), pad.cpp:27-91
template <class T>
class Split : public TypedOperation<T> {
 public:
  Split() : TypedOperation<T>("base.Split") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 1 || node.outputs.empty()) return false;
    if (!same_dtype(graph, node.outputs, this->DTYPE) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    const uint64_t axis = first_varint(node);
    auto& sm = graph.getSymbolManager();
    const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
    std::vector<Variable<T>*> outs;
    for (const std::string& name : node.outputs) outs.push_back(sm.getVariable(name, T()));
    graph.addStep([a, axis, outs] {
      std::vector<Variable<T>> parts = base::split(*a, outs.size(), static_cast<size_t>(axis));
      for (size_t i = 0; i < outs.size(); ++i) *outs[i] = std::move(parts[i]);
    });
    return true;
  }

  static uint64_t first_varint(const proto::Node& node) {
    uint64_t v = 0;
    wire::Reader r(node.operation);
    uint32_t f, t;
    while (r.next(f, t)) {
      if (f == 1 && t == 0) v = r.varint();
      else r.skip(t);
    }
    return v;
  }
};

template <class T>
class Stack : public TypedOperation<T> {
 public:
  Stack() : TypedOperation<T>("base.Stack") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.empty() || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, this->DTYPE) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    const uint64_t axis = Split<T>::first_varint(node);
    auto& sm = graph.getSymbolManager();
    std::vector<const Tensor<T>*> values;
    for (const std::string& name : node.inputs) values.push_back(sm.getTensor(name, T()));
    Variable<T>* out = sm.getVariable(node.outputs[0], T());
    graph.addStep([values, axis, out] { *out = base::stack(values, static_cast<size_t>(axis)); });
    return true;
  }
};

template <class T, class POS>
class SliceV2 : public TypedOperation<T> {
 public:
  SliceV2() : TypedOperation<T>("base.SliceV2") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (!std::is_integral<POS>::value) return false;
    if (node.inputs.size() != 3 || node.outputs.size() != 1) return false;
    auto& sm = graph.getSymbolManager();
    if (sm.getSymbolInfo(node.outputs[0]).dtype != this->DTYPE || sm.getSymbolInfo(node.inputs[0]).dtype != this->DTYPE)
      return false;
    if (sm.getSymbolInfo(node.inputs[1]).dtype != DataTypeOf<POS>::value ||
        sm.getSymbolInfo(node.inputs[2]).dtype != DataTypeOf<POS>::value)
      return false;
    const uint64_t axis = Split<T>::first_varint(node);
    const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
    const POS* start = sm.getValue(node.inputs[1], POS());
    const POS* end = sm.getValue(node.inputs[2], POS());
    Variable<T>* out = sm.getVariable(node.outputs[0], T());
    graph.addStep([a, start, end, axis, out] {
      if (axis >= a->shape().size()) throw RuntimeError("SliceV2: invalid axis");
      long long s = static_cast<long long>(*start), e = static_cast<long long>(*end);
      const long long extent = a->shape(static_cast<size_t>(axis));
      if (std::is_signed<POS>::value && extent > 0) {
        while (s < 0) s += extent;
        while (e < 0) e += extent;
      }
      if (s < 0 || e < 0) throw RuntimeError("SliceV2: invalid position");
      const unsigned limit = ~0u;
      *out = base::slice(*a, static_cast<size_t>(axis), static_cast<unsigned>(std::min<long long>(s, limit)),
                         static_cast<unsigned>(std::min<long long>(e, limit)));
    });
    return true;
  }
};

template <class T, class IDX>
class Pad : public TypedOperation<T> {
 public:
  Pad() : TypedOperation<T>("base.Pad") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (!std::is_integral<IDX>::value) return false;
    if (node.inputs.size() != 3 || node.outputs.size() != 1) return false;
    auto& sm = graph.getSymbolManager();
    if (sm.getSymbolInfo(node.outputs[0]).dtype != this->DTYPE || sm.getSymbolInfo(node.inputs[0]).dtype != this->DTYPE)
      return false;
    if (sm.getSymbolInfo(node.inputs[1]).dtype != DataTypeOf<IDX>::value ||
        sm.getSymbolInfo(node.inputs[2]).dtype != DataTypeOf<IDX>::value)
      return false;
    const uint64_t axis = Split<T>::first_varint(node);
    const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
    const IDX* head = sm.getValue(node.inputs[1], IDX());
    const IDX* tail = sm.getValue(node.inputs[2], IDX());
    Variable<T>* out = sm.getVariable(node.outputs[0], T());
    graph.addStep([a, head, tail, axis, out] {
      *out = base::pad(*a, static_cast<size_t>(axis), static_cast<unsigned>(*head), static_cast<unsigned>(*tail));
    });
    return true;
  }
};

// ---- base.At / At1 / ToTensor / ToValue / ToVector: between the three kinds of symbols ---------------------------
// tfcc_runtime/operations/base/at.cpp:27-82, at1.cpp:27-75, totensor.cpp:27-116, tovalue.cpp:27-109,
// tovector.cpp:27-110.  Reading a tensor into a value or a vector waits for the device.
template <class T, class IDX>
class At : public TypedOperation<T> {
 public:
  At() : TypedOperation<T>("base.At") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (!std::is_integral<IDX>::value) return false;
    if (node.inputs.size() != 2 || node.outputs.size() != 1) return false;
    auto& sm = graph.getSymbolManager();
    if (sm.getSymbolInfo(node.outputs[0]).dtype != this->DTYPE || sm.getSymbolInfo(node.inputs[0]).dtype != this->DTYPE ||
        sm.getSymbolInfo(node.inputs[1]).dtype != DataTypeOf<IDX>::value)
      return false;
    const std::vector<T>* a = sm.getVector(node.inputs[0], T());
    const IDX* pos = sm.getValue(node.inputs[1], IDX());
    T* out = sm.getValue(node.outputs[0], T());
    graph.addStep([a, pos, out] {
      if (*pos < IDX(0) || static_cast<size_t>(*pos) >= a->size()) throw RuntimeError("At: invalid pos");
      *out = (*a)[static_cast<size_t>(*pos)];
    });
    return true;
  }
};

template <class T>
class At1 : public TypedOperation<T> {
 public:
  At1() : TypedOperation<T>("base.At1") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 1 || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, this->DTYPE) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    size_t idx = 0;
    wire::Reader r(node.operation);
    uint32_t f, t;
    while (r.next(f, t)) {
      if (f == 1 && t == 0) idx = static_cast<size_t>(r.varint());
      else r.skip(t);
    }
    auto& sm = graph.getSymbolManager();
    const std::vector<T>* a = sm.getVector(node.inputs[0], T());
    T* out = sm.getValue(node.outputs[0], T());
    graph.addStep([a, idx, out] {
      if (idx >= a->size()) throw RuntimeError("At1: invalid pos");
      *out = (*a)[idx];
    });
    return true;
  }
};

enum class Target { TENSOR, VALUE, VECTOR };

template <Target TO, class T>
class Convert : public TypedOperation<T> {
  static const char* message() {
    return TO == Target::TENSOR ? "base.ToTensor" : TO == Target::VALUE ? "base.ToValue" : "base.ToVector";
  }

 public:
  Convert() : TypedOperation<T>(message()) {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 1 || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, this->DTYPE) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    auto& sm = graph.getSymbolManager();
    const SymbolType from = stype_of(graph, node.inputs[0]);
    // the three sources, read into a host vector when the step runs
    std::function<std::vector<T>()> read;
    if (is_tensor(from)) {
      const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
      if (TO == Target::TENSOR) {
        Variable<T>* out = sm.getVariable(node.outputs[0], T());
        graph.addStep([a, out] { *out = data::copy(*a); });
        return true;
      }
      read = [a] { return data::get(*a); };
    } else if (is_vector(from)) {
      const std::vector<T>* a = sm.getVector(node.inputs[0], T());
      read = [a] { return *a; };
    } else if (is_value(from)) {
      const T* a = sm.getValue(node.inputs[0], T());
      read = [a] { return std::vector<T>(1, *a); };
    } else {
      return false;
    }
    if (TO == Target::TENSOR) {
      Variable<T>* out = sm.getVariable(node.outputs[0], T());
      graph.addStep([read, out] {
        std::vector<T> v = read();
        const unsigned n = static_cast<unsigned>(v.size());
        *out = data::set(std::move(v), Shape({n}));
      });
    } else if (TO == Target::VALUE) {
      T* out = sm.getValue(node.outputs[0], T());
      const bool single = is_value(from);
      graph.addStep([read, out, a = is_tensor(from) ? sm.getTensor(node.inputs[0], T()) : nullptr, single] {
        if (a != nullptr && a->size() != 1) throw RuntimeError("ToValue: invalid size of input");
        std::vector<T> v = read();
        if (!single && v.size() != 1) throw RuntimeError("ToValue: invalid size of input");
        *out = v[0];
      });
    } else {
      std::vector<T>* out = sm.getVector(node.outputs[0], T());
      graph.addStep([read, out] { *out = read(); });
    }
    return true;
  }
};

// ---- base.Identity -----------------------------------------------------------------------------------------------
template <class T>
class Identity : public TypedOperation<T> {
 public:
  Identity() : TypedOperation<T>("base.Identity") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 1 || node.outputs.size() != 1) return false;
    if (!same_dtype(graph, node.outputs, this->DTYPE) || !same_dtype(graph, node.inputs, this->DTYPE)) return false;
    auto& sm = graph.getSymbolManager();
    const SymbolType si = stype_of(graph, node.inputs[0]), so = stype_of(graph, node.outputs[0]);
    if (is_tensor(si) && so == SymbolType::VARIABLE) {
      const Tensor<T>* a = sm.getTensor(node.inputs[0], T());
      Variable<T>* out = sm.getVariable(node.outputs[0], T());
      graph.addStep([a, out] { *out = data::copy(*a); });
    } else if (is_value(si) && so == SymbolType::VALUE) {
      const T* a = sm.getValue(node.inputs[0], T());
      T* out = sm.getValue(node.outputs[0], T());
      graph.addStep([a, out] { *out = *a; });
    } else if (is_vector(si) && so == SymbolType::VECTOR) {
      const std::vector<T>* a = sm.getVector(node.inputs[0], T());
      std::vector<T>* out = sm.getVector(node.outputs[0], T());
      graph.addStep([a, out] { *out = *a; });
    } else {
      return false;
    }
    return true;
  }
};

// ---- base.CreateVector: literal entries, or `pos` entries that splice in an input value / vector ---------------
template <class T>
class CreateVector : public TypedOperation<T> {
  struct Entry {
    bool fromInput = false;
    unsigned pos = 0;
    T literal = T();
  };

  template <class S>
  static bool splice(Graph& graph, const std::string& name, std::vector<T>* out) {
    auto& sm = graph.getSymbolManager();
    const SymbolInfo& info = sm.getSymbolInfo(name);
    if (info.dtype != DataTypeOf<S>::value) return false;
    if (is_value(info.stype)) {
      const S* v = sm.getValue(name, S());
      graph.addStep([v, out] { out->push_back(static_cast<T>(*v)); });
    } else if (is_vector(info.stype)) {
      const std::vector<S>* v = sm.getVector(name, S());
      graph.addStep([v, out] {
        for (S x : *v) out->push_back(static_cast<T>(x));
      });
    } else {
      return false;
    }
    return true;
  }

 public:
  CreateVector() : TypedOperation<T>("base.CreateVector") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.outputs.size() != 1) return false;
    auto& sm = graph.getSymbolManager();
    if (sm.getSymbolInfo(node.outputs[0]).dtype != this->DTYPE) return false;
    std::vector<Entry> entries;
    DataType declared = UNKNOW;
    wire::Reader r(node.operation);
    uint32_t f, t;
    while (r.next(f, t)) {
      if (f == 1 && t == 2) {
        Entry e;
        bool known = false;
        wire::Reader v = r.sub();
        uint32_t vf, vt;
        while (v.next(vf, vt)) {
          if (vf == 1 && vt == 0) { e.literal = static_cast<T>(static_cast<int64_t>(v.varint())); known = true; }
          else if (vf == 2 && vt == 0) { e.literal = static_cast<T>(v.varint()); known = true; }
          else if (vf == 3 && vt == 5) { e.literal = static_cast<T>(v.float32()); known = true; }
          else if (vf == 4 && vt == 1) { e.literal = static_cast<T>(v.float64()); known = true; }
          else if (vf == 5 && vt == 0) { e.fromInput = true; e.pos = static_cast<unsigned>(v.varint()); known = true; }
          else v.skip(vt);
        }
        if (!known) return false;
        entries.push_back(e);
      } else if (f == 2 && t == 0) {
        declared = static_cast<DataType>(r.varint());
      } else {
        r.skip(t);
      }
    }
    if (declared != this->DTYPE) return false;
    std::vector<T>* out = sm.getVector(node.outputs[0], T());
    graph.addStep([out] { out->clear(); });
    for (const Entry& e : entries) {
      if (!e.fromInput) {
        const T literal = e.literal;
        graph.addStep([out, literal] { out->push_back(literal); });
        continue;
      }
      if (e.pos >= node.inputs.size()) return false;
      const std::string& name = node.inputs[e.pos];
      bool ok = false;
#define TFCC_RUNTIME_SPLICE(S, E) ok = ok || splice<S>(graph, name, out);
      TFCC_RUNTIME_FOR_ALL_TYPES(TFCC_RUNTIME_SPLICE)
#undef TFCC_RUNTIME_SPLICE
      if (!ok) return false;
    }
    return true;
  }
};

// ---- rnn.BidirectionalLSTM ---------------------------------------------------------------------------------
// tfcc_runtime/operations/rnn/bidirectionallstm.cpp:27-128: six inputs (a [seq, batch, length]; input kernel
// [2, length, 4 hidden], state kernel [2, hidden, 4 hidden], bias [2, 4 hidden], initial h and c [2, batch, hidden],
// index 0 the forward direction) and six outputs (forward / backward outputs, h, c); hidden_size 0 is refused.
template <class T>
class BidirectionalLSTM : public TypedOperation<T> {
  static View<T> direction(const Tensor<T>& t, unsigned d) {
    View<T> v(t, t.shape(), d, d + 1);
    std::vector<unsigned> dims = t.shape().toVector();
    dims.erase(dims.begin());
    v.reshape(Shape(std::move(dims)));
    return v;
  }

 public:
  BidirectionalLSTM() : TypedOperation<T>("rnn.BidirectionalLSTM") {}
  bool process(const proto::Node& node, Graph& graph) const override {
    if (node.inputs.size() != 6 || node.outputs.size() != 6) return false;
    auto& sm = graph.getSymbolManager();
    if (sm.getSymbolInfo(node.outputs[0]).dtype != this->DTYPE) return false;
    uint64_t hiddenSize = 0;
    wire::Reader r(node.operation);
    uint32_t f, t;
    while (r.next(f, t)) {
      if (f == 1 && t == 0) hiddenSize = r.varint();
      else r.skip(t);
    }
    if (hiddenSize == 0) return false;
    const Tensor<T>* in[6];
    Variable<T>* out[6];
    for (int i = 0; i < 6; ++i) {
      in[i] = sm.getTensor(node.inputs[i], T());
      out[i] = sm.getVariable(node.outputs[i], T());
    }
    std::array<const Tensor<T>*, 6> i6{in[0], in[1], in[2], in[3], in[4], in[5]};
    std::array<Variable<T>*, 6> o6{out[0], out[1], out[2], out[3], out[4], out[5]};
    graph.addStep([i6, o6] {
      for (unsigned d = 0; d < 2; ++d) {
        for (int i = 1; i < 6; ++i)
          if (i6[i]->shape().size() < 2 || i6[i]->shape(0) != 2) throw InvalidArgumentError("invalid shape");
        View<T> ik = direction(*i6[1], d), sk = direction(*i6[2], d), bias = direction(*i6[3], d),
                ih = direction(*i6[4], d), ic = direction(*i6[5], d);
        std::tie(*o6[0 + d], *o6[2 + d], *o6[4 + d]) =
            d == 0 ? rnn::lstm_forward(*i6[0], ik, sk, bias, ih, ic) : rnn::lstm_backward(*i6[0], ik, sk, bias, ih, ic);
      }
    });
    return true;
  }
};

class Collector {
  std::map<std::string, std::vector<std::unique_ptr<Operation>>> _operations;

  void add(Operation* op) { _operations[op->getOperationTypeUrl()].emplace_back(op); }

  template <class T>
  void addForType() {
    add(new Matmul<T>());
    add(new MatmulWithBias<T>());
    add(new Arithmetic<Arith::ADD, T>());
    add(new Arithmetic<Arith::SUB, T>());
    add(new Arithmetic<Arith::MUL, T>());
    add(new Arithmetic<Arith::DIV, T>());
    add(new Arithmetic<Arith::POW, T>());
    add(new Arithmetic<Arith::MAX, T>());
    add(new Arithmetic<Arith::MIN, T>());
    add(new Reduce<Reduction::SUM, T>());
    add(new Reduce<Reduction::MEAN, T>());
    add(new Reduce<Reduction::PROD, T>());
    add(new Reduce<Reduction::MAX, T>());
    add(new Reduce<Reduction::MIN, T>());
    add(new Clip<T>());
    add(new Compare<Relation::EQUAL, T>());
    add(new Compare<Relation::UNEQUAL, T>());
    add(new Compare<Relation::GREATER, T>());
    add(new Compare<Relation::GREATER_EQUAL, T>());
    add(new Compare<Relation::LESS, T>());
    add(new Compare<Relation::LESS_EQUAL, T>());
    add(new ArgMax<T>());
    add(new Where<T>());
    add(new Triangle<T, false>());
    add(new Triangle<T, true>());
    add(new Range<T>());
    add(new LeakyRelu<T>());
    add(new Gelu<T>());
    add(new Unary<UnaryFunction::SIGMOID, T>());
    add(new Unary<UnaryFunction::TANH, T>());
    add(new Unary<UnaryFunction::RELU, T>());
    add(new Unary<UnaryFunction::SOFTPLUS, T>());
    add(new Unary<UnaryFunction::LOG, T>());
    add(new Unary<UnaryFunction::RSQRT, T>());
    add(new Unary<UnaryFunction::ERF, T>());
    add(new Unary<UnaryFunction::ABS, T>());
    add(new Unary<UnaryFunction::SIGN, T>());
    add(new Unary<UnaryFunction::NEG, T>());
    add(new Unary<UnaryFunction::RECIPROCAL, T>());
    add(new Unary<UnaryFunction::SQRT, T>());
    add(new Softmax<T>());
    add(new LayerNormalization<T>());
    add(new Transpose<T>());
    add(new Reshape<T, int32_t>());
    add(new Reshape<T, uint32_t>());
    add(new Reshape<T, int64_t>());
    add(new Reshape<T, uint64_t>());
    add(new Identity<T>());
    add(new CreateVector<T>());
    add(new BidirectionalLSTM<T>());
    add(new ShapeView<Reshaping::SQUEEZE, T>());
    add(new ShapeView<Reshaping::UNSQUEEZE, T>());
    add(new ShapeView<Reshaping::FLATTEN, T>());
    add(new GetShape<T>());
    add(new Gather<T, int32_t>());
    add(new Gather<T, uint32_t>());
    add(new Gather<T, int64_t>());
    add(new Gather<T, uint64_t>());
    add(new Concat<T>());
    add(new At1<T>());
    add(new Split<T>());
    add(new Stack<T>());
    add(new Convert<Target::TENSOR, T>());
    add(new Convert<Target::VALUE, T>());
    add(new Convert<Target::VECTOR, T>());
#define TFCC_RUNTIME_ADD_PAIR(OTHER, E) \
  add(new Cast<T, OTHER>());            \
  add(new SliceV1<T, OTHER>());         \
  add(new At<T, OTHER>());              \
  add(new SliceV2<T, OTHER>());         \
  add(new Pad<T, OTHER>());
    TFCC_RUNTIME_FOR_ALL_TYPES(TFCC_RUNTIME_ADD_PAIR)
#undef TFCC_RUNTIME_ADD_PAIR
#define TFCC_RUNTIME_ADD_SHAPED(IDX) \
  add(new Expand<T, IDX>());          \
  add(new Tile<T, IDX>());            \
  add(new CreateTensor<T, IDX>());
    TFCC_RUNTIME_ADD_SHAPED(int32_t)
    TFCC_RUNTIME_ADD_SHAPED(uint32_t)
    TFCC_RUNTIME_ADD_SHAPED(int64_t)
    TFCC_RUNTIME_ADD_SHAPED(uint64_t)
#undef TFCC_RUNTIME_ADD_SHAPED
    add(new TopK<T, int8_t>());
    add(new TopK<T, uint8_t>());
    add(new TopK<T, int16_t>());
    add(new TopK<T, uint16_t>());
    add(new TopK<T, int32_t>());
    add(new TopK<T, uint32_t>());
    add(new TopK<T, int64_t>());
    add(new TopK<T, uint64_t>());
#define TFCC_RUNTIME_ADD_DIMENSION(DST, E) add(new GetDimension<T, DST>());
    TFCC_RUNTIME_FOR_ALL_TYPES(TFCC_RUNTIME_ADD_DIMENSION)
#undef TFCC_RUNTIME_ADD_DIMENSION
  }

 public:
  Collector() {
#define TFCC_RUNTIME_ADD(T, E) addForType<T>();
    TFCC_RUNTIME_FOR_ALL_TYPES(TFCC_RUNTIME_ADD)
#undef TFCC_RUNTIME_ADD
    add(new Not());
  }
  const std::vector<std::unique_ptr<Operation>>& get(const std::string& url) const {
    static const std::vector<std::unique_ptr<Operation>> empty;
    auto it = _operations.find(url);
    return it == _operations.end() ? empty : it->second;
  }
};

}  // namespace

const std::vector<std::unique_ptr<Operation>>& operations_for(const std::string& typeUrl) {
  static const Collector collector;
  return collector.get(typeUrl);
}

}  // namespace runtime
}  // namespace tfcc
