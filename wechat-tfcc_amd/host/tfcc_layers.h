// The callers of matmul that find their weights by name: scopes, data loaders, constants, and the layers
// built on them.  Same names, argument meaning and error texts as the reference:
//   Scope / ScopeGuard       tfcc/core/framework/tfcc_scope.{h,cpp}
//   DataLoader, NPZDataLoader tfcc/core/dataloaders/tfcc_dataloader.h, tfcc_npzdataloader.cpp
//   Constant<T>              tfcc/core/framework/tfcc_constant.cpp:35-115 (loaded once per device, scope and name)
//   Configure<T>             tfcc/core/framework/tfcc_configure.h (scalars by name)
//   layer::Dense, dense()    tfcc/core/layers/tfcc_denselayer.cpp:31-125
//   rnn::LSTMCell            tfcc/core/rnn/tfcc_lstmcell.cpp:34-96
//   rnn::GRUCell             tfcc/core/rnn/tfcc_grucell.cpp:46-105
//   rnn::PyTorchGRUCell      tfcc/core/rnn/tfcc_pytorchgrucell.cpp:53-118
// On the ROCm device Dense is one launch: the bias is added in the matmul's epilogue, which gives the bits of
// matmul followed by the broadcast add the reference runs.
#pragma once

#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

#include "../runtime/archive.h"
#include "tfcc_interfaces.h"

namespace tfcc {

// ---- scopes ----------------------------------------------------------------------------------------------
class ScopeGuard {
  bool _valid;

 public:
  ScopeGuard() : _valid(true) {}
  ScopeGuard(ScopeGuard&& g) noexcept : _valid(g._valid) { g._valid = false; }
  ScopeGuard(const ScopeGuard&) = delete;
  ScopeGuard& operator=(const ScopeGuard&) = delete;
  ~ScopeGuard();
};

class Scope {
  static Scope _root;
  static thread_local Scope* _currentScope;

  Scope* _parent;
  std::string _name;
  std::map<std::string, std::unique_ptr<Scope>> _children;
  std::mutex _mtx;

  Scope(Scope* parent, const std::string& name) : _parent(parent), _name(name) {}

 public:
  Scope(const Scope&) = delete;
  Scope& operator=(const Scope&) = delete;

  Scope& getChild(const std::string& name);
  Scope* getParent() { return _parent; }
  const std::string& getName() const { return _name; }
  std::string getFullName() const;  // "a/b/" for the scope b inside a; "" for the root

  static Scope& getRootScope() { return _root; }
  static Scope& getCurrentScope() { return *_currentScope; }
  static void pushScope(const std::string& name);
  static void popScope();
  static ScopeGuard scope(const std::string& name);
};

// ---- data loaders ------------------------------------------------------------------------------------------
class DataLoader {
  static DataLoader* _defaultDataLoader;

 public:
  virtual ~DataLoader() {}
  // (shape, type, data); type is one of i1 i2 i4 i8 u1 u2 u4 u8 f4 f8, data the elements in C order
  virtual const std::tuple<Shape, std::string, std::string>& loadData(const std::string& name) const = 0;
  virtual std::vector<std::tuple<std::string, std::string>> getAllNames() const = 0;
  virtual bool hasData(const std::string& name) const = 0;

  static DataLoader* getGlobalDefault();
  static void setGlobalDefault(DataLoader* loader);
};

class NPZDataLoader : public DataLoader {
  std::map<std::string, std::tuple<Shape, std::string, std::string>> _dataMap;
  void fill(const std::map<std::string, std::string>& members);

 public:
  explicit NPZDataLoader(const std::string& path);
  NPZDataLoader(const char* data, size_t dataLen);
  const std::tuple<Shape, std::string, std::string>& loadData(const std::string& name) const override;
  std::vector<std::tuple<std::string, std::string>> getAllNames() const override;
  bool hasData(const std::string& name) const override;
};

namespace detail {
template <class T>
std::vector<T> elements_of(const std::tuple<Shape, std::string, std::string>& entry) {
  runtime::NpyArray a;
  a.shape = std::get<0>(entry).toVector();
  a.type = std::get<1>(entry);
  a.body = std::get<2>(entry);
  return runtime::convert_elements<T>(a);
}
template <class T> struct TypeKey;
#define TFCC_TYPE_KEY(T, K) template <> struct TypeKey<T> { static constexpr int value = K; };
TFCC_TYPE_KEY(float, 0) TFCC_TYPE_KEY(double, 1) TFCC_TYPE_KEY(int8_t, 2) TFCC_TYPE_KEY(uint8_t, 3)
TFCC_TYPE_KEY(int16_t, 4) TFCC_TYPE_KEY(uint16_t, 5) TFCC_TYPE_KEY(int32_t, 6) TFCC_TYPE_KEY(uint32_t, 7)
TFCC_TYPE_KEY(int64_t, 8) TFCC_TYPE_KEY(uint64_t, 9)
#undef TFCC_TYPE_KEY
}  // namespace detail

// ---- constants ---------------------------------------------------------------------------------------------
// A named tensor in device memory, loaded through the global DataLoader the first time it is asked for under
// (device, scope, name) and kept until the device goes away.
template <class T>
class Constant : public Tensor<T> {
  T* _data = nullptr;
  Allocator& _allocator;
  std::mutex _mtx;

  void setData(const Shape& shape, const std::vector<T>& data) {
    if (_data != nullptr) throw RuntimeError("Reset constant data");
    this->_shape = shape;
    if (shape.area() == 0) return;
    _data = static_cast<T*>(_allocator.malloc(sizeof(T) * static_cast<size_t>(shape.area())));
    if (_data == nullptr) throw ResourceExhaustedError();
    Device::getThreadDefault()->getInterface(T()).getDataInterface().set(_data, data.data(), shape.area());
  }

 public:
  explicit Constant(Allocator& allocator) : _allocator(allocator) {}
  ~Constant() override {
    if (_data) _allocator.free(_data);
  }

  const T* data() const override { return _data; }
  void sync() const override {
    if (Session* s = Session::getThreadDefault()) s->sync();
  }
  bool available() const override {
    Device* d = Device::getThreadDefault();
    return d != nullptr && &d->getAllocator() == &_allocator;
  }

  using ProcFunc = std::function<std::pair<Shape, std::vector<T>>(Shape, std::vector<T>)>;

  static Constant& getConstant(const std::string& name, ProcFunc preprocess = nullptr) {
    Device* device = Device::getThreadDefault();
    if (device == nullptr) throw RuntimeError("no default device on this thread: call an initialize function first");
    Scope& scope = Scope::getCurrentScope();
    std::shared_ptr<void> slot = device->getConstantSlot(&scope, name, detail::TypeKey<T>::value, [device] {
      return std::static_pointer_cast<void>(std::make_shared<Constant<T>>(device->getAllocator()));
    });
    Constant& constant = *static_cast<Constant*>(slot.get());
    std::lock_guard<std::mutex> lck(constant._mtx);
    if (constant._data != nullptr) return constant;
    const std::string fullName = scope.getFullName() + name;
    if (DataLoader::getGlobalDefault() == nullptr) throw RuntimeError("no global data loader");
    const auto& entry = DataLoader::getGlobalDefault()->loadData(fullName);
    Shape shape = std::get<0>(entry);
    std::vector<T> values = detail::elements_of<T>(entry);
    if (values.size() != shape.area()) throw RuntimeError("DataLoader return a invalid data. Constant name: " + fullName);
    if (preprocess) std::tie(shape, values) = preprocess(shape, values);
    constant.setData(shape, values);
    return constant;
  }
};

// ---- configures: scalars by name (the first element of the array stored under scope + name) --------------------
template <class T>
struct Configure {
  static T getConfigure(const std::string& name, bool& existed) {
    const std::string fullName = Scope::getCurrentScope().getFullName() + name;
    DataLoader* loader = DataLoader::getGlobalDefault();
    existed = loader != nullptr && loader->hasData(fullName);
    if (!existed) return T();
    std::vector<T> values = detail::elements_of<T>(loader->loadData(fullName));
    if (values.size() != 1) throw RuntimeError("DataLoader return a invalid data. Configure name: " + fullName);
    return values[0];
  }
  static T getConfigure(const std::string& name, T defaultValue) {
    bool existed = false;
    T v = getConfigure(name, existed);
    return existed ? v : defaultValue;
  }
  static T getConfigure(const std::string& name) {
    bool existed = false;
    T v = getConfigure(name, existed);
    if (!existed) throw RuntimeError("Configure: [" + Scope::getCurrentScope().getFullName() + name + "] not found");
    return v;
  }
};

// ---- layers --------------------------------------------------------------------------------------------------
namespace layer {

template <class T>
class Dense {
  bool _initialized = false;
  Constant<T>* _kernel = nullptr;
  Constant<T>* _bias = nullptr;
  unsigned _units;
  bool _useBias;
  std::string _name, _kernelName = "kernel", _biasName = "bias";

 public:
  Dense(unsigned units, bool useBias) : Dense(units, useBias, "dense") {}
  Dense(unsigned units, bool useBias, std::string name) : _units(units), _useBias(useBias), _name(std::move(name)) {}

  void setKernelName(std::string name) { _kernelName = std::move(name); }
  void setBiasName(std::string name) { _biasName = std::move(name); }

  Variable<T> operator()(const Tensor<T>& inputs) {
    auto scopeG = Scope::scope(_name);
    if (!_initialized) {
      _kernel = &Constant<T>::getConstant(_kernelName);
      if (_kernel->shape().size() != 2) throw InvalidDataError("invalid kernel");
      if (_units != 0 && _units != _kernel->shape(1)) throw InvalidDataError("kernel and units don't match");
      if (_useBias) {
        _bias = &Constant<T>::getConstant(_biasName);
        if (_bias->shape().size() != 1) throw InvalidDataError("invalid bias");
        if (_units != 0 && _units != _bias->shape(0)) throw InvalidDataError("bias and units don't match");
        if (_bias->shape(0) != _kernel->shape(1)) throw InvalidDataError("bias and kernel don't match");
      }
      _initialized = true;
    }
    if (inputs.shape().size() < 2) throw InvalidArgumentError("invalid inputs");
    if (inputs.shape(inputs.shape().size() - 1) != _kernel->shape(0)) throw InvalidArgumentError("inputs and kernel don't match");
    return _useBias ? blas::matmul(inputs, *_kernel, *_bias) : blas::matmul(inputs, *_kernel);
  }
};

template <class T>
Variable<T> dense(const Tensor<T>& inputs, unsigned units, bool useBias) {
  return Dense<T>(units, useBias)(inputs);
}
template <class T>
Variable<T> dense(const Tensor<T>& inputs, unsigned units, bool useBias, std::string name) {
  return Dense<T>(units, useBias, std::move(name))(inputs);
}
template <class T>
Variable<T> dense(const Tensor<T>& inputs, unsigned units, bool useBias, std::string name, std::string kernelName,
                  std::string biasName) {
  Dense<T> layer(units, useBias, std::move(name));
  layer.setKernelName(std::move(kernelName));
  layer.setBiasName(std::move(biasName));
  return layer(inputs);
}

}  // namespace layer

namespace rnn {

// One step of an LSTM whose kernel is [inputSize + units, 4 units] (rows of the inputs first, then of h) under
// "<name>/kernel" and "<name>/bias"; forget bias 1.  With sequence lengths a row whose length is at most `step` keeps
// the state it came with (tfcc/core/rnn/tfcc_lstmcell.cpp:81-91).
template <class T>
class LSTMCell {
  bool _initialized = false;
  Constant<T>* _kernel = nullptr;
  Constant<T>* _bias = nullptr;
  unsigned _units;
  std::string _name;

 public:
  struct State {
    Variable<T> cs, h;
    State() = default;
    State(unsigned batch, unsigned units) : cs({batch, units}), h({batch, units}) {}
  };

  explicit LSTMCell(unsigned units) : LSTMCell(units, "lstm_cell") {}
  LSTMCell(unsigned units, std::string name) : _units(units), _name(std::move(name)) {}

  State zeroState(unsigned batch) {
    State state(batch, _units);
    data::zeros(state.cs);
    data::zeros(state.h);
    return state;
  }

  std::pair<Variable<T>, State> operator()(const Tensor<T>& inputs, const State& state, size_t step = 0,
                                           const std::vector<unsigned>& lengths = {}) {
    if (inputs.shape().size() != 2) throw InvalidArgumentError("invalid inputs");
    if (inputs.shape(0) != state.cs.shape(0)) throw InvalidArgumentError("state and inputs don't match");
    if (lengths.size() != 0 && lengths.size() != inputs.shape(0)) throw InvalidArgumentError("invalid lengths");
    auto scopeG = Scope::scope(_name);
    if (!_initialized) {
      _kernel = &Constant<T>::getConstant("kernel");
      _bias = &Constant<T>::getConstant("bias");
      _initialized = true;
    }
    if (_kernel->shape().size() != 2 || _kernel->shape(0) <= inputs.shape(1)) throw InvalidDataError("invalid kernel");
    State next;
    Interface<T>& interface = Operation<T>::getCurrentInterface();
    std::tie(next.h, next.cs) = interface.getCellInterface().processLSTMCell(
        state.cs, blas::matmul(inputs, View<T>(*_kernel, _kernel->shape(), 0, inputs.shape(1))),
        blas::matmul(state.h, View<T>(*_kernel, _kernel->shape(), inputs.shape(1))), *_bias, static_cast<T>(1));
    // a sequence that has ended keeps its state (tfcc/core/rnn/tfcc_lstmcell.cpp:81-91)
    for (unsigned i = 0; i < lengths.size(); ++i) {
      if (step < lengths[i]) continue;
      View<T> vcs(state.cs, state.cs.shape(), i, i + 1);
      base::assign_to(vcs, 0, i, next.cs);
      View<T> vh(state.h, state.h.shape(), i, i + 1);
      base::assign_to(vh, 0, i, next.h);
    }
    Variable<T> output = data::copy(next.h);
    return std::make_pair(std::move(output), std::move(next));
  }
};

// One step of a GRU in TensorFlow's layout (tfcc/core/rnn/tfcc_grucell.cpp:46-105): "<name>/gates/kernel"
// [inputSize + units, 2 units] with "gates/bias", "<name>/candidate/kernel" [inputSize + units, units] with
// "candidate/bias".
template <class T>
class GRUCell {
  bool _initialized = false;
  unsigned _units;
  std::string _name;
  Constant<T>* _gatesKernel = nullptr;
  Constant<T>* _gatesBias = nullptr;
  Constant<T>* _candidateKernel = nullptr;
  Constant<T>* _candidateBias = nullptr;

 public:
  using State = Variable<T>;

  explicit GRUCell(unsigned units) : GRUCell(units, "gru_cell") {}
  GRUCell(unsigned units, std::string name) : _units(units), _name(std::move(name)) {}

  State zeroState(unsigned batch) {
    State state({batch, _units});
    data::zeros(state);
    return state;
  }

  std::pair<Variable<T>, State> operator()(const Tensor<T>& input, const State& state, size_t step = 0,
                                           const std::vector<unsigned>& lengths = {}) {
    if (input.shape().size() != 2) throw InvalidArgumentError("invalid inputs");
    if (input.shape(0) != state.shape(0)) throw InvalidArgumentError("state and inputs don't match");
    if (lengths.size() != 0 && lengths.size() != input.shape(0)) throw InvalidArgumentError("invalid lengths");
    auto scopeG = Scope::scope(_name);
    if (!_initialized) {
      {
        auto scopeGates = Scope::scope("gates");
        _gatesKernel = &Constant<T>::getConstant("kernel");
        _gatesBias = &Constant<T>::getConstant("bias");
      }
      {
        auto scopeCandidate = Scope::scope("candidate");
        _candidateKernel = &Constant<T>::getConstant("kernel");
        _candidateBias = &Constant<T>::getConstant("bias");
      }
      _initialized = true;
    }
    Variable<T> gi = base::concat<T>({&input, &state}, 1);
    Variable<T> value = blas::matmul(gi, *_gatesKernel);
    Interface<T>& interface = Operation<T>::getCurrentInterface();
    Variable<T> ci = interface.getCellInterface().processGRUCellGates(state, input, value, *_gatesBias);
    State h = interface.getCellInterface().processGRUCellCandidate(state, value, *_gatesBias,
                                                                   blas::matmul(ci, *_candidateKernel), *_candidateBias);
    for (unsigned i = 0; i < lengths.size(); ++i) {  // tfcc/core/rnn/tfcc_grucell.cpp:94-102
      if (step < lengths[i]) continue;
      View<T> vs(state, state.shape(), i, i + 1);
      base::assign_to(vs, 0, i, h);
    }
    Variable<T> output = data::copy(h);
    return std::make_pair(std::move(output), std::move(h));
  }
};

// One step of a GRU in PyTorch's formulation (tfcc/core/rnn/tfcc_pytorchgrucell.cpp:53-118): "weight_gates"
// [inputSize + units, 2 units], "weight_candidate_i" [inputSize, units], "weight_candidate_h" [units, units] and the
// three biases.  The reference joins them into an input kernel [inputSize, 3 units] and a state kernel
// [units, 3 units] at first use and keeps those; so does this class (slice + concat on the device).
template <class T>
class PyTorchGRUCell {
  bool _initialized = false;
  unsigned _units;
  std::string _name;
  Constant<T>* _gatesBias = nullptr;
  Constant<T>* _candidateIBias = nullptr;
  Constant<T>* _candidateHBias = nullptr;
  Variable<T> _inputKernel, _stateKernel;

 public:
  using State = Variable<T>;

  explicit PyTorchGRUCell(unsigned units) : PyTorchGRUCell(units, "gru_cell") {}
  PyTorchGRUCell(unsigned units, std::string name) : _units(units), _name(std::move(name)) {}

  State zeroState(unsigned batch) {
    State state({batch, _units});
    data::zeros(state);
    return state;
  }

  std::pair<Variable<T>, State> operator()(const Tensor<T>& input, const State& state, size_t step = 0,
                                           const std::vector<unsigned>& lengths = {}) {
    if (input.shape().size() != 2) throw InvalidArgumentError("invalid inputs");
    if (input.shape(0) != state.shape(0)) throw InvalidArgumentError("state and inputs don't match");
    if (lengths.size() != 0 && lengths.size() != input.shape(0)) throw InvalidArgumentError("invalid lengths");
    auto scopeG = Scope::scope(_name);
    if (!_initialized) {
      _gatesBias = &Constant<T>::getConstant("bias_gates");
      _candidateIBias = &Constant<T>::getConstant("bias_candidate_i");
      _candidateHBias = &Constant<T>::getConstant("bias_candidate_h");
      Constant<T>& gatesKernel = Constant<T>::getConstant("weight_gates");
      Constant<T>& candidateIKernel = Constant<T>::getConstant("weight_candidate_i");
      Constant<T>& candidateHKernel = Constant<T>::getConstant("weight_candidate_h");
      const unsigned inputSize = candidateIKernel.shape(0);
      if (gatesKernel.shape().size() != 2 || gatesKernel.shape(0) <= inputSize) throw InvalidDataError("invalid kernel");
      View<T> g1(gatesKernel, gatesKernel.shape(), 0, inputSize), g2(gatesKernel, gatesKernel.shape(), inputSize);
      _inputKernel = base::concat<T>({&g1, &candidateIKernel}, 1);
      _stateKernel = base::concat<T>({&g2, &candidateHKernel}, 1);
      _initialized = true;
    }
    Variable<T> inputValue = blas::matmul(input, _inputKernel);
    Variable<T> stateValue = blas::matmul(state, _stateKernel);
    State hy = Operation<T>::getCurrentInterface().getCellInterface().processPyTorchGRUCell(
        state, inputValue, stateValue, *_gatesBias, *_candidateIBias, *_candidateHBias);
    for (unsigned i = 0; i < lengths.size(); ++i) {  // tfcc/core/rnn/tfcc_pytorchgrucell.cpp:103-111
      if (step < lengths[i]) continue;
      View<T> vs(state, state.shape(), i, i + 1);
      base::assign_to(vs, 0, i, hy);
    }
    Variable<T> output = data::copy(hy);
    return std::make_pair(std::move(output), std::move(hy));
  }
};

}  // namespace rnn

}  // namespace tfcc
