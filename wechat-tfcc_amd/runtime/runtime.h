// tfcc_runtime on the ROCm device: loads a model archive (model.pb + model.npz in a zip), builds
// one executable step list per graph and runs it with every tensor resident in HBM.
//
// What it mirrors in the reference:
//   Model       tfcc_runtime/framework/model.h:37-103, model.cpp:57-181,283-330
//   Graph       tfcc_runtime/framework/graph.h, graph.cpp:30-123
//   SymbolManager tfcc_runtime/framework/symbolmanager.cpp:150-215
//   Operation   tfcc_runtime/operations/operation.h, operation.cpp:246-300 (lookup by the type
//               URL of the node's Any and by version; the first operation that accepts wins)
// What differs by design: no x86 code generation (the reference assembles a call sequence with
// Xbyak, graph.cpp:98-123) - a graph is a vector of bound C++ closures, and because a step list
// with fixed shapes issues the same kernel sequence every run, the whole list can be recorded once
// into a HIP graph and replayed with a single launch (Graph::enableReplay).
#pragma once

#include <deque>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <ostream>
#include <set>
#include <string>
#include <unordered_map>
#include <vector>

#include "archive.h"
#include "tfcc_interfaces.h"
#include "wire.h"

namespace tfcc {
namespace runtime {

// tfcc_runtime/proto/common.proto:5-20
enum DataType : int {
  UNKNOW = 0,
  FLOAT = 1,
  UINT8 = 2,
  INT8 = 3,
  UINT16 = 4,
  INT16 = 5,
  INT32 = 6,
  INT64 = 7,
  BOOL = 9,
  DOUBLE = 11,
  UINT32 = 12,
  UINT64 = 13,
  COMPLEX64 = 14,
};

size_t data_type_size(DataType t);  // 0 for types the runtime cannot hold
const char* data_type_name(DataType t);

enum class SymbolType { VARIABLE, VIEW, CONSTANT_TENSOR, VALUE, CONSTANT_VALUE, VECTOR, CONSTANT_VECTOR };
inline bool is_tensor(SymbolType t) {
  return t == SymbolType::VARIABLE || t == SymbolType::VIEW || t == SymbolType::CONSTANT_TENSOR;
}
inline bool is_value(SymbolType t) { return t == SymbolType::VALUE || t == SymbolType::CONSTANT_VALUE; }
inline bool is_vector(SymbolType t) { return t == SymbolType::VECTOR || t == SymbolType::CONSTANT_VECTOR; }

// ---- decoded messages (tfcc_runtime/proto/model.proto, data.proto) ---------------------------------
namespace proto {

struct Value {  // common.proto Value: oneof { int64 = 1, uint64 = 2, float = 3, double = 4 }
  enum Kind { NONE, INT64, UINT64, FLOAT, DOUBLE } kind = NONE;
  int64_t i = 0;
  uint64_t u = 0;
  float f = 0;
  double d = 0;
  template <class T>
  bool get(T& out) const {
    switch (kind) {
      case INT64: out = static_cast<T>(i); return true;
      case UINT64: out = static_cast<T>(u); return true;
      case FLOAT: out = static_cast<T>(f); return true;
      case DOUBLE: out = static_cast<T>(d); return true;
      default: return false;
    }
  }
};
Value parse_value(wire::Reader r);

struct Dimension {
  bool isParam = false;
  unsigned value = 0;
  std::string param;
};

struct Symbol {
  std::string name;
  DataType dtype = UNKNOW;
  bool hasType = false;
  SymbolType stype = SymbolType::VARIABLE;
  std::string ref;  // constant_tensor / constant_value / constant_vector
  std::vector<Dimension> shape;
};

struct Node {
  std::string name;
  std::vector<std::string> inputs, outputs;
  std::string typeUrl;    // google.protobuf.Any.type_url
  std::string operation;  // google.protobuf.Any.value: the packed operation message
  unsigned version = 0;
  std::string debugString() const;
};

struct Graph {
  std::string name;
  std::vector<std::string> inputs, outputs;
  std::vector<Symbol> symbols;
  std::vector<Node> nodes;
};

struct Model {
  uint64_t protoVersion = 0;
  std::string name;
  std::vector<Graph> graphs;
  std::string entranceGraphName;
};

Model parse_model(const std::string& bytes);

struct DataItem {  // data.proto:5-10
  std::string name;
  DataType dtype = UNKNOW;
  std::vector<unsigned> shape;
  std::string data;
};
std::vector<DataItem> parse_inputs(const std::string& bytes);          // Inputs{items = 1}
std::string serialize_inputs(const std::vector<DataItem>& items);      // for callers and tests
std::vector<DataItem> parse_outputs(const std::string& bytes);         // Outputs{items = 2}
std::string serialize_outputs(const std::vector<DataItem>& items);

}  // namespace proto

inline std::string type_url(const std::string& packageAndMessage) {
  return "type.googleapis.com/tfcc.runtime.operations." + packageAndMessage;
}

class UnknowNodeError : public Exception {
 public:
  explicit UnknowNodeError(const proto::Node& node)
      : Exception("Unknow node: " + node.name + " operation: " + node.typeUrl +
                  " version: " + std::to_string(node.version)) {}
};

// ---- element types the runtime holds ------------------------------------------------------------------
template <class T>
struct DataTypeOf;
#define TFCC_RUNTIME_FOR_ALL_TYPES(M)                                                                       \
  M(float, FLOAT) M(double, DOUBLE) M(int8_t, INT8) M(uint8_t, UINT8) M(int16_t, INT16) M(uint16_t, UINT16) \
      M(int32_t, INT32) M(uint32_t, UINT32) M(int64_t, INT64) M(uint64_t, UINT64)
#define TFCC_RUNTIME_DTYPE_OF(T, E) \
  template <>                       \
  struct DataTypeOf<T> {            \
    static constexpr DataType value = E; \
  };
TFCC_RUNTIME_FOR_ALL_TYPES(TFCC_RUNTIME_DTYPE_OF)
#undef TFCC_RUNTIME_DTYPE_OF

// A constant resident on the device: memory comes from the device allocator, lives as long as the
// model's constant store (cf. tfcc::Constant / ConstantManager, tfcc/core/framework/tfcc_constant.cpp:69-76).
template <class T>
class ConstantTensor : public Tensor<T> {
  Device* _device;
  T* _data;

 public:
  ConstantTensor(Device* device, Shape shape, const std::vector<T>& values);
  ~ConstantTensor() override;
  const T* data() const override { return _data; }
  void sync() const override {}
  bool available() const override { return true; }
};

// Weights of one model on one device, created on first use.  Keys are "<graph name>/<ref>".
class ConstantStore {
 public:
  struct Holder {
    virtual ~Holder() {}
  };

 private:
  const NpzData& _npz;
  Device* _device;
  std::mutex _mutex;
  std::map<std::pair<std::string, int>, std::unique_ptr<Holder>> _tensors;

 public:
  ConstantStore(const NpzData& npz, Device* device);
  ~ConstantStore();
  template <class T>
  const Tensor<T>& getConstant(const std::string& key);
  template <class T>
  T getConfigure(const std::string& key);
  template <class T>
  std::vector<T> getVector(const std::string& key);
  Device* device() const { return _device; }
};

// ---- symbols ------------------------------------------------------------------------------------------
struct SymbolInfo {
  DataType dtype;
  SymbolType stype;
  size_t pos;
  std::vector<proto::Dimension> shape;
};

template <class T>
struct SymbolSlot {
  Variable<T> variable;       // VARIABLE, or the owner behind a VIEW set from an rvalue
  View<T> view;               // VIEW
  const Tensor<T>* constant = nullptr;  // CONSTANT_TENSOR
  T value = T();              // VALUE / CONSTANT_VALUE
  std::vector<T> vector;      // VECTOR / CONSTANT_VECTOR
};

class SymbolManager {
  std::unordered_map<std::string, SymbolInfo> _map;
#define TFCC_RUNTIME_SLOTS(T, E) std::deque<SymbolSlot<T>> _slots_##E;
  TFCC_RUNTIME_FOR_ALL_TYPES(TFCC_RUNTIME_SLOTS)
#undef TFCC_RUNTIME_SLOTS
  std::deque<SymbolSlot<uint8_t>> _slots_BOOL;

  template <class T>
  std::deque<SymbolSlot<T>>& slots(DataType dtype);
  template <class T>
  SymbolSlot<T>& slot(const std::string& name, const SymbolInfo*& info);
  template <class T>
  void create(const proto::Symbol& symbol, ConstantStore& constants, const std::string& scope);

 public:
  SymbolManager(const std::vector<proto::Symbol>& symbols, ConstantStore& constants, const std::string& scope);
  const SymbolInfo& getSymbolInfo(const std::string& name) const;
  bool has(const std::string& name) const { return _map.count(name) != 0; }

  // pointers stay valid for the life of the manager
  template <class T>
  const Tensor<T>* getTensor(const std::string& name, T = T());
  template <class T>
  Variable<T>* getVariable(const std::string& name, T = T());
  template <class T>
  View<T>* getView(const std::string& name, T = T());
  template <class T>
  void setView(const std::string& name, Variable<T>&& v);
  template <class T>
  T* getValue(const std::string& name, T = T());
  template <class T>
  std::vector<T>* getVector(const std::string& name, T = T());
};

// ---- graph ----------------------------------------------------------------------------------------------
class Model;
class Graph;

// One registered operation: says which nodes it accepts and binds an accepted node to a step.
class Operation {
 public:
  virtual ~Operation() {}
  virtual std::string getOperationTypeUrl() const = 0;
  virtual std::set<unsigned> getOperationVersions() const { return {1}; }
  // true and steps appended to the graph when the node is accepted
  virtual bool process(const proto::Node& node, Graph& graph) const = 0;
};

const std::vector<std::unique_ptr<Operation>>& operations_for(const std::string& typeUrl);

// What the build-time fusion pass decided for one node: run it as written (NONE), skip it because a
// later node runs it as part of a fused step (ABSORBED, partner = that node), or run it fused with
// the producer `partner` of one of its inputs (side: which input of an Add the product is).
struct FusionPlan {
  enum Kind { NONE, ABSORBED, MATMUL_GELU, MATMUL_ADD, DIV_SOFTMAX, MOVE_IDENTITY, MATMUL_PERMUTED, MATMUL_GROUPED, ATTENTION } kind = NONE;
  size_t partner = 0;
  unsigned side = 0;
  // MATMUL_PERMUTED: the Transpose nodes folded into a Matmul (producer of input 0 / of input 1 /
  // consumer of the output), kNoNode where there is none
  static constexpr size_t kNoNode = ~static_cast<size_t>(0);
  size_t transposeA = kNoNode, transposeB = kNoNode, transposeC = kNoNode;
  // ATTENTION (on the second Matmul): the first Matmul, the Softmax between them, the Div folded into the
  // Softmax and the Transpose of the second Matmul's other operand; transposeA / transposeB are those of
  // the first Matmul, transposeC that of the second
  size_t scoresNode = kNoNode, softmaxNode = kNoNode, divNode = kNoNode, transposeV = kNoNode;
  // ... and the Add of a mask between the (divided) scores and the Softmax; maskSide: which input of it the mask is
  size_t maskNode = kNoNode;
  unsigned maskSide = 0;
  // MATMUL_GROUPED: the MatmulWithBias nodes (this one first) that share their first input and run as one launch
  std::vector<size_t> group;
};
std::vector<FusionPlan> plan_fusions(const proto::Graph& graph, SymbolManager& symbols);
void emit_fused(const proto::Graph& graphProto, const FusionPlan& plan, size_t node, Graph& graph);

class Graph {
  Model& _model;
  const proto::Graph& _proto;
  std::unique_ptr<SymbolManager> _symbols;
  struct Step {
    std::function<void()> run;
    size_t node;
  };
  std::vector<Step> _steps;
  size_t _currentNode = 0;
  bool _built = false;
  static thread_local bool _recordDetailError;
  static thread_local bool _fusion;

  // replay state
  bool _replayWanted = false;
  bool _warm = false;            // one step-by-step run has filled the allocator's cache
  void* _graphExec = nullptr;
  bool _captured = false;
  bool _captureFailed = false;   // a recording was tried and a step could not be recorded: run step by step
  Session* _replaySession = nullptr;  // the session the recording was made on: its stream and allocator own it
  std::vector<void*> _pinned;    // blocks the recording uses that no symbol owns
  std::set<std::string> _inputOwned;  // tensor inputs held in buffers of the graph's own
  void enableReplayReset();
  void runSteps();

  std::string errorString(const std::string& what, size_t node);

 public:
  Graph(Model& model, const proto::Graph& graphProto, ConstantStore& constants);
  ~Graph();
  Graph(const Graph&) = delete;
  Graph& operator=(const Graph&) = delete;

  std::string getGraphName() const { return _proto.name; }
  const std::vector<std::string>& getInputs() const { return _proto.inputs; }
  const std::vector<std::string>& getOutputs() const { return _proto.outputs; }

  void buildGraph();
  // runs every step in node order; a failing step raises RuntimeError with the step's message
  void process();

  // After the first process() with replay enabled, the step list is recorded into a HIP graph; every
  // later process() is one graph launch.  Inputs must then be set through setInput(name, tensor)
  // forms, which copy into the fixed input buffers the recording saw.  Only valid while shapes do
  // not change; disable to go back to step-by-step execution.
  void enableReplay(bool enable);
  bool replaying() const { return _captured; }

  template <class T>
  void setInput(const std::string& name, const Tensor<T>& tensor);
  template <class T>
  void setInput(const std::string& name, Variable<T>&& variable);
  template <class T>
  typename std::enable_if<std::is_arithmetic<T>::value, void>::type setInput(const std::string& name, T value);

  template <class T>
  const Tensor<T>& getTensor(const std::string& name, T = T()) {
    return *_symbols->getTensor(name, T());
  }
  template <class T>
  T getValue(const std::string& name, T = T()) {
    return *_symbols->getValue(name, T());
  }
  template <class T>
  const std::vector<T>& getVector(const std::string& name, T = T()) {
    return *_symbols->getVector(name, T());
  }

  SymbolManager& getSymbolManager() { return *_symbols; }
  Model& getModel() { return _model; }
  size_t stepCount() const { return _steps.size(); }  // bound steps after building (fused nodes share one)
  // used by operations while the graph is being built
  void addStep(std::function<void()> step) { _steps.push_back(Step{std::move(step), _currentNode}); }

  // graphs built afterwards on this thread fuse node sequences (default) or run every node as written
  static void setFusionThreadLocal(bool enable) { _fusion = enable; }
  static void setRecordDetailErrorThreadLocal(bool enable) { _recordDetailError = enable; }
  static bool isRecordDetailError() { return _recordDetailError; }
};

// ---- model ----------------------------------------------------------------------------------------------
class Model {
  struct PerSession {
    std::vector<std::unique_ptr<Graph>> graphs;
  };
  std::mutex _mutex;
  proto::Model _proto;
  std::string _userData;
  std::unique_ptr<NpzData> _npz;
  std::map<Device*, std::unique_ptr<ConstantStore>> _constants;
  std::unordered_map<const Session*, PerSession> _sessions;
  std::shared_ptr<bool> _alive{new bool(true)};  // lets a session's release callback outlive the model

  PerSession& initializeGraphs(Session* session);
  void releaseGraphs(const Session* session);

 public:
  // `data`: the bytes of the model archive
  explicit Model(const std::string& data);
  ~Model();
  Model(const Model&) = delete;
  Model& operator=(const Model&) = delete;

  // serialized tfcc.runtime.data.Inputs in, serialized Outputs out (model.cpp:145-181): inputs are
  // copied host -> device, the entrance graph runs, every graph output is copied back
  void run(const std::string& inputs, std::string& outputs);
  void run(const std::vector<proto::DataItem>& inputs, std::vector<proto::DataItem>& outputs);

  // runs the entrance graph on the arrays of an .npz and compares each output present there
  // (model.cpp:185-280); prints a summary to `stream`
  bool test(const std::string& npz, std::ostream& stream);

  Graph& getEntranceGraph();
  Graph& getGraph(const std::string& name);
  const std::string& getUserData() const { return _userData; }
  const proto::Model& getProto() const { return _proto; }
};

}  // namespace runtime
}  // namespace tfcc
