#include "runtime.h"

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstring>
#include <sstream>

#include "tfcc_rocm.h"
#include "tfcc_rocm_device.h"

namespace tfcc {
namespace runtime {

size_t data_type_size(DataType t) {
  switch (t) {
    case FLOAT: case INT32: case UINT32: return 4;
    case DOUBLE: case INT64: case UINT64: return 8;
    case INT8: case UINT8: case BOOL: return 1;
    case INT16: case UINT16: return 2;
    default: return 0;
  }
}

const char* data_type_name(DataType t) {
  switch (t) {
    case FLOAT: return "FLOAT";
    case UINT8: return "UINT8";
    case INT8: return "INT8";
    case UINT16: return "UINT16";
    case INT16: return "INT16";
    case INT32: return "INT32";
    case INT64: return "INT64";
    case BOOL: return "BOOL";
    case DOUBLE: return "DOUBLE";
    case UINT32: return "UINT32";
    case UINT64: return "UINT64";
    case COMPLEX64: return "COMPLEX64";
    default: return "UNKNOW";
  }
}

// ---------------------------------------------------------------------------------------------------
// message decoding
// ---------------------------------------------------------------------------------------------------
namespace proto {

Value parse_value(wire::Reader r) {
  Value v;
  uint32_t f, t;
  while (r.next(f, t)) {
    if (f == 1 && t == 0) { v.kind = Value::INT64; v.i = static_cast<int64_t>(r.varint()); }
    else if (f == 2 && t == 0) { v.kind = Value::UINT64; v.u = r.varint(); }
    else if (f == 3 && t == 5) { v.kind = Value::FLOAT; v.f = r.float32(); }
    else if (f == 4 && t == 1) { v.kind = Value::DOUBLE; v.d = r.float64(); }
    else r.skip(t);
  }
  return v;
}

static std::string parse_ref(wire::Reader r) {
  std::string ref;
  uint32_t f, t;
  while (r.next(f, t)) {
    if (f == 1 && t == 2) ref = r.bytes();
    else r.skip(t);
  }
  return ref;
}

static Symbol parse_symbol(wire::Reader r) {
  Symbol s;
  uint32_t f, t;
  while (r.next(f, t)) {
    if (f == 1 && t == 2) s.name = r.bytes();
    else if (f == 2 && t == 0) s.dtype = static_cast<DataType>(r.varint());
    else if (f >= 3 && f <= 9 && t == 2) {
      static const SymbolType kinds[] = {SymbolType::VARIABLE, SymbolType::VIEW, SymbolType::CONSTANT_TENSOR,
                                         SymbolType::VALUE, SymbolType::CONSTANT_VALUE, SymbolType::VECTOR,
                                         SymbolType::CONSTANT_VECTOR};
      s.stype = kinds[f - 3];
      s.hasType = true;
      s.ref = parse_ref(r.sub());
    } else if (f == 10 && t == 2) {
      wire::Reader shape = r.sub();
      uint32_t sf, st;
      while (shape.next(sf, st)) {
        if (sf == 1 && st == 2) {
          Dimension d;
          wire::Reader dim = shape.sub();
          uint32_t df, dt;
          while (dim.next(df, dt)) {
            if (df == 1 && dt == 0) d.value = static_cast<unsigned>(dim.varint());
            else if (df == 2 && dt == 2) { d.isParam = true; d.param = dim.bytes(); }
            else dim.skip(dt);
          }
          s.shape.push_back(std::move(d));
        } else {
          shape.skip(st);
        }
      }
    } else {
      r.skip(t);
    }
  }
  return s;
}

static Node parse_node(wire::Reader r) {
  Node n;
  uint32_t f, t;
  while (r.next(f, t)) {
    if (f == 1 && t == 2) n.name = r.bytes();
    else if (f == 2 && t == 2) n.inputs.push_back(r.bytes());
    else if (f == 3 && t == 2) n.outputs.push_back(r.bytes());
    else if (f == 4 && t == 2) {  // google.protobuf.Any{type_url = 1, value = 2}
      wire::Reader any = r.sub();
      uint32_t af, at;
      while (any.next(af, at)) {
        if (af == 1 && at == 2) n.typeUrl = any.bytes();
        else if (af == 2 && at == 2) n.operation = any.bytes();
        else any.skip(at);
      }
    } else if (f == 5 && t == 0) n.version = static_cast<unsigned>(r.varint());
    else r.skip(t);
  }
  return n;
}

static Graph parse_graph(wire::Reader r) {
  Graph g;
  uint32_t f, t;
  while (r.next(f, t)) {
    if (f == 1 && t == 2) g.name = r.bytes();
    else if (f == 2 && t == 2) g.inputs.push_back(r.bytes());
    else if (f == 3 && t == 2) g.outputs.push_back(r.bytes());
    else if (f == 4 && t == 2) g.symbols.push_back(parse_symbol(r.sub()));
    else if (f == 5 && t == 2) g.nodes.push_back(parse_node(r.sub()));
    else r.skip(t);
  }
  return g;
}

Model parse_model(const std::string& bytes) {
  Model m;
  wire::Reader r(bytes);
  uint32_t f, t;
  while (r.next(f, t)) {
    if (f == 1 && t == 0) m.protoVersion = r.varint();
    else if (f == 2 && t == 2) m.name = r.bytes();
    else if (f == 3 && t == 2) m.graphs.push_back(parse_graph(r.sub()));
    else if (f == 4 && t == 2) m.entranceGraphName = r.bytes();
    else r.skip(t);
  }
  return m;
}

std::string Node::debugString() const {
  std::ostringstream ss;
  ss << "name: \"" << name << "\"\n";
  for (auto& s : inputs) ss << "inputs: \"" << s << "\"\n";
  for (auto& s : outputs) ss << "outputs: \"" << s << "\"\n";
  ss << "operation { type_url: \"" << typeUrl << "\" value: <" << operation.size() << " bytes> }\n";
  ss << "version: " << version << "\n";
  return ss.str();
}

static DataItem parse_item(wire::Reader r) {
  DataItem item;
  uint32_t f, t;
  while (r.next(f, t)) {
    if (f == 1 && t == 2) item.name = r.bytes();
    else if (f == 2 && t == 0) item.dtype = static_cast<DataType>(r.varint());
    else if (f == 3) r.repeatedVarint(t, item.shape);
    else if (f == 4 && t == 2) item.data = r.bytes();
    else r.skip(t);
  }
  return item;
}

static std::vector<DataItem> parse_items(const std::string& bytes, uint32_t field) {
  std::vector<DataItem> items;
  wire::Reader r(bytes);
  uint32_t f, t;
  while (r.next(f, t)) {
    if (f == field && t == 2) items.push_back(parse_item(r.sub()));
    else r.skip(t);
  }
  return items;
}

static std::string serialize_items(const std::vector<DataItem>& items, uint32_t field) {
  wire::Writer w;
  for (const DataItem& item : items) {
    wire::Writer wi;
    if (!item.name.empty()) wi.bytes(1, item.name);
    if (item.dtype != UNKNOW) wi.varint(2, static_cast<uint64_t>(item.dtype));
    wi.packedVarint(3, item.shape);
    if (!item.data.empty()) wi.bytes(4, item.data);
    w.bytes(field, wi.str());
  }
  return w.take();
}

std::vector<DataItem> parse_inputs(const std::string& bytes) { return parse_items(bytes, 1); }
std::string serialize_inputs(const std::vector<DataItem>& items) { return serialize_items(items, 1); }
std::vector<DataItem> parse_outputs(const std::string& bytes) { return parse_items(bytes, 2); }
std::string serialize_outputs(const std::vector<DataItem>& items) { return serialize_items(items, 2); }

}  // namespace proto

// ---------------------------------------------------------------------------------------------------
// constants
// ---------------------------------------------------------------------------------------------------
template <class T>
ConstantTensor<T>::ConstantTensor(Device* device, Shape shape, const std::vector<T>& values)
    : Tensor<T>(std::move(shape)), _device(device), _data(nullptr) {
  if (values.size() != this->size()) throw RuntimeError("constant: element count and shape differ");
  if (values.empty()) return;
  _data = static_cast<T*>(_device->malloc(values.size() * sizeof(T)));
  if (_data == nullptr) throw ResourceExhaustedError();
  _device->getInterface(T()).getDataInterface().set(_data, values.data(), values.size());
}

template <class T>
ConstantTensor<T>::~ConstantTensor() {
  if (_data) _device->free(_data);
}

namespace {
template <class T>
struct TensorHolder : ConstantStore::Holder {
  ConstantTensor<T> tensor;
  TensorHolder(Device* d, Shape s, const std::vector<T>& v) : tensor(d, std::move(s), v) {}
};
}  // namespace

ConstantStore::ConstantStore(const NpzData& npz, Device* device) : _npz(npz), _device(device) {}
ConstantStore::~ConstantStore() {}

template <class T>
const Tensor<T>& ConstantStore::getConstant(const std::string& key) {
  std::lock_guard<std::mutex> lk(_mutex);
  const auto id = std::make_pair(key, static_cast<int>(DataTypeOf<T>::value));
  auto it = _tensors.find(id);
  if (it == _tensors.end()) {
    const NpyArray& a = _npz.get(key);
    std::vector<T> values = convert_elements<T>(a);
    if (values.size() != a.count()) throw RuntimeError("constant \"" + key + "\": unsupported element type " + a.type);
    std::unique_ptr<Holder> h(new TensorHolder<T>(_device, Shape(a.shape), values));
    it = _tensors.emplace(id, std::move(h)).first;
  }
  return static_cast<TensorHolder<T>*>(it->second.get())->tensor;
}

template <class T>
std::vector<T> ConstantStore::getVector(const std::string& key) {
  const NpyArray& a = _npz.get(key);
  std::vector<T> values = convert_elements<T>(a);
  if (values.size() != a.count()) throw RuntimeError("constant \"" + key + "\": unsupported element type " + a.type);
  return values;
}

template <class T>
T ConstantStore::getConfigure(const std::string& key) {
  std::vector<T> v = getVector<T>(key);
  if (v.empty()) throw RuntimeError("constant \"" + key + "\" is empty");
  return v[0];
}

// ---------------------------------------------------------------------------------------------------
// symbols
// ---------------------------------------------------------------------------------------------------
#define TFCC_RUNTIME_SLOT_ACCESS(T, E)                                       \
  template <>                                                                \
  std::deque<SymbolSlot<T>>& SymbolManager::slots<T>(DataType dtype) {       \
    if (dtype == E) return _slots_##E;                                       \
    throw RuntimeError("type not match");                                    \
  }
TFCC_RUNTIME_SLOT_ACCESS(float, FLOAT)
TFCC_RUNTIME_SLOT_ACCESS(double, DOUBLE)
TFCC_RUNTIME_SLOT_ACCESS(int8_t, INT8)
TFCC_RUNTIME_SLOT_ACCESS(int16_t, INT16)
TFCC_RUNTIME_SLOT_ACCESS(uint16_t, UINT16)
TFCC_RUNTIME_SLOT_ACCESS(int32_t, INT32)
TFCC_RUNTIME_SLOT_ACCESS(uint32_t, UINT32)
TFCC_RUNTIME_SLOT_ACCESS(int64_t, INT64)
TFCC_RUNTIME_SLOT_ACCESS(uint64_t, UINT64)
#undef TFCC_RUNTIME_SLOT_ACCESS
// uint8_t also carries BOOL symbols (symbolmanager.cpp:236-246)
template <>
std::deque<SymbolSlot<uint8_t>>& SymbolManager::slots<uint8_t>(DataType dtype) {
  if (dtype == UINT8) return _slots_UINT8;
  if (dtype == BOOL) return _slots_BOOL;
  throw RuntimeError("type not match");
}

template <class T>
void SymbolManager::create(const proto::Symbol& symbol, ConstantStore& constants, const std::string& scope) {
  if (_map.count(symbol.name)) throw RuntimeError("name " + symbol.name + " has existed");
  if (!symbol.hasType) throw RuntimeError("invalid stype");
  auto& target = slots<T>(symbol.dtype);
  target.emplace_back();
  SymbolInfo info{symbol.dtype, symbol.stype, target.size() - 1, symbol.shape};
  SymbolSlot<T>& slot = target.back();
  const std::string key = scope + "/" + symbol.ref;
  if (info.stype == SymbolType::CONSTANT_TENSOR) slot.constant = &constants.getConstant<T>(key);
  else if (info.stype == SymbolType::CONSTANT_VALUE) slot.value = constants.getConfigure<T>(key);
  else if (info.stype == SymbolType::CONSTANT_VECTOR) slot.vector = constants.getVector<T>(key);
  _map.emplace(symbol.name, std::move(info));
}

SymbolManager::SymbolManager(const std::vector<proto::Symbol>& symbols, ConstantStore& constants,
                             const std::string& scope) {
  for (const proto::Symbol& s : symbols) {
    switch (s.dtype) {
#define TFCC_RUNTIME_CREATE(T, E) \
  case E: create<T>(s, constants, scope); break;
      TFCC_RUNTIME_FOR_ALL_TYPES(TFCC_RUNTIME_CREATE)
#undef TFCC_RUNTIME_CREATE
      case BOOL: create<uint8_t>(s, constants, scope); break;
      default: throw RuntimeError("Invalid data type " + std::to_string(static_cast<int>(s.dtype)));
    }
  }
}

const SymbolInfo& SymbolManager::getSymbolInfo(const std::string& name) const {
  auto it = _map.find(name);
  if (it == _map.end()) throw RuntimeError("Symbol name: " + name + " not found");
  return it->second;
}

template <class T>
SymbolSlot<T>& SymbolManager::slot(const std::string& name, const SymbolInfo*& info) {
  info = &getSymbolInfo(name);
  return slots<T>(info->dtype)[info->pos];
}

template <class T>
const Tensor<T>* SymbolManager::getTensor(const std::string& name, T) {
  const SymbolInfo* info;
  SymbolSlot<T>& s = slot<T>(name, info);
  switch (info->stype) {
    case SymbolType::VARIABLE: return &s.variable;
    case SymbolType::VIEW: return &s.view;
    case SymbolType::CONSTANT_TENSOR: return s.constant;
    default: throw RuntimeError("Symbol name: " + name + " is not a tensor");
  }
}

template <class T>
Variable<T>* SymbolManager::getVariable(const std::string& name, T) {
  const SymbolInfo* info;
  SymbolSlot<T>& s = slot<T>(name, info);
  if (info->stype != SymbolType::VARIABLE) throw RuntimeError("Symbol name: " + name + " is not a variable");
  return &s.variable;
}

template <class T>
View<T>* SymbolManager::getView(const std::string& name, T) {
  const SymbolInfo* info;
  SymbolSlot<T>& s = slot<T>(name, info);
  if (info->stype != SymbolType::VIEW) throw RuntimeError("Symbol name: " + name + " is not a view");
  return &s.view;
}

template <class T>
void SymbolManager::setView(const std::string& name, Variable<T>&& v) {
  const SymbolInfo* info;
  SymbolSlot<T>& s = slot<T>(name, info);
  if (info->stype != SymbolType::VIEW) throw RuntimeError("Symbol name: " + name + " is not a view");
  s.variable = std::move(v);
  s.view = View<T>(s.variable);
}

template <class T>
T* SymbolManager::getValue(const std::string& name, T) {
  const SymbolInfo* info;
  SymbolSlot<T>& s = slot<T>(name, info);
  if (!is_value(info->stype)) throw RuntimeError("Symbol name: " + name + " is not a value");
  return &s.value;
}

template <class T>
std::vector<T>* SymbolManager::getVector(const std::string& name, T) {
  const SymbolInfo* info;
  SymbolSlot<T>& s = slot<T>(name, info);
  if (!is_vector(info->stype)) throw RuntimeError("Symbol name: " + name + " is not a vector");
  return &s.vector;
}

// ---------------------------------------------------------------------------------------------------
// graph
// ---------------------------------------------------------------------------------------------------
thread_local bool Graph::_recordDetailError = false;
thread_local bool Graph::_fusion = true;

namespace {
void rocm_check(int status) {
  if (status != TFCC_ROCM_OK) throw ROCMRuntimeError(status, tfcc_rocm_last_error_string());
}
void* session_stream() {
  auto* s = dynamic_cast<ROCMSession*>(Session::getThreadDefault());
  if (s == nullptr) throw RuntimeError("replay needs a ROCm session as the thread default");
  return s->getStream();
}
}  // namespace

Graph::Graph(Model& model, const proto::Graph& graphProto, ConstantStore& constants)
    : _model(model), _proto(graphProto), _symbols(new SymbolManager(graphProto.symbols, constants, graphProto.name)) {}

Graph::~Graph() {
  try {
    enableReplay(false);
  } catch (...) {
  }
}

void Graph::buildGraph() {
  if (_built) return;
  _steps.clear();
  std::vector<FusionPlan> fusion(_proto.nodes.size());
  if (_fusion && dynamic_cast<ROCMDevice*>(Device::getThreadDefault()) != nullptr) fusion = plan_fusions(_proto, *_symbols);
  for (size_t i = 0; i < _proto.nodes.size(); ++i) {
    const proto::Node& node = _proto.nodes[i];
    _currentNode = i;
    if (fusion[i].kind == FusionPlan::ABSORBED) continue;
    if (fusion[i].kind != FusionPlan::NONE) {
      emit_fused(_proto, fusion[i], i, *this);
      continue;
    }
    bool accepted = false;
    for (auto& op : operations_for(node.typeUrl)) {
      if (!op->getOperationVersions().count(node.version)) continue;
      const size_t before = _steps.size();
      if (op->process(node, *this)) {
        accepted = true;
        break;
      }
      _steps.resize(before);
    }
    if (!accepted) throw UnknowNodeError(node);
  }
  _built = true;
}

std::string Graph::errorString(const std::string& what, size_t node) {
  if (!_recordDetailError) return what;
  std::string reason = what + "\nerror at node " + std::to_string(node) + "\nnode proto:\n" +
                       _proto.nodes[node].debugString() + "\n====================\nnode inputs:\n";
  for (const std::string& name : _proto.nodes[node].inputs) {
    reason += "name: " + name;
    if (_symbols->has(name)) {
      const SymbolInfo& info = _symbols->getSymbolInfo(name);
      reason += std::string(" dtype: ") + data_type_name(info.dtype);
      if (is_tensor(info.stype) && info.dtype == FLOAT) {
        try {
          const Tensor<float>* t = _symbols->getTensor(name, float());
          reason += " real shape: [";
          for (size_t d = 0; t && d < t->shape().size(); ++d) reason += (d ? "," : "") + std::to_string(t->shape(d));
          reason += "]";
        } catch (std::exception& e) {
          reason += std::string(" get symbol debug error: ") + e.what();
        }
      }
    }
    reason += "\n--------------------\n";
  }
  return reason;
}

void Graph::runSteps() {
  for (const Step& step : _steps) {
    try {
      step.run();
    } catch (std::exception& e) {
      throw RuntimeError(errorString(e.what(), step.node));
    }
  }
}

void Graph::process() {
  if (!_built) buildGraph();
  if (_captured) {
    rocm_check(tfcc_rocm_graph_launch(_graphExec, session_stream()));
    return;
  }
  const bool record = _replayWanted && _warm && !_captureFailed;
  if (!record) {
    runSteps();
    _warm = true;
    return;
  }
  Session* session = Session::getThreadDefault();
  auto* rocmSession = dynamic_cast<ROCMSession*>(session);
  void* stream = session_stream();
  session->getAllocator().beginPinning();
  try {
    rocm_check(tfcc_rocm_stream_begin_capture(stream));
  } catch (...) {
    session->getAllocator().unpin(session->getAllocator().endPinning());
    throw;
  }
  // From here to the end of the recording the session refuses what a recording cannot hold (waiting for the
  // stream, copies to and from host memory) before the stream sees it: such a step throws, the recording
  // stays valid and is ended and dropped below.
  rocmSession->setRecording(true);
  bool stepFailed = false;
  try {
    runSteps();
  } catch (std::exception&) {
    stepFailed = true;  // a step that reads results on the host, or a real error: the step-by-step run below tells
  }
  rocmSession->setRecording(false);
  void* exec = nullptr;
  const int status = tfcc_rocm_stream_end_capture(stream, &exec);
  std::vector<void*> pinned = session->getAllocator().endPinning();
  if (status == TFCC_ROCM_OK && !stepFailed) {
    _graphExec = exec;
    _pinned = std::move(pinned);
    _replaySession = session;
    _captured = true;
    // the recording only described the work; run it once so this call produces its outputs
    rocm_check(tfcc_rocm_graph_launch(_graphExec, stream));
    return;
  }
  // Not recordable.  Nothing has run yet (the steps before the failure were only recorded), so this call still
  // owes its outputs: give the blocks back, remember not to try again, and run step by step.  An error that is
  // not about recording shows up again there and is reported as usual.
  if (exec) tfcc_rocm_graph_destroy(exec);
  session->getAllocator().unpin(pinned);
  _captureFailed = true;
  runSteps();
}

void Graph::enableReplay(bool enable) {
  _replayWanted = enable;
  if (!enable) {
    if (_graphExec) {
      // the stream the recording runs on and the allocator its blocks came from belong to the session it was made
      // on, whichever thread or session asks for the release
      if (_replaySession) _replaySession->sync();
      rocm_check(tfcc_rocm_graph_destroy(_graphExec));
      if (_replaySession) _replaySession->getAllocator().unpin(_pinned);
    }
    _graphExec = nullptr;
    _replaySession = nullptr;
    _pinned.clear();
    _captured = false;
    _captureFailed = false;
    _warm = false;
  }
}

template <class T>
void Graph::setInput(const std::string& name, const Tensor<T>& tensor) {
  if (_replayWanted) {
    // a recording reads its inputs from fixed buffers: copy instead of re-pointing the view
    View<T>* view = _symbols->getView(name, T());
    if (_captured && !(view->shape() == tensor.shape())) enableReplayReset();
    if (!(view->shape() == tensor.shape()) || view->size() == 0 || !_inputOwned.count(name)) {
      _symbols->setView(name, data::copy(tensor));
      _inputOwned.insert(name);
      return;
    }
    rocm_check(tfcc_rocm_memcpy_d2d_async(session_stream(), const_cast<T*>(view->data()), tensor.data(),
                                          static_cast<size_t>(tensor.size()) * sizeof(T)));
    return;
  }
  View<T>* inp = _symbols->getView(name, T());
  *inp = View<T>(tensor);
}

template <class T>
void Graph::setInput(const std::string& name, Variable<T>&& variable) {
  if (_replayWanted && _inputOwned.count(name)) {
    const Variable<T>& keep = variable;
    setInput(name, static_cast<const Tensor<T>&>(keep));
    return;  // `variable` returns to the cache when the caller's object dies; the copy is stream-ordered
  }
  _symbols->setView(name, std::move(variable));
  if (_replayWanted) _inputOwned.insert(name);
}

template <class T>
typename std::enable_if<std::is_arithmetic<T>::value, void>::type Graph::setInput(const std::string& name, T value) {
  if (_captured) enableReplayReset();  // a value input is baked into the recorded launches
  *_symbols->getValue(name, T()) = value;
}

void Graph::enableReplayReset() {
  const bool wanted = _replayWanted;
  enableReplay(false);
  _replayWanted = wanted;
}

// ---------------------------------------------------------------------------------------------------
// model
// ---------------------------------------------------------------------------------------------------
Model::Model(const std::string& data) {
  auto members = unzip(data);
  if (!members.count("model.pb")) throw RuntimeError("Invalid model data");
  if (!members.count("model.npz")) throw RuntimeError("Invalid model data");
  if (members.count("userdata")) _userData = std::move(members["userdata"]);
  try {
    _proto = proto::parse_model(members["model.pb"]);
  } catch (wire::ParseError& e) {
    throw RuntimeError(std::string("Invalid model proto: ") + e.what());
  }
  // entrance graph first, the rest by name (model.cpp:84-101)
  const std::string entrance = _proto.entranceGraphName;
  std::stable_sort(_proto.graphs.begin(), _proto.graphs.end(), [&](const proto::Graph& a, const proto::Graph& b) {
    const bool ea = a.name == entrance, eb = b.name == entrance;
    if (ea != eb) return ea;
    return a.name < b.name;
  });
  if (_proto.graphs.empty() || _proto.graphs[0].name != entrance) throw RuntimeError("Invalid model proto");
  _npz.reset(new NpzData(members["model.npz"]));
}

Model::~Model() {
  _alive.reset();
  // graphs hold Variables of their sessions: drop them before the constants
  _sessions.clear();
  _constants.clear();
}

Model::PerSession& Model::initializeGraphs(Session* session) {
  if (session == nullptr) throw RuntimeError("no default session on this thread: call an initialize function first");
  std::unique_lock<std::mutex> lk(_mutex);
  auto it = _sessions.find(session);
  if (it != _sessions.end()) return it->second;
  Device* device = &session->getDevice();
  auto& store = _constants[device];
  if (!store) store.reset(new ConstantStore(*_npz, device));
  ConstantStore& constants = *store;
  lk.unlock();
  // built aside and entered only when every graph stands: a constructor that throws (a constant that is missing,
  // a dtype nobody knows) must not leave an entry with no graphs behind for the next call to index
  PerSession fresh;
  for (const proto::Graph& g : _proto.graphs) fresh.graphs.emplace_back(new Graph(*this, g, constants));
  for (auto& g : fresh.graphs) g->buildGraph();
  std::weak_ptr<bool> alive = _alive;
  session->registerReleaseCallback([this, alive](const Session* s) {
    if (!alive.expired()) releaseGraphs(s);
  });
  lk.lock();
  return _sessions.emplace(session, std::move(fresh)).first->second;
}

void Model::releaseGraphs(const Session* session) {
  std::lock_guard<std::mutex> lk(_mutex);
  _sessions.erase(session);
}

Graph& Model::getEntranceGraph() { return *initializeGraphs(Session::getThreadDefault()).graphs[0]; }

Graph& Model::getGraph(const std::string& name) {
  for (auto& g : initializeGraphs(Session::getThreadDefault()).graphs)
    if (g->getGraphName() == name) return *g;
  throw RuntimeError("Graph name: " + name + " not found");
}

namespace {
template <class T>
void add_input(Graph& graph, const proto::DataItem& item) {
  Shape shape(item.shape);
  if (item.data.size() != static_cast<size_t>(shape.area()) * sizeof(T)) throw RuntimeError("Invalid data size");
  const SymbolInfo& info = graph.getSymbolManager().getSymbolInfo(item.name);
  if (is_value(info.stype)) {
    T v;
    if (item.data.size() < sizeof(T)) throw RuntimeError("Invalid data size");
    std::memcpy(&v, item.data.data(), sizeof(T));
    graph.setInput(item.name, v);
    return;
  }
  Variable<T> v(shape);
  if (v.size() > 0)
    data::set(v, reinterpret_cast<const T*>(item.data.data()));
  graph.setInput(item.name, std::move(v));
}

template <class T>
void get_output(Graph& graph, const std::string& name, proto::DataItem& out) {
  const SymbolInfo& info = graph.getSymbolManager().getSymbolInfo(name);
  out.name = name;
  out.dtype = info.dtype;
  if (is_value(info.stype)) {
    T v = graph.getValue(name, T());
    out.shape = {1};
    out.data.assign(reinterpret_cast<const char*>(&v), sizeof(T));
    return;
  }
  const Tensor<T>& tensor = graph.getTensor(name, T());
  out.shape = tensor.shape().toVector();
  std::vector<T> v = data::get(tensor);
  out.data.assign(reinterpret_cast<const char*>(v.data()), v.size() * sizeof(T));
}
}  // namespace

void Model::run(const std::vector<proto::DataItem>& inputs, std::vector<proto::DataItem>& outputs) {
  Graph& graph = getEntranceGraph();
  for (const proto::DataItem& item : inputs) {
    switch (item.dtype) {
#define TFCC_RUNTIME_INPUT(T, E) \
  case E: add_input<T>(graph, item); break;
      TFCC_RUNTIME_FOR_ALL_TYPES(TFCC_RUNTIME_INPUT)
#undef TFCC_RUNTIME_INPUT
      case BOOL: add_input<uint8_t>(graph, item); break;
      default: throw RuntimeError("Invalid input dtype");
    }
  }
  graph.process();
  for (const std::string& name : graph.getOutputs()) {
    outputs.emplace_back();
    switch (graph.getSymbolManager().getSymbolInfo(name).dtype) {
#define TFCC_RUNTIME_OUTPUT(T, E) \
  case E: get_output<T>(graph, name, outputs.back()); break;
      TFCC_RUNTIME_FOR_ALL_TYPES(TFCC_RUNTIME_OUTPUT)
#undef TFCC_RUNTIME_OUTPUT
      case BOOL: get_output<uint8_t>(graph, name, outputs.back()); break;
      default: throw RuntimeError("Invalid output type");
    }
  }
}

void Model::run(const std::string& inputs, std::string& outputs) {
  std::vector<proto::DataItem> in, out;
  try {
    in = proto::parse_inputs(inputs);
  } catch (wire::ParseError& e) {
    throw RuntimeError(std::string("Invalid inputs: ") + e.what());
  }
  run(in, out);
  outputs = proto::serialize_outputs(out);
}

namespace {
// tfcc::is_similar (tfcc/core/utils/tfcc_debugutils.cpp:102-129)
template <class T>
bool values_similar(const std::vector<T>& a, const std::vector<T>& b) {
  if (a.size() != b.size()) return false;
  for (size_t i = 0; i < a.size(); ++i) {
    const double x = static_cast<double>(a[i]), y = static_cast<double>(b[i]);
    if (std::isnan(x) || std::isnan(y)) return false;
    if (!(std::fabs(x - y) < 1e-3 * std::fabs(x + y) || std::fabs(x - y) < 1e-5)) return false;
  }
  return true;
}

template <class T>
void test_input(Graph& graph, const std::string& name, const NpzData& npz) {
  const SymbolInfo& info = graph.getSymbolManager().getSymbolInfo(name);
  const NpyArray& a = npz.get(name);
  std::vector<T> values = convert_elements<T>(a);
  if (is_value(info.stype)) {
    if (values.empty()) throw RuntimeError("Invalid input data");
    graph.setInput(name, values[0]);
  } else if (info.stype == SymbolType::VIEW) {
    graph.setInput(name, data::set(std::move(values), Shape(a.shape)));
  } else {
    throw RuntimeError("Invalid input stype");
  }
}

template <class T>
bool test_output(Graph& graph, const std::string& name, const NpzData& npz, std::ostream& stream) {
  const SymbolInfo& info = graph.getSymbolManager().getSymbolInfo(name);
  std::vector<T> got;
  std::vector<unsigned> shape{1};
  if (is_tensor(info.stype)) {
    const Tensor<T>& t = graph.getTensor(name, T());
    got = data::get(t);
    shape = t.shape().toVector();
  } else if (is_value(info.stype)) {
    got.push_back(graph.getValue(name, T()));
  } else {
    throw RuntimeError("Invalid output stype");
  }
  bool ok = true;
  if (npz.has(name)) {
    const NpyArray& a = npz.get(name);
    ok = values_similar(got, convert_elements<T>(a)) && (!is_tensor(info.stype) || a.shape == shape);
  } else {
    stream << "WARNING output [" << name << "] not in test data" << std::endl;
    ok = false;
  }
  stream << name << ": shape [";
  for (size_t d = 0; d < shape.size(); ++d) stream << (d ? "," : "") << shape[d];
  stream << "] " << (ok ? "similar" : "DIFFERENT") << std::endl;
  return ok;
}
}  // namespace

bool Model::test(const std::string& npzBytes, std::ostream& stream) {
  NpzData npz(npzBytes);
  Graph& graph = getEntranceGraph();
  auto t0 = std::chrono::steady_clock::now();
  for (const std::string& name : graph.getInputs()) {
    switch (graph.getSymbolManager().getSymbolInfo(name).dtype) {
#define TFCC_RUNTIME_TEST_INPUT(T, E) \
  case E: test_input<T>(graph, name, npz); break;
      TFCC_RUNTIME_FOR_ALL_TYPES(TFCC_RUNTIME_TEST_INPUT)
#undef TFCC_RUNTIME_TEST_INPUT
      case BOOL: test_input<uint8_t>(graph, name, npz); break;
      default: throw RuntimeError("Invalid input dtype");
    }
  }
  auto t1 = std::chrono::steady_clock::now();
  stream << "set inputs cost: " << std::chrono::duration<double, std::milli>(t1 - t0).count() << " ms" << std::endl;
  graph.process();
  Session::getThreadDefault()->sync();
  auto t2 = std::chrono::steady_clock::now();
  stream << "process cost: " << std::chrono::duration<double, std::milli>(t2 - t1).count() << " ms" << std::endl;
  bool ok = true;
  for (const std::string& name : graph.getOutputs()) {
    switch (graph.getSymbolManager().getSymbolInfo(name).dtype) {
#define TFCC_RUNTIME_TEST_OUTPUT(T, E) \
  case E: ok = test_output<T>(graph, name, npz, stream) && ok; break;
      TFCC_RUNTIME_FOR_ALL_TYPES(TFCC_RUNTIME_TEST_OUTPUT)
#undef TFCC_RUNTIME_TEST_OUTPUT
      case BOOL: ok = test_output<uint8_t>(graph, name, npz, stream) && ok; break;
      default: throw RuntimeError("Invalid output dtype");
    }
  }
  return ok;
}

// ---- explicit instantiations ----------------------------------------------------------------------------
#define TFCC_RUNTIME_INSTANTIATE(T, E)                                                       \
  template class ConstantTensor<T>;                                                          \
  template const Tensor<T>& ConstantStore::getConstant<T>(const std::string&);               \
  template T ConstantStore::getConfigure<T>(const std::string&);                             \
  template std::vector<T> ConstantStore::getVector<T>(const std::string&);                   \
  template const Tensor<T>* SymbolManager::getTensor<T>(const std::string&, T);              \
  template Variable<T>* SymbolManager::getVariable<T>(const std::string&, T);                \
  template View<T>* SymbolManager::getView<T>(const std::string&, T);                        \
  template void SymbolManager::setView<T>(const std::string&, Variable<T>&&);                \
  template T* SymbolManager::getValue<T>(const std::string&, T);                             \
  template std::vector<T>* SymbolManager::getVector<T>(const std::string&, T);               \
  template void Graph::setInput<T>(const std::string&, const Tensor<T>&);                    \
  template void Graph::setInput<T>(const std::string&, Variable<T>&&);                       \
  template void Graph::setInput<T>(const std::string&, T);
TFCC_RUNTIME_FOR_ALL_TYPES(TFCC_RUNTIME_INSTANTIATE)
#undef TFCC_RUNTIME_INSTANTIATE

}  // namespace runtime
}  // namespace tfcc
