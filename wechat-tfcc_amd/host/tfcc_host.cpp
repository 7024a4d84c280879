// Implementation of the host-side framework (allocators, device / session bookkeeping) and of the
// ROCm device: every GPU action goes through the C ABI of libtfcc_rocm.so.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <type_traits>

#include "tfcc_rocm.h"
#include "tfcc_layers.h"
#include "tfcc_rocm_device.h"

namespace tfcc {

// ---------------------------------------------------------------------------------------------
// framework
// ---------------------------------------------------------------------------------------------
thread_local Device* Device::_threadDevice = nullptr;
thread_local Session* Session::_threadSession = nullptr;

Device::Device(DeviceType type, unsigned index, std::unique_ptr<Allocator> allocator)
    : _deviceID((static_cast<unsigned>(type) << 24) | (index & 0x00ffffffu)),
      _allocator(std::move(allocator)),
      _interfaces(new InterfaceSet()) {}

Device::~Device() {
  if (_threadDevice == this) _threadDevice = nullptr;
}

std::shared_ptr<void> Device::getConstantSlot(const void* scope, const std::string& name, int typeKey,
                                              const std::function<std::shared_ptr<void>()>& make) {
  std::lock_guard<std::mutex> lck(_constantMutex);
  std::shared_ptr<void>& slot = _constants[std::make_tuple(scope, name, typeKey)];
  if (!slot) slot = make();
  return slot;
}

void Device::removeConstants(const void* scope) {
  std::lock_guard<std::mutex> lck(_constantMutex);
  for (auto it = _constants.begin(); it != _constants.end();)
    it = std::get<0>(it->first) == scope ? _constants.erase(it) : std::next(it);
}

// ---- scopes and data loaders (tfcc/core/framework/tfcc_scope.cpp, tfcc/core/dataloaders/) ---------------------
Scope Scope::_root(nullptr, "");
thread_local Scope* Scope::_currentScope = &Scope::_root;

ScopeGuard::~ScopeGuard() {
  if (_valid) Scope::popScope();
}

Scope& Scope::getChild(const std::string& name) {
  std::lock_guard<std::mutex> lck(_mtx);
  auto it = _children.find(name);
  if (it != _children.end()) return *it->second;
  Scope* p = new Scope(this, name);
  _children[name] = std::unique_ptr<Scope>(p);
  return *p;
}

std::string Scope::getFullName() const { return _parent == nullptr ? "" : _parent->getFullName() + _name + "/"; }

void Scope::pushScope(const std::string& name) { _currentScope = &_currentScope->getChild(name); }
void Scope::popScope() { _currentScope = _currentScope->_parent ? _currentScope->_parent : &_root; }
ScopeGuard Scope::scope(const std::string& name) {
  pushScope(name);
  return ScopeGuard();
}

DataLoader* DataLoader::_defaultDataLoader = nullptr;
DataLoader* DataLoader::getGlobalDefault() { return _defaultDataLoader; }
void DataLoader::setGlobalDefault(DataLoader* loader) { _defaultDataLoader = loader; }

void NPZDataLoader::fill(const std::map<std::string, std::string>& members) {
  for (const auto& kv : members) {
    if (kv.first.size() < 4 || kv.first.substr(kv.first.size() - 4) != ".npy") continue;
    try {  // members that are not arrays are skipped (tfcc/core/dataloaders/tfcc_npzdataloader.cpp:27-42)
      runtime::NpyArray a = runtime::parse_npy(kv.second);
      _dataMap[kv.first.substr(0, kv.first.size() - 4)] = std::make_tuple(Shape(a.shape), a.type, std::move(a.body));
    } catch (const std::exception&) {
    }
  }
}

NPZDataLoader::NPZDataLoader(const std::string& path) { fill(runtime::unzip_from_path(path)); }
NPZDataLoader::NPZDataLoader(const char* data, size_t dataLen) { fill(runtime::unzip(std::string(data, dataLen))); }

const std::tuple<Shape, std::string, std::string>& NPZDataLoader::loadData(const std::string& name) const {
  auto it = _dataMap.find(name);
  if (it == _dataMap.end()) throw RuntimeError("Name: [" + name + "] not found in data loader");
  return it->second;
}

std::vector<std::tuple<std::string, std::string>> NPZDataLoader::getAllNames() const {
  std::vector<std::tuple<std::string, std::string>> result;
  for (const auto& kv : _dataMap) result.emplace_back(kv.first, std::get<1>(kv.second));
  return result;
}

bool NPZDataLoader::hasData(const std::string& name) const { return _dataMap.count(name) != 0; }

void Session::preRelease() {
  for (auto& cb : _releaseCallbacks) cb(this);
  _releaseCallbacks.clear();
  if (_threadSession == this) _threadSession = nullptr;
}

namespace detail {

void check_same_area(const Shape& from, const Shape& to) {
  if (from.area() != to.area()) throw InvalidArgumentError("shape area couldn't be changed");
}

Shape expand_dims(const Shape& s, size_t axis) {
  if (axis > s.size()) throw InvalidArgumentError("invalid axis to expand");
  std::vector<unsigned> dims = s.toVector();
  dims.insert(dims.begin() + static_cast<std::ptrdiff_t>(axis), 1u);
  return Shape(std::move(dims));
}

Shape squeeze_all(const Shape& s) {
  std::vector<unsigned> dims;
  for (unsigned d : s.toVector())
    if (d != 1) dims.push_back(d);
  Shape r(std::move(dims));
  check_same_area(s, r);
  return r;
}

Shape squeeze_axes(const Shape& s, const std::set<size_t>& axes) {
  if (!axes.empty() && *axes.rbegin() >= s.size()) throw InvalidArgumentError("invalid axis to squeeze");
  std::vector<unsigned> dims;
  for (size_t i = 0; i < s.size(); ++i) {
    if (axes.count(i)) {
      if (s[i] != 1) throw InvalidArgumentError("invalid axis to squeeze");
    } else {
      dims.push_back(s[i]);
    }
  }
  return Shape(std::move(dims));
}

}  // namespace detail

// ---- FlexAllocator -------------------------------------------------------------------------------

size_t FlexAllocator::bucket(size_t len) {
  len += 64;  // header room, part of the accounting the reference's test pins
  const size_t grain = len < (size_t(4) << 20) ? size_t(4096) : (size_t(1) << 20);
  return (len + grain - 1) / grain * grain;
}

FlexAllocator::~FlexAllocator() {
  // blocks still handed out at this point are a bug of the owner; the cache is returned, and with it what a
  // recording left reserved or freed while pinning (its owner may be gone without having given them back)
  {
    std::lock_guard<std::mutex> lk(_mtx);
    for (auto& kv : _reserved) _cached.emplace(kv.second, kv.first);
    for (auto& kv : _pinnedFree) _cached.emplace(kv.first, kv.second);
    _reserved.clear();
    _pinnedFree.clear();
  }
  releaseDownTo(0);
}

void* FlexAllocator::malloc(size_t len) {
  if (len == 0) return nullptr;
  const size_t size = bucket(len);
  void* p = nullptr;
  {
    std::lock_guard<std::mutex> lk(_mtx);
    auto pinned = _pinning ? _pinnedFree.find(size) : _pinnedFree.end();
    if (pinned != _pinnedFree.end()) {
      p = pinned->second;
      _pinnedFree.erase(pinned);
      _live[p] = size;
      return p;
    }
    auto it = _cached.find(size);
    if (it != _cached.end()) {
      p = it->second;
      _cached.erase(it);
    }
  }
  if (p == nullptr) {
    if (_limit == 0 || _used.load() + size <= _limit) p = _realMalloc(size);
    if (p == nullptr) {
      // over the limit, or the device is out of memory: give the cache back and try once more
      releaseDownTo(0);
      if (_limit == 0 || _used.load() + size <= _limit) p = _realMalloc(size);
    }
    if (p == nullptr) return nullptr;
    _used += size;
  }
  {
    std::lock_guard<std::mutex> lk(_mtx);
    _live[p] = size;
  }
  if (_flexLimit != 0 && _used.load() > _flexLimit) releaseDownTo(_flexLimit / 2);
  return p;
}

void FlexAllocator::free(void* p) {
  if (p == nullptr) return;
  std::lock_guard<std::mutex> lk(_mtx);
  auto it = _live.find(p);
  if (it == _live.end()) return;
  (_pinning ? _pinnedFree : _cached).emplace(it->second, p);
  _live.erase(it);
}

void FlexAllocator::beginPinning() {
  std::lock_guard<std::mutex> lk(_mtx);
  _pinning = true;
}

std::vector<void*> FlexAllocator::endPinning() {
  std::lock_guard<std::mutex> lk(_mtx);
  _pinning = false;
  std::vector<void*> blocks;
  for (auto& kv : _pinnedFree) {
    _reserved[kv.second] = kv.first;
    blocks.push_back(kv.second);
  }
  _pinnedFree.clear();
  return blocks;
}

void FlexAllocator::unpin(const std::vector<void*>& blocks) {
  std::lock_guard<std::mutex> lk(_mtx);
  for (void* p : blocks) {
    auto it = _reserved.find(p);
    if (it == _reserved.end()) continue;
    _cached.emplace(it->second, p);
    _reserved.erase(it);
  }
}

void FlexAllocator::releaseDownTo(size_t target) {
  while (_used.load() > target) {
    void* p = nullptr;
    size_t size = 0;
    {
      std::lock_guard<std::mutex> lk(_mtx);
      if (_cached.empty()) return;
      auto it = _cached.begin();  // smallest bucket first
      size = it->first;
      p = it->second;
      _cached.erase(it);
    }
    _realFree(p);
    _used -= size;
  }
}

void* SimpleAllocator::malloc(size_t len) {
  if (len == 0) return nullptr;
  if (_limit != 0 && _used.load() + len > _limit) return nullptr;
  void* p = _realMalloc(len);
  if (p == nullptr) return nullptr;
  std::lock_guard<std::mutex> lk(_mtx);
  _live[p] = len;
  _used += len;
  return p;
}

void SimpleAllocator::free(void* p) {
  if (p == nullptr) return;
  {
    std::lock_guard<std::mutex> lk(_mtx);
    auto it = _live.find(p);
    if (it == _live.end()) return;
    _used -= it->second;
    _live.erase(it);
  }
  _realFree(p);
}

// ---------------------------------------------------------------------------------------------
// host device
// ---------------------------------------------------------------------------------------------
namespace {
// plain memory moves: the only interface the host device offers
template <class T>
class HostDataInterface : public DataInterface<T> {
 public:
  void set(T* dst, const T* data, size_t len) override { std::memcpy(dst, data, len * sizeof(T)); }
  void set(Variable<T>& a, const T* data) override { set(a.data(), data, a.size()); }
  void set(Variable<T>& a, std::vector<T>&& data) override { set(a.data(), data.data(), a.size()); }
  void get(const Tensor<T>& a, T* data) override { std::memcpy(data, a.data(), static_cast<size_t>(a.size()) * sizeof(T)); }
  void zeros(Variable<T>& a) override { std::fill(a.data(), a.data() + a.size(), static_cast<T>(0)); }
  void ones(Variable<T>& a) override { std::fill(a.data(), a.data() + a.size(), static_cast<T>(1)); }
  Variable<T> copy(const Tensor<T>& a) override {
    Variable<T> r(a.shape());
    std::memcpy(r.data(), a.data(), static_cast<size_t>(a.size()) * sizeof(T));
    return r;
  }
};
template <class T>
void install_host(Interface<T>& i) {
  i.setDataInterface(std::unique_ptr<DataInterface<T>>(new HostDataInterface<T>()));
}
}  // namespace

HostDevice::HostDevice() : Device(DeviceType::HOST, 0, std::unique_ptr<Allocator>(new FlexAllocator())) {
  _allocator->setRealMalloc([](size_t len) -> void* { return std::aligned_alloc(64, (len + 63) / 64 * 64); });
  _allocator->setRealFree([](void* p) { std::free(p); });
  install_host(_interfaces->f32);
  install_host(_interfaces->f64);
  install_host(_interfaces->s8);
  install_host(_interfaces->u8);
  install_host(_interfaces->s16);
  install_host(_interfaces->u16);
  install_host(_interfaces->s32);
  install_host(_interfaces->u32);
  install_host(_interfaces->s64);
  install_host(_interfaces->u64);
}

void initialize_host() {
  static HostDevice device;
  thread_local std::unique_ptr<HostSession> session;
  if (!session) session.reset(new HostSession(device));
  Device::setThreadDefault(&device);
  Session::setThreadDefault(session.get());
}

HostSession::HostSession(HostDevice& device) : Session(std::unique_ptr<Allocator>(new FlexAllocator())), _device(device) {
  _allocator->setRealMalloc([this](size_t len) { return _device.malloc(len); });
  _allocator->setRealFree([this](void* p) { _device.free(p); });
}

HostSession::~HostSession() {
  preRelease();
  _allocator->releaseCache();
}

// ---------------------------------------------------------------------------------------------
// ROCm device
// ---------------------------------------------------------------------------------------------
namespace {

inline void check(int status) {
  if (status != TFCC_ROCM_OK) throw ROCMRuntimeError(status, tfcc_rocm_last_error_string());
}

inline void* current_stream() {
  auto* s = dynamic_cast<ROCMSession*>(Session::getThreadDefault());
  if (s == nullptr) throw RuntimeError("the thread's default session is not a ROCm session");
  return s->getStream();
}

// the stream for an operation the host waits on (copies to and from host memory)
inline void* current_stream_for_host_transfer(const char* what) {
  auto* s = dynamic_cast<ROCMSession*>(Session::getThreadDefault());
  if (s == nullptr) throw RuntimeError("the thread's default session is not a ROCm session");
  if (s->recording()) throw RuntimeError(std::string(what) + ": not possible while the session's stream records a graph");
  return s->getStream();
}

template <class T>
constexpr int type_code();
template <> constexpr int type_code<int8_t>() { return TFCC_ROCM_S8; }
template <> constexpr int type_code<uint8_t>() { return TFCC_ROCM_U8; }
template <> constexpr int type_code<int16_t>() { return TFCC_ROCM_S16; }
template <> constexpr int type_code<uint16_t>() { return TFCC_ROCM_U16; }
template <> constexpr int type_code<int32_t>() { return TFCC_ROCM_S32; }
template <> constexpr int type_code<uint32_t>() { return TFCC_ROCM_U32; }

inline void require_scalar(const Tensor<float>& t, const char* what) {
  if (t.size() != 1 || t.shape().size() != 1) throw InvalidArgumentError(what);
}

// ---- data ------------------------------------------------------------------------------------
template <class T>
class ROCMDataInterface : public DataInterface<T> {
 public:
  void set(T* dst, const T* data, size_t len) override {
    check(tfcc_rocm_memcpy_h2d(current_stream_for_host_transfer("data::set"), dst, data, len * sizeof(T)));
  }
  void set(Variable<T>& a, const T* data) override { set(a.data(), data, a.size()); }
  void set(Variable<T>& a, std::vector<T>&& data) override { set(a.data(), data.data(), a.size()); }
  void get(const Tensor<T>& a, T* data) override {
    check(tfcc_rocm_memcpy_d2h(current_stream_for_host_transfer("data::get"), data, a.data(),
                               static_cast<size_t>(a.size()) * sizeof(T)));
  }
  void zeros(Variable<T>& a) override {
    check(tfcc_rocm_fill_async(current_stream(), a.data(), 0, sizeof(T), a.size()));
  }
  void ones(Variable<T>& a) override {
    T one = static_cast<T>(1);
    uint64_t bits = 0;
    std::memcpy(&bits, &one, sizeof(T));
    check(tfcc_rocm_fill_async(current_stream(), a.data(), bits, sizeof(T), a.size()));
  }
  void fill(Variable<T>& a, T value) override {
    uint64_t bits = 0;
    std::memcpy(&bits, &value, sizeof(T));
    check(tfcc_rocm_fill_async(current_stream(), a.data(), bits, sizeof(T), a.size()));
  }
  // the ten conversions of the reference's interface over the one conversion kernel
  template <class SRC>
  Variable<T> castFrom(const Tensor<SRC>& a) {
    Variable<T> result(a.shape());
    if (a.size() > 0)
      check(tfcc_rocm_cast(current_stream(), a.data(), ElementCode<SRC>::value, result.data(), ElementCode<T>::value, result.size()));
    return result;
  }
  Variable<T> cast(const Tensor<float>& a) override { return castFrom(a); }
  Variable<T> cast(const Tensor<double>& a) override { return castFrom(a); }
  Variable<T> cast(const Tensor<int8_t>& a) override { return castFrom(a); }
  Variable<T> cast(const Tensor<uint8_t>& a) override { return castFrom(a); }
  Variable<T> cast(const Tensor<int16_t>& a) override { return castFrom(a); }
  Variable<T> cast(const Tensor<uint16_t>& a) override { return castFrom(a); }
  Variable<T> cast(const Tensor<int32_t>& a) override { return castFrom(a); }
  Variable<T> cast(const Tensor<uint32_t>& a) override { return castFrom(a); }
  Variable<T> cast(const Tensor<int64_t>& a) override { return castFrom(a); }
  Variable<T> cast(const Tensor<uint64_t>& a) override { return castFrom(a); }
  // b[i] = a[i] ? 1 : 0 (tfcc/mkl/interfaces/tfcc_mkldatainterface.cpp:87-93): the comparison against zero
  Variable<uint8_t> cast_to_boolean(const Tensor<T>& a) override {
    Variable<uint8_t> result(a.shape());
    const T zero = static_cast<T>(0);
    if (a.size() > 0)
      check(tfcc_rocm_compare_value(current_stream(), TFCC_ROCM_COMPARE_UNEQUAL, a.data(), ElementCode<T>::value, a.size(), &zero,
                                    result.data()));
    return result;
  }
  Variable<T> copy(const Tensor<T>& a) override {
    Variable<T> r(a.shape());
    check(tfcc_rocm_memcpy_d2d_async(current_stream(), r.data(), a.data(), static_cast<size_t>(a.size()) * sizeof(T)));
    return r;
  }
};

// ---- blas --------------------------------------------------------------------------------------
// Stride rules of the reference's blas interface (tfcc/mkl/interfaces/tfcc_mklblasinterface.cpp:127-186):
// a rank-2 operand against a batched one is shared by the whole batch (stride 0).
// shared by the interface and by the fused forms of tfcc::rocm::blas
Variable<float> rocm_sgemm(const Tensor<float>& a, const Tensor<float>& b, const Tensor<float>* bias,
                           const Tensor<float>* residual, int activation) {
  const size_t ra = a.shape().size(), rb = b.shape().size();
  const unsigned m = a.shape(ra - 2), n = b.shape(rb - 1), k = a.shape(ra - 1);
  uint64_t strideA = static_cast<uint64_t>(m) * k, strideB = static_cast<uint64_t>(n) * k;
  if (ra != rb) {
    if (ra == 2) strideA = 0;
    if (rb == 2) strideB = 0;
  }
  std::vector<unsigned> s = tfcc::blas::detail::check<float>(a, b, bias);
  Variable<float> result{Shape(s)};
  if (residual && !(residual->shape() == result.shape())) throw InvalidArgumentError("residual and result don't match");
  bool broadcast = false;
  if (ra == rb)
    for (size_t i = 0; i + 2 < ra; ++i) broadcast = broadcast || a.shape(i) != b.shape(i);
  if (broadcast) {
    // leading dimensions of extent 1 on one side: per-dimension strides (0 where broadcast), adjacent
    // dimensions merged where the strides allow, at most two left for the kernel's outer x inner batch grid
    std::vector<unsigned> dims;
    std::vector<uint64_t> sa, sb, sc;
    uint64_t da = static_cast<uint64_t>(m) * k, db = static_cast<uint64_t>(k) * n, dc = static_cast<uint64_t>(m) * n;
    for (size_t i = ra - 2; i-- > 0;) {  // innermost leading dimension first
      const unsigned ea = a.shape(i), eb = b.shape(i), e = s[i];
      if (e > 1) {
        dims.insert(dims.begin(), e);
        sa.insert(sa.begin(), ea == 1 ? 0 : da);
        sb.insert(sb.begin(), eb == 1 ? 0 : db);
        sc.insert(sc.begin(), dc);
      }
      da *= ea; db *= eb; dc *= e;
    }
    for (size_t i = 0; i + 1 < dims.size();) {
      if (sa[i] == sa[i + 1] * dims[i + 1] && sb[i] == sb[i + 1] * dims[i + 1] && sc[i] == sc[i + 1] * dims[i + 1]) {
        dims[i + 1] *= dims[i];
        dims.erase(dims.begin() + i); sa.erase(sa.begin() + i); sb.erase(sb.begin() + i); sc.erase(sc.begin() + i);
        if (i > 0) --i;
      } else {
        ++i;
      }
    }
    if (dims.size() > 2) throw NotImplementedError("matmul: broadcast over more than two groups of batch dimensions");
    tfcc_rocm_sgemm_desc d{};
    d.a = a.data(); d.b = b.data(); d.c = result.data();
    d.bias = bias ? bias->data() : nullptr;
    d.residual = residual ? residual->data() : nullptr;
    d.stride_residual = static_cast<uint64_t>(m) * n;
    d.m = m; d.n = n; d.k = k; d.lda = k; d.ldb = n; d.ldc = n;
    d.activation = activation;
    d.batch_outer = 1; d.batch_inner = 1;
    if (dims.size() == 2) {
      d.batch_outer = dims[0]; d.stride_a = sa[0]; d.stride_b = sb[0]; d.stride_c = sc[0];
      d.batch_inner = dims[1]; d.inner_stride_a = sa[1]; d.inner_stride_b = sb[1]; d.inner_stride_c = sc[1];
    } else if (dims.size() == 1) {
      d.batch_outer = dims[0]; d.stride_a = sa[0]; d.stride_b = sb[0]; d.stride_c = sc[0];
    }
    check(tfcc_rocm_sgemm_general(current_stream(), &d));
    return result;
  }
  unsigned rows = m, batch = result.size() / (m * n);
  if (rb == 2 && ra > 2) {
    // one matrix b for the whole batch of a: the batch is just more rows of one product
    rows = m * batch;
    batch = 1;
  }
  check(tfcc_rocm_sgemm_fused(current_stream(), a.data(), strideA, b.data(), strideB, bias ? bias->data() : nullptr,
                              residual ? residual->data() : nullptr, static_cast<uint64_t>(rows) * n, result.data(),
                              static_cast<uint64_t>(rows) * n, rows, n, k, batch, activation));
  return result;
}

class ROCMBlasInterface : public BlasInterface<float> {
 public:
  Variable<float> matmul(const Tensor<float>& a, const Tensor<float>& b) override {
    return rocm_sgemm(a, b, nullptr, nullptr, 0);
  }
  Variable<float> matmul(const Tensor<float>& a, const Tensor<float>& b, const Tensor<float>& bias) override {
    return rocm_sgemm(a, b, &bias, nullptr, 0);
  }
};

// ---- quantization --------------------------------------------------------------------------------
template <class T>
class ROCMQuantizationInterface : public QuantizationInterface<T> {
  template <class TI>
  static Variable<T> requantizeImpl(const Tensor<TI>& a, const Tensor<float>& minInput, const Tensor<float>& maxInput,
                                    const Tensor<float>& minOutput, const Tensor<float>& maxOutput) {
    if (a.size() == 0) throw InvalidArgumentError("invalid tensor");
    require_scalar(minInput, "invalid minInput");
    require_scalar(maxInput, "invalid maxInput");
    require_scalar(minOutput, "invalid minOutput");
    require_scalar(maxOutput, "invalid maxOutput");
    Variable<T> result(a.shape());
    check(tfcc_rocm_requantize(current_stream(), a.data(), type_code<TI>(), result.data(), type_code<T>(), a.size(),
                               minInput.data(), maxInput.data(), minOutput.data(), maxOutput.data()));
    return result;
  }

 public:
  std::tuple<Variable<T>, Variable<float>, Variable<float>> quantize(const Tensor<float>& a) override {
    if (a.size() == 0) throw InvalidArgumentError("invalid tensor");
    Variable<T> result(a.shape());
    Variable<float> minValue({1}), maxValue({1});
    check(tfcc_rocm_quantize_minmax(current_stream(), a.data(), a.size(), result.data(), type_code<T>(),
                                    minValue.data(), maxValue.data()));
    return std::make_tuple(std::move(result), std::move(minValue), std::move(maxValue));
  }
  Variable<T> quantize(const Tensor<float>& a, const Tensor<float>& minValue, const Tensor<float>& maxValue) override {
    if (a.size() == 0) throw InvalidArgumentError("invalid tensor");
    require_scalar(minValue, "invalid minValue");
    require_scalar(maxValue, "invalid maxValue");
    Variable<T> result(a.shape());
    check(tfcc_rocm_quantize(current_stream(), a.data(), a.size(), minValue.data(), maxValue.data(), result.data(),
                             type_code<T>()));
    return result;
  }
#define TFCC_ROCM_REQUANTIZE(TI)                                                                                \
  Variable<T> requantize(const Tensor<TI>& a, const Tensor<float>& minInput, const Tensor<float>& maxInput,      \
                         const Tensor<float>& minOutput, const Tensor<float>& maxOutput) override {             \
    return requantizeImpl<TI>(a, minInput, maxInput, minOutput, maxOutput);                                     \
  }
  TFCC_ROCM_REQUANTIZE(int8_t)
  TFCC_ROCM_REQUANTIZE(uint8_t)
  TFCC_ROCM_REQUANTIZE(int16_t)
  TFCC_ROCM_REQUANTIZE(uint16_t)
  TFCC_ROCM_REQUANTIZE(int32_t)
  TFCC_ROCM_REQUANTIZE(uint32_t)
#undef TFCC_ROCM_REQUANTIZE
  Variable<float> dequantize(const Tensor<T>& a, const Tensor<float>& minValue, const Tensor<float>& maxValue) override {
    if (a.size() == 0) throw InvalidArgumentError("invalid tensor");
    require_scalar(minValue, "invalid minValue");
    require_scalar(maxValue, "invalid maxValue");
    Variable<float> result(a.shape());
    check(tfcc_rocm_dequantize(current_stream(), a.data(), type_code<T>(), a.size(), minValue.data(), maxValue.data(),
                               result.data()));
    return result;
  }
};

// ---- the element-wise neighbours (float only) ----------------------------------------------------------
class ROCMActivationInterface : public ActivationInterface<float> {
 public:
  Variable<float> softmax(const Tensor<float>& a, size_t axis) override {
    if (a.size() == 0) throw InvalidArgumentError("invalid tensor");
    if (axis + 1 != a.shape().size()) throw NotImplementedError("softmax over the last axis only");
    Variable<float> r(a.shape());
    const unsigned cols = a.shape(axis);
    check(tfcc_rocm_softmax_f32(current_stream(), a.data(), a.size() / cols, cols, r.data()));
    return r;
  }
  Variable<float> geluAccurate(const Tensor<float>& a) override {
    Variable<float> r(a.shape());
    check(tfcc_rocm_gelu_accurate_f32(current_stream(), a.data(), a.size(), r.data()));
    return r;
  }
  Variable<float> unary(const Tensor<float>& a, int function) override {
    Variable<float> r(a.shape());
    check(tfcc_rocm_unary_f32(current_stream(), function, a.data(), a.size(), r.data()));
    return r;
  }
  Variable<float> leakyRelu(const Tensor<float>& a, float alpha) override {
    Variable<float> r(a.shape());
    check(tfcc_rocm_leaky_relu_f32(current_stream(), a.data(), a.size(), alpha, r.data()));
    return r;
  }
  Variable<float> pow(const Tensor<float>& a, float exponent) override;
  Variable<float> pow(const Tensor<float>& a, const Tensor<float>& exponent) override;
  Variable<float> pow(float a, const Tensor<float>& exponent) override;
};

// Checks and error texts of tfcc/mkl/interfaces/tfcc_mklcellinterface.cpp:33-165.
class ROCMCellInterface : public CellInterface<float> {
  static void check_lstm(const Tensor<float>& stateC, const Tensor<float>& inputValue, const Tensor<float>& stateHValue,
                         const Tensor<float>& bias) {
    if (stateC.shape().size() != 2) throw InvalidArgumentError("invalid stateC");
    const unsigned batch = stateC.shape(0), units = stateC.shape(1);
    if (inputValue.shape().size() != 2 || inputValue.shape(0) != batch || inputValue.shape(1) != units * 4)
      throw InvalidArgumentError("invalid inputValue");
    if (stateHValue.shape().size() != 2 || stateHValue.shape(0) != batch || stateHValue.shape(1) != units * 4)
      throw InvalidArgumentError("invalid stateHValue");
    if (bias.shape().size() != 1 || bias.shape(0) != units * 4) throw InvalidArgumentError("invalid bias");
  }

 public:
  std::tuple<Variable<float>, Variable<float>> processLSTMCell(const Tensor<float>& stateC,
                                                               const Tensor<float>& inputValue,
                                                               const Tensor<float>& stateHValue,
                                                               const Tensor<float>& bias, float forget) override {
    check_lstm(stateC, inputValue, stateHValue, bias);
    Variable<float> h(stateC.shape()), cs(stateC.shape());
    check(tfcc_rocm_lstm_cell_f32(current_stream(), stateC.shape(0), stateC.shape(1), stateC.data(), inputValue.data(),
                                  stateHValue.data(), bias.data(), forget, h.data(), cs.data()));
    return std::make_tuple(std::move(h), std::move(cs));
  }
  void processLSTMCellInto(const Tensor<float>& stateC, const Tensor<float>& inputValue,
                           const Tensor<float>& stateHValue, const Tensor<float>& bias, float forget, float* h,
                           float* cs) override {
    check_lstm(stateC, inputValue, stateHValue, bias);
    check(tfcc_rocm_lstm_cell_f32(current_stream(), stateC.shape(0), stateC.shape(1), stateC.data(), inputValue.data(),
                                  stateHValue.data(), bias.data(), forget, h, cs));
  }
  // [units, 4 units] -> gates interleaved, [units, units, 4]: column 4 u + g is gate g of unit u
  Variable<float> prepareLSTMStateKernel(const Tensor<float>& stateKernel, unsigned batch) override {
    if (batch < 1 || batch > 8) throw NotImplementedError("one-launch LSTM step: 1 to 8 rows");
    if (stateKernel.shape().size() != 2 || stateKernel.shape(1) != stateKernel.shape(0) * 4 || stateKernel.size() == 0)
      throw InvalidArgumentError("invalid state kernel");
    const unsigned units = stateKernel.shape(0);
    Variable<float> r({units, units * 4});
    const unsigned shape[3] = {units, 4, units}, perm[3] = {0, 2, 1};
    check(tfcc_rocm_transpose_f32(current_stream(), stateKernel.data(), shape, perm, 3, r.data()));
    return r;
  }
  void processLSTMStepInto(const Tensor<float>& stateC, const Tensor<float>& inputValue, const Tensor<float>& h,
                           const Tensor<float>& preparedStateKernel, const Tensor<float>& bias, float forget, float* hOut,
                           float* csOut) override {
    if (stateC.shape().size() != 2) throw InvalidArgumentError("invalid stateC");
    const unsigned batch = stateC.shape(0), units = stateC.shape(1);
    if (inputValue.shape().size() != 2 || inputValue.shape(0) != batch || inputValue.shape(1) != units * 4)
      throw InvalidArgumentError("invalid inputValue");
    if (h.shape() != stateC.shape()) throw InvalidArgumentError("invalid h");
    if (preparedStateKernel.shape().size() != 2 || preparedStateKernel.shape(0) != units ||
        preparedStateKernel.shape(1) != units * 4)
      throw InvalidArgumentError("invalid state kernel");
    if (bias.shape().size() != 1 || bias.shape(0) != units * 4) throw InvalidArgumentError("invalid bias");
    check(tfcc_rocm_lstm_step_f32(current_stream(), batch, units, h.data(), preparedStateKernel.data(), inputValue.data(),
                                  bias.data(), forget, stateC.data(), hOut, csOut));
  }
  Variable<float> processGRUCellGates(const Tensor<float>& state, const Tensor<float>& inputs,
                                      const Tensor<float>& value, const Tensor<float>& bias) override {
    if (state.shape().size() != 2) throw InvalidArgumentError("invalid state");
    const unsigned batch = state.shape(0), units = state.shape(1);
    if (inputs.shape().size() != 2 || inputs.shape(0) != batch) throw InvalidArgumentError("invalid inputs");
    if (value.shape().size() != 2 || value.shape(0) != batch || value.shape(1) != units * 2)
      throw InvalidArgumentError("invalid value");
    if (bias.shape().size() != 1 || bias.shape(0) != units * 2) throw InvalidArgumentError("invalid bias");
    Variable<float> r({batch, inputs.shape(1) + units});
    check(tfcc_rocm_gru_cell_gates_f32(current_stream(), batch, units, inputs.shape(1), state.data(), inputs.data(),
                                       value.data(), bias.data(), r.data()));
    return r;
  }
  Variable<float> processGRUCellCandidate(const Tensor<float>& state, const Tensor<float>& value,
                                          const Tensor<float>& bias, const Tensor<float>& cValue,
                                          const Tensor<float>& cBias) override {
    if (state.shape().size() != 2) throw InvalidArgumentError("invalid state");
    const unsigned batch = state.shape(0), units = state.shape(1);
    if (value.shape().size() != 2 || value.shape(0) != batch || value.shape(1) != units * 2)
      throw InvalidArgumentError("invalid value");
    if (bias.shape().size() != 1 || bias.shape(0) != units * 2) throw InvalidArgumentError("invalid bias");
    if (cValue.shape().size() != 2 || cValue.shape(0) != batch || cValue.shape(1) != units)
      throw InvalidArgumentError("invalid cValue");
    if (cBias.shape().size() != 1 || cBias.shape(0) != units) throw InvalidArgumentError("invalid cBias");
    Variable<float> r(state.shape());
    check(tfcc_rocm_gru_cell_candidate_f32(current_stream(), batch, units, state.data(), value.data(), bias.data(),
                                           cValue.data(), cBias.data(), r.data()));
    return r;
  }
  Variable<float> processPyTorchGRUCell(const Tensor<float>& state, const Tensor<float>& inputValue,
                                        const Tensor<float>& stateValue, const Tensor<float>& gateBias,
                                        const Tensor<float>& candidateIBias,
                                        const Tensor<float>& candidateHBias) override {
    if (state.shape().size() != 2) throw InvalidArgumentError("invalid state");
    const unsigned batch = state.shape(0), units = state.shape(1);
    if (inputValue.shape().size() != 2 || inputValue.shape(0) != batch || inputValue.shape(1) != units * 3)
      throw InvalidArgumentError("invalid inputValue");
    if (stateValue.shape().size() != 2 || stateValue.shape(0) != batch || stateValue.shape(1) != units * 3)
      throw InvalidArgumentError("invalid stateValue");
    if (gateBias.shape().size() != 1 || gateBias.shape(0) != units * 2) throw InvalidArgumentError("invalid gateBias");
    if (candidateIBias.shape().size() != 1 || candidateIBias.shape(0) != units)
      throw InvalidArgumentError("invalid candidateIBias");
    if (candidateHBias.shape().size() != 1 || candidateHBias.shape(0) != units)
      throw InvalidArgumentError("invalid candidateHBias");
    Variable<float> r(state.shape());
    check(tfcc_rocm_pytorch_gru_cell_f32(current_stream(), batch, units, state.data(), inputValue.data(),
                                         stateValue.data(), gateBias.data(), candidateIBias.data(),
                                         candidateHBias.data(), r.data()));
    return r;
  }
};

class ROCMNormalizationInterface : public NormalizationInterface<float> {
 public:
  Variable<float> layerNormalize(const Tensor<float>& a, const Tensor<float>& gamma, const Tensor<float>& beta,
                                 float epsilon, size_t beginNormAxis) override {
    if (beginNormAxis >= a.shape().size()) throw InvalidArgumentError("invalid beginNormAxis");
    unsigned cols = 1;
    for (size_t i = beginNormAxis; i < a.shape().size(); ++i) cols *= a.shape(i);
    if (gamma.size() != cols || beta.size() != cols) throw InvalidArgumentError("gamma, beta and the normalized dims don't match");
    if (a.size() == 0) throw InvalidArgumentError("invalid tensor");
    Variable<float> r(a.shape());
    check(tfcc_rocm_layer_norm_f32(current_stream(), a.data(), gamma.data(), beta.data(), epsilon, a.size() / cols, cols,
                                   r.data()));
    return r;
  }
};

// slice, concat and gather move bytes and exist for every element type; transpose is the float kernel.
template <class T>
class ROCMBasicInterface : public BasicInterface<T> {
  static void split_at(const Shape& shape, size_t axis, uint64_t& s1, uint64_t& s3) {
    s1 = s3 = 1;
    for (size_t i = 0; i < axis; ++i) s1 *= shape[i];
    for (size_t i = axis + 1; i < shape.size(); ++i) s3 *= shape[i];
  }

 public:
  Variable<T> transpose(const Tensor<T>& a, const std::vector<size_t>& perm) override {
    if constexpr (std::is_same<T, float>::value) {
      if (a.size() == 0) throw InvalidArgumentError("invalid tensor");
      std::vector<unsigned> shape = a.shape().toVector(), p(perm.begin(), perm.end()), out(perm.size());
      for (size_t i = 0; i < perm.size(); ++i) out[i] = shape[perm[i]];
      Variable<float> r{Shape(std::move(out))};
      check(tfcc_rocm_transpose_f32(current_stream(), a.data(), shape.data(), p.data(), static_cast<int>(p.size()), r.data()));
      return r;
    } else {
      throw NotImplementedError("transpose: float only");
    }
  }
  Variable<T> slice(const Tensor<T>& a, size_t axis, unsigned start, unsigned end) override {
    end = std::min(end, a.shape(axis));  // tfcc/mkl/interfaces/tfcc_mklbasicinterface.cpp:490
    std::vector<unsigned> shape = a.shape().toVector();
    shape[axis] = end - start;
    Variable<T> r{Shape(shape)};
    if (r.size() == 0) return r;
    uint64_t s1, s3;
    split_at(a.shape(), axis, s1, s3);
    const uint64_t row = static_cast<uint64_t>(end - start) * s3 * sizeof(T);
    check(tfcc_rocm_copy2d(current_stream(), a.data() + static_cast<size_t>(start) * s3, a.shape(axis) * s3 * sizeof(T),
                           r.data(), row, s1, row));
    return r;
  }
  Variable<T> concat(const std::vector<const Tensor<T>*>& values, size_t axis) override {
    std::vector<unsigned> shape = values[0]->shape().toVector();
    shape[axis] = 0;
    for (const Tensor<T>* v : values) shape[axis] += v->shape(axis);
    Variable<T> r{Shape(shape)};
    if (r.size() == 0) return r;
    uint64_t s1, s3;
    split_at(r.shape(), axis, s1, s3);
    const uint64_t pitch = static_cast<uint64_t>(shape[axis]) * s3 * sizeof(T);
    size_t offset = 0;  // elements into a row of the result
    for (const Tensor<T>* v : values) {
      const uint64_t width = static_cast<uint64_t>(v->shape(axis)) * s3 * sizeof(T);
      if (width != 0) check(tfcc_rocm_copy2d(current_stream(), v->data(), width, r.data() + offset, pitch, s1, width));
      offset += static_cast<size_t>(v->shape(axis)) * s3;
    }
    return r;
  }
  // tfcc/mkl/interfaces/tfcc_mklbasicinterface.cpp:518-537: one strided copy
  void assignTo(const Tensor<T>& a, size_t axis, unsigned start, Variable<T>& b) override {
    if (a.size() == 0) return;
    uint64_t s1, s3;
    split_at(a.shape(), axis, s1, s3);
    const uint64_t width = static_cast<uint64_t>(a.shape(axis)) * s3 * sizeof(T);
    check(tfcc_rocm_copy2d(current_stream(), a.data(), width, b.data() + static_cast<size_t>(start) * s3,
                           static_cast<uint64_t>(b.shape(axis)) * s3 * sizeof(T), s1, width));
  }
  Variable<T> clip(const Tensor<T>& a, T minValue, T maxValue) override {
    if constexpr (std::is_same<T, float>::value) {
      Variable<T> r(a.shape());
      check(tfcc_rocm_clip_f32(current_stream(), a.data(), a.size(), minValue, maxValue, r.data()));
      return r;
    } else {
      throw NotImplementedError("clip: float tensors only");
    }
  }
  Variable<T> where(const Tensor<uint8_t>& condition, const Tensor<T>* x, T xValue, const Tensor<T>* y, T yValue) override {
    Variable<T> r(condition.shape());
    if (r.size() == 0) return r;
    uint64_t xBits = 0, yBits = 0;
    std::memcpy(&xBits, &xValue, sizeof(T));
    std::memcpy(&yBits, &yValue, sizeof(T));
    check(tfcc_rocm_where(current_stream(), condition.data(), x ? x->data() : nullptr, xBits, y ? y->data() : nullptr, yBits,
                          sizeof(T), r.size(), r.data()));
    return r;
  }
  Variable<T> triangle(const Tensor<T>& a, int64_t k, bool upper) override {
    if (a.size() == 0) throw InvalidArgumentError("invalid tensor");
    Variable<T> r(a.shape());
    check(tfcc_rocm_triangle(current_stream(), a.data(), a.shape(0), a.shape(1), k, upper ? 1 : 0, sizeof(T), r.data()));
    return r;
  }
  std::tuple<Variable<T>, Variable<uint32_t>> topK(const Tensor<T>& a, unsigned k) override {
    if constexpr (std::is_same<T, float>::value) {
      if (k == 0) throw InvalidArgumentError("invalid k");
      std::vector<unsigned> shape = a.shape().toVector();
      const unsigned length = shape.back();
      shape.back() = k;
      Variable<T> values{Shape(shape)};
      Variable<uint32_t> positions{Shape(shape)};
      check(tfcc_rocm_topk_f32(current_stream(), a.data(), a.size() / length, length, k, values.data(), positions.data()));
      return std::make_tuple(std::move(values), std::move(positions));
    } else {
      throw NotImplementedError("top_k: float tensors only");
    }
  }
  Variable<int64_t> argmax(const Tensor<T>& a, size_t axis) override {
    if constexpr (std::is_same<T, float>::value) {
      std::vector<unsigned> shape = a.shape().toVector();
      uint64_t s1, s3;
      split_at(a.shape(), axis, s1, s3);
      const unsigned length = shape[axis];
      shape[axis] = 1;
      Variable<int64_t> r{Shape(shape)};
      check(tfcc_rocm_argmax_f32(current_stream(), a.data(), s1, length, s3, r.data()));
      return r;
    } else {
      throw NotImplementedError("argmax: float tensors only");
    }
  }
  Variable<T> gather(const Tensor<T>& params, const void* indices, int indexCode, const Shape& indexShape) override {
    std::vector<unsigned> shape = indexShape.toVector();
    for (size_t i = 1; i < params.shape().size(); ++i) shape.push_back(params.shape(i));
    Variable<T> r{Shape(shape)};
    const uint64_t chunk = static_cast<uint64_t>(params.size() / params.shape(0)) * sizeof(T);
    check(tfcc_rocm_gather_rows(current_stream(), params.data(), params.shape(0), chunk, indices, indexCode, indexShape.area(),
                                r.data()));
    return r;
  }
};

// a and b arrive with equal rank, every dimension equal or 1 on one side (tfcc::math merges the rest away).
Variable<float> broadcast_binary_run(int op, const Tensor<float>& a, const Tensor<float>& b) {
    const size_t rank = a.shape().size();
    if (rank == 0 || rank != b.shape().size()) throw InvalidArgumentError("invalid tensor shape");
    std::vector<unsigned> dims(rank);
    for (size_t d = 0; d < rank; ++d) {
      if (a.shape(d) != b.shape(d) && a.shape(d) != 1 && b.shape(d) != 1) throw InvalidArgumentError("broadcast failed");
      dims[d] = std::max(a.shape(d), b.shape(d));
    }
    Variable<float> r{Shape(dims)};
    if (r.size() == 0) return r;
    // b repeats along the leading dimensions of a only: the one-pass kernel with a period
    bool periodic = a.size() == r.size();
    for (size_t d = 0, seenFull = 0; periodic && d < rank; ++d) {
      if (b.shape(d) == dims[d] && dims[d] != 1) seenFull = 1;
      else if (seenFull && dims[d] != 1) periodic = false;  // b broadcasts again after one of its own dimensions
    }
    if (periodic) {
      check(tfcc_rocm_binary_f32(current_stream(), op, a.data(), b.data(), a.size(), b.size(), r.data()));
      return r;
    }
    if (rank > 6) throw NotImplementedError("element-wise operation: more than six groups of broadcast dimensions");
    uint64_t sa[6], sb[6], accA = 1, accB = 1;
    for (size_t d = rank; d-- > 0;) {
      sa[d] = a.shape(d) == 1 && dims[d] != 1 ? 0 : accA;
      sb[d] = b.shape(d) == 1 && dims[d] != 1 ? 0 : accB;
      accA *= a.shape(d);
      accB *= b.shape(d);
    }
    check(tfcc_rocm_binary_broadcast_f32(current_stream(), op, a.data(), b.data(), static_cast<int>(rank), dims.data(), sa,
                                         sb, r.data()));
    return r;
}

class ROCMArithmeticInterface : public ArithmeticInterface<float> {
 public:
  Variable<float> add(const Tensor<float>& a, const Tensor<float>& b) override { return broadcast_binary_run(0, a, b); }
  Variable<float> sub(const Tensor<float>& a, const Tensor<float>& b) override { return broadcast_binary_run(1, a, b); }
  Variable<float> mul(const Tensor<float>& a, const Tensor<float>& b) override { return broadcast_binary_run(2, a, b); }
  Variable<float> div(const Tensor<float>& a, const Tensor<float>& b) override { return broadcast_binary_run(3, a, b); }
};

// a one-element tensor of the rank of `like` holding `value`
Variable<float> scalar_like(const Tensor<float>& like, float value) {
  Variable<float> v{Shape(std::vector<unsigned>(like.shape().size(), 1u))};
  uint64_t bits = 0;
  std::memcpy(&bits, &value, sizeof(float));
  check(tfcc_rocm_fill_async(current_stream(), v.data(), bits, sizeof(float), 1));
  return v;
}

class ROCMMinMaxInterface : public MinMaxInterface<float> {
 public:
  Variable<float> min(const Tensor<float>& a, const Tensor<float>& b) override { return broadcast_binary_run(6, a, b); }
  Variable<float> max(const Tensor<float>& a, const Tensor<float>& b) override { return broadcast_binary_run(5, a, b); }
  Variable<float> min(const Tensor<float>& a, float b) override {
    Variable<float> r(a.shape());
    check(tfcc_rocm_clip_f32(current_stream(), a.data(), a.size(), -std::numeric_limits<float>::infinity(), b, r.data()));
    return r;
  }
  Variable<float> max(const Tensor<float>& a, float b) override {
    Variable<float> r(a.shape());
    check(tfcc_rocm_clip_f32(current_stream(), a.data(), a.size(), b, std::numeric_limits<float>::infinity(), r.data()));
    return r;
  }
};

class ROCMReduceInterface : public ReduceInterface<float> {
  static Variable<float> run(int op, const Tensor<float>& a, size_t keep) {
    std::vector<unsigned> s = a.shape().toVector();
    size_t cols = 1;
    for (size_t d = keep; d < s.size(); ++d) {
      cols *= s[d];
      s[d] = 1;
    }
    Variable<float> r{Shape(s)};
    check(tfcc_rocm_reduce_f32(current_stream(), op, a.data(), a.size() / cols, cols, r.data()));
    return r;
  }

 public:
  Variable<float> reduceSum(const Tensor<float>& a, size_t keep) override { return run(TFCC_ROCM_REDUCE_SUM, a, keep); }
  Variable<float> reduceMean(const Tensor<float>& a, size_t keep) override { return run(TFCC_ROCM_REDUCE_MEAN, a, keep); }
  Variable<float> reduceProd(const Tensor<float>& a, size_t keep) override { return run(TFCC_ROCM_REDUCE_PROD, a, keep); }
  Variable<float> reduceMax(const Tensor<float>& a, size_t keep) override { return run(TFCC_ROCM_REDUCE_MAX, a, keep); }
  Variable<float> reduceMin(const Tensor<float>& a, size_t keep) override { return run(TFCC_ROCM_REDUCE_MIN, a, keep); }
};

Variable<float> ROCMActivationInterface::pow(const Tensor<float>& a, float exponent) {
  Variable<float> e = scalar_like(a, exponent);
  return broadcast_binary_run(4, a, e);
}
Variable<float> ROCMActivationInterface::pow(const Tensor<float>& a, const Tensor<float>& exponent) {
  return broadcast_binary_run(4, a, exponent);
}
Variable<float> ROCMActivationInterface::pow(float a, const Tensor<float>& exponent) {
  Variable<float> base = scalar_like(exponent, a);
  return broadcast_binary_run(4, base, exponent);
}

class ROCMTransformationInterface : public TransformationInterface<float> {
 public:
  Variable<float> transform(const Tensor<float>& a, float alpha, float beta) override {
    if (a.size() == 0) throw InvalidArgumentError("invalid tensor");
    Variable<float> r(a.shape());
    check(tfcc_rocm_transform_f32(current_stream(), a.data(), a.size(), alpha, beta, r.data()));
    return r;
  }
  Variable<float> transform2(const Tensor<float>& a, float alpha, float beta) override {
    if (a.size() == 0) throw InvalidArgumentError("invalid tensor");
    Variable<float> r(a.shape());
    check(tfcc_rocm_transform2_f32(current_stream(), a.data(), a.size(), alpha, beta, r.data()));
    return r;
  }
};

template <class T>
class ROCMComparisonInterface : public ComparisonInterface<T> {
 public:
  Variable<uint8_t> compare(const Tensor<T>& a, T b, Relation r) override {
    Variable<uint8_t> result(a.shape());
    check(tfcc_rocm_compare_value(current_stream(), static_cast<int>(r), a.data(), ElementCode<T>::value, a.size(), &b,
                                  result.data()));
    return result;
  }
  Variable<uint8_t> compareDifference(const Tensor<T>& a, const Tensor<T>& b, Relation r) override {
    const size_t rank = a.shape().size();
    if (rank == 0 || rank != b.shape().size()) throw InvalidArgumentError("invalid tensor shape");
    if (rank > 6) throw NotImplementedError("comparison: more than six groups of broadcast dimensions");
    std::vector<unsigned> dims(rank);
    for (size_t d = 0; d < rank; ++d) {
      if (a.shape(d) != b.shape(d) && a.shape(d) != 1 && b.shape(d) != 1) throw InvalidArgumentError("broadcast failed");
      dims[d] = std::max(a.shape(d), b.shape(d));
    }
    Variable<uint8_t> result{Shape(dims)};
    uint64_t sa[6], sb[6], accA = 1, accB = 1;
    for (size_t d = rank; d-- > 0;) {
      sa[d] = a.shape(d) == 1 && dims[d] != 1 ? 0 : accA;
      sb[d] = b.shape(d) == 1 && dims[d] != 1 ? 0 : accB;
      accA *= a.shape(d);
      accB *= b.shape(d);
    }
    check(tfcc_rocm_compare(current_stream(), static_cast<int>(r), a.data(), b.data(), ElementCode<T>::value,
                            static_cast<int>(rank), dims.data(), sa, sb, result.data()));
    return result;
  }
};

template <class T>
void install_common(Interface<T>& i) {
  i.setComparisonInterface(std::unique_ptr<ComparisonInterface<T>>(new ROCMComparisonInterface<T>()));
  i.setDataInterface(std::unique_ptr<DataInterface<T>>(new ROCMDataInterface<T>()));
  i.setBasicInterface(std::unique_ptr<BasicInterface<T>>(new ROCMBasicInterface<T>()));
}
template <class T>
void install_quantization(Interface<T>& i) {
  i.setQuantizationInterface(std::unique_ptr<QuantizationInterface<T>>(new ROCMQuantizationInterface<T>()));
}

}  // namespace

unsigned ROCMDevice::getDeviceCount() {
  int n = 0;
  if (tfcc_rocm_device_count(&n) != TFCC_ROCM_OK) return 0;
  return n > 0 ? static_cast<unsigned>(n) : 0u;
}

ROCMDevice::ROCMDevice(unsigned index) : ROCMDevice(index, std::unique_ptr<Allocator>(new FlexAllocator())) {
  // leave a tenth of the card to the runtime, like the reference's GPU device
  size_t freeBytes = 0, totalBytes = 0;
  check(tfcc_rocm_set_device(static_cast<int>(_index)));
  check(tfcc_rocm_mem_info(&freeBytes, &totalBytes));
  _allocator->setLimit(totalBytes / 10 * 9);
}

ROCMDevice::ROCMDevice(unsigned index, std::unique_ptr<Allocator> allocator)
    : Device(DeviceType::ROCM, index, std::move(allocator)), _index(index) {
  check(tfcc_rocm_set_device(static_cast<int>(_index)));
  const int idx = static_cast<int>(_index);
  _allocator->setRealMalloc([idx](size_t len) -> void* {
    void* p = nullptr;
    if (tfcc_rocm_set_device(idx) != TFCC_ROCM_OK) return nullptr;
    if (tfcc_rocm_malloc(&p, len) != TFCC_ROCM_OK) return nullptr;
    return p;
  });
  _allocator->setRealFree([](void* p) { tfcc_rocm_free(p); });

  install_common(_interfaces->f32);
  install_common(_interfaces->f64);
  install_common(_interfaces->s8);
  install_common(_interfaces->u8);
  install_common(_interfaces->s16);
  install_common(_interfaces->u16);
  install_common(_interfaces->s32);
  install_common(_interfaces->u32);
  install_common(_interfaces->s64);
  install_common(_interfaces->u64);
  // quantization for the six quantized element types (tfcc/mkl/interfaces/tfcc_mklinterface.cpp:45-50)
  install_quantization(_interfaces->s8);
  install_quantization(_interfaces->u8);
  install_quantization(_interfaces->s16);
  install_quantization(_interfaces->u16);
  install_quantization(_interfaces->s32);
  install_quantization(_interfaces->u32);
  // matmul is float only, like the reference's MKL device; other types keep the throwing default
  _interfaces->f32.setBlasInterface(std::unique_ptr<BlasInterface<float>>(new ROCMBlasInterface()));
  _interfaces->f32.setActivationInterface(std::unique_ptr<ActivationInterface<float>>(new ROCMActivationInterface()));
  _interfaces->f32.setNormalizationInterface(std::unique_ptr<NormalizationInterface<float>>(new ROCMNormalizationInterface()));
  _interfaces->f32.setArithmeticInterface(std::unique_ptr<ArithmeticInterface<float>>(new ROCMArithmeticInterface()));
  _interfaces->f32.setMinMaxInterface(std::unique_ptr<MinMaxInterface<float>>(new ROCMMinMaxInterface()));
  _interfaces->f32.setReduceInterface(std::unique_ptr<ReduceInterface<float>>(new ROCMReduceInterface()));
  _interfaces->f32.setCellInterface(std::unique_ptr<CellInterface<float>>(new ROCMCellInterface()));
  _interfaces->f32.setTransformationInterface(std::unique_ptr<TransformationInterface<float>>(new ROCMTransformationInterface()));
}

ROCMDevice::~ROCMDevice() { _allocator->releaseCache(); }

void ROCMDevice::attach() { check(tfcc_rocm_set_device(static_cast<int>(_index))); }

ROCMSession::ROCMSession(ROCMDevice& device) : ROCMSession(device, std::unique_ptr<Allocator>(new FlexAllocator())) {}

ROCMSession::ROCMSession(ROCMDevice& device, std::unique_ptr<Allocator> allocator)
    : Session(std::move(allocator)), _device(device), _stream(nullptr) {
  device.attach();
  check(tfcc_rocm_stream_create(&_stream));
  // session memory comes from the device allocator; a block only really goes back after the stream
  // has drained, because kernels still queued may be using it
  _allocator->setRealMalloc([this](size_t len) { return _device.malloc(len); });
  _allocator->setRealFree([this](void* p) {
    this->sync();
    _device.free(p);
  });
}

ROCMSession::~ROCMSession() {
  preRelease();
  tfcc_rocm_stream_synchronize(_stream);
  _allocator->releaseCache();
  tfcc_rocm_stream_destroy(_stream);
}

void ROCMSession::sync() const {
  if (_recording) throw RuntimeError("Session::sync: not possible while the session's stream records a graph");
  check(tfcc_rocm_stream_synchronize(_stream));
}

namespace {

struct RocmRuntime {
  std::mutex mtx;
  std::vector<std::unique_ptr<ROCMDevice>> devices;
};

RocmRuntime& runtime() {
  static RocmRuntime r;
  return r;
}

struct ThreadBinding {
  std::unique_ptr<ROCMSession> session;
  ~ThreadBinding() {
    if (session && Session::getThreadDefault() == session.get()) Session::setThreadDefault(nullptr);
  }
};

void bind_thread(unsigned deviceID) {
  thread_local ThreadBinding binding;
  if (Device::getThreadDefault() != nullptr && Session::getThreadDefault() != nullptr) {
    Device::getThreadDefault()->attach();
    return;
  }
  RocmRuntime& r = runtime();
  ROCMDevice* device = nullptr;
  {
    std::lock_guard<std::mutex> lk(r.mtx);
    if (r.devices.empty()) {
      unsigned n = ROCMDevice::getDeviceCount();
      if (n == 0) throw RuntimeError("no ROCm device available");
      for (unsigned i = 0; i < n; ++i) r.devices.emplace_back(new ROCMDevice(i));
    }
    if (deviceID >= r.devices.size()) throw InvalidArgumentError("invalid device id");
    device = r.devices[deviceID].get();
  }
  binding.session.reset(new ROCMSession(*device));
  Device::setThreadDefault(device);
  Session::setThreadDefault(binding.session.get());
}

}  // namespace

void initialize_rocm() { bind_thread(0); }
void initialize_rocm(unsigned deviceID) { bind_thread(deviceID); }

// ---------------------------------------------------------------------------------------------
// fused forms
// ---------------------------------------------------------------------------------------------
namespace rocm {
namespace blas {
Variable<float> matmul_fused(const Tensor<float>& a, const Tensor<float>& b, const Tensor<float>* bias,
                             const Tensor<float>* residual, Activation activation) {
  std::vector<unsigned> s = tfcc::blas::detail::check<float>(a, b, bias);
  if (a.size() == 0 || b.size() == 0) return Variable<float>(Shape(std::move(s)));
  if (dynamic_cast<ROCMDevice*>(Device::getThreadDefault()) == nullptr) throw NotImplementedError();
  return rocm_sgemm(a, b, bias, residual, static_cast<int>(activation));
}
namespace {
struct PermutedView {
  unsigned dims[4];
  uint64_t strides[4];
};
// dims and element strides of transpose(t, perm) seen on t's dense storage
// Tensors of rank 2 and 3 count as rank 4 with leading dimensions of 1.
PermutedView permuted_view(const Shape& shape, const std::vector<size_t>& perm) {
  const size_t rank = shape.size();
  if (rank < 2 || rank > 4 || (!perm.empty() && perm.size() != rank)) throw NotImplementedError("matmul_permuted: rank 2 to 4");
  const size_t pad = 4 - rank;
  unsigned full[4] = {1, 1, 1, 1};
  for (size_t i = 0; i < rank; ++i) full[pad + i] = shape[i];
  uint64_t dense[4];
  uint64_t acc = 1;
  for (int i = 3; i >= 0; --i) {
    dense[i] = acc;
    acc *= full[i];
  }
  bool seen[4] = {false, false, false, false};
  PermutedView v;
  for (size_t i = 0; i < 4; ++i) {
    const size_t src = (perm.empty() || i < pad) ? i : pad + perm[i - pad];
    if (src >= 4 || seen[src]) throw InvalidArgumentError("invalid perm");
    seen[src] = true;
    v.dims[i] = full[src];
    v.strides[i] = dense[src];
  }
  return v;
}
}  // namespace

Variable<float> matmul_permuted(const Tensor<float>& a, const std::vector<size_t>& permA, const Tensor<float>& b,
                                const std::vector<size_t>& permB, const std::vector<size_t>& permC,
                                const Tensor<float>* bias) {
  if (dynamic_cast<ROCMDevice*>(Device::getThreadDefault()) == nullptr) throw NotImplementedError();
  if (a.shape().size() != b.shape().size()) throw NotImplementedError("matmul_permuted: operands of different rank");
  const size_t rank = a.shape().size();
  if (!permC.empty() && permC.size() != rank) throw InvalidArgumentError("invalid perm");
  const PermutedView va = permuted_view(a.shape(), permA), vb = permuted_view(b.shape(), permB);
  if (va.dims[0] != vb.dims[0] || va.dims[1] != vb.dims[1] || va.dims[3] != vb.dims[2]) throw InvalidArgumentError("shape invalid");
  if (a.size() == 0 || b.size() == 0) throw NotImplementedError("matmul_permuted: empty operand");
  const unsigned m = va.dims[2], k = va.dims[3], n = vb.dims[3];
  // the result tensor: dims of [B0, B1, m, n] permuted by permC, dense
  if (bias != nullptr && (bias->shape().size() != 1 || bias->size() != n)) throw InvalidArgumentError("shape invalid");
  const unsigned logical[4] = {va.dims[0], va.dims[1], m, n};
  const size_t pad = 4 - rank;
  std::vector<unsigned> outDims4(4);
  uint64_t cStride[4] = {0, 0, 0, 0};
  {
    bool seen[4] = {false, false, false, false};
    size_t srcOf[4];
    for (size_t p = 0; p < 4; ++p) {
      const size_t src = (permC.empty() || p < pad) ? p : pad + permC[p - pad];
      if (src >= 4 || seen[src]) throw InvalidArgumentError("invalid perm");
      seen[src] = true;
      srcOf[p] = src;
      outDims4[p] = logical[src];
    }
    uint64_t acc = 1;
    for (int p = 3; p >= 0; --p) {
      cStride[srcOf[p]] = acc;
      acc *= outDims4[p];
    }
  }
  const std::vector<unsigned> outDims(outDims4.begin() + pad, outDims4.end());
  if (va.strides[3] != 1 && k != 1) throw NotImplementedError("matmul_permuted: k is not contiguous in a");
  if (cStride[3] != 1 && n != 1) throw NotImplementedError("matmul_permuted: n is not contiguous in the result");
  tfcc_rocm_sgemm_desc d{};
  if (vb.strides[3] == 1 || n == 1) {
    d.trans_b = 0;
    d.ldb = static_cast<unsigned>(vb.strides[2]);
  } else if (vb.strides[2] == 1 || k == 1) {
    d.trans_b = 1;
    d.ldb = static_cast<unsigned>(vb.strides[3]);
  } else {
    throw NotImplementedError("matmul_permuted: neither k nor n is contiguous in b");
  }
  d.lda = static_cast<unsigned>(va.strides[2]);
  d.ldc = static_cast<unsigned>(cStride[2]);
  // a dimension of extent 1 may carry any stride: give it the smallest valid one
  if (m == 1) { d.lda = std::max(d.lda, k); d.ldc = std::max(d.ldc, n); }
  if (d.lda < k) d.lda = k;
  if (d.ldc < n) d.ldc = n;
  if (d.ldb < (d.trans_b ? k : n)) d.ldb = d.trans_b ? k : n;
  // a lone product of at most eight rows with B as stored runs on the streaming kernel, whose sums are ordered
  // differently from the tiled kernel a transposed B needs: leave that case to the separate steps
  if (d.trans_b && m <= 8 && static_cast<uint64_t>(logical[0]) * logical[1] == 1)
    throw NotImplementedError("matmul_permuted: a single product of at most eight rows with a transposed b");
  Variable<float> result{Shape(outDims)};
  d.a = a.data(); d.b = b.data(); d.c = result.data();
  d.bias = bias ? bias->data() : nullptr;
  d.m = m; d.n = n; d.k = k;
  d.batch_outer = logical[0]; d.batch_inner = logical[1];
  d.stride_a = va.strides[0]; d.inner_stride_a = va.strides[1];
  d.stride_b = vb.strides[0]; d.inner_stride_b = vb.strides[1];
  d.stride_c = cStride[0]; d.inner_stride_c = cStride[1];
  check(tfcc_rocm_sgemm_general(current_stream(), &d));
  return result;
}
Variable<float> attention_permuted(const Tensor<float>& q, const std::vector<size_t>& permQ, const Tensor<float>& k,
                                   const std::vector<size_t>& permK, const Tensor<float>& v,
                                   const std::vector<size_t>& permV, const std::vector<size_t>& permOut,
                                   const float* divisor, const Tensor<float>* mask) {
  if (dynamic_cast<ROCMDevice*>(Device::getThreadDefault()) == nullptr) throw NotImplementedError();
  if (q.size() == 0 || k.size() == 0 || v.size() == 0) throw NotImplementedError("attention_permuted: empty operand");
  const PermutedView vq = permuted_view(q.shape(), permQ), vk = permuted_view(k.shape(), permK),
                     vv = permuted_view(v.shape(), permV);
  // [b0, b1, s, d] x [b0, b1, d, t] -> [b0, b1, s, t];  x [b0, b1, t, d2] -> [b0, b1, s, d2]
  const unsigned s = vq.dims[2], d = vq.dims[3], t = vk.dims[3];
  for (int i = 0; i < 2; ++i)
    if (vq.dims[i] != vk.dims[i] || vq.dims[i] != vv.dims[i]) throw InvalidArgumentError("shape invalid");
  if (vk.dims[2] != d || vv.dims[2] != t) throw InvalidArgumentError("shape invalid");
  if (vv.dims[3] != d) throw NotImplementedError("attention_permuted: value size differs from key size");
  const unsigned logical[4] = {vq.dims[0], vq.dims[1], s, d};
  std::vector<unsigned> outDims(4);
  uint64_t oStride[4] = {0, 0, 0, 0};
  {
    bool seen[4] = {false, false, false, false};
    for (size_t p = 0; p < 4; ++p) {
      const size_t src = permOut.empty() ? p : permOut[p];
      if ((!permOut.empty() && permOut.size() != 4) || src >= 4 || seen[src]) throw InvalidArgumentError("invalid perm");
      seen[src] = true;
      outDims[p] = logical[src];
    }
    uint64_t acc = 1;
    for (int p = 3; p >= 0; --p) {
      oStride[permOut.empty() ? p : permOut[p]] = acc;
      acc *= outDims[p];
    }
  }
  // size must be the contiguous dimension everywhere: q rows, k rows (k is taken as K, not K^T), v rows, result rows
  if ((vq.strides[3] != 1 || vk.strides[2] != 1 || vv.strides[3] != 1 || oStride[3] != 1) && d != 1)
    throw NotImplementedError("attention_permuted: head size is not the contiguous dimension");
  tfcc_rocm_attention_desc a{};
  a.s = s; a.t = t; a.d = d;
  a.ldq = static_cast<unsigned>(std::max<uint64_t>(vq.strides[2], d));
  a.ldk = static_cast<unsigned>(std::max<uint64_t>(vk.strides[3], d));
  a.ldv = static_cast<unsigned>(std::max<uint64_t>(vv.strides[2], d));
  a.ldo = static_cast<unsigned>(std::max<uint64_t>(oStride[2], d));
  a.batch_outer = logical[0]; a.batch_inner = logical[1];
  a.stride_q = vq.strides[0]; a.inner_stride_q = vq.strides[1];
  a.stride_k = vk.strides[0]; a.inner_stride_k = vk.strides[1];
  a.stride_v = vv.strides[0]; a.inner_stride_v = vv.strides[1];
  a.stride_out = oStride[0]; a.inner_stride_out = oStride[1];
  a.divisor = divisor ? *divisor : 1.f;
  a.has_divisor = divisor ? 1 : 0;
  a.q = q.data(); a.k = k.data(); a.v = v.data();
  if (mask != nullptr) {
    const Shape& ms = mask->shape();
    if (ms.size() != 4 || ms[3] != t || ms[2] != 1 || (ms[0] != 1 && ms[0] != logical[0]) || (ms[1] != 1 && ms[1] != logical[1]))
      throw NotImplementedError("attention_permuted: the mask is not [b0 or 1, b1 or 1, 1, keys]");
    a.mask = mask->data();
    a.stride_mask = ms[0] == 1 ? 0 : static_cast<uint64_t>(ms[1]) * t;
    a.inner_stride_mask = ms[1] == 1 ? 0 : t;
  }
  if (!tfcc_rocm_attention_f32_supported(&a)) throw NotImplementedError("attention_permuted: outside the kernel's limits");
  Variable<float> result{Shape(outDims)};
  a.out = result.data();
  check(tfcc_rocm_attention_f32(current_stream(), &a));
  return result;
}
std::vector<Variable<float>> matmul_grouped(const Tensor<float>& a, const std::vector<const Tensor<float>*>& b,
                                            const std::vector<const Tensor<float>*>& bias) {
  if (dynamic_cast<ROCMDevice*>(Device::getThreadDefault()) == nullptr) throw NotImplementedError();
  const size_t groups = b.size();
  if (groups < 1 || groups > 4 || bias.size() != groups) throw NotImplementedError("matmul_grouped: 1 to 4 products");
  const size_t ra = a.shape().size();
  if (ra < 2 || a.size() == 0) throw NotImplementedError("matmul_grouped: operand a");
  const unsigned k = a.shape(ra - 1), m = a.size() / k, n = b[0]->shape().size() == 2 ? b[0]->shape(1) : 0;
  for (size_t g = 0; g < groups; ++g) {
    if (b[g]->shape().size() != 2 || b[g]->shape(0) != k || b[g]->shape(1) != n || n == 0 || bias[g] == nullptr ||
        bias[g]->shape().size() != 1 || bias[g]->size() != n)
      throw NotImplementedError("matmul_grouped: the weight matrices need one common [k, n] shape and [n] biases");
  }
  std::vector<unsigned> shape = a.shape().toVector();
  shape.back() = n;
  std::vector<Variable<float>> results;
  const float* bp[4];
  const float* biasp[4];
  float* cp[4];
  for (size_t g = 0; g < groups; ++g) {
    results.emplace_back(Shape(shape));
    bp[g] = b[g]->data();
    biasp[g] = bias[g]->data();
    cp[g] = results.back().data();
  }
  check(tfcc_rocm_sgemm_grouped(current_stream(), a.data(), bp, biasp, cp, static_cast<unsigned>(groups), m, n, k));
  return results;
}
}  // namespace blas
namespace math {
Variable<float> softmax_div(const Tensor<float>& a, size_t axis, float divisor) {
  if (axis >= a.shape().size()) throw InvalidArgumentError("invalid axis");
  if (a.size() == 0) throw InvalidArgumentError("invalid tensor");
  if (dynamic_cast<ROCMDevice*>(Device::getThreadDefault()) == nullptr) throw NotImplementedError();
  if (axis + 1 != a.shape().size()) throw NotImplementedError("softmax over the last axis only");
  Variable<float> r(a.shape());
  const unsigned cols = a.shape(axis);
  check(tfcc_rocm_softmax_div_f32(current_stream(), a.data(), a.size() / cols, cols, divisor, r.data()));
  return r;
}
}  // namespace math
}  // namespace rocm

// ---------------------------------------------------------------------------------------------
// quantized matmul
// ---------------------------------------------------------------------------------------------
namespace rocm {
namespace quantization {

namespace {

struct QPlan {
  tfcc_rocm_qgemm_desc desc;
  std::vector<unsigned> shape;
};

// checks and batch folding of tfcc/mkl/operations/tfcc_mklquantization.cpp:75-145
QPlan plan(const Tensor<uint8_t>& a, const Tensor<int32_t>& reduceSumA, const Tensor<float>& minA,
           const Tensor<float>& maxA, const Tensor<int8_t>& b, const Tensor<int32_t>& reduceSumB,
           const Tensor<float>& minB, const Tensor<float>& maxB) {
  const size_t ra = a.shape().size(), rb = b.shape().size();
  if (a.size() == 0 || ra < 2) throw InvalidArgumentError("invalid input tensor a");
  if (reduceSumA.size() == 0) throw InvalidArgumentError("invalid tensor reduceSumA");
  require_scalar(minA, "invalid tensor minA");
  require_scalar(maxA, "invalid tensor maxA");
  if (b.size() == 0 || rb < 2) throw InvalidArgumentError("invalid input tensor b");
  if (reduceSumB.size() == 0) throw InvalidArgumentError("invalid tensor reduceSumB");
  require_scalar(minB, "invalid tensor minB");
  require_scalar(maxB, "invalid tensor maxB");
  if (a.shape(ra - 1) != b.shape(rb - 2)) throw InvalidArgumentError("tensor a and b don't match");
  if (ra != rb && ra != 2 && rb != 2) throw InvalidArgumentError("tensor a and b don't match");
  if (a.shape(ra - 2) != reduceSumA.shape(reduceSumA.shape().size() - 1))
    throw InvalidArgumentError("tensor a and reduceSumA don't match");
  if (b.shape(rb - 1) != reduceSumB.shape(reduceSumB.shape().size() - 1))
    throw InvalidArgumentError("tensor b and reduceSumB don't match");
  if (ra == rb)
    for (size_t i = 0; i + 2 < ra; ++i)
      if (a.shape(i) != b.shape(i)) throw InvalidArgumentError("tensor a and b don't match");

  QPlan p{};
  p.shape = ra > rb ? a.shape().toVector() : b.shape().toVector();
  unsigned m = a.shape(ra - 2), n = b.shape(rb - 1), k = a.shape(ra - 1);
  p.shape[p.shape.size() - 2] = m;
  p.shape[p.shape.size() - 1] = n;
  unsigned batch = 1;
  for (size_t i = 0; i + 2 < p.shape.size(); ++i) batch *= p.shape[i];
  uint64_t strideRA = reduceSumA.shape().size() == 1 ? 0 : m;
  uint64_t strideRB = reduceSumB.shape().size() == 1 ? 0 : n;
  uint64_t strideA = ra == 2 ? 0 : static_cast<uint64_t>(m) * k;
  uint64_t strideB = rb == 2 ? 0 : static_cast<uint64_t>(k) * n;
  if (rb == 2) {  // one B for the whole batch: the batch becomes extra rows
    m *= batch;
    strideRA *= batch;
    strideA *= batch;
    batch = 1;
  }
  tfcc_rocm_qgemm_desc& d = p.desc;
  d.a = a.data(); d.b = b.data(); d.rowsum_a = reduceSumA.data(); d.colsum_b = reduceSumB.data();
  d.stride_a = strideA; d.stride_b = strideB; d.stride_rowsum_a = strideRA; d.stride_colsum_b = strideRB;
  d.stride_c = static_cast<uint64_t>(m) * n;
  d.m = m; d.n = n; d.k = k; d.batch = batch;
  d.min_a = minA.data(); d.max_a = maxA.data(); d.min_b = minB.data(); d.max_b = maxB.data();
  return p;
}

}  // namespace

std::tuple<Variable<int32_t>, Variable<float>, Variable<float>> matmul(
    const Tensor<uint8_t>& a, const Tensor<int32_t>& reduceSumA, const Tensor<float>& minA,
    const Tensor<float>& maxA, const Tensor<int8_t>& b, const Tensor<int32_t>& reduceSumB,
    const Tensor<float>& minB, const Tensor<float>& maxB) {
  QPlan p = plan(a, reduceSumA, minA, maxA, b, reduceSumB, minB, maxB);
  Variable<int32_t> result{Shape(p.shape)};
  Variable<float> minResult({1}), maxResult({1});
  p.desc.min_c = minResult.data();
  p.desc.max_c = maxResult.data();
  check(tfcc_rocm_gemm_u8s8s32(current_stream(), &p.desc, result.data()));
  return std::make_tuple(std::move(result), std::move(minResult), std::move(maxResult));
}

PreparedWeights::PreparedWeights(const Tensor<int8_t>& b)
    : _b(&b), _reduceSum(reduce_sum(b, false)), _packed() {
  if (b.shape().size() != 2 || b.size() == 0) throw InvalidArgumentError("invalid weight tensor b");
  const unsigned k = b.shape(0), n = b.shape(1);
  _packed = Variable<uint8_t>({static_cast<unsigned>(tfcc_rocm_gemv_packed_size(n, k))});
  check(tfcc_rocm_gemv_pack_b(current_stream(), b.data(), n, k, _packed.data()));
}

std::tuple<Variable<int32_t>, Variable<float>, Variable<float>> matmul(
    const Tensor<uint8_t>& a, const Tensor<int32_t>& reduceSumA, const Tensor<float>& minA,
    const Tensor<float>& maxA, const PreparedWeights& w, const Tensor<float>& minB, const Tensor<float>& maxB) {
  QPlan p = plan(a, reduceSumA, minA, maxA, w.weights(), w.reduceSum(), minB, maxB);
  Variable<int32_t> result{Shape(p.shape)};
  Variable<float> minResult({1}), maxResult({1});
  p.desc.min_c = minResult.data();
  p.desc.max_c = maxResult.data();
  p.desc.packed_b = w.packed();
  p.desc.colsum_b_is_exact = 1;  // w.reduceSum() was computed from w.weights()
  check(tfcc_rocm_gemm_u8s8s32(current_stream(), &p.desc, result.data()));
  return std::make_tuple(std::move(result), std::move(minResult), std::move(maxResult));
}

std::tuple<Variable<uint8_t>, Variable<float>, Variable<float>> matmul_requantize(
    const Tensor<uint8_t>& a, const Tensor<int32_t>& reduceSumA, const Tensor<float>& minA,
    const Tensor<float>& maxA, const Tensor<int8_t>& b, const Tensor<int32_t>& reduceSumB,
    const Tensor<float>& minB, const Tensor<float>& maxB, const Tensor<float>& minOutput,
    const Tensor<float>& maxOutput, Variable<int32_t>* accumulators) {
  QPlan p = plan(a, reduceSumA, minA, maxA, b, reduceSumB, minB, maxB);
  require_scalar(minOutput, "invalid minOutput");
  require_scalar(maxOutput, "invalid maxOutput");
  Variable<uint8_t> result{Shape(p.shape)};
  Variable<float> minResult({1}), maxResult({1});
  p.desc.min_c = minResult.data();
  p.desc.max_c = maxResult.data();
  int32_t* acc = nullptr;
  if (accumulators) {
    *accumulators = Variable<int32_t>(Shape(p.shape));
    acc = accumulators->data();
  }
  check(tfcc_rocm_gemm_u8s8s32_requant_u8(current_stream(), &p.desc, acc, result.data(), 0.0, 0.0, 0.0, 0,
                                          minOutput.data(), maxOutput.data()));
  return std::make_tuple(std::move(result), std::move(minResult), std::move(maxResult));
}

template <class T>
Variable<int32_t> reduce_sum(const Tensor<T>& a, bool row) {
  const size_t rank = a.shape().size();
  if (a.size() == 0 || rank < 2) throw InvalidArgumentError("invalid input tensor a");
  std::vector<unsigned> s = a.shape().toVector();
  const unsigned r = s[rank - 2], c = s[rank - 1];
  const unsigned batch = a.size() / r / c;
  s.pop_back();
  s.pop_back();
  s.push_back(row ? r : c);
  Variable<int32_t> result{Shape(std::move(s))};
  if (row)
    check(tfcc_rocm_reduce_sum_rows(current_stream(), a.data(), type_code<T>(), batch, r, c, result.data()));
  else
    check(tfcc_rocm_reduce_sum_cols(current_stream(), a.data(), type_code<T>(), batch, r, c, result.data()));
  return result;
}

template Variable<int32_t> reduce_sum(const Tensor<int8_t>&, bool);
template Variable<int32_t> reduce_sum(const Tensor<uint8_t>&, bool);
template Variable<int32_t> reduce_sum(const Tensor<int16_t>&, bool);

}  // namespace quantization
}  // namespace rocm
}  // namespace tfcc
