// Host-side framework types the ROCm device plugs into: the part of TFCC's core/framework layer
// that the matmul path touches, with the same names, semantics and error behaviour, so that code
// written against the reference (tfcc::Variable, tfcc::View, tfcc::Session, tfcc::Device ...)
// compiles against this header unchanged.
//
//   Shape                 tfcc/core/framework/tfcc_shape.h:24-81 (unsigned dims, unsigned area, rank-0 has area 0)
//   Tensor / Variable     tfcc/core/framework/tfcc_tensor.h:25-56, tfcc_variable.cpp:27-125
//   View                  tfcc/core/framework/tfcc_view.h:24-88, tfcc_view.cpp:25-121
//   Allocator             tfcc/core/allocators/tfcc_allocator.h:22-44
//   FlexAllocator         tfcc/core/allocators/tfcc_flexallocator.cpp:26-160 (4 KiB / 1 MiB buckets, +64 bytes,
//                         limit, flex limit; accounting pinned by tfcc/test/framework.cpp:113-171)
//   Session / Device      tfcc/core/framework/tfcc_session.h:28-66, tfcc_device.h:34-135
//   exceptions            tfcc/core/exceptions/
// Plain C++17, no GPU headers: device specifics live behind the C ABI (include/tfcc_rocm.h).
#pragma once

#include <atomic>
#include <cstddef>
#include <cstdint>
#include <exception>
#include <functional>
#include <initializer_list>
#include <map>
#include <memory>
#include <mutex>
#include <set>
#include <string>
#include <tuple>
#include <vector>

namespace tfcc {

// ---------------------------------------------------------------------------------------------
// exceptions
// ---------------------------------------------------------------------------------------------
class Exception : public std::exception {
  std::string _what;

 public:
  explicit Exception(std::string what) : _what(std::move(what)) {}
  const char* what() const noexcept override { return _what.c_str(); }
};

#define TFCC_DEFINE_ERROR(NAME, DEFAULT_TEXT)                       \
  class NAME : public Exception {                                   \
   public:                                                          \
    NAME() : Exception(DEFAULT_TEXT) {}                             \
    explicit NAME(const std::string& what) : Exception(what) {}     \
  }
TFCC_DEFINE_ERROR(InvalidArgumentError, "invalid argument");
TFCC_DEFINE_ERROR(NotImplementedError, "not implemented");
TFCC_DEFINE_ERROR(ResourceExhaustedError, "resource exhausted");
TFCC_DEFINE_ERROR(RuntimeError, "runtime error");
TFCC_DEFINE_ERROR(InvalidDataError, "invalid data");
TFCC_DEFINE_ERROR(DataFormatError, "data format error");
#undef TFCC_DEFINE_ERROR

// ---------------------------------------------------------------------------------------------
// Shape
// ---------------------------------------------------------------------------------------------
class Shape {
  std::vector<unsigned> _dims;
  unsigned _area = 0;

  void recount() {
    _area = _dims.empty() ? 0u : 1u;
    for (unsigned d : _dims) _area *= d;
  }

 public:
  Shape() = default;
  Shape(std::initializer_list<unsigned> dims) : _dims(dims) { recount(); }
  Shape(std::vector<unsigned> dims) : _dims(std::move(dims)) { recount(); }  // implicit, like the reference
  Shape(const Shape&) = default;
  Shape& operator=(const Shape&) = default;
  Shape(Shape&& o) noexcept : _dims(std::move(o._dims)), _area(o._area) { o._area = 0; }
  Shape& operator=(Shape&& o) noexcept {
    _dims = std::move(o._dims);
    _area = o._area;
    o._area = 0;
    return *this;
  }

  unsigned operator[](size_t i) const { return _dims[i]; }
  size_t size() const { return _dims.size(); }
  unsigned area() const { return _area; }
  const std::vector<unsigned>& toVector() const { return _dims; }
  friend bool operator==(const Shape& a, const Shape& b) { return a._dims == b._dims; }
  friend bool operator!=(const Shape& a, const Shape& b) { return !(a == b); }
};

// ---------------------------------------------------------------------------------------------
// Allocators
// ---------------------------------------------------------------------------------------------
class Allocator {
 protected:
  std::function<void*(size_t)> _realMalloc;
  std::function<void(void*)> _realFree;

 public:
  Allocator() = default;
  Allocator(const Allocator&) = delete;
  Allocator& operator=(const Allocator&) = delete;
  virtual ~Allocator() {}

  virtual void* malloc(size_t len) = 0;
  virtual void free(void* p) = 0;
  virtual void releaseCache() = 0;
  virtual void setLimit(size_t limit) = 0;
  virtual size_t used() const = 0;

  // Pinning keeps every block that is freed between beginPinning() and endPinning() out of the
  // general cache: such a block may be handed out again only while pinning is still on.
  // endPinning() returns the blocks left over; they stay reserved until given to unpin().  A
  // recorded kernel sequence that is replayed later relies on this: no other user of the
  // allocator can be given memory the recording writes to.
  virtual void beginPinning() {}
  virtual std::vector<void*> endPinning() { return {}; }
  virtual void unpin(const std::vector<void*>&) {}

  void setRealMalloc(std::function<void*(size_t)> f) { _realMalloc = std::move(f); }
  void setRealFree(std::function<void(void*)> f) { _realFree = std::move(f); }
};

// Size-bucketed caching allocator.  A freed block goes to a free list keyed by its bucket size and
// is handed out again for the next request of that bucket; real frees happen only on
// releaseCache(), when the limit is hit, or past the flex limit.  Freed device blocks are thereby
// reused in stream order, which is what makes "destroy the inputs right after the call" safe for
// asynchronous kernels.
class FlexAllocator : public Allocator {
  std::multimap<size_t, void*> _cached;  // bucket size -> free block
  std::map<void*, size_t> _live;         // block handed out -> bucket size
  mutable std::mutex _mtx;
  std::atomic<size_t> _used{0};          // bytes obtained from the real allocator
  size_t _limit = 0, _flexLimit = 0;
  bool _pinning = false;
  std::multimap<size_t, void*> _pinnedFree;  // freed while pinning: reusable only while pinning
  std::map<void*, size_t> _reserved;         // handed to the caller of endPinning()

  static size_t bucket(size_t len);
  void releaseDownTo(size_t target);

 public:
  FlexAllocator() = default;
  ~FlexAllocator() override;

  void* malloc(size_t len) override;
  void free(void* p) override;
  void releaseCache() override { releaseDownTo(0); }
  void setLimit(size_t limit) override { _limit = limit; }
  size_t used() const override { return _used.load(); }
  void setFlexLimit(size_t flexLimit) { _flexLimit = flexLimit; }
  void beginPinning() override;
  std::vector<void*> endPinning() override;
  void unpin(const std::vector<void*>& blocks) override;
};

// Pass-through allocator (tfcc/core/allocators/tfcc_simpleallocator.*)
class SimpleAllocator : public Allocator {
  std::map<void*, size_t> _live;
  std::mutex _mtx;
  std::atomic<size_t> _used{0};
  size_t _limit = 0;

 public:
  void* malloc(size_t len) override;
  void free(void* p) override;
  void releaseCache() override {}
  void setLimit(size_t limit) override { _limit = limit; }
  size_t used() const override { return _used.load(); }
};

// ---------------------------------------------------------------------------------------------
// Device and Session
// ---------------------------------------------------------------------------------------------
template <class T>
class Interface;
struct InterfaceSet;  // one Interface<T> per element type, defined in tfcc_interfaces.h

// 8-bit device type in the top byte of the device id.  CUDA and MKL keep the reference's values
// (tfcc/core/framework/tfcc_device.h:34-37); ROCM and HOST are new.
enum class DeviceType : uint8_t { CUDA = 0, MKL = 1, ROCM = 2, HOST = 3 };

class Device {
  static thread_local Device* _threadDevice;

 protected:
  unsigned _deviceID;
  std::unique_ptr<Allocator> _allocator;
  std::unique_ptr<InterfaceSet> _interfaces;
  // Constants of this device, keyed by (scope, name, element type): tfcc/core/framework/tfcc_constantmanager.cpp:35-49.
  // Declared after the allocator so that they are released before it.
  std::mutex _constantMutex;
  std::map<std::tuple<const void*, std::string, int>, std::shared_ptr<void>> _constants;

 public:
  Device(DeviceType type, unsigned index, std::unique_ptr<Allocator> allocator);
  Device(const Device&) = delete;
  Device& operator=(const Device&) = delete;
  virtual ~Device();

  // makes the device current for the calling thread (cudaSetDevice / hipSetDevice)
  virtual void attach() = 0;

  void* malloc(size_t len) { return _allocator->malloc(len); }
  void free(void* p) { _allocator->free(p); }
  void releaseCache() { _allocator->releaseCache(); }
  Allocator& getAllocator() { return *_allocator; }

  template <class T>
  Interface<T>& getInterface(T = T());

  // The constant registered under (scope, name, typeKey), created with `make` on first use.
  std::shared_ptr<void> getConstantSlot(const void* scope, const std::string& name, int typeKey,
                                        const std::function<std::shared_ptr<void>()>& make);
  void removeConstants(const void* scope);

  unsigned getDeviceID() const { return _deviceID; }  // type << 24 | index
  DeviceType getDeviceType() const { return static_cast<DeviceType>(_deviceID >> 24); }

  static Device* getThreadDefault() { return _threadDevice; }
  static void setThreadDefault(Device* d) {
    _threadDevice = d;
    if (d) d->attach();
  }
};

class Session {
  static thread_local Session* _threadSession;

 protected:
  std::unique_ptr<Allocator> _allocator;
  std::vector<std::function<void(const Session*)>> _releaseCallbacks;
  void preRelease();  // runs the callbacks; call first in a subclass destructor

 public:
  explicit Session(std::unique_ptr<Allocator> allocator) : _allocator(std::move(allocator)) {}
  Session(const Session&) = delete;
  Session& operator=(const Session&) = delete;
  virtual ~Session() {}

  virtual void sync() const = 0;
  virtual Device& getDevice() = 0;
  virtual const Device& getDevice() const = 0;

  void registerReleaseCallback(std::function<void(const Session*)> cb) { _releaseCallbacks.push_back(std::move(cb)); }
  void* malloc(size_t len) { return _allocator->malloc(len); }
  void free(void* p) { _allocator->free(p); }
  void releaseCache() { _allocator->releaseCache(); }
  Allocator& getAllocator() { return *_allocator; }

  static Session* getThreadDefault() { return _threadSession; }
  static void setThreadDefault(Session* s) { _threadSession = s; }
};

// ---------------------------------------------------------------------------------------------
// Tensor, Variable, View
// ---------------------------------------------------------------------------------------------
template <class T>
class Tensor {
 protected:
  Shape _shape;
  Tensor() = default;
  explicit Tensor(Shape s) : _shape(std::move(s)) {}
  Tensor(Tensor&&) noexcept = default;
  Tensor& operator=(Tensor&&) noexcept = default;

 public:
  Tensor(const Tensor&) = delete;
  Tensor& operator=(const Tensor&) = delete;
  virtual ~Tensor() {}

  virtual const T* data() const = 0;  // device pointer; use tfcc::data::get to read values
  virtual void sync() const = 0;
  virtual bool available() const = 0;

  unsigned size() const { return _shape.area(); }
  const Shape& shape() const { return _shape; }
  unsigned shape(size_t n) const { return _shape[n]; }
};

namespace detail {
Shape expand_dims(const Shape& s, size_t axis);
Shape squeeze_all(const Shape& s);
Shape squeeze_axes(const Shape& s, const std::set<size_t>& axes);
void check_same_area(const Shape& from, const Shape& to);
}  // namespace detail

// Owning tensor; its memory comes from (and returns to) the Session that was the thread default
// when it was created.
template <class T>
class Variable : public Tensor<T> {
  Session* _session;
  T* _data = nullptr;

  void allocate() {
    if (this->_shape.area() == 0) return;
    _data = static_cast<T*>(_session->malloc(sizeof(T) * static_cast<size_t>(this->_shape.area())));
    if (_data == nullptr) throw ResourceExhaustedError();
  }

 public:
  Variable() : _session(Session::getThreadDefault()) {}
  explicit Variable(const Shape& s) : Tensor<T>(s), _session(Session::getThreadDefault()) { allocate(); }
  explicit Variable(Shape&& s) : Tensor<T>(std::move(s)), _session(Session::getThreadDefault()) { allocate(); }
  Variable(std::initializer_list<unsigned> dims) : Variable(Shape(dims)) {}
  Variable(Variable&& v) noexcept : Tensor<T>(std::move(v)), _session(v._session), _data(v._data) { v._data = nullptr; }
  Variable& operator=(Variable&& v) noexcept {
    if (this != &v) {
      if (_data) _session->free(_data);
      _session = v._session;
      Tensor<T>::operator=(std::move(v));
      _data = v._data;
      v._data = nullptr;
    }
    return *this;
  }
  ~Variable() override {
    if (_data) _session->free(_data);
  }

  const T* data() const override { return _data; }
  T* data() { return _data; }
  void sync() const override { _session->sync(); }
  bool available() const override { return _session == Session::getThreadDefault(); }

  void reshape(Shape s) {
    detail::check_same_area(this->_shape, s);
    this->_shape = std::move(s);
  }
  void expandDims(size_t axis) { this->_shape = detail::expand_dims(this->_shape, axis); }
  void squeeze() { this->_shape = detail::squeeze_all(this->_shape); }
  void squeeze(const std::set<size_t>& axes) { this->_shape = detail::squeeze_axes(this->_shape, axes); }
};

// Non-owning window on another tensor: the whole of it under a new shape, or rows [start, end) of
// its first dimension.
template <class T>
class View : public Tensor<T> {
  const Tensor<T>* _tensor = nullptr;
  size_t _offset = 0;

 public:
  View() = default;
  explicit View(const Tensor<T>& t) : View(t, t.shape(), 0, t.shape().size() ? t.shape(0) : 0) {}
  View(const Tensor<T>& t, const Shape& s) : View(t, s, 0, s.size() ? s[0] : 0) {}
  View(const Tensor<T>& t, const Shape& s, unsigned start) : View(t, s, start, s.size() ? s[0] : 0) {}
  View(const Tensor<T>& t, const Shape& s, unsigned start, unsigned end) : _tensor(&t) {
    if (s.size() == 0 || s.area() != t.size()) throw InvalidArgumentError("invalid shape");
    if (s[0] > 0 && start >= s[0]) throw InvalidArgumentError("invalid start");
    if (end > s[0]) end = s[0];
    std::vector<unsigned> dims = s.toVector();
    dims[0] = end - start;
    this->_shape = Shape(std::move(dims));
    _offset = start > 0 ? static_cast<size_t>(s.area() / s[0]) * start : 0;
  }
  View(const View& v) : Tensor<T>(v._shape), _tensor(v._tensor), _offset(v._offset) {}
  View& operator=(const View& v) {
    this->_shape = v._shape;
    _tensor = v._tensor;
    _offset = v._offset;
    return *this;
  }
  View(View&&) noexcept = default;
  View& operator=(View&&) noexcept = default;

  const T* data() const override { return _tensor->data() + _offset; }
  void sync() const override { _tensor->sync(); }
  bool available() const override { return _tensor->available(); }

  void reshape(Shape s) {
    detail::check_same_area(this->_shape, s);
    this->_shape = std::move(s);
  }
  void expandDims(size_t axis) { this->_shape = detail::expand_dims(this->_shape, axis); }
  void squeeze() { this->_shape = detail::squeeze_all(this->_shape); }
  void squeeze(const std::set<size_t>& axes) { this->_shape = detail::squeeze_axes(this->_shape, axes); }
};

}  // namespace tfcc
