// Protocol-buffers wire format, just enough to read the runtime's model / input messages and to
// write its output message without a protobuf library.  Field numbers are those of the reference's
// schema files (tfcc_runtime/proto/model.proto, common.proto, data.proto, operations/*.proto); the
// decoding rules are the public proto3 encoding: a key is (field << 3 | wire type) as a varint,
// wire type 0 = varint, 1 = 64-bit, 2 = length-delimited, 5 = 32-bit; repeated scalars may arrive
// packed (one length-delimited blob) or one key per element.
#pragma once

#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

namespace tfcc {
namespace runtime {
namespace wire {

class ParseError : public std::runtime_error {
 public:
  explicit ParseError(const std::string& what) : std::runtime_error("protobuf wire: " + what) {}
};

class Reader {
  const uint8_t* _p;
  const uint8_t* _end;

 public:
  Reader(const void* data, size_t len) : _p(static_cast<const uint8_t*>(data)), _end(_p + len) {}
  explicit Reader(const std::string& s) : Reader(s.data(), s.size()) {}

  bool done() const { return _p >= _end; }

  uint64_t varint() {
    uint64_t v = 0;
    for (int shift = 0; shift < 70; shift += 7) {
      if (_p >= _end) throw ParseError("truncated varint");
      const uint8_t b = *_p++;
      if (shift < 64) v |= static_cast<uint64_t>(b & 0x7f) << shift;
      if (!(b & 0x80)) return v;
    }
    throw ParseError("varint longer than 10 bytes");
  }
  uint32_t fixed32() {
    if (_end - _p < 4) throw ParseError("truncated fixed32");
    uint32_t v;
    std::memcpy(&v, _p, 4);
    _p += 4;
    return v;
  }
  uint64_t fixed64() {
    if (_end - _p < 8) throw ParseError("truncated fixed64");
    uint64_t v;
    std::memcpy(&v, _p, 8);
    _p += 8;
    return v;
  }
  // the payload of a length-delimited field (valid while the parent buffer lives)
  Reader sub() {
    const uint64_t len = varint();
    if (len > static_cast<uint64_t>(_end - _p)) throw ParseError("truncated length-delimited field");
    Reader r(_p, static_cast<size_t>(len));
    _p += len;
    return r;
  }
  std::string bytes() {
    Reader r = sub();
    return std::string(reinterpret_cast<const char*>(r._p), static_cast<size_t>(r._end - r._p));
  }
  // next key; false at the end of the message
  bool next(uint32_t& field, uint32_t& type) {
    if (done()) return false;
    const uint64_t key = varint();
    field = static_cast<uint32_t>(key >> 3);
    type = static_cast<uint32_t>(key & 7);
    if (field == 0) throw ParseError("field number 0");
    return true;
  }
  void skip(uint32_t type) {
    switch (type) {
      case 0: varint(); break;
      case 1: fixed64(); break;
      case 2: sub(); break;
      case 5: fixed32(); break;
      default: throw ParseError("unsupported wire type " + std::to_string(type));
    }
  }
  // one element or a packed run of a repeated varint field
  template <class T>
  void repeatedVarint(uint32_t type, std::vector<T>& out) {
    if (type == 2) {
      Reader r = sub();
      while (!r.done()) out.push_back(static_cast<T>(r.varint()));
    } else if (type == 0) {
      out.push_back(static_cast<T>(varint()));
    } else {
      throw ParseError("repeated varint field with wire type " + std::to_string(type));
    }
  }
  float float32() {
    const uint32_t u = fixed32();
    float f;
    std::memcpy(&f, &u, 4);
    return f;
  }
  double float64() {
    const uint64_t u = fixed64();
    double d;
    std::memcpy(&d, &u, 8);
    return d;
  }
};

class Writer {
  std::string _out;

  void raw(uint64_t v) {
    while (v >= 0x80) {
      _out.push_back(static_cast<char>((v & 0x7f) | 0x80));
      v >>= 7;
    }
    _out.push_back(static_cast<char>(v));
  }

 public:
  void varint(uint32_t field, uint64_t v) {
    raw(static_cast<uint64_t>(field) << 3);
    raw(v);
  }
  void bytes(uint32_t field, const void* data, size_t len) {
    raw(static_cast<uint64_t>(field) << 3 | 2);
    raw(len);
    _out.append(static_cast<const char*>(data), len);
  }
  void bytes(uint32_t field, const std::string& s) { bytes(field, s.data(), s.size()); }
  template <class T>
  void packedVarint(uint32_t field, const std::vector<T>& values) {
    if (values.empty()) return;
    Writer inner;
    for (T v : values) inner.raw(static_cast<uint64_t>(v));
    bytes(field, inner._out);
  }
  const std::string& str() const { return _out; }
  std::string take() { return std::move(_out); }
};

}  // namespace wire
}  // namespace runtime
}  // namespace tfcc
