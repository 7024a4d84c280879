#include "archive.h"

#include <zlib.h>

#include <cstring>
#include <fstream>
#include <sstream>

namespace tfcc {
namespace runtime {

namespace {

// Offsets and sizes come from the file: every test is written so that it cannot wrap (a - b with b <= a, never a + b).
template <class T>
T rd(const std::string& s, uint64_t pos) {
  if (pos > s.size() || s.size() - pos < sizeof(T)) throw DataFormatError("invalid zip format");
  T v;
  std::memcpy(&v, s.data() + pos, sizeof(T));
  return v;
}

// deflate expands by at most about 1032 : 1; a stored size beyond that is not a size this stream can have
constexpr uint64_t kMaxDeflateRatio = 1032;

std::string inflate_raw(const char* src, size_t srcLen, uint64_t dstLen) {
  if (dstLen / kMaxDeflateRatio > srcLen + 1) throw DataFormatError("invalid zip format: size beyond what the stream can hold");
  std::string out(dstLen, '\0');
  z_stream zs;
  std::memset(&zs, 0, sizeof(zs));
  if (inflateInit2(&zs, -MAX_WBITS) != Z_OK) throw DataFormatError("zlib init failed");
  zs.next_in = reinterpret_cast<Bytef*>(const_cast<char*>(src));
  zs.avail_in = static_cast<uInt>(srcLen);
  size_t produced = 0;
  int rc = Z_OK;
  // sizes beyond 4 GiB are fed in slices: zlib's counters are 32-bit
  size_t consumed = 0;
  while (rc == Z_OK) {
    const size_t inChunk = std::min<size_t>(srcLen - consumed, 1u << 30);
    const size_t outChunk = std::min<size_t>(dstLen - produced, 1u << 30);
    zs.next_in = reinterpret_cast<Bytef*>(const_cast<char*>(src + consumed));
    zs.avail_in = static_cast<uInt>(inChunk);
    zs.next_out = reinterpret_cast<Bytef*>(&out[0] + produced);
    zs.avail_out = static_cast<uInt>(outChunk);
    rc = inflate(&zs, Z_NO_FLUSH);
    consumed += inChunk - zs.avail_in;
    produced += outChunk - zs.avail_out;
    if (rc == Z_OK && inChunk == zs.avail_in && outChunk == zs.avail_out) break;  // no progress
  }
  inflateEnd(&zs);
  if (rc != Z_STREAM_END || produced != dstLen) throw DataFormatError("invalid zip deflate stream");
  return out;
}

// value of a key of the python-dict header of an .npy ("'key': value")
std::string dict_value(const std::string& header, const std::string& key) {
  size_t pos = header.find("'" + key + "'");
  if (pos == std::string::npos) return "";
  pos = header.find(':', pos);
  if (pos == std::string::npos) return "";
  std::string value;
  int depth = 0;
  char quote = 0;
  for (size_t i = pos + 1; i < header.size(); ++i) {
    const char c = header[i];
    if (quote) {
      if (c == quote) quote = 0;
    } else if (c == '\'' || c == '"') {
      quote = c;
    } else if (c == '(' || c == '[' || c == '{') {
      ++depth;
    } else if (c == ')' || c == ']' || (c == '}' && depth > 0)) {
      --depth;
    } else if (depth == 0 && (c == ',' || c == '}')) {
      break;
    }
    value += c;
  }
  const char* blanks = " \r\n\f\b\t";
  const size_t b = value.find_first_not_of(blanks), e = value.find_last_not_of(blanks);
  if (b == std::string::npos) return "";
  return value.substr(b, e + 1 - b);
}

std::string to_c_order(const std::string& body, const std::vector<unsigned>& shape, size_t itemSize) {
  // element (i0, i1, ...) sits at sum(i_d * prod(shape[:d])) in Fortran order
  std::string out(body.size(), '\0');
  const size_t rank = shape.size();
  size_t total = 1;
  for (unsigned d : shape) total *= d;  // the caller has checked total * itemSize <= body.size()
  std::vector<size_t> fstride(rank);
  size_t acc = 1;
  for (size_t d = 0; d < rank; ++d) {
    fstride[d] = acc;
    acc *= shape[d];
  }
  std::vector<unsigned> idx(rank, 0);
  for (size_t c = 0; c < total; ++c) {
    size_t f = 0;
    for (size_t d = 0; d < rank; ++d) f += idx[d] * fstride[d];
    std::memcpy(&out[c * itemSize], &body[f * itemSize], itemSize);
    for (size_t d = rank; d-- > 0;) {
      if (++idx[d] < shape[d]) break;
      idx[d] = 0;
    }
  }
  return out;
}

template <class T, class S>
std::vector<T> cast_body(const std::string& body) {
  const size_t n = body.size() / sizeof(S);
  std::vector<T> out;
  out.reserve(n);
  for (size_t i = 0; i < n; ++i) {
    S v;
    std::memcpy(&v, body.data() + i * sizeof(S), sizeof(S));
    out.push_back(static_cast<T>(v));
  }
  return out;
}

}  // namespace

std::map<std::string, std::string> unzip(const std::string& data) {
  std::map<std::string, std::string> result;
  // end-of-central-directory record: last occurrence of its signature within the trailing 64 KiB + 22
  if (data.size() < 22) throw DataFormatError("invalid zip format");
  size_t eocd = std::string::npos;
  const size_t lowest = data.size() > 22 + 65535 ? data.size() - 22 - 65535 : 0;
  for (size_t pos = data.size() - 22 + 1; pos-- > lowest;) {
    if (rd<uint32_t>(data, pos) == 0x06054b50u) {
      eocd = pos;
      break;
    }
  }
  if (eocd == std::string::npos) throw DataFormatError("invalid zip format");
  uint64_t entries = rd<uint16_t>(data, eocd + 10);
  uint64_t dirOffset = rd<uint32_t>(data, eocd + 16);
  if (entries == 0xffffu || dirOffset == 0xffffffffu) {
    // zip64: locator sits just before the end record and points at the zip64 end record
    if (eocd < 20 || rd<uint32_t>(data, eocd - 20) != 0x07064b50u) throw DataFormatError("invalid zip64 format");
    const uint64_t z64 = rd<uint64_t>(data, eocd - 20 + 8);
    if (rd<uint32_t>(data, z64) != 0x06064b50u) throw DataFormatError("invalid zip64 format");
    entries = rd<uint64_t>(data, z64 + 32);
    dirOffset = rd<uint64_t>(data, z64 + 48);
  }
  uint64_t pos = dirOffset;
  for (uint64_t e = 0; e < entries; ++e) {
    if (rd<uint32_t>(data, pos) != 0x02014b50u) throw DataFormatError("invalid zip format");
    const uint16_t method = rd<uint16_t>(data, pos + 10);
    uint64_t compressedSize = rd<uint32_t>(data, pos + 20);
    uint64_t size = rd<uint32_t>(data, pos + 24);
    const uint16_t nameLen = rd<uint16_t>(data, pos + 28);
    const uint16_t extraLen = rd<uint16_t>(data, pos + 30);
    const uint16_t commentLen = rd<uint16_t>(data, pos + 32);
    uint64_t localOffset = rd<uint32_t>(data, pos + 42);
    if (data.size() - pos < 46ull + nameLen + extraLen) throw DataFormatError("invalid zip format");  // pos <= size: read above
    const std::string name = data.substr(pos + 46, nameLen);
    // zip64 extra field (id 1): present values in the order size, compressed size, local offset
    size_t x = pos + 46 + nameLen;
    const size_t xEnd = x + extraLen;
    while (x + 4 <= xEnd) {
      const uint16_t id = rd<uint16_t>(data, x), len = rd<uint16_t>(data, x + 2);
      if (id == 1) {
        size_t f = x + 4;
        if (size == 0xffffffffu) { size = rd<uint64_t>(data, f); f += 8; }
        if (compressedSize == 0xffffffffu) { compressedSize = rd<uint64_t>(data, f); f += 8; }
        if (localOffset == 0xffffffffu) { localOffset = rd<uint64_t>(data, f); f += 8; }
        if (f > x + 4 + len) throw DataFormatError("invalid zip64 extra header format");
      }
      x += 4 + len;
    }
    if (method != 0 && method != 8) throw DataFormatError("invalid zip compress type: " + std::to_string(method));
    if (rd<uint32_t>(data, localOffset) != 0x04034b50u) throw DataFormatError("invalid zip format");
    // localOffset + 30 <= size after the reads below, so `body` cannot wrap
    const uint64_t body = localOffset + 30 + rd<uint16_t>(data, localOffset + 26) + rd<uint16_t>(data, localOffset + 28);
    if (body > data.size() || compressedSize > data.size() - body) throw DataFormatError("invalid zip format");
    if (method == 0 && size != compressedSize) throw DataFormatError("invalid zip format");
    if (!name.empty() && name.back() != '/') {
      result[name] = method == 0 ? data.substr(body, compressedSize)
                                 : inflate_raw(data.data() + body, compressedSize, size);
    }
    pos += 46 + nameLen + extraLen + commentLen;
  }
  return result;
}

std::map<std::string, std::string> unzip_from_path(const std::string& path) {
  std::ifstream ifs(path, std::ios::binary);
  if (!ifs) throw InvalidArgumentError("open file: \"" + path + "\" failed");
  std::ostringstream ss;
  ss << ifs.rdbuf();
  return unzip(ss.str());
}

size_t NpyArray::count() const {
  size_t n = 1;
  for (unsigned d : shape) {
    if (d != 0 && n > static_cast<size_t>(-1) / d) throw DataFormatError("invalid npy shape: too many elements");
    n *= d;
  }
  return n;
}

NpyArray parse_npy(const std::string& data) {
  if (data.size() < 10 || data.compare(0, 6, "\x93NUMPY") != 0) throw DataFormatError("invalid npy header");
  size_t pos = 8, headLength = 0;
  if (data[6] == 1) {
    headLength = rd<uint16_t>(data, pos);
    pos += 2;
  } else if (data[6] == 2 || data[6] == 3) {
    headLength = rd<uint32_t>(data, pos);
    pos += 4;
  } else {
    throw DataFormatError("unknow npy version");
  }
  if (headLength > data.size() - pos) throw DataFormatError("invalid npy header");
  const std::string header = data.substr(pos, headLength);
  const std::string descr = dict_value(header, "descr");  // quoted: '<f4'
  if (descr.size() < 5) throw DataFormatError("invalid npy descr");
  if (descr[1] != '<' && descr[1] != '|') throw DataFormatError("invalid npy endian");
  for (size_t i = 3; i + 1 < descr.size(); ++i)
    if (descr[i] < '0' || descr[i] > '9') throw DataFormatError("invalid npy type size");
  const std::string strShape = dict_value(header, "shape");
  if (strShape.size() < 2 || !((strShape.front() == '(' && strShape.back() == ')') ||
                               (strShape.front() == '[' && strShape.back() == ']')))
    throw DataFormatError("invalid npy shape");
  NpyArray a;
  std::string num;
  for (size_t i = 1; i < strShape.size(); ++i) {
    if (strShape[i] >= '0' && strShape[i] <= '9') {
      num += strShape[i];
    } else if (!num.empty()) {
      if (num.size() > 10) throw DataFormatError("invalid npy shape");  // no dimension has more than 10 digits
      const unsigned long long extent = std::stoull(num);
      if (extent > 0xffffffffull) throw DataFormatError("invalid npy shape");
      a.shape.push_back(static_cast<unsigned>(extent));
      num.clear();
    }
  }
  if (a.shape.empty()) a.shape.push_back(1u);
  const std::string order = dict_value(header, "fortran_order");
  if (order != "True" && order != "False") throw DataFormatError("invalid npy data order");
  a.type = descr.substr(2, descr.size() - 3);
  const size_t itemSize = std::stoull(a.type.substr(1));
  a.body = data.substr(pos + headLength);
  const size_t count = a.count();
  if (itemSize == 0 || count > a.body.size() / itemSize) throw DataFormatError("invalid npy body");
  if (order == "True" && a.shape.size() > 1) a.body = to_c_order(a.body, a.shape, itemSize);
  return a;
}

template <class T>
std::vector<T> convert_elements(const NpyArray& a) {
  const std::string& t = a.type;
  if (t == "f4") return cast_body<T, float>(a.body);
  if (t == "f8") return cast_body<T, double>(a.body);
  if (t == "i1") return cast_body<T, int8_t>(a.body);
  if (t == "i2") return cast_body<T, int16_t>(a.body);
  if (t == "i4") return cast_body<T, int32_t>(a.body);
  if (t == "i8") return cast_body<T, int64_t>(a.body);
  if (t == "u1" || t == "b1") return cast_body<T, uint8_t>(a.body);
  if (t == "u2") return cast_body<T, uint16_t>(a.body);
  if (t == "u4") return cast_body<T, uint32_t>(a.body);
  if (t == "u8") return cast_body<T, uint64_t>(a.body);
  return {};
}

#define TFCC_INSTANTIATE(T) template std::vector<T> convert_elements<T>(const NpyArray&);
TFCC_INSTANTIATE(float)
TFCC_INSTANTIATE(double)
TFCC_INSTANTIATE(int8_t)
TFCC_INSTANTIATE(uint8_t)
TFCC_INSTANTIATE(int16_t)
TFCC_INSTANTIATE(uint16_t)
TFCC_INSTANTIATE(int32_t)
TFCC_INSTANTIATE(uint32_t)
TFCC_INSTANTIATE(int64_t)
TFCC_INSTANTIATE(uint64_t)
#undef TFCC_INSTANTIATE

NpzData::NpzData(const std::string& npz) {
  for (auto& kv : unzip(npz)) {
    std::string name = kv.first;
    if (name.size() > 4 && name.compare(name.size() - 4, 4, ".npy") == 0) name.resize(name.size() - 4);
    _arrays.emplace(std::move(name), parse_npy(kv.second));
  }
}

const NpyArray& NpzData::get(const std::string& name) const {
  auto it = _arrays.find(name);
  if (it == _arrays.end()) throw InvalidArgumentError("data \"" + name + "\" not found");
  return it->second;
}

std::vector<std::string> NpzData::names() const {
  std::vector<std::string> out;
  for (auto& kv : _arrays) out.push_back(kv.first);
  return out;
}

}  // namespace runtime
}  // namespace tfcc
