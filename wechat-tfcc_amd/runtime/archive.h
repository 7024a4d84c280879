// Containers the runtime reads: a zip archive (stored or deflate members, zip64 sizes) and the
// .npy arrays inside an .npz.  Same accepted inputs and conversions as the reference's loaders
// (tfcc/core/utils/tfcc_commutils.cpp:106-163 unzip, :214-287 parse_npy, :411-436 element
// conversion), but read through the archive's central directory so members written with a
// trailing data descriptor are found too.
#pragma once

#include <cstdint>
#include <map>
#include <string>
#include <vector>

#include "tfcc_core.h"

namespace tfcc {
namespace runtime {

class DataFormatError : public Exception {
 public:
  explicit DataFormatError(const std::string& what) : Exception(what) {}
};

// member name -> uncompressed bytes
std::map<std::string, std::string> unzip(const std::string& data);
std::map<std::string, std::string> unzip_from_path(const std::string& path);

struct NpyArray {
  std::vector<unsigned> shape;  // a 0-d array is given shape [1]
  std::string type;             // kind + item size: "f4", "i8", "u1", ...
  std::string body;             // elements in C order, little-endian
  size_t count() const;
};

NpyArray parse_npy(const std::string& data);

// element-wise static_cast of an array body to T; empty when the type code is unknown
template <class T>
std::vector<T> convert_elements(const NpyArray& array);

// All arrays of an .npz, keyed by member name without the ".npy" suffix.
class NpzData {
  std::map<std::string, NpyArray> _arrays;

 public:
  explicit NpzData(const std::string& npz);
  bool has(const std::string& name) const { return _arrays.count(name) != 0; }
  const NpyArray& get(const std::string& name) const;
  std::vector<std::string> names() const;
};

}  // namespace runtime
}  // namespace tfcc
