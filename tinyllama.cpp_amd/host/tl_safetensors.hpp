// tl_safetensors.hpp — reader of a safetensors file for the host layer: maps the file and hands out the raw tensor bytes, so
// that bf16 weights go from the page cache to the device without a typed host copy (as tl_gguf.hpp does for GGUF files).
// Layout: u64 little-endian header length, that many bytes of JSON {name: {dtype, shape, data_offsets: [begin, end]}}
// (plus an optional "__metadata__" entry), then the data section the offsets refer to.
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

namespace tlhost {

struct SafeTensor {
  std::string name, dtype;  // dtype as spelled in the file: "BF16", "F32", "I32", ...
  std::vector<long long> shape;
  const uint8_t* data = nullptr;  // into the mapping
  size_t nbytes = 0;
};

class SafeTensorsFile {
 public:
  SafeTensorsFile() = default;
  ~SafeTensorsFile();
  SafeTensorsFile(const SafeTensorsFile&) = delete;
  SafeTensorsFile& operator=(const SafeTensorsFile&) = delete;
  // throws std::runtime_error (truncated file, offsets outside the data section, size not matching dtype x shape ...)
  void open(const std::string& path);
  void close();
  const std::vector<SafeTensor>& tensors() const { return tensors_; }  // in data order
  const SafeTensor* find(const std::string& name) const;

 private:
  int fd_ = -1;
  const uint8_t* map_ = nullptr;
  size_t size_ = 0;
  std::vector<SafeTensor> tensors_;
};

}  // namespace tlhost
