// tl_safetensors.cpp — see tl_safetensors.hpp.
#include "tl_safetensors.hpp"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cstring>
#include <stdexcept>

#include "tl_json.hpp"

namespace tlhost {

namespace {
size_t dtype_bytes(const std::string& d) {
  if (d == "F64" || d == "I64" || d == "U64") return 8;
  if (d == "F32" || d == "I32" || d == "U32") return 4;
  if (d == "BF16" || d == "F16" || d == "I16" || d == "U16") return 2;
  if (d == "I8" || d == "U8" || d == "BOOL" || d == "F8_E4M3" || d == "F8_E5M2") return 1;
  return 0;
}
}  // namespace

SafeTensorsFile::~SafeTensorsFile() { close(); }

void SafeTensorsFile::close() {
  if (map_) munmap(const_cast<uint8_t*>(map_), size_);
  if (fd_ >= 0) ::close(fd_);
  map_ = nullptr;
  fd_ = -1;
  size_ = 0;
  tensors_.clear();
}

void SafeTensorsFile::open(const std::string& path) {
  close();
  fd_ = ::open(path.c_str(), O_RDONLY);
  if (fd_ < 0) throw std::runtime_error("safetensors: cannot open " + path);
  struct stat st;
  if (fstat(fd_, &st) != 0 || st.st_size < 8) throw std::runtime_error("safetensors: " + path + " is too short");
  size_ = (size_t)st.st_size;
  void* m = mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd_, 0);
  if (m == MAP_FAILED) throw std::runtime_error("safetensors: cannot map " + path);
  map_ = static_cast<const uint8_t*>(m);
  uint64_t hlen = 0;
  for (int i = 7; i >= 0; --i) hlen = (hlen << 8) | map_[i];
  if (hlen > size_ - 8) throw std::runtime_error("safetensors: header of " + path + " runs past the end of the file");
  const char* hb = reinterpret_cast<const char*>(map_ + 8);
  const Json header = Json::parse(hb, hb + hlen);
  if (header.kind != Json::OBJECT) throw std::runtime_error("safetensors: header is not an object");
  const uint8_t* data = map_ + 8 + hlen;
  const size_t data_bytes = size_ - 8 - (size_t)hlen;
  for (const auto& kv : header.obj) {
    if (kv.first == "__metadata__") continue;
    SafeTensor t;
    t.name = kv.first;
    t.dtype = kv.second.at("dtype").as_string("dtype");
    size_t n = 1;
    for (const Json& d : kv.second.at("shape").arr) {
      const long long v = d.as_int("shape entry");
      if (v < 0) throw std::runtime_error("safetensors: negative dimension in " + t.name);
      t.shape.push_back(v);
      n *= (size_t)v;
    }
    const Json& off = kv.second.at("data_offsets");
    if (off.arr.size() != 2) throw std::runtime_error("safetensors: data_offsets of " + t.name);
    const long long b = off.arr[0].as_int("offset"), e = off.arr[1].as_int("offset");
    if (b < 0 || e < b || (size_t)e > data_bytes) throw std::runtime_error("safetensors: " + t.name + " lies outside the data section");
    t.nbytes = (size_t)(e - b);
    const size_t eb = dtype_bytes(t.dtype);
    if (eb && n * eb != t.nbytes) throw std::runtime_error("safetensors: size of " + t.name + " does not fit its dtype and shape");
    t.data = data + b;
    tensors_.push_back(std::move(t));
  }
  std::sort(tensors_.begin(), tensors_.end(), [](const SafeTensor& a, const SafeTensor& b) { return a.data < b.data; });
}

const SafeTensor* SafeTensorsFile::find(const std::string& name) const {
  for (const SafeTensor& t : tensors_)
    if (t.name == name) return &t;
  return nullptr;
}

}  // namespace tlhost
