// tl_json.hpp — a small JSON reader for the host layer: configuration files (config.json of a checkpoint folder), the
// header of a safetensors file, and the line-oriented step records of tl_trace. Values are a plain tree; numbers are kept
// as double (and as the integer they spell when they spell one). Throws std::runtime_error on malformed input.
#pragma once
#include <cstdint>
#include <map>
#include <string>
#include <vector>

namespace tlhost {

struct Json {
  enum Kind { NUL, BOOL, NUMBER, STRING, ARRAY, OBJECT } kind = NUL;
  bool b = false;
  double num = 0.0;
  int64_t inum = 0;      // NUMBER written without fraction or exponent
  bool is_int = false;
  std::string str;
  std::vector<Json> arr;
  std::vector<std::pair<std::string, Json>> obj;  // in file order

  static Json parse(const std::string& text);
  static Json parse(const char* begin, const char* end);

  bool is_null() const { return kind == NUL; }
  const Json* find(const std::string& key) const;       // OBJECT member or nullptr
  const Json& at(const std::string& key) const;         // throws when missing
  // typed reads with the path in the error text
  int64_t as_int(const char* what) const;
  double as_double(const char* what) const;
  const std::string& as_string(const char* what) const;
  bool truthy() const;  // false for null / false / 0 / "" / missing-like values
};

}  // namespace tlhost
