// tl_json.cpp — see tl_json.hpp.
#include "tl_json.hpp"

#include <cmath>
#include <cstdlib>
#include <stdexcept>

namespace tlhost {

namespace {

struct Parser {
  const char* p;
  const char* end;
  [[noreturn]] void fail(const char* why) const { throw std::runtime_error(std::string("JSON: ") + why); }
  void ws() {
    while (p < end && (*p == ' ' || *p == '\t' || *p == '\n' || *p == '\r')) ++p;
  }
  bool lit(const char* s) {
    const char* q = p;
    for (; *s; ++s, ++q)
      if (q >= end || *q != *s) return false;
    p = q;
    return true;
  }
  static void utf8(std::string& out, uint32_t c) {
    if (c < 0x80) out += (char)c;
    else if (c < 0x800) { out += (char)(0xC0 | (c >> 6)); out += (char)(0x80 | (c & 0x3F)); }
    else if (c < 0x10000) { out += (char)(0xE0 | (c >> 12)); out += (char)(0x80 | ((c >> 6) & 0x3F)); out += (char)(0x80 | (c & 0x3F)); }
    else { out += (char)(0xF0 | (c >> 18)); out += (char)(0x80 | ((c >> 12) & 0x3F)); out += (char)(0x80 | ((c >> 6) & 0x3F)); out += (char)(0x80 | (c & 0x3F)); }
  }
  uint32_t hex4() {
    if (end - p < 4) fail("truncated \\u escape");
    uint32_t v = 0;
    for (int i = 0; i < 4; ++i, ++p) {
      const char c = *p;
      v <<= 4;
      if (c >= '0' && c <= '9') v |= c - '0';
      else if (c >= 'a' && c <= 'f') v |= c - 'a' + 10;
      else if (c >= 'A' && c <= 'F') v |= c - 'A' + 10;
      else fail("bad \\u escape");
    }
    return v;
  }
  std::string string() {
    if (p >= end || *p != '"') fail("expected a string");
    ++p;
    std::string out;
    while (true) {
      if (p >= end) fail("unterminated string");
      const char c = *p++;
      if (c == '"') break;
      if (c != '\\') { out += c; continue; }
      if (p >= end) fail("unterminated escape");
      const char e = *p++;
      switch (e) {
        case '"': out += '"'; break;
        case '\\': out += '\\'; break;
        case '/': out += '/'; break;
        case 'b': out += '\b'; break;
        case 'f': out += '\f'; break;
        case 'n': out += '\n'; break;
        case 'r': out += '\r'; break;
        case 't': out += '\t'; break;
        case 'u': {
          uint32_t c1 = hex4();
          if (c1 >= 0xD800 && c1 < 0xDC00 && end - p >= 6 && p[0] == '\\' && p[1] == 'u') {
            p += 2;
            const uint32_t c2 = hex4();
            c1 = 0x10000 + ((c1 - 0xD800) << 10) + (c2 - 0xDC00);
          }
          utf8(out, c1);
          break;
        }
        default: fail("unknown escape");
      }
    }
    return out;
  }
  Json value(int depth) {
    if (depth > 200) fail("nested too deeply");
    ws();
    if (p >= end) fail("unexpected end");
    Json j;
    const char c = *p;
    if (c == '{') {
      ++p;
      j.kind = Json::OBJECT;
      ws();
      if (p < end && *p == '}') { ++p; return j; }
      while (true) {
        ws();
        std::string k = string();
        ws();
        if (p >= end || *p != ':') fail("expected ':'");
        ++p;
        j.obj.emplace_back(std::move(k), value(depth + 1));
        ws();
        if (p < end && *p == ',') { ++p; continue; }
        if (p < end && *p == '}') { ++p; break; }
        fail("expected ',' or '}'");
      }
    } else if (c == '[') {
      ++p;
      j.kind = Json::ARRAY;
      ws();
      if (p < end && *p == ']') { ++p; return j; }
      while (true) {
        j.arr.push_back(value(depth + 1));
        ws();
        if (p < end && *p == ',') { ++p; continue; }
        if (p < end && *p == ']') { ++p; break; }
        fail("expected ',' or ']'");
      }
    } else if (c == '"') {
      j.kind = Json::STRING;
      j.str = string();
    } else if (lit("true")) {
      j.kind = Json::BOOL;
      j.b = true;
    } else if (lit("false")) {
      j.kind = Json::BOOL;
    } else if (lit("null")) {
    } else {
      const char* s = p;
      bool integral = true;
      if (p < end && (*p == '-' || *p == '+')) ++p;
      while (p < end && ((*p >= '0' && *p <= '9') || *p == '.' || *p == 'e' || *p == 'E' || *p == '-' || *p == '+')) {
        if (*p == '.' || *p == 'e' || *p == 'E') integral = false;
        ++p;
      }
      if (p == s) fail("unexpected character");
      const std::string t(s, p);
      char* e = nullptr;
      j.kind = Json::NUMBER;
      j.num = strtod(t.c_str(), &e);
      if (!e || *e) fail("bad number");
      if (integral && t.size() < 19) {
        j.is_int = true;
        j.inum = strtoll(t.c_str(), nullptr, 10);
      }
    }
    return j;
  }
};

}  // namespace

Json Json::parse(const char* begin, const char* end) {
  Parser ps{begin, end};
  Json j = ps.value(0);
  ps.ws();
  if (ps.p != end) ps.fail("trailing characters");
  return j;
}
Json Json::parse(const std::string& text) { return parse(text.data(), text.data() + text.size()); }

const Json* Json::find(const std::string& key) const {
  if (kind != OBJECT) return nullptr;
  for (const auto& kv : obj)
    if (kv.first == key) return &kv.second;
  return nullptr;
}
const Json& Json::at(const std::string& key) const {
  const Json* j = find(key);
  if (!j) throw std::runtime_error("JSON: key \"" + key + "\" is missing");
  return *j;
}
int64_t Json::as_int(const char* what) const {
  if (kind == NUMBER && is_int) return inum;
  if (kind == NUMBER && std::floor(num) == num && std::fabs(num) < 9e15) return (int64_t)num;
  throw std::runtime_error(std::string("JSON: ") + what + " is not an integer");
}
double Json::as_double(const char* what) const {
  if (kind == NUMBER) return num;
  throw std::runtime_error(std::string("JSON: ") + what + " is not a number");
}
const std::string& Json::as_string(const char* what) const {
  if (kind == STRING) return str;
  throw std::runtime_error(std::string("JSON: ") + what + " is not a string");
}
bool Json::truthy() const {
  switch (kind) {
    case NUL: return false;
    case BOOL: return b;
    case NUMBER: return num != 0.0;
    case STRING: return !str.empty();
    default: return true;
  }
}

}  // namespace tlhost
