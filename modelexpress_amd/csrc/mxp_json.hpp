// Minimal JSON reader for safetensors headers and shard indexes: objects keep their
// key order, numbers are kept as int64 when integral (offsets and shapes must not pass
// through a double), strings are unescaped (\uXXXX to UTF-8).
#pragma once
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace mxp {

struct Json {
  enum Type { Null, Bool, Int, Real, String, Array, Object } type = Null;
  bool b = false;
  int64_t i = 0;
  double d = 0;
  std::string s;
  std::vector<Json> arr;
  std::vector<std::pair<std::string, Json>> obj;

  const Json* get(const std::string& key) const {
    for (const auto& kv : obj)
      if (kv.first == key) return &kv.second;
    return nullptr;
  }
};

class JsonParser {
 public:
  JsonParser(const char* p, size_t n) : p_(p), end_(p + n) {}
  Json parse() {
    Json v = value(0);
    ws();
    if (p_ != end_) fail("trailing characters");
    return v;
  }

 private:
  const char* p_;
  const char* end_;
  [[noreturn]] void fail(const char* what) { throw std::runtime_error(std::string("JSON: ") + what); }
  void ws() {
    while (p_ < end_ && (*p_ == ' ' || *p_ == '\n' || *p_ == '\r' || *p_ == '\t')) ++p_;
  }
  Json value(int depth) {
    if (depth > 64) fail("nesting too deep");
    ws();
    if (p_ >= end_) fail("unexpected end");
    Json v;
    switch (*p_) {
      case '{': {
        v.type = Json::Object;
        ++p_;
        ws();
        if (p_ < end_ && *p_ == '}') { ++p_; return v; }
        for (;;) {
          ws();
          if (p_ >= end_ || *p_ != '"') fail("expected string key");
          std::string k = string();
          ws();
          if (p_ >= end_ || *p_ != ':') fail("expected ':'");
          ++p_;
          v.obj.emplace_back(std::move(k), value(depth + 1));
          ws();
          if (p_ >= end_) fail("unexpected end in object");
          if (*p_ == ',') { ++p_; continue; }
          if (*p_ == '}') { ++p_; return v; }
          fail("expected ',' or '}'");
        }
      }
      case '[': {
        v.type = Json::Array;
        ++p_;
        ws();
        if (p_ < end_ && *p_ == ']') { ++p_; return v; }
        for (;;) {
          v.arr.push_back(value(depth + 1));
          ws();
          if (p_ >= end_) fail("unexpected end in array");
          if (*p_ == ',') { ++p_; continue; }
          if (*p_ == ']') { ++p_; return v; }
          fail("expected ',' or ']'");
        }
      }
      case '"':
        v.type = Json::String;
        v.s = string();
        return v;
      case 't':
        lit("true");
        v.type = Json::Bool;
        v.b = true;
        return v;
      case 'f':
        lit("false");
        v.type = Json::Bool;
        return v;
      case 'n':
        lit("null");
        return v;
      default:
        return number();
    }
  }
  void lit(const char* w) {
    const size_t n = std::strlen(w);
    if ((size_t)(end_ - p_) < n || std::memcmp(p_, w, n) != 0) fail("bad literal");
    p_ += n;
  }
  Json number() {
    const char* st = p_;
    bool real = false;
    if (p_ < end_ && *p_ == '-') ++p_;
    if (p_ >= end_ || *p_ < '0' || *p_ > '9') fail("bad number");
    while (p_ < end_ && ((*p_ >= '0' && *p_ <= '9') || *p_ == '.' || *p_ == 'e' || *p_ == 'E' ||
                         *p_ == '+' || *p_ == '-')) {
      if (*p_ == '.' || *p_ == 'e' || *p_ == 'E') real = true;
      ++p_;
    }
    std::string t(st, p_);
    Json v;
    if (real) {
      v.type = Json::Real;
      v.d = std::strtod(t.c_str(), nullptr);
    } else {
      v.type = Json::Int;
      errno = 0;
      v.i = std::strtoll(t.c_str(), nullptr, 10);
      if (errno) fail("integer out of range");
      v.d = (double)v.i;
    }
    return v;
  }
  static void utf8(std::string& o, uint32_t c) {
    if (c < 0x80) o += (char)c;
    else if (c < 0x800) { o += (char)(0xC0 | (c >> 6)); o += (char)(0x80 | (c & 0x3F)); }
    else if (c < 0x10000) {
      o += (char)(0xE0 | (c >> 12)); o += (char)(0x80 | ((c >> 6) & 0x3F)); o += (char)(0x80 | (c & 0x3F));
    } else {
      o += (char)(0xF0 | (c >> 18)); o += (char)(0x80 | ((c >> 12) & 0x3F));
      o += (char)(0x80 | ((c >> 6) & 0x3F)); o += (char)(0x80 | (c & 0x3F));
    }
  }
  uint32_t hex4() {
    if (end_ - p_ < 4) fail("bad \\u escape");
    uint32_t c = 0;
    for (int k = 0; k < 4; ++k) {
      const char h = *p_++;
      c <<= 4;
      if (h >= '0' && h <= '9') c |= (uint32_t)(h - '0');
      else if (h >= 'a' && h <= 'f') c |= (uint32_t)(h - 'a' + 10);
      else if (h >= 'A' && h <= 'F') c |= (uint32_t)(h - 'A' + 10);
      else fail("bad \\u escape");
    }
    return c;
  }
  std::string string() {
    ++p_;  // opening quote
    std::string o;
    for (;;) {
      if (p_ >= end_) fail("unterminated string");
      const char c = *p_++;
      if (c == '"') return o;
      if (c != '\\') { o += c; continue; }
      if (p_ >= end_) fail("unterminated escape");
      const char e = *p_++;
      switch (e) {
        case '"': o += '"'; break;
        case '\\': o += '\\'; break;
        case '/': o += '/'; break;
        case 'b': o += '\b'; break;
        case 'f': o += '\f'; break;
        case 'n': o += '\n'; break;
        case 'r': o += '\r'; break;
        case 't': o += '\t'; break;
        case 'u': {
          uint32_t c1 = hex4();
          if (c1 >= 0xD800 && c1 < 0xDC00 && end_ - p_ >= 6 && p_[0] == '\\' && p_[1] == 'u') {
            p_ += 2;
            const uint32_t c2 = hex4();
            if (c2 >= 0xDC00 && c2 < 0xE000) c1 = 0x10000 + ((c1 - 0xD800) << 10) + (c2 - 0xDC00);
          }
          utf8(o, c1);
          break;
        }
        default: fail("bad escape");
      }
    }
  }
};

}  // namespace mxp
