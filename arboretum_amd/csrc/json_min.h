// Minimal JSON document model: parser and emitter sufficient for the booster
// configuration and the model wire format (src/core/json_conversion.h:13-167,
// src/core/model_helper.cpp:16-30).  Objects keep their keys sorted, like the
// std::map-backed documents the reference emits, and floating-point numbers
// are printed as the shortest decimal that round-trips the double.
#ifndef ARBORETUM_AMD_JSON_MIN_H_
#define ARBORETUM_AMD_JSON_MIN_H_

#include <charconv>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace arb {
namespace json {

struct Value;
using Array = std::vector<Value>;
using Object = std::map<std::string, Value>;

struct Value {
  enum Type { Null, Bool, Int, Float, String, Arr, Obj } type = Null;
  bool b = false;
  int64_t i = 0;
  double d = 0.0;
  std::string s;
  std::shared_ptr<Array> a;
  std::shared_ptr<Object> o;

  Value() {}
  static Value MakeBool(bool v) { Value x; x.type = Bool; x.b = v; return x; }
  static Value MakeInt(int64_t v) { Value x; x.type = Int; x.i = v; x.d = (double)v; return x; }
  static Value MakeFloat(double v) { Value x; x.type = Float; x.d = v; return x; }
  static Value MakeString(const std::string &v) { Value x; x.type = String; x.s = v; return x; }
  static Value MakeArray() { Value x; x.type = Arr; x.a = std::make_shared<Array>(); return x; }
  static Value MakeObject() { Value x; x.type = Obj; x.o = std::make_shared<Object>(); return x; }

  bool is_null() const { return type == Null; }
  bool is_number() const { return type == Int || type == Float; }
  bool is_object() const { return type == Obj; }
  bool is_array() const { return type == Arr; }
  const Value *find(const char *key) const {
    if (type != Obj) return nullptr;
    auto it = o->find(key);
    return it == o->end() ? nullptr : &it->second;
  }
  Value &operator[](const std::string &key) { return (*o)[key]; }
  void push(const Value &v) { a->push_back(v); }

  double number() const {
    if (type == Int) return (double)i;
    if (type == Float) return d;
    if (type == Bool) return b ? 1.0 : 0.0;
    throw std::runtime_error("json: number expected");
  }
  bool boolean() const {
    if (type == Bool) return b;
    if (is_number()) return number() != 0.0;
    throw std::runtime_error("json: boolean expected");
  }
};

class Parser {
 public:
  explicit Parser(const char *text) : p_(text) {}
  Value Parse() {
    Value v = ParseValue(0);
    SkipWs();
    if (*p_ != '\0') Fail("trailing characters");
    return v;
  }

 private:
  const char *p_;
  [[noreturn]] void Fail(const char *what) { throw std::runtime_error(std::string("json: ") + what); }
  void SkipWs() {
    while (*p_ == ' ' || *p_ == '\t' || *p_ == '\n' || *p_ == '\r') ++p_;
  }
  Value ParseValue(int depth) {
    if (depth > 64) Fail("nesting too deep");
    SkipWs();
    switch (*p_) {
      case '{': return ParseObject(depth);
      case '[': return ParseArray(depth);
      case '"': return Value::MakeString(ParseString());
      case 't': Expect("true"); return Value::MakeBool(true);
      case 'f': Expect("false"); return Value::MakeBool(false);
      case 'n': Expect("null"); return Value();
      case 'N': Expect("NaN"); return Value::MakeFloat(NAN);       // python's json.dumps extension
      case 'I': Expect("Infinity"); return Value::MakeFloat(INFINITY);
      default: return ParseNumber();
    }
  }
  void Expect(const char *lit) {
    size_t n = std::strlen(lit);
    if (std::strncmp(p_, lit, n) != 0) Fail("unexpected token");
    p_ += n;
  }
  Value ParseNumber() {
    const char *start = p_;
    if (*p_ == '-') {
      ++p_;
      if (*p_ == 'I') { Expect("Infinity"); return Value::MakeFloat(-INFINITY); }
    }
    if (!(*p_ >= '0' && *p_ <= '9')) Fail("unexpected character");
    bool is_float = false;
    while ((*p_ >= '0' && *p_ <= '9') || *p_ == '.' || *p_ == 'e' || *p_ == 'E' || *p_ == '+' || *p_ == '-') {
      if (*p_ == '.' || *p_ == 'e' || *p_ == 'E') is_float = true;
      ++p_;
    }
    std::string tok(start, p_);
    if (!is_float) {
      errno = 0;
      char *end = nullptr;
      long long v = std::strtoll(tok.c_str(), &end, 10);
      if (errno == 0 && end && *end == '\0') return Value::MakeInt(v);
    }
    char *end = nullptr;
    double d = std::strtod(tok.c_str(), &end);
    if (!end || *end != '\0') Fail("bad number");
    return Value::MakeFloat(d);
  }
  std::string ParseString() {
    ++p_;
    std::string out;
    while (*p_ != '"') {
      if (*p_ == '\0') Fail("unterminated string");
      if (*p_ == '\\') {
        ++p_;
        switch (*p_) {
          case '"': out += '"'; break;
          case '\\': out += '\\'; break;
          case '/': out += '/'; break;
          case 'b': out += '\b'; break;
          case 'f': out += '\f'; break;
          case 'n': out += '\n'; break;
          case 'r': out += '\r'; break;
          case 't': out += '\t'; break;
          case 'u': {
            unsigned cp = 0;
            for (int k = 1; k <= 4; ++k) {
              char c = p_[k];
              cp <<= 4;
              if (c >= '0' && c <= '9') cp |= c - '0';
              else if (c >= 'a' && c <= 'f') cp |= c - 'a' + 10;
              else if (c >= 'A' && c <= 'F') cp |= c - 'A' + 10;
              else Fail("bad \\u escape");
            }
            p_ += 4;
            if (cp < 0x80) out += (char)cp;
            else if (cp < 0x800) { out += (char)(0xC0 | (cp >> 6)); out += (char)(0x80 | (cp & 0x3F)); }
            else { out += (char)(0xE0 | (cp >> 12)); out += (char)(0x80 | ((cp >> 6) & 0x3F)); out += (char)(0x80 | (cp & 0x3F)); }
            break;
          }
          default: Fail("bad escape");
        }
        ++p_;
      } else {
        out += *p_++;
      }
    }
    ++p_;
    return out;
  }
  Value ParseArray(int depth) {
    ++p_;
    Value v = Value::MakeArray();
    SkipWs();
    if (*p_ == ']') { ++p_; return v; }
    for (;;) {
      v.push(ParseValue(depth + 1));
      SkipWs();
      if (*p_ == ',') { ++p_; continue; }
      if (*p_ == ']') { ++p_; return v; }
      Fail("expected , or ]");
    }
  }
  Value ParseObject(int depth) {
    ++p_;
    Value v = Value::MakeObject();
    SkipWs();
    if (*p_ == '}') { ++p_; return v; }
    for (;;) {
      SkipWs();
      if (*p_ != '"') Fail("expected string key");
      std::string key = ParseString();
      SkipWs();
      if (*p_ != ':') Fail("expected :");
      ++p_;
      v[key] = ParseValue(depth + 1);
      SkipWs();
      if (*p_ == ',') { ++p_; continue; }
      if (*p_ == '}') { ++p_; return v; }
      Fail("expected , or }");
    }
  }
};

inline Value Parse(const char *text) { return Parser(text).Parse(); }

inline void DumpDouble(double d, std::string &out) {
  if (!std::isfinite(d)) { out += "null"; return; }  // json_conversion.h:28-33: non-finite <-> null
  char buf[40];
  auto r = std::to_chars(buf, buf + sizeof(buf), d);
  std::string s(buf, r.ptr);
  if (s.find_first_of(".en") == std::string::npos) s += ".0";
  out += s;
}

inline void Dump(const Value &v, std::string &out) {
  switch (v.type) {
    case Value::Null: out += "null"; break;
    case Value::Bool: out += v.b ? "true" : "false"; break;
    case Value::Int: out += std::to_string(v.i); break;
    case Value::Float: DumpDouble(v.d, out); break;
    case Value::String: {
      out += '"';
      for (char c : v.s) {
        if (c == '"' || c == '\\') { out += '\\'; out += c; }
        else if (c == '\n') out += "\\n";
        else if (c == '\t') out += "\\t";
        else if (c == '\r') out += "\\r";
        else if ((unsigned char)c < 0x20) { char b[8]; snprintf(b, sizeof b, "\\u%04x", c); out += b; }
        else out += c;
      }
      out += '"';
      break;
    }
    case Value::Arr: {
      out += '[';
      bool first = true;
      for (const Value &e : *v.a) { if (!first) out += ','; first = false; Dump(e, out); }
      out += ']';
      break;
    }
    case Value::Obj: {
      out += '{';
      bool first = true;
      for (const auto &kv : *v.o) {
        if (!first) out += ',';
        first = false;
        Dump(Value::MakeString(kv.first), out);
        out += ':';
        Dump(kv.second, out);
      }
      out += '}';
      break;
    }
  }
}

}  // namespace json
}  // namespace arb
#endif  // ARBORETUM_AMD_JSON_MIN_H_
