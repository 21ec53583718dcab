// A small JSON reader: enough for safetensors headers and the test fixtures' side files
// (objects, arrays, strings with the common escapes, numbers, true / false / null).
#pragma once

#include <cstdlib>
#include <map>
#include <memory>
#include <string>
#include <vector>

namespace atenia {
namespace json {

struct Value {
  enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
  bool b = false;
  double num = 0;
  bool is_int = false;  // the literal had no fraction or exponent (serde's as_u64 / as_i64 case)
  std::string str;
  std::vector<Value> arr;
  std::vector<std::pair<std::string, Value>> obj;  // keeps the file's order

  const Value* get(const std::string& key) const {
    for (const auto& kv : obj)
      if (kv.first == key) return &kv.second;
    return nullptr;
  }
  bool is(Kind k) const { return kind == k; }
};

class Parser {
 public:
  Parser(const char* p, size_t n) : p_(p), end_(p + n) {}
  // Parses one value; ok() tells whether the text was well formed.
  Value parse() {
    Value v = value();
    ws();
    return v;
  }
  bool ok() const { return ok_; }

 private:
  const char* p_;
  const char* end_;
  bool ok_ = true;
  void ws() {
    while (p_ < end_ && (*p_ == ' ' || *p_ == '\n' || *p_ == '\t' || *p_ == '\r')) ++p_;
  }
  bool eat(char c) {
    ws();
    if (p_ < end_ && *p_ == c) {
      ++p_;
      return true;
    }
    return false;
  }
  Value fail() {
    ok_ = false;
    p_ = end_;
    return Value();
  }
  // Containers nest by recursion; a header or config that nests deeper than any real one is
  // rejected instead of being followed down the stack.
  static constexpr int kMaxDepth = 64;
  int depth_ = 0;
  struct DepthGuard {
    int& d;
    explicit DepthGuard(int& x) : d(x) { ++d; }
    ~DepthGuard() { --d; }
  };
  Value value() {
    ws();
    if (p_ >= end_) return fail();
    Value v;
    const char c = *p_;
    if ((c == '{' || c == '[') && depth_ >= kMaxDepth) return fail();
    DepthGuard guard(depth_);
    if (c == '{') {
      ++p_;
      v.kind = Value::Object;
      if (eat('}')) return v;
      do {
        ws();
        Value k = string_value();
        if (!ok_ || !eat(':')) return fail();
        v.obj.emplace_back(std::move(k.str), value());
        if (!ok_) return Value();
      } while (eat(','));
      if (!eat('}')) return fail();
      return v;
    }
    if (c == '[') {
      ++p_;
      v.kind = Value::Array;
      if (eat(']')) return v;
      do {
        v.arr.push_back(value());
        if (!ok_) return Value();
      } while (eat(','));
      if (!eat(']')) return fail();
      return v;
    }
    if (c == '"') return string_value();
    if (end_ - p_ >= 4 && std::string(p_, 4) == "true") { p_ += 4; v.kind = Value::Bool; v.b = true; return v; }
    if (end_ - p_ >= 5 && std::string(p_, 5) == "false") { p_ += 5; v.kind = Value::Bool; return v; }
    if (end_ - p_ >= 4 && std::string(p_, 4) == "null") { p_ += 4; return v; }
    // number (also accepts the non-standard NaN / Infinity some writers emit)
    const char* q = p_;
    while (q < end_ && (*q == '-' || *q == '+' || *q == '.' || *q == 'e' || *q == 'E' ||
                        (*q >= '0' && *q <= '9') || *q == 'N' || *q == 'a' || *q == 'I' ||
                        *q == 'n' || *q == 'f' || *q == 'i' || *q == 't' || *q == 'y'))
      ++q;
    if (q == p_) return fail();
    std::string t(p_, q);
    char* e = nullptr;
    v.num = std::strtod(t.c_str(), &e);
    if (e == t.c_str()) return fail();
    v.kind = Value::Number;
    v.is_int = t.find_first_of(".eENIai") == std::string::npos;
    p_ = q;
    return v;
  }
  Value string_value() {
    ws();
    if (p_ >= end_ || *p_ != '"') return fail();
    ++p_;
    Value v;
    v.kind = Value::String;
    while (p_ < end_ && *p_ != '"') {
      if (*p_ == '\\' && p_ + 1 < end_) {
        ++p_;
        switch (*p_) {
          case 'n': v.str += '\n'; break;
          case 't': v.str += '\t'; break;
          case 'r': v.str += '\r'; break;
          case 'b': v.str += '\b'; break;
          case 'f': v.str += '\f'; break;
          case 'u':  // keep the escape as it is: tensor names are ASCII
            v.str += "\\u";
            break;
          default: v.str += *p_;
        }
        ++p_;
      } else {
        v.str += *p_++;
      }
    }
    if (p_ >= end_) return fail();
    ++p_;
    return v;
  }
};

inline bool parse(const std::string& text, Value& out) {
  Parser p(text.data(), text.size());
  out = p.parse();
  return p.ok();
}

}  // namespace json
}  // namespace atenia
