// Minimal JSON reader (objects, arrays, strings, numbers, true/false/null) for the pipeline
// configuration files.  Enough for the reference's config schema
// (pipeline/config_all/llama3-8B/1024.json); not a general-purpose parser.
#pragma once
#include <cctype>
#include <cstdlib>
#include <fstream>
#include <map>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

namespace mini_json {

struct Value {
  enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
  bool b = false;
  double num = 0;
  std::string str;
  std::vector<Value> arr;
  std::map<std::string, Value> obj;

  bool is_null() const { return kind == Null; }
  bool is_array() const { return kind == Array; }
  bool contains(const std::string& k) const { return kind == Object && obj.count(k); }
  const Value& at(const std::string& k) const {
    auto it = obj.find(k);
    if (kind != Object || it == obj.end()) throw std::out_of_range("json: missing key \"" + k + "\"");
    return it->second;
  }
  double number() const {
    if (kind != Number) throw std::invalid_argument("json: not a number");
    return num;
  }
  template <typename T>
  T value(const std::string& k, T dflt) const {
    if (!contains(k) || at(k).kind != Number) return dflt;
    return static_cast<T>(at(k).num);
  }
};

class Parser {
public:
  explicit Parser(const std::string& s) : s_(s) {}
  Value parse() {
    Value v = value();
    ws();
    if (i_ != s_.size()) fail("trailing characters");
    return v;
  }

private:
  const std::string& s_;
  size_t i_ = 0;
  [[noreturn]] void fail(const char* what) {
    throw std::invalid_argument("json: " + std::string(what) + " at offset " + std::to_string(i_));
  }
  void ws() {
    while (i_ < s_.size() && std::isspace((unsigned char)s_[i_])) ++i_;
  }
  bool lit(const char* w) {
    size_t n = std::char_traits<char>::length(w);
    if (s_.compare(i_, n, w) == 0) {
      i_ += n;
      return true;
    }
    return false;
  }
  Value value() {
    ws();
    if (i_ >= s_.size()) fail("unexpected end");
    Value v;
    char c = s_[i_];
    if (c == '{') {
      v.kind = Value::Object;
      ++i_;
      ws();
      if (s_[i_] == '}') { ++i_; return v; }
      for (;;) {
        ws();
        if (s_[i_] != '"') fail("expected key");
        std::string k = string();
        ws();
        if (s_[i_] != ':') fail("expected ':'");
        ++i_;
        v.obj[k] = value();
        ws();
        if (s_[i_] == ',') { ++i_; continue; }
        if (s_[i_] == '}') { ++i_; break; }
        fail("expected ',' or '}'");
      }
    } else if (c == '[') {
      v.kind = Value::Array;
      ++i_;
      ws();
      if (s_[i_] == ']') { ++i_; return v; }
      for (;;) {
        v.arr.push_back(value());
        ws();
        if (s_[i_] == ',') { ++i_; continue; }
        if (s_[i_] == ']') { ++i_; break; }
        fail("expected ',' or ']'");
      }
    } else if (c == '"') {
      v.kind = Value::String;
      v.str = string();
    } else if (lit("true")) {
      v.kind = Value::Bool;
      v.b = true;
    } else if (lit("false")) {
      v.kind = Value::Bool;
    } else if (lit("null")) {
      v.kind = Value::Null;
    } else {
      char* end = nullptr;
      v.num = std::strtod(s_.c_str() + i_, &end);
      if (end == s_.c_str() + i_) fail("bad value");
      v.kind = Value::Number;
      i_ = end - s_.c_str();
    }
    return v;
  }
  std::string string() {
    std::string out;
    ++i_;  // opening quote
    while (i_ < s_.size() && s_[i_] != '"') {
      if (s_[i_] == '\\' && i_ + 1 < s_.size()) {
        char e = s_[++i_];
        switch (e) {
          case 'n': out += '\n'; break;
          case 't': out += '\t'; break;
          case 'u': i_ += 4; out += '?'; break;
          default: out += e;
        }
        ++i_;
      } else {
        out += s_[i_++];
      }
    }
    if (i_ >= s_.size()) fail("unterminated string");
    ++i_;
    return out;
  }
};

inline Value parse_file(const std::string& path) {
  std::ifstream f(path);
  if (!f.is_open()) throw std::runtime_error("Could not open the file: " + path);
  std::stringstream ss;
  ss << f.rdbuf();
  std::string text = ss.str();
  return Parser(text).parse();
}

}  // namespace mini_json
