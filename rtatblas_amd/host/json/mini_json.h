// A small self-contained JSON value: enough for the plan / statistics / input files of this
// library (objects with sorted keys, arrays, strings, integers, doubles, booleans, null),
// with a parser and a pretty printer.  The reference uses nlohmann::json for the same job
// (src/methods/json_encoding.h, src/planning/planner_statistics.h:50-67); the subset of its
// interface used there — operator[], push_back, get<T>(), dump(indent), parse, == — is
// provided under the same names.
#pragma once
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <istream>
#include <iterator>
#include <map>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

namespace rtat {

class Json {
 public:
  enum class Kind { Null, Bool, Int, Real, String, Array, Object };
  using Array = std::vector<Json>;
  using Object = std::map<std::string, Json>;

  Json() = default;
  Json(std::nullptr_t) {}
  Json(bool b) : kind_(Kind::Bool), int_(b) {}
  Json(int v) : kind_(Kind::Int), int_(v) {}
  Json(long v) : kind_(Kind::Int), int_(v) {}
  Json(long long v) : kind_(Kind::Int), int_(v) {}
  Json(unsigned v) : kind_(Kind::Int), int_(v) {}
  Json(unsigned long v) : kind_(Kind::Int), int_((int64_t)v) {}
  Json(double v) : kind_(Kind::Real), real_(v) {}
  Json(float v) : kind_(Kind::Real), real_(v) {}
  Json(const char* s) : kind_(Kind::String), str_(s) {}
  Json(const std::string& s) : kind_(Kind::String), str_(s) {}
  template <typename T>
  Json(const std::vector<T>& v) : kind_(Kind::Array) {
    for (const auto& x : v) arr_.emplace_back(x);
  }
  static Json array() { Json j; j.kind_ = Kind::Array; return j; }
  static Json object() { Json j; j.kind_ = Kind::Object; return j; }

  Kind kind() const { return kind_; }
  bool is_null() const { return kind_ == Kind::Null; }
  bool is_object() const { return kind_ == Kind::Object; }
  bool is_array() const { return kind_ == Kind::Array; }
  bool is_number() const { return kind_ == Kind::Int || kind_ == Kind::Real; }
  bool is_string() const { return kind_ == Kind::String; }

  // Object member access; a null value becomes an object on first write.
  Json& operator[](const std::string& key) {
    if (kind_ == Kind::Null) kind_ = Kind::Object;
    if (kind_ != Kind::Object) throw std::runtime_error("Json: not an object");
    return obj_[key];
  }
  Json& operator[](const char* key) { return (*this)[std::string(key)]; }
  const Json& operator[](const std::string& key) const { return at(key); }
  const Json& operator[](const char* key) const { return at(std::string(key)); }
  const Json& at(const std::string& key) const {
    if (kind_ != Kind::Object) throw std::runtime_error("Json: not an object");
    auto it = obj_.find(key);
    if (it == obj_.end()) throw std::out_of_range("Json: no member \"" + key + "\"");
    return it->second;
  }
  bool contains(const std::string& key) const {
    return kind_ == Kind::Object && obj_.count(key) != 0;
  }
  // Member `key` converted to T, or `fallback` when it is absent.
  template <typename T>
  T value(const std::string& key, T fallback) const {
    return contains(key) ? at(key).get<T>() : fallback;
  }

  // Array access; a null value becomes an array on first push_back.
  void push_back(Json v) {
    if (kind_ == Kind::Null) kind_ = Kind::Array;
    if (kind_ != Kind::Array) throw std::runtime_error("Json: not an array");
    arr_.push_back(std::move(v));
  }
  const Json& operator[](size_t i) const { return items().at(i); }
  // int overloads keep a literal 0 off the const char* overload
  const Json& operator[](int i) const { return items().at((size_t)i); }
  const Json& operator[](int i) { return items().at((size_t)i); }
  const Json& operator[](size_t i) { return items().at(i); }
  size_t size() const {
    return kind_ == Kind::Array ? arr_.size() : kind_ == Kind::Object ? obj_.size() : 0;
  }
  const Array& items() const {
    if (kind_ != Kind::Array && kind_ != Kind::Null) throw std::runtime_error("Json: not an array");
    return arr_;
  }
  const Object& members() const {
    if (kind_ != Kind::Object && kind_ != Kind::Null)
      throw std::runtime_error("Json: not an object");
    return obj_;
  }
  Array::const_iterator begin() const { return items().begin(); }
  Array::const_iterator end() const { return items().end(); }

  template <typename T>
  T get() const {
    if constexpr (std::is_same_v<T, std::string>) {
      if (kind_ != Kind::String) throw std::runtime_error("Json: not a string");
      return str_;
    } else if constexpr (std::is_same_v<T, bool>) {
      if (kind_ != Kind::Bool) throw std::runtime_error("Json: not a boolean");
      return int_ != 0;
    } else if constexpr (std::is_arithmetic_v<T>) {
      if (kind_ == Kind::Int) return (T)int_;
      if (kind_ == Kind::Real) return (T)real_;
      throw std::runtime_error("Json: not a number");
    } else {
      T out;
      for (const auto& x : items()) out.push_back(x.template get<typename T::value_type>());
      return out;
    }
  }

  friend bool operator==(const Json& a, const Json& b) {
    if (a.is_number() && b.is_number()) return a.as_real() == b.as_real();
    if (a.kind_ != b.kind_) return false;
    switch (a.kind_) {
      case Kind::Null: return true;
      case Kind::Bool: return a.int_ == b.int_;
      case Kind::String: return a.str_ == b.str_;
      case Kind::Array: return a.arr_ == b.arr_;
      case Kind::Object: return a.obj_ == b.obj_;
      default: return false;
    }
  }
  friend bool operator!=(const Json& a, const Json& b) { return !(a == b); }

  // indent < 0: one line; otherwise pretty-printed with that many spaces per level.
  std::string dump(int indent = -1) const {
    std::string out;
    write(out, indent, 0);
    return out;
  }
  friend std::ostream& operator<<(std::ostream& os, const Json& j) { return os << j.dump(); }

  static Json parse(const std::string& text) {
    size_t pos = 0;
    Json v = parse_value(text, pos);
    skip_space(text, pos);
    if (pos != text.size()) fail(pos, "trailing characters");
    return v;
  }
  static Json parse(std::istream& in) {
    return parse(std::string(std::istreambuf_iterator<char>(in), std::istreambuf_iterator<char>()));
  }
  static Json parse(std::istream&& in) { return parse(in); }

 private:
  Kind kind_ = Kind::Null;
  int64_t int_ = 0;
  double real_ = 0.0;
  std::string str_;
  Array arr_;
  Object obj_;

  double as_real() const { return kind_ == Kind::Int ? (double)int_ : real_; }

  static void write_string(std::string& out, const std::string& s) {
    out += '"';
    for (unsigned char c : s) {
      switch (c) {
        case '"': out += "\\\""; break;
        case '\\': out += "\\\\"; break;
        case '\n': out += "\\n"; break;
        case '\t': out += "\\t"; break;
        case '\r': out += "\\r"; break;
        default:
          if (c < 0x20) {
            char buf[8];
            std::snprintf(buf, sizeof buf, "\\u%04x", c);
            out += buf;
          } else {
            out += (char)c;
          }
      }
    }
    out += '"';
  }
  // Shortest decimal that reads back to the same double; always looks like a real number.
  static std::string real_text(double v) {
    if (!std::isfinite(v)) return "null";
    char buf[40];
    for (int prec = 1; prec <= 17; ++prec) {
      std::snprintf(buf, sizeof buf, "%.*g", prec, v);
      if (std::strtod(buf, nullptr) == v) break;
    }
    std::string s(buf);
    if (s.find_first_of(".eEn") == std::string::npos) s += ".0";
    return s;
  }
  void write(std::string& out, int indent, int depth) const {
    const bool pretty = indent >= 0;
    auto newline = [&](int d) {
      if (pretty) {
        out += '\n';
        out.append((size_t)(indent * d), ' ');
      }
    };
    switch (kind_) {
      case Kind::Null: out += "null"; break;
      case Kind::Bool: out += int_ ? "true" : "false"; break;
      case Kind::Int: out += std::to_string(int_); break;
      case Kind::Real: out += real_text(real_); break;
      case Kind::String: write_string(out, str_); break;
      case Kind::Array:
        if (arr_.empty()) { out += "[]"; break; }
        out += '[';
        for (size_t i = 0; i < arr_.size(); ++i) {
          if (i) out += ',';
          newline(depth + 1);
          arr_[i].write(out, indent, depth + 1);
        }
        newline(depth);
        out += ']';
        break;
      case Kind::Object: {
        if (obj_.empty()) { out += "{}"; break; }
        out += '{';
        bool first = true;
        for (const auto& kv : obj_) {
          if (!first) out += ',';
          first = false;
          newline(depth + 1);
          write_string(out, kv.first);
          out += pretty ? ": " : ":";
          kv.second.write(out, indent, depth + 1);
        }
        newline(depth);
        out += '}';
        break;
      }
    }
  }

  [[noreturn]] static void fail(size_t pos, const char* what) {
    throw std::runtime_error("Json parse error at offset " + std::to_string(pos) + ": " + what);
  }
  static void skip_space(const std::string& t, size_t& p) {
    while (p < t.size() && (t[p] == ' ' || t[p] == '\n' || t[p] == '\t' || t[p] == '\r')) ++p;
  }
  static std::string parse_string(const std::string& t, size_t& p) {
    std::string s;
    ++p;  // opening quote
    while (true) {
      if (p >= t.size()) fail(p, "unterminated string");
      char c = t[p++];
      if (c == '"') return s;
      if (c != '\\') { s += c; continue; }
      if (p >= t.size()) fail(p, "unterminated escape");
      char e = t[p++];
      switch (e) {
        case '"': s += '"'; break;
        case '\\': s += '\\'; break;
        case '/': s += '/'; break;
        case 'n': s += '\n'; break;
        case 't': s += '\t'; break;
        case 'r': s += '\r'; break;
        case 'b': s += '\b'; break;
        case 'f': s += '\f'; break;
        case 'u': {
          if (p + 4 > t.size()) fail(p, "short \\u escape");
          unsigned code = (unsigned)std::strtoul(t.substr(p, 4).c_str(), nullptr, 16);
          p += 4;
          if (code < 0x80) s += (char)code;
          else if (code < 0x800) { s += (char)(0xC0 | (code >> 6)); s += (char)(0x80 | (code & 0x3F)); }
          else { s += (char)(0xE0 | (code >> 12)); s += (char)(0x80 | ((code >> 6) & 0x3F)); s += (char)(0x80 | (code & 0x3F)); }
          break;
        }
        default: fail(p, "bad escape");
      }
    }
  }
  static Json parse_value(const std::string& t, size_t& p) {
    skip_space(t, p);
    if (p >= t.size()) fail(p, "unexpected end");
    const char c = t[p];
    if (c == '{') {
      Json o = object();
      ++p;
      skip_space(t, p);
      if (p < t.size() && t[p] == '}') { ++p; return o; }
      while (true) {
        skip_space(t, p);
        if (p >= t.size() || t[p] != '"') fail(p, "expected a member name");
        std::string key = parse_string(t, p);
        skip_space(t, p);
        if (p >= t.size() || t[p] != ':') fail(p, "expected ':'");
        ++p;
        o.obj_[key] = parse_value(t, p);
        skip_space(t, p);
        if (p < t.size() && t[p] == ',') { ++p; continue; }
        if (p < t.size() && t[p] == '}') { ++p; return o; }
        fail(p, "expected ',' or '}'");
      }
    }
    if (c == '[') {
      Json a = array();
      ++p;
      skip_space(t, p);
      if (p < t.size() && t[p] == ']') { ++p; return a; }
      while (true) {
        a.arr_.push_back(parse_value(t, p));
        skip_space(t, p);
        if (p < t.size() && t[p] == ',') { ++p; continue; }
        if (p < t.size() && t[p] == ']') { ++p; return a; }
        fail(p, "expected ',' or ']'");
      }
    }
    if (c == '"') return Json(parse_string(t, p));
    if (t.compare(p, 4, "true") == 0) { p += 4; return Json(true); }
    if (t.compare(p, 5, "false") == 0) { p += 5; return Json(false); }
    if (t.compare(p, 4, "null") == 0) { p += 4; return Json(); }
    // number
    size_t q = p;
    if (q < t.size() && (t[q] == '-' || t[q] == '+')) ++q;
    bool real = false;
    while (q < t.size() && (std::isdigit((unsigned char)t[q]) || t[q] == '.' || t[q] == 'e' ||
                            t[q] == 'E' || t[q] == '-' || t[q] == '+')) {
      if (t[q] == '.' || t[q] == 'e' || t[q] == 'E') real = true;
      ++q;
    }
    if (q == p) fail(p, "unexpected character");
    const std::string num = t.substr(p, q - p);
    p = q;
    if (real) return Json(std::strtod(num.c_str(), nullptr));
    return Json((long long)std::strtoll(num.c_str(), nullptr, 10));
  }
};

}  // namespace rtat
