// A minimal JSON value, reader and writer: what the tuner's trial logs and records need
// (objects keep insertion order so that saved records diff cleanly).
#pragma once
#include <cerrno>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <optional>
#include <string>
#include <utility>
#include <vector>

namespace cutile {
namespace json {

struct Value {
  enum class Kind { Null, Bool, Int, Float, String, Array, Object };
  Kind kind = Kind::Null;
  bool b = false;
  int64_t i = 0;
  double f = 0.0;
  std::string s;
  std::vector<Value> items;
  std::vector<std::pair<std::string, Value>> fields;

  static Value null() { return Value{}; }
  static Value boolean(bool v) { Value x; x.kind = Kind::Bool; x.b = v; return x; }
  static Value integer(int64_t v) { Value x; x.kind = Kind::Int; x.i = v; return x; }
  static Value number(double v) { Value x; x.kind = Kind::Float; x.f = v; return x; }
  static Value string(std::string v) { Value x; x.kind = Kind::String; x.s = std::move(v); return x; }
  static Value array() { Value x; x.kind = Kind::Array; return x; }
  static Value object() { Value x; x.kind = Kind::Object; return x; }

  bool is_null() const { return kind == Kind::Null; }
  bool is_string() const { return kind == Kind::String; }
  bool is_number() const { return kind == Kind::Int || kind == Kind::Float; }
  bool is_object() const { return kind == Kind::Object; }
  bool is_array() const { return kind == Kind::Array; }
  double as_double() const { return kind == Kind::Int ? (double)i : f; }

  Value& set(const std::string& key, Value v) {
    for (auto& kv : fields)
      if (kv.first == key) { kv.second = std::move(v); return *this; }
    fields.emplace_back(key, std::move(v));
    return *this;
  }
  const Value* get(const std::string& key) const {
    if (kind != Kind::Object) return nullptr;
    for (auto& kv : fields)
      if (kv.first == key) return &kv.second;
    return nullptr;
  }
};

inline std::string quote(const std::string& s) {
  std::string out = "\"";
  for (unsigned char c : s) {
    switch (c) {
      case '"': out += "\\\""; break;
      case '\\': out += "\\\\"; break;
      case '\n': out += "\\n"; break;
      case '\r': out += "\\r"; break;
      case '\t': out += "\\t"; break;
      case '\b': out += "\\b"; break;
      case '\f': out += "\\f"; break;
      default:
        if (c < 0x20) { char buf[8]; snprintf(buf, sizeof(buf), "\\u%04x", c); out += buf; }
        else out += (char)c;
    }
  }
  return out + "\"";
}

// Shortest decimal text that reads back to the same f32 (timings are stored as f32).
inline std::string float_text(double v) {
  if (!std::isfinite(v)) return "null";   // JSON has no NaN / infinity
  char buf[40];
  for (int prec = 1; prec <= 9; ++prec) {
    snprintf(buf, sizeof(buf), "%.*g", prec, v);
    if ((float)strtod(buf, nullptr) == (float)v) break;
  }
  std::string t = buf;
  if (t.find_first_of(".eEn") == std::string::npos) t += ".0";
  return t;
}

inline void dump_to(const Value& v, bool pretty, int depth, std::string* out) {
  auto newline = [&](int d) { if (pretty) { *out += "\n"; out->append((size_t)d * 2, ' '); } };
  switch (v.kind) {
    case Value::Kind::Null: *out += "null"; break;
    case Value::Kind::Bool: *out += v.b ? "true" : "false"; break;
    case Value::Kind::Int: *out += std::to_string(v.i); break;
    case Value::Kind::Float: *out += float_text(v.f); break;
    case Value::Kind::String: *out += quote(v.s); break;
    case Value::Kind::Array:
      *out += "[";
      for (size_t k = 0; k < v.items.size(); ++k) {
        if (k) *out += ",";
        newline(depth + 1);
        dump_to(v.items[k], pretty, depth + 1, out);
      }
      if (!v.items.empty()) newline(depth);
      *out += "]";
      break;
    case Value::Kind::Object:
      *out += "{";
      for (size_t k = 0; k < v.fields.size(); ++k) {
        if (k) *out += ",";
        newline(depth + 1);
        *out += quote(v.fields[k].first) + (pretty ? ": " : ":");
        dump_to(v.fields[k].second, pretty, depth + 1, out);
      }
      if (!v.fields.empty()) newline(depth);
      *out += "}";
      break;
  }
}
inline std::string dump(const Value& v, bool pretty = false) {
  std::string out;
  dump_to(v, pretty, 0, &out);
  return out;
}

class Reader {
 public:
  explicit Reader(const std::string& text) : t_(text) {}
  std::optional<Value> document() {
    Value v;
    if (!value(&v)) return std::nullopt;
    space();
    if (p_ != t_.size()) return std::nullopt;
    return v;
  }

 private:
  void space() { while (p_ < t_.size() && (t_[p_] == ' ' || t_[p_] == '\n' || t_[p_] == '\t' || t_[p_] == '\r')) ++p_; }
  bool literal(const char* w) {
    size_t n = std::char_traits<char>::length(w);
    if (t_.compare(p_, n, w) != 0) return false;
    p_ += n;
    return true;
  }
  bool string(std::string* out) {
    if (p_ >= t_.size() || t_[p_] != '"') return false;
    ++p_;
    while (p_ < t_.size()) {
      char c = t_[p_++];
      if (c == '"') return true;
      if (c != '\\') { *out += c; continue; }
      if (p_ >= t_.size()) return false;
      char e = t_[p_++];
      switch (e) {
        case '"': *out += '"'; break;
        case '\\': *out += '\\'; break;
        case '/': *out += '/'; break;
        case 'n': *out += '\n'; break;
        case 'r': *out += '\r'; break;
        case 't': *out += '\t'; break;
        case 'b': *out += '\b'; break;
        case 'f': *out += '\f'; break;
        case 'u': {
          if (p_ + 4 > t_.size()) return false;
          unsigned cp = (unsigned)strtoul(t_.substr(p_, 4).c_str(), nullptr, 16);
          p_ += 4;
          if (cp < 0x80) *out += (char)cp;
          else if (cp < 0x800) { *out += (char)(0xC0 | (cp >> 6)); *out += (char)(0x80 | (cp & 0x3F)); }
          else { *out += (char)(0xE0 | (cp >> 12)); *out += (char)(0x80 | ((cp >> 6) & 0x3F)); *out += (char)(0x80 | (cp & 0x3F)); }
          break;
        }
        default: return false;
      }
    }
    return false;   // unterminated: a torn line
  }
  // Nesting deeper than any record or log line this library writes (they nest three levels) is refused: a corrupted
  // or hostile file must not be able to overflow the stack through the recursion below.
  static constexpr int kMaxDepth = 64;
  struct DepthGuard {
    int& d;
    explicit DepthGuard(int& depth) : d(depth) { ++d; }
    ~DepthGuard() { --d; }
  };
  bool value(Value* out) {
    DepthGuard guard(depth_);
    if (depth_ > kMaxDepth) return false;
    space();
    if (p_ >= t_.size()) return false;
    char c = t_[p_];
    if (c == '{') {
      ++p_;
      *out = Value::object();
      space();
      if (p_ < t_.size() && t_[p_] == '}') { ++p_; return true; }
      while (true) {
        space();
        std::string key;
        if (!string(&key)) return false;
        space();
        if (p_ >= t_.size() || t_[p_++] != ':') return false;
        Value v;
        if (!value(&v)) return false;
        out->fields.emplace_back(std::move(key), std::move(v));
        space();
        if (p_ >= t_.size()) return false;
        if (t_[p_] == ',') { ++p_; continue; }
        if (t_[p_] == '}') { ++p_; return true; }
        return false;
      }
    }
    if (c == '[') {
      ++p_;
      *out = Value::array();
      space();
      if (p_ < t_.size() && t_[p_] == ']') { ++p_; return true; }
      while (true) {
        Value v;
        if (!value(&v)) return false;
        out->items.push_back(std::move(v));
        space();
        if (p_ >= t_.size()) return false;
        if (t_[p_] == ',') { ++p_; continue; }
        if (t_[p_] == ']') { ++p_; return true; }
        return false;
      }
    }
    if (c == '"') { *out = Value::string(""); return string(&out->s); }
    if (literal("null")) { *out = Value::null(); return true; }
    if (literal("true")) { *out = Value::boolean(true); return true; }
    if (literal("false")) { *out = Value::boolean(false); return true; }
    size_t start = p_;
    bool is_float = false;
    if (t_[p_] == '-') ++p_;
    while (p_ < t_.size() && (isdigit((unsigned char)t_[p_]) || t_[p_] == '.' || t_[p_] == 'e' || t_[p_] == 'E' || t_[p_] == '+' || t_[p_] == '-')) {
      if (t_[p_] == '.' || t_[p_] == 'e' || t_[p_] == 'E') is_float = true;
      ++p_;
    }
    if (p_ == start) return false;
    // The scan above takes any run of number characters; the conversion must consume all of it, or the token is
    // not a number ("1-2", "--", "1e", "1.2.3") and the document is refused like any other torn text.
    std::string num = t_.substr(start, p_ - start);
    if (!(num[0] == '-' || isdigit((unsigned char)num[0]))) return false;   // JSON numbers do not start with '+' or '.'
    char* end = nullptr;
    errno = 0;
    if (is_float) {
      const double v = strtod(num.c_str(), &end);
      if (end != num.c_str() + num.size() || !isdigit((unsigned char)num.back())) return false;
      *out = Value::number(v);
    } else {
      const long long v = strtoll(num.c_str(), &end, 10);
      if (end != num.c_str() + num.size() || errno == ERANGE || !isdigit((unsigned char)num.back())) return false;
      *out = Value::integer(v);
    }
    return true;
  }
  const std::string& t_;
  size_t p_ = 0;
  int depth_ = 0;
};

inline std::optional<Value> parse(const std::string& text) { return Reader(text).document(); }

}  // namespace json
}  // namespace cutile
