#include "Json.h"

#include <cerrno>
#include <cmath>
#include <cstdlib>
#include <cstring>

namespace akg {
namespace json {

bool Value::asBool() const {
  if (kind_ == Kind::Bool) return bool_;
  if (kind_ == Kind::Number) return num_ != 0.0;
  throw ParseError("json: value is not a bool");
}

double Value::asDouble() const {
  if (kind_ == Kind::Number) return num_;
  if (kind_ == Kind::Bool) return bool_ ? 1.0 : 0.0;
  throw ParseError("json: value is not a number");
}

int64_t Value::asInt() const {
  if (kind_ == Kind::Number) return isInt_ ? int_ : static_cast<int64_t>(num_);
  if (kind_ == Kind::Bool) return bool_ ? 1 : 0;
  throw ParseError("json: value is not a number");
}

const std::string &Value::asString() const {
  if (kind_ != Kind::String) throw ParseError("json: value is not a string");
  return str_;
}

size_t Value::size() const {
  if (kind_ == Kind::Array) return array_.size();
  if (kind_ == Kind::Object) return object_.size();
  return 0;
}

const Value &Value::operator[](size_t i) const {
  if (kind_ != Kind::Array) throw ParseError("json: value is not an array");
  if (i >= array_.size()) throw ParseError("json: array index " + std::to_string(i) + " out of range");
  return array_[i];
}

bool Value::contains(const std::string &key) const {
  if (kind_ != Kind::Object) return false;
  for (const auto &kv : object_) {
    if (kv.first == key) return true;
  }
  return false;
}

const Value &Value::at(const std::string &key) const {
  if (kind_ != Kind::Object) throw ParseError("json: cannot look up key '" + key + "' in a non-object");
  for (const auto &kv : object_) {
    if (kv.first == key) return kv.second;
  }
  throw ParseError("json: key '" + key + "' not found");
}

std::vector<int64_t> Value::asIntVector() const {
  std::vector<int64_t> out;
  if (kind_ == Kind::Number) {
    out.push_back(asInt());
    return out;
  }
  if (kind_ != Kind::Array) throw ParseError("json: value is not an integer list");
  out.reserve(array_.size());
  for (const auto &v : array_) out.push_back(v.asInt());
  return out;
}

std::vector<double> Value::asDoubleVector() const {
  std::vector<double> out;
  if (kind_ == Kind::Number) {
    out.push_back(num_);
    return out;
  }
  if (kind_ != Kind::Array) throw ParseError("json: value is not a number list");
  out.reserve(array_.size());
  for (const auto &v : array_) out.push_back(v.asDouble());
  return out;
}

class Parser {
 public:
  explicit Parser(const std::string &text) : s_(text.data()), n_(text.size()) {}

  Value run() {
    skipWs();
    Value v = parseValue(0);
    skipWs();
    if (pos_ != n_) fail("trailing characters after the document");
    return v;
  }

 private:
  static constexpr int kMaxDepth = 256;
  const char *s_;
  size_t n_;
  size_t pos_ = 0;

  [[noreturn]] void fail(const std::string &what) const {
    throw ParseError("json: " + what + " at byte " + std::to_string(pos_));
  }

  void skipWs() {
    while (pos_ < n_ && (s_[pos_] == ' ' || s_[pos_] == '\t' || s_[pos_] == '\n' || s_[pos_] == '\r')) ++pos_;
  }

  bool consumeWord(const char *w) {
    size_t len = std::strlen(w);
    if (pos_ + len <= n_ && std::memcmp(s_ + pos_, w, len) == 0) {
      pos_ += len;
      return true;
    }
    return false;
  }

  Value parseValue(int depth) {
    if (depth > kMaxDepth) fail("nesting too deep");
    if (pos_ >= n_) fail("unexpected end of input");
    char c = s_[pos_];
    if (c == '{') return parseObject(depth);
    if (c == '[') return parseArray(depth);
    if (c == '"') {
      Value v;
      v.kind_ = Value::Kind::String;
      v.str_ = parseString();
      return v;
    }
    if (c == 't' || c == 'f') {
      Value v;
      v.kind_ = Value::Kind::Bool;
      if (consumeWord("true")) {
        v.bool_ = true;
      } else if (consumeWord("false")) {
        v.bool_ = false;
      } else {
        fail("invalid literal");
      }
      return v;
    }
    if (c == 'n') {
      if (!consumeWord("null")) fail("invalid literal");
      return Value();
    }
    // Python's json module emits these for non-finite floats; accept them as numbers.
    if (c == 'N' && consumeWord("NaN")) return makeNumber(std::nan(""));
    if (c == 'I' && consumeWord("Infinity")) return makeNumber(HUGE_VAL);
    if (c == '-' && pos_ + 1 < n_ && s_[pos_ + 1] == 'I') {
      ++pos_;
      if (!consumeWord("Infinity")) fail("invalid literal");
      return makeNumber(-HUGE_VAL);
    }
    if (c == '-' || (c >= '0' && c <= '9')) return parseNumber();
    fail(std::string("unexpected character '") + c + "'");
  }

  static Value makeNumber(double d) {
    Value v;
    v.kind_ = Value::Kind::Number;
    v.num_ = d;
    v.isInt_ = false;
    return v;
  }

  Value parseNumber() {
    size_t start = pos_;
    bool isInt = true;
    if (s_[pos_] == '-') ++pos_;
    if (pos_ >= n_ || s_[pos_] < '0' || s_[pos_] > '9') fail("malformed number");
    while (pos_ < n_ && s_[pos_] >= '0' && s_[pos_] <= '9') ++pos_;
    if (pos_ < n_ && s_[pos_] == '.') {
      isInt = false;
      ++pos_;
      if (pos_ >= n_ || s_[pos_] < '0' || s_[pos_] > '9') fail("malformed fraction");
      while (pos_ < n_ && s_[pos_] >= '0' && s_[pos_] <= '9') ++pos_;
    }
    if (pos_ < n_ && (s_[pos_] == 'e' || s_[pos_] == 'E')) {
      isInt = false;
      ++pos_;
      if (pos_ < n_ && (s_[pos_] == '+' || s_[pos_] == '-')) ++pos_;
      if (pos_ >= n_ || s_[pos_] < '0' || s_[pos_] > '9') fail("malformed exponent");
      while (pos_ < n_ && s_[pos_] >= '0' && s_[pos_] <= '9') ++pos_;
    }
    std::string tok(s_ + start, pos_ - start);
    Value v;
    v.kind_ = Value::Kind::Number;
    v.num_ = std::strtod(tok.c_str(), nullptr);
    if (isInt) {
      errno = 0;
      long long ll = std::strtoll(tok.c_str(), nullptr, 10);
      if (errno == 0) {
        v.isInt_ = true;
        v.int_ = ll;
      }
    }
    return v;
  }

  static void appendUtf8(std::string *out, uint32_t cp) {
    if (cp < 0x80) {
      out->push_back(static_cast<char>(cp));
    } else if (cp < 0x800) {
      out->push_back(static_cast<char>(0xC0 | (cp >> 6)));
      out->push_back(static_cast<char>(0x80 | (cp & 0x3F)));
    } else if (cp < 0x10000) {
      out->push_back(static_cast<char>(0xE0 | (cp >> 12)));
      out->push_back(static_cast<char>(0x80 | ((cp >> 6) & 0x3F)));
      out->push_back(static_cast<char>(0x80 | (cp & 0x3F)));
    } else {
      out->push_back(static_cast<char>(0xF0 | (cp >> 18)));
      out->push_back(static_cast<char>(0x80 | ((cp >> 12) & 0x3F)));
      out->push_back(static_cast<char>(0x80 | ((cp >> 6) & 0x3F)));
      out->push_back(static_cast<char>(0x80 | (cp & 0x3F)));
    }
  }

  uint32_t parseHex4() {
    if (pos_ + 4 > n_) fail("truncated \\u escape");
    uint32_t v = 0;
    for (int i = 0; i < 4; ++i) {
      char c = s_[pos_++];
      v <<= 4;
      if (c >= '0' && c <= '9') {
        v |= static_cast<uint32_t>(c - '0');
      } else if (c >= 'a' && c <= 'f') {
        v |= static_cast<uint32_t>(c - 'a' + 10);
      } else if (c >= 'A' && c <= 'F') {
        v |= static_cast<uint32_t>(c - 'A' + 10);
      } else {
        fail("bad hex digit in \\u escape");
      }
    }
    return v;
  }

  std::string parseString() {
    ++pos_;  // opening quote
    std::string out;
    while (true) {
      if (pos_ >= n_) fail("unterminated string");
      char c = s_[pos_++];
      if (c == '"') break;
      if (static_cast<unsigned char>(c) < 0x20) fail("control character in string");
      if (c != '\\') {
        out.push_back(c);
        continue;
      }
      if (pos_ >= n_) fail("unterminated escape");
      char e = s_[pos_++];
      switch (e) {
        case '"': out.push_back('"'); break;
        case '\\': out.push_back('\\'); break;
        case '/': out.push_back('/'); break;
        case 'b': out.push_back('\b'); break;
        case 'f': out.push_back('\f'); break;
        case 'n': out.push_back('\n'); break;
        case 'r': out.push_back('\r'); break;
        case 't': out.push_back('\t'); break;
        case 'u': {
          uint32_t cp = parseHex4();
          if (cp >= 0xD800 && cp <= 0xDBFF && pos_ + 1 < n_ && s_[pos_] == '\\' && s_[pos_ + 1] == 'u') {
            pos_ += 2;
            uint32_t lo = parseHex4();
            if (lo >= 0xDC00 && lo <= 0xDFFF) {
              cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
            } else {
              fail("unpaired surrogate");
            }
          }
          appendUtf8(&out, cp);
          break;
        }
        default: fail("unknown escape");
      }
    }
    return out;
  }

  Value parseArray(int depth) {
    ++pos_;
    Value v;
    v.kind_ = Value::Kind::Array;
    skipWs();
    if (pos_ < n_ && s_[pos_] == ']') {
      ++pos_;
      return v;
    }
    while (true) {
      skipWs();
      v.array_.push_back(parseValue(depth + 1));
      skipWs();
      if (pos_ >= n_) fail("unterminated array");
      if (s_[pos_] == ',') {
        ++pos_;
        continue;
      }
      if (s_[pos_] == ']') {
        ++pos_;
        break;
      }
      fail("expected ',' or ']'");
    }
    return v;
  }

  Value parseObject(int depth) {
    ++pos_;
    Value v;
    v.kind_ = Value::Kind::Object;
    skipWs();
    if (pos_ < n_ && s_[pos_] == '}') {
      ++pos_;
      return v;
    }
    while (true) {
      skipWs();
      if (pos_ >= n_ || s_[pos_] != '"') fail("expected a string key");
      std::string key = parseString();
      skipWs();
      if (pos_ >= n_ || s_[pos_] != ':') fail("expected ':'");
      ++pos_;
      skipWs();
      Value member = parseValue(depth + 1);
      // Duplicate keys: the last one wins, as in nlohmann::json.
      bool replaced = false;
      for (auto &kv : v.object_) {
        if (kv.first == key) {
          kv.second = std::move(member);
          replaced = true;
          break;
        }
      }
      if (!replaced) v.object_.emplace_back(std::move(key), std::move(member));
      skipWs();
      if (pos_ >= n_) fail("unterminated object");
      if (s_[pos_] == ',') {
        ++pos_;
        continue;
      }
      if (s_[pos_] == '}') {
        ++pos_;
        break;
      }
      fail("expected ',' or '}'");
    }
    return v;
  }
};

Value Value::parse(const std::string &text) { return Parser(text).run(); }

}  // namespace json
}  // namespace akg
