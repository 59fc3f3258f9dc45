/**
 * Minimal JSON document model and recursive-descent reader used by the op-description translator.
 *
 * The reference reads MindSpore graph-kernel descriptions with nlohmann::json
 * (akg-mlir/lib/Target/MindsporeDialect/TranslateToMindsporeDialect.cpp:46,295-316). That library is a
 * third-party dependency; this reader implements just what the translator needs: objects keep insertion
 * order, numbers remember whether they were written as integers, `null` is a first-class value (per-op
 * "attr" is frequently null in real descriptions).
 */
#ifndef AKG_HIP_JSON_H_
#define AKG_HIP_JSON_H_

#include <cstdint>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace akg {
namespace json {

class ParseError : public std::runtime_error {
 public:
  explicit ParseError(const std::string &msg) : std::runtime_error(msg) {}
};

class Value {
 public:
  enum class Kind { Null, Bool, Number, String, Array, Object };

  Value() = default;

  Kind kind() const { return kind_; }
  bool isNull() const { return kind_ == Kind::Null; }
  bool isBool() const { return kind_ == Kind::Bool; }
  bool isNumber() const { return kind_ == Kind::Number; }
  bool isInteger() const { return kind_ == Kind::Number && isInt_; }
  bool isString() const { return kind_ == Kind::String; }
  bool isArray() const { return kind_ == Kind::Array; }
  bool isObject() const { return kind_ == Kind::Object; }

  bool asBool() const;
  double asDouble() const;
  int64_t asInt() const;
  const std::string &asString() const;

  // Array / object size; 0 for scalars and null (iteration over a null "attr" must be a no-op).
  size_t size() const;
  const Value &operator[](size_t i) const;

  bool contains(const std::string &key) const;
  // Throws ParseError naming the key when it is absent (mirrors nlohmann's at()).
  const Value &at(const std::string &key) const;
  const std::vector<std::pair<std::string, Value>> &members() const { return object_; }
  const std::vector<Value> &elements() const { return array_; }

  std::vector<int64_t> asIntVector() const;
  std::vector<double> asDoubleVector() const;

  static Value parse(const std::string &text);

 private:
  friend class Parser;
  Kind kind_ = Kind::Null;
  bool bool_ = false;
  bool isInt_ = false;
  double num_ = 0.0;
  int64_t int_ = 0;
  std::string str_;
  std::vector<Value> array_;
  std::vector<std::pair<std::string, Value>> object_;
};

}  // namespace json
}  // namespace akg

#endif  // AKG_HIP_JSON_H_
