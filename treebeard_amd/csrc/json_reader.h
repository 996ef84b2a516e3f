// Minimal JSON DOM reader, sufficient for XGBoost model files and the
// compiler-option config files.  Numbers are converted with strtod so that
// `(float)value` equals what the reference obtains from its JSON library
// (correctly rounded double, then narrowed).
#pragma once

#include <cstdint>
#include <memory>
#include <string>
#include <utility>
#include <vector>

namespace tbamd {

class JsonValue {
public:
  enum class Kind { kNull, kBool, kNumber, kString, kArray, kNumberArray, kObject };
  Kind kind = Kind::kNull;
  bool boolean = false;
  double number = 0.0;
  std::string str;
  std::vector<JsonValue> array;
  std::vector<double> numbers; // arrays made only of numbers are kept flat
  std::vector<std::pair<std::string, JsonValue>> object;

  bool Has(const std::string &key) const;
  const JsonValue &operator[](const std::string &key) const; // throws tbamd::Error when absent
  size_t Size() const;
  // Flat view of a numeric (or empty / boolean) array.
  std::vector<double> AsNumbers() const;
  const std::string &AsString() const;
  double AsNumber() const;
};

JsonValue ParseJson(const char *begin, const char *end);
JsonValue ParseJsonFile(const std::string &path);
std::string ReadFile(const std::string &path);

} // namespace tbamd
