// A small JSON value with a strict parser: enough to read back the cost tables
// and layout plans this backend writes (the reference uses nlohmann::json,
// which is not available offline).
#ifndef FLUIDML_AMD_HOST_UTILS_JSON_H_
#define FLUIDML_AMD_HOST_UTILS_JSON_H_

#include <map>
#include <string>
#include <vector>

namespace fluidml {
namespace json {

struct Value {
  enum class Kind { Null, Bool, Number, String, Array, Object };
  Kind kind = Kind::Null;
  bool boolean = false;
  double number = 0;
  std::string string;
  std::vector<Value> array;
  std::map<std::string, Value> object;

  bool Has(const std::string &key) const { return kind == Kind::Object && object.count(key) > 0; }
  const Value &At(const std::string &key) const;  // throws std::out_of_range
};

Value Parse(const std::string &text);  // throws std::runtime_error with the byte offset
std::string Quote(const std::string &s);

}  // namespace json
}  // namespace fluidml

#endif
