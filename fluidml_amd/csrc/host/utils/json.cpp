#include "utils/json.h"

#include <cctype>
#include <cstdlib>
#include <stdexcept>

namespace fluidml {
namespace json {
namespace {

class Parser {
 public:
  explicit Parser(const std::string &text) : s_(text) {}
  Value Document() {
    Value v = ParseValue();
    SkipSpace();
    if (pos_ != s_.size()) Fail("trailing characters");
    return v;
  }

 private:
  [[noreturn]] void Fail(const char *what) const {
    throw std::runtime_error(std::string("json: ") + what + " at byte " + std::to_string(pos_));
  }
  void SkipSpace() {
    while (pos_ < s_.size() && std::isspace(static_cast<unsigned char>(s_[pos_]))) ++pos_;
  }
  bool Eat(char c) {
    SkipSpace();
    if (pos_ < s_.size() && s_[pos_] == c) {
      ++pos_;
      return true;
    }
    return false;
  }
  void Expect(const char *word) {
    for (const char *p = word; *p; ++p) {
      if (pos_ >= s_.size() || s_[pos_] != *p) Fail("unexpected token");
      ++pos_;
    }
  }
  std::string ParseString() {
    std::string out;
    while (true) {
      if (pos_ >= s_.size()) Fail("unterminated string");
      const char c = s_[pos_++];
      if (c == '"') return out;
      if (c == '\\') {
        if (pos_ >= s_.size()) Fail("unterminated escape");
        const char e = s_[pos_++];
        switch (e) {
          case 'n': out += '\n'; break;
          case 't': out += '\t'; break;
          case 'r': out += '\r'; break;
          case 'b': out += '\b'; break;
          case 'f': out += '\f'; break;
          case 'u': {
            if (pos_ + 4 > s_.size()) Fail("short \\u escape");
            const unsigned code = static_cast<unsigned>(std::strtoul(s_.substr(pos_, 4).c_str(), nullptr, 16));
            pos_ += 4;
            if (code < 0x80) out += static_cast<char>(code);
            else out += '?';
            break;
          }
          default: out += e;
        }
      } else {
        out += c;
      }
    }
  }
  Value ParseValue() {
    SkipSpace();
    if (pos_ >= s_.size()) Fail("unexpected end");
    Value v;
    const char c = s_[pos_];
    if (c == '{') {
      ++pos_;
      v.kind = Value::Kind::Object;
      if (Eat('}')) return v;
      do {
        SkipSpace();
        if (pos_ >= s_.size() || s_[pos_] != '"') Fail("object key expected");
        ++pos_;
        std::string key = ParseString();
        if (!Eat(':')) Fail("':' expected");
        v.object[key] = ParseValue();
      } while (Eat(','));
      if (!Eat('}')) Fail("'}' expected");
    } else if (c == '[') {
      ++pos_;
      v.kind = Value::Kind::Array;
      if (Eat(']')) return v;
      do {
        v.array.push_back(ParseValue());
      } while (Eat(','));
      if (!Eat(']')) Fail("']' expected");
    } else if (c == '"') {
      ++pos_;
      v.kind = Value::Kind::String;
      v.string = ParseString();
    } else if (c == 't') {
      Expect("true");
      v.kind = Value::Kind::Bool;
      v.boolean = true;
    } else if (c == 'f') {
      Expect("false");
      v.kind = Value::Kind::Bool;
    } else if (c == 'n') {
      Expect("null");
    } else {
      char *end = nullptr;
      v.number = std::strtod(s_.c_str() + pos_, &end);
      if (end == s_.c_str() + pos_) Fail("value expected");
      pos_ = static_cast<size_t>(end - s_.c_str());
      v.kind = Value::Kind::Number;
    }
    return v;
  }
  const std::string &s_;
  size_t pos_ = 0;
};

}  // namespace

const Value &Value::At(const std::string &key) const {
  if (kind != Kind::Object) throw std::out_of_range("json: not an object while looking for '" + key + "'");
  return object.at(key);
}

Value Parse(const std::string &text) { return Parser(text).Document(); }

std::string Quote(const std::string &s) {
  std::string out = "\"";
  for (char c : s) {
    switch (c) {
      case '"': out += "\\\""; break;
      case '\\': out += "\\\\"; break;
      case '\n': out += "\\n"; break;
      case '\t': out += "\\t"; break;
      default: out += c;
    }
  }
  return out + "\"";
}

}  // namespace json
}  // namespace fluidml
