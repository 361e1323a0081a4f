// A small JSON reader for the two places the convolution API takes JSON: the
// ConvParams stream reader and the planConstraints option.  Objects keep
// their members in document order.
#ifndef poplibs_amd_Json_hpp
#define poplibs_amd_Json_hpp
#include <cctype>
#include <cstdlib>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace poplibs_amd {
namespace json {

struct ParseError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

struct Value {
  enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
  bool boolean = false;
  double number = 0;
  std::string text; // string contents, or the literal text of a number
  std::vector<Value> items;
  std::vector<std::pair<std::string, Value>> members;

  bool isObject() const { return kind == Object; }
  bool isArray() const { return kind == Array; }
  const Value *find(const std::string &key) const {
    for (const auto &m : members)
      if (m.first == key)
        return &m.second;
    return nullptr;
  }
  /// Non-negative integer value; accepts numbers and numeric strings (the
  /// property-tree reader PopLibs uses stores every scalar as text).
  bool asUnsigned(unsigned long long &out) const {
    if (kind != Number && kind != String)
      return false;
    if (text.empty())
      return false;
    char *end = nullptr;
    const char *s = text.c_str();
    if (*s == '-')
      return false;
    unsigned long long v = std::strtoull(s, &end, 10);
    if (*end != '\0')
      return false;
    out = v;
    return true;
  }
  bool asBool(bool &out) const {
    if (kind == Bool) {
      out = boolean;
      return true;
    }
    if (kind == Number || kind == String) {
      if (text == "1" || text == "true") {
        out = true;
        return true;
      }
      if (text == "0" || text == "false") {
        out = false;
        return true;
      }
    }
    return false;
  }
};

class Parser {
  const std::string &s_;
  std::size_t pos_ = 0;

  [[noreturn]] void fail(const std::string &what) const {
    throw ParseError("JSON parse error at offset " + std::to_string(pos_) +
                     ": " + what);
  }
  void skipSpace() {
    while (pos_ < s_.size() && std::isspace((unsigned char)s_[pos_]))
      ++pos_;
  }
  bool consume(char c) {
    skipSpace();
    if (pos_ < s_.size() && s_[pos_] == c) {
      ++pos_;
      return true;
    }
    return false;
  }
  void expect(char c) {
    if (!consume(c))
      fail(std::string("expected '") + c + "'");
  }
  std::string parseString() {
    expect('"');
    std::string out;
    while (true) {
      if (pos_ >= s_.size())
        fail("unterminated string");
      char c = s_[pos_++];
      if (c == '"')
        break;
      if (c == '\\') {
        if (pos_ >= s_.size())
          fail("unterminated escape");
        char e = s_[pos_++];
        switch (e) {
        case 'n': out += '\n'; break;
        case 't': out += '\t'; break;
        case 'r': out += '\r'; break;
        case 'b': out += '\b'; break;
        case 'f': out += '\f'; break;
        case 'u': {
          if (pos_ + 4 > s_.size())
            fail("short \\u escape");
          unsigned code = (unsigned)std::strtoul(s_.substr(pos_, 4).c_str(),
                                                 nullptr, 16);
          pos_ += 4;
          if (code < 0x80)
            out += (char)code;
          else
            out += '?';
          break;
        }
        default: out += e; break;
        }
      } else {
        out += c;
      }
    }
    return out;
  }
  Value parseValue(int depth) {
    if (depth > 64)
      fail("nesting too deep");
    skipSpace();
    if (pos_ >= s_.size())
      fail("unexpected end of input");
    Value v;
    char c = s_[pos_];
    if (c == '{') {
      ++pos_;
      v.kind = Value::Object;
      if (consume('}'))
        return v;
      do {
        skipSpace();
        std::string key = parseString();
        expect(':');
        v.members.emplace_back(std::move(key), parseValue(depth + 1));
      } while (consume(','));
      expect('}');
    } else if (c == '[') {
      ++pos_;
      v.kind = Value::Array;
      if (consume(']'))
        return v;
      do {
        v.items.push_back(parseValue(depth + 1));
      } while (consume(','));
      expect(']');
    } else if (c == '"') {
      v.kind = Value::String;
      v.text = parseString();
    } else if (s_.compare(pos_, 4, "true") == 0) {
      pos_ += 4;
      v.kind = Value::Bool;
      v.boolean = true;
      v.text = "true";
    } else if (s_.compare(pos_, 5, "false") == 0) {
      pos_ += 5;
      v.kind = Value::Bool;
      v.text = "false";
    } else if (s_.compare(pos_, 4, "null") == 0) {
      pos_ += 4;
    } else if (c == '-' || std::isdigit((unsigned char)c)) {
      std::size_t start = pos_;
      if (c == '-')
        ++pos_;
      while (pos_ < s_.size() &&
             (std::isdigit((unsigned char)s_[pos_]) || s_[pos_] == '.' ||
              s_[pos_] == 'e' || s_[pos_] == 'E' || s_[pos_] == '+' ||
              s_[pos_] == '-'))
        ++pos_;
      v.kind = Value::Number;
      v.text = s_.substr(start, pos_ - start);
      char *end = nullptr;
      v.number = std::strtod(v.text.c_str(), &end);
      if (*end != '\0')
        fail("malformed number '" + v.text + "'");
    } else {
      fail(std::string("unexpected character '") + c + "'");
    }
    return v;
  }

public:
  explicit Parser(const std::string &s) : s_(s) {}
  Value parseDocument() {
    Value v = parseValue(0);
    skipSpace();
    if (pos_ != s_.size())
      fail("trailing characters");
    return v;
  }
};

inline Value parse(const std::string &text) {
  return Parser(text).parseDocument();
}

} // namespace json
} // namespace poplibs_amd
#endif
