// A small JSON reader and writer for config.json, generation_config.json, the safetensors header and
// the engine's own output lines.  Numbers are kept as double and as the text they were written with
// (an integer beyond 2^53 is read from the text).
#pragma once
#include <cstdint>
#include <cstdlib>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace vosti {

struct JsonError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

class Json {
 public:
  enum Kind { Null, Bool, Number, String, Array, Object };
  Kind kind = Null;
  bool boolean = false;
  double number = 0.0;
  std::string text;                           // a string's value, or a number as written
  std::vector<Json> items;                    // Array
  std::vector<std::pair<std::string, Json>> members;   // Object, in file order

  bool is_null() const { return kind == Null; }
  bool is_int() const { return kind == Number && text.find_first_of(".eE") == std::string::npos; }
  int64_t as_int() const { return std::strtoll(text.c_str(), nullptr, 10); }
  const Json* find(const std::string& key) const {
    if (kind != Object) return nullptr;
    for (const auto& m : members)
      if (m.first == key) return &m.second;
    return nullptr;
  }
  // A member that is present and not null, else nullptr.
  const Json* get(const std::string& key) const {
    const Json* j = find(key);
    return (j && !j->is_null()) ? j : nullptr;
  }

  static Json parse(const std::string& s) {
    size_t i = 0;
    Json j = value(s, i);
    skip(s, i);
    if (i != s.size()) throw JsonError("trailing characters after the JSON value");
    return j;
  }

 private:
  static void skip(const std::string& s, size_t& i) {
    while (i < s.size() && (s[i] == ' ' || s[i] == '\n' || s[i] == '\t' || s[i] == '\r')) ++i;
  }
  static Json value(const std::string& s, size_t& i) {
    skip(s, i);
    if (i >= s.size()) throw JsonError("unexpected end of JSON");
    Json j;
    const char c = s[i];
    if (c == '{') {
      j.kind = Object;
      ++i;
      skip(s, i);
      if (i < s.size() && s[i] == '}') { ++i; return j; }
      for (;;) {
        skip(s, i);
        if (i >= s.size() || s[i] != '"') throw JsonError("expected a member name");
        std::string key = string(s, i);
        skip(s, i);
        if (i >= s.size() || s[i] != ':') throw JsonError("expected ':' after a member name");
        ++i;
        j.members.emplace_back(std::move(key), value(s, i));
        skip(s, i);
        if (i < s.size() && s[i] == ',') { ++i; continue; }
        if (i < s.size() && s[i] == '}') { ++i; return j; }
        throw JsonError("expected ',' or '}' in an object");
      }
    }
    if (c == '[') {
      j.kind = Array;
      ++i;
      skip(s, i);
      if (i < s.size() && s[i] == ']') { ++i; return j; }
      for (;;) {
        j.items.push_back(value(s, i));
        skip(s, i);
        if (i < s.size() && s[i] == ',') { ++i; continue; }
        if (i < s.size() && s[i] == ']') { ++i; return j; }
        throw JsonError("expected ',' or ']' in an array");
      }
    }
    if (c == '"') {
      j.kind = String;
      j.text = string(s, i);
      return j;
    }
    if (s.compare(i, 4, "true") == 0) { j.kind = Bool; j.boolean = true; i += 4; return j; }
    if (s.compare(i, 5, "false") == 0) { j.kind = Bool; i += 5; return j; }
    if (s.compare(i, 4, "null") == 0) { i += 4; return j; }
    if (s.compare(i, 3, "NaN") == 0 || s.compare(i, 8, "Infinity") == 0 || s.compare(i, 9, "-Infinity") == 0)
      throw JsonError("a number that is not finite");
    const size_t b = i;
    while (i < s.size() && (std::string("+-0123456789.eE").find(s[i]) != std::string::npos)) ++i;
    if (i == b) throw JsonError(std::string("unexpected character '") + c + "'");
    j.kind = Number;
    j.text = s.substr(b, i - b);
    char* end = nullptr;
    j.number = std::strtod(j.text.c_str(), &end);
    if (end == j.text.c_str() || *end != 0) throw JsonError("malformed number " + j.text);
    return j;
  }
  static std::string string(const std::string& s, size_t& i) {
    std::string out;
    ++i;                                       // the opening quote
    while (i < s.size() && s[i] != '"') {
      if (s[i] == '\\') {
        if (++i >= s.size()) break;
        switch (s[i]) {
          case 'n': out += '\n'; break;
          case 't': out += '\t'; break;
          case 'r': out += '\r'; break;
          case 'b': out += '\b'; break;
          case 'f': out += '\f'; break;
          case 'u': {                          // kept as UTF-8 for the basic plane; enough for tensor names
            if (i + 4 >= s.size()) throw JsonError("short \\u escape");
            const unsigned cp = (unsigned)std::strtoul(s.substr(i + 1, 4).c_str(), nullptr, 16);
            i += 4;
            if (cp < 0x80) out += (char)cp;
            else if (cp < 0x800) { out += (char)(0xC0 | (cp >> 6)); out += (char)(0x80 | (cp & 0x3F)); }
            else { out += (char)(0xE0 | (cp >> 12)); out += (char)(0x80 | ((cp >> 6) & 0x3F)); out += (char)(0x80 | (cp & 0x3F)); }
            break;
          }
          default: out += s[i];
        }
        ++i;
      } else {
        out += s[i++];
      }
    }
    if (i >= s.size()) throw JsonError("unterminated string");
    ++i;
    return out;
  }
};

}  // namespace vosti
