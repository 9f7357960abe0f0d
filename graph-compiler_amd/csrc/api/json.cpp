#include "json.h"

#include <cerrno>
#include <cstdlib>
#include <stdexcept>

namespace gcapi {
namespace {
struct Parser {
  const std::string &s;
  size_t i = 0;
  int depth = 0;
  explicit Parser(const std::string &t) : s(t) {}
  [[noreturn]] void fail(const char *m) const {
    throw std::invalid_argument(std::string("JSON: ") + m + " at offset " + std::to_string(i));
  }
  void ws() {
    while (i < s.size() && (s[i] == ' ' || s[i] == '\t' || s[i] == '\n' || s[i] == '\r'))
      i++;
  }
  bool eat(char c) {
    ws();
    if (i < s.size() && s[i] == c) {
      i++;
      return true;
    }
    return false;
  }
  std::string str() {
    if (!eat('"'))
      fail("string expected");
    std::string o;
    while (i < s.size() && s[i] != '"') {
      char c = s[i++];
      if (c == '\\') {
        if (i >= s.size())
          fail("bad escape");
        char e = s[i++];
        switch (e) {
        case 'n': o += '\n'; break;
        case 't': o += '\t'; break;
        case 'r': o += '\r'; break;
        case 'b': o += '\b'; break;
        case 'f': o += '\f'; break;
        case 'u': {
          if (i + 4 > s.size())
            fail("bad \\u escape");
          unsigned v = (unsigned)strtoul(s.substr(i, 4).c_str(), nullptr, 16);
          i += 4;
          if (v < 0x80)
            o += (char)v;
          else if (v < 0x800) {
            o += (char)(0xC0 | (v >> 6));
            o += (char)(0x80 | (v & 0x3F));
          } else {
            o += (char)(0xE0 | (v >> 12));
            o += (char)(0x80 | ((v >> 6) & 0x3F));
            o += (char)(0x80 | (v & 0x3F));
          }
          break;
        }
        default: o += e; break; // \" \\ \/
        }
      } else {
        o += c;
      }
    }
    if (i >= s.size())
      fail("unterminated string");
    i++;
    return o;
  }
  JValue value() {
    if (++depth > 64)
      fail("nesting too deep");
    ws();
    if (i >= s.size())
      fail("value expected");
    JValue v;
    char c = s[i];
    if (c == '{') {
      i++;
      v.type = JValue::Obj;
      if (!eat('}')) {
        do {
          std::string k = str();
          if (!eat(':'))
            fail("':' expected");
          v.obj.emplace_back(std::move(k), value());
        } while (eat(','));
        if (!eat('}'))
          fail("'}' expected");
      }
    } else if (c == '[') {
      i++;
      v.type = JValue::Arr;
      if (!eat(']')) {
        do {
          v.arr.push_back(value());
        } while (eat(','));
        if (!eat(']'))
          fail("']' expected");
      }
    } else if (c == '"') {
      v.type = JValue::Str;
      v.str = str();
    } else if (s.compare(i, 4, "true") == 0) {
      v.type = JValue::Bool, v.b = true, i += 4;
    } else if (s.compare(i, 5, "false") == 0) {
      v.type = JValue::Bool, v.b = false, i += 5;
    } else if (s.compare(i, 4, "null") == 0) {
      i += 4;
    } else if (c == '-' || (c >= '0' && c <= '9')) {
      size_t j = i;
      bool integral = true;
      if (s[j] == '-')
        j++;
      while (j < s.size() && ((s[j] >= '0' && s[j] <= '9') || s[j] == '.' || s[j] == 'e' || s[j] == 'E' ||
                              s[j] == '+' || s[j] == '-')) {
        if (s[j] == '.' || s[j] == 'e' || s[j] == 'E')
          integral = false;
        j++;
      }
      std::string t = s.substr(i, j - i);
      v.type = JValue::Num;
      char *end = nullptr;
      v.num = strtod(t.c_str(), &end);
      if (end == t.c_str())
        fail("bad number");
      if (integral) {
        errno = 0;
        long long ll = strtoll(t.c_str(), nullptr, 10);
        if (errno == 0) {
          v.inum = ll;
          v.is_int = true;
        }
      }
      if (!v.is_int)
        v.inum = (int64_t)v.num;
      i = j;
    } else {
      fail("unexpected character");
    }
    depth--;
    return v;
  }
};
} // namespace

JValue parse_json(const std::string &text) {
  Parser p(text);
  JValue v = p.value();
  p.ws();
  if (p.i != text.size())
    p.fail("trailing characters");
  return v;
}

} // namespace gcapi
