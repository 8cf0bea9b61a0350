#include "json.h"

#include <cmath>
#include <cstdlib>

#include "cache_manager.h"   // Error, fail

namespace lmsf {

const Json* Json::find(const std::string& key) const {
  if (kind != kObject) return nullptr;
  for (const auto& m : members)
    if (m.first == key) return &m.second;
  return nullptr;
}

std::string Json::repr() const {
  switch (kind) {
    case kNull: return "null";
    case kBool: return boolean ? "true" : "false";
    case kNumber: return text;
    case kString: return "'" + text + "'";
    case kArray: {
      std::string s = "[";
      for (size_t i = 0; i < items.size(); ++i) s += (i ? ", " : "") + items[i].repr();
      return s + "]";
    }
    case kObject: {
      std::string s = "{";
      for (size_t i = 0; i < members.size(); ++i)
        s += (i ? ", " : "") + ("'" + members[i].first + "': ") + members[i].second.repr();
      return s + "}";
    }
  }
  return "?";
}

namespace {

struct Reader {
  const std::string& s;
  size_t at = 0;
  int depth = 0;

  [[noreturn]] void bad(const char* what) const { fail(kValueError, "not valid JSON: %s at character %zu", what, at); }
  void skip() {
    while (at < s.size() && (s[at] == ' ' || s[at] == '\t' || s[at] == '\n' || s[at] == '\r')) ++at;
  }
  bool word(const char* w) {
    const size_t n = std::char_traits<char>::length(w);
    if (s.compare(at, n, w) != 0) return false;
    at += n;
    return true;
  }
  static void utf8(unsigned cp, std::string* out) {
    if (cp < 0x80) {
      out->push_back((char)cp);
    } else if (cp < 0x800) {
      out->push_back((char)(0xC0 | (cp >> 6)));
      out->push_back((char)(0x80 | (cp & 0x3F)));
    } else if (cp < 0x10000) {
      out->push_back((char)(0xE0 | (cp >> 12)));
      out->push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
      out->push_back((char)(0x80 | (cp & 0x3F)));
    } else {
      out->push_back((char)(0xF0 | (cp >> 18)));
      out->push_back((char)(0x80 | ((cp >> 12) & 0x3F)));
      out->push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
      out->push_back((char)(0x80 | (cp & 0x3F)));
    }
  }
  unsigned hex4() {
    if (at + 4 > s.size()) bad("a short \\u escape");
    unsigned v = 0;
    for (int i = 0; i < 4; ++i) {
      const char c = s[at++];
      v <<= 4;
      if (c >= '0' && c <= '9') v |= (unsigned)(c - '0');
      else if (c >= 'a' && c <= 'f') v |= (unsigned)(c - 'a' + 10);
      else if (c >= 'A' && c <= 'F') v |= (unsigned)(c - 'A' + 10);
      else bad("a bad \\u escape");
    }
    return v;
  }
  std::string string() {
    std::string out;
    ++at;   // the opening quote
    while (true) {
      if (at >= s.size()) bad("a string without its end");
      const char c = s[at++];
      if (c == '"') return out;
      if (c != '\\') {
        out.push_back(c);
        continue;
      }
      if (at >= s.size()) bad("a string without its end");
      const char e = s[at++];
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
          unsigned cp = hex4();
          if (cp >= 0xD800 && cp < 0xDC00 && s.compare(at, 2, "\\u") == 0) {
            at += 2;
            const unsigned lo = hex4();
            cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
          }
          utf8(cp, &out);
          break;
        }
        default: bad("an unknown escape");
      }
    }
  }
  Json value() {
    if (++depth > 64) bad("nesting deeper than 64");
    skip();
    if (at >= s.size()) bad("the text ends where a value should be");
    Json v;
    const char c = s[at];
    if (c == '{') {
      v.kind = Json::kObject;
      ++at;
      skip();
      if (at < s.size() && s[at] == '}') {
        ++at;
      } else {
        while (true) {
          skip();
          if (at >= s.size() || s[at] != '"') bad("a member without a name");
          std::string key = string();
          skip();
          if (at >= s.size() || s[at] != ':') bad("a member without ':'");
          ++at;
          v.members.emplace_back(std::move(key), value());
          skip();
          if (at < s.size() && s[at] == ',') {
            ++at;
            continue;
          }
          if (at < s.size() && s[at] == '}') {
            ++at;
            break;
          }
          bad("an object without its end");
        }
      }
    } else if (c == '[') {
      v.kind = Json::kArray;
      ++at;
      skip();
      if (at < s.size() && s[at] == ']') {
        ++at;
      } else {
        while (true) {
          v.items.push_back(value());
          skip();
          if (at < s.size() && s[at] == ',') {
            ++at;
            continue;
          }
          if (at < s.size() && s[at] == ']') {
            ++at;
            break;
          }
          bad("an array without its end");
        }
      }
    } else if (c == '"') {
      v.kind = Json::kString;
      v.text = string();
    } else if (word("true")) {
      v.kind = Json::kBool;
      v.boolean = true;
    } else if (word("false")) {
      v.kind = Json::kBool;
    } else if (word("null")) {
      v.kind = Json::kNull;
    } else if (c == '-' || (c >= '0' && c <= '9')) {
      const size_t from = at;
      if (s[at] == '-') ++at;
      while (at < s.size() && ((s[at] >= '0' && s[at] <= '9') || s[at] == '.' || s[at] == 'e' || s[at] == 'E' ||
                               s[at] == '+' || s[at] == '-'))
        ++at;
      v.kind = Json::kNumber;
      v.text = s.substr(from, at - from);
      char* end = nullptr;
      v.number = std::strtod(v.text.c_str(), &end);
      if (end == v.text.c_str() || *end != 0 || !std::isfinite(v.number)) {
        at = from;
        bad("a number that cannot be read");
      }
    } else {
      bad("an unexpected character");
    }
    --depth;
    return v;
  }
};

}  // namespace

Json parse_json(const std::string& text) {
  Reader r{text};
  Json v = r.value();
  r.skip();
  if (r.at != text.size()) r.bad("text after the value");
  return v;
}

}  // namespace lmsf
