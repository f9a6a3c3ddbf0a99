// The JSON value of inference.h: a recursive-descent reader and a writer.  It serves config.json,
// the header of a safetensors file and the parameters of parts; the reference has a reader of the
// same subset for its server (/root/reference/src/json.h:14-21).
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../include/inference.h"

namespace tinyinfer {

namespace {
struct Reader {
  const std::string& s;
  size_t i = 0;
  explicit Reader(const std::string& s) : s(s) {}

  [[noreturn]] void fail(const char* what) const {
    throw Error("JSON: " + std::string(what) + " at offset " + std::to_string(i));
  }
  void skip() {
    while (i < s.size() && (s[i] == ' ' || s[i] == '\n' || s[i] == '\t' || s[i] == '\r')) ++i;
  }
  bool take(const char* word) {
    const size_t n = strlen(word);
    if (s.compare(i, n, word) == 0) {
      i += n;
      return true;
    }
    return false;
  }
  static void utf8(std::string& out, unsigned cp) {
    if (cp < 0x80) {
      out += (char)cp;
    } else if (cp < 0x800) {
      out += (char)(0xC0 | (cp >> 6));
      out += (char)(0x80 | (cp & 0x3F));
    } else if (cp < 0x10000) {
      out += (char)(0xE0 | (cp >> 12));
      out += (char)(0x80 | ((cp >> 6) & 0x3F));
      out += (char)(0x80 | (cp & 0x3F));
    } else {
      out += (char)(0xF0 | (cp >> 18));
      out += (char)(0x80 | ((cp >> 12) & 0x3F));
      out += (char)(0x80 | ((cp >> 6) & 0x3F));
      out += (char)(0x80 | (cp & 0x3F));
    }
  }
  unsigned hex4() {
    if (i + 4 > s.size()) fail("short \\u escape");
    unsigned v = 0;
    for (int k = 0; k < 4; ++k) {
      const char c = s[i++];
      v <<= 4;
      if (c >= '0' && c <= '9') v |= c - '0';
      else if (c >= 'a' && c <= 'f') v |= c - 'a' + 10;
      else if (c >= 'A' && c <= 'F') v |= c - 'A' + 10;
      else fail("bad \\u escape");
    }
    return v;
  }
  std::string string() {
    if (s[i] != '"') fail("expected a string");
    ++i;
    std::string out;
    while (true) {
      if (i >= s.size()) fail("unterminated string");
      const char c = s[i++];
      if (c == '"') break;
      if (c != '\\') {
        out += c;
        continue;
      }
      if (i >= s.size()) fail("unterminated escape");
      const char e = s[i++];
      switch (e) {
        case '"': out += '"'; break;
        case '\\': out += '\\'; break;
        case '/': out += '/'; break;
        case 'b': out += '\b'; break;
        case 'f': out += '\f'; break;
        case 'n': out += '\n'; break;
        case 'r': out += '\r'; break;
        case 't': out += '\t'; break;
        case 'u': {
          unsigned cp = hex4();
          if (cp >= 0xD800 && cp < 0xDC00 && s.compare(i, 2, "\\u") == 0) {
            i += 2;
            const unsigned lo = hex4();
            cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
          }
          utf8(out, cp);
          break;
        }
        default: fail("unknown escape");
      }
    }
    return out;
  }
  Json number() {
    const size_t start = i;
    bool integral = true;
    if (s[i] == '-') ++i;
    while (i < s.size() && (isdigit((unsigned char)s[i]) || s[i] == '.' || s[i] == 'e' || s[i] == 'E' || s[i] == '+' ||
                            s[i] == '-')) {
      if (s[i] == '.' || s[i] == 'e' || s[i] == 'E') integral = false;
      ++i;
    }
    const std::string text = s.substr(start, i - start);
    if (text.empty() || text == "-") fail("expected a number");
    if (integral && text.size() < 19) return Json((int64_t)strtoll(text.c_str(), nullptr, 10));
    const double d = strtod(text.c_str(), nullptr);
    // 3.0 and 1e3 are integers as far as a configuration is concerned
    if (std::isfinite(d) && std::fabs(d) < 9e15 && d == std::floor(d) && !integral) {
      Json j(d);
      return j;
    }
    return Json(d);
  }
  Json value(int depth = 0) {
    if (depth > 200) fail("nested too deeply");
    skip();
    if (i >= s.size()) fail("unexpected end");
    const char c = s[i];
    if (c == '{') {
      ++i;
      Json obj = Json::object();
      skip();
      if (i < s.size() && s[i] == '}') {
        ++i;
        return obj;
      }
      while (true) {
        skip();
        std::string key = string();
        skip();
        if (i >= s.size() || s[i] != ':') fail("expected ':'");
        ++i;
        obj.set(key, value(depth + 1));
        skip();
        if (i < s.size() && s[i] == ',') {
          ++i;
          continue;
        }
        if (i < s.size() && s[i] == '}') {
          ++i;
          return obj;
        }
        fail("expected ',' or '}'");
      }
    }
    if (c == '[') {
      ++i;
      Json arr = Json::array();
      skip();
      if (i < s.size() && s[i] == ']') {
        ++i;
        return arr;
      }
      while (true) {
        arr.push(value(depth + 1));
        skip();
        if (i < s.size() && s[i] == ',') {
          ++i;
          continue;
        }
        if (i < s.size() && s[i] == ']') {
          ++i;
          return arr;
        }
        fail("expected ',' or ']'");
      }
    }
    if (c == '"') return Json(string());
    if (take("true")) return Json(true);
    if (take("false")) return Json(false);
    if (take("null")) return Json();
    if (take("NaN")) return Json(std::nan(""));
    if (take("Infinity")) return Json(INFINITY);
    if (take("-Infinity")) return Json(-INFINITY);
    if (c == '-' || isdigit((unsigned char)c)) return number();
    fail("unexpected character");
  }
};

void write_string(std::string& out, const std::string& s) {
  out += '"';
  for (const unsigned char c : s) {
    switch (c) {
      case '"': out += "\\\""; break;
      case '\\': out += "\\\\"; break;
      case '\n': out += "\\n"; break;
      case '\r': out += "\\r"; break;
      case '\t': out += "\\t"; break;
      default:
        if (c < 0x20) {
          char buf[8];
          snprintf(buf, sizeof buf, "\\u%04x", c);
          out += buf;
        } else {
          out += (char)c;
        }
    }
  }
  out += '"';
}

void write(std::string& out, const Json& j) {
  switch (j.type()) {
    case Json::Null: out += "null"; break;
    case Json::Bool: out += j.as_bool() ? "true" : "false"; break;
    case Json::Int: out += std::to_string(j.as_int()); break;
    case Json::Float: {
      const double d = j.as_double();
      if (std::isnan(d)) {
        out += "NaN";
      } else if (std::isinf(d)) {
        out += d > 0 ? "Infinity" : "-Infinity";
      } else {
        char buf[40];
        snprintf(buf, sizeof buf, "%.17g", d);
        out += buf;
        if (!strpbrk(buf, ".eE")) out += ".0";
      }
      break;
    }
    case Json::String: write_string(out, j.as_string()); break;
    case Json::Array: {
      out += '[';
      bool first = true;
      for (const Json& v : j.items()) {
        if (!first) out += ',';
        first = false;
        write(out, v);
      }
      out += ']';
      break;
    }
    case Json::Object: {
      out += '{';
      bool first = true;
      for (const auto& kv : j.members()) {
        if (!first) out += ',';
        first = false;
        write_string(out, kv.first);
        out += ':';
        write(out, kv.second);
      }
      out += '}';
      break;
    }
  }
}
}  // namespace

Json Json::parse(const std::string& text) {
  Reader r(text);
  Json v = r.value();
  r.skip();
  if (r.i != text.size()) r.fail("text after the value");
  return v;
}

std::string Json::dump() const {
  std::string out;
  write(out, *this);
  return out;
}

const Json* Json::find(const std::string& key) const {
  for (const auto& kv : members_)
    if (kv.first == key) return &kv.second;
  return nullptr;
}

const Json& Json::at(const std::string& key) const {
  const Json* j = find(key);
  if (!j) throw Error("JSON: key '" + key + "' is missing");
  return *j;
}

void Json::set(const std::string& key, Json v) {
  if (type_ != Object) {
    type_ = Object;
  }
  for (auto& kv : members_)
    if (kv.first == key) {
      kv.second = std::move(v);
      return;
    }
  members_.emplace_back(key, std::move(v));
}

}  // namespace tinyinfer
