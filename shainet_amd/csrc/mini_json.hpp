// A small JSON reader for config.json, safetensors headers and shard indexes:
// objects keep their key order, numbers are kept as doubles and, where they are
// written as integers, as 64-bit integers too.
#pragma once
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <string>
#include <utility>
#include <vector>

namespace shainet {

struct Json {
  enum Kind { kNull, kBool, kNumber, kString, kArray, kObject } kind = kNull;
  bool b = false;
  double num = 0.0;
  long long inum = 0;
  bool is_int = false;
  std::string str;
  std::vector<Json> arr;
  std::vector<std::pair<std::string, Json>> obj;

  const Json *get(const char *key) const {
    if (kind != kObject) return nullptr;
    for (const auto &kv : obj)
      if (kv.first == key) return &kv.second;
    return nullptr;
  }
  bool is_null() const { return kind == kNull; }
};

class JsonParser {
 public:
  JsonParser(const char *text, size_t len) : p_(text), end_(text + len) {}
  bool parse(Json &out, std::string &err) {
    if (!value(out, 0)) {
      err = err_.empty() ? "malformed JSON" : err_;
      return false;
    }
    skip();
    if (p_ != end_) {
      err = "trailing characters after JSON value";
      return false;
    }
    return true;
  }

 private:
  const char *p_, *end_;
  std::string err_;
  void skip() {
    while (p_ < end_ && (*p_ == ' ' || *p_ == '\n' || *p_ == '\t' || *p_ == '\r')) ++p_;
  }
  bool fail(const char *m) {
    if (err_.empty()) err_ = m;
    return false;
  }
  bool literal(const char *word) {
    const size_t n = strlen(word);
    if ((size_t)(end_ - p_) < n || memcmp(p_, word, n) != 0) return fail("bad literal");
    p_ += n;
    return true;
  }
  static void put_utf8(std::string &s, unsigned cp) {
    if (cp < 0x80) {
      s += (char)cp;
    } else if (cp < 0x800) {
      s += (char)(0xC0 | (cp >> 6));
      s += (char)(0x80 | (cp & 0x3F));
    } else if (cp < 0x10000) {
      s += (char)(0xE0 | (cp >> 12));
      s += (char)(0x80 | ((cp >> 6) & 0x3F));
      s += (char)(0x80 | (cp & 0x3F));
    } else {
      s += (char)(0xF0 | (cp >> 18));
      s += (char)(0x80 | ((cp >> 12) & 0x3F));
      s += (char)(0x80 | ((cp >> 6) & 0x3F));
      s += (char)(0x80 | (cp & 0x3F));
    }
  }
  bool hex4(unsigned &v) {
    if (end_ - p_ < 4) return fail("short \\u escape");
    v = 0;
    for (int i = 0; i < 4; ++i) {
      const char c = *p_++;
      v <<= 4;
      if (c >= '0' && c <= '9') v |= (unsigned)(c - '0');
      else if (c >= 'a' && c <= 'f') v |= (unsigned)(c - 'a' + 10);
      else if (c >= 'A' && c <= 'F') v |= (unsigned)(c - 'A' + 10);
      else return fail("bad \\u escape");
    }
    return true;
  }
  bool string(std::string &s) {
    if (p_ >= end_ || *p_ != '"') return fail("expected string");
    ++p_;
    s.clear();
    while (p_ < end_ && *p_ != '"') {
      char c = *p_++;
      if (c != '\\') {
        s += c;
        continue;
      }
      if (p_ >= end_) return fail("short escape");
      c = *p_++;
      switch (c) {
        case '"': s += '"'; break;
        case '\\': s += '\\'; break;
        case '/': s += '/'; break;
        case 'b': s += '\b'; break;
        case 'f': s += '\f'; break;
        case 'n': s += '\n'; break;
        case 'r': s += '\r'; break;
        case 't': s += '\t'; break;
        case 'u': {
          unsigned cp;
          if (!hex4(cp)) return false;
          if (cp >= 0xD800 && cp < 0xDC00 && end_ - p_ >= 6 && p_[0] == '\\' && p_[1] == 'u') {
            p_ += 2;
            unsigned lo;
            if (!hex4(lo)) return false;
            cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
          }
          put_utf8(s, cp);
          break;
        }
        default: return fail("bad escape");
      }
    }
    if (p_ >= end_) return fail("unterminated string");
    ++p_;
    return true;
  }
  bool value(Json &out, int depth) {
    if (depth > 64) return fail("JSON nested too deeply");
    skip();
    if (p_ >= end_) return fail("unexpected end of JSON");
    const char c = *p_;
    if (c == '{') {
      ++p_;
      out.kind = Json::kObject;
      skip();
      if (p_ < end_ && *p_ == '}') {
        ++p_;
        return true;
      }
      for (;;) {
        skip();
        std::string key;
        if (!string(key)) return false;
        skip();
        if (p_ >= end_ || *p_ != ':') return fail("expected ':'");
        ++p_;
        out.obj.emplace_back(std::move(key), Json());
        if (!value(out.obj.back().second, depth + 1)) return false;
        skip();
        if (p_ < end_ && *p_ == ',') {
          ++p_;
          continue;
        }
        if (p_ < end_ && *p_ == '}') {
          ++p_;
          return true;
        }
        return fail("expected ',' or '}'");
      }
    }
    if (c == '[') {
      ++p_;
      out.kind = Json::kArray;
      skip();
      if (p_ < end_ && *p_ == ']') {
        ++p_;
        return true;
      }
      for (;;) {
        out.arr.emplace_back();
        if (!value(out.arr.back(), depth + 1)) return false;
        skip();
        if (p_ < end_ && *p_ == ',') {
          ++p_;
          continue;
        }
        if (p_ < end_ && *p_ == ']') {
          ++p_;
          return true;
        }
        return fail("expected ',' or ']'");
      }
    }
    if (c == '"') {
      out.kind = Json::kString;
      return string(out.str);
    }
    if (c == 't') {
      out.kind = Json::kBool;
      out.b = true;
      return literal("true");
    }
    if (c == 'f') {
      out.kind = Json::kBool;
      out.b = false;
      return literal("false");
    }
    if (c == 'n') {
      out.kind = Json::kNull;
      return literal("null");
    }
    // number
    const char *start = p_;
    bool integral = true;
    if (p_ < end_ && (*p_ == '-' || *p_ == '+')) ++p_;
    while (p_ < end_ && ((*p_ >= '0' && *p_ <= '9') || *p_ == '.' || *p_ == 'e' || *p_ == 'E' || *p_ == '-' || *p_ == '+')) {
      if (*p_ == '.' || *p_ == 'e' || *p_ == 'E') integral = false;
      ++p_;
    }
    if (p_ == start) return fail("unexpected character in JSON");
    const std::string tok(start, p_);
    char *endp = nullptr;
    out.kind = Json::kNumber;
    out.num = strtod(tok.c_str(), &endp);
    if (endp == tok.c_str() || *endp) return fail("bad number");
    out.is_int = integral;
    out.inum = integral ? strtoll(tok.c_str(), nullptr, 10) : (long long)out.num;
    return true;
  }
};

}  // namespace shainet
