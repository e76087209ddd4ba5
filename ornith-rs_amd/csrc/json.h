// A small JSON reader shared by the artifact loader, the tokenizer and the chat template:
// objects keep their keys in file order (the chat template writes them back out in that
// order), numbers remember whether they were written as whole numbers.
#pragma once

#include <cerrno>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <utility>
#include <vector>

namespace orn_json {


struct JVal {
  enum Kind { Null, Bool, Num, Str, Arr, Obj } kind = Null;
  bool b = false;
  double num = 0;
  bool integral = false;  // written without fraction or exponent, and fits uint64
  uint64_t u = 0;
  bool is_int = false;    // written without fraction or exponent (any sign, any size)
  std::string raw;        // the number as written
  std::string str;
  std::vector<JVal> arr;
  std::vector<std::pair<std::string, JVal>> obj;  // file order

  const JVal* get(const char* key) const {
    if (kind != Obj) return nullptr;
    for (auto& kv : obj)
      if (kv.first == key) return &kv.second;
    return nullptr;
  }
  bool as_usize(size_t* out) const {
    if (kind != Num) return false;
    if (integral) {
      *out = (size_t)u;
      return true;
    }
    // 1e6-style spellings of a whole number are accepted, fractions are not
    if (num < 0 || num > 9007199254740992.0 || num != std::floor(num)) return false;
    *out = (size_t)num;
    return true;
  }
};

struct JParser {
  const char* p;
  const char* end;
  const char* begin;
  std::string err;

  bool fail(const char* what) {
    if (err.empty()) {
      char buf[160];
      snprintf(buf, sizeof buf, "JSON: %s at byte %zu", what, (size_t)(p - begin));
      err = buf;
    }
    return false;
  }
  void ws() {
    while (p < end && (*p == ' ' || *p == '\t' || *p == '\n' || *p == '\r')) ++p;
  }
  static void utf8(std::string& s, uint32_t c) {
    if (c < 0x80) {
      s.push_back((char)c);
    } else if (c < 0x800) {
      s.push_back((char)(0xC0 | (c >> 6)));
      s.push_back((char)(0x80 | (c & 0x3F)));
    } else if (c < 0x10000) {
      s.push_back((char)(0xE0 | (c >> 12)));
      s.push_back((char)(0x80 | ((c >> 6) & 0x3F)));
      s.push_back((char)(0x80 | (c & 0x3F)));
    } else {
      s.push_back((char)(0xF0 | (c >> 18)));
      s.push_back((char)(0x80 | ((c >> 12) & 0x3F)));
      s.push_back((char)(0x80 | ((c >> 6) & 0x3F)));
      s.push_back((char)(0x80 | (c & 0x3F)));
    }
  }
  bool hex4(uint32_t* out) {
    if (end - p < 4) return fail("short \\u escape");
    uint32_t v = 0;
    for (int i = 0; i < 4; ++i) {
      const char c = *p++;
      v <<= 4;
      if (c >= '0' && c <= '9') v |= (uint32_t)(c - '0');
      else if (c >= 'a' && c <= 'f') v |= (uint32_t)(c - 'a' + 10);
      else if (c >= 'A' && c <= 'F') v |= (uint32_t)(c - 'A' + 10);
      else return fail("bad \\u escape");
    }
    *out = v;
    return true;
  }
  bool string(std::string* out) {
    if (p >= end || *p != '"') return fail("expected a string");
    ++p;
    out->clear();
    while (true) {
      if (p >= end) return fail("unterminated string");
      const unsigned char c = (unsigned char)*p++;
      if (c == '"') return true;
      if (c < 0x20) return fail("control character in a string");
      if (c != '\\') {
        out->push_back((char)c);
        continue;
      }
      if (p >= end) return fail("unterminated escape");
      const char e = *p++;
      switch (e) {
        case '"': out->push_back('"'); break;
        case '\\': out->push_back('\\'); break;
        case '/': out->push_back('/'); break;
        case 'b': out->push_back('\b'); break;
        case 'f': out->push_back('\f'); break;
        case 'n': out->push_back('\n'); break;
        case 'r': out->push_back('\r'); break;
        case 't': out->push_back('\t'); break;
        case 'u': {
          uint32_t c1;
          if (!hex4(&c1)) return false;
          if (c1 >= 0xD800 && c1 < 0xDC00) {  // surrogate pair
            uint32_t c2;
            if (end - p < 2 || p[0] != '\\' || p[1] != 'u') return fail("lone high surrogate");
            p += 2;
            if (!hex4(&c2)) return false;
            if (c2 < 0xDC00 || c2 > 0xDFFF) return fail("bad low surrogate");
            c1 = 0x10000 + ((c1 - 0xD800) << 10) + (c2 - 0xDC00);
          } else if (c1 >= 0xDC00 && c1 <= 0xDFFF) {
            return fail("lone low surrogate");
          }
          utf8(*out, c1);
          break;
        }
        default: return fail("unknown escape");
      }
    }
  }
  bool number(JVal* v) {
    const char* s = p;
    bool frac = false;
    if (p < end && *p == '-') ++p;
    if (p >= end || *p < '0' || *p > '9') return fail("bad number");
    if (*p == '0') {
      ++p;
    } else {
      while (p < end && *p >= '0' && *p <= '9') ++p;
    }
    if (p < end && *p == '.') {
      frac = true;
      ++p;
      if (p >= end || *p < '0' || *p > '9') return fail("bad fraction");
      while (p < end && *p >= '0' && *p <= '9') ++p;
    }
    if (p < end && (*p == 'e' || *p == 'E')) {
      frac = true;
      ++p;
      if (p < end && (*p == '+' || *p == '-')) ++p;
      if (p >= end || *p < '0' || *p > '9') return fail("bad exponent");
      while (p < end && *p >= '0' && *p <= '9') ++p;
    }
    const std::string text(s, p);
    v->kind = JVal::Num;
    v->num = strtod(text.c_str(), nullptr);
    v->is_int = !frac;
    v->raw = text;
    if (!frac && text[0] != '-' && text.size() <= 19) {
      v->integral = true;
      v->u = strtoull(text.c_str(), nullptr, 10);
    }
    return true;
  }
  bool literal(const char* word) {
    const size_t n = strlen(word);
    if ((size_t)(end - p) < n || memcmp(p, word, n) != 0) return fail("unknown literal");
    p += n;
    return true;
  }
  bool value(JVal* v, int depth) {
    if (depth > 64) return fail("nesting too deep");
    ws();
    if (p >= end) return fail("unexpected end");
    switch (*p) {
      case '{': {
        ++p;
        v->kind = JVal::Obj;
        ws();
        if (p < end && *p == '}') {
          ++p;
          return true;
        }
        while (true) {
          ws();
          std::string key;
          if (!string(&key)) return false;
          ws();
          if (p >= end || *p != ':') return fail("expected ':'");
          ++p;
          v->obj.emplace_back(std::move(key), JVal());
          if (!value(&v->obj.back().second, depth + 1)) return false;
          ws();
          if (p < end && *p == ',') {
            ++p;
            continue;
          }
          if (p < end && *p == '}') {
            ++p;
            return true;
          }
          return fail("expected ',' or '}'");
        }
      }
      case '[': {
        ++p;
        v->kind = JVal::Arr;
        ws();
        if (p < end && *p == ']') {
          ++p;
          return true;
        }
        while (true) {
          v->arr.emplace_back();
          if (!value(&v->arr.back(), depth + 1)) return false;
          ws();
          if (p < end && *p == ',') {
            ++p;
            continue;
          }
          if (p < end && *p == ']') {
            ++p;
            return true;
          }
          return fail("expected ',' or ']'");
        }
      }
      case '"':
        v->kind = JVal::Str;
        return string(&v->str);
      case 't':
        v->kind = JVal::Bool;
        v->b = true;
        return literal("true");
      case 'f':
        v->kind = JVal::Bool;
        v->b = false;
        return literal("false");
      case 'n':
        v->kind = JVal::Null;
        return literal("null");
      default:
        return number(v);
    }
  }
};

inline bool json_parse(const char* data, size_t n, JVal* out, std::string* err) {
  JParser ps{data, data + n, data, {}};
  if (!ps.value(out, 0)) {
    *err = ps.err;
    return false;
  }
  ps.ws();
  if (ps.p != ps.end) {
    ps.fail("trailing bytes after the value");
    *err = ps.err;
    return false;
  }
  return true;
}

inline bool read_file(const std::string& path, std::string* out, std::string* err) {
  FILE* f = fopen(path.c_str(), "rb");
  if (!f) {
    *err = path + ": " + strerror(errno);
    return false;
  }
  char buf[1 << 16];
  size_t n;
  out->clear();
  while ((n = fread(buf, 1, sizeof buf, f)) > 0) out->append(buf, n);
  fclose(f);
  return true;
}

inline bool json_file(const std::string& path, JVal* out, std::string* err) {
  std::string raw;
  if (!read_file(path, &raw, err)) return false;
  std::string perr;
  if (!json_parse(raw.data(), raw.size(), out, &perr)) {
    *err = path + ": " + perr;
    return false;
  }
  return true;
}

}  // namespace orn_json
