// UTF-8, Unicode classes and NFC for the tokenizer and the chat template (host only).
//
//   split pattern classes   /root/reference/src/tokenizer/split.rs:100-118 (\p{L} \p{M} \p{N} \s)
//   NFC                     /root/reference/src/tokenizer/nfc.rs:1-199 (UAX #15: decompose,
//                           canonical ordering, canonical composition; Hangul by arithmetic)
//   lossy UTF-8             String::from_utf8_lossy in src/tokenizer/mod.rs:326,362
#include "text.h"

#include <algorithm>

#include "unicode_tables.h"

namespace orn_text {

bool utf8_decode(const char* s, size_t n, std::vector<uint32_t>* out) {
  out->clear();
  out->reserve(n);
  const unsigned char* p = reinterpret_cast<const unsigned char*>(s);
  size_t i = 0;
  while (i < n) {
    const unsigned char b = p[i];
    if (b < 0x80) {
      out->push_back(b);
      ++i;
      continue;
    }
    int len;
    uint32_t cp, min;
    if (b >= 0xC2 && b <= 0xDF) {
      len = 2, cp = b & 0x1F, min = 0x80;
    } else if (b >= 0xE0 && b <= 0xEF) {
      len = 3, cp = b & 0x0F, min = 0x800;
    } else if (b >= 0xF0 && b <= 0xF4) {
      len = 4, cp = b & 0x07, min = 0x10000;
    } else {
      return false;
    }
    if (i + len > n) return false;
    for (int k = 1; k < len; ++k) {
      if ((p[i + k] & 0xC0) != 0x80) return false;
      cp = (cp << 6) | (p[i + k] & 0x3F);
    }
    if (cp < min || cp > 0x10FFFF || (cp >= 0xD800 && cp <= 0xDFFF)) return false;
    out->push_back(cp);
    i += len;
  }
  return true;
}

void utf8_append(std::string& s, uint32_t c) {
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

// The ranges a continuation byte may take after the bytes seen so far are what decides how
// long an ill-formed prefix is ("maximal subpart", Unicode 3.9 / the WHATWG decoder): after
// E0 only A0..BF, after ED only 80..9F, after F0 only 90..BF, after F4 only 80..8F.
std::string utf8_lossy(const std::string& bytes) {
  std::string out;
  out.reserve(bytes.size());
  const unsigned char* p = reinterpret_cast<const unsigned char*>(bytes.data());
  const size_t n = bytes.size();
  size_t i = 0;
  while (i < n) {
    const unsigned char b = p[i];
    if (b < 0x80) {
      out.push_back((char)b);
      ++i;
      continue;
    }
    int need = 0;
    unsigned char lo = 0x80, hi = 0xBF;
    if (b >= 0xC2 && b <= 0xDF) {
      need = 1;
    } else if (b >= 0xE0 && b <= 0xEF) {
      need = 2;
      if (b == 0xE0) lo = 0xA0;
      if (b == 0xED) hi = 0x9F;
    } else if (b >= 0xF0 && b <= 0xF4) {
      need = 3;
      if (b == 0xF0) lo = 0x90;
      if (b == 0xF4) hi = 0x8F;
    }
    size_t j = i + 1;
    bool ok = need > 0;
    for (int k = 0; ok && k < need; ++k) {
      if (j >= n || p[j] < lo || p[j] > hi) {
        ok = false;
        break;
      }
      ++j;
      lo = 0x80, hi = 0xBF;
    }
    if (ok) {
      out.append(bytes, i, j - i);
    } else {
      out.append("\xEF\xBF\xBD");  // the bytes accepted so far are the maximal subpart
    }
    i = j;
  }
  return out;
}

static bool in_ranges(const uint32_t (*t)[2], int n, uint32_t c) {
  int lo = 0, hi = n - 1;
  while (lo <= hi) {
    const int mid = (lo + hi) / 2;
    if (c < t[mid][0]) hi = mid - 1;
    else if (c > t[mid][1]) lo = mid + 1;
    else return true;
  }
  return false;
}

bool is_letter(uint32_t c) { return in_ranges(UT_LETTER, UT_LETTER_N, c); }
bool is_mark(uint32_t c) { return in_ranges(UT_MARK, UT_MARK_N, c); }
bool is_number(uint32_t c) { return in_ranges(UT_NUMBER, UT_NUMBER_N, c); }
bool is_space(uint32_t c) { return in_ranges(UT_WHITE_SPACE, UT_WHITE_SPACE_N, c); }
bool is_py_space(uint32_t c) { return in_ranges(UT_PY_WHITESPACE, UT_PY_WHITESPACE_N, c); }

int combining_class(uint32_t c) {
  int lo = 0, hi = UT_CCC_N - 1;
  while (lo <= hi) {
    const int mid = (lo + hi) / 2;
    if (c < UT_CCC[mid][0]) hi = mid - 1;
    else if (c > UT_CCC[mid][1]) lo = mid + 1;
    else return (int)UT_CCC[mid][2];
  }
  return 0;
}

namespace {
// Hangul syllables (UAX #15, D132-D133)
const uint32_t SB = 0xAC00, LB = 0x1100, VB = 0x1161, TB = 0x11A7;
const uint32_t LN = 19, VN = 21, TN = 28, NN = VN * TN, SN = LN * NN;

void decompose(uint32_t c, std::vector<uint32_t>& out) {
  if (c >= SB && c < SB + SN) {
    const uint32_t si = c - SB;
    out.push_back(LB + si / NN);
    out.push_back(VB + (si % NN) / TN);
    if (si % TN) out.push_back(TB + si % TN);
    return;
  }
  int lo = 0, hi = UT_DECOMPOSE_N - 1;
  while (lo <= hi) {
    const int mid = (lo + hi) / 2;
    if (c < UT_DECOMPOSE[mid][0]) hi = mid - 1;
    else if (c > UT_DECOMPOSE[mid][0]) lo = mid + 1;
    else {
      const uint32_t* d = UT_DECOMPOSE_DATA + UT_DECOMPOSE[mid][1];
      out.insert(out.end(), d, d + UT_DECOMPOSE[mid][2]);
      return;
    }
  }
  out.push_back(c);
}

// primary composite of (a, b), or 0
uint32_t compose(uint32_t a, uint32_t b) {
  if (a >= LB && a < LB + LN && b >= VB && b < VB + VN) return SB + ((a - LB) * VN + (b - VB)) * TN;
  if (a >= SB && a < SB + SN && (a - SB) % TN == 0 && b > TB && b < TB + TN) return a + (b - TB);
  int lo = 0, hi = UT_COMPOSE_N - 1;
  while (lo <= hi) {
    const int mid = (lo + hi) / 2;
    const uint32_t* e = UT_COMPOSE[mid];
    if (a < e[0] || (a == e[0] && b < e[1])) hi = mid - 1;
    else if (a > e[0] || b > e[1]) lo = mid + 1;
    else return e[2];
  }
  return 0;
}
}  // namespace

std::vector<uint32_t> nfc(const std::vector<uint32_t>& s) {
  bool plain = true;
  for (uint32_t c : s)
    if (in_ranges(UT_NFC_UNSAFE, UT_NFC_UNSAFE_N, c) || (c >= SB && c < SB + SN)) {
      plain = false;
      break;
    }
  // precomposed Hangul is already NFC; it only matters above when jamo follow it
  if (plain) return s;

  std::vector<uint32_t> d;
  d.reserve(s.size() + 8);
  for (uint32_t c : s) decompose(c, d);

  // canonical ordering: each run of non-starters sorted by class, stable
  for (size_t i = 0; i < d.size();) {
    if (combining_class(d[i]) == 0) {
      ++i;
      continue;
    }
    size_t j = i;
    while (j < d.size() && combining_class(d[j]) != 0) ++j;
    std::stable_sort(d.begin() + i, d.begin() + j,
                     [](uint32_t x, uint32_t y) { return combining_class(x) < combining_class(y); });
    i = j;
  }

  // canonical composition: a character joins the last starter when the pair has a primary
  // composite and nothing of an equal or higher class (or another starter) stands between
  std::vector<uint32_t> out;
  out.reserve(d.size());
  long starter = -1;
  int last_cc = 0;  // class of the last character kept after the starter; 0: none yet
  for (uint32_t c : d) {
    const int cc = combining_class(c);
    if (starter >= 0 && (last_cc == 0 || last_cc < cc)) {
      const uint32_t x = compose(out[starter], c);
      if (x) {
        out[starter] = x;
        continue;
      }
    }
    if (cc == 0) {
      starter = (long)out.size();
      last_cc = 0;
    } else {
      last_cc = cc;
    }
    out.push_back(c);
  }
  return out;
}

}  // namespace orn_text
