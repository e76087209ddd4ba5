// The tokenizer: `tokenizer.json` read and run by hand, and the streaming detokenizer (host only).
//
//   Tokenizer::{load, load_as, encode, decode, token, id, is_special}  /root/reference/src/tokenizer/mod.rs:78-349
//   Detokenizer (mlx-lm's BPEStreamingDetokenizer)                      /root/reference/src/tokenizer/mod.rs:352-417
//   pre_split / the split pattern                                       /root/reference/src/tokenizer/split.rs:1-238
//   merge_all (tokenizers' Word::merge_all)                             /root/reference/src/tokenizer/bpe.rs:1-117
//
// Pipeline, in the order `tokenizers` runs it: split the raw text on the added tokens
// (leftmost-longest), NFC on every other piece, Split(pattern, Isolated) + ByteLevel, BPE with
// ranked merges; the post-processor adds nothing. A tokenizer.json that asks for anything
// else is refused rather than tokenized differently.
#include <algorithm>
#include <queue>
#include <unordered_map>

#include "json.h"
#include "rt.h"
#include "text.h"

using namespace orn_json;
using namespace orn_text;

namespace {

const char* kPatternJson =
    "(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\\r\\n\\p{L}\\p{N}]?[\\p{L}\\p{M}]+|\\p{N}| ?[^\\s\\p{L}\\p{M}\\p{N}]+[\\r\\n]*|\\s*[\\r\\n]+|\\s+(?!\\S)|\\s+";
const char* kPatternTransformers =
    "(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\\r\\n\\p{L}\\p{N}]?\\p{L}+|\\p{N}| ?[^\\s\\p{L}\\p{N}]+[\\r\\n]*|\\s*[\\r\\n]+|\\s+(?!\\S)|\\s+";

// ---- the split pattern, matched by hand ----------------------------------------------
// oniguruma is an ordered backtracking engine and the pattern matches at least one character
// everywhere, so `Isolated` tiles the text: at the cursor take the first alternative that
// succeeds, greedy with backtracking.
struct Splitter {
  bool marks;  // [\p{L}\p{M}] (tokenizer.json's pattern) or \p{L} alone (transformers')
  bool word(uint32_t c) const { return is_letter(c) || (marks && is_mark(c)); }
  static bool prefix(uint32_t c) { return c != '\r' && c != '\n' && !is_letter(c) && !is_number(c); }
  bool punct(uint32_t c) const { return !is_space(c) && !word(c) && !is_number(c); }
  // (?i:) folds by Unicode simple case folding; of everything that folds onto s t r e v m l d
  // only U+017F (long s) is not the letter's own upper case
  static bool folds(uint32_t c, char l) { return c == (uint32_t)l || c == (uint32_t)(l - 32) || (l == 's' && c == 0x17F); }

  size_t match(const std::vector<uint32_t>& c, size_t i) const {
    const size_t n = c.size();
    // 1. (?i:'s|'t|'re|'ve|'m|'ll|'d)
    if (c[i] == '\'') {
      static const char* words[] = {"s", "t", "re", "ve", "m", "ll", "d"};
      for (const char* w : words) {
        const size_t len = strlen(w);
        if (i + 1 + len > n) continue;
        bool ok = true;
        for (size_t k = 0; k < len && ok; ++k) ok = folds(c[i + 1 + k], w[k]);
        if (ok) return i + 1 + len;
      }
    }
    // 2. [^\r\n\p{L}\p{N}]?[\p{L}\p{M}]+ : the optional character is greedy, so with it first
    for (int skip = 1; skip >= 0; --skip) {
      if (skip && !prefix(c[i])) continue;
      size_t j = i + skip;
      if (j < n && word(c[j])) {
        while (j < n && word(c[j])) ++j;
        return j;
      }
    }
    // 3. \p{N}
    if (is_number(c[i])) return i + 1;
    // 4.  ?[^\s\p{L}\p{M}\p{N}]+[\r\n]*
    {
      size_t j = i + (c[i] == ' ' ? 1 : 0);
      if (j < n && punct(c[j])) {
        while (j < n && punct(c[j])) ++j;
        while (j < n && (c[j] == '\r' || c[j] == '\n')) ++j;
        return j;
      }
    }
    // 5. \s*[\r\n]+ : all the spaces, then back off to the last line break among them
    size_t run = i;
    while (run < n && is_space(c[run])) ++run;
    for (size_t j = run; j > i; --j)
      if (c[j - 1] == '\r' || c[j - 1] == '\n') return j;
    // 6. \s+(?!\S) : give characters back until a space (or the end) follows
    for (size_t j = run; j > i; --j)
      if (j == n || is_space(c[j])) return j;
    // 7. \s+
    if (run > i) return run;
    return i + 1;  // not reachable: every character is in one of the classes above
  }
};

}  // namespace

struct ornith_tokenizer {
  int dialect = 0;
  std::unordered_map<std::string, uint32_t> vocab;  // the BPE entries
  std::vector<std::string> tokens;                  // id -> token string, added ones included
  std::unordered_map<uint64_t, std::pair<uint32_t, uint32_t>> merges;  // (a, b) -> (rank, new id)
  std::vector<std::pair<std::string, uint32_t>> added;                 // longest first
  std::vector<uint32_t> special, eos_ids;
  uint32_t byte_cp[256];                          // the GPT-2 byte alphabet
  uint32_t byte_id[256];                          // vocab id of each byte's one-character token
  std::unordered_map<uint32_t, uint8_t> cp_byte;  // and back
  bool added_first_byte[256] = {};

  const std::string& token(uint32_t id) const {
    // ids past the tokenizer's entries (the model's vocabulary is padded) read as "!", the
    // fallback of the detokenizer this mirrors
    static const std::string bang = "!";
    if (id >= tokens.size() || tokens[id].empty()) return bang;
    return tokens[id];
  }
};

struct ornith_detokenizer {
  const ornith_tokenizer* tk;
  std::string text, unflushed;
  size_t offset = 0;
  std::vector<uint32_t> tokens;
};

namespace {

uint64_t pair_key(uint32_t a, uint32_t b) { return ((uint64_t)a << 32) | b; }

// tokenizers' Word::merge_all: a queue of candidate merges ordered by (rank, position), stale
// entries skipped when popped. Lowest rank first; among equal ranks the leftmost.
void merge_all(const ornith_tokenizer& tk, const std::vector<uint32_t>& ids, std::vector<uint32_t>* out) {
  struct Sym {
    uint32_t c;
    int prev, next;
    bool live;
  };
  struct Cand {
    uint32_t rank, pos, new_id;
    bool operator<(const Cand& o) const { return rank != o.rank ? rank > o.rank : pos > o.pos; }
  };
  const int n = (int)ids.size();
  std::vector<Sym> sym(n);
  for (int i = 0; i < n; ++i) sym[i] = {ids[i], i - 1, i + 1 < n ? i + 1 : -1, true};
  std::priority_queue<Cand> q;
  auto push = [&](int pos) {
    const int nx = sym[pos].next;
    if (nx < 0) return;
    auto it = tk.merges.find(pair_key(sym[pos].c, sym[nx].c));
    if (it != tk.merges.end()) q.push({it->second.first, (uint32_t)pos, it->second.second});
  };
  for (int i = 0; i + 1 < n; ++i) push(i);
  while (!q.empty()) {
    const Cand top = q.top();
    q.pop();
    Sym& s = sym[top.pos];
    if (!s.live || s.next < 0) continue;
    const int nx = s.next;
    auto it = tk.merges.find(pair_key(s.c, sym[nx].c));
    if (it == tk.merges.end() || it->second.second != top.new_id) continue;  // the pair changed since
    s.c = top.new_id;
    s.next = sym[nx].next;
    sym[nx].live = false;
    if (s.next >= 0) sym[s.next].prev = (int)top.pos;
    if (s.prev >= 0) push(s.prev);
    push((int)top.pos);
  }
  for (int i = 0; i < n; ++i)
    if (sym[i].live) out->push_back(sym[i].c);
}

// normalize, pre-tokenize and merge one stretch of text that holds no added token
int encode_plain(const ornith_tokenizer& tk, const char* s, size_t n, std::vector<uint32_t>* out) {
  std::vector<uint32_t> cps;
  if (!utf8_decode(s, n, &cps)) return ornith_fail(ORNITH_ERR_INVALID, "tokenizer_encode: the text is not valid UTF-8");
  const std::vector<uint32_t> norm = nfc(cps);
  const Splitter sp{tk.dialect == 0};
  std::vector<uint32_t> word;
  std::string piece;
  for (size_t i = 0; i < norm.size();) {
    const size_t end = sp.match(norm, i);
    piece.clear();
    for (size_t k = i; k < end; ++k) utf8_append(piece, norm[k]);
    word.clear();
    for (unsigned char b : piece) word.push_back(tk.byte_id[b]);
    merge_all(tk, word, out);
    i = end;
  }
  return ORNITH_OK;
}

int encode(const ornith_tokenizer& tk, const char* text, size_t n, std::vector<uint32_t>* out) {
  size_t i = 0, plain_from = 0;
  while (i < n) {
    const std::pair<std::string, uint32_t>* hit = nullptr;
    if (tk.added_first_byte[(unsigned char)text[i]])
      for (auto& a : tk.added)  // longest first: the first hit is the leftmost-longest match
        if (a.first.size() <= n - i && memcmp(text + i, a.first.data(), a.first.size()) == 0) {
          hit = &a;
          break;
        }
    if (!hit) {
      ++i;
      continue;
    }
    if (plain_from < i)
      if (int rc = encode_plain(tk, text + plain_from, i - plain_from, out)) return rc;
    out->push_back(hit->second);
    i += hit->first.size();
    plain_from = i;
  }
  if (plain_from < n) return encode_plain(tk, text + plain_from, n - plain_from, out);
  return ORNITH_OK;
}

// ByteLevel decoding of token strings: each character back to the byte it stands for; a
// character outside the alphabet (added tokens may hold any) keeps its own UTF-8.
// skip_zero: the streaming detokenizer this mirrors tests the byte for truthiness, so the
// character standing for byte 0 is emitted as itself there.
void byte_decode(const ornith_tokenizer& tk, const std::string& s, bool skip_zero, std::string* bytes) {
  std::vector<uint32_t> cps;
  utf8_decode(s.data(), s.size(), &cps);  // token strings come from JSON: valid
  for (uint32_t c : cps) {
    auto it = tk.cp_byte.find(c);
    if (it != tk.cp_byte.end() && !(skip_zero && it->second == 0)) bytes->push_back((char)it->second);
    else utf8_append(*bytes, c);
  }
}

int copy_out(const std::string& s, char* out, size_t cap, size_t* n_out, const char* who) {
  if (n_out) *n_out = s.size();
  if (!out) return ORNITH_OK;  // size query
  ORN_REQUIRE(cap >= s.size(), "%s: %zu bytes do not fit the buffer (%zu)", who, s.size(), cap);
  memcpy(out, s.data(), s.size());
  return ORNITH_OK;
}

const JVal* path(const JVal& root, std::initializer_list<const char*> keys) {
  const JVal* v = &root;
  for (const char* k : keys) {
    v = v->get(k);
    if (!v) return nullptr;
  }
  return v;
}
bool str_is(const JVal* v, const char* want) { return v && v->kind == JVal::Str && v->str == want; }
bool bool_is(const JVal* v, bool want) { return v && v->kind == JVal::Bool && v->b == want; }

int load(const std::string& dir, int dialect, ornith_tokenizer* tk) {
  JVal tj, cfg;
  std::string err;
  ORN_REQUIRE(json_file(dir + "/tokenizer.json", &tj, &err), "tokenizer_load: %s", err.c_str());
  ORN_REQUIRE(json_file(dir + "/tokenizer_config.json", &cfg, &err), "tokenizer_load: %s", err.c_str());
  tk->dialect = dialect;

#define TK_NEED(cond, ...) \
  if (!(cond)) return ornith_fail(ORNITH_ERR_UNSUPPORTED, "tokenizer_load: " __VA_ARGS__)
  TK_NEED(str_is(path(tj, {"normalizer", "type"}), "NFC"), "normalizer.type is not NFC");
  TK_NEED(str_is(path(tj, {"model", "type"}), "BPE"), "model.type is not BPE");
  for (const char* k : {"dropout", "unk_token"}) {
    const JVal* v = path(tj, {"model", k});
    TK_NEED(!v || v->kind == JVal::Null, "model.%s is set; the BPE here does not implement it", k);
  }
  for (const char* k : {"fuse_unk", "byte_fallback", "ignore_merges"}) {
    const JVal* v = path(tj, {"model", k});
    TK_NEED(!v || bool_is(v, false), "model.%s is set; the BPE here does not implement it", k);
  }
  for (const char* k : {"continuing_subword_prefix", "end_of_word_suffix"}) {
    const JVal* v = path(tj, {"model", k});
    TK_NEED(!v || v->kind == JVal::Null || str_is(v, ""), "model.%s is set; the BPE here does not implement it", k);
  }
  TK_NEED(str_is(path(tj, {"pre_tokenizer", "type"}), "Sequence"), "pre_tokenizer.type is not Sequence");
  const JVal* pres = path(tj, {"pre_tokenizer", "pretokenizers"});
  TK_NEED(pres && pres->kind == JVal::Arr && pres->arr.size() == 2, "pre_tokenizer is not Split + ByteLevel");
  const JVal &p0 = pres->arr[0], &p1 = pres->arr[1];
  TK_NEED(str_is(p0.get("type"), "Split") && str_is(p0.get("behavior"), "Isolated") && bool_is(p0.get("invert"), false),
          "the first pre-tokenizer is not Split(Isolated, invert = false)");
  TK_NEED(str_is(path(p0, {"pattern", "Regex"}), kPatternJson),
          "tokenizer.json carries a split pattern that is not implemented here");
  TK_NEED(str_is(p1.get("type"), "ByteLevel") && bool_is(p1.get("add_prefix_space"), false),
          "the second pre-tokenizer is not ByteLevel(add_prefix_space = false)");
  TK_NEED(str_is(path(tj, {"post_processor", "type"}), "ByteLevel"), "post_processor.type is not ByteLevel");
  TK_NEED(str_is(path(tj, {"decoder", "type"}), "ByteLevel"), "decoder.type is not ByteLevel");
  {
    const JVal* v = cfg.get("add_bos_token");
    TK_NEED(!v || v->kind == JVal::Null || bool_is(v, false), "tokenizer_config asks for a BOS token");
  }

  const JVal* vocab = path(tj, {"model", "vocab"});
  ORN_REQUIRE(vocab && vocab->kind == JVal::Obj, "tokenizer_load: model.vocab is not an object");
  tk->tokens.assign(vocab->obj.size(), std::string());
  tk->vocab.reserve(vocab->obj.size() * 2);
  for (auto& kv : vocab->obj) {
    size_t id;
    ORN_REQUIRE(kv.second.as_usize(&id), "tokenizer_load: a vocab value is not an integer");
    ORN_REQUIRE(id < tk->tokens.size(), "tokenizer_load: vocab id %zu is past the end of the vocab", id);
    tk->tokens[id] = kv.first;
    tk->vocab.emplace(kv.first, (uint32_t)id);
  }

  const JVal* merges = path(tj, {"model", "merges"});
  ORN_REQUIRE(merges && merges->kind == JVal::Arr, "tokenizer_load: model.merges is not a list");
  tk->merges.reserve(merges->arr.size() * 2);
  for (size_t rank = 0; rank < merges->arr.size(); ++rank) {
    const JVal& m = merges->arr[rank];
    std::string a, b;
    if (m.kind == JVal::Str) {
      const size_t sp = m.str.find(' ');
      ORN_REQUIRE(sp != std::string::npos, "tokenizer_load: bad merge \"%s\"", m.str.c_str());
      a = m.str.substr(0, sp);
      b = m.str.substr(sp + 1);
    } else {  // the pair spelling newer files use
      ORN_REQUIRE(m.kind == JVal::Arr && m.arr.size() == 2 && m.arr[0].kind == JVal::Str && m.arr[1].kind == JVal::Str,
                  "tokenizer_load: merge %zu is neither a string nor a pair of strings", rank);
      a = m.arr[0].str;
      b = m.arr[1].str;
    }
    auto ia = tk->vocab.find(a), ib = tk->vocab.find(b), ij = tk->vocab.find(a + b);
    ORN_REQUIRE(ia != tk->vocab.end(), "tokenizer_load: merge lhs \"%s\" not in vocab", a.c_str());
    ORN_REQUIRE(ib != tk->vocab.end(), "tokenizer_load: merge rhs \"%s\" not in vocab", b.c_str());
    ORN_REQUIRE(ij != tk->vocab.end(), "tokenizer_load: merge result \"%s\" not in vocab", (a + b).c_str());
    tk->merges[pair_key(ia->second, ib->second)] = {(uint32_t)rank, ij->second};
  }

  // added tokens: tokenizer.json's, then those only tokenizer_config.json knows, by id
  std::vector<std::pair<size_t, const JVal*>> entries;
  if (const JVal* at = tj.get("added_tokens")) {
    ORN_REQUIRE(at->kind == JVal::Arr, "tokenizer_load: added_tokens is not a list");
    for (auto& t : at->arr) {
      size_t id;
      ORN_REQUIRE(t.get("id") && t.get("id")->as_usize(&id), "tokenizer_load: an added token has no id");
      entries.emplace_back(id, &t);
    }
  }
  if (const JVal* dec = cfg.get("added_tokens_decoder"))
    if (dec->kind == JVal::Obj)
      for (auto& kv : dec->obj) {
        char* endp = nullptr;
        const size_t id = strtoull(kv.first.c_str(), &endp, 10);
        ORN_REQUIRE(endp && *endp == 0 && !kv.first.empty(), "tokenizer_load: added_tokens_decoder key \"%s\"", kv.first.c_str());
        bool seen = false;
        for (auto& e : entries) seen |= e.first == id;
        if (!seen) entries.emplace_back(id, &kv.second);
      }
  std::stable_sort(entries.begin(), entries.end(), [](auto& x, auto& y) { return x.first < y.first; });
  for (auto& e : entries) {
    const JVal* content = e.second->get("content");
    ORN_REQUIRE(content && content->kind == JVal::Str && !content->str.empty(), "tokenizer_load: added token %zu has no content", e.first);
    for (const char* flag : {"single_word", "lstrip", "rstrip", "normalized"}) {
      const JVal* v = e.second->get(flag);
      TK_NEED(!v || bool_is(v, false), "added token \"%s\" sets %s; the split does not implement it", content->str.c_str(), flag);
    }
    if (tk->tokens.size() <= e.first) tk->tokens.resize(e.first + 1);
    tk->tokens[e.first] = content->str;
    tk->added.emplace_back(content->str, (uint32_t)e.first);
    tk->added_first_byte[(unsigned char)content->str[0]] = true;
    if (bool_is(e.second->get("special"), true)) tk->special.push_back((uint32_t)e.first);
  }
  std::sort(tk->added.begin(), tk->added.end(), [](auto& x, auto& y) {
    return x.first.size() != y.first.size() ? x.first.size() > y.first.size() : x.first < y.first;
  });
#undef TK_NEED

  // the GPT-2 byte alphabet: printable Latin-1 bytes stand for themselves, the others take
  // code points from U+0100 up in byte order
  uint32_t next = 0;
  for (int b = 0; b < 256; ++b) {
    const bool printable = (b >= 0x21 && b <= 0x7E) || (b >= 0xA1 && b <= 0xAC) || b >= 0xAE;
    tk->byte_cp[b] = printable ? (uint32_t)b : 256 + next++;
    tk->cp_byte[tk->byte_cp[b]] = (uint8_t)b;
    std::string s;
    utf8_append(s, tk->byte_cp[b]);
    auto it = tk->vocab.find(s);
    ORN_REQUIRE(it != tk->vocab.end(), "tokenizer_load: the vocab has no token for byte 0x%02X", b);
    tk->byte_id[b] = it->second;
  }

  // end-of-sequence ids: generation_config.json's, else tokenizer_config's eos_token
  JVal gen;
  std::string gerr;
  if (json_file(dir + "/generation_config.json", &gen, &gerr)) {
    if (const JVal* e = gen.get("eos_token_id")) {
      size_t id;
      if (e->kind == JVal::Arr) {
        for (auto& v : e->arr)
          if (v.as_usize(&id)) tk->eos_ids.push_back((uint32_t)id);
      } else if (e->as_usize(&id)) {
        tk->eos_ids.push_back((uint32_t)id);
      }
    }
  }
  if (tk->eos_ids.empty()) {
    const JVal* e = cfg.get("eos_token");
    const std::string eos = e && e->kind == JVal::Str ? e->str : "<|im_end|>";
    for (auto& a : tk->added)
      if (a.first == eos) {
        tk->eos_ids.push_back(a.second);
        break;
      }
  }
  return ORNITH_OK;
}

std::string trim_first_space(const ornith_detokenizer* d, const std::string& cur) {
  // a single leading space at the very start of a generation is dropped
  if (cur.empty() || cur[0] != ' ' || !d->text.empty()) return cur;
  return cur.substr(1);
}

}  // namespace

extern "C" {

int ornith_tokenizer_load(const char* model_dir, int dialect, ornith_tokenizer** out) {
  ORN_REQUIRE(model_dir && out, "tokenizer_load: null argument");
  ORN_REQUIRE(dialect == 0 || dialect == 1, "tokenizer_load: dialect %d (0 tokenizer.json's pattern, 1 transformers')", dialect);
  *out = nullptr;
  ornith_tokenizer* tk = new ornith_tokenizer();
  const int rc = load(model_dir, dialect, tk);
  if (rc) {
    delete tk;
    return rc;
  }
  *out = tk;
  return ORNITH_OK;
}

int ornith_tokenizer_destroy(ornith_tokenizer* tk) {
  delete tk;
  return ORNITH_OK;
}

int ornith_tokenizer_vocab_size(const ornith_tokenizer* tk, size_t* n_out) {
  ORN_REQUIRE(tk && n_out, "tokenizer_vocab_size: null argument");
  *n_out = tk->tokens.size();
  return ORNITH_OK;
}

int ornith_tokenizer_encode(const ornith_tokenizer* tk, const char* text, size_t text_len, uint32_t* ids_out,
                            size_t cap, size_t* n_out) {
  ORN_REQUIRE(tk && (text || !text_len) && n_out, "tokenizer_encode: null argument");
  std::vector<uint32_t> ids;
  if (int rc = encode(*tk, text, text_len, &ids)) return rc;
  *n_out = ids.size();
  if (!ids_out) return ORNITH_OK;  // size query
  ORN_REQUIRE(cap >= ids.size(), "tokenizer_encode: %zu ids do not fit the buffer (%zu)", ids.size(), cap);
  if (!ids.empty()) memcpy(ids_out, ids.data(), ids.size() * 4);
  return ORNITH_OK;
}

int ornith_tokenizer_decode(const ornith_tokenizer* tk, const uint32_t* ids, size_t n, char* out, size_t cap,
                            size_t* n_out) {
  ORN_REQUIRE(tk && (ids || !n), "tokenizer_decode: null argument");
  std::string bytes;
  for (size_t i = 0; i < n; ++i) byte_decode(*tk, tk->token(ids[i]), false, &bytes);
  return copy_out(utf8_lossy(bytes), out, cap, n_out, "tokenizer_decode");
}

int ornith_tokenizer_token(const ornith_tokenizer* tk, uint32_t id, char* out, size_t cap, size_t* n_out) {
  ORN_REQUIRE(tk, "tokenizer_token: null argument");
  return copy_out(tk->token(id), out, cap, n_out, "tokenizer_token");
}

int ornith_tokenizer_id(const ornith_tokenizer* tk, const char* token, uint32_t* id_out) {
  ORN_REQUIRE(tk && token && id_out, "tokenizer_id: null argument");
  for (auto& a : tk->added)
    if (a.first == token) {
      *id_out = a.second;
      return ORNITH_OK;
    }
  auto it = tk->vocab.find(token);
  if (it == tk->vocab.end()) return ornith_fail(ORNITH_ERR_INVALID, "tokenizer_id: no token \"%s\"", token);
  *id_out = it->second;
  return ORNITH_OK;
}

int ornith_tokenizer_is_special(const ornith_tokenizer* tk, uint32_t id) {
  if (!tk) return 0;
  return std::find(tk->special.begin(), tk->special.end(), id) != tk->special.end();
}

int ornith_tokenizer_eos_ids(const ornith_tokenizer* tk, uint32_t* ids_out, size_t cap, size_t* n_out) {
  ORN_REQUIRE(tk && n_out, "tokenizer_eos_ids: null argument");
  *n_out = tk->eos_ids.size();
  if (!ids_out) return ORNITH_OK;
  ORN_REQUIRE(cap >= tk->eos_ids.size(), "tokenizer_eos_ids: %zu ids do not fit the buffer (%zu)", tk->eos_ids.size(), cap);
  if (!tk->eos_ids.empty()) memcpy(ids_out, tk->eos_ids.data(), tk->eos_ids.size() * 4);
  return ORNITH_OK;
}

int ornith_detokenizer_create(const ornith_tokenizer* tk, ornith_detokenizer** out) {
  ORN_REQUIRE(tk && out, "detokenizer_create: null argument");
  *out = new ornith_detokenizer{tk, {}, {}, 0, {}};
  return ORNITH_OK;
}

int ornith_detokenizer_destroy(ornith_detokenizer* d) {
  delete d;
  return ORNITH_OK;
}

int ornith_detokenizer_add_token(ornith_detokenizer* d, uint32_t token) {
  ORN_REQUIRE(d, "detokenizer_add_token: null argument");
  d->tokens.push_back(token);
  const std::string& v = d->tk->token(token);
  d->unflushed += v;
  std::string bytes;
  byte_decode(*d->tk, d->unflushed, true, &bytes);
  const std::string text = utf8_lossy(bytes);
  // a partial UTF-8 sequence waits for its rest; a lone space waits for the next token, which
  // decides whether it is the leading one
  std::vector<uint32_t> vc;
  utf8_decode(v.data(), v.size(), &vc);
  bool lone_space = false;
  if (vc.size() == 1) {
    auto it = d->tk->cp_byte.find(vc[0]);
    lone_space = it != d->tk->cp_byte.end() && it->second == 32;
  }
  const bool partial = text.size() >= 3 && text.compare(text.size() - 3, 3, "\xEF\xBF\xBD") == 0;
  if (!partial && !lone_space) {
    d->text += trim_first_space(d, text);
    d->unflushed.clear();
  }
  return ORNITH_OK;
}

int ornith_detokenizer_finalize(ornith_detokenizer* d) {
  ORN_REQUIRE(d, "detokenizer_finalize: null argument");
  std::string bytes;
  byte_decode(*d->tk, d->unflushed, false, &bytes);
  d->text += trim_first_space(d, utf8_lossy(bytes));
  d->unflushed.clear();
  return ORNITH_OK;
}

int ornith_detokenizer_last_segment(ornith_detokenizer* d, char* out, size_t cap, size_t* n_out) {
  ORN_REQUIRE(d, "detokenizer_last_segment: null argument");
  const std::string seg = d->text.substr(d->offset);
  const int rc = copy_out(seg, out, cap, n_out, "detokenizer_last_segment");
  if (!rc && out) d->offset = d->text.size();  // a size query does not consume the segment
  return rc;
}

int ornith_detokenizer_text(const ornith_detokenizer* d, char* out, size_t cap, size_t* n_out) {
  ORN_REQUIRE(d, "detokenizer_text: null argument");
  return copy_out(d->text, out, cap, n_out, "detokenizer_text");
}

int ornith_text_nfc(const char* text, size_t n, char* out, size_t cap, size_t* n_out) {
  ORN_REQUIRE(text || !n, "text_nfc: null argument");
  std::vector<uint32_t> cps;
  ORN_REQUIRE(utf8_decode(text, n, &cps), "text_nfc: the text is not valid UTF-8");
  std::string s;
  for (uint32_t c : nfc(cps)) utf8_append(s, c);
  return copy_out(s, out, cap, n_out, "text_nfc");
}

int ornith_text_pre_split(const char* text, size_t n, int dialect, size_t* ends_out, size_t cap, size_t* n_out) {
  ORN_REQUIRE((text || !n) && n_out, "text_pre_split: null argument");
  std::vector<uint32_t> cps;
  ORN_REQUIRE(utf8_decode(text, n, &cps), "text_pre_split: the text is not valid UTF-8");
  const Splitter sp{dialect == 0};
  std::vector<size_t> ends;
  size_t bytes = 0;
  for (size_t i = 0; i < cps.size();) {
    const size_t e = sp.match(cps, i);
    for (size_t k = i; k < e; ++k) bytes += cps[k] < 0x80 ? 1 : cps[k] < 0x800 ? 2 : cps[k] < 0x10000 ? 3 : 4;
    ends.push_back(bytes);
    i = e;
  }
  *n_out = ends.size();
  if (!ends_out) return ORNITH_OK;
  ORN_REQUIRE(cap >= ends.size(), "text_pre_split: %zu pieces do not fit the buffer (%zu)", ends.size(), cap);
  if (!ends.empty()) memcpy(ends_out, ends.data(), ends.size() * sizeof(size_t));
  return ORNITH_OK;
}

int ornith_text_char_class(uint32_t cp) {
  // 1 letter or mark, 2 number, 3 white space, 0 other: the classes the split pattern asks about
  if (is_letter(cp) || is_mark(cp)) return 1;
  if (is_number(cp)) return 2;
  if (is_space(cp)) return 3;
  return 0;
}

const char* ornith_tokenizer_split_pattern(int dialect) { return dialect == 0 ? kPatternJson : kPatternTransformers; }

}  // extern "C"
