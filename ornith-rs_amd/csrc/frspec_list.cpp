// FR-Spec id lists on the host: the file format, the default location, and the superset
// merge.
//
// Mirrors /root/reference/src/frspec.rs:101-135 (file = u32 n, then n x u32 little endian;
// the same four rejections), :153-158 (default_path: ORNITH_FRSPEC, else
// <refs root>/frspec/ids_64k.bin with the refs root from ORNITH_REFS, src/refs.rs:179-184) and
// the list arithmetic of /root/reference/tools/merge_frspec.py:74-92,176-204: a merged list
// only ever ADDS to the base list (ids a corpus used at least min_count times and the base
// lacks, plus an explicit extra set such as every id of one script), is written sorted and
// de-duplicated, and must stay a strict pruning of the vocabulary. Tokenizing a corpus is
// the caller's business: this takes token ids.
#include <algorithm>
#include <cstdlib>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "rt.h"

// reads and validates a list file; on success ids holds the n ids in file order
int frspec_read_file(const char* path, std::vector<uint32_t>& ids) {
  FILE* fp = fopen(path, "rb");
  if (!fp) return ornith_fail(ORNITH_ERR_IO, "%s: cannot open", path);
  fseek(fp, 0, SEEK_END);
  const long size = ftell(fp);
  fseek(fp, 0, SEEK_SET);
  uint32_t n = 0;
  if (size < 4 || fread(&n, 4, 1, fp) != 1) {
    fclose(fp);
    return ornith_fail(ORNITH_ERR_IO, "%s: %ld bytes is too short to hold a count", path, size);
  }
  if (size != 4 + 4 * (long)n) {
    fclose(fp);
    return ornith_fail(ORNITH_ERR_IO, "%s: says %u ids but carries %ld bytes", path, n, size - 4);
  }
  ids.resize(n);
  const size_t got = n ? fread(ids.data(), 4, n, fp) : 0;
  fclose(fp);
  if (got != n) return ornith_fail(ORNITH_ERR_IO, "%s: short read", path);
  return ORNITH_OK;
}

extern "C" {

int ornith_frspec_default_path(char* buf, size_t len) {
  ORN_REQUIRE(buf && len > 0, "frspec_default_path: null buffer");
  std::string p;
  if (const char* e = getenv("ORNITH_FRSPEC")) {
    p = e;
  } else {
    const char* r = getenv("ORNITH_REFS");
    p = std::string(r ? r : "refs") + "/frspec/ids_64k.bin";
  }
  ORN_REQUIRE(p.size() + 1 <= len, "frspec_default_path: the path needs %zu bytes, the buffer has %zu", p.size() + 1, len);
  memcpy(buf, p.c_str(), p.size() + 1);
  return ORNITH_OK;
}

int ornith_frspec_read_ids(const char* path, uint32_t* ids_out, size_t cap, size_t* n_out) {
  ORN_REQUIRE(path && n_out, "frspec_read_ids: null argument");
  std::vector<uint32_t> ids;
  if (int rc = frspec_read_file(path, ids)) return rc;
  *n_out = ids.size();
  if (!ids_out) return ORNITH_OK;  // size query
  ORN_REQUIRE(cap >= ids.size(), "frspec_read_ids: %zu ids do not fit a buffer of %zu", ids.size(), cap);
  if (!ids.empty()) memcpy(ids_out, ids.data(), 4 * ids.size());
  return ORNITH_OK;
}

int ornith_frspec_write_ids(const char* path, const uint32_t* ids, size_t n, uint32_t vocab, size_t* n_written) {
  ORN_REQUIRE(path && (ids || n == 0), "frspec_write_ids: null argument");
  std::vector<uint32_t> v(ids, ids + n);
  std::sort(v.begin(), v.end());
  v.erase(std::unique(v.begin(), v.end()), v.end());
  ORN_REQUIRE(!v.empty(), "frspec_write_ids: no ids");
  ORN_REQUIRE(v.size() < vocab, "frspec_write_ids: %zu ids is not a pruning of %u", v.size(), vocab);
  ORN_REQUIRE(v.back() < vocab, "frspec_write_ids: an id is outside the %u-row vocabulary", vocab);
  FILE* fp = fopen(path, "wb");
  if (!fp) return ornith_fail(ORNITH_ERR_IO, "%s: cannot create", path);
  const uint32_t cnt = (uint32_t)v.size();
  const bool ok = fwrite(&cnt, 4, 1, fp) == 1 && fwrite(v.data(), 4, v.size(), fp) == v.size();
  if (fclose(fp) != 0 || !ok) return ornith_fail(ORNITH_ERR_IO, "%s: write failed", path);
  if (n_written) *n_written = v.size();
  return ORNITH_OK;
}

int ornith_frspec_merge(const uint32_t* base, size_t n_base, const uint32_t* corpus, size_t n_corpus,
                        uint32_t min_count, const uint32_t* extra, size_t n_extra, uint32_t vocab,
                        uint32_t* out, size_t out_cap, ornith_frspec_merge_stats* stats) {
  ORN_REQUIRE(base && n_base > 0 && stats, "frspec_merge: null argument");
  ORN_REQUIRE((corpus || n_corpus == 0) && (extra || n_extra == 0), "frspec_merge: null list");
  ORN_REQUIRE(n_corpus > 0 || n_extra > 0, "frspec_merge: nothing to add: give a corpus, or extra ids, or both");
  std::unordered_set<uint32_t> inside(base, base + n_base);
  for (size_t i = 0; i < n_base; ++i) ORN_REQUIRE(base[i] < vocab, "frspec_merge: a base id is outside the vocabulary");
  std::unordered_map<uint32_t, uint64_t> missing;
  uint64_t covered = 0;
  for (size_t i = 0; i < n_corpus; ++i) {
    ORN_REQUIRE(corpus[i] < vocab, "frspec_merge: corpus token %u is outside the %u-row vocabulary", corpus[i], vocab);
    if (inside.count(corpus[i])) ++covered;
    else ++missing[corpus[i]];
  }
  std::vector<uint32_t> merged(base, base + n_base);
  uint64_t after = covered;
  size_t kept = 0;
  for (const auto& kv : missing)
    if (kv.second >= min_count) {
      merged.push_back(kv.first);
      after += kv.second;
      ++kept;
    }
  size_t extra_new = 0;
  std::unordered_set<uint32_t> extra_seen;
  for (size_t i = 0; i < n_extra; ++i) {
    ORN_REQUIRE(extra[i] < vocab, "frspec_merge: an extra id is outside the vocabulary");
    if (!inside.count(extra[i]) && extra_seen.insert(extra[i]).second) ++extra_new;
    merged.push_back(extra[i]);
  }
  std::sort(merged.begin(), merged.end());
  merged.erase(std::unique(merged.begin(), merged.end()), merged.end());
  ORN_REQUIRE(merged.size() < vocab, "frspec_merge: %zu ids is not a pruning of %u", merged.size(), vocab);
  stats->n_merged = merged.size();
  stats->corpus_tokens = n_corpus;
  stats->covered_before = covered;
  stats->covered_after = after;
  stats->missing_distinct = missing.size();
  stats->missing_kept = kept;
  stats->extra_new = extra_new;
  if (!out) return ORNITH_OK;  // size query
  ORN_REQUIRE(out_cap >= merged.size(), "frspec_merge: %zu ids do not fit a buffer of %zu", merged.size(), out_cap);
  memcpy(out, merged.data(), 4 * merged.size());
  return ORNITH_OK;
}

}  // extern "C"
