// Host-side model objects: the named-tensor store, the trunk, the MTP head, the
// caches and the FR-Spec head. Mirrors WeightStore (/root/reference/src/weights.rs),
// TextModel / DecoderLayer / GatedDeltaNet / Attention
// (/root/reference/src/model/qwen3_5.rs), MtpHead (/root/reference/src/model/mtp.rs),
// KvCache / GdnCache (/root/reference/src/model/cache.rs) and FrSpec
// (/root/reference/src/frspec.rs). Everything here is host bookkeeping over device
// pointers; the arithmetic lives in the .hip files.
#pragma once

#include <map>
#include <string>
#include <vector>

#include "rt.h"

struct Tensor {
  int dtype = 0;
  std::vector<int64_t> shape;
  void* d = nullptr;
  size_t bytes = 0;
  int64_t numel() const {
    int64_t n = 1;
    for (auto s : shape) n *= s;
    return n;
  }
};

// One module's entry in config.json's `quantization` block
// (/root/reference/src/weights.rs:31-37).
struct QuantSpec {
  int group_size = 0, bits = 0, mode = ORNITH_QM_AFFINE;
};
struct QuantTable {
  bool loaded = false;
  QuantSpec def;
  std::map<std::string, QuantSpec> per_module;
  // per-module override, else the top-level default (/root/reference/src/weights.rs:96-98)
  QuantSpec lookup(const std::string& path) const {
    auto it = per_module.find(path);
    return it == per_module.end() ? def : it->second;
  }
};
int quant_table_load(const std::string& model_dir, QuantTable* qt);

struct ornith_weights_files;  // the mapped shards behind a store opened from a directory
struct ornith_weights;
const Tensor* ws_fault_in(const ornith_weights* ws, const std::string& name);
void ws_release_files(ornith_weights* ws);

struct ornith_weights {
  ornith_ctx* ctx = nullptr;
  // resident tensors; a store opened from a directory copies each one in on first use
  // (WeightStore::tensor, /root/reference/src/weights.rs:101-108), hence mutable
  mutable std::map<std::string, Tensor> t;
  mutable size_t total_bytes = 0;
  // set when copying a tensor in on first use failed (allocation / upload): find() then
  // returns null for a tensor that does exist, and the caller reports this code instead of
  // "no such tensor" (the message of the failing call is already recorded)
  mutable int fault_rc = 0;
  ornith_weights_files* files = nullptr;
  QuantTable quant;
  const Tensor* find(const std::string& name) const {
    auto it = t.find(name);
    if (it != t.end()) return &it->second;
    return files ? ws_fault_in(this, name) : nullptr;
  }
};

// A lookup came back null: the reason is a failed copy-in if there was one, else a missing tensor.
#define ORN_REQUIRE_TENSOR(ws, t, ...)                               \
  do {                                                               \
    if (!(t)) {                                                      \
      if ((ws)->fault_rc) {                                          \
        const int rc__ = (ws)->fault_rc;                             \
        (ws)->fault_rc = 0;                                          \
        return rc__;                                                 \
      }                                                              \
      return ornith_fail(ORNITH_ERR_INVALID, __VA_ARGS__);           \
    }                                                                \
  } while (0)

// After lookups that may legitimately come back null (an optional tensor): a failed copy-in
// is reported as itself rather than read as "the tensor is absent".
#define ORN_RETURN_FAULT(ws)               \
  do {                                     \
    if ((ws)->fault_rc) {                  \
      const int rc__ = (ws)->fault_rc;     \
      (ws)->fault_rc = 0;                  \
      return rc__;                         \
    }                                      \
  } while (0)

// Resolves module `path` into a Linear by the tensors present (k-quant / affine8 / dense).
int ws_linear(const ornith_weights* ws, const std::string& path, ornith_linear* out);
// A routed k-quant module [E, O, K].
int ws_kmatrix(const ornith_weights* ws, const std::string& path, ornith_kmatrix* out);
// A plain tensor with an expected element count and dtype.
int ws_tensor(const ornith_weights* ws, const std::string& name, int dtype, int64_t numel,
              const void** out);
// <prefix>.<e>.<suffix> for e in 0..experts copied into one [experts, ...] tensor, kept under
// "<prefix>.*.<suffix>" (WeightStore::stacked_experts, /root/reference/src/weights.rs:237-279).
int ws_stacked(const ornith_weights* ws, const std::string& prefix, const std::string& suffix,
               int experts, int dtype, int64_t numel, const void** out);
size_t ornith_dt_size(int dt);

struct GdnLayer {
  ornith_linear in_proj_qkv, in_proj_z, out_proj, in_proj_a, in_proj_b;
  const void *conv1d, *dt_bias, *a_log, *norm;
};
struct AttnLayer {
  ornith_linear q_proj, k_proj, v_proj, o_proj;
  const void *q_norm, *k_norm;
};
struct Layer {
  bool linear = false;
  const void *input_ln = nullptr, *post_ln = nullptr;
  GdnLayer gdn{};
  AttnLayer attn{};
  ornith_moe_weights moe{};
};

struct ornith_model {
  ornith_ctx* ctx = nullptr;
  ornith_text_config cfg{};
  ornith_linear embed_tokens{};
  ornith_linear lm_head{};
  const void* final_norm = nullptr;
  std::vector<Layer> layers;
  // step buffers, sized for `max_rows` activation rows
  int max_rows = 0;
  void* ws_buf = nullptr;
  size_t ws_bytes = 0;
  // rope tables, grown on demand to the largest cache capacity seen
  float *d_cos = nullptr, *d_sin = nullptr;
  int rope_npos = 0;
  int key_dim() const { return cfg.linear_num_key_heads * cfg.linear_key_head_dim; }
  int value_dim() const { return cfg.linear_num_value_heads * cfg.linear_value_head_dim; }
  int conv_dim() const { return 2 * key_dim() + value_dim(); }
};

struct LayerCache {
  // full attention
  void *k = nullptr, *v = nullptr;  // bf16 [Hkv, cap, hd]
  // gated delta
  void* conv[2] = {nullptr, nullptr};  // bf16 [K-1+max_rows, D] each
  float* state = nullptr;              // f32 [slots][Hv, Dv, Dk]
};

struct ornith_caches {
  ornith_model* m = nullptr;
  int capacity = 0, max_window = 0, conv_rows = 0;
  bool growable = true;  // a forward past the capacity grows the KV tensors (else it is refused)
  std::vector<LayerCache> layers;
  // one set of cursors serves every layer: they all advance together
  int offset = 0;     // tokens held
  int conv_cur = 0;   // which conv buffer holds the live window
  int conv_off = 0;   // first row of the live K-1 rows in it
  int state_cur = 0;  // slot holding the live recurrent state
  int last_T = 0;     // rows of the last forward (for rewind)
  bool last_capture = false;
};

struct ornith_frspec {
  ornith_model* m = nullptr;
  int n = 0, vocab = 0;
  std::vector<uint32_t> ids;
  uint32_t* d_ids = nullptr;
  ornith_linear head{};
  void* owned[3] = {nullptr, nullptr, nullptr};
};

struct ornith_mtp_head {
  ornith_model* m = nullptr;
  const void *pre_fc_norm_embedding, *pre_fc_norm_hidden, *input_ln, *post_ln, *norm;
  ornith_linear fc;
  AttnLayer attn{};
  ornith_moe_weights moe{};
  // one-layer KV cache
  void *k = nullptr, *v = nullptr;
  int capacity = 0, offset = 0;
  bool growable = true;
  void* buf = nullptr;  // step buffers
  int max_rows = 0;
  // tokens that replace the drafts (ornith_mtp_force_drafts), indexed by output position
  uint32_t* d_forced = nullptr;
  size_t n_forced = 0;
};

// grows the model's RoPE tables to cover `npos` positions
int model_ensure_rope(ornith_model* m, int npos);
// What a loop asks before it starts: `rows` rows must fit. Growable caches always say yes (they
// grow as the rows arrive); fixed ones are checked against their capacity.
inline bool caches_fit(const ornith_caches* c, size_t rows) { return c->growable || rows <= (size_t)c->capacity; }
inline bool mtp_cache_fits(const ornith_mtp_head* h, size_t rows) { return h->growable || rows <= (size_t)h->capacity; }
