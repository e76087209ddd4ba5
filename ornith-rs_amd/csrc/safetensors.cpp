// Reading a model artifact from disk: a small JSON reader, memory-mapped safetensors
// shards, config.json's text and quantization blocks, and the store that hands tensors to
// the device on first use.
//
//   SafeTensors::{open, open_many, add_file, get, bytes}  /root/reference/src/safetensors.rs:196-285
//   shards_from_index                                      /root/reference/src/safetensors.rs:296-310
//   WeightStore::{open, quant_config, tensor}              /root/reference/src/weights.rs:41-122
//   WeightStore::stacked_experts                           /root/reference/src/weights.rs:237-279
//   TextConfig::from_value                                 /root/reference/src/model/config.rs:53-133
//   QuantMode::from_config                                 /root/reference/src/ops/quantized.rs:60-75
//
// A shard is `u64 header_len`, a JSON object {name: {dtype, shape, data_offsets}} and the
// tensor bytes packed back to back. Tensors start on odd byte offsets, so each one is copied
// into its own device allocation; the mapping is only ever read.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cmath>
#include <cstdlib>
#include <memory>

#include "json.h"
#include "model.h"

namespace {
using namespace orn_json;

// ------------------------------------------------------------------ mapped shards
struct Mapping {
  void* addr = nullptr;
  size_t map_len = 0, file_len = 0;
  Mapping() = default;
  Mapping(const Mapping&) = delete;
  Mapping& operator=(const Mapping&) = delete;
  ~Mapping() {
    if (addr) munmap(addr, map_len);
  }
  bool open(const std::string& path, std::string* err) {
    const int fd = ::open(path.c_str(), O_RDONLY);
    if (fd < 0) {
      *err = "mmap " + path + ": " + strerror(errno);
      return false;
    }
    struct stat st;
    if (fstat(fd, &st) != 0) {
      *err = "stat " + path + ": " + strerror(errno);
      ::close(fd);
      return false;
    }
    file_len = (size_t)st.st_size;
    map_len = file_len ? file_len : 1;
    if (file_len) {
      addr = mmap(nullptr, map_len, PROT_READ, MAP_PRIVATE, fd, 0);
      if (addr == MAP_FAILED) {
        addr = nullptr;
        *err = "mmap " + path + ": " + strerror(errno);
        ::close(fd);
        return false;
      }
    }
    ::close(fd);
    return true;
  }
  void will_need() const {
    if (addr) madvise(addr, map_len, MADV_WILLNEED);
  }
  const uint8_t* bytes() const { return (const uint8_t*)addr; }
};

struct DtName {
  const char* name;
  int dt;
};
const DtName kDtNames[] = {
    {"F32", ORNITH_DT_F32},   {"BF16", ORNITH_DT_BF16}, {"F16", ORNITH_DT_F16}, {"U8", ORNITH_DT_U8},
    {"U32", ORNITH_DT_U32},   {"I32", ORNITH_DT_I32},   {"I8", ORNITH_DT_I8},   {"I16", ORNITH_DT_I16},
    {"U16", ORNITH_DT_U16},   {"I64", ORNITH_DT_I64},   {"U64", ORNITH_DT_U64}, {"F64", ORNITH_DT_F64},
    {"BOOL", ORNITH_DT_BOOL},
};

}  // namespace

size_t ornith_dt_size(int dt) {
  switch (dt) {
    case ORNITH_DT_F64: case ORNITH_DT_I64: case ORNITH_DT_U64: return 8;
    case ORNITH_DT_F32: case ORNITH_DT_U32: case ORNITH_DT_I32: return 4;
    case ORNITH_DT_BF16: case ORNITH_DT_F16: case ORNITH_DT_I16: case ORNITH_DT_U16: return 2;
    case ORNITH_DT_U8: case ORNITH_DT_I8: case ORNITH_DT_BOOL: return 1;
    default: return 0;
  }
}

struct StTensor {
  int file = 0, dtype = 0;
  std::vector<int64_t> shape;
  size_t offset = 0, nbytes = 0;  // offset from the start of the file
};

struct ornith_safetensors {
  std::vector<std::unique_ptr<Mapping>> files;
  std::map<std::string, StTensor> tensors;
  std::vector<const std::string*> order;  // names, sorted (the map's own order)

  const StTensor* get(const std::string& name) const {
    auto it = tensors.find(name);
    return it == tensors.end() ? nullptr : &it->second;
  }
  const uint8_t* bytes(const StTensor& t) const { return files[t.file]->bytes() + t.offset; }

  int add_file(const std::string& path) {
    std::unique_ptr<Mapping> map(new Mapping());
    std::string err;
    if (!map->open(path, &err)) return ornith_fail(ORNITH_ERR_IO, "%s", err.c_str());
    if (map->file_len < 8)
      return ornith_fail(ORNITH_ERR_IO, "%s: too short for a safetensors header", path.c_str());
    uint64_t hdr_len = 0;
    for (int i = 7; i >= 0; --i) hdr_len = (hdr_len << 8) | map->bytes()[i];
    if (hdr_len > map->file_len - 8)
      return ornith_fail(ORNITH_ERR_IO, "%s: header length %llu past EOF", path.c_str(),
                         (unsigned long long)hdr_len);
    JVal header;
    if (!json_parse((const char*)map->bytes() + 8, (size_t)hdr_len, &header, &err))
      return ornith_fail(ORNITH_ERR_IO, "%s: %s", path.c_str(), err.c_str());
    if (header.kind != JVal::Obj)
      return ornith_fail(ORNITH_ERR_IO, "%s: header is not an object", path.c_str());
    const size_t data_start = 8 + (size_t)hdr_len;
    const int file_idx = (int)files.size();
    for (auto& kv : header.obj) {
      const std::string& name = kv.first;
      if (name == "__metadata__") continue;
      const JVal& meta = kv.second;
      const JVal* jd = meta.get("dtype");
      if (!jd || jd->kind != JVal::Str)
        return ornith_fail(ORNITH_ERR_IO, "%s: missing dtype", name.c_str());
      StTensor t;
      t.file = file_idx;
      t.dtype = -1;
      for (auto& d : kDtNames)
        if (jd->str == d.name) t.dtype = d.dt;
      if (t.dtype < 0)
        return ornith_fail(ORNITH_ERR_IO, "%s: unsupported dtype %s", name.c_str(), jd->str.c_str());
      const JVal* js = meta.get("shape");
      if (!js || js->kind != JVal::Arr)
        return ornith_fail(ORNITH_ERR_IO, "%s: missing shape", name.c_str());
      if (js->arr.size() > 8)
        return ornith_fail(ORNITH_ERR_IO, "%s: %zu dims", name.c_str(), js->arr.size());
      size_t numel = 1;
      for (auto& d : js->arr) {
        size_t v = 0;
        if (!d.as_usize(&v)) return ornith_fail(ORNITH_ERR_IO, "%s: bad shape entry", name.c_str());
        t.shape.push_back((int64_t)v);
        if (v && numel > SIZE_MAX / v)
          return ornith_fail(ORNITH_ERR_IO, "%s: shape overflows", name.c_str());
        numel *= v;
      }
      const JVal* jo = meta.get("data_offsets");
      size_t begin = 0, end = 0;
      if (!jo || jo->kind != JVal::Arr || jo->arr.size() != 2 || !jo->arr[0].as_usize(&begin) ||
          !jo->arr[1].as_usize(&end) || end < begin)
        return ornith_fail(ORNITH_ERR_IO, "%s: missing data_offsets", name.c_str());
      t.nbytes = end - begin;
      const size_t expect = numel * ornith_dt_size(t.dtype);
      if (t.nbytes != expect)
        return ornith_fail(ORNITH_ERR_IO,
                           "%s: data_offsets span %zu bytes but its shape x %s needs %zu",
                           name.c_str(), t.nbytes, jd->str.c_str(), expect);
      if (end > map->file_len - data_start)
        return ornith_fail(ORNITH_ERR_IO, "%s: data past EOF in %s", name.c_str(), path.c_str());
      t.offset = data_start + begin;
      tensors[name] = std::move(t);  // a later file wins, as HashMap::insert does
    }
    files.push_back(std::move(map));
    return ORNITH_OK;
  }
  void index() {
    order.clear();
    for (auto& kv : tensors) order.push_back(&kv.first);
  }
};

// model.safetensors.index.json -> the shard paths, sorted and de-duplicated.
static int shards_from_index(const std::string& dir, std::vector<std::string>* out) {
  const std::string idx_path = dir + "/model.safetensors.index.json";
  JVal idx;
  std::string err;
  if (!json_file(idx_path, &idx, &err)) return ornith_fail(ORNITH_ERR_IO, "%s", err.c_str());
  const JVal* map = idx.get("weight_map");
  if (!map || map->kind != JVal::Obj)
    return ornith_fail(ORNITH_ERR_IO, "%s: no weight_map", idx_path.c_str());
  std::vector<std::string> files;
  for (auto& kv : map->obj)
    if (kv.second.kind == JVal::Str) files.push_back(kv.second.str);
  std::sort(files.begin(), files.end());
  files.erase(std::unique(files.begin(), files.end()), files.end());
  for (auto& f : files) out->push_back(dir + "/" + f);
  return ORNITH_OK;
}

static int open_paths(const std::vector<std::string>& paths, ornith_safetensors** out) {
  std::unique_ptr<ornith_safetensors> st(new ornith_safetensors());
  for (auto& p : paths) {
    int rc = st->add_file(p);
    if (rc) return rc;
  }
  st->index();
  *out = st.release();
  return ORNITH_OK;
}

// ------------------------------------------------------------------ config.json
static int quant_mode_from(const std::string& s, int* mode) {
  if (s == "affine") *mode = ORNITH_QM_AFFINE;
  else if (s == "q4k") *mode = ORNITH_QM_Q4K;
  else if (s == "q6k") *mode = ORNITH_QM_Q6K;
  else if (s == "nvfp4" || s == "mxfp4" || s == "mxfp8")
    return ornith_fail(ORNITH_ERR_UNSUPPORTED,
                       "quantization mode \"%s\" is not carried by this library", s.c_str());
  else
    return ornith_fail(ORNITH_ERR_INVALID, "unknown quantization mode \"%s\"", s.c_str());
  return ORNITH_OK;
}

int quant_table_load(const std::string& dir, QuantTable* qt) {
  JVal cfg;
  std::string err;
  if (!json_file(dir + "/config.json", &cfg, &err))
    return ornith_fail(ORNITH_ERR_IO, "config.json: %s", err.c_str());
  const JVal* q = cfg.get("quantization");
  ORN_REQUIRE(q && q->kind == JVal::Obj, "config.json has no quantization block");
  size_t gs = 0, bits = 0;
  const JVal* v = q->get("group_size");
  ORN_REQUIRE(v && v->as_usize(&gs), "quantization.group_size");
  v = q->get("bits");
  ORN_REQUIRE(v && v->as_usize(&bits), "quantization.bits");
  // artifacts older than the fp modes carry no `mode`; it defaults to affine
  std::string mode = "affine";
  v = q->get("mode");
  if (v && v->kind == JVal::Str) mode = v->str;
  qt->def.group_size = (int)gs;
  qt->def.bits = (int)bits;
  int rc = quant_mode_from(mode, &qt->def.mode);
  if (rc) return rc;
  for (auto& kv : q->obj) {
    if (kv.second.kind != JVal::Obj) continue;
    QuantSpec s = qt->def;
    size_t x;
    const JVal* o = kv.second.get("group_size");
    if (o && o->as_usize(&x)) s.group_size = (int)x;
    o = kv.second.get("bits");
    if (o && o->as_usize(&x)) s.bits = (int)x;
    o = kv.second.get("mode");
    if (o && o->kind == JVal::Str) {
      rc = quant_mode_from(o->str, &s.mode);
      if (rc) return rc;
    }
    qt->per_module[kv.first] = s;
  }
  qt->loaded = true;
  return ORNITH_OK;
}

static int text_config_from(const JVal& cfg, ornith_text_config* c, int* mtp_layers) {
  // the text model's keys sit under `text_config` when the artifact also has a vision tower
  const JVal* t = cfg.get("text_config");
  if (!t) t = &cfg;
  int rc = ORNITH_OK;
  auto need = [&](const char* k, int* out) {
    size_t v = 0;
    const JVal* j = t->get(k);
    if (!j || !j->as_usize(&v)) {
      if (!rc) rc = ornith_fail(ORNITH_ERR_INVALID, "config.json: missing %s", k);
      return;
    }
    *out = (int)v;
  };
  auto opt = [&](const char* k, int d) {
    size_t v = 0;
    const JVal* j = t->get(k);
    return j && j->as_usize(&v) ? (int)v : d;
  };
  auto num = [&](const JVal* o, const char* k, float d) {
    const JVal* j = o ? o->get(k) : nullptr;
    return j && j->kind == JVal::Num ? (float)j->num : d;
  };
  memset(c, 0, sizeof *c);
  need("hidden_size", &c->hidden_size);
  need("num_attention_heads", &c->num_attention_heads);
  need("num_hidden_layers", &c->num_hidden_layers);
  need("num_key_value_heads", &c->num_key_value_heads);
  need("vocab_size", &c->vocab_size);
  need("linear_num_value_heads", &c->linear_num_value_heads);
  need("linear_num_key_heads", &c->linear_num_key_heads);
  need("linear_key_head_dim", &c->linear_key_head_dim);
  need("linear_value_head_dim", &c->linear_value_head_dim);
  need("linear_conv_kernel_dim", &c->linear_conv_kernel_dim);
  if (rc) return rc;
  ORN_REQUIRE(c->num_attention_heads > 0, "config.json: num_attention_heads is 0");
  c->head_dim = opt("head_dim", c->hidden_size / c->num_attention_heads);
  c->rms_norm_eps = num(t, "rms_norm_eps", 1e-6f);
  c->full_attention_interval = opt("full_attention_interval", 4);
  c->num_experts = opt("num_experts", 0);
  c->num_experts_per_tok = opt("num_experts_per_tok", 0);
  c->moe_intermediate_size = opt("moe_intermediate_size", 0);
  c->shared_expert_intermediate_size = opt("shared_expert_intermediate_size", 0);
  const JVal* ntp = t->get("norm_topk_prob");
  c->norm_topk_prob = ntp && ntp->kind == JVal::Bool ? (ntp->b ? 1 : 0) : 1;
  // rope settings live in `rope_parameters` when present; both are read as fp32
  const JVal* rope = t->get("rope_parameters");
  c->rope_theta = (double)num(rope, "rope_theta", num(t, "rope_theta", 100000.0f));
  const float prf = num(rope, "partial_rotary_factor", num(t, "partial_rotary_factor", 0.25f));
  c->rope_dims = (int)((float)c->head_dim * prf);
  if (mtp_layers) {
    size_t v = 0;
    const JVal* j = cfg.get("num_nextn_predict_layers");
    if (!j) j = t->get("num_nextn_predict_layers");
    *mtp_layers = j && j->as_usize(&v) ? (int)v : 0;
  }
  return ORNITH_OK;
}

// ------------------------------------------------------------------ the store's file side
struct ornith_weights_files {
  ornith_safetensors* st = nullptr;
  ~ornith_weights_files() { delete st; }
};

void ws_release_files(ornith_weights* ws) {
  delete ws->files;
  ws->files = nullptr;
}

// First use of a tensor that lives in a mapped shard: allocate and copy.
const Tensor* ws_fault_in(const ornith_weights* ws, const std::string& name) {
  if (!ws->files) return nullptr;
  const ornith_safetensors* st = ws->files->st;
  const StTensor* info = st->get(name);
  if (!info) return nullptr;
  if (info->nbytes == 0) {
    ws->fault_rc = ornith_fail(ORNITH_ERR_INVALID, "%s: empty tensor", name.c_str());
    return nullptr;
  }
  Tensor t;
  t.dtype = info->dtype;
  t.shape = info->shape;
  t.bytes = info->nbytes;
  if (int rc = ornith_alloc(ws->ctx, t.bytes, &t.d)) {
    ws->fault_rc = rc;
    return nullptr;
  }
  if (int rc = ornith_upload(ws->ctx, t.d, st->bytes(*info), t.bytes)) {
    ornith_free(ws->ctx, t.d);
    ws->fault_rc = rc;
    return nullptr;
  }
  ws->total_bytes += t.bytes;
  auto it = ws->t.emplace(name, std::move(t)).first;
  return &it->second;
}

int ws_stacked(const ornith_weights* ws, const std::string& prefix, const std::string& suffix,
               int experts, int dtype, int64_t numel, const void** out) {
  const std::string key = prefix + ".*." + suffix;
  auto hit = ws->t.find(key);
  if (hit != ws->t.end()) {
    ORN_REQUIRE(hit->second.dtype == dtype && hit->second.numel() == numel,
                "%s: stacked tensor disagrees with the config", key.c_str());
    *out = hit->second.d;
    return ORNITH_OK;
  }
  ORN_REQUIRE(ws->files, "%s.0.%s: no such tensor", prefix.c_str(), suffix.c_str());
  const ornith_safetensors* st = ws->files->st;
  const StTensor* first = st->get(prefix + ".0." + suffix);
  ORN_REQUIRE(first, "no tensor named %s.0.%s", prefix.c_str(), suffix.c_str());
  ORN_REQUIRE(first->dtype == dtype, "%s.0.%s: dtype %d, expected %d", prefix.c_str(),
              suffix.c_str(), first->dtype, dtype);
  const size_t stride = first->nbytes;
  ORN_REQUIRE(experts >= 1 && stride > 0, "%s: nothing to stack", key.c_str());
  Tensor t;
  t.dtype = dtype;
  t.shape.push_back(experts);
  for (auto s : first->shape) t.shape.push_back(s);
  t.bytes = stride * (size_t)experts;
  ORN_REQUIRE(t.numel() == numel, "%s: %lld elements, expected %lld", key.c_str(),
              (long long)t.numel(), (long long)numel);
  int rc = ornith_alloc(ws->ctx, t.bytes, &t.d);
  if (rc) return rc;
  for (int e = 0; e < experts && !rc; ++e) {
    const std::string name = prefix + "." + std::to_string(e) + "." + suffix;
    const StTensor* info = st->get(name);
    if (!info) rc = ornith_fail(ORNITH_ERR_INVALID, "no tensor named %s", name.c_str());
    else if (info->shape != first->shape)
      rc = ornith_fail(ORNITH_ERR_INVALID, "%s has a different shape from expert 0", name.c_str());
    else if (info->dtype != first->dtype)
      rc = ornith_fail(ORNITH_ERR_INVALID, "%s has a different dtype from expert 0", name.c_str());
    else
      rc = ornith_upload(ws->ctx, (uint8_t*)t.d + (size_t)e * stride, st->bytes(*info), stride);
  }
  if (rc) {
    ornith_free(ws->ctx, t.d);
    return rc;
  }
  ws->total_bytes += t.bytes;
  *out = t.d;
  ws->t.emplace(key, std::move(t));
  return ORNITH_OK;
}

// ------------------------------------------------------------------ C ABI
extern "C" {

int ornith_safetensors_open(const char* const* paths, int n_paths, ornith_safetensors** out) {
  ORN_REQUIRE(out && n_paths >= 0 && (n_paths == 0 || paths), "safetensors_open: null argument");
  std::vector<std::string> v;
  for (int i = 0; i < n_paths; ++i) {
    ORN_REQUIRE(paths[i], "safetensors_open: path %d is null", i);
    v.push_back(paths[i]);
  }
  return open_paths(v, out);
}

int ornith_safetensors_open_model(const char* model_dir, const char* const* extra, int n_extra,
                                  ornith_safetensors** out) {
  ORN_REQUIRE(model_dir && out && n_extra >= 0 && (n_extra == 0 || extra),
              "safetensors_open_model: null argument");
  std::vector<std::string> v;
  int rc = shards_from_index(model_dir, &v);
  if (rc) return rc;
  for (int i = 0; i < n_extra; ++i) {
    ORN_REQUIRE(extra[i], "safetensors_open_model: extra path %d is null", i);
    v.push_back(extra[i]);
  }
  return open_paths(v, out);
}

int ornith_safetensors_close(ornith_safetensors* st) {
  delete st;
  return ORNITH_OK;
}

int ornith_safetensors_count(const ornith_safetensors* st, int64_t* n_tensors, int64_t* n_files) {
  ORN_REQUIRE(st, "safetensors_count: null handle");
  if (n_tensors) *n_tensors = (int64_t)st->tensors.size();
  if (n_files) *n_files = (int64_t)st->files.size();
  return ORNITH_OK;
}

int ornith_safetensors_name(const ornith_safetensors* st, int64_t i, const char** name) {
  ORN_REQUIRE(st && name, "safetensors_name: null argument");
  ORN_REQUIRE(i >= 0 && i < (int64_t)st->order.size(), "safetensors_name: index %lld of %zu",
              (long long)i, st->order.size());
  *name = st->order[(size_t)i]->c_str();
  return ORNITH_OK;
}

int ornith_safetensors_info(const ornith_safetensors* st, const char* name, int* dtype,
                            int64_t* shape, int* ndim, const void** data, size_t* nbytes) {
  ORN_REQUIRE(st && name, "safetensors_info: null argument");
  const StTensor* t = st->get(name);
  ORN_REQUIRE(t, "no tensor named %s", name);
  if (dtype) *dtype = t->dtype;
  if (ndim) *ndim = (int)t->shape.size();
  if (shape)
    for (size_t i = 0; i < t->shape.size(); ++i) shape[i] = t->shape[i];
  if (data) *data = st->bytes(*t);
  if (nbytes) *nbytes = t->nbytes;
  return ORNITH_OK;
}

int ornith_text_config_load(const char* model_dir, ornith_text_config* out, int* mtp_layers) {
  ORN_REQUIRE(model_dir && out, "text_config_load: null argument");
  JVal cfg;
  std::string err;
  if (!json_file(std::string(model_dir) + "/config.json", &cfg, &err))
    return ornith_fail(ORNITH_ERR_IO, "config.json: %s", err.c_str());
  return text_config_from(cfg, out, mtp_layers);
}

int ornith_quant_config_load(const char* model_dir, const char* module_path, int* group_size,
                             int* bits, int* mode) {
  ORN_REQUIRE(model_dir && module_path, "quant_config_load: null argument");
  QuantTable qt;
  int rc = quant_table_load(model_dir, &qt);
  if (rc) return rc;
  const QuantSpec s = qt.lookup(module_path);
  if (group_size) *group_size = s.group_size;
  if (bits) *bits = s.bits;
  if (mode) *mode = s.mode;
  return ORNITH_OK;
}

int ornith_weights_open(ornith_ctx* ctx, const char* model_dir, const char* const* extra,
                        int n_extra, ornith_weights** out) {
  ORN_REQUIRE(ctx && model_dir && out, "weights_open: null argument");
  std::unique_ptr<ornith_weights_files> files(new ornith_weights_files());
  int rc = ornith_safetensors_open_model(model_dir, extra, n_extra, &files->st);
  if (rc) return rc;
  QuantTable qt;
  rc = quant_table_load(model_dir, &qt);
  if (rc) return rc;
  for (auto& f : files->st->files) f->will_need();
  ornith_weights* w = new ornith_weights();
  w->ctx = ctx;
  w->files = files.release();
  w->quant = std::move(qt);
  *out = w;
  return ORNITH_OK;
}

int ornith_weights_quant_config(const ornith_weights* ws, const char* module_path,
                                int* group_size, int* bits, int* mode) {
  ORN_REQUIRE(ws && module_path, "weights_quant_config: null argument");
  ORN_REQUIRE(ws->quant.loaded, "weights_quant_config: the store was not opened from a model directory");
  const QuantSpec s = ws->quant.lookup(module_path);
  if (group_size) *group_size = s.group_size;
  if (bits) *bits = s.bits;
  if (mode) *mode = s.mode;
  return ORNITH_OK;
}

int ornith_weights_has(const ornith_weights* ws, const char* name) {
  if (!ws || !name) return 0;
  if (ws->t.count(name)) return 1;
  return ws->files && ws->files->st->get(name) ? 1 : 0;
}

int ornith_weights_fetch(const ornith_weights* ws, const char* name, int* dtype, int64_t* shape,
                         int* ndim, void* host_out, size_t host_bytes) {
  ORN_REQUIRE(ws && name, "weights_fetch: null argument");
  const Tensor* t = ws->find(name);
  ORN_REQUIRE_TENSOR(ws, t, "no tensor named %s", name);
  if (dtype) *dtype = t->dtype;
  if (ndim) *ndim = (int)t->shape.size();
  if (shape)
    for (size_t i = 0; i < t->shape.size(); ++i) shape[i] = t->shape[i];
  if (host_out) {
    ORN_REQUIRE(host_bytes == t->bytes, "weights_fetch: %s holds %zu bytes, buffer has %zu", name,
                t->bytes, host_bytes);
    return ornith_download(ws->ctx, host_out, t->d, t->bytes);
  }
  return ORNITH_OK;
}

}  // extern "C"
