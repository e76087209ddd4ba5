// The named-tensor store and the module resolution rules of
// WeightStore::{tensor, linear, kquant_matrix, quant_matrix}
// (/root/reference/src/weights.rs:101-227): a module <path> is
//   k-quant   <path>.weight (u32 / u8 codes), <path>.scales (u8), <path>.dm (f16)
//   affine 8  <path>.weight (u32 / u8), <path>.scales (bf16), <path>.biases (bf16)
//   dense     <path>.weight (bf16)
// with the tensor shapes of /root/reference/src/ops/kquant.rs:20-26.
#include "model.h"

// config.json's mode for a module must agree with the tensors the artifact holds for it
// (/root/reference/src/weights.rs:132-150, 199-220); stores filled by ornith_weights_put carry
// no config and resolve by the tensors alone.
static int check_mode(const ornith_weights* ws, const std::string& path, bool is_k, int kind) {
  if (!ws->quant.loaded) return ORNITH_OK;
  const QuantSpec s = ws->quant.lookup(path);
  const bool says_k = s.mode == ORNITH_QM_Q4K || s.mode == ORNITH_QM_Q6K;
  if (is_k) {
    ORN_REQUIRE(says_k, "%s holds a .dm tensor but config.json's quantization block says affine",
                path.c_str());
    ORN_REQUIRE(s.group_size == 256, "%s: a k-quant's super-block is 256 weights, not %d",
                path.c_str(), s.group_size);
    ORN_REQUIRE((s.mode == ORNITH_QM_Q4K) == (kind == ORNITH_Q4K),
                "%s: config.json says %s but the scales are laid out as %s", path.c_str(),
                s.mode == ORNITH_QM_Q4K ? "q4k" : "q6k", kind == ORNITH_Q4K ? "q4k" : "q6k");
    ORN_REQUIRE(!ornith_weights_has(ws, (path + ".biases").c_str()) &&
                    !ornith_weights_has(ws, (path + ".global_scale").c_str()),
                "%s is a k-quant but the artifact has a .biases or .global_scale for it",
                path.c_str());
  } else {
    ORN_REQUIRE(!says_k, "%s is a k-quant in config.json but the artifact has no %s.dm",
                path.c_str(), path.c_str());
  }
  return ORNITH_OK;
}

static int kq_from(const ornith_weights* ws, const std::string& path, bool routed,
                   ornith_kmatrix* out) {
  ws->fault_rc = 0;
  const Tensor* w = ws->find(path + ".weight");
  const Tensor* s = ws->find(path + ".scales");
  const Tensor* d = ws->find(path + ".dm");
  ORN_RETURN_FAULT(ws);
  if (routed && w && s && !d && ornith_weights_has(ws, (path + ".biases").c_str())) {
    // stacked experts in the 4-bit affine group-32 format (the published artifact's switch_mlp)
    const Tensor* b = ws->find(path + ".biases");
    ORN_REQUIRE_TENSOR(ws, b, "%s.biases: no such tensor", path.c_str());
    int rc = check_mode(ws, path, false, 0);
    if (rc) return rc;
    ORN_REQUIRE(w->dtype == ORNITH_DT_U32 || w->dtype == ORNITH_DT_U8, "%s.weight must be uint32", path.c_str());
    ORN_REQUIRE(s->dtype == ORNITH_DT_BF16 && b->dtype == ORNITH_DT_BF16, "%s: affine scales/biases must be bfloat16",
                path.c_str());
    ORN_REQUIRE(s->shape.size() == 3 && b->shape == s->shape, "%s: scales/biases must be [E, O, K/32]", path.c_str());
    if (ws->quant.loaded) {
      const QuantSpec q = ws->quant.lookup(path);
      ORN_REQUIRE(q.bits == 4 && q.group_size == 32,
                  "%s: affine %d-bit group %d experts are not carried (4-bit group 32 only)", path.c_str(), q.bits,
                  q.group_size);
    }
    out->kind = ORNITH_AFFINE4_G32;
    out->E = (int)s->shape[0];
    out->O = (int)s->shape[1];
    out->K = (int)s->shape[2] * 32;
    out->d_qs = w->d;
    out->d_scales = s->d;
    out->d_dm = b->d;
    return ornith_kmatrix_check(out, w->bytes, s->bytes, b->bytes);
  }
  ORN_REQUIRE_TENSOR(ws, w && s && d, "%s: k-quant module needs .weight, .scales and .dm", path.c_str());
  ORN_REQUIRE(w->dtype == ORNITH_DT_U32 || w->dtype == ORNITH_DT_U8, "%s.weight must be uint32",
              path.c_str());
  ORN_REQUIRE(s->dtype == ORNITH_DT_U8, "%s.scales must be uint8", path.c_str());
  ORN_REQUIRE(d->dtype == ORNITH_DT_F16, "%s.dm must be float16", path.c_str());
  const size_t nd = s->shape.size();
  ORN_REQUIRE(nd == (routed ? 4u : 3u), "%s.scales: expected %d dims, got %zu", path.c_str(),
              routed ? 4 : 3, nd);
  const int64_t per = s->shape[nd - 1], nb = s->shape[nd - 2], O = s->shape[nd - 3];
  const int64_t E = routed ? s->shape[0] : 1;
  ORN_REQUIRE(per == 12 || per == 16, "%s.scales: %lld bytes a block is neither Q4_K nor Q6_K",
              path.c_str(), (long long)per);
  out->kind = per == 12 ? ORNITH_Q4K : ORNITH_Q6K;
  out->E = (int)E;
  out->O = (int)O;
  out->K = (int)(nb * 256);
  out->d_qs = w->d;
  out->d_scales = s->d;
  out->d_dm = d->d;
  int rc = check_mode(ws, path, true, out->kind);
  if (rc) return rc;
  return ornith_kmatrix_check(out, w->bytes, s->bytes, d->bytes);
}

int ws_kmatrix(const ornith_weights* ws, const std::string& path, ornith_kmatrix* out) {
  return kq_from(ws, path, true, out);
}

int ws_linear(const ornith_weights* ws, const std::string& path, ornith_linear* out) {
  memset(out, 0, sizeof *out);
  ws->fault_rc = 0;
  const Tensor* w = ws->find(path + ".weight");
  ORN_REQUIRE_TENSOR(ws, w, "%s.weight: no such tensor", path.c_str());
  if (ornith_weights_has(ws, (path + ".dm").c_str())) {
    out->mode = ORNITH_LIN_KQUANT;
    int rc = kq_from(ws, path, false, &out->km);
    if (rc) return rc;
    out->O = out->km.O;
    out->K = out->km.K;
    return ORNITH_OK;
  }
  int rc = check_mode(ws, path, false, 0);
  if (rc) return rc;
  const Tensor* b = ws->find(path + ".biases");
  ORN_RETURN_FAULT(ws);  // a .biases that exists but could not be copied in is not a dense module
  if (b) {
    const Tensor* s = ws->find(path + ".scales");
    ORN_REQUIRE_TENSOR(ws, s, "%s: affine module needs .scales", path.c_str());
    ORN_REQUIRE(s->dtype == ORNITH_DT_BF16 && b->dtype == ORNITH_DT_BF16,
                "%s: affine scales/biases must be bfloat16", path.c_str());
    ORN_REQUIRE(w->dtype == ORNITH_DT_U32 || w->dtype == ORNITH_DT_U8, "%s.weight must be uint32",
                path.c_str());
    ORN_REQUIRE(s->shape.size() == 2 && b->shape == s->shape, "%s: scales/biases must be [O, K/group]",
                path.c_str());
    // two affine layouts are carried: 8-bit group 64 and 4-bit group 32 (the published
    // artifact's). The quantization block says which; without one the byte count does
    // (64 weight bytes per group against 16).
    const size_t groups = (size_t)s->shape[0] * (size_t)s->shape[1];
    ORN_REQUIRE(groups > 0, "%s: empty scales", path.c_str());
    int bits = w->bytes == groups * 64 ? 8 : w->bytes == groups * 16 ? 4 : 0, group = bits == 8 ? 64 : 32;
    if (ws->quant.loaded) {
      const QuantSpec q = ws->quant.lookup(path);
      ORN_REQUIRE((q.bits == 8 && q.group_size == 64) || (q.bits == 4 && q.group_size == 32),
                  "%s: affine %d-bit group %d is not carried (8-bit group 64 and 4-bit group 32 only)",
                  path.c_str(), q.bits, q.group_size);
      ORN_REQUIRE(bits == q.bits, "%s.weight: %zu bytes is not %d-bit group-%d for its %zu groups", path.c_str(),
                  w->bytes, q.bits, q.group_size, groups);
    }
    ORN_REQUIRE(bits != 0, "%s.weight: %zu bytes is neither 8-bit group-64 nor 4-bit group-32 for [%lld, %lld] groups",
                path.c_str(), w->bytes, (long long)s->shape[0], (long long)s->shape[1]);
    out->mode = bits == 8 ? ORNITH_LIN_AFFINE8 : ORNITH_LIN_AFFINE4;
    out->O = (int)s->shape[0];
    out->K = (int)s->shape[1] * group;
    out->d_w = w->d;
    out->d_scales = s->d;
    out->d_biases = b->d;
    return ORNITH_OK;
  }
  ORN_REQUIRE(w->dtype == ORNITH_DT_BF16 && w->shape.size() == 2,
              "%s.weight: a dense projection must be bfloat16 [O, K]", path.c_str());
  out->mode = ORNITH_LIN_DENSE;
  out->O = (int)w->shape[0];
  out->K = (int)w->shape[1];
  out->d_w = w->d;
  return ORNITH_OK;
}

int ws_tensor(const ornith_weights* ws, const std::string& name, int dtype, int64_t numel,
              const void** out) {
  ws->fault_rc = 0;
  const Tensor* t = ws->find(name);
  ORN_REQUIRE_TENSOR(ws, t, "%s: no such tensor", name.c_str());
  ORN_REQUIRE(t->dtype == dtype, "%s: dtype %d, expected %d", name.c_str(), t->dtype, dtype);
  ORN_REQUIRE(t->numel() == numel, "%s: %lld elements, expected %lld", name.c_str(),
              (long long)t->numel(), (long long)numel);
  *out = t->d;
  return ORNITH_OK;
}

extern "C" {

int ornith_weights_create(ornith_ctx* ctx, ornith_weights** out) {
  ORN_REQUIRE(ctx && out, "weights_create: null argument");
  ornith_weights* w = new ornith_weights();
  w->ctx = ctx;
  *out = w;
  return ORNITH_OK;
}

int ornith_weights_put(ornith_weights* ws, const char* name, int dtype, const int64_t* shape,
                       int ndim, const void* host_data) {
  ORN_REQUIRE(ws && name && shape && host_data, "weights_put: null argument");
  ORN_REQUIRE(ndim >= 1 && ndim <= 8, "weights_put: %s has %d dims", name, ndim);
  const size_t es = ornith_dt_size(dtype);
  ORN_REQUIRE(es, "weights_put: %s has unknown dtype %d", name, dtype);
  ORN_REQUIRE(!ws->find(name), "weights_put: %s is already in the store", name);
  Tensor t;
  t.dtype = dtype;
  int64_t n = 1;
  for (int i = 0; i < ndim; ++i) {
    ORN_REQUIRE(shape[i] >= 1, "weights_put: %s dim %d is %lld", name, i, (long long)shape[i]);
    t.shape.push_back(shape[i]);
    n *= shape[i];
  }
  t.bytes = (size_t)n * es;
  int rc = ornith_alloc(ws->ctx, t.bytes, &t.d);
  if (rc) return rc;
  rc = ornith_upload(ws->ctx, t.d, host_data, t.bytes);
  if (rc) {
    ornith_free(ws->ctx, t.d);
    return rc;
  }
  ws->total_bytes += t.bytes;
  ws->t.emplace(name, std::move(t));
  return ORNITH_OK;
}

int ornith_weights_destroy(ornith_weights* ws) {
  if (!ws) return ORNITH_OK;
  for (auto& kv : ws->t) ornith_free(ws->ctx, kv.second.d);
  ws_release_files(ws);
  delete ws;
  return ORNITH_OK;
}

int ornith_weights_stats(const ornith_weights* ws, int64_t* n_tensors, int64_t* bytes) {
  ORN_REQUIRE(ws, "weights_stats: null store");
  if (n_tensors) *n_tensors = (int64_t)ws->t.size();
  if (bytes) *bytes = (int64_t)ws->total_bytes;
  return ORNITH_OK;
}

}  // extern "C"
