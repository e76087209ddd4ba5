// TextModel, its caches, the MTP head and the FR-Spec head: load, forward, rewind.
//
// Mirrors /root/reference/src/model/qwen3_5.rs:102-279 (load, forward_hidden,
// forward_capture), :301-349 (TrunkCapture::rewind), :374-390 (layer wiring),
// :430-474 (attention), :478-695 (gated delta), /root/reference/src/model/cache.rs,
// /root/reference/src/model/mtp.rs:96-268 and /root/reference/src/frspec.rs:38-158.
//
// Cache design (differs from the reference on purpose): every cache has a fixed
// capacity and is addressed through a few host-side cursors, so taking rows back
// after a rejected draft moves integers, never bytes:
//   KV        rows [0, offset) are live; a forward appends at `offset`.
//   conv      two buffers of K-1+rows rows; a forward reads the live K-1 rows from
//             one and writes the whole concatenated window into the other; the live
//             rows afterwards are [keep, keep+K-1) of that window.
//   state     `max_window` fp32 slots; a captured forward writes the state after
//             token t into slot t; the live slot afterwards is keep-1.
#include "model.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <set>

static const int kMaxRows = 16;  // activation rows a single forward may carry

// frspec_list.cpp: reads and validates an FR-Spec id file
int frspec_read_file(const char* path, std::vector<uint32_t>& ids);

#define TRY(e)         \
  do {                 \
    int rc__ = (e);    \
    if (rc__) return rc__; \
  } while (0)

static std::string lname(const char* prefix, int i, const char* rest) {
  char buf[256];
  snprintf(buf, sizeof buf, "%slayers.%d.%s", prefix, i, rest);
  return buf;
}

static int load_moe(const ornith_weights* ws, const std::string& mlp, const ornith_text_config& c,
                    bool dense_experts, ornith_moe_weights* w) {
  memset(w, 0, sizeof *w);
  TRY(ws_linear(ws, mlp + "gate", &w->router));
  TRY(ws_linear(ws, mlp + "shared_expert.gate_proj", &w->sh_gate));
  TRY(ws_linear(ws, mlp + "shared_expert.up_proj", &w->sh_up));
  TRY(ws_linear(ws, mlp + "shared_expert.down_proj", &w->sh_down));
  TRY(ws_linear(ws, mlp + "shared_expert_gate", &w->sh_egate));
  const int E = c.num_experts, H = c.hidden_size, I = c.moe_intermediate_size;
  if (dense_experts) {
    const int64_t n = (int64_t)E * I * H;
    w->ex_dense = 1;
    if (ornith_weights_has(ws, (mlp + "switch_mlp.gate_proj.weight").c_str())) {
      TRY(ws_tensor(ws, mlp + "switch_mlp.gate_proj.weight", ORNITH_DT_BF16, n, &w->d_ex_gate));
      TRY(ws_tensor(ws, mlp + "switch_mlp.up_proj.weight", ORNITH_DT_BF16, n, &w->d_ex_up));
      TRY(ws_tensor(ws, mlp + "switch_mlp.down_proj.weight", ORNITH_DT_BF16, n, &w->d_ex_down));
    } else {
      // the sidecar file keeps the experts as numbered tensors
      // (/root/reference/src/model/mtp.rs:118-135)
      const std::string ex = mlp + "experts";
      TRY(ws_stacked(ws, ex, "gate_proj.weight", E, ORNITH_DT_BF16, n, &w->d_ex_gate));
      TRY(ws_stacked(ws, ex, "up_proj.weight", E, ORNITH_DT_BF16, n, &w->d_ex_up));
      TRY(ws_stacked(ws, ex, "down_proj.weight", E, ORNITH_DT_BF16, n, &w->d_ex_down));
    }
    w->ex_gate.E = w->ex_up.E = w->ex_down.E = E;
    w->ex_gate.O = w->ex_up.O = I;
    w->ex_gate.K = w->ex_up.K = H;
    w->ex_down.O = H;
    w->ex_down.K = I;
  } else {
    TRY(ws_kmatrix(ws, mlp + "switch_mlp.gate_proj", &w->ex_gate));
    TRY(ws_kmatrix(ws, mlp + "switch_mlp.up_proj", &w->ex_up));
    TRY(ws_kmatrix(ws, mlp + "switch_mlp.down_proj", &w->ex_down));
  }
  w->top_k = c.num_experts_per_tok;
  w->norm_topk_prob = c.norm_topk_prob;
  ORN_REQUIRE(w->router.O == E && w->router.K == H, "%sgate is [%d,%d], config says [%d,%d]",
              mlp.c_str(), w->router.O, w->router.K, E, H);
  ORN_REQUIRE(w->ex_gate.E == E && w->ex_gate.O == I && w->ex_gate.K == H && w->ex_down.O == H &&
                  w->ex_down.K == I,
              "%sswitch_mlp shapes disagree with the config", mlp.c_str());
  ORN_REQUIRE(w->sh_gate.O == c.shared_expert_intermediate_size && w->sh_gate.K == H,
              "%sshared_expert shapes disagree with the config", mlp.c_str());
  return ORNITH_OK;
}

static int load_attn(const ornith_weights* ws, const std::string& p, const ornith_text_config& c,
                     AttnLayer* a) {
  TRY(ws_linear(ws, p + "q_proj", &a->q_proj));
  TRY(ws_linear(ws, p + "k_proj", &a->k_proj));
  TRY(ws_linear(ws, p + "v_proj", &a->v_proj));
  TRY(ws_linear(ws, p + "o_proj", &a->o_proj));
  TRY(ws_tensor(ws, p + "q_norm.weight", ORNITH_DT_BF16, c.head_dim, &a->q_norm));
  TRY(ws_tensor(ws, p + "k_norm.weight", ORNITH_DT_BF16, c.head_dim, &a->k_norm));
  const int H = c.hidden_size, hd = c.head_dim;
  ORN_REQUIRE(a->q_proj.O == c.num_attention_heads * 2 * hd && a->q_proj.K == H &&
                  a->k_proj.O == c.num_key_value_heads * hd && a->v_proj.O == a->k_proj.O &&
                  a->o_proj.O == H && a->o_proj.K == c.num_attention_heads * hd,
              "%s projection shapes disagree with the config", p.c_str());
  return ORNITH_OK;
}

struct StepBufs {
  char *x, *normed, *r, *h, *normed2, *mo;
  char *qkv, *z, *a, *b, *q, *k, *v, *beta, *y, *gated;
  float* g;
  char *qg, *kx, *vx, *q_rot, *att;
};

// Lays the step buffers for R rows out from `base`; *total receives the bytes used, so the
// allocation is sized by the very layout it has to hold.
static StepBufs carve(const ornith_model* m, void* base, int R, size_t* total = nullptr) {
  const auto& c = m->cfg;
  const size_t H = c.hidden_size, D = m->conv_dim(), Vd = m->value_dim(), Kd = m->key_dim();
  const size_t Hv = c.linear_num_value_heads;
  const size_t aq = (size_t)c.num_attention_heads * c.head_dim, akv = (size_t)c.num_key_value_heads * c.head_dim;
  ScratchCursor sc(base);
  StepBufs s;
  s.x = sc.take<char>(2 * H * R);
  s.normed = sc.take<char>(2 * H * R);
  s.r = sc.take<char>(2 * H * R);
  s.h = sc.take<char>(2 * H * R);
  s.normed2 = sc.take<char>(2 * H * R);
  s.mo = sc.take<char>(2 * H * R);
  s.qkv = sc.take<char>(2 * D * R);
  s.z = sc.take<char>(2 * Vd * R);
  s.a = sc.take<char>(2 * Hv * R);
  s.b = sc.take<char>(2 * Hv * R);
  s.q = sc.take<char>(2 * Kd * R);
  s.k = sc.take<char>(2 * Kd * R);
  s.v = sc.take<char>(2 * Vd * R);
  s.beta = sc.take<char>(2 * Hv * R);
  s.y = sc.take<char>(2 * Vd * R);
  s.gated = sc.take<char>(2 * Vd * R);
  s.g = sc.take<float>(Hv * R);
  s.qg = sc.take<char>(2 * 2 * aq * R);
  s.kx = sc.take<char>(2 * akv * R);
  s.vx = sc.take<char>(2 * akv * R);
  s.q_rot = sc.take<char>(2 * aq * R);
  s.att = sc.take<char>(2 * aq * R);
  if (total) *total = sc.off;
  return s;
}

// bytes of step buffers for R rows (trunk)
static size_t step_bytes(const ornith_model* m, int R) {
  size_t n = 0;
  carve(m, nullptr, R, &n);
  return n + 256;
}

int model_ensure_rope(ornith_model* m, int npos) {
  if (npos <= m->rope_npos) return ORNITH_OK;
  ornith_ctx* ctx = m->ctx;
  if (m->d_cos) ornith_free(ctx, m->d_cos);
  if (m->d_sin) ornith_free(ctx, m->d_sin);
  m->d_cos = m->d_sin = nullptr;
  m->rope_npos = 0;
  const size_t bytes = (size_t)npos * (m->cfg.rope_dims / 2) * 4;
  TRY(ornith_alloc(ctx, bytes, (void**)&m->d_cos));
  TRY(ornith_alloc(ctx, bytes, (void**)&m->d_sin));
  TRY(ornith_rope_table(ctx, npos, m->cfg.rope_dims, m->cfg.rope_theta, m->d_cos, m->d_sin));
  m->rope_npos = npos;
  return ORNITH_OK;
}

// q/k/v projections, per-head norm + rope + append, attention + gate; the caller applies
// o_proj to `att`. qg, kx, vx, q_rot, att hold at least T rows.
// With `pend`, d_x is not ready yet: it is rms_norm(pend->res + pend->y) and the q/k/v launch
// makes it (and stores it to d_x, and the sum to pend->h_out).
struct PendingNorm {
  const void *res, *y, *w;
  void* h_out;
};
static int attention_block(ornith_model* m, const AttnLayer& a, void* d_x, int T, void* k_cache,
                           void* v_cache, int offset, int cap, char* qg, char* kx, char* vx,
                           char* q_rot, char* att, const PendingNorm* pend) {
  ornith_ctx* ctx = m->ctx;
  const auto& c = m->cfg;
  {
    const ornith_linear* ws[3] = {&a.q_proj, &a.k_proj, &a.v_proj};
    void* ys[3] = {qg, kx, vx};
    if (pend)
      TRY(ornith_add_rms_linear_multi(ctx, ws, 3, pend->res, pend->y, pend->w, c.rms_norm_eps, T,
                                      pend->h_out, d_x, ys));
    else
      TRY(ornith_linear_matmul_multi(ctx, ws, 3, d_x, T, ys));
  }
  const float scale = 1.0f / sqrtf((float)c.head_dim);
  return ornith_attn_decode(ctx, qg, kx, vx, a.q_norm, a.k_norm, T, c.num_attention_heads,
                            c.num_key_value_heads, c.head_dim, c.rope_dims, c.rms_norm_eps, m->d_cos, m->d_sin,
                            m->rope_npos, offset, cap, scale, q_rot, k_cache, v_cache, att);
}

static int forward_rows(ornith_model* m, ornith_caches* cc, const uint32_t* d_tokens, int T,
                        bool capture, void* d_hidden_out) {
  ornith_ctx* ctx = m->ctx;
  const auto& c = m->cfg;
  const int H = c.hidden_size;
  StepBufs s = carve(m, m->ws_buf, m->max_rows);
  TRY(ornith_embedding(ctx, &m->embed_tokens, d_tokens, T, s.x));
  TRY(ornith_rms_norm(ctx, s.x, m->layers[0].input_ln, T, H, c.rms_norm_eps, s.normed));
  const int Hk = c.linear_num_key_heads, Hv = c.linear_num_value_heads;
  const int Dk = c.linear_key_head_dim, Dv = c.linear_value_head_dim, K = c.linear_conv_kernel_dim;
  const size_t D = m->conv_dim(), ssz = (size_t)Hv * Dv * Dk;
  for (size_t i = 0; i < m->layers.size(); ++i) {
    const Layer& L = m->layers[i];
    LayerCache& lc = cc->layers[i];
    // From the second layer on the layer's input norm is still owed: x = h + mo of the layer
    // before, normed = rms_norm(x, input_ln). The first projections of the mixer make it.
    const PendingNorm pend{s.h, s.mo, L.input_ln, s.x};
    const PendingNorm* pp = i > 0 ? &pend : nullptr;
    if (L.linear) {
      const GdnLayer& g = L.gdn;
      const ornith_linear* big[2] = {&g.in_proj_qkv, &g.in_proj_z};
      void* ybig[2] = {s.qkv, s.z};
      if (pp)
        TRY(ornith_add_rms_linear_multi(ctx, big, 2, pp->res, pp->y, pp->w, c.rms_norm_eps, T, pp->h_out,
                                        s.normed, ybig));
      else
        TRY(ornith_linear_matmul_multi(ctx, big, 2, s.normed, T, ybig));
      const char* conv_state = (const char*)lc.conv[cc->conv_cur] + (size_t)cc->conv_off * D * 2;
      const float* state_in = lc.state + (size_t)cc->state_cur * ssz;
      const bool dense_ab = g.in_proj_a.mode == ORNITH_LIN_DENSE && g.in_proj_b.mode == ORNITH_LIN_DENSE;
      const bool fused = T <= 16 && Dk == 128 && Dv == 128 && ornith_option_fuse_gdn();
      if (!(fused && dense_ab)) {
        const ornith_linear* ab[2] = {&g.in_proj_a, &g.in_proj_b};
        void* yab[2] = {s.a, s.b};
        TRY(ornith_linear_matmul_multi(ctx, ab, 2, s.normed, T, yab));
      }
      if (fused) {
        TRY(ornith_gdn_step(ctx, conv_state, s.qkv, g.conv1d, dense_ab ? nullptr : s.a,
                            dense_ab ? nullptr : s.b, dense_ab ? g.in_proj_a.d_w : nullptr,
                            dense_ab ? g.in_proj_b.d_w : nullptr, dense_ab ? s.normed : nullptr, H, g.a_log,
                            g.dt_bias, T, K, Hk, Dk, Hv, Dv, 1e-6f, state_in, lc.state, capture ? 1 : 0,
                            g.norm, s.z, c.rms_norm_eps, lc.conv[1 - cc->conv_cur], s.gated));
      } else {
        TRY(ornith_gdn_front(ctx, conv_state, s.qkv, g.conv1d, s.a, s.b, g.a_log, g.dt_bias, T, K, Hk,
                             Dk, Hv, Dv, 1e-6f, s.q, s.k, s.v, s.beta, s.g, lc.conv[1 - cc->conv_cur]));
        TRY(ornith_gdn_recurrence(ctx, s.q, s.k, s.v, s.g, s.beta, state_in, T, Hk, Hv, Dk, Dv, s.y,
                                  lc.state, capture ? 1 : 0));
        TRY(ornith_rms_norm_gated(ctx, s.y, g.norm, s.z, T * Hv, Dv, c.rms_norm_eps, s.gated));
      }
      TRY(ornith_linear_matmul(ctx, &g.out_proj, s.gated, T, s.r));
    } else {
      TRY(attention_block(m, L.attn, s.normed, T, lc.k, lc.v, cc->offset, cc->capacity, s.qg, s.kx,
                          s.vx, s.q_rot, s.att, pp));
      TRY(ornith_linear_matmul(ctx, &L.attn.o_proj, s.att, T, s.r));
    }
    TRY(ornith_add_rms_moe_block(ctx, &L.moe, s.x, s.r, L.post_ln, c.rms_norm_eps, T, s.h, s.normed2, s.mo));
  }
  // the last layer's closing add and the model's final norm
  TRY(ornith_add_rms_norm(ctx, s.h, s.mo, m->final_norm, T, H, c.rms_norm_eps, s.x, d_hidden_out));
  // every layer advanced together
  cc->conv_cur = 1 - cc->conv_cur;
  cc->conv_off = T;
  cc->state_cur = capture ? T - 1 : 0;
  cc->offset += T;
  cc->last_T = T;
  cc->last_capture = capture;
  return ORNITH_OK;
}

extern "C" {

int ornith_model_load(ornith_ctx* ctx, const ornith_weights* ws, const ornith_text_config* cfg,
                      ornith_model** out) {
  ORN_REQUIRE(ctx && ws && cfg && out, "model_load: null argument");
  const ornith_text_config& c = *cfg;
  ORN_REQUIRE(c.num_hidden_layers >= 1 && c.full_attention_interval >= 1, "model_load: bad layer config");
  ORN_REQUIRE(c.linear_key_head_dim == 128 && c.linear_value_head_dim == 128,
              "model_load: gated-delta head dims %d/%d (128 only)", c.linear_key_head_dim,
              c.linear_value_head_dim);
  ORN_REQUIRE(c.hidden_size % 64 == 0 && c.num_experts % 64 == 0, "model_load: hidden=%d experts=%d",
              c.hidden_size, c.num_experts);
  ornith_model* m = new ornith_model();
  m->ctx = ctx;
  m->cfg = c;
  const char* P = "language_model.model.";
  int rc = ORNITH_OK;
  auto fail = [&](int code) {
    ornith_model_destroy(m);
    return code;
  };
#define LTRY(e)                    \
  do {                             \
    rc = (e);                      \
    if (rc) return fail(rc);       \
  } while (0)
  LTRY(ws_linear(ws, std::string(P) + "embed_tokens", &m->embed_tokens));
  if (!((m->embed_tokens.mode == ORNITH_LIN_AFFINE8 || m->embed_tokens.mode == ORNITH_LIN_AFFINE4) &&
        m->embed_tokens.O == c.vocab_size && m->embed_tokens.K == c.hidden_size))
    return fail(ornith_fail(ORNITH_ERR_INVALID, "model_load: embed_tokens must be an affine [vocab, hidden] table"));
  LTRY(ws_linear(ws, "language_model.lm_head", &m->lm_head));
  if (!(m->lm_head.O == c.vocab_size && m->lm_head.K == c.hidden_size))
    return fail(ornith_fail(ORNITH_ERR_INVALID, "model_load: lm_head is [%d,%d]", m->lm_head.O, m->lm_head.K));
  LTRY(ws_tensor(ws, std::string(P) + "norm.weight", ORNITH_DT_BF16, c.hidden_size, &m->final_norm));
  const int Hv = c.linear_num_value_heads, H = c.hidden_size;
  m->layers.resize(c.num_hidden_layers);
  for (int i = 0; i < c.num_hidden_layers; ++i) {
    Layer& L = m->layers[i];
    L.linear = ((i + 1) % c.full_attention_interval) != 0;
    LTRY(ws_tensor(ws, lname(P, i, "input_layernorm.weight"), ORNITH_DT_BF16, H, &L.input_ln));
    LTRY(ws_tensor(ws, lname(P, i, "post_attention_layernorm.weight"), ORNITH_DT_BF16, H, &L.post_ln));
    if (L.linear) {
      GdnLayer& g = L.gdn;
      const std::string p = lname(P, i, "linear_attn.");
      LTRY(ws_linear(ws, p + "in_proj_qkv", &g.in_proj_qkv));
      LTRY(ws_linear(ws, p + "in_proj_z", &g.in_proj_z));
      LTRY(ws_linear(ws, p + "out_proj", &g.out_proj));
      LTRY(ws_linear(ws, p + "in_proj_a", &g.in_proj_a));
      LTRY(ws_linear(ws, p + "in_proj_b", &g.in_proj_b));
      LTRY(ws_tensor(ws, p + "conv1d.weight", ORNITH_DT_BF16, (int64_t)m->conv_dim() * c.linear_conv_kernel_dim, &g.conv1d));
      LTRY(ws_tensor(ws, p + "dt_bias", ORNITH_DT_BF16, Hv, &g.dt_bias));
      LTRY(ws_tensor(ws, p + "A_log", ORNITH_DT_BF16, Hv, &g.a_log));
      LTRY(ws_tensor(ws, p + "norm.weight", ORNITH_DT_BF16, c.linear_value_head_dim, &g.norm));
      if (!(g.in_proj_qkv.O == m->conv_dim() && g.in_proj_qkv.K == H && g.in_proj_z.O == m->value_dim() &&
            g.out_proj.O == H && g.out_proj.K == m->value_dim() && g.in_proj_a.O == Hv && g.in_proj_b.O == Hv)) {
        ornith_fail(ORNITH_ERR_INVALID, "%s projection shapes disagree with the config", p.c_str());
        return fail(ORNITH_ERR_INVALID);
      }
    } else {
      LTRY(load_attn(ws, lname(P, i, "self_attn."), c, &L.attn));
    }
    LTRY(load_moe(ws, lname(P, i, "mlp."), c, false, &L.moe));
  }
  m->max_rows = kMaxRows;
  m->ws_bytes = step_bytes(m, m->max_rows);
  LTRY(ornith_alloc(ctx, m->ws_bytes, &m->ws_buf));
#undef LTRY
  *out = m;
  return ORNITH_OK;
}

int ornith_model_moe_weights(const ornith_model* m, int layer, ornith_moe_weights* out) {
  ORN_REQUIRE(m && out, "model_moe_weights: null argument");
  ORN_REQUIRE(layer >= 0 && layer < (int)m->layers.size(), "model_moe_weights: layer %d of %zu", layer,
              m->layers.size());
  *out = m->layers[layer].moe;
  return ORNITH_OK;
}

int ornith_model_set_max_rows(ornith_model* m, int rows) {
  ORN_REQUIRE(m, "model_set_max_rows: null model");
  ORN_REQUIRE(rows >= kMaxRows && rows <= 8192, "model_set_max_rows: rows=%d (%d..8192)", rows, kMaxRows);
  if (rows == m->max_rows) return ORNITH_OK;
  TRY(ornith_sync(m->ctx));
  void* buf = nullptr;
  const size_t bytes = step_bytes(m, rows);
  TRY(ornith_alloc(m->ctx, bytes, &buf));
  ornith_free(m->ctx, m->ws_buf);
  m->ws_buf = buf;
  m->ws_bytes = bytes;
  m->max_rows = rows;
  return ORNITH_OK;
}

int ornith_model_destroy(ornith_model* m) {
  if (!m) return ORNITH_OK;
  ornith_free(m->ctx, m->ws_buf);
  ornith_free(m->ctx, m->d_cos);
  ornith_free(m->ctx, m->d_sin);
  delete m;
  return ORNITH_OK;
}

// KvCache::update_and_fetch's growth (/root/reference/src/model/cache.rs:38-79): a KV pair
// [Hkv, cap, hd] that must hold `need` rows moves to tensors of a larger capacity, a multiple of
// 256 rows as the reference's steps are and at least half as large again as before (so a long
// generation copies its cache a logarithmic number of times, not once per 256 tokens). Rows
// [0, offset) of every head are carried over; what lies past them was never committed.
static int kv_new_capacity(int capacity, int need) {
  const long grown = (long)capacity + capacity / 2;
  const long want = need > grown ? need : grown;
  return (int)((want + 255) / 256 * 256);
}

static int kv_move(ornith_model* m, void** buf, int old_cap, int new_cap, int offset) {
  const auto& c = m->cfg;
  const size_t row = (size_t)c.head_dim * 2;
  void* nb = nullptr;
  TRY(ornith_alloc(m->ctx, (size_t)c.num_key_value_heads * new_cap * row, &nb));
  if (offset > 0) {
    hipError_t e = hipMemcpy2DAsync(nb, (size_t)new_cap * row, *buf, (size_t)old_cap * row, (size_t)offset * row,
                                    c.num_key_value_heads, hipMemcpyDeviceToDevice, m->ctx->stream);
    if (e != hipSuccess) {
      ornith_free(m->ctx, nb);
      return ornith_fail(ORNITH_ERR_HIP, "growing a KV cache: %s", hipGetErrorString(e));
    }
  }
  const int rc = ornith_sync(m->ctx);  // the old tensor is freed next: everything that reads it has run
  if (rc) {
    ornith_free(m->ctx, nb);
    return rc;
  }
  ornith_free(m->ctx, *buf);
  *buf = nb;
  return ORNITH_OK;
}

int ornith_caches_reserve(ornith_caches* cc, int rows) {
  ORN_REQUIRE(cc && rows >= 0, "caches_reserve: bad argument");
  if (rows <= cc->capacity) return ORNITH_OK;
  ornith_model* m = cc->m;
  const int ncap = kv_new_capacity(cc->capacity, rows);
  TRY(model_ensure_rope(m, ncap));
  for (size_t i = 0; i < cc->layers.size(); ++i) {
    if (m->layers[i].linear) continue;
    TRY(kv_move(m, &cc->layers[i].k, cc->capacity, ncap, cc->offset));
    TRY(kv_move(m, &cc->layers[i].v, cc->capacity, ncap, cc->offset));
  }
  cc->capacity = ncap;
  return ORNITH_OK;
}

int ornith_caches_set_growable(ornith_caches* cc, int growable) {
  ORN_REQUIRE(cc, "caches_set_growable: null caches");
  cc->growable = growable != 0;
  return ORNITH_OK;
}

int ornith_caches_capacity(const ornith_caches* cc, int* capacity_out) {
  ORN_REQUIRE(cc && capacity_out, "caches_capacity: null argument");
  *capacity_out = cc->capacity;
  return ORNITH_OK;
}

int ornith_caches_create(ornith_model* m, int capacity, int max_window, ornith_caches** out) {
  ORN_REQUIRE(m && out, "caches_create: null argument");
  ORN_REQUIRE(capacity >= 1 && max_window >= 1 && max_window <= kMaxRows,
              "caches_create: capacity=%d max_window=%d (window at most %d)", capacity, max_window,
              kMaxRows);
  const auto& c = m->cfg;
  ornith_caches* cc = new ornith_caches();
  cc->m = m;
  cc->capacity = capacity;
  cc->max_window = max_window;
  cc->conv_rows = c.linear_conv_kernel_dim - 1 + m->max_rows;
  cc->layers.resize(m->layers.size());
  const size_t kv = (size_t)c.num_key_value_heads * capacity * c.head_dim * 2;
  const size_t conv = (size_t)cc->conv_rows * m->conv_dim() * 2;
  const size_t st = (size_t)max_window * c.linear_num_value_heads * c.linear_value_head_dim *
                    c.linear_key_head_dim * 4;
  int rc = model_ensure_rope(m, capacity);
  for (size_t i = 0; i < m->layers.size() && !rc; ++i) {
    LayerCache& lc = cc->layers[i];
    if (m->layers[i].linear) {
      rc = ornith_alloc(m->ctx, conv, &lc.conv[0]);
      if (!rc) rc = ornith_alloc(m->ctx, conv, &lc.conv[1]);
      if (!rc) rc = ornith_alloc(m->ctx, st, (void**)&lc.state);
    } else {
      rc = ornith_alloc(m->ctx, kv, &lc.k);
      if (!rc) rc = ornith_alloc(m->ctx, kv, &lc.v);
    }
  }
  if (!rc) rc = ornith_caches_reset(cc);
  if (rc) {
    ornith_caches_destroy(cc);
    return rc;
  }
  *out = cc;
  return ORNITH_OK;
}

int ornith_caches_reset(ornith_caches* cc) {
  ORN_REQUIRE(cc, "caches_reset: null caches");
  ornith_model* m = cc->m;
  const auto& c = m->cfg;
  const size_t conv = (size_t)cc->conv_rows * m->conv_dim() * 2;
  const size_t st = (size_t)c.linear_num_value_heads * c.linear_value_head_dim * c.linear_key_head_dim * 4;
  for (size_t i = 0; i < cc->layers.size(); ++i) {
    LayerCache& lc = cc->layers[i];
    if (m->layers[i].linear) {
      // conv_or_zeros / state_or_zeros (src/model/cache.rs:90-133)
      TRY(ornith_memset(m->ctx, lc.conv[0], 0, conv));
      TRY(ornith_memset(m->ctx, lc.state, 0, st));
    }
  }
  cc->offset = cc->conv_cur = cc->conv_off = cc->state_cur = cc->last_T = 0;
  cc->last_capture = false;
  return ORNITH_OK;
}

int ornith_caches_destroy(ornith_caches* cc) {
  if (!cc) return ORNITH_OK;
  for (auto& lc : cc->layers) {
    ornith_free(cc->m->ctx, lc.k);
    ornith_free(cc->m->ctx, lc.v);
    ornith_free(cc->m->ctx, lc.conv[0]);
    ornith_free(cc->m->ctx, lc.conv[1]);
    ornith_free(cc->m->ctx, lc.state);
  }
  delete cc;
  return ORNITH_OK;
}

int ornith_caches_offset(const ornith_caches* cc, int* offset_out) {
  ORN_REQUIRE(cc && offset_out, "caches_offset: null argument");
  *offset_out = cc->offset;
  return ORNITH_OK;
}

int ornith_model_forward(ornith_model* m, ornith_caches* cc, const uint32_t* d_tokens, int T,
                         int capture, void* d_hidden_out) {
  ORN_REQUIRE(m && cc && d_tokens && d_hidden_out, "model_forward: null argument");
  ORN_REQUIRE(cc->m == m, "model_forward: caches belong to another model");
  ORN_REQUIRE(T >= 1 && T <= m->max_rows, "model_forward: T=%d (1..%d rows a call)", T, m->max_rows);
  ORN_REQUIRE(m->cfg.linear_conv_kernel_dim - 1 + T <= cc->conv_rows,
              "model_forward: %d rows, but these caches were created for %d rows a call", T,
              cc->conv_rows - (m->cfg.linear_conv_kernel_dim - 1));
  ORN_REQUIRE(!capture || T <= cc->max_window, "model_forward: capture of %d rows, window is %d", T,
              cc->max_window);
  ORN_REQUIRE(cc->growable || cc->offset + T <= cc->capacity, "model_forward: %d + %d rows exceed cache capacity %d",
              cc->offset, T, cc->capacity);
  TRY(ornith_caches_reserve(cc, cc->offset + T));
  return forward_rows(m, cc, d_tokens, T, capture != 0, d_hidden_out);
}

int ornith_model_rewind(ornith_model* m, ornith_caches* cc, int keep) {
  ORN_REQUIRE(m && cc && cc->m == m, "model_rewind: bad argument");
  ORN_REQUIRE(cc->last_capture, "model_rewind: the last forward did not capture");
  ORN_REQUIRE(keep >= 1 && keep <= cc->last_T, "model_rewind: keep=%d of %d rows", keep, cc->last_T);
  cc->offset -= cc->last_T - keep;
  cc->conv_off = keep;
  cc->state_cur = keep - 1;
  cc->last_T = keep;
  return ORNITH_OK;
}

int ornith_model_logits(ornith_model* m, const void* d_hidden, int T, void* d_logits) {
  ORN_REQUIRE(m && d_hidden && d_logits, "model_logits: null argument");
  return ornith_linear_matmul(m->ctx, &m->lm_head, d_hidden, T, d_logits);
}

// ---- FR-Spec ---------------------------------------------------------------------

static int gather_rows_dev(ornith_ctx* ctx, const void* src, size_t row_bytes, const std::vector<uint32_t>& ids,
                           void** out) {
  // FrSpec::prune is a load-time row gather (src/frspec.rs:67-93): one launch per tensor
  void* d_ids = nullptr;
  TRY(ornith_alloc(ctx, ids.size() * 4, &d_ids));
  int rc = ornith_upload(ctx, d_ids, ids.data(), ids.size() * 4);
  if (!rc) rc = ornith_alloc(ctx, row_bytes * ids.size(), out);
  if (!rc) rc = ornith_gather_rows(ctx, src, row_bytes, (const uint32_t*)d_ids, (int)ids.size(), *out);
  if (!rc) rc = ornith_sync(ctx);
  ornith_free(ctx, d_ids);
  return rc;
}

int ornith_frspec_from_ids(ornith_model* m, const uint32_t* ids, int n, ornith_frspec** out) {
  ORN_REQUIRE(m && ids && out, "frspec: null argument");
  const int vocab = m->cfg.vocab_size;
  ORN_REQUIRE(n > 0, "FR-Spec list is empty");
  ORN_REQUIRE(n < vocab, "FR-Spec list has %d ids, the vocabulary has %d: nothing to prune", n, vocab);
  std::set<uint32_t> seen;
  for (int i = 0; i < n; ++i) {
    ORN_REQUIRE(ids[i] < (uint32_t)vocab, "FR-Spec id %u at %d is outside the vocabulary (%d)", ids[i], i, vocab);
    ORN_REQUIRE(seen.insert(ids[i]).second, "FR-Spec id %u is listed twice", ids[i]);
  }
  ornith_frspec* f = new ornith_frspec();
  f->m = m;
  f->n = n;
  f->vocab = vocab;
  f->ids.assign(ids, ids + n);
  const ornith_linear& lm = m->lm_head;
  f->head = lm;
  f->head.O = n;
  int rc = ornith_alloc(m->ctx, (size_t)n * 4, (void**)&f->d_ids);
  if (!rc) rc = ornith_upload(m->ctx, f->d_ids, ids, (size_t)n * 4);
  if (!rc) {
    if (lm.mode == ORNITH_LIN_KQUANT) {
      const size_t nb = lm.K / 256;
      const size_t cb = lm.km.kind == ORNITH_Q4K ? 128 : 192, sb = lm.km.kind == ORNITH_Q4K ? 12 : 16,
                   db = lm.km.kind == ORNITH_Q4K ? 4 : 2;
      rc = gather_rows_dev(m->ctx, lm.km.d_qs, nb * cb, f->ids, &f->owned[0]);
      if (!rc) rc = gather_rows_dev(m->ctx, lm.km.d_scales, nb * sb, f->ids, &f->owned[1]);
      if (!rc) rc = gather_rows_dev(m->ctx, lm.km.d_dm, nb * db, f->ids, &f->owned[2]);
      f->head.km.O = n;
      f->head.km.d_qs = f->owned[0];
      f->head.km.d_scales = f->owned[1];
      f->head.km.d_dm = f->owned[2];
    } else if (lm.mode == ORNITH_LIN_AFFINE8) {
      rc = gather_rows_dev(m->ctx, lm.d_w, (size_t)lm.K, f->ids, &f->owned[0]);
      if (!rc) rc = gather_rows_dev(m->ctx, lm.d_scales, (size_t)lm.K / 64 * 2, f->ids, &f->owned[1]);
      if (!rc) rc = gather_rows_dev(m->ctx, lm.d_biases, (size_t)lm.K / 64 * 2, f->ids, &f->owned[2]);
      f->head.d_w = f->owned[0];
      f->head.d_scales = f->owned[1];
      f->head.d_biases = f->owned[2];
    } else if (lm.mode == ORNITH_LIN_AFFINE4) {
      rc = gather_rows_dev(m->ctx, lm.d_w, (size_t)lm.K / 2, f->ids, &f->owned[0]);
      if (!rc) rc = gather_rows_dev(m->ctx, lm.d_scales, (size_t)lm.K / 32 * 2, f->ids, &f->owned[1]);
      if (!rc) rc = gather_rows_dev(m->ctx, lm.d_biases, (size_t)lm.K / 32 * 2, f->ids, &f->owned[2]);
      f->head.d_w = f->owned[0];
      f->head.d_scales = f->owned[1];
      f->head.d_biases = f->owned[2];
    } else {
      rc = gather_rows_dev(m->ctx, lm.d_w, (size_t)lm.K * 2, f->ids, &f->owned[0]);
      f->head.d_w = f->owned[0];
    }
  }
  if (rc) {
    ornith_frspec_destroy(f);
    return rc;
  }
  *out = f;
  return ORNITH_OK;
}

int ornith_frspec_load(ornith_model* m, const char* path, ornith_frspec** out) {
  ORN_REQUIRE(m && out, "frspec_load: null argument");
  char dflt[4096];
  if (!path) {
    TRY(ornith_frspec_default_path(dflt, sizeof dflt));
    path = dflt;
  }
  std::vector<uint32_t> ids;
  TRY(frspec_read_file(path, ids));
  ORN_REQUIRE(!ids.empty(), "%s: FR-Spec list is empty", path);
  return ornith_frspec_from_ids(m, ids.data(), (int)ids.size(), out);
}

int ornith_frspec_destroy(ornith_frspec* f) {
  if (!f) return ORNITH_OK;
  for (void* p : f->owned) ornith_free(f->m->ctx, p);
  ornith_free(f->m->ctx, f->d_ids);
  delete f;
  return ORNITH_OK;
}

int ornith_frspec_head(const ornith_frspec* f, ornith_linear* head_out, int* n_out) {
  ORN_REQUIRE(f && head_out, "frspec_head: null argument");
  *head_out = f->head;
  if (n_out) *n_out = f->n;
  return ORNITH_OK;
}

// ---- MTP head ---------------------------------------------------------------------

int ornith_mtp_load(ornith_model* m, const ornith_weights* ws, int capacity, ornith_mtp_head** out) {
  ORN_REQUIRE(m && ws && out && capacity >= 1, "mtp_load: bad argument");
  const auto& c = m->cfg;
  const int H = c.hidden_size;
  ornith_mtp_head* h = new ornith_mtp_head();
  h->m = m;
  int rc = ORNITH_OK;
#define MTRY(e)                 \
  do {                          \
    rc = (e);                   \
    if (rc) {                   \
      ornith_mtp_destroy(h);    \
      return rc;                \
    }                           \
  } while (0)
  MTRY(ws_tensor(ws, "mtp.pre_fc_norm_embedding.weight", ORNITH_DT_BF16, H, &h->pre_fc_norm_embedding));
  MTRY(ws_tensor(ws, "mtp.pre_fc_norm_hidden.weight", ORNITH_DT_BF16, H, &h->pre_fc_norm_hidden));
  MTRY(ws_linear(ws, "mtp.fc", &h->fc));
  if (!(h->fc.O == H && h->fc.K == 2 * H)) {
    ornith_mtp_destroy(h);
    return ornith_fail(ORNITH_ERR_INVALID, "mtp.fc is [%d,%d], expected [%d,%d]", h->fc.O, h->fc.K, H, 2 * H);
  }
  MTRY(ws_tensor(ws, "mtp.layers.0.input_layernorm.weight", ORNITH_DT_BF16, H, &h->input_ln));
  MTRY(ws_tensor(ws, "mtp.layers.0.post_attention_layernorm.weight", ORNITH_DT_BF16, H, &h->post_ln));
  MTRY(ws_tensor(ws, "mtp.norm.weight", ORNITH_DT_BF16, H, &h->norm));
  MTRY(load_attn(ws, "mtp.layers.0.self_attn.", c, &h->attn));
  MTRY(load_moe(ws, "mtp.layers.0.mlp.", c, !ornith_weights_has(ws, "mtp.layers.0.mlp.switch_mlp.gate_proj.dm"), &h->moe));
  h->capacity = capacity;
  h->max_rows = m->max_rows;
  const size_t kv = (size_t)c.num_key_value_heads * capacity * c.head_dim * 2;
  MTRY(ornith_alloc(m->ctx, kv, &h->k));
  MTRY(ornith_alloc(m->ctx, kv, &h->v));
  const size_t aq = (size_t)c.num_attention_heads * c.head_dim, akv = (size_t)c.num_key_value_heads * c.head_dim;
  const size_t per_row = 2 * ((size_t)9 * H + 4 * aq + 2 * akv) + 4096;
  MTRY(ornith_alloc(m->ctx, per_row * h->max_rows + 64 * 256, &h->buf));
  MTRY(model_ensure_rope(m, capacity));
#undef MTRY
  *out = h;
  return ORNITH_OK;
}

int ornith_mtp_destroy(ornith_mtp_head* h) {
  if (!h) return ORNITH_OK;
  ornith_free(h->m->ctx, h->k);
  ornith_free(h->m->ctx, h->v);
  ornith_free(h->m->ctx, h->buf);
  ornith_free(h->m->ctx, h->d_forced);
  delete h;
  return ORNITH_OK;
}

int ornith_mtp_force_drafts(ornith_mtp_head* h, const uint32_t* tokens, size_t n) {
  ORN_REQUIRE(h && (tokens || n == 0), "mtp_force_drafts: null argument");
  ornith_ctx* ctx = h->m->ctx;
  // a generation that still reads the old list has been queued at most; let it finish
  TRY(ornith_sync(ctx));
  ornith_free(ctx, h->d_forced);
  h->d_forced = nullptr;
  h->n_forced = 0;
  if (n == 0) return ORNITH_OK;
  void* d = nullptr;
  TRY(ornith_alloc(ctx, n * 4, &d));
  const int rc = ornith_upload(ctx, d, tokens, n * 4);
  if (rc) {
    ornith_free(ctx, d);
    return rc;
  }
  h->d_forced = (uint32_t*)d;
  h->n_forced = n;
  return ORNITH_OK;
}

int ornith_mtp_cache_reserve(ornith_mtp_head* h, int rows) {
  ORN_REQUIRE(h && rows >= 0, "mtp_cache_reserve: bad argument");
  if (rows <= h->capacity) return ORNITH_OK;
  const int ncap = kv_new_capacity(h->capacity, rows);
  TRY(model_ensure_rope(h->m, ncap));
  TRY(kv_move(h->m, &h->k, h->capacity, ncap, h->offset));
  TRY(kv_move(h->m, &h->v, h->capacity, ncap, h->offset));
  h->capacity = ncap;
  return ORNITH_OK;
}

int ornith_mtp_cache_set_growable(ornith_mtp_head* h, int growable) {
  ORN_REQUIRE(h, "mtp_cache_set_growable: null head");
  h->growable = growable != 0;
  return ORNITH_OK;
}

int ornith_mtp_cache_set_offset(ornith_mtp_head* h, int offset) {
  ORN_REQUIRE(h && offset >= 0 && offset <= h->capacity, "mtp_cache_set_offset: offset=%d", offset);
  h->offset = offset;
  return ORNITH_OK;
}

int ornith_mtp_cache_offset(const ornith_mtp_head* h, int* offset_out) {
  ORN_REQUIRE(h && offset_out, "mtp_cache_offset: null argument");
  *offset_out = h->offset;
  return ORNITH_OK;
}

int ornith_mtp_forward(ornith_mtp_head* h, const ornith_frspec* frspec, const void* d_trunk_hidden,
                       const uint32_t* d_next_ids, int T, void* d_hidden_out, void* d_logits) {
  ORN_REQUIRE(h && d_trunk_hidden && d_next_ids && d_hidden_out, "mtp_forward: null argument");
  ORN_REQUIRE(T >= 1 && T <= h->max_rows, "mtp_forward: T=%d", T);
  ORN_REQUIRE(h->growable || h->offset + T <= h->capacity, "mtp_forward: %d + %d rows exceed the head's cache (%d)",
              h->offset, T, h->capacity);
  TRY(ornith_mtp_cache_reserve(h, h->offset + T));
  ornith_model* m = h->m;
  ornith_ctx* ctx = m->ctx;
  const auto& c = m->cfg;
  const size_t H = c.hidden_size, R = h->max_rows;
  const size_t aq = (size_t)c.num_attention_heads * c.head_dim, akv = (size_t)c.num_key_value_heads * c.head_dim;
  ScratchCursor sc(h->buf);
  char* emb = sc.take<char>(2 * H * R);
  char* joined = sc.take<char>(2 * 2 * H * R);  // [T, 2H]: e | h
  char* x = sc.take<char>(2 * H * R);
  char* normed = sc.take<char>(2 * H * R);
  char* r = sc.take<char>(2 * H * R);
  char* hh = sc.take<char>(2 * H * R);
  char* normed2 = sc.take<char>(2 * H * R);
  char* mo = sc.take<char>(2 * H * R);
  char* qg = sc.take<char>(2 * 2 * aq * R);
  char* kx = sc.take<char>(2 * akv * R);
  char* vx = sc.take<char>(2 * akv * R);
  char* q_rot = sc.take<char>(2 * aq * R);
  char* att = sc.take<char>(2 * aq * R);

  TRY(ornith_embedding(ctx, &m->embed_tokens, d_next_ids, T, emb));
  // e = norm(embed), h = norm(trunk hidden); concat order "embedding_hidden": the two
  // norms write the halves of each joined row directly
  for (int t = 0; t < T; ++t) {
    TRY(ornith_rms_norm(ctx, emb + (size_t)t * H * 2, h->pre_fc_norm_embedding, 1, (int)H, c.rms_norm_eps,
                        joined + (size_t)t * 4 * H));
    TRY(ornith_rms_norm(ctx, (const char*)d_trunk_hidden + (size_t)t * H * 2, h->pre_fc_norm_hidden, 1, (int)H,
                        c.rms_norm_eps, joined + (size_t)t * 4 * H + 2 * H));
  }
  TRY(ornith_linear_matmul(ctx, &h->fc, joined, T, x));
  TRY(ornith_rms_norm(ctx, x, h->input_ln, T, (int)H, c.rms_norm_eps, normed));
  TRY(attention_block(m, h->attn, normed, T, h->k, h->v, h->offset, h->capacity, qg, kx, vx, q_rot, att,
                      nullptr));
  TRY(ornith_linear_matmul(ctx, &h->attn.o_proj, att, T, r));
  TRY(ornith_add_rms_norm(ctx, x, r, h->post_ln, T, (int)H, c.rms_norm_eps, hh, normed2));
  // add(h, m) then mtp.norm; the un-normed sum is not needed afterwards
  TRY(ornith_moe_block(ctx, &h->moe, normed2, T, mo, nullptr, nullptr));
  TRY(ornith_add_rms_norm(ctx, hh, mo, h->norm, T, (int)H, c.rms_norm_eps, x, d_hidden_out));
  h->offset += T;
  if (d_logits) {
    const ornith_linear* lm = frspec ? &frspec->head : &m->lm_head;
    TRY(ornith_linear_matmul(ctx, lm, d_hidden_out, T, d_logits));
  }
  return ORNITH_OK;
}

}  // extern "C"
