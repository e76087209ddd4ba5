/*
 * CPU oracle -- TEST INFRASTRUCTURE (see orc_common.h). The trunk, the MTP head,
 * the caches with capture/rewind and the two generation loops, composed from the
 * operator restatements in the other orc_*.c files.
 *
 * Restates /root/reference/src/model/qwen3_5.rs:190-279 (forward_hidden /
 * forward_capture), :301-349 (rewind), :374-390 (layer wiring), :430-474, :478-695;
 * /root/reference/src/model/mtp.rs:150-262; /root/reference/src/generate.rs:86-206;
 * /root/reference/src/mtp_generate.rs:99-317; /root/reference/src/frspec.rs:67-142.
 * Caches here are plain copies (snapshots are memcpy'd back on rewind), which is
 * the reference's own formulation and deliberately not the device library's
 * cursor scheme.
 */
#include "orc_common.h"
#include "orc_types.h"



void orc_linear_fwd(const orc_linear* L, const bf16_t* x, int M, bf16_t* y);
float orc_dense_row_dot(const bf16_t* w, int K, const float* x);
void orc_moe_block(const orc_moe_weights* W, const bf16_t* x, int T, bf16_t* out, uint32_t* inds_out,
                   bf16_t* scores_out, bf16_t* probs_out);
void orc_softmax_bf16(const bf16_t* x, int rows, int n, bf16_t* out);
void orc_router_topk(const bf16_t* p, int rows, int n, int k, uint32_t* inds, bf16_t* scores);
void orc_swiglu_bf16(const bf16_t* gate, const bf16_t* up, int64_t n, bf16_t* out);
void orc_moe_combine(const bf16_t* scores, const bf16_t* y, const bf16_t* gate, const bf16_t* shared,
                     int tokens, int k, int dim, int normalize, bf16_t* out);
void orc_dense_gather_mv(const bf16_t* w, int O, int K, const bf16_t* x, const uint32_t* lhs,
                         const uint32_t* rhs, int rows, bf16_t* y);
void orc_embedding(const uint8_t* w, const bf16_t* scales, const bf16_t* biases, int K,
                   const uint32_t* ids, int n, bf16_t* out);
void orc_embedding4(const uint8_t* w, const bf16_t* scales, const bf16_t* biases, int K,
                    const uint32_t* ids, int n, bf16_t* out);
/* the token embedding through whichever affine format the table is in */
static void embed_rows(const orc_linear* t, int K, const uint32_t* ids, int n, bf16_t* out) {
  if (t->mode == 3) orc_embedding4(t->aw, t->as, t->ab, K, ids, n, out);
  else orc_embedding(t->aw, t->as, t->ab, K, ids, n, out);
}
void orc_rms_norm(const bf16_t* x, const bf16_t* w, int rows, int n, float eps, bf16_t* out);
void orc_add_rms_norm(const bf16_t* a, const bf16_t* b, const bf16_t* w, int rows, int n, float eps,
                      bf16_t* h_out, bf16_t* out);
void orc_rms_norm_gated(const bf16_t* y, const bf16_t* w, const bf16_t* z, int rows, int n, float eps,
                        bf16_t* out);
void orc_gdn_front(const bf16_t* conv_state, const bf16_t* qkv, const bf16_t* cw, const bf16_t* a_in,
                   const bf16_t* b_in, const bf16_t* a_log, const bf16_t* dt_bias, int T, int K, int Hk,
                   int Dk, int Hv, int Dv, float eps, bf16_t* q, bf16_t* k, bf16_t* v, bf16_t* beta,
                   float* g, bf16_t* conv_input);
void orc_gdn_recurrence(const bf16_t* q, const bf16_t* k, const bf16_t* v, const float* g,
                        const bf16_t* beta, const float* state_in, int T, int Hk, int Hv, int Dk, int Dv,
                        bf16_t* y, float* snapshots);
void orc_rope_table(int npos, int dims, double theta, float* cos_t, float* sin_t);
void orc_attn_prep(const bf16_t* qg, const bf16_t* kx, const bf16_t* vx, const bf16_t* q_norm_w,
                   const bf16_t* k_norm_w, int T, int Hq, int Hkv, int hd, int rope_dims, float eps,
                   const float* cos_t, const float* sin_t, int offset, int cap, bf16_t* q_rot,
                   bf16_t* gate, bf16_t* k_cache, bf16_t* v_cache);
void orc_sdpa_decode_gated(const bf16_t* q_rot, const bf16_t* k_cache, const bf16_t* v_cache,
                           const bf16_t* gate, int T, int Hq, int Hkv, int hd, int offset, int cap,
                           float scale, bf16_t* out);
void orc_greedy_rows(const bf16_t* logits, int rows, int V, uint32_t* tokens, bf16_t* lse_out);
void orc_argmax_rows(const bf16_t* logits, int rows, int V, uint32_t* out);

typedef struct orc_config {
  int hidden_size, num_hidden_layers, vocab_size;
  int num_experts, num_experts_per_tok, moe_intermediate_size, shared_expert_intermediate_size;
  int linear_num_key_heads, linear_num_value_heads, linear_key_head_dim, linear_value_head_dim;
  int linear_conv_kernel_dim;
  int num_attention_heads, num_key_value_heads, head_dim, rope_dims;
  int full_attention_interval;
  int norm_topk_prob;
  float rms_norm_eps;
  double rope_theta;
} orc_config;

typedef struct orc_attn_w { orc_linear q, k, v, o; const bf16_t* q_norm; const bf16_t* k_norm; } orc_attn_w;
typedef struct orc_gdn_w {
  orc_linear in_proj_qkv, in_proj_z, out_proj, in_proj_a, in_proj_b;
  const bf16_t *conv1d, *dt_bias, *a_log, *norm;
} orc_gdn_w;
typedef struct orc_layer_w {
  int linear;
  const bf16_t *input_ln, *post_ln;
  orc_gdn_w gdn;
  orc_attn_w attn;
  orc_moe_weights moe;
} orc_layer_w;
typedef struct orc_model_w {
  orc_config cfg;
  orc_linear embed, lm_head;
  const bf16_t* final_norm;
  const orc_layer_w* layers;
} orc_model_w;
typedef struct orc_mtp_w {
  const bf16_t *pre_fc_norm_embedding, *pre_fc_norm_hidden, *input_ln, *post_ln, *norm;
  orc_linear fc;
  orc_attn_w attn;
  orc_moe_weights moe; /* router / shared as linears; experts dense below */
  const bf16_t *ex_gate, *ex_up, *ex_down; /* [E, I, H], [E, I, H], [E, H, I] bf16 */
} orc_mtp_w;

typedef struct orc_lcache {
  bf16_t *k, *v;           /* [Hkv, cap, hd] */
  bf16_t* conv;            /* [K-1, D] */
  float* state;            /* [Hv, Dv, Dk] */
  bf16_t* conv_input;      /* capture: [K-1+T, D] */
  float* snaps;            /* capture: [T][state] */
} orc_lcache;
typedef struct orc_state {
  const orc_model_w* m;
  int cap, offset, last_T, max_T;
  orc_lcache* l;
  float *cos_t, *sin_t;
  /* the MTP head's one-layer cache */
  bf16_t *mk, *mv;
  int moffset;
} orc_state;

/* Test hook: while a log is set, every MoE block run by orc_forward / orc_mtp_hidden appends
 * the experts its router picked ([T, top_k] u32 per block, in call order), so a test can
 * evaluate an independent model on the same experts. NULL turns it off. */
static struct { uint32_t* buf; int cap, n; } g_picks;
ORC_API void orc_debug_log_picks(uint32_t* buf, int cap) { g_picks.buf = buf; g_picks.cap = cap; g_picks.n = 0; }
ORC_API int orc_debug_picks_logged(void) { return g_picks.n; }
static void log_picks(const uint32_t* inds, int n) {
  if (!g_picks.buf) return;
  for (int i = 0; i < n && g_picks.n < g_picks.cap; ++i) g_picks.buf[g_picks.n++] = inds[i];
}

static int key_dim(const orc_config* c) { return c->linear_num_key_heads * c->linear_key_head_dim; }
static int value_dim(const orc_config* c) { return c->linear_num_value_heads * c->linear_value_head_dim; }
static int conv_dim(const orc_config* c) { return 2 * key_dim(c) + value_dim(c); }
static size_t state_elems(const orc_config* c) {
  return (size_t)c->linear_num_value_heads * c->linear_value_head_dim * c->linear_key_head_dim;
}

ORC_API orc_state* orc_state_create(const orc_model_w* m, int cap, int max_T) {
  const orc_config* c = &m->cfg;
  orc_state* s = (orc_state*)calloc(1, sizeof *s);
  s->m = m;
  s->cap = cap;
  s->max_T = max_T;
  s->l = (orc_lcache*)calloc((size_t)c->num_hidden_layers, sizeof(orc_lcache));
  const size_t kv = (size_t)c->num_key_value_heads * cap * c->head_dim;
  const int S = c->linear_conv_kernel_dim - 1, D = conv_dim(c);
  for (int i = 0; i < c->num_hidden_layers; ++i) {
    if (m->layers[i].linear) {
      s->l[i].conv = (bf16_t*)calloc((size_t)S * D, 2);
      s->l[i].state = (float*)calloc(state_elems(c), 4);
      s->l[i].conv_input = (bf16_t*)calloc((size_t)(S + max_T) * D, 2);
      s->l[i].snaps = (float*)calloc(state_elems(c) * (size_t)max_T, 4);
    } else {
      s->l[i].k = (bf16_t*)calloc(kv, 2);
      s->l[i].v = (bf16_t*)calloc(kv, 2);
    }
  }
  s->cos_t = (float*)malloc(sizeof(float) * (size_t)cap * (c->rope_dims / 2));
  s->sin_t = (float*)malloc(sizeof(float) * (size_t)cap * (c->rope_dims / 2));
  orc_rope_table(cap, c->rope_dims, c->rope_theta, s->cos_t, s->sin_t);
  s->mk = (bf16_t*)calloc(kv, 2);
  s->mv = (bf16_t*)calloc(kv, 2);
  return s;
}

ORC_API void orc_state_destroy(orc_state* s) {
  if (!s) return;
  for (int i = 0; i < s->m->cfg.num_hidden_layers; ++i) {
    free(s->l[i].k); free(s->l[i].v); free(s->l[i].conv); free(s->l[i].state);
    free(s->l[i].conv_input); free(s->l[i].snaps);
  }
  free(s->l); free(s->cos_t); free(s->sin_t); free(s->mk); free(s->mv); free(s);
}

ORC_API int orc_state_offset(const orc_state* s) { return s->offset; }

static void attention(const orc_config* c, const orc_attn_w* a, const orc_state* s, const bf16_t* x, int T,
                      bf16_t* kc, bf16_t* vc, int offset, bf16_t* out) {
  const int Hq = c->num_attention_heads, Hkv = c->num_key_value_heads, hd = c->head_dim;
  bf16_t* qg = (bf16_t*)malloc(2 * (size_t)T * Hq * 2 * hd);
  bf16_t* kx = (bf16_t*)malloc(2 * (size_t)T * Hkv * hd);
  bf16_t* vx = (bf16_t*)malloc(2 * (size_t)T * Hkv * hd);
  bf16_t* q_rot = (bf16_t*)malloc(2 * (size_t)T * Hq * hd);
  bf16_t* gate = (bf16_t*)malloc(2 * (size_t)T * Hq * hd);
  bf16_t* att = (bf16_t*)malloc(2 * (size_t)T * Hq * hd);
  orc_linear_fwd(&a->q, x, T, qg);
  orc_linear_fwd(&a->k, x, T, kx);
  orc_linear_fwd(&a->v, x, T, vx);
  orc_attn_prep(qg, kx, vx, a->q_norm, a->k_norm, T, Hq, Hkv, hd, c->rope_dims, c->rms_norm_eps,
                s->cos_t, s->sin_t, offset, s->cap, q_rot, gate, kc, vc);
  orc_sdpa_decode_gated(q_rot, kc, vc, gate, T, Hq, Hkv, hd, offset, s->cap, 1.0f / sqrtf((float)hd), att);
  orc_linear_fwd(&a->o, att, T, out);
  free(qg); free(kx); free(vx); free(q_rot); free(gate); free(att);
}

/* T tokens through the trunk; hidden_out = post-norm rows [T, H]. capture keeps
 * per-layer windows and per-token states so orc_rewind can take rows back. */
ORC_API void orc_forward(orc_state* s, const uint32_t* tokens, int T, int capture, bf16_t* hidden_out) {
  const orc_model_w* m = s->m;
  const orc_config* c = &m->cfg;
  const int H = c->hidden_size, L = c->num_hidden_layers;
  const int Hk = c->linear_num_key_heads, Hv = c->linear_num_value_heads, Dk = c->linear_key_head_dim,
            Dv = c->linear_value_head_dim, K = c->linear_conv_kernel_dim, S = K - 1, D = conv_dim(c);
  const size_t hb = 2 * (size_t)T * H, se = state_elems(c);
  bf16_t *x = malloc(hb), *normed = malloc(hb), *r = malloc(hb), *h = malloc(hb), *n2 = malloc(hb), *mo = malloc(hb);
  embed_rows(&m->embed, H, tokens, T, x);
  orc_rms_norm(x, m->layers[0].input_ln, T, H, c->rms_norm_eps, normed);
  for (int i = 0; i < L; ++i) {
    const orc_layer_w* Lw = &m->layers[i];
    orc_lcache* lc = &s->l[i];
    if (Lw->linear) {
      const orc_gdn_w* g = &Lw->gdn;
      bf16_t *qkv = malloc(2 * (size_t)T * D), *z = malloc(2 * (size_t)T * value_dim(c));
      bf16_t *a = malloc(2 * (size_t)T * Hv), *b = malloc(2 * (size_t)T * Hv);
      bf16_t *q = malloc(2 * (size_t)T * key_dim(c)), *k = malloc(2 * (size_t)T * key_dim(c));
      bf16_t *v = malloc(2 * (size_t)T * value_dim(c)), *beta = malloc(2 * (size_t)T * Hv);
      float* gg = malloc(4 * (size_t)T * Hv);
      bf16_t *y = malloc(2 * (size_t)T * value_dim(c)), *gated = malloc(2 * (size_t)T * value_dim(c));
      bf16_t* ci = malloc(2 * (size_t)(S + T) * D);
      float* snaps = malloc(4 * se * (size_t)T);
      orc_linear_fwd(&g->in_proj_qkv, normed, T, qkv);
      orc_linear_fwd(&g->in_proj_z, normed, T, z);
      orc_linear_fwd(&g->in_proj_a, normed, T, a);
      orc_linear_fwd(&g->in_proj_b, normed, T, b);
      orc_gdn_front(lc->conv, qkv, g->conv1d, a, b, g->a_log, g->dt_bias, T, K, Hk, Dk, Hv, Dv, 1e-6f, q, k,
                    v, beta, gg, ci);
      orc_gdn_recurrence(q, k, v, gg, beta, lc->state, T, Hk, Hv, Dk, Dv, y, snaps);
      memcpy(lc->conv, ci + (size_t)T * D, 2 * (size_t)S * D); /* the last K-1 rows */
      memcpy(lc->state, snaps + se * (size_t)(T - 1), 4 * se);
      if (capture) {
        memcpy(lc->conv_input, ci, 2 * (size_t)(S + T) * D);
        memcpy(lc->snaps, snaps, 4 * se * (size_t)T);
      }
      orc_rms_norm_gated(y, g->norm, z, T * Hv, Dv, c->rms_norm_eps, gated);
      orc_linear_fwd(&g->out_proj, gated, T, r);
      free(qkv); free(z); free(a); free(b); free(q); free(k); free(v); free(beta); free(gg); free(y);
      free(gated); free(ci); free(snaps);
    } else {
      attention(c, &Lw->attn, s, normed, T, lc->k, lc->v, s->offset, r);
    }
    orc_add_rms_norm(x, r, Lw->post_ln, T, H, c->rms_norm_eps, h, n2);
    if (g_picks.buf) {
      uint32_t* picked = malloc(4 * (size_t)T * Lw->moe.top_k);
      orc_moe_block(&Lw->moe, n2, T, mo, picked, NULL, NULL);
      log_picks(picked, T * Lw->moe.top_k);
      free(picked);
    } else {
      orc_moe_block(&Lw->moe, n2, T, mo, NULL, NULL, NULL);
    }
    orc_add_rms_norm(h, mo, i + 1 < L ? m->layers[i + 1].input_ln : m->final_norm, T, H, c->rms_norm_eps, x,
                     normed);
  }
  memcpy(hidden_out, normed, hb);
  s->offset += T;
  s->last_T = T;
  free(x); free(normed); free(r); free(h); free(n2); free(mo);
}

/* TrunkCapture::rewind: keep the first `keep` rows of the last captured forward */
ORC_API void orc_rewind(orc_state* s, int keep) {
  const orc_config* c = &s->m->cfg;
  const int S = c->linear_conv_kernel_dim - 1, D = conv_dim(c);
  const size_t se = state_elems(c);
  for (int i = 0; i < c->num_hidden_layers; ++i) {
    if (!s->m->layers[i].linear) continue;
    memcpy(s->l[i].conv, s->l[i].conv_input + (size_t)keep * D, 2 * (size_t)S * D);
    memcpy(s->l[i].state, s->l[i].snaps + se * (size_t)(keep - 1), 4 * se);
  }
  s->offset -= s->last_T - keep;
  s->last_T = keep;
}

ORC_API void orc_logits(const orc_model_w* m, const bf16_t* hidden, int T, bf16_t* logits) {
  orc_linear_fwd(&m->lm_head, hidden, T, logits);
}

/* the MTP head's MoE with dense experts (src/ops/moe.rs:863-937) */
static void mtp_moe(const orc_config* c, const orc_mtp_w* w, const bf16_t* x, int T, bf16_t* out) {
  const int E = c->num_experts, H = c->hidden_size, I = c->moe_intermediate_size, k = c->num_experts_per_tok;
  const int SI = c->shared_expert_intermediate_size;
  bf16_t *gates = malloc(2 * (size_t)T * E), *probs = malloc(2 * (size_t)T * E), *scores = malloc(2 * (size_t)T * k);
  uint32_t *inds = malloc(4 * (size_t)T * k), *lhs = malloc(4 * (size_t)T * k), *rows = malloc(4 * (size_t)T * k);
  bf16_t *xg = malloc(2 * (size_t)T * k * I), *xu = malloc(2 * (size_t)T * k * I), *act = malloc(2 * (size_t)T * k * I);
  bf16_t *y = malloc(2 * (size_t)T * k * H), *sg = malloc(2 * (size_t)T * SI), *su = malloc(2 * (size_t)T * SI);
  bf16_t *sact = malloc(2 * (size_t)T * SI), *sy = malloc(2 * (size_t)T * H), *eg = malloc(2 * (size_t)T);
  orc_linear_fwd(&w->moe.router, x, T, gates);
  orc_softmax_bf16(gates, T, E, probs);
  orc_router_topk(probs, T, E, k, inds, scores);
  log_picks(inds, T * k);
  for (int r = 0; r < T * k; ++r) { lhs[r] = (uint32_t)(r / k); rows[r] = (uint32_t)r; }
  orc_dense_gather_mv(w->ex_gate, I, H, x, lhs, inds, T * k, xg);
  orc_dense_gather_mv(w->ex_up, I, H, x, lhs, inds, T * k, xu);
  orc_swiglu_bf16(xg, xu, (int64_t)T * k * I, act);
  orc_dense_gather_mv(w->ex_down, H, I, act, rows, inds, T * k, y);
  orc_linear_fwd(&w->moe.sh_gate, x, T, sg);
  orc_linear_fwd(&w->moe.sh_up, x, T, su);
  orc_swiglu_bf16(sg, su, (int64_t)T * SI, sact);
  orc_linear_fwd(&w->moe.sh_down, sact, T, sy);
  orc_linear_fwd(&w->moe.sh_egate, x, T, eg);
  orc_moe_combine(scores, y, eg, sy, T, k, H, c->norm_topk_prob, out);
  free(gates); free(probs); free(scores); free(inds); free(lhs); free(rows); free(xg); free(xu); free(act);
  free(y); free(sg); free(su); free(sact); free(sy); free(eg);
}

/* MtpHead::hidden: T trunk-hidden rows + the T ids that follow them -> post-norm hidden */
ORC_API void orc_mtp_hidden(orc_state* s, const orc_mtp_w* w, const bf16_t* trunk_hidden,
                            const uint32_t* next_ids, int T, bf16_t* hidden_out) {
  const orc_model_w* m = s->m;
  const orc_config* c = &m->cfg;
  const int H = c->hidden_size;
  const size_t hb = 2 * (size_t)T * H;
  bf16_t *emb = malloc(hb), *e = malloc(hb), *hh = malloc(hb), *joined = malloc(2 * hb), *x = malloc(hb);
  bf16_t *normed = malloc(hb), *r = malloc(hb), *h2 = malloc(hb), *n2 = malloc(hb), *mo = malloc(hb), *sum = malloc(hb);
  embed_rows(&m->embed, H, next_ids, T, emb);
  orc_rms_norm(emb, w->pre_fc_norm_embedding, T, H, c->rms_norm_eps, e);
  orc_rms_norm(trunk_hidden, w->pre_fc_norm_hidden, T, H, c->rms_norm_eps, hh);
  for (int t = 0; t < T; ++t) {
    memcpy(joined + (size_t)t * 2 * H, e + (size_t)t * H, 2 * (size_t)H);
    memcpy(joined + (size_t)t * 2 * H + H, hh + (size_t)t * H, 2 * (size_t)H);
  }
  orc_linear_fwd(&w->fc, joined, T, x);
  orc_rms_norm(x, w->input_ln, T, H, c->rms_norm_eps, normed);
  attention(c, &w->attn, s, normed, T, s->mk, s->mv, s->moffset, r);
  orc_add_rms_norm(x, r, w->post_ln, T, H, c->rms_norm_eps, h2, n2);
  mtp_moe(c, w, n2, T, mo);
  orc_add_rms_norm(h2, mo, w->norm, T, H, c->rms_norm_eps, sum, hidden_out);
  s->moffset += T;
  free(emb); free(e); free(hh); free(joined); free(x); free(normed); free(r); free(h2); free(n2); free(mo); free(sum);
}

ORC_API void orc_mtp_set_offset(orc_state* s, int off) { s->moffset = off; }

/* The sampler the two loops below drive (generate.rs:36-64): greedy unless
 * orc_set_sampler chose the top-p / top-k / temperature one (sample.rs:192-225). Each
 * loop call starts from the seed, as a freshly built TopSampler does. */
static struct {
  int kind;
  double temp, top_p;
  int top_k;
  uint64_t seed;
  int accept; /* 0: token equality (the reference), 1: probability ratio (speculative sampling) */
  int rng;    /* 0: threefry key sequence (the reference), 1: Philox4x32-10 counter stream */
  uint32_t key[2];
  uint64_t philox_n;
} g_sampler;
extern void orc_key_from_seed(uint64_t seed, uint32_t key[2]);
extern void orc_key_next(uint32_t state[2], uint32_t sub[2]);
extern void orc_random_bits(const uint32_t key[2], int n, uint32_t* out);
extern uint32_t orc_philox_draw(uint64_t seed, uint64_t n);
extern uint32_t orc_top_sample_bits(const bf16_t* logits, int V, double temp, double top_p, int top_k, uint32_t raw);
extern float orc_sampler_weights(const bf16_t* logits, int V, double temp, double top_p, int top_k, float* w);
extern uint32_t orc_draw_weights(const float* w, int V, uint32_t bits);
extern int orc_spec_accept(const float* wp, float sp, const float* wq, float sq, uint32_t x, uint32_t bits);
extern uint32_t orc_spec_resample(const float* wp, float sp, const float* wq, float sq, int V, uint32_t bits);
ORC_API void orc_set_sampler2(int kind, double temp, double top_p, int top_k, uint64_t seed, int accept, int rng) {
  g_sampler.kind = kind;
  g_sampler.temp = temp;
  g_sampler.top_p = top_p;
  g_sampler.top_k = top_k;
  g_sampler.seed = seed;
  g_sampler.accept = accept;
  g_sampler.rng = rng;
}
ORC_API void orc_set_sampler(int kind, double temp, double top_p, int top_k, uint64_t seed) {
  orc_set_sampler2(kind, temp, top_p, top_k, seed, 0, 0);
}
static void sampler_begin(void) {
  orc_key_from_seed(g_sampler.seed, g_sampler.key);
  g_sampler.philox_n = 0;
}
/* the next raw random word of the sampler's stream: one key split (threefry) or one counter
 * value (Philox) per draw */
static uint32_t next_bits(void) {
  if (g_sampler.rng == 1) return orc_philox_draw(g_sampler.seed, g_sampler.philox_n++);
  uint32_t sub[2], raw;
  orc_key_next(g_sampler.key, sub);
  orc_random_bits(sub, 1, &raw);
  return raw;
}
static uint32_t sample_row(const bf16_t* logits, int V) {
  if (g_sampler.kind == 0) {
    uint32_t t;
    orc_greedy_rows(logits, 1, V, &t, NULL);
    return t;
  }
  return orc_top_sample_bits(logits, V, g_sampler.temp, g_sampler.top_p, g_sampler.top_k, next_bits());
}

/* generate_step; returns the number of tokens written */
ORC_API int orc_generate(orc_state* s, const uint32_t* prompt, int n_prompt, int max_tokens, int prefill_step,
                         uint32_t* out) {
  const orc_model_w* m = s->m;
  const int H = m->cfg.hidden_size, V = m->cfg.vocab_size;
  bf16_t* hid = malloc(2 * (size_t)(prefill_step > n_prompt ? prefill_step : n_prompt) * H);
  bf16_t* logits = malloc(2 * (size_t)V);
  int processed = 0;
  while (n_prompt - processed > 1) {
    int n = prefill_step < n_prompt - processed - 1 ? prefill_step : n_prompt - processed - 1;
    orc_forward(s, prompt + processed, n, 0, hid);
    processed += n;
  }
  int rows = n_prompt - processed;
  uint32_t y, next;
  sampler_begin();
  orc_forward(s, prompt + processed, rows, 0, hid);
  orc_logits(m, hid + (size_t)(rows - 1) * H, 1, logits);
  y = sample_row(logits, V);
  int n = 0;
  while (n != max_tokens) {
    orc_forward(s, &y, 1, 0, hid);
    orc_logits(m, hid, 1, logits);
    next = sample_row(logits, V);
    out[n++] = y;
    y = next;
  }
  free(hid); free(logits);
  return n;
}

/* Scripted drafts (test hook, the counterpart of the device library's measurement aid): while
 * a list is set, the draft for output position p is forced[p] instead of the head's own
 * (the head still runs). n = 0 clears it. */
static struct { const uint32_t* toks; int n; } g_forced;
ORC_API void orc_mtp_force_drafts(const uint32_t* toks, int n) { g_forced.toks = toks; g_forced.n = n; }

typedef struct orc_mtp_stats { int64_t cycles, drafted, accepted, reached[8], accepted_by[8]; } orc_mtp_stats;

/* generate_step_mtp. With the greedy sampler every row's target is taken at once; with a
 * sampler whose rows depend on each other (each draw advances the key) the rows are
 * sampled one by one and only as far as the accept loop asks (mtp_generate.rs:236-279).
 * fr_ids/fr_head: the FR-Spec list and its
 * pruned head (NULL for the full lm_head). policy: 0 Cycle, 1 Committed. */
ORC_API int orc_mtp_generate(orc_state* s, const orc_mtp_w* w, const uint32_t* fr_ids, int fr_n,
                             const orc_linear* fr_head, const uint32_t* prompt, int n_prompt, int depth,
                             int max_tokens, int prefill_step, int policy, uint32_t* out,
                             orc_mtp_stats* stats) {
  const orc_model_w* m = s->m;
  const int H = m->cfg.hidden_size, V = m->cfg.vocab_size, W = depth + 1;
  memset(stats, 0, sizeof *stats);
  int big = prefill_step > W ? prefill_step : W;
  if (n_prompt > big) big = n_prompt;
  bf16_t *hid = malloc(2 * (size_t)big * H), *h = malloc(2 * (size_t)H), *mh = malloc(2 * (size_t)W * H);
  bf16_t *vlogits = malloc(2 * (size_t)W * V), *dlogits = malloc(2 * (size_t)V), *tmp = malloc(2 * (size_t)W * H);
  uint32_t* window = malloc(4 * (size_t)W);
  uint32_t* targets = malloc(4 * (size_t)W);
  /* probability-ratio acceptance: the drafts are DRAWN from the head's distribution q (under the
   * sampler's own temperature / top-p / top-k) and kept, in vocabulary space, for the verify */
  const int ratio = g_sampler.kind != 0 && g_sampler.accept == 1;
  float *wq = NULL, *wp = NULL, *wloc = NULL, *sq = NULL;
  if (ratio) {
    wq = calloc((size_t)depth * V, 4);
    wp = malloc(4 * (size_t)V);
    wloc = malloc(4 * (size_t)V);
    sq = malloc(4 * (size_t)depth);
  }
  int processed = 0;
  while (n_prompt - processed > 1) {
    int n = prefill_step < n_prompt - processed - 1 ? prefill_step : n_prompt - processed - 1;
    orc_forward(s, prompt + processed, n, 0, hid);
    processed += n;
  }
  const int rows = n_prompt - processed;
  orc_forward(s, prompt + processed, rows, 0, hid);
  orc_logits(m, hid + (size_t)(rows - 1) * H, 1, vlogits);
  sampler_begin();
  uint32_t primary = sample_row(vlogits, V);
  memcpy(h, hid + (size_t)(rows - 1) * H, 2 * (size_t)H);
  int emitted = 0;
  s->moffset = 0;
  for (;;) {
    if (policy == 0) s->moffset = 0;
    const int cycle_off = s->moffset;
    int want = max_tokens - (emitted + 1);
    if (want < 0) want = 0;
    if (want > depth) want = depth;
    memset(window, 0, 4 * (size_t)W);
    window[0] = primary;
    const bf16_t* hcur = h;
    for (int i = 0; i < want; ++i) {
      bf16_t* hi = mh + (size_t)i * H;
      orc_mtp_hidden(s, w, hcur, window + i, 1, hi);
      if (ratio) {
        const int Vd = fr_head ? fr_n : V;
        orc_linear_fwd(fr_head ? fr_head : &m->lm_head, hi, 1, dlogits);
        sq[i] = orc_sampler_weights(dlogits, Vd, g_sampler.temp, g_sampler.top_p, g_sampler.top_k, wloc);
        const uint32_t local = orc_draw_weights(wloc, Vd, next_bits());
        window[i + 1] = fr_head ? fr_ids[local] : local;
        float* q = wq + (size_t)i * V;
        memset(q, 0, 4 * (size_t)V);
        for (int l = 0; l < Vd; ++l) q[fr_head ? fr_ids[l] : (uint32_t)l] = wloc[l];
      } else if (fr_head) {
        uint32_t local;
        orc_linear_fwd(fr_head, hi, 1, dlogits);
        orc_argmax_rows(dlogits, 1, fr_n, &local);
        window[i + 1] = fr_ids[local];
      } else {
        orc_linear_fwd(&m->lm_head, hi, 1, dlogits);
        orc_argmax_rows(dlogits, 1, V, &window[i + 1]);
      }
      if (emitted + 1 + i < g_forced.n) window[i + 1] = g_forced.toks[emitted + 1 + i];
      hcur = hi;
    }
    if (want > 0) { stats->cycles++; stats->drafted += want; }
    const int n_rows = want + 1;
    orc_forward(s, window, n_rows, 1, hid);
    orc_logits(m, hid, n_rows, vlogits);
    const int independent = g_sampler.kind == 0;
    if (independent) orc_greedy_rows(vlogits, n_rows, V, targets, NULL);
    int k = 0, have = 0;
    uint32_t next_primary = 0;
    while (k < want) {
      if (ratio) {
        const float sp = orc_sampler_weights(vlogits + (size_t)k * V, V, g_sampler.temp, g_sampler.top_p,
                                             g_sampler.top_k, wp);
        const float* q = wq + (size_t)k * V;
        stats->reached[k]++;
        if (!orc_spec_accept(wp, sp, q, sq[k], window[1 + k], next_bits())) {
          next_primary = orc_spec_resample(wp, sp, q, sq[k], V, next_bits());
          have = 1;
          break;
        }
      } else {
        const uint32_t target = independent ? targets[k] : sample_row(vlogits + (size_t)k * V, V);
        stats->reached[k]++;
        if (target != window[1 + k]) { next_primary = target; have = 1; break; }
      }
      stats->accepted_by[k]++;
      stats->accepted++;
      k++;
    }
    if (!have) next_primary = independent ? targets[k] : sample_row(vlogits + (size_t)k * V, V);
    orc_rewind(s, k + 1);
    if (policy == 1) {
      s->moffset = cycle_off + 1;
      if (k > 0) orc_mtp_hidden(s, w, hid, window + 1, k, tmp);
    }
    memcpy(h, hid + (size_t)k * H, 2 * (size_t)H);
    for (int i = 0; i <= k; ++i) {
      out[emitted++] = i == 0 ? primary : window[i];
      if (emitted == max_tokens) goto done;
    }
    primary = next_primary;
  }
done:
  free(hid); free(h); free(mh); free(vlogits); free(dlogits); free(tmp); free(window); free(targets);
  free(wq); free(wp); free(wloc); free(sq);
  return emitted;
}
