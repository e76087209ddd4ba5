/*
 * CPU oracle -- TEST INFRASTRUCTURE (see orc_common.h). RMS norms and the
 * gated-delta (linear attention) layer.
 *
 * Restates vendored rms_norm.metal:12-81 and
 * /root/reference/kernels/ornith_norm.metal:28-183 (rms, add_rms, rms_gated),
 * kernels/gdn_front.metal:65-190 (conv + silu + q/k norm + beta + decay),
 * kernels/gated_delta.metal:36-142 (the recurrence),
 * src/model/qwen3_5.rs:478-695 (layer wiring and per-token snapshots) and
 * :301-349 (rewind).
 *
 * Reduction orders are this build's (64-lane): a row of n values is cut into 64
 * contiguous pieces, each lane runs one fma chain over its piece, then tree64.
 * The recurrence gives each state row (128 wide) to 8 lanes; lane j owns
 * dk = 32m + 4j + i (m < 4, i < 4) in that order, and the 8 lane sums go through
 * the butterfly (xor 4, 2, 1).
 */
#include "orc_common.h"

static float row_sumsq(const float* x, int n) {
  const int per = n / 64;
  float lanes[64];
  for (int l = 0; l < 64; ++l) {
    float a = 0.f;
    for (int i = 0; i < per; ++i) a = fmaf(x[l * per + i], x[l * per + i], a);
    lanes[l] = a;
  }
  return orc_tree64(lanes);
}

/* out = bf16(w * bf16(x * inv)), inv = 1/sqrt(sum(x^2)/n + eps); w may be NULL (== 1) */
ORC_API void orc_rms_norm(const bf16_t* x, const bf16_t* w, int rows, int n, float eps,
                          bf16_t* out) {
  float* xf = (float*)malloc(sizeof(float) * (size_t)n);
  for (int r = 0; r < rows; ++r) {
    for (int i = 0; i < n; ++i) xf[i] = orc_bf16_to_f32(x[(size_t)r * n + i]);
    const float inv = orc_rsqrtf(row_sumsq(xf, n) / (float)n + eps);
    for (int i = 0; i < n; ++i) {
      float v = orc_rb(xf[i] * inv);
      if (w) v = orc_rb(orc_bf16_to_f32(w[i]) * v);
      out[(size_t)r * n + i] = orc_f32_to_bf16(v);
    }
  }
  free(xf);
}

/* h = bf16(a + b) (written out), then rms_norm(h) */
ORC_API void orc_add_rms_norm(const bf16_t* a, const bf16_t* b, const bf16_t* w, int rows, int n,
                              float eps, bf16_t* h_out, bf16_t* out) {
  for (int64_t i = 0; i < (int64_t)rows * n; ++i)
    h_out[i] = orc_f32_to_bf16(orc_bf16_to_f32(a[i]) + orc_bf16_to_f32(b[i]));
  orc_rms_norm(h_out, w, rows, n, eps, out);
}

/* Qwen3NextRMSNormGated: normed = bf16(w * bf16(y * inv)); out = bf16(silu_f32(z) * normed) */
ORC_API void orc_rms_norm_gated(const bf16_t* y, const bf16_t* w, const bf16_t* z, int rows, int n,
                                float eps, bf16_t* out) {
  float* xf = (float*)malloc(sizeof(float) * (size_t)n);
  for (int r = 0; r < rows; ++r) {
    for (int i = 0; i < n; ++i) xf[i] = orc_bf16_to_f32(y[(size_t)r * n + i]);
    const float inv = orc_rsqrtf(row_sumsq(xf, n) / (float)n + eps);
    for (int i = 0; i < n; ++i) {
      float normed = orc_rb(orc_bf16_to_f32(w[i]) * orc_rb(xf[i] * inv));
      float g = orc_bf16_to_f32(z[(size_t)r * n + i]);
      g = g * orc_sigmoid_f32(g);
      out[(size_t)r * n + i] = orc_f32_to_bf16(g * normed);
    }
  }
  free(xf);
}

/* softplus in bf16: logaddexp(x, 0) (kernels/ornith_logaddexp.h:12-23 at T = bf16) */
static float softplus_bf16(float x) {
  if (x != x) return x;
  float mx = x > 0.f ? x : 0.f, mn = x > 0.f ? 0.f : x;
  if (mn == -INFINITY || mx == INFINITY) return mx;
  float d = orc_rb(mn - mx);
  float e = orc_rb(orc_expf(d));
  float l = orc_rb(orc_log1pf(e));
  return orc_rb(mx + l);
}

/*
 * Front end. Shapes (B = 1):
 *   conv_state [K-1, D], qkv [T, D], cw [D, K], a,b [T, Hv], a_log, dt_bias [Hv]
 *   -> q,k [T, Hk, Dk], v [T, Hv, Dv], beta bf16 [T, Hv], g f32 [T, Hv],
 *      conv_input [K-1+T, D] (the concatenation; the next state is a 3-row slice)
 * D = 2*Hk*Dk + Hv*Dv; q scale Dk^-1, k scale Dk^-0.5 (as bf16).
 */
ORC_API void orc_gdn_front(const bf16_t* conv_state, const bf16_t* qkv, const bf16_t* cw,
                           const bf16_t* a_in, const bf16_t* b_in, const bf16_t* a_log,
                           const bf16_t* dt_bias, int T, int K, int Hk, int Dk, int Hv, int Dv,
                           float eps, bf16_t* q, bf16_t* k, bf16_t* v, bf16_t* beta, float* g,
                           bf16_t* conv_input) {
  const int S = K - 1, key_dim = Hk * Dk, D = 2 * key_dim + Hv * Dv;
  memcpy(conv_input, conv_state, 2 * (size_t)S * D);
  memcpy(conv_input + (size_t)S * D, qkv, 2 * (size_t)T * D);
  const float inv_scale = orc_rb(1.0f / sqrtf((float)Dk));
  const float q_scale = orc_rb((1.0f / sqrtf((float)Dk)) * (1.0f / sqrtf((float)Dk)));
  float* s = (float*)malloc(sizeof(float) * (size_t)D);
  for (int t = 0; t < T; ++t) {
    for (int c = 0; c < D; ++c) {
      float acc = 0.f;
      for (int i = 0; i < K; ++i)
        acc = fmaf(orc_bf16_to_f32(conv_input[(size_t)(t + i) * D + c]),
                   orc_bf16_to_f32(cw[(size_t)c * K + i]), acc);
      float cv = orc_rb(acc);
      s[c] = orc_rb(cv * orc_sigmoid_bf16(cv));
    }
    for (int slot = 0; slot < 2 * Hk; ++slot) {
      const float* xs = s + slot * Dk;
      const float inv = orc_rsqrtf(row_sumsq(xs, Dk) / (float)Dk + eps);
      const int is_q = slot < Hk;
      bf16_t* dst = (is_q ? q : k) + ((size_t)t * Hk + (is_q ? slot : slot - Hk)) * Dk;
      const float sc = is_q ? q_scale : inv_scale;
      for (int i = 0; i < Dk; ++i) dst[i] = orc_f32_to_bf16(sc * orc_rb(xs[i] * inv));
    }
    for (int i = 0; i < Hv * Dv; ++i) v[(size_t)t * Hv * Dv + i] = orc_f32_to_bf16(s[2 * key_dim + i]);
    for (int h = 0; h < Hv; ++h) {
      const int idx = t * Hv + h;
      float sp = softplus_bf16(orc_rb(orc_bf16_to_f32(a_in[idx]) + orc_bf16_to_f32(dt_bias[h])));
      float decay = orc_expf(orc_bf16_to_f32(a_log[h]));
      g[idx] = orc_expf(-decay * sp);
      beta[idx] = orc_f32_to_bf16(orc_sigmoid_bf16(orc_bf16_to_f32(b_in[idx])));
    }
  }
  free(s);
}

static float row8_sum(const float* st, const float* vec) {
  /* st, vec: 128 wide. lane j: dk = 32m + 4j + i */
  float lanes[8];
  for (int j = 0; j < 8; ++j) {
    float a = 0.f;
    for (int m = 0; m < 4; ++m)
      for (int i = 0; i < 4; ++i) a = fmaf(st[32 * m + 4 * j + i], vec[32 * m + 4 * j + i], a);
    lanes[j] = a;
  }
  float w[8];
  for (int s = 4; s >= 1; s >>= 1) {
    for (int j = 0; j < 8; ++j) w[j] = lanes[j] + lanes[j ^ s];
    memcpy(lanes, w, sizeof w);
  }
  return lanes[0];
}

/*
 * Recurrence over T tokens. state_in [Hv, Dv, Dk] f32; snapshots [T][Hv, Dv, Dk]
 * (the state after each token; snapshots[T-1] is the new state). Dk == 128.
 *   S *= g; kv = S.k; delta = (v - kv) * beta; S = fma(k, delta, S); y = bf16(S.q)
 */
ORC_API void orc_gdn_recurrence(const bf16_t* q, const bf16_t* k, const bf16_t* v, const float* g,
                                const bf16_t* beta, const float* state_in, int T, int Hk, int Hv,
                                int Dk, int Dv, bf16_t* y, float* snapshots) {
  const size_t ssz = (size_t)Hv * Dv * Dk;
#pragma omp parallel for schedule(static)
  for (int hv = 0; hv < Hv; ++hv) {
    const int hk = hv / (Hv / Hk);
    float kf[128], qf[128];
    float* st = (float*)malloc(sizeof(float) * (size_t)Dv * Dk);
    memcpy(st, state_in + (size_t)hv * Dv * Dk, sizeof(float) * (size_t)Dv * Dk);
    for (int t = 0; t < T; ++t) {
      for (int i = 0; i < Dk; ++i) {
        kf[i] = orc_bf16_to_f32(k[((size_t)t * Hk + hk) * Dk + i]);
        qf[i] = orc_bf16_to_f32(q[((size_t)t * Hk + hk) * Dk + i]);
      }
      const float gt = g[t * Hv + hv], bt = orc_bf16_to_f32(beta[t * Hv + hv]);
      for (int dv = 0; dv < Dv; ++dv) {
        float* row = st + (size_t)dv * Dk;
        for (int i = 0; i < Dk; ++i) row[i] = row[i] * gt;
        const float kv = row8_sum(row, kf);
        const float delta = (orc_bf16_to_f32(v[((size_t)t * Hv + hv) * Dv + dv]) - kv) * bt;
        for (int i = 0; i < Dk; ++i) row[i] = fmaf(kf[i], delta, row[i]);
        y[((size_t)t * Hv + hv) * Dv + dv] = orc_f32_to_bf16(row8_sum(row, qf));
      }
      memcpy(snapshots + (size_t)t * ssz + (size_t)hv * Dv * Dk, st,
             sizeof(float) * (size_t)Dv * Dk);
    }
    free(st);
  }
}
