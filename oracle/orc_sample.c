/*
 * CPU oracle -- TEST INFRASTRUCTURE (see orc_common.h). Greedy token selection.
 *
 * Restates /root/reference/src/ops/sample.rs:1-19,134-191: the target token is
 * argmax(logits - logsumexp(logits)) evaluated in bf16 (the subtraction can merge
 * neighbouring logits, so it is kept), ties to the lowest index (vendored
 * arg_reduce.metal:54-64); the draft chain takes argmax of the raw logits.
 *
 * logsumexp order (this build's): the vocabulary is cut into chunks of 1024; a
 * chunk's m_c = max and l_c = sum exp(x - m_c) (16 tree64 of 64 consecutive
 * values, folded left to right); chunks merge ascending:
 * L = fma(l_c, exp(m_c - M), L); lse = bf16(log(L) + M).
 */
#include "orc_common.h"

#define LSE_CHUNK 1024

ORC_API float orc_logsumexp_bf16(const bf16_t* x, int V) {
  const int nch = (V + LSE_CHUNK - 1) / LSE_CHUNK;
  float* mc = (float*)malloc(sizeof(float) * (size_t)nch);
  float* lc = (float*)malloc(sizeof(float) * (size_t)nch);
  for (int c = 0; c < nch; ++c) {
    const int n = (V - c * LSE_CHUNK) < LSE_CHUNK ? (V - c * LSE_CHUNK) : LSE_CHUNK;
    float m = -INFINITY;
    for (int i = 0; i < n; ++i) {
      float v = orc_bf16_to_f32(x[c * LSE_CHUNK + i]);
      m = v > m ? v : m;
    }
    float e[LSE_CHUNK];
    for (int i = 0; i < LSE_CHUNK; ++i)
      e[i] = i < n ? orc_expf(orc_bf16_to_f32(x[c * LSE_CHUNK + i]) - m) : 0.f;
    float l = orc_tree64(e);
    for (int w = 1; w < 16; ++w) l = l + orc_tree64(e + 64 * w);
    mc[c] = m;
    lc[c] = l;
  }
  float M = -INFINITY;
  for (int c = 0; c < nch; ++c) M = mc[c] > M ? mc[c] : M;
  float L = 0.f;
  for (int c = 0; c < nch; ++c) L = fmaf(lc[c], orc_expf(mc[c] - M), L);
  free(mc);
  free(lc);
  return orc_rb(orc_logf(L) + M);
}

/* tokens[r] = argmax_i bf16(x[r,i] - lse_r), lowest index on ties */
ORC_API void orc_greedy_rows(const bf16_t* logits, int rows, int V, uint32_t* tokens,
                             bf16_t* lse_out) {
  for (int r = 0; r < rows; ++r) {
    const bf16_t* x = logits + (size_t)r * V;
    const float lse = orc_logsumexp_bf16(x, V);
    if (lse_out) lse_out[r] = orc_f32_to_bf16(lse);
    int best = 0;
    float bv = -INFINITY;
    for (int i = 0; i < V; ++i) {
      float lp = orc_rb(orc_bf16_to_f32(x[i]) - lse);
      if (lp > bv) {
        bv = lp;
        best = i;
      }
    }
    tokens[r] = (uint32_t)best;
  }
}

/* plain argmax of the raw logits (the draft chain), lowest index on ties */
ORC_API void orc_argmax_rows(const bf16_t* logits, int rows, int V, uint32_t* out) {
  for (int r = 0; r < rows; ++r) {
    int best = 0;
    float bv = -INFINITY;
    for (int i = 0; i < V; ++i) {
      float v = orc_bf16_to_f32(logits[(size_t)r * V + i]);
      if (v > bv) {
        bv = v;
        best = i;
      }
    }
    out[r] = (uint32_t)best;
  }
}
