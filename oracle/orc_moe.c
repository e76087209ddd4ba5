/*
 * CPU oracle -- TEST INFRASTRUCTURE (see orc_common.h). The sparse MoE block and
 * the small operators around it. Activations are bf16 (raw uint16) in memory.
 *
 * Restates /root/reference/src/ops/moe.rs:662-741 (block wiring),
 * kernels/moe.metal:207-244 (combine), :568-614 (router top-k),
 * kernels/ornith_elementwise.metal:97-105 (swiglu),
 * vendored softmax.h:10-98 (precise softmax, bf16 out),
 * vendored quantized.h:283-289,756-821 (8-bit affine mat-vec).
 */
#include "orc_common.h"
#include "orc_types.h"

float orc_kq_row_dot(int kind, const uint8_t* qs, const uint8_t* scales, const f16_t* dm, int K,
                     int64_t row, const float* x);

/* ---- row softmax, fp32 inside, bf16 out -----------------------------------
 * n must be a multiple of 64. Lane l owns elements [l*n/64, (l+1)*n/64); the
 * sum of exp(x - max) is lane-sequential then tree64; p = bf16(e * (1/sum)). */
ORC_API void orc_softmax_bf16(const bf16_t* x, int rows, int n, bf16_t* out) {
  const int per = n / 64;
  float* e = (float*)malloc(sizeof(float) * (size_t)n);
  for (int r = 0; r < rows; ++r) {
    const bf16_t* xr = x + (size_t)r * n;
    float m = -INFINITY;
    for (int i = 0; i < n; ++i) {
      float v = orc_bf16_to_f32(xr[i]);
      m = v > m ? v : m;
    }
    float lanes[64];
    for (int l = 0; l < 64; ++l) {
      float s = 0.f;
      for (int i = 0; i < per; ++i) {
        float ev = orc_expf(orc_bf16_to_f32(xr[l * per + i]) - m);
        e[l * per + i] = ev;
        s = s + ev;
      }
      lanes[l] = s;
    }
    const float inv = 1.0f / orc_tree64(lanes);
    for (int i = 0; i < n; ++i) out[(size_t)r * n + i] = orc_f32_to_bf16(e[i] * inv);
  }
  free(e);
}

/* ---- top-k by (value, then larger index); slot k-1-r holds the r-th pick ----
 * i.e. the slots are the last k of a stable ascending sort. Brute force. */
ORC_API void orc_router_topk(const bf16_t* p, int rows, int n, int k, uint32_t* inds,
                             bf16_t* scores) {
  uint8_t* taken = (uint8_t*)malloc((size_t)n);
  for (int r = 0; r < rows; ++r) {
    const bf16_t* pr = p + (size_t)r * n;
    memset(taken, 0, (size_t)n);
    for (int round = 0; round < k; ++round) {
      int best = -1;
      float bv = 0.f;
      for (int i = 0; i < n; ++i) {
        if (taken[i]) continue;
        float v = orc_bf16_to_f32(pr[i]);
        if (best < 0 || v > bv || (v == bv && i > best)) {
          best = i;
          bv = v;
        }
      }
      taken[best] = 1;
      inds[(size_t)r * k + (k - 1 - round)] = (uint32_t)best;
      scores[(size_t)r * k + (k - 1 - round)] = pr[best];
    }
  }
  free(taken);
}

/* swiglu, every intermediate in bf16: bf16(bf16(g * sigmoid_bf16(g)) * up) */
static inline bf16_t swiglu1(bf16_t g, bf16_t up) {
  float gf = orc_bf16_to_f32(g);
  float s = orc_rb(gf * orc_sigmoid_bf16(gf));
  return orc_f32_to_bf16(s * orc_bf16_to_f32(up));
}
ORC_API void orc_swiglu_bf16(const bf16_t* gate, const bf16_t* up, int64_t n, bf16_t* out) {
  for (int64_t i = 0; i < n; ++i) out[i] = swiglu1(gate[i], up[i]);
}

/* the block's tail (kernels/moe.metal:207-244), T = bf16:
 * denom = ((0+s0)+s1)...; w_j = bf16(s_j/denom); acc = bf16(bf16(y_j*w_j) + acc);
 * out = bf16(acc + bf16(sigmoid_bf16(gate) * shared)) */
ORC_API void orc_moe_combine(const bf16_t* scores, const bf16_t* y, const bf16_t* gate,
                             const bf16_t* shared, int tokens, int k, int dim, int normalize,
                             bf16_t* out) {
  for (int t = 0; t < tokens; ++t) {
    const bf16_t* s = scores + (size_t)t * k;
    float denom = 0.f;
    if (normalize)
      for (int j = 0; j < k; ++j) denom = orc_rb(orc_bf16_to_f32(s[j]) + denom);
    const float g = orc_sigmoid_bf16(orc_bf16_to_f32(gate[t]));
    for (int c = 0; c < dim; ++c) {
      float acc = 0.f;
      for (int j = 0; j < k; ++j) {
        float w = normalize ? orc_rb(orc_bf16_to_f32(s[j]) / denom) : orc_bf16_to_f32(s[j]);
        float weighted = orc_rb(orc_bf16_to_f32(y[((size_t)t * k + j) * dim + c]) * w);
        acc = orc_rb(weighted + acc);
      }
      float gated = orc_rb(g * orc_bf16_to_f32(shared[(size_t)t * dim + c]));
      out[(size_t)t * dim + c] = orc_f32_to_bf16(acc + gated);
    }
  }
}

/* ---- 8-bit affine, group 64: y = sum_g (s_g * sum x q + b_g * sum x) ---------
 * w u8[O,K], scales/biases bf16[O,K/64]. Lane l owns 8-element chunks
 * j = l + 64c; per chunk p = fma(sum_x, bias, scale * accum); tree64. */
extern int orc_row_order; /* orc_ref_order.c: > 0 selects the reference's 32-lane schedule */
float orc_affine4_row_dot_ref32(const uint8_t* w, const bf16_t* scales, const bf16_t* biases, int K, const float* x,
                                int fma, int tree);
float orc_affine8_row_dot_ref32(const uint8_t* w, const bf16_t* scales, const bf16_t* biases, int K, const float* x,
                                int fma, int tree);

float orc_affine8_row_dot(const uint8_t* w, const bf16_t* scales, const bf16_t* biases, int K,
                          const float* x) {
  if (orc_row_order > 0) return orc_affine8_row_dot_ref32(w, scales, biases, K, x, (orc_row_order - 1) / 3, (orc_row_order - 1) % 3);
  float lanes[64];
  for (int l = 0; l < 64; ++l) lanes[l] = 0.f;
  for (int j = 0; j < K / 8; ++j) {
    const float s = orc_bf16_to_f32(scales[j / 8]), b = orc_bf16_to_f32(biases[j / 8]);
    float acc = 0.f, sum = 0.f;
    for (int i = 0; i < 8; ++i) {
      acc = fmaf(x[8 * j + i], (float)w[8 * j + i], acc);
      sum = sum + x[8 * j + i];
    }
    float pp = s * acc;
    pp = fmaf(sum, b, pp);
    lanes[j % 64] = lanes[j % 64] + pp;
  }
  return orc_tree64(lanes);
}

ORC_API void orc_affine8_qmv(const uint8_t* w, const bf16_t* scales, const bf16_t* biases, int O,
                             int K, const bf16_t* x, int M, bf16_t* y) {
  float* xf = (float*)malloc(sizeof(float) * (size_t)K);
  for (int m = 0; m < M; ++m) {
    for (int i = 0; i < K; ++i) xf[i] = orc_bf16_to_f32(x[(size_t)m * K + i]);
    for (int o = 0; o < O; ++o)
      y[(size_t)m * O + o] = orc_f32_to_bf16(orc_affine8_row_dot(
          w + (size_t)o * K, scales + (size_t)o * (K / 64), biases + (size_t)o * (K / 64), K, xf));
  }
  free(xf);
}

/* ---- 4-bit affine, group 32 (the published artifact's format: mlx affine, bits 4, group 32;
 * /root/reference/src/ops/quantized.rs:311-333, vendored quantized.h:235-244 qdot at bits = 4):
 * w holds K/2 bytes a row, element i in the low (even i) or high (odd i) nibble of byte i/2
 * (mlx packs eight nibbles into a u32, lowest first); scales/biases bf16[O,K/32].
 * y = sum_g (s_g * sum x q + b_g * sum x). Lane l owns 16-element chunks j = l + 64c (two a
 * group); per chunk one fma chain over x*q and one plain sum of x, p = fma(sum_x, bias,
 * scale * accum); tree64. */
float orc_affine4_row_dot(const uint8_t* w, const bf16_t* scales, const bf16_t* biases, int K,
                          const float* x) {
  if (orc_row_order > 0) return orc_affine4_row_dot_ref32(w, scales, biases, K, x, (orc_row_order - 1) / 3, (orc_row_order - 1) % 3);
  float lanes[64];
  for (int l = 0; l < 64; ++l) lanes[l] = 0.f;
  for (int j = 0; j < K / 16; ++j) {
    const float s = orc_bf16_to_f32(scales[j / 2]), b = orc_bf16_to_f32(biases[j / 2]);
    float acc = 0.f, sum = 0.f;
    for (int i = 0; i < 16; ++i) {
      const uint8_t byte = w[8 * j + i / 2];
      const float q = (float)((i & 1) ? (byte >> 4) : (byte & 0xF));
      acc = fmaf(x[16 * j + i], q, acc);
      sum = sum + x[16 * j + i];
    }
    float pp = s * acc;
    pp = fmaf(sum, b, pp);
    lanes[j % 64] = lanes[j % 64] + pp;
  }
  return orc_tree64(lanes);
}

/* E == 1, lhs == rhs == NULL: plain mat-vec over M = rows rows of x. Otherwise the gathered
 * form (quantized.rs:531-589): y[r] = x[lhs[r]] . W[rhs[r]]^T over stacked experts [E,O,K]. */
ORC_API void orc_affine4_gather_qmv(const uint8_t* w, const bf16_t* scales, const bf16_t* biases, int E, int O,
                                    int K, const bf16_t* x, const uint32_t* lhs, const uint32_t* rhs, int rows,
                                    bf16_t* y) {
  (void)E;
#pragma omp parallel for schedule(dynamic)
  for (int r = 0; r < rows; ++r) {
    float* xf = (float*)malloc(sizeof(float) * (size_t)K);
    const size_t xr = lhs ? lhs[r] : (size_t)r, e = rhs ? rhs[r] : 0;
    for (int i = 0; i < K; ++i) xf[i] = orc_bf16_to_f32(x[xr * K + i]);
    for (int o = 0; o < O; ++o) {
      const size_t row = e * O + o;
      y[(size_t)r * O + o] = orc_f32_to_bf16(orc_affine4_row_dot(w + row * (K / 2), scales + row * (K / 32),
                                                                 biases + row * (K / 32), K, xf));
    }
    free(xf);
  }
}

/* 4-bit embedding rows: out = bf16(bf16(q * scale) + bias), as the 8-bit lookup below */
ORC_API void orc_embedding4(const uint8_t* w, const bf16_t* scales, const bf16_t* biases, int K,
                            const uint32_t* ids, int n, bf16_t* out) {
  for (int r = 0; r < n; ++r) {
    const size_t row = ids[r];
    for (int i = 0; i < K; ++i) {
      const uint8_t byte = w[row * (K / 2) + i / 2];
      const float q = (float)((i & 1) ? (byte >> 4) : (byte & 0xF));
      const float s = orc_bf16_to_f32(scales[row * (K / 32) + i / 32]);
      const float b = orc_bf16_to_f32(biases[row * (K / 32) + i / 32]);
      out[(size_t)r * K + i] = orc_f32_to_bf16(orc_rb(q * s) + b);
    }
  }
}

/* embedding row lookup: out = bf16(bf16(q * scale) + bias)
 * (vendored quantized.h affine_dequantize at T = bf16; src/ops/embedding.rs:18-46) */
ORC_API void orc_embedding(const uint8_t* w, const bf16_t* scales, const bf16_t* biases, int K,
                           const uint32_t* ids, int n, bf16_t* out) {
  for (int r = 0; r < n; ++r) {
    const size_t row = ids[r];
    for (int i = 0; i < K; ++i) {
      float s = orc_bf16_to_f32(scales[row * (K / 64) + i / 64]);
      float b = orc_bf16_to_f32(biases[row * (K / 64) + i / 64]);
      float v = orc_rb((float)w[row * K + i] * s);
      out[(size_t)r * K + i] = orc_f32_to_bf16(v + b);
    }
  }
}

/* ---- the whole block ------------------------------------------------------- */


float orc_dense_row_dot(const bf16_t* w, int K, const float* x);

/* y[M,O] bf16 = x[M,K] bf16 through any linear */
void orc_linear_fwd(const orc_linear* L, const bf16_t* x, int M, bf16_t* y) {
  const int O = L->km.O, K = L->km.K;
  float* xf = (float*)malloc(sizeof(float) * (size_t)K);
  for (int m = 0; m < M; ++m) {
    for (int i = 0; i < K; ++i) xf[i] = orc_bf16_to_f32(x[(size_t)m * K + i]);
#pragma omp parallel for schedule(static)
    for (int o = 0; o < O; ++o) {
      float v;
      if (L->mode == 0)
        v = orc_kq_row_dot(L->km.kind, L->km.qs, L->km.scales, L->km.dm, K, o, xf);
      else if (L->mode == 1)
        v = orc_affine8_row_dot(L->aw + (size_t)o * K, L->as + (size_t)o * (K / 64),
                                L->ab + (size_t)o * (K / 64), K, xf);
      else if (L->mode == 3)
        v = orc_affine4_row_dot(L->aw + (size_t)o * (K / 2), L->as + (size_t)o * (K / 32),
                                L->ab + (size_t)o * (K / 32), K, xf);
      else
        v = orc_dense_row_dot((const bf16_t*)L->aw + (size_t)o * K, K, xf);
      y[(size_t)m * O + o] = orc_f32_to_bf16(v);
    }
  }
  free(xf);
}



/* x [T,H] bf16 -> out [T,H] bf16; also returns router picks for the index check.
 * Optional taps (may be NULL): probs [T,E], act [T*k, I], ydown [T*k, H]. */
ORC_API void orc_moe_block(const orc_moe_weights* W, const bf16_t* x, int T, bf16_t* out,
                           uint32_t* inds_out, bf16_t* scores_out, bf16_t* probs_out) {
  const int E = W->router.km.O, H = W->router.km.K, I = W->ex_gate.O, k = W->top_k;
  bf16_t* gates = (bf16_t*)malloc(2 * (size_t)T * E);
  bf16_t* probs = (bf16_t*)malloc(2 * (size_t)T * E);
  uint32_t* inds = (uint32_t*)malloc(4 * (size_t)T * k);
  bf16_t* scores = (bf16_t*)malloc(2 * (size_t)T * k);
  bf16_t* sg = (bf16_t*)malloc(2 * (size_t)T * I);
  bf16_t* su = (bf16_t*)malloc(2 * (size_t)T * I);
  bf16_t* sact = (bf16_t*)malloc(2 * (size_t)T * I);
  bf16_t* sy = (bf16_t*)malloc(2 * (size_t)T * H);
  bf16_t* eg = (bf16_t*)malloc(2 * (size_t)T);
  bf16_t* act = (bf16_t*)malloc(2 * (size_t)T * k * I);
  bf16_t* y = (bf16_t*)malloc(2 * (size_t)T * k * H);

  orc_linear_fwd(&W->router, x, T, gates);
  orc_softmax_bf16(gates, T, E, probs);
  orc_router_topk(probs, T, E, k, inds, scores);
  orc_linear_fwd(&W->sh_gate, x, T, sg);
  orc_linear_fwd(&W->sh_up, x, T, su);
  orc_swiglu_bf16(sg, su, (int64_t)T * I, sact);
  orc_linear_fwd(&W->sh_down, sact, T, sy);
  orc_linear_fwd(&W->sh_egate, x, T, eg);

#pragma omp parallel for schedule(dynamic)
  for (int r = 0; r < T * k; ++r) {
    const int t = r / k;
    const int64_t e = inds[r];
    float* xf = (float*)malloc(sizeof(float) * (size_t)(H > I ? H : I));
    for (int i = 0; i < H; ++i) xf[i] = orc_bf16_to_f32(x[(size_t)t * H + i]);
    for (int o = 0; o < I; ++o) {
      bf16_t g = orc_f32_to_bf16(orc_kq_row_dot(W->ex_gate.kind, W->ex_gate.qs, W->ex_gate.scales,
                                                W->ex_gate.dm, H, e * I + o, xf));
      bf16_t u = orc_f32_to_bf16(orc_kq_row_dot(W->ex_up.kind, W->ex_up.qs, W->ex_up.scales,
                                                W->ex_up.dm, H, e * I + o, xf));
      act[(size_t)r * I + o] = swiglu1(g, u);
    }
    for (int i = 0; i < I; ++i) xf[i] = orc_bf16_to_f32(act[(size_t)r * I + i]);
    for (int o = 0; o < H; ++o)
      y[(size_t)r * H + o] = orc_f32_to_bf16(orc_kq_row_dot(
          W->ex_down.kind, W->ex_down.qs, W->ex_down.scales, W->ex_down.dm, I, e * H + o, xf));
    free(xf);
  }
  orc_moe_combine(scores, y, eg, sy, T, k, H, W->normalize, out);

  if (inds_out) memcpy(inds_out, inds, 4 * (size_t)T * k);
  if (scores_out) memcpy(scores_out, scores, 2 * (size_t)T * k);
  if (probs_out) memcpy(probs_out, probs, 2 * (size_t)T * E);
  free(gates); free(probs); free(inds); free(scores); free(sg); free(su); free(sact);
  free(sy); free(eg); free(act); free(y);
}
