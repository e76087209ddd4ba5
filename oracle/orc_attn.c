/*
 * CPU oracle -- TEST INFRASTRUCTURE (see orc_common.h). Full-attention layer pieces
 * at decode / verify width: per-head q/k RMS, partial RoPE, KV append, causal
 * attention over the cache, sigmoid output gate.
 *
 * Restates /root/reference/src/model/qwen3_5.rs:430-474 (wiring),
 * src/ops/rope.rs:6-60 with vendored rope.metal:11-67 (non-traditional rotation of
 * pairs (i, i + dims/2) of the first `dims` channels), src/model/cache.rs:38-79
 * (append at `offset`), vendored sdpa_vector.h:15-177 (q scaled in fp32, fp32
 * online softmax, key i visible to query row r iff i <= offset + r) and
 * kernels/ornith_elementwise.metal sigmoid_gate.
 *
 * Summation order (this build's): keys are cut into blocks of 256 by absolute
 * position. Inside a block the score of a key is one fma chain over the head
 * dimension ascending; p = exp(s - m_block); the block's sum of p is four tree64
 * (64 keys each) folded left to right; the block's value sum is one fma chain per
 * channel over keys ascending. Blocks are merged in ascending order with weights
 * exp(m_block - M). Keys a row may not see contribute p = 0, so row r of a T-row
 * call equals a one-row call at that position bit for bit.
 */
#include "orc_common.h"

#define ATT_KB 256

/* cos/sin tables [npos][dims/2], fp32 from double libm */
ORC_API void orc_rope_table(int npos, int dims, double theta, float* cos_t, float* sin_t) {
  const int half = dims / 2;
  for (int pos = 0; pos < npos; ++pos)
    for (int i = 0; i < half; ++i) {
      const double inv_freq = pow(theta, -(double)i / (double)half);
      const double ang = (double)pos * inv_freq;
      cos_t[(size_t)pos * half + i] = (float)cos(ang);
      sin_t[(size_t)pos * half + i] = (float)sin(ang);
    }
}

static float head_sumsq(const float* x, int n) {
  const int per = n / 64;
  float lanes[64];
  for (int l = 0; l < 64; ++l) {
    float a = 0.f;
    for (int i = 0; i < per; ++i) a = fmaf(x[l * per + i], x[l * per + i], a);
    lanes[l] = a;
  }
  return orc_tree64(lanes);
}

/* one head: rms(w) then rope at `pos`; in/out bf16 [hd] */
static void norm_rope_head(const bf16_t* in, const bf16_t* w, int hd, int dims, float eps,
                           const float* cos_p, const float* sin_p, bf16_t* out) {
  float x[512];
  for (int i = 0; i < hd; ++i) x[i] = orc_bf16_to_f32(in[i]);
  const float inv = orc_rsqrtf(head_sumsq(x, hd) / (float)hd + eps);
  for (int i = 0; i < hd; ++i) x[i] = orc_rb(orc_bf16_to_f32(w[i]) * orc_rb(x[i] * inv));
  const int half = dims / 2;
  for (int i = 0; i < hd; ++i) out[i] = orc_f32_to_bf16(x[i]);
  for (int i = 0; i < half; ++i) {
    const float x1 = x[i], x2 = x[i + half], c = cos_p[i], s = sin_p[i];
    float a = x1 * c;
    a = fmaf(-x2, s, a);
    float b = x1 * s;
    b = fmaf(x2, c, b);
    out[i] = orc_f32_to_bf16(a);
    out[i + half] = orc_f32_to_bf16(b);
  }
}

/*
 * qg [T, Hq, 2*hd] (query | gate per head), kx, vx [T, Hkv, hd] straight from the
 * projections. Writes q_rot [T, Hq, hd], gate [T, Hq, hd], and appends K (normed,
 * rotated) and V at rows [offset, offset+T) of k_cache/v_cache [Hkv, cap, hd].
 */
ORC_API void orc_attn_prep(const bf16_t* qg, const bf16_t* kx, const bf16_t* vx,
                           const bf16_t* q_norm_w, const bf16_t* k_norm_w, int T, int Hq, int Hkv,
                           int hd, int rope_dims, float eps, const float* cos_t,
                           const float* sin_t, int offset, int cap, bf16_t* q_rot, bf16_t* gate,
                           bf16_t* k_cache, bf16_t* v_cache) {
  const int half = rope_dims / 2;
  for (int t = 0; t < T; ++t) {
    const float* cp = cos_t + (size_t)(offset + t) * half;
    const float* sp = sin_t + (size_t)(offset + t) * half;
    for (int h = 0; h < Hq; ++h) {
      const bf16_t* src = qg + ((size_t)t * Hq + h) * 2 * hd;
      norm_rope_head(src, q_norm_w, hd, rope_dims, eps, cp, sp, q_rot + ((size_t)t * Hq + h) * hd);
      memcpy(gate + ((size_t)t * Hq + h) * hd, src + hd, 2 * (size_t)hd);
    }
    for (int h = 0; h < Hkv; ++h) {
      norm_rope_head(kx + ((size_t)t * Hkv + h) * hd, k_norm_w, hd, rope_dims, eps, cp, sp,
                     k_cache + ((size_t)h * cap + offset + t) * hd);
      memcpy(v_cache + ((size_t)h * cap + offset + t) * hd, vx + ((size_t)t * Hkv + h) * hd,
             2 * (size_t)hd);
    }
  }
}

/* n = 1, 2, 4 or 8 values added pairwise: (p0 + p1) + (p2 + p3), ... */
static float pair_tree(const float* p, int n) {
  float t[8];
  for (int i = 0; i < n; ++i) t[i] = p[i];
  for (int w = n; w > 1; w /= 2)
    for (int i = 0; i < w / 2; ++i) t[i] = t[2 * i] + t[2 * i + 1];
  return t[0];
}

/*
 * q_rot [T, Hq, hd], caches [Hkv, cap, hd] holding offset+T rows, gate [T, Hq, hd]
 * -> out [T, Hq*hd] = bf16(sigmoid_bf16(gate) * bf16(attn)). hd <= 512.
 */
ORC_API void orc_sdpa_decode_gated(const bf16_t* q_rot, const bf16_t* k_cache,
                                   const bf16_t* v_cache, const bf16_t* gate, int T, int Hq,
                                   int Hkv, int hd, int offset, int cap, float scale, bf16_t* out) {
  const int gqa = Hq / Hkv;
#pragma omp parallel for schedule(dynamic) collapse(2)
  for (int t = 0; t < T; ++t) {
    for (int h = 0; h < Hq; ++h) {
      const int hk = h / gqa;
      const int last = offset + t; /* last visible key */
      const int nblk = last / ATT_KB + 1;
      float qs[512];
      for (int d = 0; d < hd; ++d) qs[d] = scale * orc_bf16_to_f32(q_rot[((size_t)t * Hq + h) * hd + d]);
      float* mb = (float*)malloc(sizeof(float) * (size_t)nblk);
      float* lb = (float*)malloc(sizeof(float) * (size_t)nblk);
      float* ob = (float*)malloc(sizeof(float) * (size_t)nblk * hd);
      for (int b = 0; b < nblk; ++b) {
        float s[ATT_KB], pr[ATT_KB];
        float m = -INFINITY;
        for (int i = 0; i < ATT_KB; ++i) {
          const int key = b * ATT_KB + i;
          if (key > last) {
            s[i] = -INFINITY;
            continue;
          }
          const bf16_t* kr = k_cache + ((size_t)hk * cap + key) * hd;
          /* one chain per 64 channels, the chains added pairwise */
          float part[8];
          const int nch = hd / 64;
          for (int c = 0; c < nch; ++c) {
            float a = 0.f;
            for (int d = 64 * c; d < 64 * c + 64; ++d) a = fmaf(qs[d], orc_bf16_to_f32(kr[d]), a);
            part[c] = a;
          }
          const float a = pair_tree(part, nch);
          s[i] = a;
          m = a > m ? a : m;
        }
        for (int i = 0; i < ATT_KB; ++i)
          pr[i] = (b * ATT_KB + i > last) ? 0.f : orc_expf(s[i] - m);
        float l = orc_tree64(pr);
        l = l + orc_tree64(pr + 64);
        l = l + orc_tree64(pr + 128);
        l = l + orc_tree64(pr + 192);
        for (int d = 0; d < hd; ++d) {
          /* one chain per 64 keys (keys past the last visible one are not added), the four
           * chains added pairwise */
          float part[ATT_KB / 64];
          for (int c = 0; c < ATT_KB / 64; ++c) {
            float a = 0.f;
            for (int i = 64 * c; i < 64 * c + 64; ++i) {
              const int key = b * ATT_KB + i;
              if (key > last) break;
              a = fmaf(pr[i], orc_bf16_to_f32(v_cache[((size_t)hk * cap + key) * hd + d]), a);
            }
            part[c] = a;
          }
          ob[(size_t)b * hd + d] = pair_tree(part, ATT_KB / 64);
        }
        mb[b] = m;
        lb[b] = l;
      }
      float M = -INFINITY;
      for (int b = 0; b < nblk; ++b) M = mb[b] > M ? mb[b] : M;
      float L = 0.f;
      float O[512];
      for (int d = 0; d < hd; ++d) O[d] = 0.f;
      for (int b = 0; b < nblk; ++b) {
        const float w = orc_expf(mb[b] - M);
        L = fmaf(lb[b], w, L);
        for (int d = 0; d < hd; ++d) O[d] = fmaf(ob[(size_t)b * hd + d], w, O[d]);
      }
      for (int d = 0; d < hd; ++d) {
        const float att = orc_rb(O[d] / L);
        const float g = orc_sigmoid_bf16(orc_bf16_to_f32(gate[((size_t)t * Hq + h) * hd + d]));
        out[((size_t)t * Hq + h) * hd + d] = orc_f32_to_bf16(g * att);
      }
      free(mb); free(lb); free(ob);
    }
  }
}
