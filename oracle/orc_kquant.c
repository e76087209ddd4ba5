/*
 * CPU oracle -- TEST INFRASTRUCTURE (see orc_common.h). k-quant formats and
 * mat-vecs.
 *
 * Storage is the reference's three-tensor split (src/ops/kquant.rs:20-26):
 *   Q4_K  qs     u8 [O, K/256, 128]   4-bit codes
 *         scales u8 [O, K/256, 12]    8 x 6-bit scale + 8 x 6-bit min
 *         dm     f16[O, K/256, 2]     d, dmin
 *   Q6_K  qs     u8 [O, K/256, 192]   ql[128] then qh[64]
 *         scales i8 [O, K/256, 16]
 *         dm     f16[O, K/256, 1]     d
 *
 * Dequantizers restate kernels/q4k.metal:43-96 and kernels/q6k.metal:47-77.
 *
 * The mat-vec's summation ORDER is this build's own (the reference's 32-lane
 * schedule is its schedule, not its contract; its contract is fp32
 * accumulation, agreement with the float64 product to 1e-5 and row
 * independence, tests/q4k.rs:10-26,120-163). The order is written for one
 * 64-lane wavefront per output row:
 *
 *   Q4_K  a row is cut into chunks of 16 code bytes (32 weights: 16 low
 *         nibbles = weights 64g+16h+i, 16 high nibbles = the same +32).
 *         chunk j -> lane j % 64, lanes accumulate their chunks ascending.
 *   Q6_K  chunk = 16 positions l of one 128-half: ql[l], ql[l+32], qh[l]
 *         -> 64 weights (l, l+32, l+64, l+96), 48 bytes.
 *
 *   y = tree64(lane partials), see orc_tree64.
 */
#include "orc_common.h"

/* ---- Q4_K field packing ------------------------------------------------- */

ORC_API void orc_q4k_get_scale_min(int j, const uint8_t* q, uint8_t* sc, uint8_t* m) {
  if (j < 4) {
    *sc = q[j] & 63;
    *m = q[j + 4] & 63;
  } else {
    *sc = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
    *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
  }
}

/* inverse of the above: 8 scales + 8 mins (each 0..63) -> 12 bytes. */
ORC_API void orc_q4k_put_scale_min(const uint8_t* sc, const uint8_t* m, uint8_t* q) {
  memset(q, 0, 12);
  for (int j = 0; j < 4; ++j) {
    q[j] = (uint8_t)(sc[j] & 63);
    q[j + 4] = (uint8_t)(m[j] & 63);
  }
  for (int j = 4; j < 8; ++j) {
    q[j + 4] = (uint8_t)((sc[j] & 0xF) | ((m[j] & 0xF) << 4));
    q[j - 4] |= (uint8_t)((sc[j] >> 4) << 6);
    q[j] |= (uint8_t)((m[j] >> 4) << 6);
  }
}

/* ---- dequantizers ------------------------------------------------------- */

ORC_API void orc_q4k_dequant(const uint8_t* qs, const uint8_t* scales, const f16_t* dm,
                             int64_t nblocks, float* out) {
  for (int64_t ib = 0; ib < nblocks; ++ib) {
    const uint8_t* q = qs + ib * 128;
    const uint8_t* sc = scales + ib * 12;
    const float d = orc_f16_to_f32(dm[ib * 2 + 0]);
    const float dmin = orc_f16_to_f32(dm[ib * 2 + 1]);
    float* y = out + ib * 256;
    for (int c = 0; c < 4; ++c) {
      uint8_t s1, m1, s2, m2;
      orc_q4k_get_scale_min(2 * c, sc, &s1, &m1);
      orc_q4k_get_scale_min(2 * c + 1, sc, &s2, &m2);
      const float d1 = d * (float)s1, mm1 = dmin * (float)m1;
      const float d2 = d * (float)s2, mm2 = dmin * (float)m2;
      for (int l = 0; l < 32; ++l) {
        y[64 * c + l] = d1 * (float)(q[32 * c + l] & 0xF) - mm1;
        y[64 * c + 32 + l] = d2 * (float)(q[32 * c + l] >> 4) - mm2;
      }
    }
  }
}

static inline void q6k_codes(const uint8_t* ql, const uint8_t* qh, int l, int q[4]) {
  q[0] = (int)((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
  q[1] = (int)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
  q[2] = (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
  q[3] = (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
}

ORC_API void orc_q6k_dequant(const uint8_t* w, const uint8_t* scales, const f16_t* dm,
                             int64_t nblocks, float* out) {
  for (int64_t ib = 0; ib < nblocks; ++ib) {
    const float d = orc_f16_to_f32(dm[ib]);
    for (int n = 0; n < 2; ++n) {
      const uint8_t* ql = w + ib * 192 + 64 * n;
      const uint8_t* qh = w + ib * 192 + 128 + 32 * n;
      const int8_t* sc = (const int8_t*)(scales + ib * 16) + 8 * n;
      float* y = out + ib * 256 + 128 * n;
      for (int l = 0; l < 32; ++l) {
        int q[4];
        q6k_codes(ql, qh, l, q);
        const int is = l / 16;
        for (int g = 0; g < 4; ++g)
          y[l + 32 * g] = d * (float)sc[is + 2 * g] * (float)q[g];
      }
    }
  }
}

/* A packer written independently of the dequantizer, for the brute-force
 * round-trip: 256 codes in 0..63 -> ql[128] qh[64]. Weight index i of a block:
 * half n = i/128, r = i%128, group g = r/32, l = r%32. */
ORC_API void orc_q6k_pack_codes(const uint8_t* codes, uint8_t* w) {
  memset(w, 0, 192);
  for (int i = 0; i < 256; ++i) {
    int n = i / 128, r = i % 128, g = r / 32, l = r % 32;
    uint8_t c = codes[i] & 63;
    uint8_t lo = c & 0xF, hi = c >> 4;
    uint8_t* ql = w + 64 * n;
    uint8_t* qh = w + 128 + 32 * n;
    int qlpos = l + ((g & 1) ? 32 : 0);
    if (g < 2)
      ql[qlpos] |= lo;
    else
      ql[qlpos] |= (uint8_t)(lo << 4);
    qh[l] |= (uint8_t)(hi << (2 * g));
  }
}

/* and for Q4_K: 256 codes in 0..15 -> qs[128]. weight i: chunk c = i/64,
 * r = i%64; r<32 low nibble of byte 32c+r, else high nibble of byte 32c+r-32. */
ORC_API void orc_q4k_pack_codes(const uint8_t* codes, uint8_t* qs) {
  memset(qs, 0, 128);
  for (int i = 0; i < 256; ++i) {
    int c = i / 64, r = i % 64;
    if (r < 32)
      qs[32 * c + r] |= codes[i] & 0xF;
    else
      qs[32 * c + r - 32] |= (uint8_t)((codes[i] & 0xF) << 4);
  }
}

/* ---- float64 yardstick (tools/dump_q4k.py:98-99) ------------------------- */

ORC_API void orc_kq_matvec_f64(int kind, const uint8_t* qs, const uint8_t* scales,
                               const f16_t* dm, int O, int K, const float* x, int M,
                               double* y) {
  const int nb = K / 256;
  float* wrow = (float*)malloc(sizeof(float) * (size_t)K);
  for (int o = 0; o < O; ++o) {
    if (kind == ORC_Q4K)
      orc_q4k_dequant(qs + (size_t)o * nb * 128, scales + (size_t)o * nb * 12,
                      dm + (size_t)o * nb * 2, nb, wrow);
    else
      orc_q6k_dequant(qs + (size_t)o * nb * 192, scales + (size_t)o * nb * 16,
                      dm + (size_t)o * nb, nb, wrow);
    for (int m = 0; m < M; ++m) {
      double acc = 0.0;
      for (int k = 0; k < K; ++k) acc += (double)wrow[k] * (double)x[(size_t)m * K + k];
      y[(size_t)m * O + o] = acc;
    }
  }
  free(wrow);
}

/* ---- canonical fp32 mat-vec, one row ------------------------------------ */

float orc_q4k_row_dot(const uint8_t* qs, const uint8_t* scales, const f16_t* dm, int K,
                      const float* x) {
  const int nb = K / 256;
  float lanes[64];
  for (int l = 0; l < 64; ++l) lanes[l] = 0.0f;
  for (int j = 0; j < nb * 8; ++j) {
    const int b = j / 8, c = j % 8, g = c / 2, h = c % 2;
    const uint8_t* q = qs + b * 128 + 32 * g + 16 * h;
    uint8_t s1, m1, s2, m2;
    orc_q4k_get_scale_min(2 * g, scales + b * 12, &s1, &m1);
    orc_q4k_get_scale_min(2 * g + 1, scales + b * 12, &s2, &m2);
    const float d = orc_f16_to_f32(dm[b * 2]), dmin = orc_f16_to_f32(dm[b * 2 + 1]);
    const float* xlo = x + b * 256 + 64 * g + 16 * h;
    const float* xhi = xlo + 32;
    float lo = 0.f, hi = 0.f, sl = 0.f, sh = 0.f;
    for (int i = 0; i < 16; ++i) {
      lo = fmaf(xlo[i], (float)(q[i] & 0xF), lo);
      hi = fmaf(xhi[i], (float)(q[i] >> 4), hi);
      sl = sl + xlo[i];
      sh = sh + xhi[i];
    }
    float t1 = lo * (float)s1;
    t1 = fmaf(hi, (float)s2, t1);
    float t2 = sl * (float)m1;
    t2 = fmaf(sh, (float)m2, t2);
    float p = d * t1;
    p = fmaf(-dmin, t2, p);
    lanes[j % 64] = lanes[j % 64] + p;
  }
  return orc_tree64(lanes);
}

float orc_q6k_row_dot(const uint8_t* w, const uint8_t* scales, const f16_t* dm, int K,
                      const float* x) {
  const int nb = K / 256;
  float lanes[64];
  for (int l = 0; l < 64; ++l) lanes[l] = 0.0f;
  for (int j = 0; j < nb * 4; ++j) {
    const int b = j / 4, n = (j % 4) / 2, u = j % 2;
    const uint8_t* ql = w + b * 192 + 64 * n;
    const uint8_t* qh = w + b * 192 + 128 + 32 * n;
    const int8_t* sc = (const int8_t*)(scales + b * 16) + 8 * n + u;
    const float d = orc_f16_to_f32(dm[b]);
    const float* xx = x + b * 256 + 128 * n + 16 * u;
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    for (int i = 0; i < 16; ++i) {
      int q[4];
      q6k_codes(ql, qh, 16 * u + i, q);
      for (int g = 0; g < 4; ++g) s[g] = fmaf(xx[i + 32 * g], (float)q[g], s[g]);
    }
    float t = s[0] * (float)sc[0];
    t = fmaf(s[1], (float)sc[2], t);
    t = fmaf(s[2], (float)sc[4], t);
    t = fmaf(s[3], (float)sc[6], t);
    float p = d * t;
    lanes[j % 64] = lanes[j % 64] + p;
  }
  return orc_tree64(lanes);
}

static inline size_t kq_qs_row(int kind, int K) { return (size_t)(K / 256) * (kind == ORC_Q4K ? 128 : 192); }
static inline size_t kq_sc_row(int kind, int K) { return (size_t)(K / 256) * (kind == ORC_Q4K ? 12 : 16); }
static inline size_t kq_dm_row(int kind, int K) { return (size_t)(K / 256) * (kind == ORC_Q4K ? 2 : 1); }

/* orc_ref_order.c: the same dot product in the reference's 32-lane schedule, selected for
 * every k-quant mat-vec of the oracle by orc_set_row_order (a measurement aid) */
extern int orc_row_order;
float orc_q4k_row_dot_ref32(const uint8_t* qs, const uint8_t* scales, const f16_t* dm, int K, const float* x,
                            int fma, int tree);
float orc_q6k_row_dot_ref32(const uint8_t* w, const uint8_t* scales, const f16_t* dm, int K, const float* x,
                            int fma, int tree);

float orc_affine4_row_dot(const uint8_t* w, const bf16_t* scales, const bf16_t* biases, int K, const float* x);  /* orc_moe.c */

float orc_kq_row_dot(int kind, const uint8_t* qs, const uint8_t* scales, const f16_t* dm,
                     int K, int64_t row, const float* x) {
  if (kind == ORC_AFFINE4_G32)  /* quantized::gather_qmv, 4-bit affine (src/ops/quantized.rs:531-589) */
    return orc_affine4_row_dot(qs + row * (K / 2), (const bf16_t*)scales + row * (K / 32),
                               (const bf16_t*)dm + row * (K / 32), K, x);
  const uint8_t* q = qs + row * kq_qs_row(kind, K);
  const uint8_t* s = scales + row * kq_sc_row(kind, K);
  const f16_t* d = dm + row * kq_dm_row(kind, K);
  if (orc_row_order > 0) {
    const int v = orc_row_order - 1, tree = v % 3, fma = v / 3;
    return kind == ORC_Q4K ? orc_q4k_row_dot_ref32(q, s, d, K, x, fma, tree)
                           : orc_q6k_row_dot_ref32(q, s, d, K, x, fma, tree);
  }
  return kind == ORC_Q4K ? orc_q4k_row_dot(q, s, d, K, x) : orc_q6k_row_dot(q, s, d, K, x);
}

/* x: [M,K] fp32 (already widened from bf16 by the caller if needed)
 * y: [M,O] fp32; if round_bf16 each output is rounded to bf16 precision. */
ORC_API void orc_kq_qmv(int kind, const uint8_t* qs, const uint8_t* scales, const f16_t* dm,
                        int O, int K, const float* x, int M, float* y, int round_bf16) {
#pragma omp parallel for schedule(static)
  for (int o = 0; o < O; ++o) {
    for (int m = 0; m < M; ++m) {
      float v = orc_kq_row_dot(kind, qs, scales, dm, K, o, x + (size_t)m * K);
      y[(size_t)m * O + o] = round_bf16 ? orc_rb(v) : v;
    }
  }
}

/* out[r] = x[lhs[r]] . W[rhs[r]]^T  (src/ops/kquant.rs:741-770) */
ORC_API void orc_kq_gather_qmv(int kind, const uint8_t* qs, const uint8_t* scales,
                               const f16_t* dm, int E, int O, int K, const float* x,
                               const uint32_t* lhs, const uint32_t* rhs, int rows, float* y,
                               int round_bf16) {
  (void)E;
#pragma omp parallel for schedule(static) collapse(2)
  for (int r = 0; r < rows; ++r) {
    for (int o = 0; o < O; ++o) {
      int64_t row = (int64_t)rhs[r] * O + o;
      float v = orc_kq_row_dot(kind, qs, scales, dm, K, row, x + (size_t)lhs[r] * K);
      y[(size_t)r * O + o] = round_bf16 ? orc_rb(v) : v;
    }
  }
}

/* ---- helpers exported for tests ---------------------------------------- */

ORC_API void orc_bf16_to_f32_n(const bf16_t* in, float* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = orc_bf16_to_f32(in[i]);
}
ORC_API void orc_f32_to_bf16_n(const float* in, bf16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = orc_f32_to_bf16(in[i]);
}
ORC_API void orc_f16_to_f32_n(const f16_t* in, float* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = orc_f16_to_f32(in[i]);
}
ORC_API void orc_f32_to_f16_n(const float* in, f16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = orc_f32_to_f16(in[i]);
}
ORC_API void orc_expf_n(const float* in, float* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = orc_expf(in[i]);
}
ORC_API void orc_logf_n(const float* in, float* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = orc_logf(in[i]);
}
ORC_API void orc_log1pf_n(const float* in, float* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = orc_log1pf(in[i]);
}
ORC_API void orc_sigmoid_bf16_n(const bf16_t* in, bf16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i)
    out[i] = orc_f32_to_bf16(orc_sigmoid_bf16(orc_bf16_to_f32(in[i])));
}
ORC_API float orc_tree64_export(const float* lanes) { return orc_tree64(lanes); }
