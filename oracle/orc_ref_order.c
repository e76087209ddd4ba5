/*
 * CPU oracle -- TEST INFRASTRUCTURE (see orc_common.h). The k-quant mat-vec in the
 * REFERENCE's own lane schedule, for measuring how often integer results (router expert
 * ids, argmax tokens) depend on the summation order.
 *
 * The library and the rest of this oracle sum a row in an order made for 64-lane wavefronts
 * (orc_kquant.c). The reference sums it in a 32-lane schedule:
 *   Q4_K  /root/reference/kernels/q4k.metal:120-222: lane -> ix = lane / 8 (block phase, blocks
 *         ix, ix + 4, ...), it = lane % 8, iq = it / 4, ir = it % 4; 32 activations a lane a
 *         block; four interleaved accumulators per 64-group with the unshifted-mask scaling
 *         (x 256, x 16, x 4096 undone by exact factors); then simd_sum over the 32 lanes.
 *   Q6_K  /root/reference/kernels/q6k.metal:87-169: ix = lane % 2 (block phase), tid = lane / 2,
 *         ip = tid / 8, il = tid % 8, 16 weights a lane a block; then simd_sum.
 * Two things about that schedule are not in the reference's source: how Metal's simd_sum
 * folds the 32 lanes, and whether its compiler contracts a * b + c into a fused multiply-add
 * (the reference's own src/bin/cpu_row.rs:53-90 tries three trees with and without
 * contraction for this reason). Both are parameters here:
 *   tree 0: shuffle_xor butterfly (masks 1, 2, 4, 8, 16), 1: shuffle_down halving (16 .. 1),
 *        2: lane order;   fma 0: every product rounded, 1: accumulations and sums of
 *        products contracted where the source has the shape a * b + c.
 * None of the six variants is "the" reference; the spread over them is the measurement.
 *
 * The mlx affine formats (4-bit group 32, 8-bit group 64) in the reference's schedule as well:
 *   vendored kernels/mlx/mlx/backend/metal/kernels/quantized.h:757-821 (qmv_fast_impl), :62-70 and
 *   :98-101 (load_vector), :235-244 and :282-288 (qdot): lane l of 32 takes values_per_thread
 *   = 16 (4-bit) or 8 (8-bit) consecutive values of every block of 512 / 256; 4-bit: the
 *   activations are summed four at a time (sum += x0 + x1 + x2 + x3) and pre-divided by 1, 16,
 *   256, 4096 against the unshifted nibble masks (exact: the products are those of x and the
 *   nibble), the four products of a 16-bit word are added up and then added to the accumulator;
 *   8-bit: accum += x * w one value at a time; a lane's block result scale * accum + sum * bias is
 *   added to its running result; then simd_sum. The same two parameters apply.
 */
#include "orc_common.h"

static float fold32(const float* v, int tree) {
  float a[32];
  memcpy(a, v, sizeof a);
  if (tree == 0) {
    for (int d = 1; d < 32; d <<= 1) {
      float n[32];
      for (int i = 0; i < 32; ++i) n[i] = a[i] + a[i ^ d];
      memcpy(a, n, sizeof a);
    }
    return a[0];
  }
  if (tree == 1) {
    for (int d = 16; d >= 1; d >>= 1)
      for (int i = 0; i < d; ++i) a[i] = a[i] + a[i + d];
    return a[0];
  }
  float s = 0.f;
  for (int i = 0; i < 32; ++i) s = s + a[i];
  return s;
}

static inline float mac(float acc, float a, float b, int fma) { return fma ? fmaf(a, b, acc) : acc + a * b; }

float orc_q4k_row_dot_ref32(const uint8_t* qs8, const uint8_t* scales8, const f16_t* dm, int K, const float* x,
                            int fma, int tree) {
  const uint16_t* qs = (const uint16_t*)qs8;         /* 64 u16 a block */
  const uint16_t* scales = (const uint16_t*)scales8; /* 6 u16 a block */
  const int nb = K / 256;
  float lanes[32];
  for (int lane = 0; lane < 32; ++lane) {
    const int ix = lane / 8, it = lane % 8, iq = it / 4, ir = it % 4;
    float sumf = 0.f;
    for (int ib = ix; ib < nb; ib += 4) {
      const float* y4 = x + ib * 256 + 64 * iq + 8 * ir;
      float yl[16], yh[16], sumy[4] = {0.f, 0.f, 0.f, 0.f};
      for (int i = 0; i < 8; ++i) {
        yl[i] = y4[i];          sumy[0] += yl[i];
        yl[i + 8] = y4[i + 32]; sumy[1] += yl[i + 8];
        yh[i] = y4[i + 128];    sumy[2] += yh[i];
        yh[i + 8] = y4[i + 160]; sumy[3] += yh[i + 8];
      }
      const uint16_t* sc = scales + ib * 6 + iq;
      const uint16_t* q1 = qs + ib * 64 + 16 * iq + 4 * ir;
      const uint16_t* q2 = q1 + 32;
      uint16_t sc16[4];
      sc16[0] = sc[0] & 0x3f3f;
      sc16[1] = sc[2] & 0x3f3f;
      sc16[2] = (uint16_t)(((sc[4] >> 0) & 0x0f0f) | ((sc[0] & 0xc0c0) >> 2));
      sc16[3] = (uint16_t)(((sc[4] >> 4) & 0x0f0f) | ((sc[2] & 0xc0c0) >> 2));
      float sc8[8];
      for (int j = 0; j < 4; ++j) {
        sc8[2 * j] = (float)(sc16[j] & 0xff);
        sc8[2 * j + 1] = (float)(sc16[j] >> 8);
      }
      float acc1[4] = {0, 0, 0, 0}, acc2[4] = {0, 0, 0, 0};
      for (int i = 0; i < 4; ++i) {
        acc1[0] = mac(acc1[0], yl[2 * i + 0], (float)(q1[i] & 0x000F), fma);
        acc1[1] = mac(acc1[1], yl[2 * i + 1], (float)(q1[i] & 0x0F00), fma);
        acc1[2] = mac(acc1[2], yl[2 * i + 8], (float)(q1[i] & 0x00F0), fma);
        acc1[3] = mac(acc1[3], yl[2 * i + 9], (float)(q1[i] & 0xF000), fma);
        acc2[0] = mac(acc2[0], yh[2 * i + 0], (float)(q2[i] & 0x000F), fma);
        acc2[1] = mac(acc2[1], yh[2 * i + 1], (float)(q2[i] & 0x0F00), fma);
        acc2[2] = mac(acc2[2], yh[2 * i + 8], (float)(q2[i] & 0x00F0), fma);
        acc2[3] = mac(acc2[3], yh[2 * i + 9], (float)(q2[i] & 0xF000), fma);
      }
      const float k256 = 1.f / 256.f;
      const float a0 = mac(acc1[0], k256, acc1[1], fma), a1 = mac(acc1[2], k256, acc1[3], fma);
      const float a2 = mac(acc2[0], k256, acc2[1], fma), a3 = mac(acc2[2], k256, acc2[3], fma);
      float t = a0 * sc8[0];
      t = t + ((a1 * sc8[1]) * 1.f) / 16.f;
      t = mac(t, a2, sc8[4], fma);
      t = t + ((a3 * sc8[5]) * 1.f) / 16.f;
      float ms = sumy[0] * sc8[2];
      ms = mac(ms, sumy[1], sc8[3], fma);
      ms = mac(ms, sumy[2], sc8[6], fma);
      ms = mac(ms, sumy[3], sc8[7], fma);
      const float d = orc_f16_to_f32(dm[ib * 2]), dmin = orc_f16_to_f32(dm[ib * 2 + 1]);
      const float block = fma ? fmaf(d, t, -(dmin * ms)) : d * t - dmin * ms;
      sumf = sumf + block;
    }
    lanes[lane] = sumf;
  }
  return fold32(lanes, tree);
}

float orc_q6k_row_dot_ref32(const uint8_t* w, const uint8_t* scales, const f16_t* dm, int K, const float* x,
                            int fma, int tree) {
  const int nb = K / 256;
  float lanes[32];
  for (int lane = 0; lane < 32; ++lane) {
    const int tid = lane / 2, ix = lane % 2, ip = tid / 8, il = tid % 8, l0 = 4 * il, is = 8 * ip + l0 / 16;
    const int y_offset = 128 * ip + l0, q_offset_l = 64 * ip + l0, q_offset_h = 32 * ip + l0;
    float sumf = 0.f;
    for (int i = ix; i < nb; i += 2) {
      const uint8_t* q1 = w + i * 192 + q_offset_l;
      const uint8_t* q2 = q1 + 32;
      const uint8_t* qh = w + i * 192 + 128 + q_offset_h;
      const int8_t* sc = (const int8_t*)(scales + i * 16) + is;
      const float* y = x + i * 256 + y_offset;
      float sums[4] = {0, 0, 0, 0};
      for (int l = 0; l < 4; ++l) {
        sums[0] = mac(sums[0], y[l + 0], (float)((int8_t)((q1[l] & 0xF) | ((qh[l] & 0x03) << 4)) - 32), fma);
        sums[1] = mac(sums[1], y[l + 32], (float)((int8_t)((q2[l] & 0xF) | ((qh[l] & 0x0C) << 2)) - 32), fma);
        sums[2] = mac(sums[2], y[l + 64], (float)((int8_t)((q1[l] >> 4) | ((qh[l] & 0x30) << 0)) - 32), fma);
        sums[3] = mac(sums[3], y[l + 96], (float)((int8_t)((q2[l] >> 4) | ((qh[l] & 0xC0) >> 2)) - 32), fma);
      }
      float t = sums[0] * (float)sc[0];
      t = mac(t, sums[1], (float)sc[2], fma);
      t = mac(t, sums[2], (float)sc[4], fma);
      t = mac(t, sums[3], (float)sc[6], fma);
      sumf = mac(sumf, orc_f16_to_f32(dm[i]), t, fma);
    }
    lanes[lane] = sumf;
  }
  return fold32(lanes, tree);
}

float orc_affine4_row_dot_ref32(const uint8_t* w, const bf16_t* scales, const bf16_t* biases, int K, const float* x,
                                int fma, int tree) {
  float lanes[32];
  for (int lane = 0; lane < 32; ++lane) {
    float result = 0.f;
    for (int k = 0; k + 16 * lane < K; k += 512) {
      const int e0 = k + 16 * lane; /* K % 16 == 0: a lane's 16 values are inside the row or not at all */
      const float* xv = x + e0;
      float xt[16], sum = 0.f;
      for (int i = 0; i < 16; i += 4) {
        sum = sum + (((xv[i] + xv[i + 1]) + xv[i + 2]) + xv[i + 3]);
        xt[i] = xv[i];
        xt[i + 1] = xv[i + 1] / 16.0f;
        xt[i + 2] = xv[i + 2] / 256.0f;
        xt[i + 3] = xv[i + 3] / 4096.0f;
      }
      const uint16_t* ws = (const uint16_t*)(w + e0 / 2);
      float accum = 0.f;
      for (int i = 0; i < 4; ++i) {
        float t = xt[4 * i] * (float)(ws[i] & 0x000f);
        t = mac(t, xt[4 * i + 1], (float)(ws[i] & 0x00f0), fma);
        t = mac(t, xt[4 * i + 2], (float)(ws[i] & 0x0f00), fma);
        t = mac(t, xt[4 * i + 3], (float)(ws[i] & 0xf000), fma);
        accum = accum + t;
      }
      const float sc = orc_bf16_to_f32(scales[e0 / 32]), bi = orc_bf16_to_f32(biases[e0 / 32]);
      result = result + (fma ? fmaf(sc, accum, sum * bi) : sc * accum + sum * bi);
    }
    lanes[lane] = result;
  }
  return fold32(lanes, tree);
}

float orc_affine8_row_dot_ref32(const uint8_t* w, const bf16_t* scales, const bf16_t* biases, int K, const float* x,
                                int fma, int tree) {
  float lanes[32];
  for (int lane = 0; lane < 32; ++lane) {
    float result = 0.f;
    for (int k = 0; k + 8 * lane < K; k += 256) {
      const int e0 = k + 8 * lane;
      float sum = 0.f, accum = 0.f;
      for (int i = 0; i < 8; ++i) sum = sum + x[e0 + i];
      for (int i = 0; i < 8; ++i) accum = mac(accum, x[e0 + i], (float)w[e0 + i], fma);
      const float sc = orc_bf16_to_f32(scales[e0 / 64]), bi = orc_bf16_to_f32(biases[e0 / 64]);
      result = result + (fma ? fmaf(sc, accum, sum * bi) : sc * accum + sum * bi);
    }
    lanes[lane] = result;
  }
  return fold32(lanes, tree);
}

/* 0: this build's 64-lane order (the default, what the library implements);
 * 1 + tree + 3 * fma: the reference's 32-lane schedule in one of its six readings (k-quant and
 * affine mat-vecs alike). Process-global; tests that change it put it back. */
int orc_row_order = 0;
ORC_API void orc_set_row_order(int mode) { orc_row_order = mode; }
