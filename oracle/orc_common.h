/*
 * CPU oracle for the ornith speculative-decode hot path -- TEST INFRASTRUCTURE.
 *
 * Nothing in the shipped library may include, link or call this directory. It
 * exists so the tests, the smoke check and the benchmark's cpu_baseline leg have
 * an independent, scalar restatement of every result the HIP path produces.
 *
 * This header: scalar types, bf16/f16 conversion, the deterministic
 * transcendental functions and the canonical 64-lane reduction tree.
 *
 * Why "deterministic" functions: router indices, argmax tokens and accepted
 * counts must be bit-identical between this CPU code and the GPU. libm and the
 * GPU's math library do not agree in the last bit, so every transcendental the
 * path needs is written out here with nothing but IEEE fp32 add/mul/fma,
 * correctly rounded divide/sqrt and integer bit moves; the GPU side carries its
 * own copy of the same formulae. Accuracy of each is pinned against libm's
 * double routines in tests/test_oracle_math.py (<= 2 ulp).
 *
 * Rounding points follow the reference (activations are bf16 in memory, fp32 in
 * registers, /root/reference/kernels/q4k.metal:216-221; bf16 RNE as in
 * /root/reference/src/array.rs:229-237).
 */
#ifndef ORC_COMMON_H
#define ORC_COMMON_H

#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_API __attribute__((visibility("default")))

typedef uint16_t bf16_t; /* raw bits */
typedef uint16_t f16_t;  /* raw bits */

enum { ORC_F32 = 0, ORC_BF16 = 1 };
enum { ORC_Q4K = 0, ORC_Q6K = 1,
       /* stacked experts in the 4-bit affine group-32 format riding in an orc_kmat: qs = packed
        * codes u8[E,O,K/2], scales = bf16 scales [E,O,K/32], dm = bf16 biases [E,O,K/32] */
       ORC_AFFINE4_G32 = 2 };

static inline uint32_t orc_f2u(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
static inline float orc_u2f(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* bf16 round-to-nearest-even; NaN -> quiet NaN (src/array.rs:229-237). */
static inline bf16_t orc_f32_to_bf16(float f) {
  uint32_t u = orc_f2u(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x0040u);
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  return (bf16_t)(u >> 16);
}
static inline float orc_bf16_to_f32(bf16_t b) { return orc_u2f((uint32_t)b << 16); }
/* Round an fp32 value to bf16 precision and back ("->T" in the reference). */
static inline float orc_rb(float f) { return orc_bf16_to_f32(orc_f32_to_bf16(f)); }

/* IEEE half -> float, exact, including subnormals. */
static inline float orc_f16_to_f32(f16_t h) {
  uint32_t s = (uint32_t)(h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1fu;
  uint32_t m = h & 0x3ffu;
  if (e == 0) {
    if (m == 0) return orc_u2f(s);
    /* subnormal: value = m * 2^-24, exact in fp32 */
    float v = (float)m * 5.9604644775390625e-08f;
    return s ? -v : v;
  }
  if (e == 31) return orc_u2f(s | 0x7f800000u | (m << 13));
  return orc_u2f(s | ((e + 112u) << 23) | (m << 13));
}
/* float -> IEEE half, RNE (only used to build synthetic weights). */
static inline f16_t orc_f32_to_f16(float f) {
  uint32_t u = orc_f2u(f);
  uint32_t s = (u >> 16) & 0x8000u;
  uint32_t a = u & 0x7fffffffu;
  if (a >= 0x7f800000u) return (f16_t)(s | 0x7c00u | (a > 0x7f800000u ? 0x200u : 0));
  if (a >= 0x477ff000u) return (f16_t)(s | 0x7c00u); /* overflow after rounding */
  if (a < 0x33000001u) return (f16_t)s;             /* rounds to zero */
  int e = (int)(a >> 23) - 127;
  uint32_t m = (a & 0x7fffffu) | 0x800000u;
  int shift = (e < -14) ? (13 + (-14 - e)) : 13;
  uint32_t half = 1u << (shift - 1);
  uint32_t r = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  if (rem > half || (rem == half && (r & 1u))) r++;
  if (e < -14) return (f16_t)(s | r); /* subnormal (r may carry into exponent, still right) */
  /* r holds 1.mmmmmmmmmm (11 bits) possibly carried to 12 bits */
  uint32_t out = ((uint32_t)(e + 15) << 10) + (r - 0x400u);
  return (f16_t)(s | out);
}

/* ---- deterministic transcendentals ------------------------------------- */

/* exp(x): Cody-Waite reduction by ln2 (two constants), degree-5 minimax in the
 * reduced argument evaluated with fma, scaled by an exponent built from bits.
 * Inputs below -87 return +0 and above 88 return +inf so the result never
 * depends on subnormal handling. */
static inline float orc_expf(float x) {
  if (x != x) return x;
  if (x > 88.0f) return INFINITY;
  if (x < -87.0f) return 0.0f;
  float n = rintf(x * 1.44269504088896341f);
  float r = fmaf(n, -0.693359375f, x);
  r = fmaf(n, 2.12194440e-4f, r);
  float p = 1.9875691500e-4f;
  p = fmaf(p, r, 1.3981999507e-3f);
  p = fmaf(p, r, 8.3334519073e-3f);
  p = fmaf(p, r, 4.1665795894e-2f);
  p = fmaf(p, r, 1.6666665459e-1f);
  p = fmaf(p, r, 5.0000001201e-1f);
  float r2 = r * r;
  float e = fmaf(p, r2, r) + 1.0f;
  int ni = (int)n;
  return e * orc_u2f((uint32_t)(ni + 127) << 23);
}

/* log(x) for finite x > 0 (normal numbers): mantissa in [sqrt(1/2), sqrt(2)),
 * degree-8 polynomial in f = m - 1, exponent added back in two pieces. */
static inline float orc_logf(float x) {
  if (x != x || x < 0.0f) return NAN;
  if (x == 0.0f) return -INFINITY;
  if (x == INFINITY) return INFINITY;
  uint32_t u = orc_f2u(x);
  int e = (int)(u >> 23) - 126;
  float m = orc_u2f((u & 0x007fffffu) | 0x3f000000u); /* [0.5, 1) */
  if (m < 0.707106781186547524f) {
    e -= 1;
    m = m + m;
  }
  float f = m - 1.0f;
  float z = f * f;
  float p = 7.0376836292e-2f;
  p = fmaf(p, f, -1.1514610310e-1f);
  p = fmaf(p, f, 1.1676998740e-1f);
  p = fmaf(p, f, -1.2420140846e-1f);
  p = fmaf(p, f, 1.4249322787e-1f);
  p = fmaf(p, f, -1.6668057665e-1f);
  p = fmaf(p, f, 2.0000714765e-1f);
  p = fmaf(p, f, -2.4999993993e-1f);
  p = fmaf(p, f, 3.3333331174e-1f);
  float y = f * z * p;
  float fe = (float)e;
  y = fmaf(fe, -2.12194440e-4f, y);
  y = fmaf(-0.5f, z, y);
  float r = f + y;
  r = fmaf(fe, 0.693359375f, r);
  return r;
}

/* log1p(u) for u >= 0: log(w) * u / (w - 1) with w = fl(1 + u) recovers the
 * bits lost when 1 + u rounds. */
static inline float orc_log1pf(float u) {
  float w = 1.0f + u;
  if (w == 1.0f) return u;
  if (w == INFINITY) return INFINITY;
  return orc_logf(w) * (u / (w - 1.0f));
}

static inline float orc_rsqrtf(float x) { return 1.0f / sqrtf(x); }

/* sigmoid with every intermediate held in bf16
 * (/root/reference/kernels/ornith_sigmoid.h:27-31, T = bfloat16). */
static inline float orc_sigmoid_bf16(float x_bf16) {
  float e = orc_rb(orc_expf(fabsf(x_bf16)));
  float s = orc_rb(1.0f + e);
  float y = orc_rb(1.0f / s);
  return (x_bf16 < 0.0f) ? y : orc_rb(1.0f - y);
}
/* the same operator evaluated in fp32 (ornith_sigmoid.h, T = float). */
static inline float orc_sigmoid_f32(float x) {
  float y = 1.0f / (1.0f + orc_expf(fabsf(x)));
  return (x < 0.0f) ? y : 1.0f - y;
}

/* ---- the canonical wave reduction -------------------------------------- */

/* Butterfly over 64 lanes: v[l] += v[l ^ s] for s = 32,16,8,4,2,1. fp32 add is
 * commutative, so every lane ends with the same bits; lane 0 is returned. */
static inline float orc_tree64(const float* lanes) {
  float v[64], w[64];
  memcpy(v, lanes, sizeof v);
  for (int s = 32; s >= 1; s >>= 1) {
    for (int l = 0; l < 64; ++l) w[l] = v[l] + v[l ^ s];
    memcpy(v, w, sizeof v);
  }
  return v[0];
}
static inline float orc_treemax64(const float* lanes) {
  float m = lanes[0];
  for (int l = 1; l < 64; ++l) m = lanes[l] > m ? lanes[l] : m;
  return m;
}

#ifdef __cplusplus
}
#endif
#endif
