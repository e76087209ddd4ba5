// Device-side scalar arithmetic with fully specified results.
//
// Router indices, argmax tokens and accepted-token counts have to come out the
// same on every run and agree with a scalar CPU evaluation, so nothing here
// calls the device math library: exp/log are written out with fp32 add, mul and
// fma only, divide and sqrt are the correctly rounded IEEE ones (hipcc's
// default), and conversions are integer bit moves. The file is compiled with
// -ffp-contract=off, so the only fused operations are the explicit __builtin_fmaf.
//
// Rounding points follow the reference: activations are bf16 in memory and fp32
// in registers (/root/reference/kernels/q4k.metal:216-221), bf16 rounding is
// round-to-nearest-even (/root/reference/src/array.rs:229-237).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint16_t bf16_t;  // raw bits
typedef uint16_t f16_t;   // raw bits

#define DM_INF (__builtin_inff())

__device__ __forceinline__ float dm_fma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }

__device__ __forceinline__ float dm_bf2f(bf16_t b) { return __uint_as_float((uint32_t)b << 16); }

__device__ __forceinline__ bf16_t dm_f2bf(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (bf16_t)(u >> 16);
}
// round to bf16 precision, keep as float
__device__ __forceinline__ float dm_rb(float f) { return dm_bf2f(dm_f2bf(f)); }

// low / high bf16 of a packed pair (little endian: element 0 in the low half)
__device__ __forceinline__ float dm_bf2f_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float dm_bf2f_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// IEEE half -> float, exact. v_cvt_f32_f16 is exact for every input (subnormals
// included: gfx9 keeps fp16 denormals), so the hardware conversion is used.
__device__ __forceinline__ float dm_h2f(f16_t h) {
  _Float16 v;
  __builtin_memcpy(&v, &h, 2);
  return (float)v;
}

// exp(x): reduce by ln2 in two pieces, degree-5 polynomial, exponent from bits.
// x < -87 gives +0 and x > 88 gives +inf, so subnormal results never occur.
__device__ __forceinline__ float dm_exp(float x) {
  if (x != x) return x;
  if (x > 88.0f) return DM_INF;
  if (x < -87.0f) return 0.0f;
  float n = __builtin_rintf(x * 1.44269504088896341f);
  float r = dm_fma(n, -0.693359375f, x);
  r = dm_fma(n, 2.12194440e-4f, r);
  float p = 1.9875691500e-4f;
  p = dm_fma(p, r, 1.3981999507e-3f);
  p = dm_fma(p, r, 8.3334519073e-3f);
  p = dm_fma(p, r, 4.1665795894e-2f);
  p = dm_fma(p, r, 1.6666665459e-1f);
  p = dm_fma(p, r, 5.0000001201e-1f);
  float r2 = r * r;
  float e = dm_fma(p, r2, r) + 1.0f;
  int ni = (int)n;
  return e * __uint_as_float((uint32_t)(ni + 127) << 23);
}

// log(x), x finite normal > 0.
__device__ __forceinline__ float dm_log(float x) {
  if (x != x || x < 0.0f) return __builtin_nanf("");
  if (x == 0.0f) return -DM_INF;
  if (x == DM_INF) return DM_INF;
  uint32_t u = __float_as_uint(x);
  int e = (int)(u >> 23) - 126;
  float m = __uint_as_float((u & 0x007fffffu) | 0x3f000000u);
  if (m < 0.707106781186547524f) {
    e -= 1;
    m = m + m;
  }
  float f = m - 1.0f;
  float z = f * f;
  float p = 7.0376836292e-2f;
  p = dm_fma(p, f, -1.1514610310e-1f);
  p = dm_fma(p, f, 1.1676998740e-1f);
  p = dm_fma(p, f, -1.2420140846e-1f);
  p = dm_fma(p, f, 1.4249322787e-1f);
  p = dm_fma(p, f, -1.6668057665e-1f);
  p = dm_fma(p, f, 2.0000714765e-1f);
  p = dm_fma(p, f, -2.4999993993e-1f);
  p = dm_fma(p, f, 3.3333331174e-1f);
  float y = f * z * p;
  float fe = (float)e;
  y = dm_fma(fe, -2.12194440e-4f, y);
  y = dm_fma(-0.5f, z, y);
  float r = f + y;
  r = dm_fma(fe, 0.693359375f, r);
  return r;
}

__device__ __forceinline__ float dm_log1p(float u) {
  float w = 1.0f + u;
  if (w == 1.0f) return u;
  if (w == DM_INF) return DM_INF;
  return dm_log(w) * (u / (w - 1.0f));
}

__device__ __forceinline__ float dm_rsqrt(float x) { return 1.0f / __builtin_sqrtf(x); }

// sigmoid with every intermediate held in bf16
// (/root/reference/kernels/ornith_sigmoid.h:27-31 at T = bfloat16).
__device__ __forceinline__ float dm_sigmoid_bf16(float x) {
  float e = dm_rb(dm_exp(__builtin_fabsf(x)));
  float s = dm_rb(1.0f + e);
  float y = dm_rb(1.0f / s);
  return (x < 0.0f) ? y : dm_rb(1.0f - y);
}
__device__ __forceinline__ float dm_sigmoid_f32(float x) {
  float y = 1.0f / (1.0f + dm_exp(__builtin_fabsf(x)));
  return (x < 0.0f) ? y : 1.0f - y;
}

// ---- wavefront reductions: v[l] += v[l ^ s], s = 32,16,...,1 ---------------
// fp32 add commutes, so all 64 lanes finish with identical bits.
template <int WIDTH>
__device__ __forceinline__ float dm_wave_sum(float v) {
#pragma unroll
  for (int s = WIDTH / 2; s >= 1; s >>= 1) v = v + __shfl_xor(v, s, 64);
  return v;
}
template <int WIDTH>
__device__ __forceinline__ float dm_wave_max(float v) {
#pragma unroll
  for (int s = WIDTH / 2; s >= 1; s >>= 1) {
    float o = __shfl_xor(v, s, 64);
    v = o > v ? o : v;
  }
  return v;
}
