// Device-side scalar arithmetic with fully specified results.
//
// Router indices, argmax tokens and accepted-token counts have to come out the
// same on every run and agree with a scalar CPU evaluation, so nothing here
// calls the device math library: exp/log are written out with fp32 add, mul and
// fma only, divide and sqrt are the correctly rounded IEEE ones (hipcc's
// default), and conversions are integer bit moves or the hardware's exact / round-to-
// nearest-even ones. The file is compiled with -ffp-contract=off, so the only fused
// operations are the explicit __builtin_fmaf.
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

// A pointer rebuilt from an integer that is known to address device memory. Going through the
// global address space lets the compiler use global loads (counted by vmcnt alone, so a kernel
// can wait for its loads one by one) where a bare integer-to-pointer cast gives flat loads.
template <class T>
__device__ __forceinline__ T* dm_global_ptr(uint64_t bits) {
  return (T*)(__attribute__((address_space(1))) T*)bits;
}

__device__ __forceinline__ float dm_fma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }

__device__ __forceinline__ float dm_bf2f(bf16_t b) { return __uint_as_float((uint32_t)b << 16); }

// fp32 -> bf16, round to nearest even: gfx950's v_cvt_pk_bf16_f32 (one instruction for
// two values; subnormals are kept, fp32 denormals being on). Equal to the integer
// formulation u += 0x7fff + ((u >> 16) & 1) for every non-NaN input.
__device__ __forceinline__ bf16_t dm_f2bf(float f) {
  const __bf16 b = (__bf16)f;
  return __builtin_bit_cast(bf16_t, b);
}
// two values in one instruction, element 0 in the low half; each half equals dm_f2bf of its value
__device__ __forceinline__ uint32_t dm_f2bf2(float lo, float hi) {
  typedef float f2v __attribute__((ext_vector_type(2)));
  typedef __bf16 b2v __attribute__((ext_vector_type(2)));
  const f2v v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, b2v));
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
  // no branches: the polynomial is worked out for every input and the special cases are
  // selected afterwards (outside [-87, 88] its value is never used; a NaN stays that NaN)
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
  // n as an integer: n is integral and, where the result is used, within [-126, 127]
  const int ni = (int)__builtin_fminf(__builtin_fmaxf(n, -200.0f), 200.0f);
  float v = e * __uint_as_float((uint32_t)(ni + 127) << 23);
  v = x < -87.0f ? 0.0f : v;
  v = x > 88.0f ? DM_INF : v;
  return x != x ? x : v;
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

// Everything here stays in the vector ALU: a trip through the LDS crossbar (ds_swizzle,
// ds_bpermute) costs an LDS round trip each, and a 64-lane sum would take four of them in series.

// The halves of a wavefront (ROWS = 32) or the 16-lane rows of each half (ROWS = 16) trade
// places: given v in both operands, on return a holds the even rows' values in every row pair
// and b the odd rows' (v_permlane32_swap / v_permlane16_swap exchange the odd rows of the
// first operand with the even rows of the second).
template <int ROWS>
__device__ __forceinline__ void dm_row_swap(float v, float& a, float& b) {
  a = v;
  b = v;
  if constexpr (ROWS == 32)
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  else
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}

// value of lane (l ^ S): DPP quad permutes for 1 and 2 and a row rotate for 8 (they fold
// into the consuming add), two bank-masked row shifts for 4, a row swap and a select for 16, 32.
template <int S>
__device__ __forceinline__ float dm_xor_lane(float v) {
  int i = __builtin_bit_cast(int, v);
  if constexpr (S == 1)
    i = __builtin_amdgcn_mov_dpp(i, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
  else if constexpr (S == 2)
    i = __builtin_amdgcn_mov_dpp(i, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
  else if constexpr (S == 4) {
    const int up = __builtin_amdgcn_update_dpp(i, i, 0x104, 0xF, 0x5, false);  // row_shl:4 into lanes 0-3, 8-11
    i = __builtin_amdgcn_update_dpp(up, i, 0x114, 0xF, 0xA, false);            // row_shr:4 into lanes 4-7, 12-15
  } else if constexpr (S == 8)
    i = __builtin_amdgcn_update_dpp(0, i, 0x128, 0xF, 0xF, false);  // row_ror:8 (every lane has a source)
  else {
    float a, b;
    dm_row_swap<S>(v, a, b);
    return (__lane_id() & S) ? a : b;
  }
  return __builtin_bit_cast(float, i);
}

template <int WIDTH>
__device__ __forceinline__ float dm_wave_sum(float v) {
  // a + b after a row swap is v[l] + v[l ^ ROWS] with the operands in one order for both
  // partners, which is the same bits
  if constexpr (WIDTH >= 64) { float a, b; dm_row_swap<32>(v, a, b); v = a + b; }
  if constexpr (WIDTH >= 32) { float a, b; dm_row_swap<16>(v, a, b); v = a + b; }
  if constexpr (WIDTH >= 16) {
    v = v + dm_xor_lane<8>(v);
    // v now repeats every 8 lanes, so the lane 4 further round the row holds the bits of lane
    // l ^ 4: one rotate that folds into the add
    v = v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xF, 0xF, false));
  } else if constexpr (WIDTH >= 8) {
    v = v + dm_xor_lane<4>(v);
  }
  if constexpr (WIDTH >= 4) v = v + dm_xor_lane<2>(v);
  if constexpr (WIDTH >= 2) v = v + dm_xor_lane<1>(v);
  return v;
}
template <int WIDTH>
__device__ __forceinline__ float dm_wave_max(float v) {
  float o;
  if constexpr (WIDTH >= 64) { float a, b; dm_row_swap<32>(v, a, b); v = b > a ? b : a; }
  if constexpr (WIDTH >= 32) { float a, b; dm_row_swap<16>(v, a, b); v = b > a ? b : a; }
  if constexpr (WIDTH >= 16) { o = dm_xor_lane<8>(v); v = o > v ? o : v; }
  if constexpr (WIDTH >= 8) { o = dm_xor_lane<4>(v); v = o > v ? o : v; }
  if constexpr (WIDTH >= 4) { o = dm_xor_lane<2>(v); v = o > v ? o : v; }
  if constexpr (WIDTH >= 2) { o = dm_xor_lane<1>(v); v = o > v ? o : v; }
  return v;
}

// Four 64-lane butterfly sums for the price of one and a bit: at the 32 and 16 steps
// each lane sends the value its partner is going to keep, so two sums share a permute.
// Every addition pairs the same two operands as the plain butterfly, so the bits are
// those of dm_wave_sum<64>. On return lanes [0,16) hold sum(a), [16,32) sum(c),
// [32,48) sum(b), [48,64) sum(d).
__device__ __forceinline__ float dm_wave_sum4(float a, float b, float c, float d, int lane) {
  const bool h32 = lane & 32, h16 = lane & 16;
  const float r1 = (h32 ? b : a) + dm_xor_lane<32>(h32 ? a : b);
  const float r2 = (h32 ? d : c) + dm_xor_lane<32>(h32 ? c : d);
  float r = (h16 ? r2 : r1) + dm_xor_lane<16>(h16 ? r1 : r2);
  r = r + dm_xor_lane<8>(r);
  r = r + dm_xor_lane<4>(r);
  r = r + dm_xor_lane<2>(r);
  r = r + dm_xor_lane<1>(r);
  return r;
}
__device__ __forceinline__ float dm_lane_value(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// byte k of a dword as a float, one instruction (the compiler's own pattern match gives
// a bit-field extract plus a convert once the operand carries a nibble mask)
__device__ __forceinline__ float dm_ubyte0(uint32_t w) { float r; asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(r) : "v"(w)); return r; }
__device__ __forceinline__ float dm_ubyte1(uint32_t w) { float r; asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(r) : "v"(w)); return r; }
__device__ __forceinline__ float dm_ubyte2(uint32_t w) { float r; asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(r) : "v"(w)); return r; }
__device__ __forceinline__ float dm_ubyte3(uint32_t w) { float r; asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(r) : "v"(w)); return r; }
template <int K>
__device__ __forceinline__ float dm_ubyte(uint32_t w) {
  if constexpr (K == 0) return dm_ubyte0(w);
  else if constexpr (K == 1) return dm_ubyte1(w);
  else if constexpr (K == 2) return dm_ubyte2(w);
  else return dm_ubyte3(w);
}
