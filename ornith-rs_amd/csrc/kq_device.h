// Device-side pieces of the k-quant mat-vec shared by the plain, gathered and fused
// MoE kernels: the per-lane activation registers, the row loads and the per-chunk
// accumulation for Q4_K and Q6_K.
//
// Formats: /root/reference/kernels/q4k.metal:43-96, /root/reference/kernels/q6k.metal:47-77.
// A row of K weights is cut into chunks, one per lane:
//   Q4_K  16 code bytes = 32 weights: low nibbles are weights 64g+16h+i, high nibbles
//         the same +32 (g = 64-weight group, h = half, i < 16); one 16-byte load.
//   Q6_K  16 positions of one 128-half: ql[l], ql[l+32], qh[l] -> 64 weights
//         (l, l+32, l+64, l+96); three 16-byte loads.
// chunk j belongs to lane j % 64 and a lane accumulates its chunks in ascending order;
// the per-chunk arithmetic below is the summation order every k-quant kernel of this
// library shares, which is what keeps their results bit-identical to each other.
#pragma once

#include "../../include/ornith_hip.h"
#include "dmath.h"

// 16 consecutive activations -> fp32 registers. COH: the row was written by another
// workgroup of this launch (handoff.h), so it is read with agent-scope loads (bf16 only).
template <bool XF32, bool COH = false>
__device__ __forceinline__ void load_x16(const void* xrow, int off, float (&v)[16]) {
  if constexpr (COH) {
    static_assert(!XF32, "hand-off rows are bf16");
    const uint64_t* p = reinterpret_cast<const uint64_t*>(static_cast<const bf16_t*>(xrow) + off);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint64_t w = __hip_atomic_load(p + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const uint32_t lo = (uint32_t)w, hi = (uint32_t)(w >> 32);
      v[4 * i + 0] = dm_bf2f_lo(lo);
      v[4 * i + 1] = dm_bf2f_hi(lo);
      v[4 * i + 2] = dm_bf2f_lo(hi);
      v[4 * i + 3] = dm_bf2f_hi(hi);
    }
  } else if constexpr (XF32) {
    const float4* p = reinterpret_cast<const float4*>(static_cast<const float*>(xrow) + off);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float4 f = p[i];
      v[4 * i + 0] = f.x;
      v[4 * i + 1] = f.y;
      v[4 * i + 2] = f.z;
      v[4 * i + 3] = f.w;
    }
  } else {
    const uint4* p = reinterpret_cast<const uint4*>(static_cast<const bf16_t*>(xrow) + off);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      uint4 w = p[i];
      v[8 * i + 0] = dm_bf2f_lo(w.x);
      v[8 * i + 1] = dm_bf2f_hi(w.x);
      v[8 * i + 2] = dm_bf2f_lo(w.y);
      v[8 * i + 3] = dm_bf2f_hi(w.y);
      v[8 * i + 4] = dm_bf2f_lo(w.z);
      v[8 * i + 5] = dm_bf2f_hi(w.z);
      v[8 * i + 6] = dm_bf2f_lo(w.w);
      v[8 * i + 7] = dm_bf2f_hi(w.w);
    }
  }
}

__device__ __forceinline__ float kq_ub(uint32_t w, int k) { return (float)((w >> (8 * k)) & 0xffu); }
__device__ __forceinline__ float kq_sb(uint32_t w, int k) {
  return (float)(int)(int8_t)((w >> (8 * k)) & 0xffu);
}

// ---- Q4_K ---------------------------------------------------------------
template <int M>
struct Q4Lane {
  float xl[M][16], xh[M][16], sl[M], sh[M];
  int b, g, h;  // block, 64-group, half

  // which block / group / half chunk `chunk` of a row is (needed by the row loads)
  __device__ __forceinline__ void set_chunk(int chunk) {
    b = chunk >> 3;
    g = (chunk & 7) >> 1;
    h = chunk & 1;
  }

  template <bool XF32, bool COH = false>
  __device__ __forceinline__ void load_x(const void* const (&xrow)[M], int chunk) {
    set_chunk(chunk);
    const int off = 256 * b + 64 * g + 16 * h;
#pragma unroll
    for (int t = 0; t < M; ++t) {
      load_x16<XF32, COH>(xrow[t], off, xl[t]);
      load_x16<XF32, COH>(xrow[t], off + 32, xh[t]);
      float a = 0.f, c = 0.f;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        a = a + xl[t][i];
        c = c + xh[t][i];
      }
      sl[t] = a;
      sh[t] = c;
    }
  }
};

struct Q4Row {
  uint4 q;
  uint32_t s0, s1, s2, dmw;
};

// `row` counts rows of nb blocks from the start of the three tensors
template <int M>
__device__ __forceinline__ Q4Row q4_load(const uint8_t* qs, const uint8_t* scales, const uint16_t* dm,
                                         int64_t row, int nb, const Q4Lane<M>& L) {
  Q4Row r;
  const uint8_t* qrow = qs + row * (int64_t)nb * 128;
  r.q = *reinterpret_cast<const uint4*>(qrow + L.b * 128 + 32 * L.g + 16 * L.h);
  const uint32_t* sc = reinterpret_cast<const uint32_t*>(scales + (row * nb + L.b) * 12);
  r.s0 = sc[0];
  r.s1 = sc[1];
  r.s2 = sc[2];
  r.dmw = *reinterpret_cast<const uint32_t*>(dm + (row * nb + L.b) * 2);
  return r;
}

template <int M>
__device__ __forceinline__ void q4_accumulate(const Q4Row& r, const Q4Lane<M>& L, float (&acc)[M]) {
  const int sh16 = (L.g & 1) * 16;
  const uint32_t a = (r.s0 >> sh16) & 0xffffu, b = (r.s1 >> sh16) & 0xffffu,
                 c = (r.s2 >> sh16) & 0xffffu;
  // both field layouts evaluated, one selected: no branch in the row loop
  const bool low = L.g < 2;
  const uint32_t sc16 = low ? (a & 0x3f3fu) : ((c & 0x0f0fu) | ((a & 0xc0c0u) >> 2));
  const uint32_t m16 = low ? (b & 0x3f3fu) : (((c >> 4) & 0x0f0fu) | ((b & 0xc0c0u) >> 2));
  const float s1 = (float)(sc16 & 0xffu), s2 = (float)(sc16 >> 8);
  const float m1 = (float)(m16 & 0xffu), m2 = (float)(m16 >> 8);
  const float d = dm_h2f((f16_t)(r.dmw & 0xffffu)), dmin = dm_h2f((f16_t)(r.dmw >> 16));

  const uint32_t w[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
  float lo[M], hi[M];
#pragma unroll
  for (int t = 0; t < M; ++t) lo[t] = hi[t] = 0.f;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const uint32_t wl = w[k] & 0x0f0f0f0fu;
    // high nibbles left in place: 16*n. Scaling by a power of two commutes with
    // every rounding below, so 16*sum == sum of 16*terms bit for bit.
    const uint32_t wh = w[k] & 0xf0f0f0f0u;
#define ORN_Q4_STEP(I)                                              \
  {                                                                 \
    const float fl = dm_ubyte<I>(wl), fh = dm_ubyte<I>(wh);         \
    _Pragma("unroll") for (int t = 0; t < M; ++t) {                 \
      lo[t] = dm_fma(L.xl[t][4 * k + I], fl, lo[t]);                \
      hi[t] = dm_fma(L.xh[t][4 * k + I], fh, hi[t]);                \
    }                                                               \
  }
    ORN_Q4_STEP(0)
    ORN_Q4_STEP(1)
    ORN_Q4_STEP(2)
    ORN_Q4_STEP(3)
#undef ORN_Q4_STEP
  }
#pragma unroll
  for (int t = 0; t < M; ++t) {
    float t1 = lo[t] * s1;
    t1 = dm_fma(hi[t] * 0.0625f, s2, t1);
    float t2 = L.sl[t] * m1;
    t2 = dm_fma(L.sh[t], m2, t2);
    float p = d * t1;
    p = dm_fma(-dmin, t2, p);
    acc[t] = acc[t] + p;
  }
}

// ---- Q6_K ---------------------------------------------------------------
template <int M>
struct Q6Lane {
  float x[M][4][16];
  int b, n, u;

  __device__ __forceinline__ void set_chunk(int chunk) {
    b = chunk >> 2;
    n = (chunk & 3) >> 1;
    u = chunk & 1;
  }

  template <bool XF32, bool COH = false>
  __device__ __forceinline__ void load_x(const void* const (&xrow)[M], int chunk) {
    set_chunk(chunk);
    const int off = 256 * b + 128 * n + 16 * u;
#pragma unroll
    for (int t = 0; t < M; ++t)
#pragma unroll
      for (int g = 0; g < 4; ++g) load_x16<XF32, COH>(xrow[t], off + 32 * g, x[t][g]);
  }
};

struct Q6Row {
  uint4 qa, qb, qh;  // ql[l], ql[l+32], qh[l]
  uint2 sc;
  uint16_t d;
};

template <int M>
__device__ __forceinline__ Q6Row q6_load(const uint8_t* qs, const uint8_t* scales, const uint16_t* dm,
                                         int64_t row, int nb, const Q6Lane<M>& L) {
  Q6Row r;
  const uint8_t* blk = qs + (row * nb + L.b) * 192;
  r.qa = *reinterpret_cast<const uint4*>(blk + 64 * L.n + 16 * L.u);
  r.qb = *reinterpret_cast<const uint4*>(blk + 64 * L.n + 32 + 16 * L.u);
  r.qh = *reinterpret_cast<const uint4*>(blk + 128 + 32 * L.n + 16 * L.u);
  r.sc = *reinterpret_cast<const uint2*>(scales + (row * nb + L.b) * 16 + 8 * L.n);
  r.d = dm[row * nb + L.b];
  return r;
}

template <int M>
__device__ __forceinline__ void q6_accumulate(const Q6Row& r, const Q6Lane<M>& L, float (&acc)[M]) {
  const uint32_t A[4] = {r.qa.x, r.qa.y, r.qa.z, r.qa.w};
  const uint32_t B[4] = {r.qb.x, r.qb.y, r.qb.z, r.qb.w};
  const uint32_t H[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
  float s[M][4];
#pragma unroll
  for (int t = 0; t < M; ++t)
#pragma unroll
    for (int g = 0; g < 4; ++g) s[t][g] = 0.f;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    uint32_t c[4];
    c[0] = (A[k] & 0x0f0f0f0fu) | ((H[k] << 4) & 0x30303030u);
    c[1] = (B[k] & 0x0f0f0f0fu) | ((H[k] << 2) & 0x30303030u);
    c[2] = ((A[k] >> 4) & 0x0f0f0f0fu) | (H[k] & 0x30303030u);
    c[3] = ((B[k] >> 4) & 0x0f0f0f0fu) | ((H[k] >> 2) & 0x30303030u);
    // code - 32, exact either as an integer or (as here) as a float subtract
#define ORN_Q6_STEP(I)                                                                        \
  _Pragma("unroll") for (int g = 0; g < 4; ++g) {                                             \
    const float q = dm_ubyte<I>(c[g]) - 32.0f;                                                \
    _Pragma("unroll") for (int t = 0; t < M; ++t) s[t][g] = dm_fma(L.x[t][g][4 * k + I], q, s[t][g]); \
  }
    ORN_Q6_STEP(0)
    ORN_Q6_STEP(1)
    ORN_Q6_STEP(2)
    ORN_Q6_STEP(3)
#undef ORN_Q6_STEP
  }
  // scales: bytes u, u+2, u+4, u+6 of the half's eight
  const uint32_t lo = r.sc.x >> (8 * L.u), hi = r.sc.y >> (8 * L.u);
  const float c0 = kq_sb(lo, 0), c1 = kq_sb(lo, 2), c2 = kq_sb(hi, 0), c3 = kq_sb(hi, 2);
  const float d = dm_h2f(r.d);
#pragma unroll
  for (int t = 0; t < M; ++t) {
    float v = s[t][0] * c0;
    v = dm_fma(s[t][1], c1, v);
    v = dm_fma(s[t][2], c2, v);
    v = dm_fma(s[t][3], c3, v);
    acc[t] = acc[t] + d * v;
  }
}

// format-generic front: lane registers, row load, accumulate
template <int KIND, int M>
struct KqLane;
template <int M>
struct KqLane<ORNITH_Q4K, M> {
  using Lane = Q4Lane<M>;
  using Row = Q4Row;
  static __device__ __forceinline__ Row load(const uint8_t* qs, const uint8_t* sc, const uint16_t* dm,
                                             int64_t row, int nb, const Lane& L) {
    return q4_load(qs, sc, dm, row, nb, L);
  }
  static __device__ __forceinline__ void accumulate(const Row& r, const Lane& L, float (&acc)[M]) {
    q4_accumulate(r, L, acc);
  }
  static constexpr int kChunksPerBlock = 8;
};
template <int M>
struct KqLane<ORNITH_Q6K, M> {
  using Lane = Q6Lane<M>;
  using Row = Q6Row;
  static __device__ __forceinline__ Row load(const uint8_t* qs, const uint8_t* sc, const uint16_t* dm,
                                             int64_t row, int nb, const Lane& L) {
    return q6_load(qs, sc, dm, row, nb, L);
  }
  static __device__ __forceinline__ void accumulate(const Row& r, const Lane& L, float (&acc)[M]) {
    q6_accumulate(r, L, acc);
  }
  static constexpr int kChunksPerBlock = 4;
};
