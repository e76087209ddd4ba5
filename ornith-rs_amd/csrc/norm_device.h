// One row of an RMS norm by one wavefront, shared by the norm kernels and by kernels
// that apply a norm to their own input.
//
// Arithmetic of vendored rms_norm.metal:12-81 and
// /root/reference/kernels/ornith_norm.metal:28-183: lane l owns the contiguous piece
// [l*PER, (l+1)*PER) of the row, one fma chain of squares per lane, butterfly over the
// 64 lanes, inv = 1/sqrt(sum/n + eps), out = bf16(w * bf16(x * inv)).
#pragma once

#include "dmath.h"
#include "handoff.h"

// PER consecutive bf16 values <-> fp32 registers, widest aligned access
template <int PER>
__device__ __forceinline__ void load_bf16(const bf16_t* p, float (&v)[PER]) {
  if constexpr (PER >= 8) {
#pragma unroll
    for (int c = 0; c < PER / 8; ++c) {
      const uint4 w = reinterpret_cast<const uint4*>(p)[c];
      v[8 * c + 0] = dm_bf2f_lo(w.x);
      v[8 * c + 1] = dm_bf2f_hi(w.x);
      v[8 * c + 2] = dm_bf2f_lo(w.y);
      v[8 * c + 3] = dm_bf2f_hi(w.y);
      v[8 * c + 4] = dm_bf2f_lo(w.z);
      v[8 * c + 5] = dm_bf2f_hi(w.z);
      v[8 * c + 6] = dm_bf2f_lo(w.w);
      v[8 * c + 7] = dm_bf2f_hi(w.w);
    }
  } else if constexpr (PER == 4) {
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    v[0] = dm_bf2f_lo(w.x);
    v[1] = dm_bf2f_hi(w.x);
    v[2] = dm_bf2f_lo(w.y);
    v[3] = dm_bf2f_hi(w.y);
  } else if constexpr (PER == 2) {
    const uint32_t w = *reinterpret_cast<const uint32_t*>(p);
    v[0] = dm_bf2f_lo(w);
    v[1] = dm_bf2f_hi(w);
  } else {
    v[0] = dm_bf2f(p[0]);
  }
}

__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  return (uint32_t)dm_f2bf(a) | ((uint32_t)dm_f2bf(b) << 16);
}

// rounds each value to bf16 and stores
template <int PER>
__device__ __forceinline__ void store_bf16(bf16_t* p, const float (&v)[PER]) {
  if constexpr (PER >= 8) {
#pragma unroll
    for (int c = 0; c < PER / 8; ++c)
      reinterpret_cast<uint4*>(p)[c] =
          make_uint4(pack_bf16x2(v[8 * c], v[8 * c + 1]), pack_bf16x2(v[8 * c + 2], v[8 * c + 3]),
                     pack_bf16x2(v[8 * c + 4], v[8 * c + 5]), pack_bf16x2(v[8 * c + 6], v[8 * c + 7]));
  } else if constexpr (PER == 4) {
    *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
  } else if constexpr (PER == 2) {
    *reinterpret_cast<uint32_t*>(p) = pack_bf16x2(v[0], v[1]);
  } else {
    p[0] = dm_f2bf(v[0]);
  }
}

enum { NORM_PLAIN = 0, NORM_ADD = 1, NORM_GATED = 2 };

// One row. a (and b for NORM_ADD, z for NORM_GATED) point at the row; w at the weights
// (may be null for NORM_PLAIN); h_out receives bf16(a + b) for NORM_ADD.
template <int PER, int MODE>
__device__ __forceinline__ void rms_row(const bf16_t* a, const bf16_t* b, const bf16_t* w,
                                        const bf16_t* z, bf16_t* h_out, bf16_t* out, int n,
                                        float eps, int lane) {
  const int base = lane * PER;
  float x[PER], wv[PER];
  load_bf16<PER>(a + base, x);
  if (w) load_bf16<PER>(w + base, wv);
  if constexpr (MODE == NORM_ADD) {
    float y[PER];
    load_bf16<PER>(b + base, y);
#pragma unroll
    for (int i = 0; i < PER; ++i) x[i] = dm_rb(x[i] + y[i]);
    store_bf16<PER>(h_out + base, x);
  }
  float acc = 0.f;
#pragma unroll
  for (int i = 0; i < PER; ++i) acc = dm_fma(x[i], x[i], acc);
  const float inv = dm_rsqrt(dm_wave_sum<64>(acc) / (float)n + eps);
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    x[i] = dm_rb(x[i] * inv);
    if (w) x[i] = dm_rb(wv[i] * x[i]);
  }
  if constexpr (MODE == NORM_GATED) {
    float g[PER];
    load_bf16<PER>(z + base, g);
#pragma unroll
    for (int i = 0; i < PER; ++i) x[i] = (g[i] * dm_sigmoid_f32(g[i])) * x[i];
  }
  store_bf16<PER>(out + base, x);
}

// Residual add + RMS norm of T <= 4 rows of 2048 values by one 256-thread workgroup, for
// kernels that consume the normed rows themselves: h = bf16(res + y),
// normed = bf16(w * bf16(h * inv)). The rows land in LDS (xn); the workgroup for which
// `write_global` holds also stores h and normed for later consumers. Same arithmetic and
// order as rms_wide_kernel<32, NORM_ADD> (wavefront t sums row t), so a consumer that
// recomputes the norm per workgroup sees the bits the stand-alone kernel would have written.
struct PreNorm {
  const bf16_t* res;     // [T, 2048]
  const bf16_t* y;       // [T, 2048]
  const bf16_t* w;       // [2048]
  bf16_t* h_out;         // [T, 2048]
  bf16_t* normed_out;    // [T, 2048]
  float eps;
};

constexpr int kPreN = 2048;

template <int T>
struct PreNormLds {
  float xs[T * kPreN];
  __attribute__((aligned(16))) bf16_t xn[T][kPreN];
  float inv[4];
};

// COH: the normed rows stored by the `write_global` workgroup are read by other workgroups of
// the same launch (handoff.h), so they go out as agent-scope stores.
template <int T, bool COH = false>
__device__ __forceinline__ void prenorm_rows(const PreNorm& p, bool write_global, PreNormLds<T>& s) {
  static_assert(T >= 1 && T <= 4, "one wavefront per row");
  constexpr int PER = kPreN / 64;
  const int tid = threadIdx.x, e0 = tid * 8, lane = tid & 63, wave = tid >> 6;
  const int lane_of = e0 / PER, pos0 = e0 % PER;
  float x[T][8], wv[8];
  load_bf16<8>(p.w + e0, wv);
#pragma unroll
  for (int t = 0; t < T; ++t) {
    float yv[8];
    load_bf16<8>(p.res + (size_t)t * kPreN + e0, x[t]);
    load_bf16<8>(p.y + (size_t)t * kPreN + e0, yv);
#pragma unroll
    for (int i = 0; i < 8; ++i) x[t][i] = dm_rb(x[t][i] + yv[i]);
    if (write_global) store_bf16<8>(p.h_out + (size_t)t * kPreN + e0, x[t]);
#pragma unroll
    for (int i = 0; i < 8; ++i) s.xs[t * kPreN + (pos0 + i) * 64 + lane_of] = x[t][i];
  }
  __syncthreads();
  if (wave < T) {
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const float v = s.xs[wave * kPreN + i * 64 + lane];
      acc = dm_fma(v, v, acc);
    }
    const float inv = dm_rsqrt(dm_wave_sum<64>(acc) / (float)kPreN + p.eps);
    if (lane == 0) s.inv[wave] = inv;
  }
  __syncthreads();
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const float inv = s.inv[t];
#pragma unroll
    for (int i = 0; i < 8; ++i) x[t][i] = dm_rb(wv[i] * dm_rb(x[t][i] * inv));
    store_bf16<8>(&s.xn[t][e0], x[t]);
    if (write_global) {
      if constexpr (COH) {
        uint64_t* dst = reinterpret_cast<uint64_t*>(p.normed_out + (size_t)t * kPreN + e0);
        ho_store_u64(dst, (uint64_t)pack_bf16x2(x[t][0], x[t][1]) | ((uint64_t)pack_bf16x2(x[t][2], x[t][3]) << 32));
        ho_store_u64(dst + 1, (uint64_t)pack_bf16x2(x[t][4], x[t][5]) | ((uint64_t)pack_bf16x2(x[t][6], x[t][7]) << 32));
      } else {
        store_bf16<8>(p.normed_out + (size_t)t * kPreN + e0, x[t]);
      }
    }
  }
  __syncthreads();
}
