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

__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) { return dm_f2bf2(a, b); }

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
// order as rms_wide_kernel<32, NORM_ADD> (64 lane chains of 32 squares, then the 64-lane
// butterfly), so a consumer that recomputes the norm per workgroup sees the bits the
// stand-alone kernel would have written.
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
  __attribute__((aligned(16))) bf16_t xn[T][kPreN];
  float part[T][64];  // the 64 canonical lanes' sums of squares
};

// The global loads of the prologue, kept apart from the arithmetic: loads return in issue
// order, so a kernel that also has cold weight rows to fetch issues these first (they hit in
// cache and come back early) and the weight loads right after, and the norm is worked out
// while the weights are still on their way.
template <int T>
struct PreNormRegs {
  uint4 w, r[T], y[T];
};

__device__ __forceinline__ void unpack_bf16x8(const uint4& w, float (&v)[8]) {
  v[0] = dm_bf2f_lo(w.x);
  v[1] = dm_bf2f_hi(w.x);
  v[2] = dm_bf2f_lo(w.y);
  v[3] = dm_bf2f_hi(w.y);
  v[4] = dm_bf2f_lo(w.z);
  v[5] = dm_bf2f_hi(w.z);
  v[6] = dm_bf2f_lo(w.w);
  v[7] = dm_bf2f_hi(w.w);
}

template <int T>
__device__ __forceinline__ void prenorm_issue(const PreNorm& p, PreNormRegs<T>& g) {
  const int e0 = threadIdx.x * 8;
  g.w = *reinterpret_cast<const uint4*>(p.w + e0);
#pragma unroll
  for (int t = 0; t < T; ++t) {
    g.r[t] = *reinterpret_cast<const uint4*>(p.res + (size_t)t * kPreN + e0);
    g.y[t] = *reinterpret_cast<const uint4*>(p.y + (size_t)t * kPreN + e0);
  }
}

// COH: the normed rows stored by the `write_global` workgroup are read by other workgroups of
// the same launch (handoff.h), so they go out as agent-scope stores.
template <int T, bool COH = false>
__device__ __forceinline__ void prenorm_finish(const PreNorm& p, const PreNormRegs<T>& g, bool write_global,
                                               PreNormLds<T>& s) {
  static_assert(T >= 1 && T <= 4, "rows of the exact window");
  // Thread tid holds values [8 tid, 8 tid + 8): canonical lane l = tid / 4 (32 values, one
  // fma chain in ascending order) is the four threads of a quad. The chain runs down the quad:
  // every thread continues from what its left neighbour handed over, so after four steps the
  // quad's last thread holds the lane's sum with the canonical association.
  const int tid = threadIdx.x, e0 = tid * 8, lane = tid & 63;
  float x[T][8], wv[8];
  unpack_bf16x8(g.w, wv);
#pragma unroll
  for (int t = 0; t < T; ++t) {
    float rv[8], yv[8];
    unpack_bf16x8(g.r[t], rv);
    unpack_bf16x8(g.y[t], yv);
    // h = bf16(res + y), two values a conversion; the packed words are what gets stored
    uint32_t hp[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      hp[j] = dm_f2bf2(rv[2 * j] + yv[2 * j], rv[2 * j + 1] + yv[2 * j + 1]);
      x[t][2 * j] = dm_bf2f_lo(hp[j]);
      x[t][2 * j + 1] = dm_bf2f_hi(hp[j]);
    }
    if (write_global)
      *reinterpret_cast<uint4*>(p.h_out + (size_t)t * kPreN + e0) = make_uint4(hp[0], hp[1], hp[2], hp[3]);
    float acc = 0.f;
#pragma unroll
    for (int step = 0; step < 4; ++step) {
      // quad_perm [0,0,1,2]: each thread reads its left neighbour in the quad
      float in = 0.f;
      if (step > 0)
        in = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, acc), 0x90, 0xF, 0xF, false));
      acc = in;
#pragma unroll
      for (int i = 0; i < 8; ++i) acc = dm_fma(x[t][i], x[t][i], acc);
    }
    if ((tid & 3) == 3) s.part[t][tid >> 2] = acc;
  }
  __syncthreads();
  float invs[T];
#pragma unroll
  for (int t = 0; t < T; ++t)
    invs[t] = dm_rsqrt(dm_wave_sum<64>(s.part[t][lane]) / (float)kPreN + p.eps);
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const float inv = invs[t];
    uint32_t np[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t a = dm_f2bf2(x[t][2 * j] * inv, x[t][2 * j + 1] * inv);
      np[j] = dm_f2bf2(wv[2 * j] * dm_bf2f_lo(a), wv[2 * j + 1] * dm_bf2f_hi(a));
    }
    *reinterpret_cast<uint4*>(&s.xn[t][e0]) = make_uint4(np[0], np[1], np[2], np[3]);
    if (write_global) {
      if constexpr (COH) {
        uint64_t* dst = reinterpret_cast<uint64_t*>(p.normed_out + (size_t)t * kPreN + e0);
        ho_store_u64(dst, (uint64_t)np[0] | ((uint64_t)np[1] << 32));
        ho_store_u64(dst + 1, (uint64_t)np[2] | ((uint64_t)np[3] << 32));
      } else {
        *reinterpret_cast<uint4*>(p.normed_out + (size_t)t * kPreN + e0) = make_uint4(np[0], np[1], np[2], np[3]);
      }
    }
  }
  __syncthreads();
}

template <int T, bool COH = false>
__device__ __forceinline__ void prenorm_rows(const PreNorm& p, bool write_global, PreNormLds<T>& s) {
  PreNormRegs<T> g;
  prenorm_issue<T>(p, g);
  prenorm_finish<T, COH>(p, g, write_global, s);
}
