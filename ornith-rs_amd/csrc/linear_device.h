// One row of the dense bf16 mat-vec by one wavefront: groups of 8 weights, group j on lane
// j mod 64, one fma chain per lane in group order, butterfly over the 64 lanes. Shared by the
// dense kernels of linear.hip and by kernels that fold a small projection into their head
// (ops::matmul::gemv, /root/reference/src/ops/matmul.rs:334-438, fp32 accumulate).
#pragma once

#include "dmath.h"

// a group's eight products onto the lane's chain
__device__ __forceinline__ float dense_group_chain(const uint4& wv, const uint4& xv, float a) {
  a = dm_fma(dm_bf2f_lo(wv.x), dm_bf2f_lo(xv.x), a);
  a = dm_fma(dm_bf2f_hi(wv.x), dm_bf2f_hi(xv.x), a);
  a = dm_fma(dm_bf2f_lo(wv.y), dm_bf2f_lo(xv.y), a);
  a = dm_fma(dm_bf2f_hi(wv.y), dm_bf2f_hi(xv.y), a);
  a = dm_fma(dm_bf2f_lo(wv.z), dm_bf2f_lo(xv.z), a);
  a = dm_fma(dm_bf2f_hi(wv.z), dm_bf2f_hi(xv.z), a);
  a = dm_fma(dm_bf2f_lo(wv.w), dm_bf2f_lo(xv.w), a);
  a = dm_fma(dm_bf2f_hi(wv.w), dm_bf2f_hi(xv.w), a);
  return a;
}

// NR rows over the same activations. A lane asks for NU groups of every row (and of the
// activations) before it uses the first: written as a plain loop over a row's groups every
// group was its own trip to memory, eight in a row for K = 4096, and the rows of a call came
// one after the other. The chains and the butterflies are those of that loop.
template <int NR, int NU>
__device__ __forceinline__ void dense_rows_dot(const bf16_t* const (&wr)[NR], const bf16_t* xr, int K, int lane,
                                               float (&out)[NR]) {
  float a[NR];
#pragma unroll
  for (int r = 0; r < NR; ++r) a[r] = 0.f;
  const int n = K / 8;
  for (int j0 = lane; j0 < n; j0 += 64 * NU) {
    uint4 wv[NR][NU], xv[NU];
#pragma unroll
    for (int u = 0; u < NU; ++u) {
      const int j = j0 + 64 * u;
      if (j < n) {
        xv[u] = *reinterpret_cast<const uint4*>(xr + 8 * j);
#pragma unroll
        for (int r = 0; r < NR; ++r) wv[r][u] = *reinterpret_cast<const uint4*>(wr[r] + 8 * j);
      }
    }
#pragma unroll
    for (int r = 0; r < NR; ++r)
#pragma unroll
      for (int u = 0; u < NU; ++u)
        if (j0 + 64 * u < n) a[r] = dense_group_chain(wv[r][u], xv[u], a[r]);
  }
#pragma unroll
  for (int r = 0; r < NR; ++r) out[r] = dm_wave_sum<64>(a[r]);
}

// one row; NU = 1 for a caller that has no registers to spare for groups in flight
template <int NU = 8>
__device__ __forceinline__ float dense_row_dot(const bf16_t* wr, const bf16_t* xr, int K, int lane) {
  const bf16_t* const rows[1] = {wr};
  float v[1];
  dense_rows_dot<1, NU>(rows, xr, K, lane, v);
  return v[0];
}
