// One row of the dense bf16 mat-vec by one wavefront: groups of 8 weights, group j on lane
// j mod 64, one fma chain per lane in group order, butterfly over the 64 lanes. Shared by the
// dense kernels of linear.hip and by kernels that fold a small projection into their head
// (ops::matmul::gemv, /root/reference/src/ops/matmul.rs:334-438, fp32 accumulate).
#pragma once

#include "dmath.h"

__device__ __forceinline__ float dense_row_dot(const bf16_t* wr, const bf16_t* xr, int K, int lane) {
  float a = 0.f;
  for (int j = lane; j < K / 8; j += 64) {
    const uint4 wv = *reinterpret_cast<const uint4*>(wr + 8 * j);
    const uint4 xv = *reinterpret_cast<const uint4*>(xr + 8 * j);
    a = dm_fma(dm_bf2f_lo(wv.x), dm_bf2f_lo(xv.x), a);
    a = dm_fma(dm_bf2f_hi(wv.x), dm_bf2f_hi(xv.x), a);
    a = dm_fma(dm_bf2f_lo(wv.y), dm_bf2f_lo(xv.y), a);
    a = dm_fma(dm_bf2f_hi(wv.y), dm_bf2f_hi(xv.y), a);
    a = dm_fma(dm_bf2f_lo(wv.z), dm_bf2f_lo(xv.z), a);
    a = dm_fma(dm_bf2f_hi(wv.z), dm_bf2f_hi(xv.z), a);
    a = dm_fma(dm_bf2f_lo(wv.w), dm_bf2f_lo(xv.w), a);
    a = dm_fma(dm_bf2f_hi(wv.w), dm_bf2f_hi(xv.w), a);
  }
  return dm_wave_sum<64>(a);
}
