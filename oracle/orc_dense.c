/*
 * CPU oracle -- TEST INFRASTRUCTURE (see orc_common.h). Dense bf16 mat-vec, used
 * by the MTP head and the gated-delta a/b projections
 * (/root/reference/src/ops/matmul.rs:334-438; vendored gemv.h: `result +=
 * T(mat) * float(vec)`, fp32 accumulate, output rounded to bf16).
 *
 * Order: lane l owns the 8-element chunks j = l + 64c (c ascending) and runs one
 * fma chain over its elements in memory order; then tree64. K % 8 == 0.
 */
#include "orc_common.h"

float orc_dense_row_dot(const bf16_t* w, int K, const float* x) {
  float lanes[64];
  for (int l = 0; l < 64; ++l) lanes[l] = 0.f;
  for (int j = 0; j < K / 8; ++j) {
    float a = lanes[j % 64];
    for (int i = 0; i < 8; ++i) a = fmaf(orc_bf16_to_f32(w[8 * j + i]), x[8 * j + i], a);
    lanes[j % 64] = a;
  }
  return orc_tree64(lanes);
}

ORC_API void orc_dense_gemv(const bf16_t* w, int O, int K, const bf16_t* x, int M, bf16_t* y) {
  float* xf = (float*)malloc(sizeof(float) * (size_t)K);
  for (int m = 0; m < M; ++m) {
    for (int i = 0; i < K; ++i) xf[i] = orc_bf16_to_f32(x[(size_t)m * K + i]);
#pragma omp parallel for schedule(static)
    for (int o = 0; o < O; ++o)
      y[(size_t)m * O + o] = orc_f32_to_bf16(orc_dense_row_dot(w + (size_t)o * K, K, xf));
  }
  free(xf);
}

/* out[r] = x[lhs[r]] . W[rhs[r]]^T over stacked dense experts W[E,O,K]
 * (src/ops/matmul.rs:649-, `gather_mv`). */
ORC_API void orc_dense_gather_mv(const bf16_t* w, int O, int K, const bf16_t* x,
                                 const uint32_t* lhs, const uint32_t* rhs, int rows, bf16_t* y) {
#pragma omp parallel for schedule(dynamic)
  for (int r = 0; r < rows; ++r) {
    float* xf = (float*)malloc(sizeof(float) * (size_t)K);
    for (int i = 0; i < K; ++i) xf[i] = orc_bf16_to_f32(x[(size_t)lhs[r] * K + i]);
    for (int o = 0; o < O; ++o)
      y[(size_t)r * O + o] =
          orc_f32_to_bf16(orc_dense_row_dot(w + ((size_t)rhs[r] * O + o) * K, K, xf));
    free(xf);
  }
}
