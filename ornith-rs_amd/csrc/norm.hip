// RMS norms: plain, fused residual add, and the gated output norm of the
// gated-delta layer.
//
// Replaces norm::{rms_norm, add_rms_norm, rms_norm_gated}
// (/root/reference/src/ops/norm.rs:19-220; vendored rms_norm.metal:12-81,
// /root/reference/kernels/ornith_norm.metal:28-183).
//
// One wavefront per row. Lane l owns the contiguous piece [l*n/64, (l+1)*n/64),
// sums its squares with one fma chain, and the 64 lane sums go through the
// butterfly. Two roundings on the way out, as in the reference:
//   out = bf16(w * bf16(x * inv)),  inv = 1 / sqrt(sum / n + eps).
#include "dmath.h"
#include "rt.h"

namespace {

enum { NORM_PLAIN = 0, NORM_ADD = 1, NORM_GATED = 2 };

template <int PER, int MODE>
__global__ __launch_bounds__(64) void rms_kernel(const bf16_t* a, const bf16_t* b, const bf16_t* w,
                                                 const bf16_t* z, bf16_t* h_out, bf16_t* out, int n,
                                                 float eps) {
  const int r = blockIdx.x, lane = threadIdx.x;
  const size_t base = (size_t)r * n + lane * PER;
  float x[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    x[i] = dm_bf2f(a[base + i]);
    if constexpr (MODE == NORM_ADD) {
      const bf16_t h = dm_f2bf(x[i] + dm_bf2f(b[base + i]));
      h_out[base + i] = h;
      x[i] = dm_bf2f(h);
    }
  }
  float acc = 0.f;
#pragma unroll
  for (int i = 0; i < PER; ++i) acc = dm_fma(x[i], x[i], acc);
  const float inv = dm_rsqrt(dm_wave_sum<64>(acc) / (float)n + eps);
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    float v = dm_rb(x[i] * inv);
    if (w) v = dm_rb(dm_bf2f(w[lane * PER + i]) * v);
    if constexpr (MODE == NORM_GATED) {
      float g = dm_bf2f(z[base + i]);
      g = g * dm_sigmoid_f32(g);
      v = g * v;
    }
    out[base + i] = dm_f2bf(v);
  }
}

template <int MODE>
int launch_rms(ornith_ctx* ctx, const void* a, const void* b, const void* w, const void* z,
               void* h_out, void* out, int rows, int n, float eps, const char* who) {
  ORN_REQUIRE(rows >= 1 && n >= 64 && n % 64 == 0, "%s: rows=%d n=%d", who, rows, n);
#define RMS_CASE(P)                                                                              \
  case P:                                                                                        \
    hipLaunchKernelGGL((rms_kernel<P, MODE>), dim3(rows), dim3(64), 0, ctx->stream,              \
                       (const bf16_t*)a, (const bf16_t*)b, (const bf16_t*)w, (const bf16_t*)z,   \
                       (bf16_t*)h_out, (bf16_t*)out, n, eps);                                    \
    break;
  switch (n / 64) {
    RMS_CASE(1)
    RMS_CASE(2)
    RMS_CASE(4)
    RMS_CASE(8)
    RMS_CASE(16)
    RMS_CASE(32)
    RMS_CASE(64)
    default:
      return ornith_fail(ORNITH_ERR_UNSUPPORTED, "%s: row width %d (need 64 * 2^j, j <= 6)", who, n);
  }
#undef RMS_CASE
  ORN_LAUNCH_CHECK("rms_kernel");
  return ORNITH_OK;
}

}  // namespace

extern "C" {

int ornith_rms_norm(ornith_ctx* ctx, const void* d_x, const void* d_w, int rows, int n, float eps,
                    void* d_out) {
  ORN_REQUIRE(ctx && d_x && d_out, "rms_norm: null argument");
  return launch_rms<NORM_PLAIN>(ctx, d_x, nullptr, d_w, nullptr, nullptr, d_out, rows, n, eps,
                                "rms_norm");
}

int ornith_add_rms_norm(ornith_ctx* ctx, const void* d_a, const void* d_b, const void* d_w, int rows,
                        int n, float eps, void* d_h_out, void* d_out) {
  ORN_REQUIRE(ctx && d_a && d_b && d_h_out && d_out, "add_rms_norm: null argument");
  return launch_rms<NORM_ADD>(ctx, d_a, d_b, d_w, nullptr, d_h_out, d_out, rows, n, eps,
                              "add_rms_norm");
}

int ornith_rms_norm_gated(ornith_ctx* ctx, const void* d_y, const void* d_w, const void* d_z,
                          int rows, int n, float eps, void* d_out) {
  ORN_REQUIRE(ctx && d_y && d_w && d_z && d_out, "rms_norm_gated: null argument");
  return launch_rms<NORM_GATED>(ctx, d_y, nullptr, d_w, d_z, nullptr, d_out, rows, n, eps,
                                "rms_norm_gated");
}

}  // extern "C"
