// RMS norms: plain, fused residual add, and the gated output norm of the
// gated-delta layer.
//
// Replaces norm::{rms_norm, add_rms_norm, rms_norm_gated}
// (/root/reference/src/ops/norm.rs:19-220; vendored rms_norm.metal:12-81,
// /root/reference/kernels/ornith_norm.metal:28-183).
//
// Rows up to 512 wide: one wavefront per row (see norm_device.h for the arithmetic and
// its order). Wider rows: one workgroup of n/8 threads per row, eight values (16 bytes)
// per thread, because a single wavefront walking 32 or 64 values per lane through the
// add / round / scale / round steps is a chain of thousands of dependent instructions.
// The element-wise steps are spread over the workgroup; only the sum of squares keeps
// its defined order (lane l of the first wavefront owns [l*PER, (l+1)*PER), one fma
// chain, butterfly), reading the values from LDS laid out so that lane l's i-th value
// sits at [i][l].
#include "norm_device.h"
#include "rt.h"

namespace {

template <int PER, int MODE>
__global__ __launch_bounds__(64) void rms_kernel(const bf16_t* a, const bf16_t* b, const bf16_t* w,
                                                 const bf16_t* z, bf16_t* h_out, bf16_t* out, int n,
                                                 float eps) {
  const size_t off = (size_t)blockIdx.x * n;
  rms_row<PER, MODE>(a + off, b ? b + off : nullptr, w, z ? z + off : nullptr,
                     h_out ? h_out + off : nullptr, out + off, n, eps, threadIdx.x);
}

template <int PER, int MODE>
__global__ __launch_bounds__(PER * 8) void rms_wide_kernel(const bf16_t* a, const bf16_t* b,
                                                           const bf16_t* w, bf16_t* h_out,
                                                           bf16_t* out, int n, float eps) {
  static_assert(PER % 8 == 0 && MODE != NORM_GATED, "wide rows: plain and add only");
  __shared__ float xs[PER * 64];
  __shared__ float s_inv;
  const size_t off = (size_t)blockIdx.x * n;
  const int tid = threadIdx.x, e0 = tid * 8;
  float x[8], wv[8];
  load_bf16<8>(a + off + e0, x);
  if (w) load_bf16<8>(w + e0, wv);
  if constexpr (MODE == NORM_ADD) {
    float y[8];
    load_bf16<8>(b + off + e0, y);
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = dm_rb(x[i] + y[i]);
    store_bf16<8>(h_out + off + e0, x);
  }
  // value e belongs to lane e / PER, position e % PER
  const int lane_of = e0 / PER, pos0 = e0 % PER;
#pragma unroll
  for (int i = 0; i < 8; ++i) xs[(pos0 + i) * 64 + lane_of] = x[i];
  __syncthreads();
  if (tid < 64) {
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const float v = xs[i * 64 + tid];
      acc = dm_fma(v, v, acc);
    }
    const float inv = dm_rsqrt(dm_wave_sum<64>(acc) / (float)n + eps);
    if (tid == 0) s_inv = inv;
  }
  __syncthreads();
  const float inv = s_inv;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    x[i] = dm_rb(x[i] * inv);
    if (w) x[i] = dm_rb(wv[i] * x[i]);
  }
  store_bf16<8>(out + off + e0, x);
}

template <int MODE>
int launch_rms(ornith_ctx* ctx, const void* a, const void* b, const void* w, const void* z,
               void* h_out, void* out, int rows, int n, float eps, const char* who) {
  ORN_REQUIRE(rows >= 1 && n >= 64 && n % 64 == 0, "%s: rows=%d n=%d", who, rows, n);
  // vector accesses need the row pieces aligned: rows start on n*2 bytes, pieces on PER*2
  const uintptr_t all = (uintptr_t)a | (uintptr_t)b | (uintptr_t)w | (uintptr_t)z | (uintptr_t)h_out |
                        (uintptr_t)out;
  ORN_REQUIRE((all & 15) == 0, "%s: operands must be 16-byte aligned", who);
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
#undef RMS_CASE
#define RMS_CASE(P)                                                                              \
  case P:                                                                                        \
    if constexpr (MODE == NORM_GATED)                                                            \
      hipLaunchKernelGGL((rms_kernel<P, MODE>), dim3(rows), dim3(64), 0, ctx->stream,            \
                         (const bf16_t*)a, (const bf16_t*)b, (const bf16_t*)w, (const bf16_t*)z, \
                         (bf16_t*)h_out, (bf16_t*)out, n, eps);                                  \
    else                                                                                         \
      hipLaunchKernelGGL((rms_wide_kernel<P, MODE>), dim3(rows), dim3(P * 8), 0, ctx->stream,    \
                         (const bf16_t*)a, (const bf16_t*)b, (const bf16_t*)w, (bf16_t*)h_out,   \
                         (bf16_t*)out, n, eps);                                                  \
    break;
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
