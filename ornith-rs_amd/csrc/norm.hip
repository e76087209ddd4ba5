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
// A lane's piece is moved with the widest aligned vector access (16 bytes for
// pieces of 8 or more values), so a 2048-wide row is four loads per lane.
#include "dmath.h"
#include "rt.h"

namespace {

enum { NORM_PLAIN = 0, NORM_ADD = 1, NORM_GATED = 2 };

// PER consecutive bf16 values <-> fp32 registers
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

__device__ __forceinline__ uint32_t pack2(float a, float b) {
  return (uint32_t)dm_f2bf(a) | ((uint32_t)dm_f2bf(b) << 16);
}

// rounds each value to bf16 and stores
template <int PER>
__device__ __forceinline__ void store_bf16(bf16_t* p, const float (&v)[PER]) {
  if constexpr (PER >= 8) {
#pragma unroll
    for (int c = 0; c < PER / 8; ++c)
      reinterpret_cast<uint4*>(p)[c] =
          make_uint4(pack2(v[8 * c], v[8 * c + 1]), pack2(v[8 * c + 2], v[8 * c + 3]),
                     pack2(v[8 * c + 4], v[8 * c + 5]), pack2(v[8 * c + 6], v[8 * c + 7]));
  } else if constexpr (PER == 4) {
    *reinterpret_cast<uint2*>(p) = make_uint2(pack2(v[0], v[1]), pack2(v[2], v[3]));
  } else if constexpr (PER == 2) {
    *reinterpret_cast<uint32_t*>(p) = pack2(v[0], v[1]);
  } else {
    p[0] = dm_f2bf(v[0]);
  }
}

template <int PER, int MODE>
__global__ __launch_bounds__(64) void rms_kernel(const bf16_t* a, const bf16_t* b, const bf16_t* w,
                                                 const bf16_t* z, bf16_t* h_out, bf16_t* out, int n,
                                                 float eps) {
  const int r = blockIdx.x, lane = threadIdx.x;
  const size_t base = (size_t)r * n + lane * PER;
  float x[PER];
  load_bf16<PER>(a + base, x);
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
  float wv[PER];
  if (w) load_bf16<PER>(w + lane * PER, wv);
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
