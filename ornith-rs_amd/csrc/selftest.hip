// Element-wise evaluation of the device scalar functions, so a caller can check
// them bit for bit against a CPU evaluation of the same formulae.
#include "dmath.h"
#include "rt.h"

namespace {
__global__ void unary_kernel(int op, const float* in, float* out, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float x = in[i];
  float y;
  switch (op) {
    case ORNITH_FN_EXP: y = dm_exp(x); break;
    case ORNITH_FN_LOG: y = dm_log(x); break;
    case ORNITH_FN_LOG1P: y = dm_log1p(x); break;
    case ORNITH_FN_SIGMOID_BF16: y = dm_sigmoid_bf16(dm_rb(x)); break;
    case ORNITH_FN_SIGMOID_F32: y = dm_sigmoid_f32(x); break;
    case ORNITH_FN_RSQRT: y = dm_rsqrt(x); break;
    case ORNITH_FN_RECIP: y = 1.0f / x; break;
    case ORNITH_FN_ROUND_BF16: y = dm_rb(x); break;
    case ORNITH_FN_WAVE_SUM: y = dm_wave_sum<64>(x); break;
    case ORNITH_FN_XOR_LANE + 0: y = dm_xor_lane<1>(x); break;
    case ORNITH_FN_XOR_LANE + 1: y = dm_xor_lane<2>(x); break;
    case ORNITH_FN_XOR_LANE + 2: y = dm_xor_lane<4>(x); break;
    case ORNITH_FN_XOR_LANE + 3: y = dm_xor_lane<8>(x); break;
    case ORNITH_FN_XOR_LANE + 4: y = dm_xor_lane<16>(x); break;
    case ORNITH_FN_XOR_LANE + 5: y = dm_xor_lane<32>(x); break;
    default: y = x;
  }
  out[i] = y;
}
}  // namespace

extern "C" int ornith_selftest_unary(ornith_ctx* ctx, int fn, const float* d_in, float* d_out,
                                     int64_t n) {
  ORN_REQUIRE(ctx && d_in && d_out && n >= 0, "selftest_unary: bad argument");
  ORN_REQUIRE(fn >= 0 && fn <= ORNITH_FN_XOR_LANE + 5, "selftest_unary: unknown function %d", fn);
  // the lane-crossing functions need whole wavefronts: n a multiple of the 256-thread block
  ORN_REQUIRE(fn < ORNITH_FN_WAVE_SUM || n % 256 == 0, "selftest_unary: function %d needs n %% 256 == 0", fn);
  if (n == 0) return ORNITH_OK;
  hipLaunchKernelGGL(unary_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, ctx->stream, fn,
                     d_in, d_out, n);
  ORN_LAUNCH_CHECK("unary_kernel");
  return ORNITH_OK;
}
