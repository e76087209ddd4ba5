// The non-k-quant projections and the polymorphic Linear.
//
// Replaces Linear::matmul (/root/reference/src/ops/linear.rs:23-110), the 8-bit
// affine mat-vec `affine_qmv_fast` (/root/reference/src/ops/quantized.rs:311-333,
// vendored quantized.h:283-289,756-821), the dense bf16 mat-vec and its gathered
// form (/root/reference/src/ops/matmul.rs:334-438,649-) and the embedding lookup
// (/root/reference/src/ops/embedding.rs:18-46).
//
// All are one wavefront per output row: lane l owns the 8-element chunks
// j = l + 64c in ascending c, accumulates them in fp32 and the 64 lane sums go
// through the butterfly. These matrices are small (router-sized or the MTP
// head), so the layout favours a fixed summation order over tuning.
#include "dmath.h"
#include "linear_device.h"
#include "rt.h"

// kquant.hip
extern "C" int kq_qmv_multi_prenorm(ornith_ctx* ctx, const ornith_kmatrix* const* ws, int n,
                                    const void* d_res, const void* d_y, const void* d_wnorm, float eps,
                                    int M, void* d_h_out, void* d_normed_out, void* const* d_ys);

namespace {

// ---- 8-bit affine, group 64 ---------------------------------------------
__global__ __launch_bounds__(64) void affine8_qmv_kernel(const uint8_t* w, const bf16_t* scales,
                                                         const bf16_t* biases, const bf16_t* x,
                                                         bf16_t* y, int O, int K) {
  const int o = blockIdx.x, m = blockIdx.y, lane = threadIdx.x;
  const uint8_t* wr = w + (size_t)o * K;
  const bf16_t* sr = scales + (size_t)o * (K / 64);
  const bf16_t* br = biases + (size_t)o * (K / 64);
  const bf16_t* xr = x + (size_t)m * K;
  float acc_lane = 0.f;
  for (int j = lane; j < K / 8; j += 64) {
    const uint2 q = *reinterpret_cast<const uint2*>(wr + 8 * j);
    const uint4 xv = *reinterpret_cast<const uint4*>(xr + 8 * j);
    const float xs[8] = {dm_bf2f_lo(xv.x), dm_bf2f_hi(xv.x), dm_bf2f_lo(xv.y), dm_bf2f_hi(xv.y),
                         dm_bf2f_lo(xv.z), dm_bf2f_hi(xv.z), dm_bf2f_lo(xv.w), dm_bf2f_hi(xv.w)};
    const uint32_t qw[2] = {q.x, q.y};
    float acc = 0.f, sum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float qf = (float)((qw[i >> 2] >> (8 * (i & 3))) & 0xffu);
      acc = dm_fma(xs[i], qf, acc);
      sum = sum + xs[i];
    }
    const float s = dm_bf2f(sr[j >> 3]), b = dm_bf2f(br[j >> 3]);
    float p = s * acc;
    p = dm_fma(sum, b, p);
    acc_lane = acc_lane + p;
  }
  const float v = dm_wave_sum<64>(acc_lane);
  if (lane == 0) y[(size_t)m * O + o] = dm_f2bf(v);
}

// ---- 4-bit affine, group 32 ------------------------------------------------
// One wavefront per output row (four rows a workgroup); lane l owns the 16-element chunks
// j = l + 64c: 8 code bytes and 16 activations, both one aligned load. GATHER selects the
// expert and the activation row through lhs / rhs.
template <bool GATHER>
__global__ __launch_bounds__(256) void affine4_qmv_kernel(const uint8_t* w, const bf16_t* scales,
                                                          const bf16_t* biases, const bf16_t* x, bf16_t* y,
                                                          int E, int O, int K, int x_rows, const uint32_t* lhs,
                                                          const uint32_t* rhs) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int o = blockIdx.x * 4 + wave, r = blockIdx.y;
  if (o >= O) return;
  size_t row = o, xi = r;
  if constexpr (GATHER) {
    xi = min(lhs[r], (uint32_t)(x_rows - 1));
    row = (size_t)min(rhs[r], (uint32_t)(E - 1)) * O + o;
  }
  const uint8_t* wr = w + row * (K / 2);
  const bf16_t* sr = scales + row * (K / 32);
  const bf16_t* br = biases + row * (K / 32);
  const bf16_t* xr = x + xi * K;
  float acc_lane = 0.f;
  for (int j = lane; j < K / 16; j += 64) {
    const uint2 q = *reinterpret_cast<const uint2*>(wr + 8 * j);
    const uint4 xa = *reinterpret_cast<const uint4*>(xr + 16 * j);
    const uint4 xb = *reinterpret_cast<const uint4*>(xr + 16 * j + 8);
    const float xs[16] = {dm_bf2f_lo(xa.x), dm_bf2f_hi(xa.x), dm_bf2f_lo(xa.y), dm_bf2f_hi(xa.y),
                          dm_bf2f_lo(xa.z), dm_bf2f_hi(xa.z), dm_bf2f_lo(xa.w), dm_bf2f_hi(xa.w),
                          dm_bf2f_lo(xb.x), dm_bf2f_hi(xb.x), dm_bf2f_lo(xb.y), dm_bf2f_hi(xb.y),
                          dm_bf2f_lo(xb.z), dm_bf2f_hi(xb.z), dm_bf2f_lo(xb.w), dm_bf2f_hi(xb.w)};
    const uint32_t qw[2] = {q.x, q.y};
    float acc = 0.f, sum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float qf = (float)((qw[i >> 3] >> (4 * (i & 7))) & 0xfu);
      acc = dm_fma(xs[i], qf, acc);
      sum = sum + xs[i];
    }
    const float s = dm_bf2f(sr[j >> 1]), b = dm_bf2f(br[j >> 1]);
    float p = s * acc;
    p = dm_fma(sum, b, p);
    acc_lane = acc_lane + p;
  }
  const float v = dm_wave_sum<64>(acc_lane);
  if (lane == 0) y[(size_t)r * O + o] = dm_f2bf(v);
}

// ---- dense bf16 ------------------------------------------------------------
// grid.x covers rows four at a time (one per wavefront), grid.y is the
// activation row; GATHER selects expert / activation row through lhs, rhs.
// Up to four matrices over the same activations in one launch: the rows of the
// segments follow each other along grid.x, each segment with its own output.
struct DenseSegs {
  const bf16_t* w[4];
  bf16_t* y[4];
  int O[4];
  int n;
};

template <bool GATHER>
__global__ __launch_bounds__(256) void dense_gemv_kernel(DenseSegs s, const bf16_t* x, int K, int E,
                                                         int x_rows, const uint32_t* lhs,
                                                         const uint32_t* rhs) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int o = blockIdx.x * 4 + wave;
  const bf16_t* w = s.w[0];
  bf16_t* y = s.y[0];
  int O = s.O[0];
#pragma unroll
  for (int i = 1; i < 4; ++i) {
    if (i < s.n && o >= O) {
      o -= O;
      w = s.w[i];
      y = s.y[i];
      O = s.O[i];
    }
  }
  if (o >= O) return;
  const int r = blockIdx.y;
  const bf16_t* wr;
  const bf16_t* xr;
  if constexpr (GATHER) {
    const uint32_t xi = min(lhs[r], (uint32_t)(x_rows - 1));
    const uint32_t ei = min(rhs[r], (uint32_t)(E - 1));
    wr = w + ((size_t)ei * O + o) * K;
    xr = x + (size_t)xi * K;
  } else {
    wr = w + (size_t)o * K;
    xr = x + (size_t)r * K;
  }
  const float v = dense_row_dot(wr, xr, K, lane);
  if (lane == 0) y[(size_t)r * O + o] = dm_f2bf(v);
}

// ---- embedding: out = bf16(bf16(q * scale) + bias) ------------------------------
__global__ void embedding_kernel(const uint8_t* w, const bf16_t* scales, const bf16_t* biases,
                                 const uint32_t* ids, bf16_t* out, int V, int K) {
  const int r = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= K) return;
  const size_t row = min(ids[r], (uint32_t)(V - 1));
  const float s = dm_bf2f(scales[row * (K / 64) + i / 64]);
  const float b = dm_bf2f(biases[row * (K / 64) + i / 64]);
  const float v = dm_rb((float)w[row * K + i] * s);
  out[(size_t)r * K + i] = dm_f2bf(v + b);
}

// 4-bit table rows: out = bf16(bf16(q * scale) + bias)
__global__ void embedding4_kernel(const uint8_t* w, const bf16_t* scales, const bf16_t* biases,
                                  const uint32_t* ids, bf16_t* out, int V, int K) {
  const int r = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= K) return;
  const size_t row = min(ids[r], (uint32_t)(V - 1));
  const uint8_t byte = w[row * (K / 2) + i / 2];
  const float q = (float)((i & 1) ? (byte >> 4) : (byte & 0xF));
  const float s = dm_bf2f(scales[row * (K / 32) + i / 32]);
  const float b = dm_bf2f(biases[row * (K / 32) + i / 32]);
  out[(size_t)r * K + i] = dm_f2bf(dm_rb(q * s) + b);
}

// ---- dense bf16 at prefill widths: a small GEMM on the matrix cores -------------------
// y[M, O] = x[M, K] . W[O, K]^T for the narrow dense projections (the gated-delta a / b heads,
// the shared expert's gate: O of 1 .. 64): as mat-vecs every activation row is read by O / 4
// workgroups. One workgroup = 16 rows; its four wavefronts split K and add up through LDS; a
// wavefront feeds v_mfma_f32_16x16x32_bf16 straight from global memory (A: 16 rows x 32
// channels, B: 16 outputs x 32 channels, 16 bytes a lane each). grid.y covers O in 64s.
typedef __bf16 dmm_bf16x8_t __attribute__((ext_vector_type(8)));
typedef float dmm_f32x4_t __attribute__((ext_vector_type(4)));

struct DenseMmSegs {
  const bf16_t* w[4];
  bf16_t* y[4];
  int O[4];
  int n;
};

__global__ __launch_bounds__(256) void dense_mm_kernel(DenseMmSegs s, const bf16_t* x, int M, int K) {
  __shared__ float red[3][4][64][4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l16 = lane & 15, lg = lane >> 4;
  const int row0 = blockIdx.x * 16;
  const int kw = K / 4, k0 = wave * kw;  // K is a multiple of 128
  const bf16_t* xp = x + (size_t)min(row0 + l16, M - 1) * K + k0 + 8 * lg;
  // the four 16-output tiles of this workgroup: tile 4 * blockIdx.y + nt of the segments' tiles
  // laid end to end (a segment's last tile may be ragged)
  const bf16_t* wp[4];
  bf16_t* yp[4];
  int ocol[4], oend[4], ostride[4];
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) {
    int t = 4 * blockIdx.y + nt, seg = -1;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (seg < 0 && i < s.n) {
        const int tiles = (s.O[i] + 15) / 16;
        if (t < tiles) seg = i; else t -= tiles;
      }
    const int sg = seg < 0 ? 0 : seg;
    ocol[nt] = 16 * t + l16;
    oend[nt] = seg < 0 ? 0 : s.O[sg];
    ostride[nt] = s.O[sg];
    yp[nt] = s.y[sg];
    wp[nt] = s.w[sg] + (size_t)min(ocol[nt], s.O[sg] - 1) * K + k0 + 8 * lg;
  }
  dmm_f32x4_t acc[4];
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) acc[nt] = dmm_f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int k = 0; k < kw; k += 32) {
    const dmm_bf16x8_t a = *reinterpret_cast<const dmm_bf16x8_t*>(xp + k);
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
      if (oend[nt] > 0) {  // (the same for every lane of the wavefront)
        const dmm_bf16x8_t b = *reinterpret_cast<const dmm_bf16x8_t*>(wp[nt] + k);
        acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[nt], 0, 0, 0);
      }
  }
  if (wave > 0) {
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave - 1][nt][lane][r] = acc[nt][r];
  }
  __syncthreads();
  if (wave > 0) return;
  // D[m = 4 * lg + r][n = l16]
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = row0 + 4 * lg + r;
      const float v = ((acc[nt][r] + red[0][nt][lane][r]) + red[1][nt][lane][r]) + red[2][nt][lane][r];
      if (ocol[nt] < oend[nt] && row < M) yp[nt][(size_t)row * ostride[nt] + ocol[nt]] = dm_f2bf(v);
    }
  }
}

// up to four dense matrices of one K over the same activations at prefill width; false when
// the shapes do not allow it
static bool launch_dense_mm(ornith_ctx* ctx, const ornith_linear* const* ws, int n, const void* d_x, int M,
                            void* const* d_ys) {
  if (n < 1 || n > 4 || ((uintptr_t)d_x & 15) != 0) return false;
  DenseMmSegs s{};
  s.n = n;
  int tiles = 0;
  for (int i = 0; i < n; ++i) {
    if (ws[i]->mode != ORNITH_LIN_DENSE || !ws[i]->d_w || ws[i]->K != ws[0]->K || ws[i]->K % 128 != 0 || ws[i]->O < 1 ||
        ((uintptr_t)ws[i]->d_w & 15) != 0)
      return false;
    s.w[i] = (const bf16_t*)ws[i]->d_w;
    s.y[i] = (bf16_t*)d_ys[i];
    s.O[i] = ws[i]->O;
    tiles += (ws[i]->O + 15) / 16;
  }
  hipLaunchKernelGGL(dense_mm_kernel, dim3((M + 15) / 16, (tiles + 3) / 4), dim3(256), 0, ctx->stream, s,
                     (const bf16_t*)d_x, M, ws[0]->K);
  return true;
}

template <bool GATHER>
int launch_dense(ornith_ctx* ctx, const DenseSegs& s, const void* d_x, int K, int E, int x_rows,
                 const uint32_t* d_lhs, const uint32_t* d_rhs, int rows) {
  int total = 0;
  for (int i = 0; i < s.n; ++i) total += s.O[i];
  hipLaunchKernelGGL(dense_gemv_kernel<GATHER>, dim3((total + 3) / 4, rows), dim3(256), 0, ctx->stream, s,
                     (const bf16_t*)d_x, K, E, x_rows, d_lhs, d_rhs);
  ORN_LAUNCH_CHECK(GATHER ? "dense_gemv_kernel<gather>" : "dense_gemv_kernel");
  return ORNITH_OK;
}

}  // namespace

// Several stacked expert tensors [E, O, K] gathered over the same (activation row, expert)
// pairs in one launch (the gate and up projections of dense experts).
extern "C" int dense_gather_mv_multi(ornith_ctx* ctx, const void* const* d_ws, int n, int E, int O, int K,
                                     const void* d_x, int x_rows, const uint32_t* d_lhs,
                                     const uint32_t* d_rhs, int rows, void* const* d_ys) {
  ORN_REQUIRE(ctx && d_ws && d_ys && d_x && d_lhs && d_rhs && n >= 1 && n <= 4, "dense_gather_mv_multi: bad argument");
  ORN_REQUIRE(E >= 1 && O >= 1 && K % 8 == 0 && x_rows >= 1 && rows >= 0 && rows <= 65535,
              "dense_gather_mv: E=%d O=%d K=%d rows=%d", E, O, K, rows);
  if (rows == 0) return ORNITH_OK;
  DenseSegs s{};
  s.n = n;
  for (int i = 0; i < n; ++i) {
    ORN_REQUIRE(d_ws[i] && d_ys[i], "dense_gather_mv_multi: null entry %d", i);
    s.w[i] = (const bf16_t*)d_ws[i];
    s.y[i] = (bf16_t*)d_ys[i];
    s.O[i] = O;
  }
  return launch_dense<true>(ctx, s, d_x, K, E, x_rows, d_lhs, d_rhs, rows);
}

extern "C" {

int ornith_linear_matmul(ornith_ctx* ctx, const ornith_linear* w, const void* d_x, int M,
                         void* d_y) {
  ORN_REQUIRE(ctx && w && d_x && d_y, "linear_matmul: null argument");
  ORN_REQUIRE(M >= 1, "linear_matmul: M=%d", M);
  switch (w->mode) {
    case ORNITH_LIN_KQUANT:
      ORN_REQUIRE(w->km.O == w->O && w->km.K == w->K, "linear_matmul: k-quant dims disagree");
      // kquant::matmul (src/ops/kquant.rs:783-800): rows within the exact window go through
      // the mat-vec (each row as if alone), prefill widths through the tiled GEMM
      if (M >= kPrefillRows) return ornith_kq_matmul(ctx, &w->km, d_x, M, d_y);
      return ornith_kq_qmv(ctx, &w->km, d_x, ORNITH_BF16, M, d_y, ORNITH_BF16);
    case ORNITH_LIN_AFFINE8:
      ORN_REQUIRE(w->d_w && w->d_scales && w->d_biases, "linear_matmul: affine tensor missing");
      ORN_REQUIRE(w->K % 64 == 0 && w->O >= 1 && M <= 65535, "linear_matmul: affine O=%d K=%d",
                  w->O, w->K);
      hipLaunchKernelGGL(affine8_qmv_kernel, dim3(w->O, M), dim3(64), 0, ctx->stream,
                         (const uint8_t*)w->d_w, (const bf16_t*)w->d_scales,
                         (const bf16_t*)w->d_biases, (const bf16_t*)d_x, (bf16_t*)d_y, w->O, w->K);
      ORN_LAUNCH_CHECK("affine8_qmv_kernel");
      return ORNITH_OK;
    case ORNITH_LIN_AFFINE4:
      ORN_REQUIRE(w->d_w && w->d_scales && w->d_biases, "linear_matmul: affine tensor missing");
      ORN_REQUIRE(w->K % 32 == 0 && w->O >= 1 && M <= 65535, "linear_matmul: 4-bit affine O=%d K=%d", w->O, w->K);
      hipLaunchKernelGGL(affine4_qmv_kernel<false>, dim3((w->O + 3) / 4, M), dim3(256), 0, ctx->stream,
                         (const uint8_t*)w->d_w, (const bf16_t*)w->d_scales, (const bf16_t*)w->d_biases,
                         (const bf16_t*)d_x, (bf16_t*)d_y, 1, w->O, w->K, M, (const uint32_t*)nullptr,
                         (const uint32_t*)nullptr);
      ORN_LAUNCH_CHECK("affine4_qmv_kernel");
      return ORNITH_OK;
    case ORNITH_LIN_DENSE:
      ORN_REQUIRE(w->d_w, "linear_matmul: dense weight missing");
      ORN_REQUIRE(w->K % 8 == 0 && w->O >= 1 && M <= 65535, "linear_matmul: dense O=%d K=%d", w->O,
                  w->K);
      // prefill widths (outside the exact window, like the k-quant GEMM): on the matrix cores
      if (M >= kPrefillRows && launch_dense_mm(ctx, &w, 1, d_x, M, &d_y)) {
        ORN_LAUNCH_CHECK("dense_mm_kernel");
        return ORNITH_OK;
      }
      {
        DenseSegs s{};
        s.n = 1;
        s.w[0] = (const bf16_t*)w->d_w;
        s.y[0] = (bf16_t*)d_y;
        s.O[0] = w->O;
        return launch_dense<false>(ctx, s, d_x, w->K, 1, M, nullptr, nullptr, M);
      }
    default:
      return ornith_fail(ORNITH_ERR_INVALID, "linear_matmul: unknown mode %d", w->mode);
  }
}

int ornith_linear_matmul_multi(ornith_ctx* ctx, const ornith_linear* const* ws, int n,
                               const void* d_x, int M, void* const* d_ys) {
  ORN_REQUIRE(ctx && ws && d_x && d_ys && n >= 1, "linear_matmul_multi: bad argument");
  bool fuse = ornith_option_fuse_proj() && n >= 2 && n <= 4 && M < kPrefillRows;
  for (int i = 0; i < n; ++i) {
    ORN_REQUIRE(ws[i] && d_ys[i], "linear_matmul_multi: null entry %d", i);
    fuse = fuse && ws[i]->mode == ws[0]->mode && ws[i]->K == ws[0]->K;
    if (ws[i]->mode == ORNITH_LIN_KQUANT) fuse = fuse && ws[i]->km.kind == ws[0]->km.kind;
  }
  if (fuse && ws[0]->mode == ORNITH_LIN_KQUANT) {
    const ornith_kmatrix* kms[4];
    for (int i = 0; i < n; ++i) kms[i] = &ws[i]->km;
    return ornith_kq_qmv_multi(ctx, kms, n, d_x, ORNITH_BF16, M, d_ys, ORNITH_BF16);
  }
  if (fuse && ws[0]->mode == ORNITH_LIN_DENSE && ws[0]->K % 8 == 0 && M <= 65535) {
    DenseSegs s{};
    s.n = n;
    for (int i = 0; i < n; ++i) {
      ORN_REQUIRE(ws[i]->d_w && ws[i]->O >= 1, "linear_matmul_multi: dense weight %d missing", i);
      s.w[i] = (const bf16_t*)ws[i]->d_w;
      s.y[i] = (bf16_t*)d_ys[i];
      s.O[i] = ws[i]->O;
    }
    return launch_dense<false>(ctx, s, d_x, ws[0]->K, 1, M, nullptr, nullptr, M);
  }
  // prefill widths: dense matrices of one K share a launch
  if (M >= kPrefillRows && ornith_option_fuse_proj() && n >= 2 && launch_dense_mm(ctx, ws, n, d_x, M, d_ys)) {
    ORN_LAUNCH_CHECK("dense_mm_kernel");
    return ORNITH_OK;
  }
  // prefill widths: runs of k-quant matrices of one K share a GEMM launch. A run of one kind may
  // be large (it picks its tile by size); a matrix of the other kind joins a run only while the
  // run is narrow (a mixed launch takes 128-row tiles, which wide matrices should not pay for).
  for (int i = 0; i < n;) {
    int j = i + 1;
    if (M >= kPrefillRows && ornith_option_fuse_proj() && ws[i]->mode == ORNITH_LIN_KQUANT) {
      int cols = ws[i]->O;
      bool mixed = false;
      while (j < n && j - i < 4 && ws[j]->mode == ORNITH_LIN_KQUANT && ws[j]->K == ws[i]->K) {
        const bool other = ws[j]->km.kind != ws[i]->km.kind;
        if ((other || mixed) && cols + ws[j]->O > 2048) break;
        mixed = mixed || other;
        cols += ws[j]->O;
        ++j;
      }
    }
    int rc;
    if (j - i >= 2) {
      const ornith_kmatrix* kms[4];
      for (int t = i; t < j; ++t) {
        ORN_REQUIRE(ws[t]->km.O == ws[t]->O && ws[t]->km.K == ws[t]->K, "linear_matmul_multi: k-quant dims disagree");
        kms[t - i] = &ws[t]->km;
      }
      rc = ornith_kq_matmul_multi(ctx, kms, j - i, d_x, M, d_ys + i);
    } else {
      rc = ornith_linear_matmul(ctx, ws[i], d_x, M, d_ys[i]);
    }
    if (rc) return rc;
    i = j;
  }
  return ORNITH_OK;
}

int ornith_add_rms_linear_multi(ornith_ctx* ctx, const ornith_linear* const* ws, int n,
                                const void* d_res, const void* d_y, const void* d_wnorm, float eps, int M,
                                void* d_h_out, void* d_normed_out, void* const* d_ys) {
  ORN_REQUIRE(ctx && ws && d_res && d_y && d_wnorm && d_h_out && d_normed_out && d_ys && n >= 1,
              "add_rms_linear_multi: bad argument");
  bool fuse = ornith_option_fuse_norm() && n <= 4 && M <= 4;
  const ornith_kmatrix* kms[4];
  for (int i = 0; i < n && fuse; ++i) {
    fuse = ws[i] && ws[i]->mode == ORNITH_LIN_KQUANT && ws[i]->K == 2048;
    if (fuse) kms[i] = &ws[i]->km;
  }
  if (fuse) {
    const int rc = kq_qmv_multi_prenorm(ctx, kms, n, d_res, d_y, d_wnorm, eps, M, d_h_out, d_normed_out, d_ys);
    if (rc >= 0) return rc;
  }
  int rc = ornith_add_rms_norm(ctx, d_res, d_y, d_wnorm, M, ws[0]->K, eps, d_h_out, d_normed_out);
  if (rc) return rc;
  return ornith_linear_matmul_multi(ctx, ws, n, d_normed_out, M, d_ys);
}

int ornith_dense_gather_mv(ornith_ctx* ctx, const void* d_w, int E, int O, int K, const void* d_x,
                           int x_rows, const uint32_t* d_lhs, const uint32_t* d_rhs, int rows,
                           void* d_y) {
  ORN_REQUIRE(ctx && d_w && d_x && d_lhs && d_rhs && d_y, "dense_gather_mv: null argument");
  ORN_REQUIRE(E >= 1 && O >= 1 && K % 8 == 0 && x_rows >= 1 && rows >= 0 && rows <= 65535,
              "dense_gather_mv: E=%d O=%d K=%d rows=%d", E, O, K, rows);
  if (rows == 0) return ORNITH_OK;
  const void* ws[1] = {d_w};
  void* ys[1] = {d_y};
  return dense_gather_mv_multi(ctx, ws, 1, E, O, K, d_x, x_rows, d_lhs, d_rhs, rows, ys);
}

int ornith_affine4_gather_qmv(ornith_ctx* ctx, const void* d_w, const void* d_scales, const void* d_biases,
                              int E, int O, int K, const void* d_x, int x_rows, const uint32_t* d_lhs,
                              const uint32_t* d_rhs, int rows, void* d_y) {
  ORN_REQUIRE(ctx && d_w && d_scales && d_biases && d_x && d_lhs && d_rhs && d_y, "affine4_gather_qmv: null argument");
  ORN_REQUIRE(E >= 1 && O >= 1 && K % 32 == 0 && x_rows >= 1 && rows >= 0 && rows <= 65535,
              "affine4_gather_qmv: E=%d O=%d K=%d rows=%d", E, O, K, rows);
  if (rows == 0) return ORNITH_OK;
  hipLaunchKernelGGL(affine4_qmv_kernel<true>, dim3((O + 3) / 4, rows), dim3(256), 0, ctx->stream,
                     (const uint8_t*)d_w, (const bf16_t*)d_scales, (const bf16_t*)d_biases, (const bf16_t*)d_x,
                     (bf16_t*)d_y, E, O, K, x_rows, d_lhs, d_rhs);
  ORN_LAUNCH_CHECK("affine4_qmv_kernel<gather>");
  return ORNITH_OK;
}

int ornith_embedding(ornith_ctx* ctx, const ornith_linear* table, const uint32_t* d_ids, int n,
                     void* d_out) {
  ORN_REQUIRE(ctx && table && d_ids && d_out, "embedding: null argument");
  ORN_REQUIRE(table->mode == ORNITH_LIN_AFFINE8 || table->mode == ORNITH_LIN_AFFINE4,
              "embedding: table mode %d; the lookup is defined for the affine tables only",
              table->mode);
  ORN_REQUIRE(table->K % 64 == 0 && n >= 0 && n <= 65535, "embedding: K=%d n=%d", table->K, n);
  if (n == 0) return ORNITH_OK;
  if (table->mode == ORNITH_LIN_AFFINE4) {
    hipLaunchKernelGGL(embedding4_kernel, dim3((table->K + 255) / 256, n), dim3(256), 0, ctx->stream,
                       (const uint8_t*)table->d_w, (const bf16_t*)table->d_scales,
                       (const bf16_t*)table->d_biases, d_ids, (bf16_t*)d_out, table->O, table->K);
    ORN_LAUNCH_CHECK("embedding4_kernel");
    return ORNITH_OK;
  }
  hipLaunchKernelGGL(embedding_kernel, dim3((table->K + 255) / 256, n), dim3(256), 0, ctx->stream,
                     (const uint8_t*)table->d_w, (const bf16_t*)table->d_scales,
                     (const bf16_t*)table->d_biases, d_ids, (bf16_t*)d_out, table->O, table->K);
  ORN_LAUNCH_CHECK("embedding_kernel");
  return ORNITH_OK;
}

}  // extern "C"
