// The expert half of the MoE block for the two formats whose row dot is one wavefront a row:
// the published artifact's (routed and shared experts in mlx 4-bit affine, group 32,
// /root/reference/src/ops/quantized.rs:311-333,531-589) and the MTP head's (dense bf16 experts,
// /root/reference/src/model/mtp.rs, gather_mm over [E, O, K] tensors). The operator path is
// moe.hip. Two launches that mirror moe_up_kernel / moe_down_kernel
// (moe_fused.hip) in place of five (two gathered mat-vecs, swiglu, the shared expert's down
// projection, the gathered down projection, the combine):
//
// moe_up_affine4:   a wavefront per (token, expert slot | shared, output row): the gate and the
//                   up row over the same activation registers, swiglu -> act. With `gates` the
//                   softmax + top-k of the row's token is made in the head of the launch.
// moe_down_affine4: a workgroup per (token, eight output columns), wavefront j = expert slot j
//                   (the last the shared expert): eight row dots each, met in LDS, then the
//                   block's tail (router weights, bf16 accumulation in slot order, sigmoid-gated
//                   shared expert).
//
// A 4-bit row dot is affine4_qmv_kernel's (linear.hip), operation for operation: lane l owns the
// 16-code chunks l + 64c in ascending c, one fma chain a chunk in code order beside the plain
// sum of its activations, scale * chain + bias * sum per chunk added to the lane's running
// value, then the 64-lane butterfly; a dense one is dense_row_dot (linear_device.h), the
// function the operator path's kernels call. So the two launches give the bits of the operator
// path and of the oracle (oracle/orc_moe.c).
#include "linear_device.h"
#include "moe_device.h"
#include "rt.h"

namespace {

constexpr int kA4MaxK = 8;  // routed experts a token the down kernel's workgroup holds

struct A4Mat {
  const uint8_t* w;      // [rows, K/2]
  const bf16_t* scales;  // [rows, K/32]
  const bf16_t* biases;  // [rows, K/32]
};

// 16 activations of chunk j as floats, and their sum in code order
struct A4X {
  float v[16];
  float sum;
  __device__ __forceinline__ void load(const bf16_t* xr, int j) {
    const uint4 xa = *reinterpret_cast<const uint4*>(xr + 16 * j);
    const uint4 xb = *reinterpret_cast<const uint4*>(xr + 16 * j + 8);
    const uint32_t wds[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
    sum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      v[2 * i] = dm_bf2f_lo(wds[i]);
      v[2 * i + 1] = dm_bf2f_hi(wds[i]);
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) sum = sum + v[i];
  }
};

// one chunk's contribution: scale * sum_i x_i q_i + bias * sum_i x_i
__device__ __forceinline__ float a4_chunk(const A4Mat& m, size_t row, int K, int j, const A4X& x) {
  const uint2 q = *reinterpret_cast<const uint2*>(m.w + row * (K / 2) + 8 * j);
  const uint32_t qw[2] = {q.x, q.y};
  float acc = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const float qf = (float)((qw[i >> 3] >> (4 * (i & 7))) & 0xfu);
    acc = dm_fma(x.v[i], qf, acc);
  }
  const float s = dm_bf2f(m.scales[row * (K / 32) + (j >> 1)]), b = dm_bf2f(m.biases[row * (K / 32) + (j >> 1)]);
  float p = s * acc;
  return dm_fma(x.sum, b, p);
}

// The two formats behind one pair of kernels: a matrix handle, the gate and up rows' dots over
// one activation row, and NC rows' dots of one matrix.
struct FmtA4 {
  using Mat = A4Mat;
  static __device__ __forceinline__ void dot2(const Mat& wg, const Mat& wu, size_t row, int K, const bf16_t* xr,
                                              int lane, float& g, float& u) {
    float ag = 0.f, au = 0.f;
    for (int j = lane; j < K / 16; j += 64) {
      A4X x;
      x.load(xr, j);
      ag = ag + a4_chunk(wg, row, K, j, x);
      au = au + a4_chunk(wu, row, K, j, x);
    }
    g = dm_wave_sum<64>(ag);
    u = dm_wave_sum<64>(au);
  }
  template <int NC>
  static __device__ __forceinline__ void dotn(const Mat& w, size_t row0, int c0, int O, int K, const bf16_t* xr,
                                              int lane, float (&v)[NC]) {
    float acc[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) acc[c] = 0.f;
    for (int jj = lane; jj < K / 16; jj += 64) {
      A4X x;
      x.load(xr, jj);
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int o = c0 + c < O ? c0 + c : O - 1;
        acc[c] = acc[c] + a4_chunk(w, row0 + o, K, jj, x);
      }
    }
#pragma unroll
    for (int c = 0; c < NC; ++c) v[c] = dm_wave_sum<64>(acc[c]);
  }
};

struct DenseMat {
  const bf16_t* w;  // [rows, K]
};
struct FmtDense {
  using Mat = DenseMat;
  static __device__ __forceinline__ void dot2(const Mat& wg, const Mat& wu, size_t row, int K, const bf16_t* xr,
                                              int lane, float& g, float& u) {
    const bf16_t* const rows[2] = {wg.w + row * K, wu.w + row * K};
    float v[2];
    dense_rows_dot<2, 4>(rows, xr, K, lane, v);
    g = v[0];
    u = v[1];
  }
  template <int NC>
  static __device__ __forceinline__ void dotn(const Mat& w, size_t row0, int c0, int O, int K, const bf16_t* xr,
                                              int lane, float (&v)[NC]) {
    const bf16_t* rows[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int o = c0 + c < O ? c0 + c : O - 1;
      rows[c] = w.w + (row0 + o) * K;
    }
    dense_rows_dot<NC, 1>(rows, xr, K, lane, v);
  }
};

template <class F>
struct A4UpArgs {
  typename F::Mat gate, up;    // routed [E * I, K]
  typename F::Mat sgate, sup;  // shared [I, K]
  const bf16_t* x;       // [T, K]
  const uint32_t* inds;  // [T*k], read unless gates is given
  bf16_t* act;           // [T*k + T, I]
  int T, k, E, I, K;
  const bf16_t* gates;   // [T, E] or null
  uint32_t* inds_out;    // [T*k]
  bf16_t* scores_out;    // [T*k]
};

// grid (ceil(I / 4), T*k + T), 256 threads: a wavefront an output row
template <class F, bool ROUTE>
__global__ __launch_bounds__(256) void moe_up_affine4_kernel(A4UpArgs<F> a) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = blockIdx.y, routed = a.T * a.k;
  int token;
  size_t row0;
  typename F::Mat wg, wu;
  if (r < routed) {
    token = r / a.k;
    uint32_t e;
    if constexpr (ROUTE) {
      __shared__ uint32_t s_inds[16];
      __shared__ bf16_t s_scores[16];
      if (wave == 0) {
        const bf16_t* g = a.gates + (size_t)token * a.E;
        switch (a.E / 64) {
          case 1: router_topk_wave<1>(g, a.k, s_inds, s_scores, nullptr, lane); break;
          case 2: router_topk_wave<2>(g, a.k, s_inds, s_scores, nullptr, lane); break;
          case 4: router_topk_wave<4>(g, a.k, s_inds, s_scores, nullptr, lane); break;
          case 8: router_topk_wave<8>(g, a.k, s_inds, s_scores, nullptr, lane); break;
          default: router_topk_wave<16>(g, a.k, s_inds, s_scores, nullptr, lane); break;
        }
      }
      __syncthreads();
      e = s_inds[r - token * a.k];
      if (blockIdx.x == 0 && r == token * a.k && (int)threadIdx.x < a.k) {
        a.inds_out[r + threadIdx.x] = s_inds[threadIdx.x];
        a.scores_out[r + threadIdx.x] = s_scores[threadIdx.x];
      }
    } else {
      e = a.inds[r];
    }
    row0 = (size_t)min(e, (uint32_t)(a.E - 1)) * a.I;
    wg = a.gate;
    wu = a.up;
  } else {
    token = r - routed;
    row0 = 0;
    wg = a.sgate;
    wu = a.sup;
  }
  const int o = blockIdx.x * 4 + wave;
  if (o >= a.I) return;
  const bf16_t* xr = a.x + (size_t)token * a.K;
  float g, u;
  F::dot2(wg, wu, row0 + o, a.K, xr, lane, g, u);
  if (lane == 0) a.act[(size_t)r * a.I + o] = swiglu_bf16(g, u);
}

template <class F>
struct A4DownArgs {
  typename F::Mat down;   // routed [E * H, I]
  typename F::Mat sdown;  // shared [H, I]
  const bf16_t* act;     // [T*k + T, I]
  const uint32_t* inds;  // [T*k]
  const bf16_t* scores;  // [T*k]
  const bf16_t* egate;   // [T]
  bf16_t* out;           // [T, H]
  int T, k, E, H, I, normalize;
};

constexpr int kA4Cols = 8;

// grid (ceil(H / 8), T), 64 * (k + 1) threads
template <class F>
__global__ __launch_bounds__(64 * (kA4MaxK + 1)) void moe_down_affine4_kernel(A4DownArgs<F> a) {
  const int lane = threadIdx.x & 63, j = threadIdx.x >> 6;  // j: expert slot, k = shared
  const int t = blockIdx.y, k = a.k, c0 = blockIdx.x * kA4Cols;
  __shared__ float yl[kA4MaxK + 1][kA4Cols];
  __shared__ float wj[kA4MaxK];
  __shared__ float gsig;
  const bool shared = j == k;
  const int arow = shared ? a.T * k + t : t * k + j;
  const typename F::Mat w = shared ? a.sdown : a.down;
  const size_t row0 = shared ? 0 : (size_t)min(a.inds[t * k + j], (uint32_t)(a.E - 1)) * a.H;
  // the token's router scores (lane i < k holds score i) and shared-expert gate are asked for
  // ahead of the rows and turned into the combine weights once the rows' sums are made: a
  // loop of loads here, one score a trip to memory, held wavefront 0's rows back by all of them
  const uint16_t score_bits = a.scores[(size_t)t * k + (lane < k ? lane : 0)];
  const uint16_t egate_bits = a.egate[t];
  const bf16_t* xr = a.act + (size_t)arow * a.I;
  float v[kA4Cols];
  F::template dotn<kA4Cols>(w, row0, c0, a.H, a.I, xr, lane, v);
  if (j == 0) {
    // the router weights of this token: denom = ((0+s0)+s1)..., w_j = bf16(s_j / denom)
    float denom = 0.f;
    if (a.normalize) {
#pragma unroll
      for (int i = 0; i < kA4MaxK; ++i)
        if (i < k) denom = dm_rb(dm_bf2f((bf16_t)__builtin_amdgcn_readlane((int)score_bits, i)) + denom);
    }
    if (lane < k) wj[lane] = a.normalize ? dm_rb(dm_bf2f(score_bits) / denom) : dm_bf2f(score_bits);
    if (lane == 0) gsig = dm_sigmoid_bf16(dm_bf2f(egate_bits));
  }
#pragma unroll
  for (int c = 0; c < kA4Cols; ++c)
    if (lane == 0) yl[j][c] = dm_rb(v[c]);  // expert outputs are bf16 in the operator path
  __syncthreads();
  const int col = threadIdx.x;
  if (col < kA4Cols && c0 + col < a.H) {
    float s = 0.f;
    for (int i = 0; i < k; ++i) {
      const float weighted = dm_rb(yl[i][col] * wj[i]);
      s = dm_rb(weighted + s);
    }
    const float gated = dm_rb(gsig * yl[k][col]);
    a.out[(size_t)t * a.H + c0 + col] = dm_f2bf(s + gated);
  }
}

A4Mat mat_of(const ornith_kmatrix& m) {
  return A4Mat{(const uint8_t*)m.d_qs, (const bf16_t*)m.d_scales, (const bf16_t*)m.d_dm};
}
A4Mat mat_of(const ornith_linear& l) {
  return A4Mat{(const uint8_t*)l.d_w, (const bf16_t*)l.d_scales, (const bf16_t*)l.d_biases};
}

}  // namespace

// Whether the two launches cover this block: routed and shared experts all 4-bit affine
// group 32, shapes that chain, at most 8 routed experts a token.
bool moe_affine4_supported(const ornith_moe_weights* w) {
  if (w->ex_dense) return false;
  if (w->ex_gate.kind != ORNITH_AFFINE4_G32 || w->ex_up.kind != ORNITH_AFFINE4_G32 ||
      w->ex_down.kind != ORNITH_AFFINE4_G32)
    return false;
  const ornith_linear* sh[3] = {&w->sh_gate, &w->sh_up, &w->sh_down};
  for (auto* l : sh)
    if (l->mode != ORNITH_LIN_AFFINE4) return false;
  if (w->sh_gate.O != w->ex_gate.O || w->sh_up.O != w->ex_gate.O || w->sh_down.K != w->ex_gate.O) return false;
  if (w->top_k < 1 || w->top_k > kA4MaxK) return false;
  return w->ex_gate.K % 32 == 0 && w->ex_gate.O % 32 == 0;
}

namespace {

template <class F>
int launch_pair(ornith_ctx* ctx, const ornith_moe_weights* w, const typename F::Mat (&m)[6], const void* d_x, int T,
                const uint32_t* d_inds, const void* d_scores, const void* d_egate, void* d_act, void* d_out,
                const void* d_gates) {
  const int E = w->router.O, H = w->router.K, I = w->sh_gate.O, k = w->top_k;
  A4UpArgs<F> u{};
  u.gate = m[0];
  u.up = m[1];
  u.sgate = m[2];
  u.sup = m[3];
  u.x = (const bf16_t*)d_x;
  u.inds = d_inds;
  u.act = (bf16_t*)d_act;
  u.T = T;
  u.k = k;
  u.E = E;
  u.I = I;
  u.K = H;
  u.gates = (const bf16_t*)d_gates;
  u.inds_out = const_cast<uint32_t*>(d_inds);
  u.scores_out = (bf16_t*)const_cast<void*>(d_scores);
  const dim3 ugrid((I + 3) / 4, T * k + T);
  if (d_gates)
    hipLaunchKernelGGL((moe_up_affine4_kernel<F, true>), ugrid, dim3(256), 0, ctx->stream, u);
  else
    hipLaunchKernelGGL((moe_up_affine4_kernel<F, false>), ugrid, dim3(256), 0, ctx->stream, u);
  ORN_LAUNCH_CHECK("moe_up_affine4_kernel");
  A4DownArgs<F> d{};
  d.down = m[4];
  d.sdown = m[5];
  d.act = (const bf16_t*)d_act;
  d.inds = d_inds;
  d.scores = (const bf16_t*)d_scores;
  d.egate = (const bf16_t*)d_egate;
  d.out = (bf16_t*)d_out;
  d.T = T;
  d.k = k;
  d.E = E;
  d.H = H;
  d.I = I;
  d.normalize = w->norm_topk_prob;
  hipLaunchKernelGGL(moe_down_affine4_kernel<F>, dim3((H + kA4Cols - 1) / kA4Cols, T), dim3(64 * (k + 1)), 0,
                     ctx->stream, d);
  ORN_LAUNCH_CHECK("moe_down_affine4_kernel");
  return ORNITH_OK;
}

}  // namespace

// act: scratch bf16 [(T*k + T), I]. With d_gates the up launch makes the routing and stores it
// to d_inds / d_scores (which then are outputs).
int moe_affine4_experts(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_x, int T, const uint32_t* d_inds,
                        const void* d_scores, const void* d_egate, void* d_act, void* d_out, const void* d_gates) {
  const A4Mat m[6] = {mat_of(w->ex_gate), mat_of(w->ex_up), mat_of(w->sh_gate),
                      mat_of(w->sh_up),   mat_of(w->ex_down), mat_of(w->sh_down)};
  return launch_pair<FmtA4>(ctx, w, m, d_x, T, d_inds, d_scores, d_egate, d_act, d_out, d_gates);
}

// The same two launches for dense bf16 experts (the MTP head's block): routed tensors [E, O, K]
// and dense shared-expert linears.
bool moe_dense_supported(const ornith_moe_weights* w) {
  if (!w->ex_dense || !w->d_ex_gate || !w->d_ex_up || !w->d_ex_down) return false;
  const ornith_linear* sh[3] = {&w->sh_gate, &w->sh_up, &w->sh_down};
  for (auto* l : sh)
    if (l->mode != ORNITH_LIN_DENSE || !l->d_w) return false;
  if (w->sh_up.O != w->sh_gate.O || w->sh_down.K != w->sh_gate.O || w->sh_gate.K != w->router.K ||
      w->sh_down.O != w->router.K)
    return false;
  if (w->top_k < 1 || w->top_k > kA4MaxK) return false;
  return w->router.K % 8 == 0 && w->sh_gate.O % 8 == 0;
}

int moe_dense_experts(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_x, int T, const uint32_t* d_inds,
                      const void* d_scores, const void* d_egate, void* d_act, void* d_out, const void* d_gates) {
  const DenseMat m[6] = {{(const bf16_t*)w->d_ex_gate}, {(const bf16_t*)w->d_ex_up},   {(const bf16_t*)w->sh_gate.d_w},
                         {(const bf16_t*)w->sh_up.d_w}, {(const bf16_t*)w->d_ex_down}, {(const bf16_t*)w->sh_down.d_w}};
  return launch_pair<FmtDense>(ctx, w, m, d_x, T, d_inds, d_scores, d_egate, d_act, d_out, d_gates);
}
