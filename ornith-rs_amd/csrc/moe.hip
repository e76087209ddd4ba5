// The sparse MoE block: router softmax + top-k, expert FFNs, shared expert, tail.
//
// Replaces moe::sparse_moe_block and its helpers
// (/root/reference/src/ops/moe.rs:113-134,256-338,548-596,662-741) and the
// kernels router_top_k / moe_combine / swiglu
// (/root/reference/kernels/moe.metal:207-258,568-614,
//  /root/reference/kernels/ornith_elementwise.metal:97-105) and the vendored
// precise softmax (softmax.h:10-98).
//
// Rounding points are the reference's: gates, probabilities, every expert output
// and every step of the tail are bf16; sums inside a kernel are fp32.
#include "moe_device.h"
#include "norm_device.h"
#include "rt.h"

// linear.hip
extern "C" int dense_gather_mv_multi(ornith_ctx* ctx, const void* const* d_ws, int n, int E, int O, int K,
                                     const void* d_x, int x_rows, const uint32_t* d_lhs,
                                     const uint32_t* d_rhs, int rows, void* const* d_ys);
// moe_fused.hip
bool moe_fused_supported(const ornith_moe_weights* w);
bool moe_fused_router(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_x, int T,
                      void* d_gates, void* d_egate, int* rc, const PreNorm* pre);
bool moe_one_launch(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_x, int T, void* d_gates,
                    void* d_egate, uint32_t* d_inds, void* d_scores, void* d_act, void* d_out,
                    const PreNorm* pre, int* rc);
// moe_affine4.hip: the expert half for routed and shared experts in 4-bit affine group 32
bool moe_affine4_supported(const ornith_moe_weights* w);
int moe_affine4_experts(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_x, int T, const uint32_t* d_inds,
                        const void* d_scores, const void* d_egate, void* d_act, void* d_out, const void* d_gates);
// ... and for dense bf16 experts (the MTP head's block)
bool moe_dense_supported(const ornith_moe_weights* w);
int moe_dense_experts(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_x, int T, const uint32_t* d_inds,
                      const void* d_scores, const void* d_egate, void* d_act, void* d_out, const void* d_gates);
int moe_fused_experts(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_x, int T,
                      const uint32_t* d_inds, const void* d_scores, const void* d_egate, void* d_act,
                      void* d_out, int phases, const void* d_gates);

namespace {

// One wavefront per token. Lane l holds gates [l*PER, (l+1)*PER).
//   softmax: fp32 max, e = exp(g - max), lane-sequential sum then butterfly,
//            p = bf16(e * (1/sum))
//   top-k:   k rounds of (value, then larger index) selection; round r -> slot k-1-r
// Also writes the gather index lists the expert mat-vecs use:
//   lhs_tok[t*k+j] = t (row of x), lhs_row[t*k+j] = t*k+j (row of act).
template <int PER>
__global__ __launch_bounds__(64) void router_topk_kernel(const bf16_t* gates, int E, int k,
                                                         uint32_t* inds, bf16_t* scores,
                                                         bf16_t* probs, uint32_t* lhs_tok,
                                                         uint32_t* lhs_row) {
  const int t = blockIdx.x, lane = threadIdx.x;
  router_topk_wave<PER>(gates + (size_t)t * E, k, inds + (size_t)t * k, scores + (size_t)t * k,
                        probs ? probs + (size_t)t * E : nullptr, lane);
  if (lane < k) {
    if (lhs_tok) lhs_tok[t * k + lane] = t;
    if (lhs_row) lhs_row[t * k + lane] = t * k + lane;
  }
}

// V consecutive elements a thread (V = 8: 16-byte loads and stores; V = 1 for odd sizes)
template <int V>
struct BfPack;
template <>
struct BfPack<8> { typedef unsigned int type __attribute__((ext_vector_type(4))); };
template <>
struct BfPack<1> { typedef bf16_t type; };
template <int V>
__device__ __forceinline__ float bf_get(const typename BfPack<V>::type& p, int i) {
  if constexpr (V == 1) return dm_bf2f(p);
  else return (i & 1) ? dm_bf2f_hi(p[i >> 1]) : dm_bf2f_lo(p[i >> 1]);
}
template <int V>
__device__ __forceinline__ void bf_put(typename BfPack<V>::type& p, int i, float v) {
  if constexpr (V == 1) p = dm_f2bf(v);
  else p[i >> 1] = (i & 1) ? (p[i >> 1] & 0xffffu) | ((uint32_t)dm_f2bf(v) << 16) : (uint32_t)dm_f2bf(v);
}

template <int V>
__global__ void swiglu_kernel(const bf16_t* gate, const bf16_t* up, bf16_t* out, int64_t n,
                              const bf16_t* gate2 = nullptr, const bf16_t* up2 = nullptr,
                              bf16_t* out2 = nullptr, int64_t n2 = 0) {
  typedef typename BfPack<V>::type P;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  // a second, independent range follows the first (two activations in one launch)
  if (i >= n / V) {
    i -= n / V;
    if (i >= n2 / V) return;
    gate = gate2;
    up = up2;
    out = out2;
  }
  const P g8 = reinterpret_cast<const P*>(gate)[i], u8 = reinterpret_cast<const P*>(up)[i];
  P o8;
#pragma unroll
  for (int e = 0; e < V; ++e) {
    const float g = bf_get<V>(g8, e);
    const float s = dm_rb(g * dm_sigmoid_bf16(g));
    bf_put<V>(o8, e, s * bf_get<V>(u8, e));
  }
  reinterpret_cast<P*>(out)[i] = o8;
}

// one thread per V output elements of a token; j ascends, every step rounds to bf16
template <int V>
__global__ void moe_combine_kernel(const bf16_t* scores, const bf16_t* y, const bf16_t* gate,
                                   const bf16_t* shared, bf16_t* out, int T, int k, int dim,
                                   int normalize) {
  typedef typename BfPack<V>::type P;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int per_row = dim / V;
  if (idx >= (int64_t)T * per_row) return;
  const int t = (int)(idx / per_row), c = (int)(idx - (int64_t)t * per_row) * V;
  const bf16_t* s = scores + (size_t)t * k;
  float denom = 0.f;
  if (normalize)
    for (int j = 0; j < k; ++j) denom = dm_rb(dm_bf2f(s[j]) + denom);
  float acc[V];
#pragma unroll
  for (int e = 0; e < V; ++e) acc[e] = 0.f;
  for (int j = 0; j < k; ++j) {
    const float w = normalize ? dm_rb(dm_bf2f(s[j]) / denom) : dm_bf2f(s[j]);
    const P yj = *reinterpret_cast<const P*>(y + ((size_t)t * k + j) * dim + c);
#pragma unroll
    for (int e = 0; e < V; ++e) {
      const float weighted = dm_rb(bf_get<V>(yj, e) * w);
      acc[e] = dm_rb(weighted + acc[e]);
    }
  }
  const float g = dm_sigmoid_bf16(dm_bf2f(gate[t]));
  const P sh = *reinterpret_cast<const P*>(shared + (size_t)t * dim + c);
  P o;
#pragma unroll
  for (int e = 0; e < V; ++e) {
    const float gated = dm_rb(g * bf_get<V>(sh, e));
    bf_put<V>(o, e, acc[e] + gated);
  }
  *reinterpret_cast<P*>(out + (size_t)t * dim + c) = o;
}

int launch_router(ornith_ctx* ctx, const bf16_t* gates, int T, int E, int k, uint32_t* inds,
                  bf16_t* scores, bf16_t* probs, uint32_t* lhs_tok, uint32_t* lhs_row) {
#define ROUTER_CASE(P)                                                                       \
  case P:                                                                                    \
    hipLaunchKernelGGL(router_topk_kernel<P>, dim3(T), dim3(64), 0, ctx->stream, gates, E, k, \
                       inds, scores, probs, lhs_tok, lhs_row);                               \
    break;
  switch (E / 64) {
    ROUTER_CASE(1)
    ROUTER_CASE(2)
    ROUTER_CASE(4)
    ROUTER_CASE(8)
    ROUTER_CASE(16)
    default:
      return ornith_fail(ORNITH_ERR_UNSUPPORTED, "router_topk: E=%d (need 64,128,256,512,1024)", E);
  }
#undef ROUTER_CASE
  ORN_LAUNCH_CHECK("router_topk_kernel");
  return ORNITH_OK;
}

// Prefill widths: the same block with every projection as a matrix-core GEMM and the routed
// experts as three expert-grouped GEMMs over one sorted pair list
// (/root/reference/src/ops/moe.rs:662-741 at T above the exact window; gather_qmm_t).
int moe_block_prefill(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_x, int T, void* d_out) {
  const int E = w->router.O, H = w->router.K, I = w->ex_gate.O, k = w->top_k, SI = w->sh_gate.O;
  const int pairs = T * k;
  const size_t plan_bytes = ornith_kq_gather_plan_bytes(pairs, E);
  const size_t need = 2 * ((size_t)T * E + (size_t)T * SI * 3 + (size_t)T * H + T + (size_t)pairs * (3 * I + H) +
                           (size_t)pairs) + 4 * (size_t)pairs + plan_bytes + 24 * 256;
  void* base = nullptr;
  int rc = ornith_scratch(ctx, need, &base);
  if (rc) return rc;
  ScratchCursor sc(base);
  bf16_t* gates = sc.take<bf16_t>((size_t)T * E);
  uint32_t* inds = sc.take<uint32_t>(pairs);
  bf16_t* scores = sc.take<bf16_t>(pairs);
  bf16_t* sg = sc.take<bf16_t>((size_t)T * SI);
  bf16_t* su = sc.take<bf16_t>((size_t)T * SI);
  bf16_t* sact = sc.take<bf16_t>((size_t)T * SI);
  bf16_t* sy = sc.take<bf16_t>((size_t)T * H);
  bf16_t* eg = sc.take<bf16_t>(T);
  bf16_t* xg = sc.take<bf16_t>((size_t)pairs * I);
  bf16_t* xu = sc.take<bf16_t>((size_t)pairs * I);
  bf16_t* act = sc.take<bf16_t>((size_t)pairs * I);
  bf16_t* y = sc.take<bf16_t>((size_t)pairs * H);
  void* plan = sc.take<char>(plan_bytes);
#define TRY(e)          \
  do {                  \
    rc = (e);           \
    if (rc) return rc;  \
  } while (0)
  {
    // the router and the shared expert's gate / up read the same rows: one launch where their
    // formats allow (alone, the 256-column router is 64 workgroups)
    const ornith_linear* in3[3] = {&w->router, &w->sh_gate, &w->sh_up};
    void* y3[3] = {gates, sg, su};
    TRY(ornith_linear_matmul_multi(ctx, in3, 3, d_x, T, y3));
  }
  TRY(ornith_linear_matmul(ctx, &w->sh_egate, d_x, T, eg));
  TRY(launch_router(ctx, gates, T, E, k, inds, scores, nullptr, nullptr, nullptr));
  TRY(ornith_swiglu(ctx, sg, su, (int64_t)T * SI, sact));
  TRY(ornith_linear_matmul(ctx, &w->sh_down, sact, T, sy));
  TRY(ornith_kq_gather_matmul(ctx, &w->ex_gate, d_x, inds, pairs, k, 1, plan, 1, xg));
  TRY(ornith_kq_gather_matmul(ctx, &w->ex_up, d_x, inds, pairs, k, 1, plan, 0, xu));
  TRY(ornith_swiglu(ctx, xg, xu, (int64_t)pairs * I, act));
  TRY(ornith_kq_gather_matmul(ctx, &w->ex_down, act, inds, pairs, k, 0, plan, 0, y));
  TRY(ornith_moe_combine(ctx, scores, y, eg, sy, T, k, H, w->norm_topk_prob, d_out));
#undef TRY
  return ORNITH_OK;
}

}  // namespace

extern "C" {

int ornith_router_topk(ornith_ctx* ctx, const void* d_gates, int T, int E, int k, uint32_t* d_inds,
                       void* d_scores, void* d_probs) {
  ORN_REQUIRE(ctx && d_gates && d_inds && d_scores, "router_topk: null argument");
  ORN_REQUIRE(T >= 1 && E % 64 == 0 && k >= 1 && k <= 16 && k <= E, "router_topk: T=%d E=%d k=%d",
              T, E, k);
  return launch_router(ctx, (const bf16_t*)d_gates, T, E, k, d_inds, (bf16_t*)d_scores,
                       (bf16_t*)d_probs, nullptr, nullptr);
}

int ornith_swiglu(ornith_ctx* ctx, const void* d_gate, const void* d_up, int64_t n, void* d_out) {
  ORN_REQUIRE(ctx && d_gate && d_up && d_out && n >= 0, "swiglu: bad argument");
  if (n == 0) return ORNITH_OK;
  // 16-byte pieces when the size and the addresses allow
  if (n % 8 == 0 && (((uintptr_t)d_gate | (uintptr_t)d_up | (uintptr_t)d_out) & 15) == 0)
    hipLaunchKernelGGL(swiglu_kernel<8>, dim3((unsigned)((n / 8 + 255) / 256)), dim3(256), 0, ctx->stream,
                       (const bf16_t*)d_gate, (const bf16_t*)d_up, (bf16_t*)d_out, n);
  else
    hipLaunchKernelGGL(swiglu_kernel<1>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, ctx->stream,
                       (const bf16_t*)d_gate, (const bf16_t*)d_up, (bf16_t*)d_out, n);
  ORN_LAUNCH_CHECK("swiglu_kernel");
  return ORNITH_OK;
}

}  // extern "C"

// swiglu over two independent ranges in one launch
static int swiglu_pair(ornith_ctx* ctx, const void* g1, const void* u1, int64_t n1, void* o1, const void* g2,
                       const void* u2, int64_t n2, void* o2) {
  ORN_REQUIRE(g1 && u1 && o1 && g2 && u2 && o2 && n1 >= 0 && n2 >= 0, "swiglu_pair: bad argument");
  if (n1 + n2 == 0) return ORNITH_OK;
  const uintptr_t bits = (uintptr_t)g1 | (uintptr_t)u1 | (uintptr_t)o1 | (uintptr_t)g2 | (uintptr_t)u2 | (uintptr_t)o2;
  if (n1 % 8 == 0 && n2 % 8 == 0 && (bits & 15) == 0)
    hipLaunchKernelGGL(swiglu_kernel<8>, dim3((unsigned)(((n1 + n2) / 8 + 255) / 256)), dim3(256), 0, ctx->stream,
                       (const bf16_t*)g1, (const bf16_t*)u1, (bf16_t*)o1, n1, (const bf16_t*)g2,
                       (const bf16_t*)u2, (bf16_t*)o2, n2);
  else
    hipLaunchKernelGGL(swiglu_kernel<1>, dim3((unsigned)((n1 + n2 + 255) / 256)), dim3(256), 0, ctx->stream,
                       (const bf16_t*)g1, (const bf16_t*)u1, (bf16_t*)o1, n1, (const bf16_t*)g2,
                       (const bf16_t*)u2, (bf16_t*)o2, n2);
  ORN_LAUNCH_CHECK("swiglu_kernel<pair>");
  return ORNITH_OK;
}

extern "C" {

int ornith_moe_combine(ornith_ctx* ctx, const void* d_scores, const void* d_y, const void* d_gate,
                       const void* d_shared, int T, int k, int dim, int normalize, void* d_out) {
  ORN_REQUIRE(ctx && d_scores && d_y && d_gate && d_shared && d_out, "moe_combine: null argument");
  ORN_REQUIRE(T >= 1 && k >= 1 && dim >= 1, "moe_combine: T=%d k=%d dim=%d", T, k, dim);
  const int64_t n = (int64_t)T * dim;
  if (dim % 8 == 0 && (((uintptr_t)d_y | (uintptr_t)d_shared | (uintptr_t)d_out) & 15) == 0)
    hipLaunchKernelGGL(moe_combine_kernel<8>, dim3((unsigned)((n / 8 + 255) / 256)), dim3(256), 0,
                       ctx->stream, (const bf16_t*)d_scores, (const bf16_t*)d_y, (const bf16_t*)d_gate,
                       (const bf16_t*)d_shared, (bf16_t*)d_out, T, k, dim, normalize);
  else
    hipLaunchKernelGGL(moe_combine_kernel<1>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                       ctx->stream, (const bf16_t*)d_scores, (const bf16_t*)d_y, (const bf16_t*)d_gate,
                       (const bf16_t*)d_shared, (bf16_t*)d_out, T, k, dim, normalize);
  ORN_LAUNCH_CHECK("moe_combine_kernel");
  return ORNITH_OK;
}

// The block. With `pre`, x is rms_norm(pre->res + pre->y): made inside the router launch when
// the fused kernels cover the shapes (d_x then is where the normed rows get stored, and read
// back by the expert kernels), by a separate add_rms_norm otherwise.
static int moe_block_impl(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_x, int T,
                          void* d_out, uint32_t* d_inds_out, void* d_scores_out, const PreNorm* pre) {
  ORN_REQUIRE(ctx && w && d_x && d_out, "moe_block: null argument");
  const int E = w->router.O, H = w->router.K, I = w->ex_gate.O, k = w->top_k;
  ORN_REQUIRE(T >= 1 && T <= 8192, "moe_block: T=%d", T);
  ORN_REQUIRE(k >= 1 && k <= 16 && k <= E, "moe_block: top_k=%d of %d", k, E);
  ORN_REQUIRE(w->ex_gate.E == E && w->ex_up.E == E && w->ex_down.E == E,
              "moe_block: expert tensors carry %d/%d/%d experts, router has %d", w->ex_gate.E,
              w->ex_up.E, w->ex_down.E, E);
  ORN_REQUIRE(w->ex_gate.K == H && w->ex_up.K == H && w->ex_up.O == I && w->ex_down.K == I &&
                  w->ex_down.O == H,
              "moe_block: expert shapes do not chain (H=%d I=%d)", H, I);
  ORN_REQUIRE(w->sh_gate.K == H && w->sh_up.K == H && w->sh_up.O == w->sh_gate.O &&
                  w->sh_down.K == w->sh_gate.O && w->sh_down.O == H && w->sh_egate.K == H &&
                  w->sh_egate.O == 1,
              "moe_block: shared expert shapes do not chain");
  const int SI = w->sh_gate.O;
  const bool pre_in_kernel = pre && T <= 4 && H == kPreN && ornith_option_fuse_norm() &&
                             ornith_option_fuse_moe() && moe_fused_supported(w) &&
                             w->router.mode == ORNITH_LIN_KQUANT;
  if (pre && !pre_in_kernel) {
    int rcn = ornith_add_rms_norm(ctx, pre->res, pre->y, pre->w, T, H, pre->eps, pre->h_out, pre->normed_out);
    if (rcn) return rcn;
    pre = nullptr;
  }
  const bool ex_affine4 = !w->ex_dense && w->ex_gate.kind == ORNITH_AFFINE4_G32;
  if (ex_affine4)
    ORN_REQUIRE(w->ex_up.kind == ORNITH_AFFINE4_G32 && w->ex_down.kind == ORNITH_AFFINE4_G32,
                "moe_block: the three expert stacks must share the 4-bit affine format");
  if (T >= kPrefillRows && !w->ex_dense && !ex_affine4) {
    ORN_REQUIRE(!d_inds_out && !d_scores_out, "moe_block: index outputs are a decode-width feature");
    return moe_block_prefill(ctx, w, d_x, T, d_out);
  }
  if (T > 64) {
    // dense and 4-bit affine experts have no prefill-width form: the operator path takes the
    // rows in blocks of 64 (rows are independent of each other, so the result is the same)
    for (int t0 = 0; t0 < T; t0 += 64) {
      const int n = T - t0 < 64 ? T - t0 : 64;
      const int rcb = moe_block_impl(ctx, w, static_cast<const bf16_t*>(d_x) + (size_t)t0 * H, n,
                                     static_cast<bf16_t*>(d_out) + (size_t)t0 * H,
                                     d_inds_out ? d_inds_out + (size_t)t0 * k : nullptr,
                                     d_scores_out ? static_cast<bf16_t*>(d_scores_out) + (size_t)t0 * k : nullptr, nullptr);
      if (rcb) return rcb;
    }
    return ORNITH_OK;
  }

  const size_t need = 2 * ((size_t)T * E * 2 + (size_t)T * SI * 3 + (size_t)T * H + T +
                           (size_t)(T * k + T) * (2 * I + I + SI + H + 1)) +
                      4 * (size_t)T * k * 3 + 64 * 256;
  void* base = nullptr;
  int rc = ornith_scratch(ctx, need, &base);
  if (rc) return rc;
  ScratchCursor sc(base);
  bf16_t* gates = sc.take<bf16_t>((size_t)T * E);
  uint32_t* inds = sc.take<uint32_t>((size_t)T * k);
  bf16_t* scores = sc.take<bf16_t>((size_t)T * k);
  uint32_t* lhs_tok = sc.take<uint32_t>((size_t)T * k);
  uint32_t* lhs_row = sc.take<uint32_t>((size_t)T * k);
  bf16_t* sg = sc.take<bf16_t>((size_t)T * SI);
  bf16_t* su = sc.take<bf16_t>((size_t)T * SI);
  bf16_t* sact = sc.take<bf16_t>((size_t)T * SI);
  bf16_t* sy = sc.take<bf16_t>((size_t)T * H);
  bf16_t* eg = sc.take<bf16_t>((size_t)T);
  bf16_t* xg = sc.take<bf16_t>((size_t)T * k * I);
  bf16_t* xu = sc.take<bf16_t>((size_t)T * k * I);
  bf16_t* act = sc.take<bf16_t>((size_t)(T * k + T) * (I > SI ? I : SI));
  bf16_t* y = sc.take<bf16_t>((size_t)T * k * H);

#define TRY(e)          \
  do {                  \
    rc = (e);           \
    if (rc) return rc;  \
  } while (0)
  if (ornith_option_fuse_moe() && moe_fused_supported(w)) {
    int rrc = ORNITH_OK;
    // router, up and down as one launch where the shapes are in its family
    if (moe_one_launch(ctx, w, d_x, T, gates, eg, inds, scores, act, d_out, pre, &rrc)) {
      if (rrc) return rrc;
      if (d_inds_out)
        ORN_HIP(hipMemcpyAsync(d_inds_out, inds, 4 * (size_t)T * k, hipMemcpyDeviceToDevice, ctx->stream));
      if (d_scores_out)
        ORN_HIP(hipMemcpyAsync(d_scores_out, scores, 2 * (size_t)T * k, hipMemcpyDeviceToDevice, ctx->stream));
      return ORNITH_OK;
    }
    // gates + shared-expert gate, softmax + top-k, then the two expert kernels
    if (moe_fused_router(ctx, w, d_x, T, gates, eg, &rrc, pre)) {
      if (rrc) return rrc;
    } else {
      if (pre) TRY(ornith_add_rms_norm(ctx, pre->res, pre->y, pre->w, T, H, pre->eps, pre->h_out, pre->normed_out));
      TRY(ornith_linear_matmul(ctx, &w->router, d_x, T, gates));
      TRY(ornith_linear_matmul(ctx, &w->sh_egate, d_x, T, eg));
    }
    // softmax + top-k ride in the head of the up kernel (the reference folds its routing
    // tail the same way, ORNITH_FUSE_MOE_TAIL); E must be one of the wavefront layouts
    const bool topk_in_up = E % 64 == 0 && E <= 1024 && ((E / 64) & (E / 64 - 1)) == 0 && k <= 16;
    if (!topk_in_up) TRY(launch_router(ctx, gates, T, E, k, inds, scores, nullptr, nullptr, nullptr));
    TRY(moe_fused_experts(ctx, w, d_x, T, inds, scores, eg, act, d_out, 3, topk_in_up ? gates : nullptr));
    if (d_inds_out)
      ORN_HIP(hipMemcpyAsync(d_inds_out, inds, 4 * (size_t)T * k, hipMemcpyDeviceToDevice,
                             ctx->stream));
    if (d_scores_out)
      ORN_HIP(hipMemcpyAsync(d_scores_out, scores, 2 * (size_t)T * k, hipMemcpyDeviceToDevice,
                             ctx->stream));
    return ORNITH_OK;
  }
  const bool pair_a4 = ex_affine4 && moe_affine4_supported(w), pair_dense = w->ex_dense && moe_dense_supported(w);
  if (ornith_option_fuse_moe() && (pair_a4 || pair_dense)) {
    // the published artifact's block, and the MTP head's dense one, in three launches: router +
    // shared-expert gate (one launch when their formats match), then the two expert launches of
    // moe_affine4.hip, the softmax + top-k in the head of the first where the expert count allows
    const ornith_linear* in2[2] = {&w->router, &w->sh_egate};
    void* out2[2] = {gates, eg};
    TRY(ornith_linear_matmul_multi(ctx, in2, 2, d_x, T, out2));
    const bool topk_in_up = E % 64 == 0 && E <= 1024 && ((E / 64) & (E / 64 - 1)) == 0 && k <= 16;
    if (!topk_in_up) TRY(launch_router(ctx, gates, T, E, k, inds, scores, nullptr, nullptr, nullptr));
    if (pair_a4)
      TRY(moe_affine4_experts(ctx, w, d_x, T, inds, scores, eg, act, d_out, topk_in_up ? gates : nullptr));
    else
      TRY(moe_dense_experts(ctx, w, d_x, T, inds, scores, eg, act, d_out, topk_in_up ? gates : nullptr));
    if (d_inds_out)
      ORN_HIP(hipMemcpyAsync(d_inds_out, inds, 4 * (size_t)T * k, hipMemcpyDeviceToDevice, ctx->stream));
    if (d_scores_out)
      ORN_HIP(hipMemcpyAsync(d_scores_out, scores, 2 * (size_t)T * k, hipMemcpyDeviceToDevice, ctx->stream));
    return ORNITH_OK;
  }
  {
    // the four projections of the block's input: one launch when their formats allow
    const ornith_linear* in4[4] = {&w->router, &w->sh_gate, &w->sh_up, &w->sh_egate};
    void* out4[4] = {gates, sg, su, eg};
    TRY(ornith_linear_matmul_multi(ctx, in4, 4, d_x, T, out4));
  }
  TRY(launch_router(ctx, gates, T, E, k, inds, scores, nullptr, lhs_tok, lhs_row));
  if (w->ex_dense) {
    ORN_REQUIRE(w->d_ex_gate && w->d_ex_up && w->d_ex_down, "moe_block: dense expert tensor missing");
    const void* gu[2] = {w->d_ex_gate, w->d_ex_up};
    void* xgu[2] = {xg, xu};
    TRY(dense_gather_mv_multi(ctx, gu, 2, E, I, H, d_x, T, lhs_tok, inds, T * k, xgu));
    // the shared expert's activation and the routed experts' in one launch
    TRY(swiglu_pair(ctx, sg, su, (int64_t)T * SI, sact, xg, xu, (int64_t)T * k * I, act));
    TRY(ornith_linear_matmul(ctx, &w->sh_down, sact, T, sy));
    TRY(ornith_dense_gather_mv(ctx, w->d_ex_down, E, H, I, act, T * k, lhs_row, inds, T * k, y));
  } else if (ex_affine4) {
    // quantized::gather_qmv over the stacked 4-bit affine experts (src/ops/quantized.rs:531-589)
    TRY(ornith_affine4_gather_qmv(ctx, w->ex_gate.d_qs, w->ex_gate.d_scales, w->ex_gate.d_dm, E, I, H, d_x, T,
                                  lhs_tok, inds, T * k, xg));
    TRY(ornith_affine4_gather_qmv(ctx, w->ex_up.d_qs, w->ex_up.d_scales, w->ex_up.d_dm, E, I, H, d_x, T, lhs_tok,
                                  inds, T * k, xu));
    TRY(swiglu_pair(ctx, sg, su, (int64_t)T * SI, sact, xg, xu, (int64_t)T * k * I, act));
    TRY(ornith_linear_matmul(ctx, &w->sh_down, sact, T, sy));
    TRY(ornith_affine4_gather_qmv(ctx, w->ex_down.d_qs, w->ex_down.d_scales, w->ex_down.d_dm, E, H, I, act, T * k,
                                  lhs_row, inds, T * k, y));
  } else {
    TRY(ornith_kq_gather_qmv(ctx, &w->ex_gate, d_x, ORNITH_BF16, T, lhs_tok, inds, T * k, xg,
                             ORNITH_BF16));
    TRY(ornith_kq_gather_qmv(ctx, &w->ex_up, d_x, ORNITH_BF16, T, lhs_tok, inds, T * k, xu,
                             ORNITH_BF16));
    TRY(swiglu_pair(ctx, sg, su, (int64_t)T * SI, sact, xg, xu, (int64_t)T * k * I, act));
    TRY(ornith_linear_matmul(ctx, &w->sh_down, sact, T, sy));
    TRY(ornith_kq_gather_qmv(ctx, &w->ex_down, act, ORNITH_BF16, T * k, lhs_row, inds, T * k, y,
                             ORNITH_BF16));
  }
  TRY(ornith_moe_combine(ctx, scores, y, eg, sy, T, k, H, w->norm_topk_prob, d_out));
  if (d_inds_out)
    ORN_HIP(hipMemcpyAsync(d_inds_out, inds, 4 * (size_t)T * k, hipMemcpyDeviceToDevice,
                           ctx->stream));
  if (d_scores_out)
    ORN_HIP(hipMemcpyAsync(d_scores_out, scores, 2 * (size_t)T * k, hipMemcpyDeviceToDevice,
                           ctx->stream));
#undef TRY
  return ORNITH_OK;
}

int ornith_moe_block(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_x, int T,
                     void* d_out, uint32_t* d_inds_out, void* d_scores_out) {
  return moe_block_impl(ctx, w, d_x, T, d_out, d_inds_out, d_scores_out, nullptr);
}

int ornith_add_rms_moe_block(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_res,
                             const void* d_y, const void* d_wnorm, float eps, int T, void* d_h_out,
                             void* d_normed_out, void* d_out) {
  ORN_REQUIRE(d_res && d_y && d_wnorm && d_h_out && d_normed_out, "add_rms_moe_block: null argument");
  const PreNorm pre{(const bf16_t*)d_res, (const bf16_t*)d_y, (const bf16_t*)d_wnorm, (bf16_t*)d_h_out,
                    (bf16_t*)d_normed_out, eps};
  return moe_block_impl(ctx, w, d_normed_out, T, d_out, nullptr, nullptr, &pre);
}

}  // extern "C"
