// The expert half of the MoE block in two launches.
//
// moe_up:   for every (token, routed expert) pair and for the shared expert:
//           gate and up projections over the same activation registers, then
//           swiglu -> act. One launch replaces two gather mat-vecs, two plain
//           mat-vecs and two swiglu launches.
// moe_down: for every (token, column group): the k routed down projections and the
//           shared one run in k+1 wavefronts of one workgroup, meet in LDS, and the
//           block's tail (weights from the router scores, bf16 accumulation in slot
//           order, sigmoid-gated shared expert) writes the block's output. One launch
//           replaces a gather mat-vec, a plain mat-vec and the combine kernel.
//
// Same arithmetic, in the same order, as the separate operators
// (/root/reference/src/ops/moe.rs:256-338,548-596,
// /root/reference/kernels/moe.metal:207-244,
// /root/reference/kernels/ornith_elementwise.metal:97-105): only the launch structure
// changes, so the two paths agree bit for bit (the reference checks its own fusions
// the same way, ORNITH_FUSE_MOE_TAIL).
//
// These two kernels are the expert gather-GEMV: per distinct expert they stream
// 2 x I x K Q4_K codes and H x I Q6_K codes once, with nothing but the activations
// and index lists read besides.
#include "kq_device.h"
#include "rt.h"

namespace {

struct KqPtr {
  const uint8_t* qs;
  const uint8_t* scales;
  const uint16_t* dm;
};

struct UpArgs {
  KqPtr gate, up;        // routed [E, I, K]
  KqPtr sgate, sup;      // shared [I, K]
  const bf16_t* x;       // [T, K]
  const uint32_t* inds;  // [T*k]
  bf16_t* act;           // [T*k + T, I]
  int T, k, E, I, K, iters;
};

__device__ __forceinline__ bf16_t swiglu_bf16(float g, float u) {
  const float gb = dm_rb(g), ub = dm_rb(u);
  const float s = dm_rb(gb * dm_sigmoid_bf16(gb));
  return dm_f2bf(s * ub);
}

// grid (ceil(I / rows_per_block), T*k + T), 256 threads
template <int KIND, int LPR>
__global__ __launch_bounds__(256) void moe_up_kernel(UpArgs a) {
  using KL = KqLane<KIND, 1>;
  constexpr int RPW = 64 / LPR;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int slot = lane / LPR, c = lane % LPR;
  const int nb = a.K >> 8;
  const int r = blockIdx.y;
  const int routed = a.T * a.k;
  int token;
  int64_t row0;
  KqPtr wg, wu;
  if (r < routed) {
    token = r / a.k;
    row0 = (int64_t)min(a.inds[r], (uint32_t)(a.E - 1)) * a.I;
    wg = a.gate;
    wu = a.up;
  } else {
    token = r - routed;
    row0 = 0;
    wg = a.sgate;
    wu = a.sup;
  }
  const void* xrow[1] = {a.x + (size_t)token * a.K};
  typename KL::Lane L;
  L.template load_x<false>(xrow, c);

  const int rows_per_wave = RPW * a.iters;
  const int base = (blockIdx.x * 4 + wave) * rows_per_wave;
#pragma unroll 2
  for (int it = 0; it < a.iters; ++it) {
    const int o = base + it * RPW + slot;
    const bool valid = o < a.I;
    const int64_t row = row0 + (valid ? o : a.I - 1);
    const typename KL::Row rg = KL::load(wg.qs, wg.scales, wg.dm, row, nb, L);
    const typename KL::Row ru = KL::load(wu.qs, wu.scales, wu.dm, row, nb, L);
    float ag[1] = {0.f}, au[1] = {0.f};
    KL::accumulate(rg, L, ag);
    KL::accumulate(ru, L, au);
    const float g = dm_wave_sum<LPR>(ag[0]);
    const float u = dm_wave_sum<LPR>(au[0]);
    if (c == 0 && valid) a.act[(size_t)r * a.I + o] = swiglu_bf16(g, u);
  }
}

struct DownArgs {
  KqPtr down;   // routed [E, H, I]
  KqPtr sdown;  // shared [H, I]
  const bf16_t* act;     // [T*k + T, I]
  const uint32_t* inds;  // [T*k]
  const bf16_t* scores;  // [T*k]
  const bf16_t* egate;   // [T]
  bf16_t* out;           // [T, H]
  int T, k, E, H, I, iters, normalize;
};

constexpr int kMaxK = 8;
constexpr int kMaxCols = 64 * 4;  // RPW * iters upper bound (LPR >= 4, iters <= 16)

// grid (ceil(H / (RPW * iters)), T), 64 * (k + 1) threads
template <int KIND, int LPR>
__global__ __launch_bounds__(64 * (kMaxK + 1)) void moe_down_kernel(DownArgs a) {
  using KL = KqLane<KIND, 1>;
  constexpr int RPW = 64 / LPR;
  const int lane = threadIdx.x & 63, j = threadIdx.x >> 6;  // j: expert slot, k = shared
  const int slot = lane / LPR, c = lane % LPR;
  const int nb = a.I >> 8;
  const int t = blockIdx.y, k = a.k;
  const int cols = RPW * a.iters, c0 = blockIdx.x * cols;

  __shared__ float yl[kMaxK + 1][kMaxCols];
  __shared__ float wj[kMaxK];
  __shared__ float gsig;

  if (j == 0) {
    // the router weights of this token: denom = ((0+s0)+s1)..., w_j = bf16(s_j / denom)
    const bf16_t* s = a.scores + (size_t)t * k;
    float denom = 0.f;
    if (a.normalize)
      for (int i = 0; i < k; ++i) denom = dm_rb(dm_bf2f(s[i]) + denom);
    if (lane < k) wj[lane] = a.normalize ? dm_rb(dm_bf2f(s[lane]) / denom) : dm_bf2f(s[lane]);
    if (lane == 0) gsig = dm_sigmoid_bf16(dm_bf2f(a.egate[t]));
  }

  const bool shared = j == k;
  const int arow = shared ? a.T * k + t : t * k + j;
  const KqPtr w = shared ? a.sdown : a.down;
  const int64_t row0 = shared ? 0 : (int64_t)min(a.inds[t * k + j], (uint32_t)(a.E - 1)) * a.H;
  const void* xrow[1] = {a.act + (size_t)arow * a.I};
  typename KL::Lane L;
  L.template load_x<false>(xrow, c);
#pragma unroll 2
  for (int it = 0; it < a.iters; ++it) {
    const int col = it * RPW + slot;
    const int o = c0 + col;
    const bool valid = o < a.H;
    const typename KL::Row r = KL::load(w.qs, w.scales, w.dm, row0 + (valid ? o : a.H - 1), nb, L);
    float acc[1] = {0.f};
    KL::accumulate(r, L, acc);
    const float v = dm_wave_sum<LPR>(acc[0]);
    if (c == 0) yl[j][col] = dm_rb(v);  // expert outputs are bf16 in the unfused path
  }
  __syncthreads();
  const int col = threadIdx.x;
  if (col < cols && c0 + col < a.H) {
    float acc = 0.f;
    for (int i = 0; i < k; ++i) {
      const float weighted = dm_rb(yl[i][col] * wj[i]);
      acc = dm_rb(weighted + acc);
    }
    const float gated = dm_rb(gsig * yl[k][col]);
    a.out[(size_t)t * a.H + c0 + col] = dm_f2bf(acc + gated);
  }
}

KqPtr ptr_of(const ornith_kmatrix& m) {
  return KqPtr{(const uint8_t*)m.d_qs, (const uint8_t*)m.d_scales, (const uint16_t*)m.d_dm};
}

int chunks_of(const ornith_kmatrix& m) { return (m.K >> 8) * (m.kind == ORNITH_Q4K ? 8 : 4); }

}  // namespace

// Whether the two fused kernels cover this block's shapes and formats.
bool moe_fused_supported(const ornith_moe_weights* w) {
  if (w->ex_dense) return false;
  const ornith_linear* sh[3] = {&w->sh_gate, &w->sh_up, &w->sh_down};
  for (auto* l : sh)
    if (l->mode != ORNITH_LIN_KQUANT) return false;
  if (w->ex_up.kind != w->ex_gate.kind || w->sh_gate.km.kind != w->ex_gate.kind ||
      w->sh_up.km.kind != w->ex_gate.kind || w->sh_down.km.kind != w->ex_down.kind)
    return false;
  if (w->sh_gate.O != w->ex_gate.O || w->sh_up.O != w->ex_gate.O) return false;
  if (w->top_k > kMaxK) return false;
  const int cu = chunks_of(w->ex_gate), cd = chunks_of(w->ex_down);
  auto ok = [](int n) { return n == 4 || n == 8 || n == 16 || n == 32 || n == 64; };
  return ok(cu) && ok(cd);
}

// act: scratch bf16 [(T*k + T), I]
int moe_fused_experts(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_x, int T,
                      const uint32_t* d_inds, const void* d_scores, const void* d_egate, void* d_act,
                      void* d_out) {
  const int E = w->router.O, H = w->router.K, I = w->ex_gate.O, k = w->top_k;
  {
    UpArgs a{};
    a.gate = ptr_of(w->ex_gate);
    a.up = ptr_of(w->ex_up);
    a.sgate = ptr_of(w->sh_gate.km);
    a.sup = ptr_of(w->sh_up.km);
    a.x = (const bf16_t*)d_x;
    a.inds = d_inds;
    a.act = (bf16_t*)d_act;
    a.T = T;
    a.k = k;
    a.E = E;
    a.I = I;
    a.K = H;
    const int nch = chunks_of(w->ex_gate), rpw = 64 / nch;
    const int rows_y = T * k + T;
    // enough workgroups to fill the chip; each wavefront keeps >= 2 row loads in flight
    int iters = (int)(((long)I * rows_y) / ((long)rpw * 4 * ctx->compute_units * 4));
    iters = iters < 2 ? 2 : (iters > 8 ? 8 : iters);
    a.iters = iters;
    dim3 grid((I + rpw * 4 * iters - 1) / (rpw * 4 * iters), rows_y);
#define UP_CASE(KIND, N)                                                                     \
  case N:                                                                                    \
    hipLaunchKernelGGL((moe_up_kernel<KIND, N>), grid, dim3(256), 0, ctx->stream, a);        \
    break;
    if (w->ex_gate.kind == ORNITH_Q4K) {
      switch (nch) { UP_CASE(ORNITH_Q4K, 4) UP_CASE(ORNITH_Q4K, 8) UP_CASE(ORNITH_Q4K, 16) UP_CASE(ORNITH_Q4K, 32) UP_CASE(ORNITH_Q4K, 64) }
    } else {
      switch (nch) { UP_CASE(ORNITH_Q6K, 4) UP_CASE(ORNITH_Q6K, 8) UP_CASE(ORNITH_Q6K, 16) UP_CASE(ORNITH_Q6K, 32) UP_CASE(ORNITH_Q6K, 64) }
    }
#undef UP_CASE
    ORN_LAUNCH_CHECK("moe_up_kernel");
  }
  {
    DownArgs a{};
    a.down = ptr_of(w->ex_down);
    a.sdown = ptr_of(w->sh_down.km);
    a.act = (const bf16_t*)d_act;
    a.inds = d_inds;
    a.scores = (const bf16_t*)d_scores;
    a.egate = (const bf16_t*)d_egate;
    a.out = (bf16_t*)d_out;
    a.T = T;
    a.k = k;
    a.E = E;
    a.H = H;
    a.I = I;
    a.normalize = w->norm_topk_prob;
    const int nch = chunks_of(w->ex_down), rpw = 64 / nch;
    // columns per workgroup: aim for >= 2 workgroups per CU, at least 2 iterations
    int iters = (int)(((long)H * T) / ((long)rpw * ctx->compute_units * 2));
    iters = iters < 1 ? 1 : (iters > 4 ? 4 : iters);
    while (rpw * iters > kMaxCols) --iters;
    a.iters = iters;
    const int cols = rpw * iters;
    dim3 grid((H + cols - 1) / cols, T);
    dim3 block(64 * (k + 1));
#define DOWN_CASE(KIND, N)                                                                   \
  case N:                                                                                    \
    hipLaunchKernelGGL((moe_down_kernel<KIND, N>), grid, block, 0, ctx->stream, a);          \
    break;
    if (w->ex_down.kind == ORNITH_Q4K) {
      switch (nch) { DOWN_CASE(ORNITH_Q4K, 4) DOWN_CASE(ORNITH_Q4K, 8) DOWN_CASE(ORNITH_Q4K, 16) DOWN_CASE(ORNITH_Q4K, 32) DOWN_CASE(ORNITH_Q4K, 64) }
    } else {
      switch (nch) { DOWN_CASE(ORNITH_Q6K, 4) DOWN_CASE(ORNITH_Q6K, 8) DOWN_CASE(ORNITH_Q6K, 16) DOWN_CASE(ORNITH_Q6K, 32) DOWN_CASE(ORNITH_Q6K, 64) }
    }
#undef DOWN_CASE
    ORN_LAUNCH_CHECK("moe_down_kernel");
  }
  return ORNITH_OK;
}
