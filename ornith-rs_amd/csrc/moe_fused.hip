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
// and index lists read besides. Both are latency-shaped, not throughput-shaped: at
// verify width 2 a launch moves ~19 MB / ~15 MB, less than the chip can hold in
// flight, so every wavefront issues ALL of its weight loads first (they depend on
// nothing but the index list), then the activation loads, and only then computes.
#include "handoff.h"
#include "kq_device.h"
#ifdef ORN_TIMING
#include "rt.h"
// debug build only: per-workgroup phase time stamps (100 MHz wall clock) of the last launch
__device__ long long g_up_marks[2048][8];
#define UP_MARK(i) do { const int bl__ = blockIdx.y * gridDim.x + blockIdx.x; if (threadIdx.x == 0 && bl__ < 2048) g_up_marks[bl__][i] = wall_clock64(); } while (0)
#define ORN_TOPK_STAMP() UP_MARK(6)  // in the top-k: the gates have arrived
#endif
#include "moe_device.h"
#include "norm_device.h"
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
  int T, k, E, I, K;
  // gates != null: the routing is not read but made -- every workgroup of a routed row runs
  // softmax + top-k over its token's gates (one wavefront, ~300 instructions) and the first
  // workgroup of each token stores inds / scores for the down kernel
  const bf16_t* gates;   // [T, E]
  uint32_t* inds_out;    // [T*k]
  bf16_t* scores_out;    // [T*k]
};

// grid (ceil(I / (RPW * 4 * ITERS)), T*k + T), 256 threads
#ifdef ORN_TIMING
__device__ long long g_down_marks[1024][8];
#define DOWN_MARK(i) do { const int bl__ = blockIdx.y * gridDim.x + blockIdx.x; if ((threadIdx.x & 63) == 0 && (threadIdx.x >> 6) == (i >> 3) && bl__ < 1024) g_down_marks[bl__][i & 7] = wall_clock64(); } while (0)
// every wavefront's own stamps: [0, 16) its rows in registers (it waits for them: a wait the
// plain build does not have), [16, 32) its sums done
__device__ long long g_down_wave_marks[1024][32];
#define DOWN_WAVE_MARK(slot) do { const int bl__ = blockIdx.y * gridDim.x + blockIdx.x; if ((threadIdx.x & 63) == 0 && bl__ < 1024) g_down_wave_marks[bl__][(slot) * 16 + ((threadIdx.x >> 6) & 15)] = wall_clock64(); } while (0)
#else
#define UP_MARK(i)
#define DOWN_MARK(i)
#define DOWN_WAVE_MARK(slot)
#endif

// ROUTE: the routing is made in the head of the launch (a.gates) instead of read (a.inds)
#ifdef ORN_NOACC
// measurement build only (-DORN_NOACC): the two expert kernels with the dequantizing arithmetic
// taken out -- every load, the routing, the activation conversion, the reductions, swiglu and
// the combine stay; a row's sum is a fold of its loaded registers. What such a build takes is
// what the launch structure costs without the mat-vec's own vector work (results are garbage).
__device__ __forceinline__ float noacc_fold(const Q4Row& r, float x) {
  return __uint_as_float((r.q.x ^ r.q.y ^ r.q.z ^ r.q.w ^ r.s0 ^ r.s1 ^ r.s2 ^ r.dmw) & 0x3fffffffu) + x;
}
__device__ __forceinline__ float noacc_fold(const Q6Row& r, float x) {
  return __uint_as_float((r.qa.x ^ r.qa.y ^ r.qa.z ^ r.qa.w ^ r.qb.x ^ r.qb.y ^ r.qb.z ^ r.qb.w ^ r.qh.x ^ r.qh.y ^
                          r.qh.z ^ r.qh.w ^ r.sc.x ^ r.sc.y ^ r.d) & 0x3fffffffu) + x;
}
__device__ __forceinline__ float noacc_x(const Q4Lane<1>& L) { return L.sl[0] + L.sh[0]; }
__device__ __forceinline__ float noacc_x(const Q6Lane<1>& L) { return L.x[0][0][0] + L.x[0][1][5] + L.x[0][2][9] + L.x[0][3][15]; }
#define ORN_KL_ACC(row, L, acc) acc[0] = noacc_fold(row, noacc_x(L))
#else
#define ORN_KL_ACC(row, L, acc) KL::accumulate(row, L, acc)
#endif

// The leading flat arguments repeat what decides a workgroup's expert (the library is built with
// kernel-argument preloading: they are in scalar registers when the wavefront starts, so the
// gates / ids are asked for while the argument block is still being fetched).
template <int KIND, int LPR, int ITERS, bool ROUTE>
__global__ __launch_bounds__(256) void moe_up_kernel(const bf16_t* h_gates, const uint32_t* h_inds, int h_T, int h_k,
                                                     int h_E, UpArgs a) {
  UP_MARK(0);
  using KL = KqLane<KIND, 1>;
  constexpr int RPW = 64 / LPR;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int slot = lane / LPR, c = lane % LPR;
  const int nb = a.K >> 8;
  const int r = blockIdx.y;
  const int routed = h_T * h_k;
  const bool is_routed = r < routed;  // the same for the whole workgroup
  const int token = is_routed ? r / h_k : r - routed;
  // the expert first: its chain (gates -> softmax + top-k, or the id) starts from the preloaded
  // arguments alone
  uint32_t e = 0;
  if constexpr (ROUTE) {
    __shared__ uint32_t s_inds[16];
    __shared__ bf16_t s_scores[16];
    if (is_routed) {
      if (wave == 0) {
        const bf16_t* g = h_gates + (size_t)token * h_E;
        switch (h_E / 64) {
          case 1: router_topk_wave<1>(g, h_k, s_inds, s_scores, nullptr, lane); break;
          case 2: router_topk_wave<2>(g, h_k, s_inds, s_scores, nullptr, lane); break;
          case 4: router_topk_wave<4>(g, h_k, s_inds, s_scores, nullptr, lane); break;
          case 8: router_topk_wave<8>(g, h_k, s_inds, s_scores, nullptr, lane); break;
          default: router_topk_wave<16>(g, h_k, s_inds, s_scores, nullptr, lane); break;
        }
      }
      __syncthreads();
      UP_MARK(5);
      e = s_inds[r - token * h_k];
      if (blockIdx.x == 0 && r == token * h_k && threadIdx.x < h_k) {
        a.inds_out[r + threadIdx.x] = s_inds[threadIdx.x];
        a.scores_out[r + threadIdx.x] = s_scores[threadIdx.x];
      }
    }
  } else {
    if (is_routed) e = h_inds[r];
  }
  // both sets of weight pointers as values in scalar registers before the choice is made:
  // chosen by address instead, the pointers would be loaded in a second trip after the first
  KqPtr pin[4] = {a.gate, a.up, a.sgate, a.sup};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    uint64_t q = (uint64_t)pin[i].qs, sc = (uint64_t)pin[i].scales, d = (uint64_t)pin[i].dm;
    asm volatile("" : "+s"(q), "+s"(sc), "+s"(d));
    pin[i].qs = dm_global_ptr<const uint8_t>(q);
    pin[i].scales = dm_global_ptr<const uint8_t>(sc);
    pin[i].dm = dm_global_ptr<const uint16_t>(d);
  }
  const int64_t row0 = is_routed ? (int64_t)min(e, (uint32_t)(h_E - 1)) * a.I : 0;
  const KqPtr wg = is_routed ? pin[0] : pin[2], wu = is_routed ? pin[1] : pin[3];
  typename KL::Lane L;
  L.set_chunk(c);
  const int base = (blockIdx.x * 4 + wave) * (RPW * ITERS);
  typename KL::Row rg[ITERS], ru[ITERS];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int o = base + it * RPW + slot;
    const int64_t row = row0 + (o < a.I ? o : a.I - 1);
    rg[it] = KL::load(wg.qs, wg.scales, wg.dm, row, nb, L);
    ru[it] = KL::load(wu.qs, wu.scales, wu.dm, row, nb, L);
  }
  __builtin_amdgcn_sched_barrier(0);  // keep the weight loads ahead of the activation loads
  UP_MARK(1);
  const void* xrow[1] = {a.x + (size_t)token * a.K};
  L.template load_x<false>(xrow, c);
  UP_MARK(2);
  if constexpr (LPR == 64 && ITERS % 2 == 0) {
    // one row per wavefront pass: reduce two rows' gate and up sums together
#pragma unroll
    for (int it = 0; it < ITERS; it += 2) {
      float g0[1] = {0.f}, u0[1] = {0.f}, g1[1] = {0.f}, u1[1] = {0.f};
      ORN_KL_ACC(rg[it], L, g0);
      ORN_KL_ACC(ru[it], L, u0);
      ORN_KL_ACC(rg[it + 1], L, g1);
      ORN_KL_ACC(ru[it + 1], L, u1);
      const float red = dm_wave_sum4(g0[0], u0[0], g1[0], u1[0], lane);
      // lanes [0,16): gate row it, [32,48): up row it, [16,32): gate row it+1, [48,64): up row it+1;
      // after the halves trade places every lane holds a row's gate and up sums, and lanes 0
      // and 16 finish the two rows in one pass over the swiglu code
      float gsum, usum;
      dm_row_swap<32>(red, gsum, usum);
      const int o = base + it + ((lane >> 4) & 1);
      if ((lane & 47) == 0 && o < a.I) a.act[(size_t)r * a.I + o] = swiglu_bf16(gsum, usum);
      if (it == 0) UP_MARK(3);
    }
  } else {
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int o = base + it * RPW + slot;
      float ag[1] = {0.f}, au[1] = {0.f};
      ORN_KL_ACC(rg[it], L, ag);
      ORN_KL_ACC(ru[it], L, au);
      const float g = dm_wave_sum<LPR>(ag[0]);
      const float u = dm_wave_sum<LPR>(au[0]);
      if (c == 0 && o < a.I) a.act[(size_t)r * a.I + o] = swiglu_bf16(g, u);
    }
  }
  UP_MARK(4);
}

struct DownArgs {
  KqPtr down;   // routed [E, H, I]
  KqPtr sdown;  // shared [H, I]
  const bf16_t* act;     // [T*k + T, I]
  const uint32_t* inds;  // [T*k]
  const bf16_t* scores;  // [T*k]
  const bf16_t* egate;   // [T]
  bf16_t* out;           // [T, H]
  int T, k, E, H, I, normalize;
};

constexpr int kMaxK = 8;

// grid (ceil(H / (RPW * ITERS)), T), 64 * (k + 1) threads
// The leading flat arguments repeat what a routed wavefront needs for its first weight request
// (the library is built with kernel-argument preloading: they are in scalar registers when the
// wavefront starts, while the argument block is still being fetched).
//
// Wavefront j < k takes routed expert j over the workgroup's ITERS column groups. At ITERS = 4
// the shared expert's column groups go one each to wavefronts k .. k + 3, so that the compute
// unit's four SIMDs (wavefronts go round them in order) carry 9 / 9 / 9 / 9 row passes instead of
// 12 / 8 / 8 / 8 with a single shared wavefront (the passes are what is left to do when the rows
// arrive: 1.1 us of a 29.5 us block at T = 4); at ITERS = 2 the same split (5 / 5 / 4 / 4 against
// 6 / 4 / 4 / 4) measured no better, so there one wavefront k takes both groups.
template <int ITERS>
constexpr int down_shared_waves() { return ITERS >= 4 ? ITERS : 1; }
template <int KIND, int LPR, int ITERS>
__global__ __launch_bounds__(64 * (kMaxK + down_shared_waves<ITERS>())) void moe_down_kernel(const uint8_t* h_qs, const uint8_t* h_scales,
                                                                        const uint16_t* h_dm, const uint32_t* h_inds,
                                                                        int h_k, int h_E, int h_H, int h_I, DownArgs a) {
  using KL = KqLane<KIND, 1>;
  constexpr int RPW = 64 / LPR, COLS = RPW * ITERS;
  const int lane = threadIdx.x & 63, j = threadIdx.x >> 6;  // j < k: expert slot; j >= k: the shared expert's group j - k
  const int slot = lane / LPR, c = lane % LPR;
  const int nb = h_I >> 8;
  const int t = blockIdx.y, k = h_k;
  const int c0 = blockIdx.x * COLS;
  DOWN_MARK(0);

  __shared__ float yl[kMaxK + 1][COLS];
  __shared__ float wj[kMaxK];
  __shared__ float gsig;

  constexpr bool SPLIT = down_shared_waves<ITERS>() > 1;
  const bool shared = SPLIT ? j >= k : j == k;
  const int only = j - k;  // SPLIT: the one column group a shared-expert wavefront takes
  const int arow = shared ? a.T * k + t : t * k + j;
  const KqPtr w = shared ? a.sdown : KqPtr{h_qs, h_scales, h_dm};
  const int64_t row0 = shared ? 0 : (int64_t)min(h_inds[t * k + j], (uint32_t)(h_E - 1)) * h_H;
  typename KL::Lane L;
  L.set_chunk(c);
  // the activation row first: it is a kilobyte the up launch has just written, back long before
  // the weights, and its conversion then runs under the weights' trip (loads return in issue
  // order: asked for behind the weights it was converted only after the last of them had arrived;
  // 0.5 us a pair at T = 2)
  // With fewer than 64 lanes a row the rows of a wavefront pass share their activations: a
  // lane asks for one 16-byte piece of the row (one load instruction a wavefront where every
  // lane fetching its own 64 or 128 bytes takes four or eight; 0.2 us a pair at T = 2, 0.4-0.5
  // at T = 3 and 4) and LDS hands out the chunks once the piece is there.
  constexpr int XROW = LPR * (KIND == ORNITH_Q4K ? 32 : 64);  // activations a row (== I)
  constexpr bool X_VIA_LDS = LPR < 64;
  constexpr int XP = X_VIA_LDS ? (XROW / 8 + 63) / 64 : 1;  // 16-byte pieces a lane
  __shared__ __align__(16) bf16_t xs[X_VIA_LDS ? kMaxK + down_shared_waves<ITERS>() : 1][X_VIA_LDS ? XROW : 8];
  const bf16_t* arow_p = a.act + (size_t)arow * a.I;
  uint4 xpiece[XP];
  if constexpr (X_VIA_LDS) {
#pragma unroll
    for (int p = 0; p < XP; ++p)
      if (8 * (lane + 64 * p) < XROW) xpiece[p] = *reinterpret_cast<const uint4*>(arow_p + 8 * (lane + 64 * p));
  } else {
    const void* xrow[1] = {arow_p};
    L.template load_x<false>(xrow, c);
  }
  // likewise the token's router scores (lane i < k holds score i) and its shared-expert gate:
  // wavefront 0 turns them into the combine weights while its weight rows are on their way
  const uint16_t score_bits = a.scores[(size_t)t * k + (lane < k ? lane : 0)];
  const uint16_t egate_bits = a.egate[t];
  __builtin_amdgcn_sched_barrier(0);
  typename KL::Row rr[ITERS];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    if (SPLIT && shared && it != only) continue;
    const int o = c0 + it * RPW + slot;
    rr[it] = KL::load(w.qs, w.scales, w.dm, row0 + (o < h_H ? o : h_H - 1), nb, L);
  }
  __builtin_amdgcn_sched_barrier(0);  // keep the weight loads ahead of everything that follows
  DOWN_MARK(1);
  if constexpr (X_VIA_LDS) {
    // (a wavefront reads back only what it wrote itself: its LDS accesses complete in order)
#pragma unroll
    for (int p = 0; p < XP; ++p)
      if (8 * (lane + 64 * p) < XROW) *reinterpret_cast<uint4*>(&xs[j][8 * (lane + 64 * p)]) = xpiece[p];
    const void* xrow[1] = {&xs[j][0]};
    L.template load_x<false>(xrow, c);
  }
  DOWN_MARK(2);

  if (j == 0) {
    // the router weights of this token: denom = ((0+s0)+s1)..., w_j = bf16(s_j / denom)
    float denom = 0.f;
    if (a.normalize) {
#pragma unroll
      for (int i = 0; i < kMaxK; ++i)
        if (i < k) denom = dm_rb(dm_bf2f((bf16_t)__builtin_amdgcn_readlane((int)score_bits, i)) + denom);
    }
    if (lane < k) wj[lane] = a.normalize ? dm_rb(dm_bf2f(score_bits) / denom) : dm_bf2f(score_bits);
    if (lane == 0) gsig = dm_sigmoid_bf16(dm_bf2f(egate_bits));
  }
#ifdef ORN_TIMING
  __builtin_amdgcn_s_waitcnt(0);  // vmcnt(0) with the other counters: the rows are here
  DOWN_WAVE_MARK(0);
#endif
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    if (SPLIT && shared && it != only) continue;
    float acc[1] = {0.f};
    ORN_KL_ACC(rr[it], L, acc);
    const float v = dm_wave_sum<LPR>(acc[0]);
    if (c == 0) yl[SPLIT && shared ? k : j][it * RPW + slot] = dm_rb(v);  // expert outputs are bf16 in the unfused path
  }
  DOWN_MARK(3);
  DOWN_WAVE_MARK(1);
  __syncthreads();
  DOWN_MARK(4);
  const int col = threadIdx.x;
  if (col < COLS && c0 + col < a.H) {
    float acc = 0.f;
    for (int i = 0; i < k; ++i) {
      const float weighted = dm_rb(yl[i][col] * wj[i]);
      acc = dm_rb(weighted + acc);
    }
    const float gated = dm_rb(gsig * yl[k][col]);
    a.out[(size_t)t * a.H + c0 + col] = dm_f2bf(acc + gated);
  }
  DOWN_MARK(5);
}

// ---- router: the gates mat-vec and, in one extra workgroup, the shared expert's scalar
// gate for every token (one wavefront per token). Softmax + top-k follow in their own
// small launch: a hand-off inside this one needs device-wide release fences, which on a
// multi-die part write the L2 back and cost more than the launch they would save. ------
struct RouterArgs {
  KqPtr w;               // router [E, K]
  const bf16_t* x;       // [M, K]
  bf16_t* gates;         // [M, E]
  bf16_t* egate;         // [M]
  const void* eg_w;      // shared_expert_gate weights: affine8 u8[K] or dense bf16[K]
  const bf16_t* eg_s;    // affine8 scales [K/64]
  const bf16_t* eg_b;    // affine8 biases [K/64]
  int eg_affine;
  int E, K;
  PreNorm pre;           // pre.res != null: x is not read but made, x = rms_norm(res + y) (K == 2048),
                         // by every workgroup; workgroup 0 stores h and x
};

// One row of the 8-bit affine / dense mat-vec by one wavefront (the order of linear.hip): group
// j of eight weights on lane j mod 64, a lane's groups in ascending order. The row is a few KB
// that no earlier launch has touched: a lane asks for all of its groups at once (egate_issue),
// ahead of the norm's arithmetic, and works them off when the normed row is there (egate_finish).
// Up to kEgGroups groups a lane (K <= 2048); wider rows take the plain loop.
constexpr int kEgGroups = 4;
struct EgRegs {
  uint4 w[kEgGroups];          // dense: eight bf16 weights; affine: .x .y the eight codes
  bf16_t s[kEgGroups], b[kEgGroups];
};
__device__ __forceinline__ void egate_issue(const RouterArgs& a, int lane, EgRegs& g) {
#pragma unroll
  for (int u = 0; u < kEgGroups; ++u) {
    const int j = lane + 64 * u;
    if (j >= a.K / 8) continue;
    if (a.eg_affine) {
      const uint2 q = *reinterpret_cast<const uint2*>(static_cast<const uint8_t*>(a.eg_w) + 8 * j);
      g.w[u] = make_uint4(q.x, q.y, 0, 0);
      g.s[u] = a.eg_s[j >> 3];
      g.b[u] = a.eg_b[j >> 3];
    } else {
      g.w[u] = *reinterpret_cast<const uint4*>(static_cast<const bf16_t*>(a.eg_w) + 8 * j);
    }
  }
}
__device__ __forceinline__ float egate_group(const RouterArgs& a, const uint4& wv, bf16_t sc, bf16_t bi, const uint4& xv,
                                             float acc_lane) {
  const float xs[8] = {dm_bf2f_lo(xv.x), dm_bf2f_hi(xv.x), dm_bf2f_lo(xv.y), dm_bf2f_hi(xv.y),
                       dm_bf2f_lo(xv.z), dm_bf2f_hi(xv.z), dm_bf2f_lo(xv.w), dm_bf2f_hi(xv.w)};
  if (a.eg_affine) {
    const uint32_t qw[2] = {wv.x, wv.y};
    float acc = 0.f, sum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float qf = (float)((qw[i >> 2] >> (8 * (i & 3))) & 0xffu);
      acc = dm_fma(xs[i], qf, acc);
      sum = sum + xs[i];
    }
    float p = dm_bf2f(sc) * acc;
    p = dm_fma(sum, dm_bf2f(bi), p);
    return acc_lane + p;
  }
  acc_lane = dm_fma(dm_bf2f_lo(wv.x), xs[0], acc_lane);
  acc_lane = dm_fma(dm_bf2f_hi(wv.x), xs[1], acc_lane);
  acc_lane = dm_fma(dm_bf2f_lo(wv.y), xs[2], acc_lane);
  acc_lane = dm_fma(dm_bf2f_hi(wv.y), xs[3], acc_lane);
  acc_lane = dm_fma(dm_bf2f_lo(wv.z), xs[4], acc_lane);
  acc_lane = dm_fma(dm_bf2f_hi(wv.z), xs[5], acc_lane);
  acc_lane = dm_fma(dm_bf2f_lo(wv.w), xs[6], acc_lane);
  acc_lane = dm_fma(dm_bf2f_hi(wv.w), xs[7], acc_lane);
  return acc_lane;
}
__device__ __forceinline__ float egate_finish(const RouterArgs& a, const EgRegs& g, const bf16_t* xr, int lane) {
  float acc_lane = 0.f;
#pragma unroll
  for (int u = 0; u < kEgGroups; ++u) {
    const int j = lane + 64 * u;
    if (j >= a.K / 8) continue;
    acc_lane = egate_group(a, g.w[u], g.s[u], g.b[u], *reinterpret_cast<const uint4*>(xr + 8 * j), acc_lane);
  }
  return dm_wave_sum<64>(acc_lane);
}
__device__ __forceinline__ float egate_row_dot(const RouterArgs& a, const bf16_t* xr, int lane) {
  float acc_lane = 0.f;
  for (int j = lane; j < a.K / 8; j += 64) {
    uint4 wv;
    bf16_t sc = 0, bi = 0;
    if (a.eg_affine) {
      const uint2 q = *reinterpret_cast<const uint2*>(static_cast<const uint8_t*>(a.eg_w) + 8 * j);
      wv = make_uint4(q.x, q.y, 0, 0);
      sc = a.eg_s[j >> 3];
      bi = a.eg_b[j >> 3];
    } else {
      wv = *reinterpret_cast<const uint4*>(static_cast<const bf16_t*>(a.eg_w) + 8 * j);
    }
    acc_lane = egate_group(a, wv, sc, bi, *reinterpret_cast<const uint4*>(xr + 8 * j), acc_lane);
  }
  return dm_wave_sum<64>(acc_lane);
}

// grid ceil(E / (RPW * 4)) + 1, 256 threads, M <= 4 tokens
// The leading flat arguments repeat what the first loads need (the norm's inputs and the router's
// rows): preloaded into scalar registers, they let those loads leave while the argument block is
// still being fetched.
template <int KIND, int LPR, int M>
__global__ __launch_bounds__(256) void moe_router_kernel(const bf16_t* h_res, const bf16_t* h_y, const bf16_t* h_w,
                                                         const uint8_t* h_qs, const uint8_t* h_scales,
                                                         const uint16_t* h_dm, int h_E, int h_K, RouterArgs a) {
  using KL = KqLane<KIND, M>;
  constexpr int RPW = 64 / LPR;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __shared__ PreNormLds<M> pn;
  const bool pre = h_res != nullptr;
  if (blockIdx.x == gridDim.x - 1) {
    const bool narrow = a.K / 8 <= 64 * kEgGroups;
    PreNormRegs<M> pg;
    EgRegs eg;
    if (pre) prenorm_issue<M>(a.pre, pg);
    if (narrow && wave < M) egate_issue(a, lane, eg);
    __builtin_amdgcn_sched_barrier(0);
    if (pre) prenorm_finish<M>(a.pre, pg, false, pn);
    if (wave < M) {
      const bf16_t* xr = pre ? &pn.xn[wave][0] : a.x + (size_t)wave * a.K;
      const float e = narrow ? egate_finish(a, eg, xr, lane) : egate_row_dot(a, xr, lane);
      if (lane == 0) a.egate[wave] = dm_f2bf(e);
    }
    return;
  }
  const int slot = lane / LPR, c = lane % LPR;
  const int nb = h_K >> 8;
  typename KL::Lane L;
  L.set_chunk(c);
  const int o = (blockIdx.x * 4 + wave) * RPW + slot;
  // the norm's inputs first (cached, back early), the weight row right behind them: loads
  // return in issue order
  PreNormRegs<M> pg;
  if (pre) {
    PreNorm ph{};
    ph.res = h_res;
    ph.y = h_y;
    ph.w = h_w;
    prenorm_issue<M>(ph, pg);
  }
  __builtin_amdgcn_sched_barrier(0);
  const typename KL::Row row = KL::load(h_qs, h_scales, h_dm, o < h_E ? o : h_E - 1, nb, L);
  __builtin_amdgcn_sched_barrier(0);  // keep the weight loads ahead of everything that follows
  if (pre) prenorm_finish<M>(a.pre, pg, blockIdx.x == 0, pn);
  const void* xrow[M];
#pragma unroll
  for (int t = 0; t < M; ++t) xrow[t] = pre ? (const void*)&pn.xn[t][0] : (const void*)(a.x + (size_t)t * a.K);
  L.template load_x<false>(xrow, c);
  float acc[M];
#pragma unroll
  for (int t = 0; t < M; ++t) acc[t] = 0.f;
  KL::accumulate(row, L, acc);
#pragma unroll
  for (int t = 0; t < M; ++t) {
    const float v = dm_wave_sum<LPR>(acc[t]);
    if (c == 0 && o < a.E) a.gates[(size_t)t * a.E + o] = dm_f2bf(v);
  }
}

#define ORN_ROUTER_HEAD(a) (a).pre.res, (a).pre.y, (a).pre.w, (a).w.qs, (a).w.scales, (a).w.dm, (a).E, (a).K
template <int KIND, int LPR>
void launch_router_fused(ornith_ctx* ctx, const RouterArgs& a, int M) {
  constexpr int RPW = 64 / LPR;
  dim3 grid((a.E + RPW * 4 - 1) / (RPW * 4) + 1);
  switch (M) {
    case 1: hipLaunchKernelGGL((moe_router_kernel<KIND, LPR, 1>), grid, dim3(256), 0, ctx->stream, ORN_ROUTER_HEAD(a), a); break;
    case 2: hipLaunchKernelGGL((moe_router_kernel<KIND, LPR, 2>), grid, dim3(256), 0, ctx->stream, ORN_ROUTER_HEAD(a), a); break;
    case 3: hipLaunchKernelGGL((moe_router_kernel<KIND, LPR, 3>), grid, dim3(256), 0, ctx->stream, ORN_ROUTER_HEAD(a), a); break;
    default: hipLaunchKernelGGL((moe_router_kernel<KIND, LPR, 4>), grid, dim3(256), 0, ctx->stream, ORN_ROUTER_HEAD(a), a); break;
  }
}

// ---- the whole block in ONE launch ---------------------------------------------------
// Router, expert up and expert down as three ranges of workgroups of one grid, handing
// their small intermediates (gates, the normed input rows, the routing, the expert
// activations) over through memory as handoff.h describes. Same arithmetic as the three
// kernels above, operation for operation; what changes is that two launch boundaries are
// gone, that the down workgroups have their weight rows in flight while the up workgroups
// still compute, and that nothing but flag words is waited for.
//
//   [0, n_router)            router rows (+ the shared expert's scalar gate in the last one);
//                            workgroup 0 also stores h and the normed rows
//   [n_router, +n_up)        (row r, column block bx): waits for the router, makes the top-k,
//                            gate + up + swiglu -> act; one workgroup per token stores the routing
//   [.., +n_down)            (token t, column block bx): waits for the routing, requests its
//                            down rows, waits for its act rows, down + combine -> out
struct OneArgs {
  RouterArgs r;
  UpArgs u;
  DownArgs d;
  uint32_t* rflag;  // [n_router]
  uint32_t* iflag;  // [T]
  uint32_t* aflag;  // [(T*k + T) * up_x]
  uint32_t* err;
  uint32_t epoch;
  int n_router, up_x, n_up, down_x, max_spins;
};

template <int KIND, int LPR, int M>
__device__ __forceinline__ void one_router(const OneArgs& o, int wg, char* lds) {
  if (threadIdx.x >= 256) return;
  const RouterArgs& a = o.r;
  using KL = KqLane<KIND, 1>;
  constexpr int RPW = 64 / LPR;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  PreNormLds<M>& pn = *reinterpret_cast<PreNormLds<M>*>(lds);
  const bool pre = a.pre.res != nullptr;
  if (wg == o.n_router - 1) {
    if (pre) prenorm_rows<M, true>(a.pre, false, pn);
    if (wave < M) {
      const float e = egate_row_dot(a, pre ? &pn.xn[wave][0] : a.x + (size_t)wave * a.K, lane);
      if (lane == 0) ho_store_u16(&a.egate[wave], dm_f2bf(e));
    }
    ho_publish(&o.rflag[wg], o.epoch);
    return;
  }
  const int slot = lane / LPR, c = lane % LPR;
  const int nb = a.K >> 8;
  typename KL::Lane L;
  L.set_chunk(c);
  const int row_o = (wg * 4 + wave) * RPW + slot;
  const typename KL::Row row = KL::load(a.w.qs, a.w.scales, a.w.dm, row_o < a.E ? row_o : a.E - 1, nb, L);
  __builtin_amdgcn_sched_barrier(0);  // keep the weight loads ahead of the activation loads
  if (pre) prenorm_rows<M, true>(a.pre, wg == 0, pn);
  // one token at a time over the same weight registers (a row's sum does not depend on how
  // many rows share the pass)
#pragma unroll
  for (int t = 0; t < M; ++t) {
    const void* xrow[1] = {pre ? (const void*)&pn.xn[t][0] : (const void*)(a.x + (size_t)t * a.K)};
    L.template load_x<false>(xrow, c);
    float acc[1] = {0.f};
    KL::accumulate(row, L, acc);
    const float v = dm_wave_sum<LPR>(acc[0]);
    if (c == 0 && row_o < a.E) ho_store_u16(&a.gates[(size_t)t * a.E + row_o], dm_f2bf(v));
  }
  ho_publish(&o.rflag[wg], o.epoch);
}

// RIN: the router runs inside this launch (gates and input rows are hand-offs); otherwise they
// were written by earlier launches and are read the ordinary way.
template <int KIND, int LPR, bool RIN>
__device__ __forceinline__ void one_up(const OneArgs& o, int u, char* lds) {
  if (threadIdx.x >= 256) return;
  const UpArgs& a = o.u;
  using KL = KqLane<KIND, 1>;
  constexpr int RPW = 64 / LPR, ITERS = 2;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int slot = lane / LPR, c = lane % LPR;
  const int nb = a.K >> 8;
  const int bx = u % o.up_x, r = u / o.up_x;
  const int routed = a.T * a.k;
  uint32_t* s_inds = reinterpret_cast<uint32_t*>(lds);
  bf16_t* s_scores = reinterpret_cast<bf16_t*>(lds + 64);
  KqPtr pin[4] = {a.gate, a.up, a.sgate, a.sup};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    uint64_t q = (uint64_t)pin[i].qs, sc = (uint64_t)pin[i].scales, d = (uint64_t)pin[i].dm;
    asm volatile("" : "+s"(q), "+s"(sc), "+s"(d));
    pin[i].qs = dm_global_ptr<const uint8_t>(q);
    pin[i].scales = dm_global_ptr<const uint8_t>(sc);
    pin[i].dm = dm_global_ptr<const uint16_t>(d);
  }
  int token;
  int64_t row0;
  KqPtr wg_, wu_;
  const bool is_routed = r < routed;
  if (is_routed) {
    token = r / a.k;
    if (wave == 0) {
      if constexpr (RIN) ho_wait(o.rflag, o.n_router, o.epoch, o.max_spins, o.err, lane);
      const bf16_t* g = a.gates + (size_t)token * a.E;
      switch (a.E / 64) {
        case 1: router_topk_wave<1, RIN>(g, a.k, s_inds, s_scores, nullptr, lane); break;
        case 2: router_topk_wave<2, RIN>(g, a.k, s_inds, s_scores, nullptr, lane); break;
        case 4: router_topk_wave<4, RIN>(g, a.k, s_inds, s_scores, nullptr, lane); break;
        case 8: router_topk_wave<8, RIN>(g, a.k, s_inds, s_scores, nullptr, lane); break;
        default: router_topk_wave<16, RIN>(g, a.k, s_inds, s_scores, nullptr, lane); break;
      }
    }
    __syncthreads();
    const uint32_t e = s_inds[r - token * a.k];
    row0 = (int64_t)min(e, (uint32_t)(a.E - 1)) * a.I;
    wg_ = pin[0];
    wu_ = pin[1];
  } else {
    token = r - routed;
    row0 = 0;
    wg_ = pin[2];
    wu_ = pin[3];
  }
  typename KL::Lane L;
  L.set_chunk(c);
  const int base = (bx * 4 + wave) * (RPW * ITERS);
  typename KL::Row rg[ITERS], ru[ITERS];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int oo = base + it * RPW + slot;
    const int64_t row = row0 + (oo < a.I ? oo : a.I - 1);
    rg[it] = KL::load(wg_.qs, wg_.scales, wg_.dm, row, nb, L);
    ru[it] = KL::load(wu_.qs, wu_.scales, wu_.dm, row, nb, L);
  }
  __builtin_amdgcn_sched_barrier(0);  // keep the weight loads ahead of everything below
  if (is_routed) {
    // one workgroup per token stores the routing: for the down workgroups when the router runs
    // in this launch (a hand-off), for the caller otherwise
    if (bx == 0 && r == token * a.k && wave == 0) {
      if (lane < a.k) {
        ho_store_u32(&a.inds_out[r + lane], s_inds[lane]);
        ho_store_u16(&a.scores_out[r + lane], s_scores[lane]);
      }
      if constexpr (RIN) {
        ho_wait_stores();
        if (lane == 0) ho_store_u32(&o.iflag[token], o.epoch);
      }
    }
  } else if constexpr (RIN) {
    // the shared expert's rows need no routing, only the normed input rows
    ho_wait(o.rflag, o.n_router, o.epoch, o.max_spins, o.err, lane);
  }
  const void* xrow[1] = {a.x + (size_t)token * a.K};
  L.template load_x<false, RIN>(xrow, c);
  if constexpr (LPR == 64) {
#pragma unroll
    for (int it = 0; it < ITERS; it += 2) {
      float g0[1] = {0.f}, u0[1] = {0.f}, g1[1] = {0.f}, u1[1] = {0.f};
      KL::accumulate(rg[it], L, g0);
      KL::accumulate(ru[it], L, u0);
      KL::accumulate(rg[it + 1], L, g1);
      KL::accumulate(ru[it + 1], L, u1);
      const float red = dm_wave_sum4(g0[0], u0[0], g1[0], u1[0], lane);
      float gsum, usum;
      dm_row_swap<32>(red, gsum, usum);
      const int oo = base + it + ((lane >> 4) & 1);
      if ((lane & 47) == 0 && oo < a.I) ho_store_u16(&a.act[(size_t)r * a.I + oo], swiglu_bf16(gsum, usum));
    }
  } else {
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int oo = base + it * RPW + slot;
      float ag[1] = {0.f}, au[1] = {0.f};
      KL::accumulate(rg[it], L, ag);
      KL::accumulate(ru[it], L, au);
      const float g = dm_wave_sum<LPR>(ag[0]);
      const float uu = dm_wave_sum<LPR>(au[0]);
      if (c == 0 && oo < a.I) ho_store_u16(&a.act[(size_t)r * a.I + oo], swiglu_bf16(g, uu));
    }
  }
  ho_publish(&o.aflag[(size_t)r * o.up_x + bx], o.epoch);
}

// Down role: wavefront w of the workgroup takes expert slots 2w and 2w+1 (slot k is the shared
// expert), so (k + 1 + 1) / 2 wavefronts cover the k + 1 rows that meet in LDS.
template <int KIND, int LPR, bool RIN>
__device__ __forceinline__ void one_down(const OneArgs& o, int dd, char* lds) {
  const DownArgs& a = o.d;
  using KL = KqLane<KIND, 1>;
  constexpr int RPW = 64 / LPR, COLS = RPW;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int slot = lane / LPR, c = lane % LPR;
  const int nb = a.I >> 8;
  const int t = dd / o.down_x, k = a.k;
  const int c0 = (dd % o.down_x) * COLS;
  float(*yl)[COLS] = reinterpret_cast<float(*)[COLS]>(lds);
  float* wj = reinterpret_cast<float*>(lds + sizeof(float) * (kMaxK + 1) * COLS);
  float* gsig = wj + kMaxK;
  const int j0 = 2 * wave;

  typename KL::Lane L;
  L.set_chunk(c);
  const int oo = c0 + slot;
  const int64_t orow = oo < a.H ? oo : a.H - 1;
  typename KL::Row rr[2];
  int arow[2];
  uint32_t* s_inds = reinterpret_cast<uint32_t*>(gsig + 1);
  bf16_t* s_scores = reinterpret_cast<bf16_t*>(s_inds + 16);
  if constexpr (RIN) {
    if (j0 < k) ho_wait(&o.iflag[t], 1, o.epoch, o.max_spins, o.err, lane);
  } else {
    // the gates are an earlier launch's: every workgroup makes its token's routing itself,
    // so nothing but its own act rows is ever waited for
    if (wave == 0) {
      const bf16_t* g = o.u.gates + (size_t)t * a.E;
      switch (a.E / 64) {
        case 1: router_topk_wave<1>(g, k, s_inds, s_scores, nullptr, lane); break;
        case 2: router_topk_wave<2>(g, k, s_inds, s_scores, nullptr, lane); break;
        case 4: router_topk_wave<4>(g, k, s_inds, s_scores, nullptr, lane); break;
        case 8: router_topk_wave<8>(g, k, s_inds, s_scores, nullptr, lane); break;
        default: router_topk_wave<16>(g, k, s_inds, s_scores, nullptr, lane); break;
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int j = j0 + q;
    const bool shared = j >= k;  // also the unused second slot of the last wavefront (harmless reload)
    arow[q] = shared ? a.T * k + t : t * k + j;
    const KqPtr w = shared ? a.sdown : a.down;
    int64_t row0 = 0;
    if (!shared) {
      const uint32_t e = RIN ? ho_load_u32(&a.inds[t * k + j]) : s_inds[j];
      row0 = (int64_t)min(e, (uint32_t)(a.E - 1)) * a.H;
    }
    rr[q] = KL::load(w.qs, w.scales, w.dm, row0 + orow, nb, L);
  }
  __builtin_amdgcn_sched_barrier(0);  // the weight rows are in flight while the act rows are awaited
  if (wave == 0) {
    // with the router in this launch the scores arrived with the routing (iflag), and the shared
    // expert's scalar gate was published before any routing could be made
    const bf16_t* s = a.scores + (size_t)t * k;
    float denom = 0.f;
    if (a.normalize)
      for (int i = 0; i < k; ++i) denom = dm_rb(dm_bf2f(RIN ? ho_load_u16(&s[i]) : s_scores[i]) + denom);
    if (lane < k) {
      const float sv = dm_bf2f(RIN ? ho_load_u16(&s[lane]) : s_scores[lane]);
      wj[lane] = a.normalize ? dm_rb(sv / denom) : sv;
    }
    if (lane == 0) *gsig = dm_sigmoid_bf16(dm_bf2f(RIN ? ho_load_u16(&a.egate[t]) : a.egate[t]));
  }
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    if (j0 + q > k) break;  // a slot past the shared expert
    ho_wait(&o.aflag[(size_t)arow[q] * o.up_x], o.up_x, o.epoch, o.max_spins, o.err, lane);
    const void* xrow[1] = {a.act + (size_t)arow[q] * a.I};
    L.template load_x<false, true>(xrow, c);
    float acc[1] = {0.f};
    KL::accumulate(rr[q], L, acc);
    const float v = dm_wave_sum<LPR>(acc[0]);
    if (c == 0) yl[j0 + q][slot] = dm_rb(v);
  }
  __syncthreads();
  const int col = threadIdx.x;
  if (col < COLS && c0 + col < a.H) {
    float acc = 0.f;
    for (int i = 0; i < k; ++i) {
      const float weighted = dm_rb(yl[i][col] * wj[i]);
      acc = dm_rb(weighted + acc);
    }
    const float gated = dm_rb(*gsig * yl[k][col]);
    a.out[(size_t)t * a.H + c0 + col] = dm_f2bf(acc + gated);
  }
  DOWN_MARK(5);
}

template <int M>
constexpr size_t one_lds_bytes() {
  constexpr size_t down = sizeof(float) * ((kMaxK + 1) * 16 + kMaxK + 1) + 16 * 4 + 16 * 2;
  return sizeof(PreNormLds<M>) > down ? sizeof(PreNormLds<M>) : down;
}

constexpr int kOneThreads = 64 * ((kMaxK + 2) / 2);  // 320: five wavefronts, of which up / router use four

template <int RK, int RLPR, int M, int UK, int ULPR, int DK, int DLPR>
__global__ __launch_bounds__(kOneThreads) void moe_one_kernel(OneArgs a) {
  __shared__ __attribute__((aligned(16))) char lds[one_lds_bytes<M>()];
  const int wg = blockIdx.x;
  if (wg < a.n_router) {
    one_router<RK, RLPR, M>(a, wg, lds);
  } else if (wg < a.n_router + a.n_up) {
    one_up<UK, ULPR, true>(a, wg - a.n_router, lds);
  } else {
    one_down<DK, DLPR, true>(a, wg - a.n_router - a.n_up, lds);
  }
}

// up + down only: the router (and the norm in its head) stays a launch of its own
template <int UK, int ULPR, int DK, int DLPR>
__global__ __launch_bounds__(kOneThreads) void moe_updown_kernel(OneArgs a) {
  __shared__ __attribute__((aligned(16))) char lds[one_lds_bytes<1>() > 1024 ? 1024 : one_lds_bytes<1>()];
  const int wg = blockIdx.x;
  if (wg < a.n_up) {
    one_up<UK, ULPR, false>(a, wg, lds);
  } else {
    one_down<DK, DLPR, false>(a, wg - a.n_up, lds);
  }
}

KqPtr ptr_of(const ornith_kmatrix& m) {
  return KqPtr{(const uint8_t*)m.d_qs, (const uint8_t*)m.d_scales, (const uint16_t*)m.d_dm};
}

int chunks_of(const ornith_kmatrix& m) { return (m.K >> 8) * (m.kind == ORNITH_Q4K ? 8 : 4); }

template <int KIND, int LPR>
void launch_up(ornith_ctx* ctx, const UpArgs& a, int rows_y) {
  constexpr int RPW = 64 / LPR;
  // Two rows per wavefront measured faster than four at every decode/verify width (four
  // rows of gate + up codes in flight cost enough registers to halve the occupancy);
  // four stays selectable for wider inputs.
  if (ornith_option_moe_up_iters() == 4) {
    dim3 grid((a.I + RPW * 4 * 4 - 1) / (RPW * 4 * 4), rows_y);
    if (a.gates)
      hipLaunchKernelGGL((moe_up_kernel<KIND, LPR, 4, true>), grid, dim3(256), 0, ctx->stream, a.gates, a.inds, a.T,
                         a.k, a.E, a);
    else
      hipLaunchKernelGGL((moe_up_kernel<KIND, LPR, 4, false>), grid, dim3(256), 0, ctx->stream, a.gates, a.inds, a.T,
                         a.k, a.E, a);
  } else {
    dim3 grid((a.I + RPW * 4 * 2 - 1) / (RPW * 4 * 2), rows_y);
    if (a.gates)
      hipLaunchKernelGGL((moe_up_kernel<KIND, LPR, 2, true>), grid, dim3(256), 0, ctx->stream, a.gates, a.inds, a.T,
                         a.k, a.E, a);
    else
      hipLaunchKernelGGL((moe_up_kernel<KIND, LPR, 2, false>), grid, dim3(256), 0, ctx->stream, a.gates, a.inds, a.T,
                         a.k, a.E, a);
  }
}

template <int KIND, int LPR>
void launch_down(ornith_ctx* ctx, const DownArgs& a) {
  constexpr int RPW = 64 / LPR;
  const long groups1 = (long)(a.H + RPW - 1) / RPW * a.T;
  const int forced = ornith_option_moe_down_iters();
  // About one workgroup (k + 1 wavefronts) per compute unit is the fastest shape at every verify
  // width: measured (us, 1 / 2 / 4 column groups a workgroup) T = 1: 5.4 / 6.1 / 8.7, T = 2:
  // 9.0 / 6.8 / 9.2, T = 3: 12.6 / 11.4 / 10.0, T = 4: 16.2 / 12.1 / 10.9
  const long cu = ctx->compute_units;
  const int iters = forced ? forced : groups1 >= 3 * cu ? 4 : groups1 >= 2 * cu ? 2 : 1;
  // k routed wavefronts and the shared expert's (one, or one a column group at four groups)
  const dim3 block(64 * (a.k + (iters >= 4 ? 4 : 1)));
  if (iters >= 4) {
    dim3 grid((a.H + RPW * 4 - 1) / (RPW * 4), a.T);
    hipLaunchKernelGGL((moe_down_kernel<KIND, LPR, 4>), grid, block, 0, ctx->stream, a.down.qs, a.down.scales,
                       a.down.dm, a.inds, a.k, a.E, a.H, a.I, a);
  } else if (iters == 2) {
    dim3 grid((a.H + RPW * 2 - 1) / (RPW * 2), a.T);
    hipLaunchKernelGGL((moe_down_kernel<KIND, LPR, 2>), grid, block, 0, ctx->stream, a.down.qs, a.down.scales,
                       a.down.dm, a.inds, a.k, a.E, a.H, a.I, a);
  } else {
    dim3 grid((a.H + RPW - 1) / RPW, a.T);
    hipLaunchKernelGGL((moe_down_kernel<KIND, LPR, 1>), grid, block, 0, ctx->stream, a.down.qs, a.down.scales,
                       a.down.dm, a.inds, a.k, a.E, a.H, a.I, a);
  }
}

}  // namespace

#ifdef ORN_TIMING
extern "C" __attribute__((visibility("default"))) int ornith_debug_marks_up(long long* out) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_up_marks), sizeof(long long) * 2048 * 8);
}
extern "C" __attribute__((visibility("default"))) int ornith_debug_marks_down(long long* out) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_down_marks), sizeof(long long) * 1024 * 8);
}
extern "C" __attribute__((visibility("default"))) int ornith_debug_marks_down_waves(long long* out) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_down_wave_marks), sizeof(long long) * 1024 * 32);
}
#endif

// Whether the two fused kernels cover this block's shapes and formats.
bool moe_fused_supported(const ornith_moe_weights* w) {
  if (w->ex_dense) return false;
  if (w->ex_gate.kind > ORNITH_Q6K || w->ex_down.kind > ORNITH_Q6K) return false;  // 4-bit affine stacks
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

// Router mat-vec + shared_expert_gate in one launch. Returns false (nothing launched)
// when the shapes / formats are outside what the kernel covers.
bool moe_fused_router(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_x, int T,
                      void* d_gates, void* d_egate, int* rc, const PreNorm* pre) {
  *rc = ORNITH_OK;
  const ornith_linear& r = w->router;
  const ornith_linear& g = w->sh_egate;
  if (T > 4 || r.mode != ORNITH_LIN_KQUANT) return false;
  if (g.mode != ORNITH_LIN_AFFINE8 && g.mode != ORNITH_LIN_DENSE) return false;
  if (g.K % 64 != 0) return false;
  const int E = r.O;
  const int nch = chunks_of(r.km);
  if (!(nch == 8 || nch == 16 || nch == 32 || nch == 64)) return false;
  RouterArgs a{};
  a.w = ptr_of(r.km);
  a.x = (const bf16_t*)d_x;
  a.gates = (bf16_t*)d_gates;
  a.egate = (bf16_t*)d_egate;
  a.eg_w = g.d_w;
  a.eg_s = (const bf16_t*)g.d_scales;
  a.eg_b = (const bf16_t*)g.d_biases;
  a.eg_affine = g.mode == ORNITH_LIN_AFFINE8;
  a.E = E;
  a.K = r.K;
  if (pre) {
    if (r.K != kPreN) return false;
    a.pre = *pre;
  }
#define R_CASE(KIND, N) \
  case N:               \
    launch_router_fused<KIND, N>(ctx, a, T); \
    break;
  if (r.km.kind == ORNITH_Q4K) {
    switch (nch) { R_CASE(ORNITH_Q4K, 8) R_CASE(ORNITH_Q4K, 16) R_CASE(ORNITH_Q4K, 32) R_CASE(ORNITH_Q4K, 64) }
  } else {
    switch (nch) { R_CASE(ORNITH_Q6K, 8) R_CASE(ORNITH_Q6K, 16) R_CASE(ORNITH_Q6K, 32) R_CASE(ORNITH_Q6K, 64) }
  }
#undef R_CASE
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) *rc = ornith_fail(ORNITH_ERR_HIP, "launch of moe_router_kernel failed: %s", hipGetErrorString(e));
  return true;
}

// act: scratch bf16 [(T*k + T), I]. phases: 1 = up, 2 = down, 3 = both.
// d_gates != null (phases & 1): the up kernel makes the routing from the gates and stores it
// to d_inds / d_scores (which then are outputs).
int moe_fused_experts(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_x, int T,
                      const uint32_t* d_inds, const void* d_scores, const void* d_egate, void* d_act,
                      void* d_out, int phases, const void* d_gates) {
  const int E = w->router.O, H = w->router.K, I = w->ex_gate.O, k = w->top_k;
  if (phases & 1) {
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
    a.gates = (const bf16_t*)d_gates;
    a.inds_out = const_cast<uint32_t*>(d_inds);
    a.scores_out = (bf16_t*)const_cast<void*>(d_scores);
    const int nch = chunks_of(w->ex_gate), rows_y = T * k + T;
#define UP_CASE(KIND, N) \
  case N:                \
    launch_up<KIND, N>(ctx, a, rows_y); \
    break;
    if (w->ex_gate.kind == ORNITH_Q4K) {
      switch (nch) { UP_CASE(ORNITH_Q4K, 8) UP_CASE(ORNITH_Q4K, 16) UP_CASE(ORNITH_Q4K, 32) UP_CASE(ORNITH_Q4K, 64) }
    } else {
      switch (nch) { UP_CASE(ORNITH_Q6K, 4) UP_CASE(ORNITH_Q6K, 8) UP_CASE(ORNITH_Q6K, 16) UP_CASE(ORNITH_Q6K, 32) UP_CASE(ORNITH_Q6K, 64) }
    }
#undef UP_CASE
    ORN_LAUNCH_CHECK("moe_up_kernel");
  }
  if (phases & 2) {
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
    const int nch = chunks_of(w->ex_down);
#define DOWN_CASE(KIND, N) \
  case N:                  \
    launch_down<KIND, N>(ctx, a); \
    break;
    if (w->ex_down.kind == ORNITH_Q4K) {
      switch (nch) { DOWN_CASE(ORNITH_Q4K, 8) DOWN_CASE(ORNITH_Q4K, 16) DOWN_CASE(ORNITH_Q4K, 32) DOWN_CASE(ORNITH_Q4K, 64) }
    } else {
      switch (nch) { DOWN_CASE(ORNITH_Q6K, 4) DOWN_CASE(ORNITH_Q6K, 8) DOWN_CASE(ORNITH_Q6K, 16) DOWN_CASE(ORNITH_Q6K, 32) DOWN_CASE(ORNITH_Q6K, 64) }
    }
#undef DOWN_CASE
    ORN_LAUNCH_CHECK("moe_down_kernel");
  }
  return ORNITH_OK;
}

// The block in one launch (moe_one_kernel). Returns false with nothing launched when the
// shapes / formats are outside the instantiated family: hidden size 2048 and expert width
// 512 in one of the format mixes (router, gate/up, down) = (Q6_K, Q4_K, Q6_K), all Q4_K or
// all Q6_K, T <= 4, a power-of-two expert count the top-k wavefront covers.
// d_x: the block's input rows, or with `pre` where the normed rows are to be stored.
bool moe_one_launch(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_x, int T, void* d_gates,
                    void* d_egate, uint32_t* d_inds, void* d_scores, void* d_act, void* d_out,
                    const PreNorm* pre, int* rc) {
  *rc = ORNITH_OK;
  const ornith_linear& r = w->router;
  const ornith_linear& g = w->sh_egate;
  const int E = r.O, H = r.K, I = w->ex_gate.O, k = w->top_k;
  const int how = ornith_option_fuse_moe_one();  // 1: router + up + down, 2: up + down (router launched first)
  if (!how || !moe_fused_supported(w) || T < 1 || T > 4) return false;
  if (r.mode != ORNITH_LIN_KQUANT || (g.mode != ORNITH_LIN_AFFINE8 && g.mode != ORNITH_LIN_DENSE)) return false;
  if (H != kPreN || I != 512 || w->sh_gate.O != I || g.K != H) return false;
  if (E % 64 != 0 || E > 1024 || ((E / 64) & (E / 64 - 1)) != 0 || k > kMaxK || k > E) return false;
  const int rk = r.km.kind, uk = w->ex_gate.kind, dk = w->ex_down.kind;
  const int mix = rk == ORNITH_Q6K && uk == ORNITH_Q4K && dk == ORNITH_Q6K   ? 0
                  : rk == ORNITH_Q4K && uk == ORNITH_Q4K && dk == ORNITH_Q4K ? 1
                  : rk == ORNITH_Q6K && uk == ORNITH_Q6K && dk == ORNITH_Q6K ? 2
                                                                              : -1;
  if (mix < 0) return false;
  // flag words: router | routing | act, all inside the context's block
  const int rlpr = rk == ORNITH_Q4K ? 64 : 32, ulpr = uk == ORNITH_Q4K ? 64 : 32, dlpr = dk == ORNITH_Q4K ? 16 : 8;
  OneArgs a{};
  a.n_router = how == 1 ? (E + (64 / rlpr) * 4 - 1) / ((64 / rlpr) * 4) + 1 : 0;
  if (how != 1) {
    // the router (with the norm in its head) as its own launch first
    if (!moe_fused_router(ctx, w, d_x, T, d_gates, d_egate, rc, pre)) return false;
    if (*rc) return true;
    pre = nullptr;
  }
  a.up_x = (I + (64 / ulpr) * 4 * 2 - 1) / ((64 / ulpr) * 4 * 2);
  const int rows_y = T * k + T;
  a.n_up = a.up_x * rows_y;
  a.down_x = (H + (64 / dlpr) - 1) / (64 / dlpr);
  const int n_down = a.down_x * T;
  if ((size_t)a.n_router + 4 + (size_t)rows_y * a.up_x > ornith_ctx::kHoFlagWords) return false;
  if (ctx->ho_epoch == 0xffffffffu) {
    // the epoch numbers are used up: start over from clean flag words
    if (hipStreamSynchronize(ctx->stream) != hipSuccess ||
        hipMemset(ctx->ho_flags, 0, sizeof(uint32_t) * ornith_ctx::kHoFlagWords) != hipSuccess) {
      *rc = ornith_fail(ORNITH_ERR_HIP, "moe_block: resetting the hand-off flags failed");
      return true;
    }
    ctx->ho_epoch = 0;
  }
  a.epoch = ++ctx->ho_epoch;
  a.rflag = ctx->ho_flags;
  a.iflag = a.rflag + a.n_router;
  a.aflag = a.iflag + 4;
  a.err = ctx->ho_err_dev;
  a.max_spins = ornith_option_ho_spins();

  a.r.w = ptr_of(r.km);
  a.r.x = (const bf16_t*)d_x;
  a.r.gates = (bf16_t*)d_gates;
  a.r.egate = (bf16_t*)d_egate;
  a.r.eg_w = g.d_w;
  a.r.eg_s = (const bf16_t*)g.d_scales;
  a.r.eg_b = (const bf16_t*)g.d_biases;
  a.r.eg_affine = g.mode == ORNITH_LIN_AFFINE8;
  a.r.E = E;
  a.r.K = H;
  if (pre) a.r.pre = *pre;

  a.u.gate = ptr_of(w->ex_gate);
  a.u.up = ptr_of(w->ex_up);
  a.u.sgate = ptr_of(w->sh_gate.km);
  a.u.sup = ptr_of(w->sh_up.km);
  a.u.x = (const bf16_t*)d_x;
  a.u.inds = d_inds;
  a.u.act = (bf16_t*)d_act;
  a.u.T = T;
  a.u.k = k;
  a.u.E = E;
  a.u.I = I;
  a.u.K = H;
  a.u.gates = (const bf16_t*)d_gates;
  a.u.inds_out = d_inds;
  a.u.scores_out = (bf16_t*)d_scores;

  a.d.down = ptr_of(w->ex_down);
  a.d.sdown = ptr_of(w->sh_down.km);
  a.d.act = (const bf16_t*)d_act;
  a.d.inds = d_inds;
  a.d.scores = (const bf16_t*)d_scores;
  a.d.egate = (const bf16_t*)d_egate;
  a.d.out = (bf16_t*)d_out;
  a.d.T = T;
  a.d.k = k;
  a.d.E = E;
  a.d.H = H;
  a.d.I = I;
  a.d.normalize = w->norm_topk_prob;

  const dim3 grid(a.n_router + a.n_up + n_down), block(kOneThreads);
#define ONE_M(RK, RL, UK, UL, DK, DL)                                                                         \
  switch (T) {                                                                                                \
    case 1: hipLaunchKernelGGL((moe_one_kernel<RK, RL, 1, UK, UL, DK, DL>), grid, block, 0, ctx->stream, a); break; \
    case 2: hipLaunchKernelGGL((moe_one_kernel<RK, RL, 2, UK, UL, DK, DL>), grid, block, 0, ctx->stream, a); break; \
    case 3: hipLaunchKernelGGL((moe_one_kernel<RK, RL, 3, UK, UL, DK, DL>), grid, block, 0, ctx->stream, a); break; \
    default: hipLaunchKernelGGL((moe_one_kernel<RK, RL, 4, UK, UL, DK, DL>), grid, block, 0, ctx->stream, a); break; \
  }
  if (how != 1) {
    if (mix == 0)
      hipLaunchKernelGGL((moe_updown_kernel<ORNITH_Q4K, 64, ORNITH_Q6K, 8>), grid, block, 0, ctx->stream, a);
    else if (mix == 1)
      hipLaunchKernelGGL((moe_updown_kernel<ORNITH_Q4K, 64, ORNITH_Q4K, 16>), grid, block, 0, ctx->stream, a);
    else
      hipLaunchKernelGGL((moe_updown_kernel<ORNITH_Q6K, 32, ORNITH_Q6K, 8>), grid, block, 0, ctx->stream, a);
  } else if (mix == 0) {
    ONE_M(ORNITH_Q6K, 32, ORNITH_Q4K, 64, ORNITH_Q6K, 8)
  } else if (mix == 1) {
    ONE_M(ORNITH_Q4K, 64, ORNITH_Q4K, 64, ORNITH_Q4K, 16)
  } else {
    ONE_M(ORNITH_Q6K, 32, ORNITH_Q6K, 32, ORNITH_Q6K, 8)
  }
#undef ONE_M
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) *rc = ornith_fail(ORNITH_ERR_HIP, "launch of moe_one_kernel failed: %s", hipGetErrorString(e));
  return true;
}

extern "C" {

int ornith_moe_experts(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_x, int T,
                       const uint32_t* d_inds, const void* d_scores, const void* d_egate, void* d_act,
                       void* d_out, int phases) {
  ORN_REQUIRE(ctx && w && d_x && d_inds && d_scores && d_egate && d_act && d_out,
              "moe_experts: null argument");
  ORN_REQUIRE(T >= 1 && T <= 64 && phases >= 1 && phases <= 3, "moe_experts: T=%d phases=%d", T, phases);
  if (!moe_fused_supported(w))
    return ornith_fail(ORNITH_ERR_UNSUPPORTED,
                       "moe_experts: the fused expert kernels need k-quant routed and shared experts "
                       "of matching formats and top_k <= %d", kMaxK);
  return moe_fused_experts(ctx, w, d_x, T, d_inds, d_scores, d_egate, d_act, d_out, phases, nullptr);
}

int ornith_moe_experts_from_gates(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_x, int T,
                                  const void* d_gates, const void* d_egate, uint32_t* d_inds_out,
                                  void* d_scores_out, void* d_act, void* d_out) {
  ORN_REQUIRE(ctx && w && d_x && d_gates && d_egate && d_inds_out && d_scores_out && d_act && d_out,
              "moe_experts_from_gates: null argument");
  ORN_REQUIRE(T >= 1 && T <= 64, "moe_experts_from_gates: T=%d", T);
  const int E = w->router.O, k = w->top_k;
  if (!moe_fused_supported(w) || E % 64 != 0 || E > 1024 || ((E / 64) & (E / 64 - 1)) != 0 || k > 16)
    return ornith_fail(ORNITH_ERR_UNSUPPORTED,
                       "moe_experts_from_gates: needs k-quant routed and shared experts of matching formats, "
                       "top_k <= %d and a power-of-two multiple of 64 experts up to 1024", kMaxK);
  return moe_fused_experts(ctx, w, d_x, T, d_inds_out, d_scores_out, d_egate, d_act, d_out, 3, d_gates);
}

}  // extern "C"
