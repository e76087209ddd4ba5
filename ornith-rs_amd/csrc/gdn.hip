// Gated-delta (linear attention) layer: fused front end and the recurrence.
//
// Replaces gdn::gdn_front and gdn::gated_delta_kernel[_into]
// (/root/reference/src/ops/gdn.rs:131-271,331-413; kernels
// /root/reference/kernels/gdn_front.metal:65-190,
// /root/reference/kernels/gated_delta.metal:36-142) and the per-token snapshot
// loop of GatedDeltaNet::forward_capture (/root/reference/src/model/qwen3_5.rs:650-677).
//
// Front: one wavefront per (token, 128-channel head slot); lane l holds channels
// 2l, 2l+1 from the convolution through the q/k normalisation, so the causal
// conv, silu, RMS and scale never leave registers. It also writes the
// concatenated window [K-1+T, D]; the next conv state is a 3-row slice of it
// (rows [keep, keep+3) after a rollback to `keep` tokens).
//
// Recurrence: the fp32 state [Hv, Dv, 128] stays in registers across the T verify
// tokens. Eight lanes share a state row (lane j owns dk = 32m + 4j + i, which
// makes every load and store a contiguous 128 bytes per row), one wavefront
// carries eight rows, and the state after EACH token is written out as a
// snapshot, so rejecting a draft is a pointer move to snapshot keep-1.
#include "dmath.h"
#include "linear_device.h"
#include "rt.h"

namespace {

struct FrontArgs {
  const bf16_t* conv_state;  // [S, D]
  const bf16_t* qkv;         // [T, D]
  const bf16_t* cw;          // [D, K]
  const bf16_t* a_in;        // [T, Hv]
  const bf16_t* b_in;        // [T, Hv]
  const bf16_t* a_log;       // [Hv]
  const bf16_t* dt_bias;     // [Hv]
  bf16_t* q;                 // [T, Hk, 128]
  bf16_t* k;                 // [T, Hk, 128]
  bf16_t* v;                 // [T, Hv, 128]
  bf16_t* beta;              // [T, Hv]
  float* g;                  // [T, Hv]
  bf16_t* conv_input;        // [S + T, D]
  int T, K, Hk, Hv, D;
  float q_scale, k_scale, eps;
};

__device__ __forceinline__ float softplus_bf16(float x) {
  if (x != x) return x;
  const float mx = x > 0.f ? x : 0.f, mn = x > 0.f ? 0.f : x;
  if (mn == -DM_INF || mx == DM_INF) return mx;
  const float d = dm_rb(mn - mx);
  const float e = dm_rb(dm_exp(d));
  const float l = dm_rb(dm_log1p(e));
  return dm_rb(mx + l);
}

__global__ __launch_bounds__(64) void gdn_front_kernel(FrontArgs p) {
  const int slot = blockIdx.x, t = blockIdx.y, lane = threadIdx.x;
  const int S = p.K - 1, D = p.D;
  const int c0 = slot * 128 + 2 * lane;
  const int key_dim = p.Hk * 128;

  float acc0 = 0.f, acc1 = 0.f;
  for (int i = 0; i < p.K; ++i) {
    const int j = t + i;
    const bf16_t* src = (j < S) ? (p.conv_state + (size_t)j * D) : (p.qkv + (size_t)(j - S) * D);
    const uint32_t xv = *reinterpret_cast<const uint32_t*>(src + c0);
    acc0 = dm_fma(dm_bf2f_lo(xv), dm_bf2f(p.cw[(size_t)c0 * p.K + i]), acc0);
    acc1 = dm_fma(dm_bf2f_hi(xv), dm_bf2f(p.cw[(size_t)(c0 + 1) * p.K + i]), acc1);
  }
  const float cv0 = dm_rb(acc0), cv1 = dm_rb(acc1);
  const float y0 = dm_rb(cv0 * dm_sigmoid_bf16(cv0)), y1 = dm_rb(cv1 * dm_sigmoid_bf16(cv1));

  // the concatenated window
  {
    uint32_t* ci = reinterpret_cast<uint32_t*>(p.conv_input + (size_t)(S + t) * D + c0);
    *ci = *reinterpret_cast<const uint32_t*>(p.qkv + (size_t)t * D + c0);
    if (t == 0) {
      for (int j = 0; j < S; ++j)
        *reinterpret_cast<uint32_t*>(p.conv_input + (size_t)j * D + c0) =
            *reinterpret_cast<const uint32_t*>(p.conv_state + (size_t)j * D + c0);
    }
  }

  if (slot < 2 * p.Hk) {
    float ss = dm_fma(y0, y0, 0.f);
    ss = dm_fma(y1, y1, ss);
    const float inv = dm_rsqrt(dm_wave_sum<64>(ss) / 128.0f + p.eps);
    const bool is_q = slot < p.Hk;
    bf16_t* dst = (is_q ? p.q : p.k) + (size_t)t * key_dim + (is_q ? c0 : c0 - key_dim);
    const float sc = is_q ? p.q_scale : p.k_scale;
    const uint32_t lo = dm_f2bf(sc * dm_rb(y0 * inv)), hi = dm_f2bf(sc * dm_rb(y1 * inv));
    *reinterpret_cast<uint32_t*>(dst) = lo | (hi << 16);
  } else {
    bf16_t* dst = p.v + (size_t)t * (D - 2 * key_dim) + (c0 - 2 * key_dim);
    *reinterpret_cast<uint32_t*>(dst) = (uint32_t)dm_f2bf(y0) | ((uint32_t)dm_f2bf(y1) << 16);
  }

  if (slot == 0) {
    for (int h = lane; h < p.Hv; h += 64) {
      const int i = t * p.Hv + h;
      const float sp = softplus_bf16(dm_rb(dm_bf2f(p.a_in[i]) + dm_bf2f(p.dt_bias[h])));
      const float decay = dm_exp(dm_bf2f(p.a_log[h]));
      p.g[i] = dm_exp(-decay * sp);
      p.beta[i] = dm_f2bf(dm_sigmoid_bf16(dm_bf2f(p.b_in[i])));
    }
  }
}

// The same for a run of tokens per workgroup (kernel size 4, prefill widths): the taps are
// loaded once and each token's inputs are read once and kept as the sliding window, instead of
// one 64-thread workgroup per token and 128 channels. Per token the arithmetic and its order
// are those of gdn_front_kernel. grid (D / 128, ceil(T / kFrontRun)), 64 threads.
constexpr int kFrontRun = 16;
__global__ __launch_bounds__(64) void gdn_front_run_kernel(FrontArgs p) {
  constexpr int K = 4, S = K - 1;
  const int slot = blockIdx.x, t0 = blockIdx.y * kFrontRun, lane = threadIdx.x;
  const int D = p.D, c0 = slot * 128 + 2 * lane, key_dim = p.Hk * 128;
  const int t1 = min(t0 + kFrontRun, p.T);
  float w0[K], w1[K];
  {
    const uint2 a = *reinterpret_cast<const uint2*>(p.cw + (size_t)c0 * K);
    const uint2 b = *reinterpret_cast<const uint2*>(p.cw + (size_t)(c0 + 1) * K);
    w0[0] = dm_bf2f_lo(a.x); w0[1] = dm_bf2f_hi(a.x); w0[2] = dm_bf2f_lo(a.y); w0[3] = dm_bf2f_hi(a.y);
    w1[0] = dm_bf2f_lo(b.x); w1[1] = dm_bf2f_hi(b.x); w1[2] = dm_bf2f_lo(b.y); w1[3] = dm_bf2f_hi(b.y);
  }
  // window position j holds conv_state[j] for j < S, qkv[j - S] from there on
  auto input = [&](int j) {
    const bf16_t* src = (j < S) ? (p.conv_state + (size_t)j * D) : (p.qkv + (size_t)(j - S) * D);
    return *reinterpret_cast<const uint32_t*>(src + c0);
  };
  uint32_t win[K];
#pragma unroll
  for (int i = 0; i < S; ++i) win[i] = input(t0 + i);
  if (t0 == 0) {
#pragma unroll
    for (int j = 0; j < S; ++j) *reinterpret_cast<uint32_t*>(p.conv_input + (size_t)j * D + c0) = win[j];
  }
  const bool is_qk = slot < 2 * p.Hk, is_q = slot < p.Hk;
  const float sc = is_q ? p.q_scale : p.k_scale;
  // the run's inputs are asked for together (one after the other, every token would wait out a
  // memory latency of its own); rows past the end of the call read the last row, unused
  uint32_t in[kFrontRun];
#pragma unroll
  for (int u = 0; u < kFrontRun; ++u) in[u] = input(min(t0 + u, p.T - 1) + S);
#pragma unroll
  for (int u = 0; u < kFrontRun; ++u) {
    const int t = t0 + u;
    if (t >= t1) break;
    win[S] = in[u];  // = qkv[t]
    float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
    for (int i = 0; i < K; ++i) {
      acc0 = dm_fma(dm_bf2f_lo(win[i]), w0[i], acc0);
      acc1 = dm_fma(dm_bf2f_hi(win[i]), w1[i], acc1);
    }
    *reinterpret_cast<uint32_t*>(p.conv_input + (size_t)(S + t) * D + c0) = win[S];
#pragma unroll
    for (int i = 0; i < S; ++i) win[i] = win[i + 1];
    const float cv0 = dm_rb(acc0), cv1 = dm_rb(acc1);
    const float y0 = dm_rb(cv0 * dm_sigmoid_bf16(cv0)), y1 = dm_rb(cv1 * dm_sigmoid_bf16(cv1));
    if (is_qk) {
      float ss = dm_fma(y0, y0, 0.f);
      ss = dm_fma(y1, y1, ss);
      const float inv = dm_rsqrt(dm_wave_sum<64>(ss) / 128.0f + p.eps);
      bf16_t* dst = (is_q ? p.q : p.k) + (size_t)t * key_dim + (is_q ? c0 : c0 - key_dim);
      const uint32_t lo = dm_f2bf(sc * dm_rb(y0 * inv)), hi = dm_f2bf(sc * dm_rb(y1 * inv));
      *reinterpret_cast<uint32_t*>(dst) = lo | (hi << 16);
    } else {
      bf16_t* dst = p.v + (size_t)t * (D - 2 * key_dim) + (c0 - 2 * key_dim);
      *reinterpret_cast<uint32_t*>(dst) = (uint32_t)dm_f2bf(y0) | ((uint32_t)dm_f2bf(y1) << 16);
    }
  }
  if (slot == 0) {
    for (int i = t0 * p.Hv + lane; i < t1 * p.Hv; i += 64) {
      const int h = i % p.Hv;
      const float sp = softplus_bf16(dm_rb(dm_bf2f(p.a_in[i]) + dm_bf2f(p.dt_bias[h])));
      const float decay = dm_exp(dm_bf2f(p.a_log[h]));
      p.g[i] = dm_exp(-decay * sp);
      p.beta[i] = dm_f2bf(dm_sigmoid_bf16(dm_bf2f(p.b_in[i])));
    }
  }
}

struct RecArgs {
  const bf16_t* q;
  const bf16_t* k;
  const bf16_t* v;
  const float* g;
  const bf16_t* beta;
  const float* state_in;  // [Hv, Dv, 128]
  bf16_t* y;              // [T, Hv, Dv]
  float* snapshots;       // [T][Hv, Dv, 128]
  int T, Hk, Hv, Dv;
  int snap_all;  // 1: a snapshot per token; 0: only the final state, in slot 0
};

__global__ __launch_bounds__(64) void gdn_recurrence_kernel(RecArgs p) {
  const int lane = threadIdx.x, row = lane >> 3, j = lane & 7;
  const int hv = blockIdx.y, dv = blockIdx.x * 8 + row;
  const int hk = hv / (p.Hv / p.Hk);
  const size_t ssz = (size_t)p.Hv * p.Dv * 128;
  const size_t roff = ((size_t)hv * p.Dv + dv) * 128 + 4 * j;

  float s[16];
#pragma unroll
  for (int m = 0; m < 4; ++m) {
    const float4 f = *reinterpret_cast<const float4*>(p.state_in + roff + 32 * m);
    s[4 * m + 0] = f.x;
    s[4 * m + 1] = f.y;
    s[4 * m + 2] = f.z;
    s[4 * m + 3] = f.w;
  }
  // Each token's step is a short dependent chain, far shorter than a trip to L2 for its
  // operands: the operands of the next GP tokens are requested while this group is worked
  // through (token indices past the end are clamped and their loads unused).
  constexpr int GP = 4;
  typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
  u32x2 kw[GP][4], qw[GP][4];
  float gg[GP], bb[GP], vv[GP];
  auto fetch = [&](int t, u32x2 (&kd)[4], u32x2 (&qd)[4], float& gd, float& bd, float& vd) {
    const int tc = t < p.T ? t : p.T - 1;
    const bf16_t* kp = p.k + ((size_t)tc * p.Hk + hk) * 128 + 4 * j;
    const bf16_t* qp = p.q + ((size_t)tc * p.Hk + hk) * 128 + 4 * j;
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      kd[m] = *reinterpret_cast<const u32x2*>(kp + 32 * m);
      qd[m] = *reinterpret_cast<const u32x2*>(qp + 32 * m);
    }
    gd = p.g[tc * p.Hv + hv];
    bd = dm_bf2f(p.beta[tc * p.Hv + hv]);
    vd = dm_bf2f(p.v[((size_t)tc * p.Hv + hv) * p.Dv + dv]);
  };
#pragma unroll
  for (int i = 0; i < GP; ++i) fetch(i, kw[i], qw[i], gg[i], bb[i], vv[i]);
  for (int t0 = 0; t0 < p.T; t0 += GP) {
    u32x2 kwn[GP][4], qwn[GP][4];
    float ggn[GP], bbn[GP], vvn[GP];
#pragma unroll
    for (int i = 0; i < GP; ++i) fetch(t0 + GP + i, kwn[i], qwn[i], ggn[i], bbn[i], vvn[i]);
    __builtin_amdgcn_sched_barrier(0);
    // a full group with only the final state wanted runs as straight-line code: the output
    // chain of one token and the k-chain of the next do not depend on each other, and without
    // branches between them the scheduler interleaves the two
    const bool straight = t0 + GP <= p.T && !p.snap_all;
    if (straight) {
#pragma unroll
      for (int i = 0; i < GP; ++i) {
        float kf[16], qf[16];
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          kf[4 * m + 0] = dm_bf2f_lo(kw[i][m].x);
          kf[4 * m + 1] = dm_bf2f_hi(kw[i][m].x);
          kf[4 * m + 2] = dm_bf2f_lo(kw[i][m].y);
          kf[4 * m + 3] = dm_bf2f_hi(kw[i][m].y);
          qf[4 * m + 0] = dm_bf2f_lo(qw[i][m].x);
          qf[4 * m + 1] = dm_bf2f_hi(qw[i][m].x);
          qf[4 * m + 2] = dm_bf2f_lo(qw[i][m].y);
          qf[4 * m + 3] = dm_bf2f_hi(qw[i][m].y);
        }
        const float gt = gg[i], bt = bb[i], vt = vv[i];
        float a = 0.f;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          s[e] = s[e] * gt;
          a = dm_fma(s[e], kf[e], a);
        }
        const float kv = dm_wave_sum<8>(a);
        const float delta = (vt - kv) * bt;
        float o = 0.f;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          s[e] = dm_fma(kf[e], delta, s[e]);
          o = dm_fma(s[e], qf[e], o);
        }
        o = dm_wave_sum<8>(o);
        if (j == 0) p.y[((size_t)(t0 + i) * p.Hv + hv) * p.Dv + dv] = dm_f2bf(o);
      }
      if (t0 + GP == p.T) {
        float* snap = p.snapshots + roff;
#pragma unroll
        for (int m = 0; m < 4; ++m)
          *reinterpret_cast<float4*>(snap + 32 * m) =
              make_float4(s[4 * m + 0], s[4 * m + 1], s[4 * m + 2], s[4 * m + 3]);
      }
    } else
#pragma unroll
    for (int i = 0; i < GP; ++i) {
      const int t = t0 + i;
      if (t < p.T) {
        float kf[16], qf[16];
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          kf[4 * m + 0] = dm_bf2f_lo(kw[i][m].x);
          kf[4 * m + 1] = dm_bf2f_hi(kw[i][m].x);
          kf[4 * m + 2] = dm_bf2f_lo(kw[i][m].y);
          kf[4 * m + 3] = dm_bf2f_hi(kw[i][m].y);
          qf[4 * m + 0] = dm_bf2f_lo(qw[i][m].x);
          qf[4 * m + 1] = dm_bf2f_hi(qw[i][m].x);
          qf[4 * m + 2] = dm_bf2f_lo(qw[i][m].y);
          qf[4 * m + 3] = dm_bf2f_hi(qw[i][m].y);
        }
        const float gt = gg[i], bt = bb[i], vt = vv[i];
        float a = 0.f;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          s[e] = s[e] * gt;
          a = dm_fma(s[e], kf[e], a);
        }
        const float kv = dm_wave_sum<8>(a);
        const float delta = (vt - kv) * bt;
        float o = 0.f;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          s[e] = dm_fma(kf[e], delta, s[e]);
          o = dm_fma(s[e], qf[e], o);
        }
        o = dm_wave_sum<8>(o);
        if (j == 0) p.y[((size_t)t * p.Hv + hv) * p.Dv + dv] = dm_f2bf(o);
        if (p.snap_all || t + 1 == p.T) {
          float* snap = p.snapshots + (p.snap_all ? (size_t)t * ssz : 0) + roff;
#pragma unroll
          for (int m = 0; m < 4; ++m)
            *reinterpret_cast<float4*>(snap + 32 * m) =
                make_float4(s[4 * m + 0], s[4 * m + 1], s[4 * m + 2], s[4 * m + 3]);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < GP; ++i) {
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        kw[i][m] = kwn[i][m];
        qw[i][m] = qwn[i][m];
      }
      gg[i] = ggn[i];
      bb[i] = bbn[i];
      vv[i] = vvn[i];
    }
  }
}

// ---- the recurrence at prefill widths ---------------------------------------------------
// A long prompt chunk is a chain of T dependent steps per state row; what a step costs is the
// instructions a wavefront issues for it and the memory trips that are not hidden. Like every
// prefill kernel this one agrees with the exact kernel above to rounding, not bit for bit,
// which frees the order of the sums: 16 lanes share a state row (8 columns a lane), each
// lane's dot products run as two chains of four, and only the final state is written. Keys
// and queries of 32 tokens are converted to f32 once and parked in LDS while the next 32
// tokens' loads are in flight, so no step waits on memory. grid (Dv / 4, Hv), 64 threads.
__global__ __launch_bounds__(64) void gdn_recurrence_wide_kernel(RecArgs p) {
  constexpr int C = 32;                          // tokens staged at a time
  __shared__ __align__(16) float kq[C + 1][2][128];  // k then q of a token, f32
  __shared__ __align__(16) float gbv[C + 1][8];      // g, beta, -, -, v of the four rows
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  const int lane = threadIdx.x, row = lane >> 4, j = lane & 15;
  const int hv = blockIdx.y, dv0 = blockIdx.x * 4, dv = dv0 + row;
  const int hk = hv / (p.Hv / p.Hk);
  const size_t roff = ((size_t)hv * p.Dv + dv) * 128 + 4 * j;  // columns 64*m + 4*j .. +4

  float s[8];
#pragma unroll
  for (int m = 0; m < 2; ++m) {
    const float4 f = *reinterpret_cast<const float4*>(p.state_in + roff + 64 * m);
    s[4 * m + 0] = f.x;
    s[4 * m + 1] = f.y;
    s[4 * m + 2] = f.z;
    s[4 * m + 3] = f.w;
  }
  // a lane's share of 32 tokens: eight columns (8*j ..) of tokens 4*i + row, i < 8; g and beta
  // of token lane (lanes below 32); v of tokens lane/4 and 16 + lane/4, row lane%4
  u32x4 kr[C / 4], qr[C / 4];
  float gr = 1.f, br = 0.f, vr[2];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < C / 4; ++i) {
      const int t = min(t0 + 4 * i + row, p.T - 1);
      const size_t o = ((size_t)t * p.Hk + hk) * 128 + 8 * j;
      kr[i] = *reinterpret_cast<const u32x4*>(p.k + o);
      qr[i] = *reinterpret_cast<const u32x4*>(p.q + o);
    }
    const int tg = min(t0 + (lane & 31), p.T - 1);
    gr = p.g[tg * p.Hv + hv];
    br = dm_bf2f(p.beta[tg * p.Hv + hv]);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int tv = min(t0 + 16 * h + (lane >> 2), p.T - 1);
      vr[h] = dm_bf2f(p.v[((size_t)tv * p.Hv + hv) * p.Dv + dv0 + (lane & 3)]);
    }
  };
  auto park = [&](int t0) {
#pragma unroll
    for (int i = 0; i < C / 4; ++i) {
      float* kd = &kq[4 * i + row][0][8 * j];
      float* qd = &kq[4 * i + row][1][8 * j];
      *reinterpret_cast<float4*>(kd) = make_float4(dm_bf2f_lo(kr[i].x), dm_bf2f_hi(kr[i].x), dm_bf2f_lo(kr[i].y), dm_bf2f_hi(kr[i].y));
      *reinterpret_cast<float4*>(kd + 4) = make_float4(dm_bf2f_lo(kr[i].z), dm_bf2f_hi(kr[i].z), dm_bf2f_lo(kr[i].w), dm_bf2f_hi(kr[i].w));
      *reinterpret_cast<float4*>(qd) = make_float4(dm_bf2f_lo(qr[i].x), dm_bf2f_hi(qr[i].x), dm_bf2f_lo(qr[i].y), dm_bf2f_hi(qr[i].y));
      *reinterpret_cast<float4*>(qd + 4) = make_float4(dm_bf2f_lo(qr[i].z), dm_bf2f_hi(qr[i].z), dm_bf2f_lo(qr[i].w), dm_bf2f_hi(qr[i].w));
    }
    if (lane < 32) {
      // tokens past the end of the call leave the state alone: g = 1, beta = 0
      const bool live = t0 + lane < p.T;
      *reinterpret_cast<float2*>(&gbv[lane][0]) = make_float2(live ? gr : 1.f, live ? br : 0.f);
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) gbv[16 * h + (lane >> 2)][4 + (lane & 3)] = vr[h];
  };

  struct Tok {
    float4 k0, k1, q0, q1;
    float2 gb;
    float vt;
  };
  auto token = [&](int i) {
    Tok t;
    t.k0 = *reinterpret_cast<const float4*>(&kq[i][0][4 * j]);
    t.k1 = *reinterpret_cast<const float4*>(&kq[i][0][64 + 4 * j]);
    t.q0 = *reinterpret_cast<const float4*>(&kq[i][1][4 * j]);
    t.q1 = *reinterpret_cast<const float4*>(&kq[i][1][64 + 4 * j]);
    t.gb = *reinterpret_cast<const float2*>(&gbv[i][0]);
    t.vt = gbv[i][4 + row];
    return t;
  };

  fetch(0);
  for (int t0 = 0; t0 < p.T; t0 += C) {
    __syncthreads();  // the steps before have read their tokens
    park(t0);
    __syncthreads();
    if (t0 + C < p.T) fetch(t0 + C);
    Tok cur = token(0);
    for (int h = 0; h < 2; ++h) {
      float yo = 0.f;
#pragma unroll 8
      for (int ii = 0; ii < 16; ++ii) {
        // the next token's operands leave LDS while this one computes (row C is padding)
        const Tok nxt = token(16 * h + ii + 1);
        __builtin_amdgcn_sched_barrier(0);
        const float kf[8] = {cur.k0.x, cur.k0.y, cur.k0.z, cur.k0.w, cur.k1.x, cur.k1.y, cur.k1.z, cur.k1.w};
        const float qf[8] = {cur.q0.x, cur.q0.y, cur.q0.z, cur.q0.w, cur.q1.x, cur.q1.y, cur.q1.z, cur.q1.w};
        const float gt = cur.gb.x, bt = cur.gb.y;
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          a0 = dm_fma(s[e], kf[e], a0);
          a1 = dm_fma(s[4 + e], kf[4 + e], a1);
        }
        const float kv = gt * dm_wave_sum<16>(a0 + a1);  // sum_e (g s_e) k_e
        const float delta = (cur.vt - kv) * bt;
#pragma unroll
        for (int e = 0; e < 8; ++e) s[e] = dm_fma(s[e], gt, kf[e] * delta);
        float o0 = 0.f, o1 = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          o0 = dm_fma(s[e], qf[e], o0);
          o1 = dm_fma(s[4 + e], qf[4 + e], o1);
        }
        const float o = dm_wave_sum<16>(o0 + o1);
        yo = j == ii ? o : yo;  // lane j of a row keeps token j of these sixteen
        cur = nxt;
      }
      const int t = t0 + 16 * h + j;
      if (t < p.T) p.y[((size_t)t * p.Hv + hv) * p.Dv + dv] = dm_f2bf(yo);
    }
  }
  float* snap = p.snapshots + roff;
#pragma unroll
  for (int m = 0; m < 2; ++m)
    *reinterpret_cast<float4*>(snap + 64 * m) = make_float4(s[4 * m + 0], s[4 * m + 1], s[4 * m + 2], s[4 * m + 3]);
}

// ---- the whole mixer core in one launch, decode / verify widths -------------------------
// One workgroup per value head (16 wavefronts):
//   1. every thread issues the loads of its slice of the recurrent state (they depend on
//      nothing), then
//   2. the wavefronts share out the head's front-end work: conv + silu (+ norm, scale) of
//      the head's q, k and v channels for each token, the in_proj_a / in_proj_b dot
//      products of this head, g and beta -- results stay in LDS;
//   3. the recurrence runs on the state registers, reading q, k, v, g, beta from LDS,
//      writing the per-token snapshots and leaving y in LDS;
//   4. one wavefront per token applies the gated RMS norm to the head's 128 outputs.
// Arithmetic and its order are those of gdn_front_kernel, dense_gemv, gdn_recurrence_kernel
// and rms_norm_gated: the fused launch is bit-identical to the four separate ones.
constexpr int kStepMaxT = 16;

struct StepArgs {
  FrontArgs f;
  const bf16_t* wa;      // in_proj_a [Hv, H] dense bf16, or null: f.a_in / f.b_in hold the projections
  const bf16_t* wb;
  const bf16_t* xn;      // [T, H] input of the projections
  int H;
  const float* state_in;  // [Hv, 128, 128]
  float* snapshots;       // [T][Hv, 128, 128]
  int snap_all;
  const bf16_t* norm_w;   // [128]
  const bf16_t* z;        // [T, Hv*128]
  float norm_eps;
  bf16_t* gated;          // [T, Hv*128]
};

#ifdef ORN_TIMING
// debug build only: per-workgroup phase time stamps (100 MHz wall clock) of the last launch
__device__ long long g_gdn_marks[64][8];
#define GDN_MARK(i) do { if (threadIdx.x == 0 && blockIdx.x < 64) g_gdn_marks[blockIdx.x][i] = wall_clock64(); } while (0)
// by lane 0 of wavefront w
#define GDN_MARK_W(i, w) do { if ((int)threadIdx.x == 64 * (w) && blockIdx.x < 64) g_gdn_marks[blockIdx.x][i] = wall_clock64(); } while (0)
#else
#define GDN_MARK(i)
#define GDN_MARK_W(i, w)
#endif

__global__ __launch_bounds__(1024) void gdn_step_kernel(StepArgs a) {
  GDN_MARK(0);
  const FrontArgs& p = a.f;
  __shared__ float qs[kStepMaxT][128], ks[kStepMaxT][128], vs[kStepMaxT][128], ys[kStepMaxT][128];
  __shared__ float gs[kStepMaxT], bs[kStepMaxT];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int hv = blockIdx.x, ratio = p.Hv / p.Hk, hk = hv / ratio;
  const int T = p.T, S = p.K - 1, D = p.D;

  // 1. state slice of this thread: row dv = 8*wave + lane/8, columns 32*m + 4*(lane%8) ..+4
  const int row = lane >> 3, j = lane & 7, dv = wave * 8 + row;
  const size_t ssz = (size_t)p.Hv * 128 * 128;
  const size_t roff = ((size_t)hv * 128 + dv) * 128 + 4 * j;
  // Loads return in issue order, and the state is 64 KB a workgroup straight from memory: asked
  // for first, it would hold back the few cached operands of the front-end tasks until it had
  // arrived, and the front end (conv, norms, projections: 1 - 2 us of dependent arithmetic)
  // would only start then. So a wavefront asks for its first task's operands first, then for
  // what the later phases need, then for its state, and works its task off under the state's
  // trip.
  const int n_conv = 3 * T, n_ab = a.wa ? 2 * T : 0;
  const bool early_conv = wave < n_conv && p.K == 4;
  const bool early_ab = wave >= n_conv && wave < n_conv + n_ab && a.H <= 2048;
  // with more than 16 tasks (four rows: 12 + 8) a conv wavefront's second task is a projection:
  // its operands go out now as well, into the registers a projection wavefront uses
  const bool early_ab2 = !early_ab && wave + 16 >= n_conv && wave + 16 < n_conv + n_ab && a.H <= 2048;
  uint4 e_w8 = make_uint4(0, 0, 0, 0);
  uint32_t e_xv[4] = {0, 0, 0, 0};
  uint4 e_dw[4], e_dx[4];
  if (early_conv) {
    const int which = wave / T, t = wave - which * T;
    const int slot = which == 0 ? hk : which == 1 ? p.Hk + hk : 2 * p.Hk + hv;
    const int c0 = slot * 128 + 2 * lane;
    e_w8 = *reinterpret_cast<const uint4*>(p.cw + (size_t)c0 * 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int jj = t + i;
      const bf16_t* src = (jj < S) ? (p.conv_state + (size_t)jj * D) : (p.qkv + (size_t)(jj - S) * D);
      e_xv[i] = *reinterpret_cast<const uint32_t*>(src + c0);
    }
  }
  if (early_ab || early_ab2) {
    const int u = (early_ab ? wave : wave + 16) - n_conv, which = u / T, t = u - which * T;
    const bf16_t* wr = (which == 0 ? a.wa : a.wb) + (size_t)hv * a.H;
    const bf16_t* xr = a.xn + (size_t)t * a.H;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int jc = lane + 64 * c;
      if (jc < a.H / 8) {
        e_dw[c] = *reinterpret_cast<const uint4*>(wr + 8 * jc);
        e_dx[c] = *reinterpret_cast<const uint4*>(xr + 8 * jc);
      }
    }
  }
  // operands of the later phases that depend on nothing computed here: requested now, so that
  // no phase starts with a trip to memory of its own
  uint32_t wv_pre = 0, zv_pre = 0;
  if (wave < T) {
    wv_pre = *reinterpret_cast<const uint32_t*>(a.norm_w + 2 * lane);
    zv_pre = *reinterpret_cast<const uint32_t*>(a.z + ((size_t)wave * p.Hv + hv) * 128 + 2 * lane);
  }
  const bf16_t dtb_pre = p.dt_bias[hv], alog_pre = p.a_log[hv];
  bf16_t ain_pre = 0, bin_pre = 0;
  if (!a.wa && tid < T) {
    ain_pre = p.a_in[tid * p.Hv + hv];
    bin_pre = p.b_in[tid * p.Hv + hv];
  }
  __builtin_amdgcn_sched_barrier(0);
  float s[16];
#pragma unroll
  for (int m = 0; m < 4; ++m) {
    const float4 f = *reinterpret_cast<const float4*>(a.state_in + roff + 32 * m);
    s[4 * m + 0] = f.x;
    s[4 * m + 1] = f.y;
    s[4 * m + 2] = f.z;
    s[4 * m + 3] = f.w;
  }
  __builtin_amdgcn_sched_barrier(0);
  GDN_MARK(4);  // every request of this wavefront is out
  const float decay_pre = dm_exp(dm_bf2f(alog_pre));  // needs only a parameter: made under the loads

  // 2. front-end tasks: [0, 3T) conv of (q | k | v, token); then the a / b projections
  for (int task = wave; task < n_conv + n_ab; task += 16) {
    if (task < n_conv) {
      const int which = task / T, t = task - which * T;  // 0 q, 1 k, 2 v
      const int slot = which == 0 ? hk : which == 1 ? p.Hk + hk : 2 * p.Hk + hv;
      const int c0 = slot * 128 + 2 * lane;
      float acc0 = 0.f, acc1 = 0.f;
      if (p.K == 4) {
        // the usual window: the four taps of both channels are one 16-byte load, and the four
        // input rows are requested together
        uint4 w8 = e_w8;
        uint32_t xv[4] = {e_xv[0], e_xv[1], e_xv[2], e_xv[3]};
        if (task != wave) {  // a second task of this wavefront (more than 16 tasks): asked for here
          w8 = *reinterpret_cast<const uint4*>(p.cw + (size_t)c0 * 4);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int jj = t + i;
            const bf16_t* src = (jj < S) ? (p.conv_state + (size_t)jj * D) : (p.qkv + (size_t)(jj - S) * D);
            xv[i] = *reinterpret_cast<const uint32_t*>(src + c0);
          }
        }
        acc0 = dm_fma(dm_bf2f_lo(xv[0]), dm_bf2f_lo(w8.x), acc0);
        acc0 = dm_fma(dm_bf2f_lo(xv[1]), dm_bf2f_hi(w8.x), acc0);
        acc0 = dm_fma(dm_bf2f_lo(xv[2]), dm_bf2f_lo(w8.y), acc0);
        acc0 = dm_fma(dm_bf2f_lo(xv[3]), dm_bf2f_hi(w8.y), acc0);
        acc1 = dm_fma(dm_bf2f_hi(xv[0]), dm_bf2f_lo(w8.z), acc1);
        acc1 = dm_fma(dm_bf2f_hi(xv[1]), dm_bf2f_hi(w8.z), acc1);
        acc1 = dm_fma(dm_bf2f_hi(xv[2]), dm_bf2f_lo(w8.w), acc1);
        acc1 = dm_fma(dm_bf2f_hi(xv[3]), dm_bf2f_hi(w8.w), acc1);
      } else {
        for (int i = 0; i < p.K; ++i) {
          const int jj = t + i;
          const bf16_t* src = (jj < S) ? (p.conv_state + (size_t)jj * D) : (p.qkv + (size_t)(jj - S) * D);
          const uint32_t xv = *reinterpret_cast<const uint32_t*>(src + c0);
          acc0 = dm_fma(dm_bf2f_lo(xv), dm_bf2f(p.cw[(size_t)c0 * p.K + i]), acc0);
          acc1 = dm_fma(dm_bf2f_hi(xv), dm_bf2f(p.cw[(size_t)(c0 + 1) * p.K + i]), acc1);
        }
      }
      const float cv0 = dm_rb(acc0), cv1 = dm_rb(acc1);
      const float y0 = dm_rb(cv0 * dm_sigmoid_bf16(cv0)), y1 = dm_rb(cv1 * dm_sigmoid_bf16(cv1));
      // the window: v channels belong to this head alone, q / k channels to the first head of the group
      if (which == 2 || hv % ratio == 0) {
        *reinterpret_cast<uint32_t*>(p.conv_input + (size_t)(S + t) * D + c0) =
            *reinterpret_cast<const uint32_t*>(p.qkv + (size_t)t * D + c0);
        if (t == 0)
          for (int r = 0; r < S; ++r)
            *reinterpret_cast<uint32_t*>(p.conv_input + (size_t)r * D + c0) =
                *reinterpret_cast<const uint32_t*>(p.conv_state + (size_t)r * D + c0);
      }
      if (which < 2) {
        float ss = dm_fma(y0, y0, 0.f);
        ss = dm_fma(y1, y1, ss);
        const float inv = dm_rsqrt(dm_wave_sum<64>(ss) / 128.0f + p.eps);
        const float sc = which == 0 ? p.q_scale : p.k_scale;
        float* dst = which == 0 ? qs[t] : ks[t];
        dst[2 * lane] = dm_rb(sc * dm_rb(y0 * inv));
        dst[2 * lane + 1] = dm_rb(sc * dm_rb(y1 * inv));
      } else {
        vs[t][2 * lane] = y0;
        vs[t][2 * lane + 1] = y1;
      }
    } else {
      const int u = task - n_conv, which = u / T, t = u - which * T;  // 0 a, 1 b
      const bf16_t* wr = (which == 0 ? a.wa : a.wb) + (size_t)hv * a.H;
      float v;
      if ((task == wave && early_ab) || (task == wave + 16 && early_ab2)) {
        // dense_row_dot over the operands asked for at the start: the same chain, the same fold
        float acc = 0.f;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          if (lane + 64 * c < a.H / 8) {
            const uint4 wv4 = e_dw[c], xv4 = e_dx[c];
            acc = dm_fma(dm_bf2f_lo(wv4.x), dm_bf2f_lo(xv4.x), acc);
            acc = dm_fma(dm_bf2f_hi(wv4.x), dm_bf2f_hi(xv4.x), acc);
            acc = dm_fma(dm_bf2f_lo(wv4.y), dm_bf2f_lo(xv4.y), acc);
            acc = dm_fma(dm_bf2f_hi(wv4.y), dm_bf2f_hi(xv4.y), acc);
            acc = dm_fma(dm_bf2f_lo(wv4.z), dm_bf2f_lo(xv4.z), acc);
            acc = dm_fma(dm_bf2f_hi(wv4.z), dm_bf2f_hi(xv4.z), acc);
            acc = dm_fma(dm_bf2f_lo(wv4.w), dm_bf2f_lo(xv4.w), acc);
            acc = dm_fma(dm_bf2f_hi(wv4.w), dm_bf2f_hi(xv4.w), acc);
          }
        }
        v = dm_rb(dm_wave_sum<64>(acc));
      } else {
        v = dm_rb(dense_row_dot<1>(wr, a.xn + (size_t)t * a.H, a.H, lane));
      }
      // the wavefront that made the projection turns it into the token's decay / beta at
      // once: the two chains of exp / log run side by side in different wavefronts instead of
      // one after the other behind a barrier
      if (which == 0) {
        const float sp = softplus_bf16(dm_rb(v + dm_bf2f(dtb_pre)));
        const float g = dm_exp(-decay_pre * sp);
        if (lane == 0) gs[t] = g;
      } else {
        const float bt = dm_rb(dm_sigmoid_bf16(v));
        if (lane == 0) bs[t] = bt;
      }
    }
  }
  GDN_MARK_W(7, 0);       // the first conv task's wavefront is through
  GDN_MARK_W(6, n_conv);  // the first a / b projection's wavefront is through
  if (!a.wa && tid < T) {
    // projections given: decay and beta of token `tid`
    const float sp = softplus_bf16(dm_rb(dm_bf2f(ain_pre) + dm_bf2f(dtb_pre)));
    gs[tid] = dm_exp(-decay_pre * sp);
    bs[tid] = dm_rb(dm_sigmoid_bf16(dm_bf2f(bin_pre)));
  }
  __syncthreads();
  GDN_MARK(1);
  GDN_MARK(2);

  // 3. recurrence (gdn_recurrence_kernel, operands from LDS)
  for (int t = 0; t < T; ++t) {
    float kf[16], qf[16];
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const float4 kv4 = *reinterpret_cast<const float4*>(&ks[t][32 * m + 4 * j]);
      const float4 qv4 = *reinterpret_cast<const float4*>(&qs[t][32 * m + 4 * j]);
      kf[4 * m + 0] = kv4.x; kf[4 * m + 1] = kv4.y; kf[4 * m + 2] = kv4.z; kf[4 * m + 3] = kv4.w;
      qf[4 * m + 0] = qv4.x; qf[4 * m + 1] = qv4.y; qf[4 * m + 2] = qv4.z; qf[4 * m + 3] = qv4.w;
    }
    const float gt = gs[t], bt = bs[t], vt = vs[t][dv];
    float acc = 0.f;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      s[e] = s[e] * gt;
      acc = dm_fma(s[e], kf[e], acc);
    }
    const float kv = dm_wave_sum<8>(acc);
    const float delta = (vt - kv) * bt;
    float o = 0.f;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      s[e] = dm_fma(kf[e], delta, s[e]);
      o = dm_fma(s[e], qf[e], o);
    }
    o = dm_wave_sum<8>(o);
    if (j == 0) ys[t][dv] = dm_rb(o);
    if (a.snap_all || t + 1 == T) {
      float* snap = a.snapshots + (a.snap_all ? (size_t)t * ssz : 0) + roff;
#pragma unroll
      for (int m = 0; m < 4; ++m)
        *reinterpret_cast<float4*>(snap + 32 * m) =
            make_float4(s[4 * m + 0], s[4 * m + 1], s[4 * m + 2], s[4 * m + 3]);
    }
  }
  __syncthreads();
  GDN_MARK(3);

  // 4. gated norm of the head's 128 outputs, one wavefront per token (rms_norm_gated, two
  //    values per lane)
  for (int t = wave; t < T; t += 16) {
    float x0 = ys[t][2 * lane], x1 = ys[t][2 * lane + 1];
    float acc = dm_fma(x0, x0, 0.f);
    acc = dm_fma(x1, x1, acc);
    const float inv = dm_rsqrt(dm_wave_sum<64>(acc) / 128.0f + a.norm_eps);
    const uint32_t wv = wv_pre, zv = zv_pre;  // t == wave: T never exceeds the wavefront count
    const size_t off = ((size_t)t * p.Hv + hv) * 128 + 2 * lane;
    x0 = dm_rb(dm_bf2f_lo(wv) * dm_rb(x0 * inv));
    x1 = dm_rb(dm_bf2f_hi(wv) * dm_rb(x1 * inv));
    const float g0 = dm_bf2f_lo(zv), g1 = dm_bf2f_hi(zv);
    x0 = (g0 * dm_sigmoid_f32(g0)) * x0;
    x1 = (g1 * dm_sigmoid_f32(g1)) * x1;
    *reinterpret_cast<uint32_t*>(a.gated + off) = (uint32_t)dm_f2bf(x0) | ((uint32_t)dm_f2bf(x1) << 16);
  }
  GDN_MARK(5);
}

}  // namespace

#ifdef ORN_TIMING
extern "C" __attribute__((visibility("default"))) int ornith_debug_marks_gdn(long long* out) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_gdn_marks), sizeof(long long) * 64 * 8);
}
#endif

// fills the front-end part of the arguments (shared by gdn_front and gdn_step)
static void fill_front(FrontArgs& p, const void* d_conv_state, const void* d_qkv, const void* d_cw,
                       const void* d_a, const void* d_b, const void* d_a_log, const void* d_dt_bias, int T,
                       int K, int Hk, int Dk, int Hv, float eps, void* d_q, void* d_k, void* d_v,
                       void* d_beta, float* d_g, void* d_conv_input) {
  p.conv_state = (const bf16_t*)d_conv_state;
  p.qkv = (const bf16_t*)d_qkv;
  p.cw = (const bf16_t*)d_cw;
  p.a_in = (const bf16_t*)d_a;
  p.b_in = (const bf16_t*)d_b;
  p.a_log = (const bf16_t*)d_a_log;
  p.dt_bias = (const bf16_t*)d_dt_bias;
  p.q = (bf16_t*)d_q;
  p.k = (bf16_t*)d_k;
  p.v = (bf16_t*)d_v;
  p.beta = (bf16_t*)d_beta;
  p.g = d_g;
  p.conv_input = (bf16_t*)d_conv_input;
  p.T = T;
  p.K = K;
  p.Hk = Hk;
  p.Hv = Hv;
  p.D = 2 * Hk * 128 + Hv * 128;
  const float inv_scale = 1.0f / sqrtf((float)Dk);
  // both scales are applied as bf16 values (the reference casts them to T)
  uint32_t u;
  float f = inv_scale * inv_scale;
  memcpy(&u, &f, 4);
  u = (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u;
  memcpy(&p.q_scale, &u, 4);
  f = inv_scale;
  memcpy(&u, &f, 4);
  u = (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u;
  memcpy(&p.k_scale, &u, 4);
  p.eps = eps;
}

// gdn_chunk.hip
int gdn_chunked_recurrence(ornith_ctx* ctx, const void* d_q, const void* d_k, const void* d_v, const float* d_g,
                           const void* d_beta, const float* d_state_in, int T, int Hk, int Hv, int Dk, int Dv,
                           void* d_y, float* d_state_out);
constexpr int kChunkedRows = 128;  // from here a call's recurrence runs in 64-token chunks

extern "C" {

int ornith_gdn_step(ornith_ctx* ctx, const void* d_conv_state, const void* d_qkv, const void* d_cw,
                    const void* d_a, const void* d_b, const void* d_wa, const void* d_wb, const void* d_xn,
                    int H, const void* d_a_log, const void* d_dt_bias, int T, int K, int Hk, int Dk, int Hv,
                    int Dv, float eps, const float* d_state_in, float* d_snapshots, int snapshot_every_token,
                    const void* d_norm_w, const void* d_z, float norm_eps, void* d_conv_input,
                    void* d_gated_out) {
  ORN_REQUIRE(ctx && d_conv_state && d_qkv && d_cw && d_a_log && d_dt_bias && d_state_in && d_snapshots &&
                  d_norm_w && d_z && d_conv_input && d_gated_out,
              "gdn_step: null argument");
  ORN_REQUIRE((d_wa && d_wb && d_xn && H >= 8 && H % 8 == 0) || (!d_wa && !d_wb && d_a && d_b),
              "gdn_step: give either the a / b projections or their weights and input");
  ORN_REQUIRE(Dk == 128 && Dv == 128, "gdn_step: head dims %d/%d (128 only)", Dk, Dv);
  ORN_REQUIRE(T >= 1 && T <= kStepMaxT && K >= 2 && K <= 8 && Hk >= 1 && Hv >= Hk && Hv % Hk == 0,
              "gdn_step: T=%d (1..%d) K=%d Hk=%d Hv=%d", T, kStepMaxT, K, Hk, Hv);
  ORN_REQUIRE(d_conv_input != d_conv_state, "gdn_step: conv_input must not alias conv_state");
  StepArgs a{};
  fill_front(a.f, d_conv_state, d_qkv, d_cw, d_a, d_b, d_a_log, d_dt_bias, T, K, Hk, Dk, Hv, eps, nullptr,
             nullptr, nullptr, nullptr, nullptr, d_conv_input);
  a.wa = (const bf16_t*)d_wa;
  a.wb = (const bf16_t*)d_wb;
  a.xn = (const bf16_t*)d_xn;
  a.H = H;
  a.state_in = d_state_in;
  a.snapshots = d_snapshots;
  a.snap_all = snapshot_every_token ? 1 : 0;
  a.norm_w = (const bf16_t*)d_norm_w;
  a.z = (const bf16_t*)d_z;
  a.norm_eps = norm_eps;
  a.gated = (bf16_t*)d_gated_out;
  hipLaunchKernelGGL(gdn_step_kernel, dim3(Hv), dim3(1024), 0, ctx->stream, a);
  ORN_LAUNCH_CHECK("gdn_step_kernel");
  return ORNITH_OK;
}

int ornith_gdn_front(ornith_ctx* ctx, const void* d_conv_state, const void* d_qkv, const void* d_cw,
                     const void* d_a, const void* d_b, const void* d_a_log, const void* d_dt_bias,
                     int T, int K, int Hk, int Dk, int Hv, int Dv, float eps, void* d_q, void* d_k,
                     void* d_v, void* d_beta, float* d_g, void* d_conv_input) {
  ORN_REQUIRE(ctx && d_conv_state && d_qkv && d_cw && d_a && d_b && d_a_log && d_dt_bias && d_q &&
                  d_k && d_v && d_beta && d_g && d_conv_input,
              "gdn_front: null argument");
  ORN_REQUIRE(Dk == 128 && Dv == 128, "gdn_front: head dims %d/%d (128 only)", Dk, Dv);
  ORN_REQUIRE(T >= 1 && T <= 65535 && K >= 2 && K <= 8 && Hk >= 1 && Hv >= Hk && Hv % Hk == 0,
              "gdn_front: T=%d K=%d Hk=%d Hv=%d", T, K, Hk, Hv);
  ORN_REQUIRE(d_conv_input != d_conv_state, "gdn_front: conv_input must not alias conv_state");
  FrontArgs p{};
  p.conv_state = (const bf16_t*)d_conv_state;
  p.qkv = (const bf16_t*)d_qkv;
  p.cw = (const bf16_t*)d_cw;
  p.a_in = (const bf16_t*)d_a;
  p.b_in = (const bf16_t*)d_b;
  p.a_log = (const bf16_t*)d_a_log;
  p.dt_bias = (const bf16_t*)d_dt_bias;
  p.q = (bf16_t*)d_q;
  p.k = (bf16_t*)d_k;
  p.v = (bf16_t*)d_v;
  p.beta = (bf16_t*)d_beta;
  p.g = d_g;
  p.conv_input = (bf16_t*)d_conv_input;
  p.T = T;
  p.K = K;
  p.Hk = Hk;
  p.Hv = Hv;
  p.D = 2 * Hk * 128 + Hv * 128;
  const float inv_scale = 1.0f / sqrtf((float)Dk);
  // both scales are applied as bf16 values (the reference casts them to T)
  uint32_t u;
  float f = inv_scale * inv_scale;
  memcpy(&u, &f, 4);
  u = (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u;
  memcpy(&p.q_scale, &u, 4);
  f = inv_scale;
  memcpy(&u, &f, 4);
  u = (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u;
  memcpy(&p.k_scale, &u, 4);
  p.eps = eps;
  if (p.K == 4 && T >= 2 * kFrontRun)
    hipLaunchKernelGGL(gdn_front_run_kernel, dim3(p.D / 128, (T + kFrontRun - 1) / kFrontRun), dim3(64), 0,
                       ctx->stream, p);
  else
    hipLaunchKernelGGL(gdn_front_kernel, dim3(p.D / 128, T), dim3(64), 0, ctx->stream, p);
  ORN_LAUNCH_CHECK("gdn_front_kernel");
  return ORNITH_OK;
}

int ornith_gdn_recurrence(ornith_ctx* ctx, const void* d_q, const void* d_k, const void* d_v,
                          const float* d_g, const void* d_beta, const float* d_state_in, int T,
                          int Hk, int Hv, int Dk, int Dv, void* d_y, float* d_snapshots,
                          int snapshot_every_token) {
  ORN_REQUIRE(ctx && d_q && d_k && d_v && d_g && d_beta && d_state_in && d_y && d_snapshots,
              "gdn_recurrence: null argument");
  ORN_REQUIRE(Dk == 128 && Dv % 8 == 0 && Dv >= 8, "gdn_recurrence: Dk=%d Dv=%d", Dk, Dv);
  ORN_REQUIRE(T >= 1 && Hk >= 1 && Hv >= Hk && Hv % Hk == 0 && Hv <= 65535,
              "gdn_recurrence: T=%d Hk=%d Hv=%d", T, Hk, Hv);
  RecArgs p{(const bf16_t*)d_q, (const bf16_t*)d_k, (const bf16_t*)d_v, d_g, (const bf16_t*)d_beta,
            d_state_in,         (bf16_t*)d_y,       d_snapshots,        T,   Hk, Hv, Dv,
            snapshot_every_token ? 1 : 0};
  if (T >= kChunkedRows && !snapshot_every_token && ornith_option_gdn_chunked()) {
    // long prompt chunks: the chunked form on the matrix cores (agrees to rounding)
    const int rc = gdn_chunked_recurrence(ctx, d_q, d_k, d_v, d_g, d_beta, d_state_in, T, Hk, Hv, Dk, Dv, d_y,
                                          d_snapshots);
    if (rc != -1) return rc;
  }
  if (T >= kPrefillRows && !snapshot_every_token) {
    // prompt chunks: the form with the short dependent chain (agrees to rounding)
    hipLaunchKernelGGL(gdn_recurrence_wide_kernel, dim3(Dv / 4, Hv), dim3(64), 0, ctx->stream, p);
    ORN_LAUNCH_CHECK("gdn_recurrence_wide_kernel");
    return ORNITH_OK;
  }
  hipLaunchKernelGGL(gdn_recurrence_kernel, dim3(Dv / 8, Hv), dim3(64), 0, ctx->stream, p);
  ORN_LAUNCH_CHECK("gdn_recurrence_kernel");
  return ORNITH_OK;
}

}  // extern "C"
