// Device-side router: precise softmax (fp32 inside, bf16 out) and top-k selection for
// one token by one wavefront. Shared by the stand-alone router kernel and the fused
// router launch.
//
// Restates vendored softmax.h:10-98 and /root/reference/kernels/moe.metal:568-614:
// p = bf16(exp(g - max) * (1 / sum)); k rounds of selection under "by value, then by
// larger index"; round r fills slot k-1-r, so the slots are the tail of a stable
// ascending sort.
#pragma once

#include "dmath.h"

// swiglu of one gate / up pair as the separate operators leave it: both mat-vec outputs rounded
// to bf16, silu and the product in bf16 steps
// (/root/reference/kernels/ornith_elementwise.metal:97-105)
__device__ __forceinline__ bf16_t swiglu_bf16(float g, float u) {
  const float gb = dm_rb(g), ub = dm_rb(u);
  const float s = dm_rb(gb * dm_sigmoid_bf16(gb));
  return dm_f2bf(s * ub);
}

#ifndef ORN_TOPK_STAMP
#define ORN_TOPK_STAMP()
#endif

template <int S>
__device__ __forceinline__ uint32_t dm_xor_lane_u32(uint32_t v) {
  return __builtin_bit_cast(uint32_t, dm_xor_lane<S>(__builtin_bit_cast(float, v)));
}
__device__ __forceinline__ uint32_t dm_wave_max_u32(uint32_t v) {
  float a, b;
  dm_row_swap<32>(__builtin_bit_cast(float, v), a, b);
  v = max(__builtin_bit_cast(uint32_t, a), __builtin_bit_cast(uint32_t, b));
  dm_row_swap<16>(__builtin_bit_cast(float, v), a, b);
  v = max(__builtin_bit_cast(uint32_t, a), __builtin_bit_cast(uint32_t, b));
  // max() with a DPP operand is one instruction a step; after the step over 8 the value
  // repeats every 8 lanes, so a rotate by 4 stands for the exchange with lane l ^ 4
  v = max(v, dm_xor_lane_u32<8>(v));
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x124, 0xF, 0xF, false));
  v = max(v, dm_xor_lane_u32<2>(v));
  v = max(v, dm_xor_lane_u32<1>(v));
  return v;
}

// max over the 64 lanes with v_max_f32 (NaN operands lose, as under `v > m ? v : m`; +0 / -0 may
// come out with the other sign, which exp(v - m) does not see)
__device__ __forceinline__ float router_wave_max(float v) {
  float a, b;
  dm_row_swap<32>(v, a, b);
  v = __builtin_fmaxf(a, b);
  dm_row_swap<16>(v, a, b);
  v = __builtin_fmaxf(a, b);
  v = __builtin_fmaxf(v, dm_xor_lane<8>(v));
  v = __builtin_fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xF, 0xF, false)));
  v = __builtin_fmaxf(v, dm_xor_lane<2>(v));
  v = __builtin_fmaxf(v, dm_xor_lane<1>(v));
  return v;
}

// Lane l holds gates [l*PER, (l+1)*PER) of the row. All 64 lanes must be active.
// E = 64 * PER <= 1024 so an index fits 10 bits: a candidate is the single integer
// (bf16 probability bits << 16 | index) + 1, whose order is exactly (value, index) for
// the non-negative probabilities a softmax produces; 0 marks a taken entry.
// COH: the gates were written by other workgroups of this launch (handoff.h) and are read
// with agent-scope loads.
template <int PER, bool COH = false>
__device__ __forceinline__ void router_topk_wave(const bf16_t* gates_row, int k, uint32_t* inds_row,
                                                 bf16_t* scores_row, bf16_t* probs_row, int lane) {
  const bf16_t* g = gates_row + lane * PER;
  float v[PER];
  float m = -DM_INF;
  if constexpr (COH) {
    if constexpr (PER == 1) {
      v[0] = dm_bf2f(__hip_atomic_load(g, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    } else if constexpr (PER == 2) {
      const uint32_t w = __hip_atomic_load(reinterpret_cast<const uint32_t*>(g), __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
      v[0] = dm_bf2f_lo(w);
      v[1] = dm_bf2f_hi(w);
    } else {
#pragma unroll
      for (int q = 0; q < PER / 4; ++q) {
        const uint64_t w = __hip_atomic_load(reinterpret_cast<const uint64_t*>(g) + q, __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT);
        v[4 * q + 0] = dm_bf2f_lo((uint32_t)w);
        v[4 * q + 1] = dm_bf2f_hi((uint32_t)w);
        v[4 * q + 2] = dm_bf2f_lo((uint32_t)(w >> 32));
        v[4 * q + 3] = dm_bf2f_hi((uint32_t)(w >> 32));
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < PER; ++i) v[i] = dm_bf2f(g[i]);
  }
#pragma unroll
  for (int i = 0; i < PER; ++i) m = __builtin_fmaxf(m, v[i]);
  m = router_wave_max(m);
  ORN_TOPK_STAMP();  // debug builds: the gates are in registers here
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    v[i] = dm_exp(v[i] - m);
    s = s + v[i];
  }
  const float inv = 1.0f / dm_wave_sum<64>(s);
  uint32_t key[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const bf16_t pb = dm_f2bf(v[i] * inv);
    if (probs_row) probs_row[lane * PER + i] = pb;
    // a NaN probability (NaN gates) never wins
    key[i] = (pb & 0x7fffu) > 0x7f80u ? 0u : ((((uint32_t)(pb & 0x7fffu)) << 16) | (uint32_t)(lane * PER + i)) + 1u;
  }
  // the lane's keys in descending order (odd-even transposition), so that a round's candidate is
  // key[0] and the lane that wins shifts its list up by one
#pragma unroll
  for (int pass = 0; pass < PER; ++pass)
#pragma unroll
    for (int i = pass & 1; i + 1 < PER; i += 2) {
      const uint32_t hi = max(key[i], key[i + 1]), lo = min(key[i], key[i + 1]);
      key[i] = hi;
      key[i + 1] = lo;
    }
  uint32_t mine = 0;  // lane r keeps round r's winner; one store after the rounds
  for (int r = 0; r < k; ++r) {
    const uint32_t win = dm_wave_max_u32(key[0]);
    // keys are distinct (the index is in them) unless 0; the winner's list moves up through a
    // lane mask (bit selects: no condition register between the steps)
    const uint32_t stay = key[0] == win ? 0u : 0xffffffffu;
#pragma unroll
    for (int i = 0; i + 1 < PER; ++i) key[i] = (key[i] & stay) | (key[i + 1] & ~stay);
    key[PER - 1] &= stay;
    mine = lane == r ? win : mine;
  }
  if (lane < k) {
    const uint32_t w = mine - 1u;  // mine == 0 only if every entry is NaN / taken: id wraps, clamped by users
    inds_row[k - 1 - lane] = mine ? (w & 0xffffu) : 0xffffffffu;
    scores_row[k - 1 - lane] = mine ? (bf16_t)(w >> 16) : (bf16_t)0;
  }
}
