// Causal attention at prefill width on the matrix cores (flash-attention form).
//
// Replaces sdpa_unfused (/root/reference/src/ops/sdpa.rs:386-461) for the rows of a prompt
// chunk: scores = scale * q . k^T over the cached keys [0, offset + t], causal inside the
// chunk, precise softmax, . v, then the output gate sigmoid(gate) of
// Attention::forward (/root/reference/src/model/qwen3_5.rs:455-474). The decode / verify
// widths keep the exact split-K kernel of attn.hip; like every prefill kernel this one
// agrees with it to rounding, not bit for bit.
//
// One workgroup = 64 query rows of one head; each of its four wavefronts owns 16 rows and
// walks the key blocks (64 keys) with the online softmax, so no wavefront ever waits for
// another's row statistics:
//   S[16 x 64]   = Q[16 x 256] . K^T      8 x 4 v_mfma_f32_16x16x32_bf16 (Q fragments live in
//                                           registers for the whole kernel)
//   P = exp(S - m), rescale O and l        fp32, in the MFMA accumulator layout
//   O[16 x 256] += P[16 x 64] . V          P goes through 2 KB of LDS to become an A operand;
//                                           V is stored transposed in LDS so that a B fragment
//                                           (8 consecutive keys of one channel) is 16 bytes
// K and V blocks are shared by the four wavefronts through LDS; the 8 query heads of a kv
// head re-read them from L2.
#include "dmath.h"
#include "rt.h"

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

constexpr int HD = 256, BQ = 64, BKV = 64;
constexpr int LDK = HD + 8, LDV = BKV + 8, LDP = BKV + 8;

struct FaArgs {
  const bf16_t* q_rot;    // [T, Hq, HD]
  const bf16_t* k_cache;  // [Hkv, cap, HD]
  const bf16_t* v_cache;
  const bf16_t* qg;       // [T, Hq, 2*HD], gate in the second half
  bf16_t* out;            // [T, Hq*HD]
  int T, Hq, Hkv, offset, cap;
  float scale;
};

__device__ __forceinline__ float max16(float v) {  // over the 16 lanes sharing lane / 16
  v = fmaxf(v, dm_xor_lane<1>(v));
  v = fmaxf(v, dm_xor_lane<2>(v));
  v = fmaxf(v, dm_xor_lane<4>(v));
  v = fmaxf(v, dm_xor_lane<8>(v));
  return v;
}
__device__ __forceinline__ float sum16(float v) {
  v = v + dm_xor_lane<1>(v);
  v = v + dm_xor_lane<2>(v);
  v = v + dm_xor_lane<4>(v);
  v = v + dm_xor_lane<8>(v);
  return v;
}

__global__ __launch_bounds__(256) void sdpa_prefill_kernel(FaArgs p) {
  __shared__ __attribute__((aligned(16))) bf16_t Ks[BKV][LDK];
  __shared__ __attribute__((aligned(16))) bf16_t Vt[HD][LDV];
  __shared__ __attribute__((aligned(16))) bf16_t Ps[4][16][LDP];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, lg = lane >> 4;  // column / row group inside a 16x16 tile
  const int h = blockIdx.y, hk = h / (p.Hq / p.Hkv);
  const int q0 = blockIdx.x * BQ, r0 = q0 + 16 * wave;
  const int last_row = min(p.T, q0 + BQ) - 1;
  const int n_kb = (p.offset + last_row) / BKV + 1;
  const int n_keys = p.offset + p.T;  // keys present in the cache for this call

  // Q fragments: row r0 + l16, channels 32*ks + 8*lg .. +8
  bf16x8_t qf[HD / 32];
  {
    const int row = r0 + l16;
    const bf16_t* qp = p.q_rot + ((size_t)min(row, p.T - 1) * p.Hq + h) * HD + 8 * lg;
#pragma unroll
    for (int ks = 0; ks < HD / 32; ++ks) qf[ks] = *reinterpret_cast<const bf16x8_t*>(qp + 32 * ks);
  }
  f32x4_t o[HD / 16];
#pragma unroll
  for (int t = 0; t < HD / 16; ++t) o[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m_i[4], l_i[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    m_i[i] = -DM_INF;
    l_i[i] = 0.f;
  }

  const bf16_t* kbase = p.k_cache + (size_t)hk * p.cap * HD;
  const bf16_t* vbase = p.v_cache + (size_t)hk * p.cap * HD;
  // A key block travels in registers one block ahead of its use. Keys: thread = (key tid/32 + 8i,
  // 8-channel piece tid%32), stored as they are. Values: thread = (8 keys 8*(lane%8).., piece
  // tid/8), an 8 x 8 tile that is transposed in registers, so each channel's 8 keys go to LDS as
  // one 16-byte store.
  constexpr int NPC = BKV * HD / 8 / 256;  // 8 pieces of each kind per thread
  static_assert(NPC == 8, "one 8 x 8 value tile per thread");
  typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
  const int vkg = lane & 7, vc8 = tid >> 3;
  u32x4_t kr[NPC], vr[NPC];
  auto fetch = [&](int kb) {
#pragma unroll
    for (int i = 0; i < NPC; ++i) {
      const int kkey = kb * BKV + (tid >> 5) + 8 * i, vkey = kb * BKV + 8 * vkg + i;
      kr[i] = u32x4_t{0, 0, 0, 0};
      vr[i] = u32x4_t{0, 0, 0, 0};
      if (kkey < n_keys) kr[i] = *reinterpret_cast<const u32x4_t*>(kbase + (size_t)kkey * HD + 8 * (tid & 31));
      if (vkey < n_keys) vr[i] = *reinterpret_cast<const u32x4_t*>(vbase + (size_t)vkey * HD + 8 * vc8);
    }
  };
  fetch(0);
  for (int kb = 0; kb < n_kb; ++kb) {
    // ---- K block as is, V block transposed
#pragma unroll
    for (int i = 0; i < NPC; ++i)
      *reinterpret_cast<u32x4_t*>(&Ks[(tid >> 5) + 8 * i][8 * (tid & 31)]) = kr[i];
#pragma unroll
    for (int ch = 0; ch < 8; ++ch) {
      const int w = ch >> 1;
      const unsigned sel = (ch & 1) ? 0x07060302u : 0x05040100u;  // high / low halves of a word pair
      u32x4_t col;
#pragma unroll
      for (int kp = 0; kp < 4; ++kp)
        col[kp] = __builtin_amdgcn_perm(vr[2 * kp + 1][w], vr[2 * kp][w], sel);
      *reinterpret_cast<u32x4_t*>(&Vt[8 * vc8 + ch][8 * vkg]) = col;
    }
    __syncthreads();
    if (kb + 1 < n_kb) fetch(kb + 1);  // in flight under this block's matrix work

    // ---- S = Q K^T
    f32x4_t s[BKV / 16];
#pragma unroll
    for (int nt = 0; nt < BKV / 16; ++nt) s[nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < HD / 32; ++ks)
#pragma unroll
      for (int nt = 0; nt < BKV / 16; ++nt) {
        const bf16x8_t kf = *reinterpret_cast<const bf16x8_t*>(&Ks[nt * 16 + l16][32 * ks + 8 * lg]);
        s[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[ks], kf, s[nt], 0, 0, 0);
      }
    // ---- online softmax on rows 4*lg + i of this wavefront's 16
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int pos = p.offset + r0 + 4 * lg + i;
      float mx = -DM_INF;
#pragma unroll
      for (int nt = 0; nt < BKV / 16; ++nt) {
        const int key = kb * BKV + nt * 16 + l16;
        const float v = key <= pos ? s[nt][i] * p.scale : -DM_INF;
        s[nt][i] = v;
        mx = fmaxf(mx, v);
      }
      mx = max16(mx);
      const float m_new = fmaxf(m_i[i], mx);
      const float alpha = m_new == -DM_INF ? 1.f : __expf(m_i[i] - m_new);
      float rs = 0.f;
#pragma unroll
      for (int nt = 0; nt < BKV / 16; ++nt) {
        const float pv = m_new == -DM_INF ? 0.f : __expf(s[nt][i] - m_new);
        s[nt][i] = pv;
        rs += pv;
      }
      rs = sum16(rs);
      l_i[i] = l_i[i] * alpha + rs;
      m_i[i] = m_new;
#pragma unroll
      for (int t = 0; t < HD / 16; ++t) o[t][i] *= alpha;
#pragma unroll
      for (int nt = 0; nt < BKV / 16; ++nt) Ps[wave][4 * lg + i][nt * 16 + l16] = dm_f2bf(s[nt][i]);
    }
    __syncthreads();
    // ---- O += P V
#pragma unroll
    for (int k2 = 0; k2 < BKV / 32; ++k2) {
      const bf16x8_t pf = *reinterpret_cast<const bf16x8_t*>(&Ps[wave][l16][32 * k2 + 8 * lg]);
#pragma unroll
      for (int t = 0; t < HD / 16; ++t) {
        const bf16x8_t vf = *reinterpret_cast<const bf16x8_t*>(&Vt[t * 16 + l16][32 * k2 + 8 * lg]);
        o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, vf, o[t], 0, 0, 0);
      }
    }
    __syncthreads();
  }

  // ---- normalise, gate, store: rows 4*lg + i, channels 16*t + l16
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = r0 + 4 * lg + i;
    if (row >= p.T) continue;
    const float inv = 1.0f / l_i[i];
    const bf16_t* gate = p.qg + ((size_t)row * p.Hq + h) * 2 * HD + HD;
    bf16_t* dst = p.out + ((size_t)row * p.Hq + h) * HD;
#pragma unroll
    for (int t = 0; t < HD / 16; ++t) {
      const int d = 16 * t + l16;
      const float att = dm_rb(o[t][i] * inv);
      const float g = dm_sigmoid_bf16(dm_bf2f(gate[d]));
      dst[d] = dm_f2bf(g * att);
    }
  }
}

}  // namespace

extern "C" int ornith_sdpa_prefill_gated(ornith_ctx* ctx, const void* d_q_rot, const void* d_k_cache,
                                         const void* d_v_cache, const void* d_qg, int T, int Hq, int Hkv,
                                         int hd, int offset, int cap, float scale, void* d_out) {
  ORN_REQUIRE(ctx && d_q_rot && d_k_cache && d_v_cache && d_qg && d_out, "sdpa_prefill: null argument");
  ORN_REQUIRE(hd == HD, "sdpa_prefill: head_dim %d (256 only; other widths use sdpa_decode_gated)", hd);
  ORN_REQUIRE(T >= 1 && Hq >= 1 && Hkv >= 1 && Hq % Hkv == 0 && Hq <= 65535, "sdpa_prefill: T=%d Hq=%d Hkv=%d",
              T, Hq, Hkv);
  ORN_REQUIRE(offset >= 0 && offset + T <= cap, "sdpa_prefill: rows [%d,%d) exceed cache capacity %d", offset,
              offset + T, cap);
  FaArgs p{(const bf16_t*)d_q_rot, (const bf16_t*)d_k_cache, (const bf16_t*)d_v_cache, (const bf16_t*)d_qg,
           (bf16_t*)d_out, T, Hq, Hkv, offset, cap, scale};
  hipLaunchKernelGGL(sdpa_prefill_kernel, dim3((T + BQ - 1) / BQ, Hq), dim3(256), 0, ctx->stream, p);
  ORN_LAUNCH_CHECK("sdpa_prefill_kernel");
  return ORNITH_OK;
}
