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
// another's row statistics. K and V blocks are shared by the four wavefronts through LDS (V
// transposed, so that 8 keys of one channel are 16 bytes); the 8 query heads of a kv head
// re-read them from L2. The products and their operand layouts are described in the kernel.
#include "dmath.h"
#include "rt.h"

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

constexpr int HD = 256, BQ = 64, BKV = 64;
constexpr int LDK = HD + 8, LDV = BKV + 8;

struct FaArgs {
  const bf16_t* q_rot;    // [T, Hq, HD]
  const bf16_t* k_cache;  // [Hkv, cap, HD]
  const bf16_t* v_cache;
  const bf16_t* qg;       // [T, Hq, 2*HD], gate in the second half
  bf16_t* out;            // [T, Hq*HD]
  int T, Hq, Hkv, offset, cap;
  float scale;
};

#ifdef ORN_TIMING
__device__ long long g_fa_marks[1024][8];
#define FA_MARK(i) do { if (threadIdx.x == 0 && blockIdx.y == 3 && blockIdx.x < 1024 && kb == 40) g_fa_marks[blockIdx.x][i] = wall_clock64(); } while (0)
extern "C" __attribute__((visibility("default"))) int ornith_debug_marks_fa(long long* out) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_fa_marks), sizeof(g_fa_marks));
}
#else
#define FA_MARK(i)
#endif

// position of key j (0..31) of a 32-key group in a row of Vt: the order in which the lanes of
// the transposed score tiles hold the keys (see below)
__device__ __forceinline__ int vt_pos(int j) { return 8 * ((j & 15) >> 2) + 4 * (j >> 4) + (j & 3); }

// G: 16-row groups a wavefront owns (the workgroup covers 64 * G query rows). With two, every
// K and V fragment read from LDS feeds two MFMAs and a key block is loaded once for 128 rows:
// both the LDS and the L1 traffic per flop halve, at one wavefront a SIMD.
template <int G>
__global__ __launch_bounds__(256) void sdpa_prefill_kernel(FaArgs p) {
  __shared__ __attribute__((aligned(16))) bf16_t Ks[BKV][LDK];
  __shared__ __attribute__((aligned(16))) bf16_t Vt[HD][LDV];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, lg = lane >> 4;
  // workgroups start in the order of their number: the longest (last rows of a causal chunk)
  // first, over all heads, and the heads of one KV group next to each other
  const int wg = (int)blockIdx.x + (int)gridDim.x * (int)blockIdx.y;
  const int h = wg % p.Hq, hk = h / (p.Hq / p.Hkv);
  const int qb = (int)gridDim.x - 1 - wg / p.Hq;
  const int q0 = qb * BQ * G, r0 = q0 + 16 * G * wave;  // group g: rows r0 + 16 * g + l16
  const int last_row = min(p.T, q0 + BQ * G) - 1;
  const int n_kb = (p.offset + last_row) / BKV + 1;
  const int n_keys = p.offset + p.T;  // keys present in the cache for this call

  // Both products run transposed, so that a LANE owns a query row (row r0 + l16) from the
  // scores to the output and the probabilities never leave the registers:
  //   S^T[key, row] = K . Q^T   A = K fragment (16 keys x 32 channels, from LDS), B = Q fragment
  //                             (the row's channels 32*ks + 8*lg .. + 8, in registers throughout);
  //                             the lane then holds keys 16*nt + 4*lg + r of its row
  //   O^T[ch, row] += V^T . P^T A = V^T fragment (16 channels x 32 keys, from LDS), B = the lane's
  //                             eight probabilities of key group k2: keys 32*k2 + 4*lg + r and
  //                             32*k2 + 16 + 4*lg + r. An MFMA does not care in which order the
  //                             k index runs as long as both operands agree, so V^T is stored
  //                             with its keys in that order (vt_pos) and stays one 16-byte read.
  // Row maximum and sum are then one value a lane, reduced over the four lanes of a row.
  bf16x8_t qf[G][HD / 32];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const int row = r0 + 16 * g + l16;
    const bf16_t* qp = p.q_rot + ((size_t)min(row, p.T - 1) * p.Hq + h) * HD + 8 * lg;
#pragma unroll
    for (int ks = 0; ks < HD / 32; ++ks) qf[g][ks] = *reinterpret_cast<const bf16x8_t*>(qp + 32 * ks);
  }
  f32x4_t o[G][HD / 16];  // o[g][t][r]: channel 16*t + 4*lg + r of the lane's row of group g
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int t = 0; t < HD / 16; ++t) o[g][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  // base-2 exponentials: exp(scale * (s - m)) = exp2(s * c2 - m * c2) with c2 = scale * log2(e)
  constexpr float kNone = -1e30f;
  const float c2 = p.scale * 1.44269504088896340736f;
  float m_i[G], l_i[G];  // l_i: this lane's share of the row sum
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m_i[g] = kNone;
    l_i[g] = 0.f;
  }

  const bf16_t* kbase = p.k_cache + (size_t)hk * p.cap * HD;
  const bf16_t* vbase = p.v_cache + (size_t)hk * p.cap * HD;
  // A key block travels in registers one block ahead of its use. Keys: thread = (key tid/32 + 8i,
  // 8-channel piece tid%32), stored as they are. Values: thread = (8 keys 8*(lane%8).., piece
  // tid/8), an 8 x 8 tile that is transposed in registers, so each channel's 8 keys go to LDS as
  // two 8-byte stores (keys 8*vkg .. + 4 and + 4 .. + 8 are 8 positions apart in vt_pos order).
  constexpr int NPC = BKV * HD / 8 / 256;  // 8 pieces of each kind per thread
  static_assert(NPC == 8, "one 8 x 8 value tile per thread");
  typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
  typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
  const int vkg = lane & 7, vc8 = tid >> 3;
  const int vcol = 32 * (vkg >> 2) + vt_pos(8 * (vkg & 3));
  u32x4_t kr[NPC], vr[NPC];
  // (keys past the end of the cache's filled part read the last filled row instead: causal
  // masking keeps every row from them, and no load needs a branch)
  auto fetch_k = [&](int kb) {
#pragma unroll
    for (int i = 0; i < NPC; ++i) {
      const int kkey = min(kb * BKV + (tid >> 5) + 8 * i, n_keys - 1);
      kr[i] = *reinterpret_cast<const u32x4_t*>(kbase + (size_t)kkey * HD + 8 * (tid & 31));
    }
  };
  auto fetch_v = [&](int kb) {
#pragma unroll
    for (int i = 0; i < NPC; ++i) {
      const int vkey = min(kb * BKV + 8 * vkg + i, n_keys - 1);
      vr[i] = *reinterpret_cast<const u32x4_t*>(vbase + (size_t)vkey * HD + 8 * vc8);
    }
  };
  fetch_k(0);
  fetch_v(0);
  for (int kb = 0; kb < n_kb; ++kb) {
    FA_MARK(0);
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
      *reinterpret_cast<u32x2_t*>(&Vt[8 * vc8 + ch][vcol]) = u32x2_t{col[0], col[1]};
      *reinterpret_cast<u32x2_t*>(&Vt[8 * vc8 + ch][vcol + 8]) = u32x2_t{col[2], col[3]};
    }
    FA_MARK(1);
    __syncthreads();
    FA_MARK(2);
    // the next block's keys and values are asked for under this block's matrix work (past the
    // last block the same block again, to no effect)
    const int kb_next = min(kb + 1, n_kb - 1);
    fetch_k(kb_next);
    __builtin_amdgcn_sched_barrier(0);

    // ---- S^T = K Q^T
    f32x4_t st[G][BKV / 16];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int nt = 0; nt < BKV / 16; ++nt) st[g][nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    {
      // the fragments of step ks + 1 leave LDS while the matrix cores work on step ks
      bf16x8_t kf[2][BKV / 16];
      auto kfrags = [&](int ks, bf16x8_t (&f)[BKV / 16]) {
#pragma unroll
        for (int nt = 0; nt < BKV / 16; ++nt)
          f[nt] = *reinterpret_cast<const bf16x8_t*>(&Ks[nt * 16 + l16][32 * ks + 8 * lg]);
      };
      kfrags(0, kf[0]);
#pragma unroll
      for (int ks = 0; ks < HD / 32; ++ks) {
        if (ks + 1 < HD / 32) kfrags(ks + 1, kf[(ks + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);  // or the reads are sunk to just before their use
#pragma unroll
        for (int nt = 0; nt < BKV / 16; ++nt)
#pragma unroll
          for (int g = 0; g < G; ++g)
            st[g][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[ks & 1][nt], qf[g][ks], st[g][nt], 0, 0, 0);
      }
    }
    FA_MARK(3);
    // ---- online softmax of the lane's rows; only blocks that reach past a row's position mask
    bf16x8_t pb[G][BKV / 32];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const int pos = p.offset + r0 + 16 * g + l16;
      const bool diag = kb * BKV + BKV - 1 > p.offset + r0 + 16 * g;
      float mx = kNone;
#pragma unroll
      for (int nt = 0; nt < BKV / 16; ++nt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if (diag && kb * BKV + nt * 16 + 4 * lg + r > pos) st[g][nt][r] = kNone;
          mx = fmaxf(mx, st[g][nt][r]);
        }
      mx = fmaxf(mx, dm_xor_lane<16>(mx));
      mx = fmaxf(mx, dm_xor_lane<32>(mx));
      // the maximum is kept unscaled (scale > 0): a probability is then one fma and one exp2
      // The reference point of a row's exponentials only moves when the maximum has grown by
      // more than 8 binary orders: until then probabilities up to 2^8 are accumulated (harmless
      // in fp32 sums and bf16 operands, and the final division by the row sum takes it out
      // again), and the running output needs no rescaling, which costs three instructions an
      // accumulator register.
      const bool grow = (mx - m_i[g]) * c2 > 8.f;
      const float m_new = grow ? mx : m_i[g];
      const float alpha = grow ? __builtin_amdgcn_exp2f((m_i[g] - m_new) * c2) : 1.f;
      m_i[g] = m_new;
      const float mc = -(m_new * c2);
      float rs = 0.f;
#pragma unroll
      for (int nt = 0; nt < BKV / 16; ++nt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float pv = __builtin_amdgcn_exp2f(dm_fma(st[g][nt][r], c2, mc));
          st[g][nt][r] = pv;
          rs += pv;
        }
      l_i[g] = l_i[g] * alpha + rs;
      // the running output only needs rescaling when some row's maximum moved
      // (the accumulators live in accumulation registers, which vector arithmetic cannot read:
      // written out by hand so that the moves to a vector register and back stay inside this
      // rarely taken branch; left to the compiler they are made on both paths)
      if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
        for (int t = 0; t < HD / 16; ++t)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float x = o[g][t][r], tmp;
            asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\tv_accvgpr_write_b32 %0, %1"
                         : "+a"(x), "=&v"(tmp)
                         : "v"(alpha));
            o[g][t][r] = x;
          }
      }
#pragma unroll
      for (int k2 = 0; k2 < BKV / 32; ++k2) {
        u32x4_t w;
        w[0] = dm_f2bf2(st[g][2 * k2][0], st[g][2 * k2][1]);
        w[1] = dm_f2bf2(st[g][2 * k2][2], st[g][2 * k2][3]);
        w[2] = dm_f2bf2(st[g][2 * k2 + 1][0], st[g][2 * k2 + 1][1]);
        w[3] = dm_f2bf2(st[g][2 * k2 + 1][2], st[g][2 * k2 + 1][3]);
        pb[g][k2] = __builtin_bit_cast(bf16x8_t, w);
      }
    }
    FA_MARK(4);
    FA_MARK(5);
    // ---- O^T += V^T P^T
    fetch_v(kb_next);
    __builtin_amdgcn_sched_barrier(0);
    {
      // 32 fragments (2 key groups x 16 channel tiles), four at a time, one batch ahead
      bf16x8_t vf[2][4];
      auto vfrags = [&](int b, bf16x8_t (&f)[4]) {
        const int k2 = b >> 2, t0 = 4 * (b & 3);
#pragma unroll
        for (int u = 0; u < 4; ++u) f[u] = *reinterpret_cast<const bf16x8_t*>(&Vt[(t0 + u) * 16 + l16][32 * k2 + 8 * lg]);
      };
      vfrags(0, vf[0]);
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        if (b + 1 < 8) vfrags(b + 1, vf[(b + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
        const int k2 = b >> 2, t0 = 4 * (b & 3);
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int g = 0; g < G; ++g)
            o[g][t0 + u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[b & 1][u], pb[g][k2], o[g][t0 + u], 0, 0, 0);
      }
    }
    FA_MARK(6);
    __syncthreads();
    FA_MARK(7);
  }

  // ---- normalise, gate, store: the lane's rows, channels 16*t + 4*lg .. + 4
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float l = l_i[g] + dm_xor_lane<16>(l_i[g]);
    l = l + dm_xor_lane<32>(l);
    const int row = r0 + 16 * g + l16;
    if (row < p.T) {
      const float inv = 1.0f / l;
      const bf16_t* gate = p.qg + ((size_t)row * p.Hq + h) * 2 * HD + HD + 4 * lg;
      bf16_t* dst = p.out + ((size_t)row * p.Hq + h) * HD + 4 * lg;
#pragma unroll
      for (int t = 0; t < HD / 16; ++t) {
        const u32x2_t gw = *reinterpret_cast<const u32x2_t*>(gate + 16 * t);
        float y[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float att = dm_rb(o[g][t][r] * inv);
          const float gv = (r & 1) ? dm_bf2f_hi(gw[r >> 1]) : dm_bf2f_lo(gw[r >> 1]);
          y[r] = dm_sigmoid_bf16(gv) * att;
        }
        *reinterpret_cast<u32x2_t*>(dst + 16 * t) = u32x2_t{dm_f2bf2(y[0], y[1]), dm_f2bf2(y[2], y[3])};
      }
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
  // 128-row workgroups once there is one for every compute unit
  if ((long)((T + 2 * BQ - 1) / (2 * BQ)) * Hq >= (long)ctx->compute_units)
    hipLaunchKernelGGL(sdpa_prefill_kernel<2>, dim3((T + 2 * BQ - 1) / (2 * BQ), Hq), dim3(256), 0, ctx->stream, p);
  else
    hipLaunchKernelGGL(sdpa_prefill_kernel<1>, dim3((T + BQ - 1) / BQ, Hq), dim3(256), 0, ctx->stream, p);
  ORN_LAUNCH_CHECK("sdpa_prefill_kernel");
  return ORNITH_OK;
}
