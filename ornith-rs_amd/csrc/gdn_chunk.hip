// The gated-delta recurrence of a long prompt chunk on the matrix cores (chunked form).
//
// Replaces, for prefill widths, the token-by-token walk of gated_delta_kernel
// (/root/reference/src/ops/gdn.rs:131-271, kernels/gated_delta.metal:36-142): per value head
//   S <- g_t S;  d_t = beta_t (v_t - S k_t);  S <- S + d_t k_t^T;  y_t = S q_t
// with S [Dv, Dk] in fp32. Like every prefill kernel this one agrees with the exact kernel to
// rounding, not bit for bit.
//
// Over a chunk of C = 64 tokens the walk is linear algebra. With l_i the running sum of
// log g inside the chunk (l_0 = 0), e_ij = exp(l_i - l_j) <= 1 for j <= i, and S_0 the state
// entering the chunk:
//   (I + A) D = diag(beta) V - diag(beta e_i0) K S_0^T,   A_ij = beta_i e_ij (k_i . k_j), j < i
//   Y        = diag(e_i0) Q S_0^T + P D,                    P_ij = e_ij (q_i . k_j),       j <= i
//   S_C      = e_C0 S_0 + (diag(e_Cj) D)^T K
// where D holds the d_t as rows. T = (I + A)^-1 does not depend on the state, so a first
// kernel makes, for every (chunk, head) at once,
//   W = -T diag(beta e_i0) K,   U = T diag(beta) V,   P,   K^T,   l
// and a second one walks the chunks of a head in order: D = U + W S_0^T, Y, S_C - three small
// matrix products a chunk instead of 64 dependent steps. fp32 values that enter a product as
// bf16 operands (T, W, P, S_0, D) go in as a high and a low bf16 part, so the state stays at fp32
// accuracy (the products against raw bf16 inputs q, k, v are exact in their operands).
#include "dmath.h"
#include "rt.h"

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

constexpr int C = 64;        // tokens a chunk
constexpr int DK = 128;      // key width (fixed by the model)
constexpr int LDT = C + 8;   // row stride of token-major LDS tiles (bf16)
constexpr int LDS0 = DK + 8; // row stride of the state tile (bf16)

struct ChunkArgs {
  const bf16_t* q;      // [T, Hk, 128]
  const bf16_t* k;
  const bf16_t* v;      // [T, Hv, Dv]
  const float* g;       // [T, Hv]
  const bf16_t* beta;   // [T, Hv]
  const float* state_in;  // [Hv, Dv, 128]
  float* state_out;
  bf16_t* y;            // [T, Hv, Dv]
  // made by the first kernel, per (chunk, head)
  bf16_t* wh;           // [n, Hv, 64, 128]  high part of W
  bf16_t* wl;           //                  low part
  float* u;             // [n, Hv, 64, Dv]
  bf16_t* pm;           // [n, Hv, 64, 64]  high part of P
  bf16_t* pl;           //                  low part
  float* ell;           // [n, Hv, 64]
  bf16_t* kt;           // [n, Hk, 128, 64]  K transposed
  bf16_t* qf;           // [n, Hk, 64, 128]  Q
  // Everything the first kernel writes is laid out as the second kernel's wavefronts hold it: the
  // 8 values of lane l for (16-row tile, 32-wide k slab) sit at ((tile * slabs + slab) * 64 + l) * 8,
  // so that one load instruction of a wavefront is one contiguous KB (row-major, the same loads
  // touch 16 half-used cache lines each and the L1's line rate bounds the scan).
  int T, Hk, Hv, Dv, nchunks;
};

__device__ __forceinline__ bf16x8_t ld8(const bf16_t* p) { return *reinterpret_cast<const bf16x8_t*>(p); }
__device__ __forceinline__ void split_bf16(float v, bf16_t* hi, bf16_t* lo) {
  const bf16_t h = dm_f2bf(v);
  *hi = h;
  *lo = dm_f2bf(v - dm_bf2f(h));
}
__device__ __forceinline__ f32x4_t mfma(bf16x8_t a, bf16x8_t b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

#ifdef ORN_TIMING
// debug build only: phase time stamps (100 MHz wall clock) of chunk 10 of every workgroup of the
// scan, and of the prep workgroups of head 5
__device__ long long g_chunk_marks[512][8];
__device__ long long g_prep_marks[512][8];
#define CH_MARK(i) do { if (threadIdx.x == 0 && chunk == 10 && blockIdx.x < 512) g_chunk_marks[blockIdx.x][i] = wall_clock64(); } while (0)
#define PR_MARK(i) do { if (threadIdx.x == 0 && blockIdx.x == 5 && blockIdx.y < 512) g_prep_marks[blockIdx.y][i] = wall_clock64(); } while (0)
extern "C" __attribute__((visibility("default"))) int ornith_debug_marks_chunk(long long* out) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_chunk_marks), sizeof(long long) * 512 * 8);
}
extern "C" __attribute__((visibility("default"))) int ornith_debug_marks_prep(long long* out) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_prep_marks), sizeof(long long) * 512 * 8);
}
#else
#define CH_MARK(i)
#define PR_MARK(i)
#endif

// ---- first kernel: everything of a chunk that does not depend on the state --------------
// grid (Hv, nchunks), 256 threads (the heads of a chunk start together: they read neighbouring
// pieces of the same token rows and write neighbouring operand blocks). Operand layout of v_mfma_f32_16x16x32_bf16: lane (l16, lg)
// holds A[m = l16][k = 8 lg ..+8], B^T[n = l16][k = 8 lg ..+8] of a 32-wide k slab and
// D[m = 4 lg + r][n = l16], r < 4.
__global__ __launch_bounds__(256) void gdn_chunk_prep_kernel(ChunkArgs p) {
  // A is kept as four planes, plane j % 4 holding A[i][j] at [i][j / 4] (rows of 16 + 4 pad, the
  // planes 4 words apart in bank): the solve below reads a plane row by row, 16 bytes a read
  constexpr int AROW = 20, APLANE = C * AROW + 4;
  __shared__ float lg_s[C], ell_s[C], bet_s[C];
  __shared__ __attribute__((aligned(16))) bf16_t Kt[DK][LDT];
  __shared__ __attribute__((aligned(16))) bf16_t Vt[DK][LDT];  // Dv <= 128 rows used
  __shared__ __attribute__((aligned(16))) float Ap[4 * APLANE];  // A, later T in two bf16 parts
  bf16_t(*Th)[LDT] = reinterpret_cast<bf16_t(*)[LDT]>(&Ap[0]);
  bf16_t(*Tl)[LDT] = Th + C;
  static_assert(sizeof(float) * 4 * APLANE >= sizeof(bf16_t) * 2 * C * LDT, "T fits where A was");

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, lg = lane >> 4;
  const int chunk = blockIdx.y, hv = blockIdx.x, hk = hv / (p.Hv / p.Hk);
  const int t0 = chunk * C, Dv = p.Dv;
  const size_t ch = (size_t)chunk * p.Hv + hv;

  PR_MARK(0);
  // decay logs and beta of the chunk's tokens; tokens past the end leave the state alone
  if (tid < C) {
    const int t = t0 + tid;
    const bool live = t < p.T;
    const float gv = live ? p.g[(size_t)t * p.Hv + hv] : 1.f;
    lg_s[tid] = live ? fmaxf(__logf(gv), -100.f) : 0.f;
    bet_s[tid] = live ? dm_bf2f(p.beta[(size_t)t * p.Hv + hv]) : 0.f;
  }
  // Operand fragments of the K K^T / Q K^T products below, asked for now (they depend on
  // nothing made here): tokens i = 16 wave + l16 as the n side, tokens j of the tiles nt < wave as
  // the m side (tile nt = wave has the same rows as the n side).
  bf16x8_t bki[4], bqi[4], akj[3][4];
  {
    const int ti = min(t0 + 16 * wave + l16, p.T - 1);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      bki[ks] = ld8(p.k + ((size_t)ti * p.Hk + hk) * DK + 32 * ks + 8 * lg);
      bqi[ks] = ld8(p.q + ((size_t)ti * p.Hk + hk) * DK + 32 * ks + 8 * lg);
    }
#pragma unroll
    for (int nt = 0; nt < 3; ++nt) {
      if (nt < wave) {
        const int tj = min(t0 + 16 * nt + l16, p.T - 1);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) akj[nt][ks] = ld8(p.k + ((size_t)tj * p.Hk + hk) * DK + 32 * ks + 8 * lg);
      }
    }
  }
  // K and V of the chunk, transposed into LDS: thread = (token pair, 8-wide piece); the two
  // tokens' values of a channel are one 4-byte write, and a wavefront's 64 writes of a channel
  // (32 pairs of two pieces) fall on 64 different banks. All loads first, then the writes.
  {
    uint4 kr[2][2], vr[2][2];
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int idx = tid + 256 * it, tp = idx & 31, pc = idx >> 5;
      const int ta = min(t0 + 2 * tp, p.T - 1), tb = min(t0 + 2 * tp + 1, p.T - 1);
      kr[it][0] = *reinterpret_cast<const uint4*>(p.k + ((size_t)ta * p.Hk + hk) * DK + 8 * pc);
      kr[it][1] = *reinterpret_cast<const uint4*>(p.k + ((size_t)tb * p.Hk + hk) * DK + 8 * pc);
      if (8 * pc < Dv) {
        vr[it][0] = *reinterpret_cast<const uint4*>(p.v + ((size_t)ta * p.Hv + hv) * Dv + 8 * pc);
        vr[it][1] = *reinterpret_cast<const uint4*>(p.v + ((size_t)tb * p.Hv + hv) * Dv + 8 * pc);
      }
    }
    auto put = [&](bf16_t(*dst)[LDT], const uint4& a, const uint4& b, int pc, int tp) {
      const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, bw[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t w = (e & 1) ? ((aw[e >> 1] >> 16) | (bw[e >> 1] & 0xffff0000u))
                                   : ((aw[e >> 1] & 0xffffu) | (bw[e >> 1] << 16));
        *reinterpret_cast<uint32_t*>(&dst[8 * pc + e][2 * tp]) = w;
      }
    };
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int idx = tid + 256 * it, tp = idx & 31, pc = idx >> 5;
      put(Kt, kr[it][0], kr[it][1], pc, tp);
      if (8 * pc < Dv) put(Vt, vr[it][0], vr[it][1], pc, tp);
    }
  }
  __syncthreads();
  PR_MARK(1);
  if (tid < C) {
    float s = 0.f;
    for (int j = 0; j <= tid; ++j) s += lg_s[j];
    ell_s[tid] = s;
    p.ell[ch * C + tid] = s;
  }
  // K^T and Q for the second kernel, once per key head
  if (hv % (p.Hv / p.Hk) == 0) {
    bf16_t* dst = p.kt + ((size_t)chunk * p.Hk + hk) * DK * C;
    for (int idx = tid; idx < DK * (C / 8); idx += 256) {
      const int r = idx / (C / 8), pc = idx % (C / 8);  // row dk = r, tokens 8 pc ..
      *reinterpret_cast<bf16x8_t*>(dst + ((size_t)((r >> 4) * 2 + (pc >> 2)) * 64 + (pc & 3) * 16 + (r & 15)) * 8) =
          ld8(&Kt[r][8 * pc]);
    }
    bf16_t* qdst = p.qf + ((size_t)chunk * p.Hk + hk) * C * DK;
    for (int idx = tid; idx < C * (DK / 8); idx += 256) {
      const int tok = idx / (DK / 8), pc = idx % (DK / 8);  // row token, channels 8 pc ..
      const int t = min(t0 + tok, p.T - 1);
      *reinterpret_cast<bf16x8_t*>(qdst + ((size_t)((tok >> 4) * 4 + (pc >> 2)) * 64 + (pc & 3) * 16 + (tok & 15)) * 8) =
          ld8(p.q + ((size_t)t * p.Hk + hk) * DK + 8 * pc);
    }
  }
  __syncthreads();
  PR_MARK(2);

  // ---- K K^T and Q K^T for the chunk's tokens i = 16 wave + l16 (the n side of the product, so
  // that a lane ends up with four consecutive j of one i: packed stores); lower triangle only
  {
    const int i = 16 * wave + l16;
    const float ell_i = ell_s[i], bet_i = bet_s[i];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      f32x4_t kk = {0.f, 0.f, 0.f, 0.f}, qk = {0.f, 0.f, 0.f, 0.f};
      if (nt <= wave) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          const bf16x8_t a = nt < wave ? akj[nt < 3 ? nt : 0][ks] : bki[ks];
          kk = mfma(a, bki[ks], kk);  // [j][i]
          qk = mfma(a, bqi[ks], qk);
        }
      }
      bf16_t ph[4], pl[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int j = 16 * nt + 4 * lg + r;
        const float e = j <= i ? __expf(ell_i - ell_s[j]) : 0.f;
        Ap[r * APLANE + i * AROW + 4 * nt + lg] = j < i ? bet_i * e * kk[r] : 0.f;
        split_bf16(e * qk[r], &ph[r], &pl[r]);
      }
      // element (i, j = 16 nt + 4 lg + r): tile i / 16, slab j / 32, lane (j % 32 / 8) * 16 + i % 16
      const size_t po = ch * C * C + ((size_t)(wave * 2 + (nt >> 1)) * 64 + (2 * (nt & 1) + (lg >> 1)) * 16 + l16) * 8 + 4 * (lg & 1);
      *reinterpret_cast<uint2*>(p.pm + po) = make_uint2(ph[0] | ((uint32_t)ph[1] << 16), ph[2] | ((uint32_t)ph[3] << 16));
      *reinterpret_cast<uint2*>(p.pl + po) = make_uint2(pl[0] | ((uint32_t)pl[1] << 16), pl[2] | ((uint32_t)pl[3] << 16));
    }
  }
  __syncthreads();
  PR_MARK(3);

  // ---- T = (I + A)^-1 by forward substitution. Thread (column c = tid / 4, part q4 = tid % 4)
  // keeps T[j][c] for j = q4 mod 4; a row's sum over j is four partial sums met inside the quad.
  const int col = tid >> 2, q4 = tid & 3;
  float tq[C / 4];
#pragma unroll
  for (int m = 0; m < C / 4; ++m) tq[m] = 0.f;
  {
    const float* arow = &Ap[q4 * APLANE];
#pragma unroll
    for (int i = 0; i < C; ++i) {
      float acc = 0.f;
#pragma unroll
      for (int m4 = 0; m4 < (i + 3) / 4; m4 += 4) {
        const float4 a4 = *reinterpret_cast<const float4*>(arow + i * AROW + m4);
        acc = dm_fma(a4.x, tq[m4], acc);
        if (m4 + 1 < (i + 3) / 4) acc = dm_fma(a4.y, tq[m4 + 1], acc);
        if (m4 + 2 < (i + 3) / 4) acc = dm_fma(a4.z, tq[m4 + 2], acc);
        if (m4 + 3 < (i + 3) / 4) acc = dm_fma(a4.w, tq[m4 + 3], acc);
      }
      acc = acc + dm_xor_lane<1>(acc);
      acc = acc + dm_xor_lane<2>(acc);
      const float ti = (i == col ? 1.f : 0.f) - acc;
      tq[i >> 2] = q4 == (i & 3) ? ti : tq[i >> 2];
    }
  }
  __syncthreads();  // A has been read; its memory becomes T
  PR_MARK(4);

  // two passes over T with its columns scaled: by beta e_j0 against K (W), by beta against V (U).
  // The products are made transposed (K^T or V^T as the m side), so a lane holds four consecutive
  // columns of one token's row and stores them in one piece.
  for (int pass = 0; pass < 2; ++pass) {
    {
      const float sc = pass == 0 ? bet_s[col] * __expf(ell_s[col]) : bet_s[col];
#pragma unroll
      for (int m = 0; m < C / 4; ++m) split_bf16(tq[m] * sc, &Th[4 * m + q4][col], &Tl[4 * m + q4][col]);
    }
    __syncthreads();
    const int i = 16 * wave + l16;
    bf16x8_t bh[2], bl[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      bh[ks] = ld8(&Th[i][32 * ks + 8 * lg]);
      bl[ks] = ld8(&Tl[i][32 * ks + 8 * lg]);
    }
    const int ntiles = pass == 0 ? DK / 16 : Dv / 16;
    for (int nt = 0; nt < ntiles; ++nt) {
      f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        if (pass == 0) {
          const bf16x8_t a = ld8(&Kt[16 * nt + l16][32 * ks + 8 * lg]);
          acc = mfma(a, bh[ks], acc);  // [dk 16 nt + 4 lg + r][token i]
          acc = mfma(a, bl[ks], acc);
        } else {
          const bf16x8_t b = ld8(&Vt[16 * nt + l16][32 * ks + 8 * lg]);
          acc = mfma(bh[ks], b, acc);  // [token 16 wave + 4 lg + r][dv 16 nt + l16]
          acc = mfma(bl[ks], b, acc);
        }
      }
      if (pass == 0) {
        bf16_t hi[4], lo[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) split_bf16(-acc[r], &hi[r], &lo[r]);
        // element (i, dk = 16 nt + 4 lg + r): tile i / 16, slab dk / 32, lane (dk % 32 / 8) * 16 + i % 16
        const size_t wo = ch * C * DK + ((size_t)(wave * 4 + (nt >> 1)) * 64 + (2 * (nt & 1) + (lg >> 1)) * 16 + l16) * 8 + 4 * (lg & 1);
        *reinterpret_cast<uint2*>(p.wh + wo) = make_uint2(hi[0] | ((uint32_t)hi[1] << 16), hi[2] | ((uint32_t)hi[3] << 16));
        *reinterpret_cast<uint2*>(p.wl + wo) = make_uint2(lo[0] | ((uint32_t)lo[1] << 16), lo[2] | ((uint32_t)lo[3] << 16));
      } else {
        // U is wanted as an accumulator tile [token][dv]: this product is made the other way round
        // (T the m side), and a lane's four values are four tokens of one dv, one 16-byte store
        *reinterpret_cast<float4*>(p.u + ch * C * Dv + ((size_t)(wave * (Dv / 16) + nt) * 64 + lane) * 4) =
            make_float4(acc[0], acc[1], acc[2], acc[3]);
      }
    }
    __syncthreads();  // T's first scaling has been read before the second is written
    PR_MARK(5 + pass);
  }
}


// four fp32 values as their high and low bf16 parts, each quad one 8-byte LDS write
__device__ __forceinline__ void split4_bf16(const f32x4_t& v, bf16_t* hi, bf16_t* lo) {
  const uint32_t h01 = dm_f2bf2(v[0], v[1]), h23 = dm_f2bf2(v[2], v[3]);  // two conversions an instruction
  const uint32_t l01 = dm_f2bf2(v[0] - dm_bf2f_lo(h01), v[1] - dm_bf2f_hi(h01));
  const uint32_t l23 = dm_f2bf2(v[2] - dm_bf2f_lo(h23), v[3] - dm_bf2f_hi(h23));
  *reinterpret_cast<uint2*>(hi) = make_uint2(h01, h23);
  *reinterpret_cast<uint2*>(lo) = make_uint2(l01, l23);
}

// ---- second kernel: the chunks of a head in order ------------------------------------------
// 512 threads: a workgroup owns 16 rows of a head's state. Only D and the state are links of the
// chain from chunk to chunk; Y is not. So the eight wavefronts have two roles, and a SIMD runs
// one of each:
//   chain  (wavefronts 0..3)  D = U + W S_0^T for the tokens 16 w .., then the state columns 32 w ..
//   output (wavefronts 4..7)  Y = diag(e_i0) Q S_0^T + P D for the tokens 16 w .., stored as y
// Both read the state as two bf16 parts (S0h, S0l) and D (Dh, Dl) from LDS; two barriers a chunk.
// The Dv / 16 workgroups of a head read the same W, P, Q, K^T, so they are placed on one XCD
// (workgroup ids go round the 8 XCDs, each with its own L2): workgroup L sits on XCD L % 8 and
// takes head (L % 8) * heads_per_xcd + ...
__global__ __launch_bounds__(512) void gdn_chunk_scan_kernel(ChunkArgs p) {
  __shared__ __attribute__((aligned(16))) bf16_t S0h[16][LDS0], S0l[16][LDS0];
  __shared__ __attribute__((aligned(16))) bf16_t Dh[16][LDT], Dl[16][LDT], Fh[16][LDT], Fl[16][LDT];

  const int tid = threadIdx.x, lane = tid & 63, wave = (tid >> 6) & 3;
  const bool chain = tid < 256;
  const int l16 = lane & 15, lg = lane >> 4;
  const int Dv = p.Dv, nb = Dv / 16;
  const int xcd = blockIdx.x % 8, slot = blockIdx.x / 8, hpx = (p.Hv + 7) / 8;
  const int hv = xcd * hpx + slot / nb, dvb = slot % nb;
  if (slot / nb >= hpx || hv >= p.Hv) return;  // uniform over the workgroup
  const int hk = hv / (p.Hv / p.Hk), dv0 = dvb * 16;

  // A chunk's operands come straight from memory into registers, one chunk ahead of their use:
  // the chunks of a head are a dependent chain, and a trip to memory inside a link would be
  // most of its length.
  if (chain) {
    // The state products are made transposed (K^T the m side), so that a lane holds four
    // consecutive key channels of one state row: s[n2][r] = S[dv0 + l16][16 (2 w + n2) + 4 lg + r],
    // 16 bytes in memory and 8 bytes of each bf16 part in LDS.
    f32x4_t s[2];
#pragma unroll
    for (int n2 = 0; n2 < 2; ++n2)
      s[n2] = *reinterpret_cast<const f32x4_t*>(p.state_in + ((size_t)hv * Dv + dv0 + l16) * DK + 16 * (2 * wave + n2) + 4 * lg);
    struct Ops {
      bf16x8_t awh[4], awl[4], bk[2][2];
      f32x4_t u, ellr;
      float ell_c;
    };
    // in two halves, issued at different points of a chunk so that the memory pipe's work runs
    // beside the matrix products instead of ahead of them
    auto fetch_a = [&](int chunk, Ops& o) {
      const size_t ch = (size_t)chunk * p.Hv + hv;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        o.awh[ks] = ld8(p.wh + ch * C * DK + ((size_t)(wave * 4 + ks) * 64 + lane) * 8);
        o.awl[ks] = ld8(p.wl + ch * C * DK + ((size_t)(wave * 4 + ks) * 64 + lane) * 8);
      }
      o.u = *reinterpret_cast<const f32x4_t*>(p.u + ch * C * Dv + ((size_t)(wave * nb + dvb) * 64 + lane) * 4);
    };
    auto fetch_b = [&](int chunk, Ops& o) {
      const size_t ch = (size_t)chunk * p.Hv + hv, ck = (size_t)chunk * p.Hk + hk;
#pragma unroll
      for (int k2 = 0; k2 < 2; ++k2)
#pragma unroll
        for (int n2 = 0; n2 < 2; ++n2)
          o.bk[n2][k2] = ld8(p.kt + ck * DK * C + ((size_t)((2 * wave + n2) * 2 + k2) * 64 + lane) * 8);
      o.ell_c = p.ell[ch * C + C - 1];
#pragma unroll
      for (int r = 0; r < 4; ++r) o.ellr[r] = p.ell[ch * C + 16 * wave + 4 * lg + r];
    };
    // three operand sets in turn, asked for two chunks ahead of their use (one chunk of a chain
    // this short is less than a trip to memory); the sets are named, not indexed or copied
    auto link = [&](int chunk, const Ops& cur, Ops& fill) {
      const bool more = chunk + 2 < p.nchunks;
      CH_MARK(0);
      const bf16x8_t(&awh)[4] = cur.awh, (&awl)[4] = cur.awl;
      const bf16x8_t(&bk)[2][2] = cur.bk;
      f32x4_t d = cur.u;
      const f32x4_t ellr = cur.ellr;
      const float ell_c = cur.ell_c;

      // 1. the state as two bf16 parts
#pragma unroll
      for (int n2 = 0; n2 < 2; ++n2)
        split4_bf16(s[n2], &S0h[l16][16 * (2 * wave + n2) + 4 * lg], &S0l[l16][16 * (2 * wave + n2) + 4 * lg]);
      __syncthreads();
      CH_MARK(1);

      // 2. D = U + W S_0^T; three accumulators, so that no product waits for the one before it
      if (more) fetch_a(chunk + 2, fill);
      f32x4_t d1 = {0.f, 0.f, 0.f, 0.f}, d2 = d1;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const bf16x8_t bh = ld8(&S0h[l16][32 * ks + 8 * lg]), bl = ld8(&S0l[l16][32 * ks + 8 * lg]);
        d = mfma(awh[ks], bh, d);
        d1 = mfma(awh[ks], bl, d1);
        d2 = mfma(awl[ks], bh, d2);
      }
      d = d + (d1 + d2);
      f32x4_t f;
#pragma unroll
      for (int r = 0; r < 4; ++r) f[r] = d[r] * __expf(ell_c - ellr[r]);
      split4_bf16(d, &Dh[l16][16 * wave + 4 * lg], &Dl[l16][16 * wave + 4 * lg]);
      split4_bf16(f, &Fh[l16][16 * wave + 4 * lg], &Fl[l16][16 * wave + 4 * lg]);
      CH_MARK(2);
      __syncthreads();
      CH_MARK(3);

      // 3. S = e_C0 S + (diag(e_Cj) D)^T K
      if (more) fetch_b(chunk + 2, fill);
      CH_MARK(4);
      const float gc = __expf(ell_c);
#pragma unroll
      for (int n2 = 0; n2 < 2; ++n2) {
#pragma unroll
        for (int r = 0; r < 4; ++r) s[n2][r] *= gc;
#pragma unroll
        for (int k2 = 0; k2 < 2; ++k2) {
          s[n2] = mfma(bk[n2][k2], ld8(&Fh[l16][32 * k2 + 8 * lg]), s[n2]);  // [dk][dv]
          s[n2] = mfma(bk[n2][k2], ld8(&Fl[l16][32 * k2 + 8 * lg]), s[n2]);
        }
      }
      CH_MARK(5);
      // the tiles read here are rewritten behind the next chunk's first barrier, the state tiles
      // behind the barrier above
      CH_MARK(6);
    };
    Ops o0, o1, o2;
    fetch_a(0, o0);
    fetch_b(0, o0);
    if (p.nchunks > 1) {
      fetch_a(1, o1);
      fetch_b(1, o1);
    }
    for (int chunk = 0; chunk < p.nchunks; chunk += 3) {
      link(chunk, o0, o2);
      if (chunk + 1 < p.nchunks) link(chunk + 1, o1, o0);
      if (chunk + 2 < p.nchunks) link(chunk + 2, o2, o1);
    }
#pragma unroll
    for (int n2 = 0; n2 < 2; ++n2)
      *reinterpret_cast<f32x4_t*>(p.state_out + ((size_t)hv * Dv + dv0 + l16) * DK + 16 * (2 * wave + n2) + 4 * lg) = s[n2];
  } else {
    struct Ops {
      bf16x8_t aq[4], ap[2], apl[2];
      f32x4_t ellr;
    };
    auto fetch = [&](int chunk, Ops& o) {
      const size_t ch = (size_t)chunk * p.Hv + hv, ck = (size_t)chunk * p.Hk + hk;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) o.aq[ks] = ld8(p.qf + ck * C * DK + ((size_t)(wave * 4 + ks) * 64 + lane) * 8);
#pragma unroll
      for (int k2 = 0; k2 < 2; ++k2) {
        o.ap[k2] = ld8(p.pm + ch * C * C + ((size_t)(wave * 2 + k2) * 64 + lane) * 8);
        o.apl[k2] = ld8(p.pl + ch * C * C + ((size_t)(wave * 2 + k2) * 64 + lane) * 8);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) o.ellr[r] = p.ell[ch * C + 16 * wave + 4 * lg + r];
    };
    auto link = [&](int chunk, const Ops& cur, Ops& fill) {
      const int t0 = chunk * C;
      __syncthreads();  // the state's two parts are in LDS
      if (chunk + 2 < p.nchunks) fetch(chunk + 2, fill);
      // the start of Y = diag(e_i0) Q S_0^T, two accumulators
      f32x4_t yv = {0.f, 0.f, 0.f, 0.f}, y1 = yv;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const bf16x8_t bh = ld8(&S0h[l16][32 * ks + 8 * lg]), bl = ld8(&S0l[l16][32 * ks + 8 * lg]);
        yv = mfma(cur.aq[ks], bh, yv);
        y1 = mfma(cur.aq[ks], bl, y1);
      }
      yv = yv + y1;
#pragma unroll
      for (int r = 0; r < 4; ++r) yv[r] *= __expf(cur.ellr[r]);
      __syncthreads();  // D is in LDS (and the state's parts have been read)
      // Y += P D
#pragma unroll
      for (int k2 = 0; k2 < 2; ++k2) {
        const bf16x8_t dh = ld8(&Dh[l16][32 * k2 + 8 * lg]);
        yv = mfma(cur.ap[k2], dh, yv);
        yv = mfma(cur.ap[k2], ld8(&Dl[l16][32 * k2 + 8 * lg]), yv);
        yv = mfma(cur.apl[k2], dh, yv);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int tk = t0 + 16 * wave + 4 * lg + r;
        if (tk < p.T) p.y[((size_t)tk * p.Hv + hv) * Dv + dv0 + l16] = dm_f2bf(yv[r]);
      }
    };
    Ops o0, o1, o2;
    fetch(0, o0);
    if (p.nchunks > 1) fetch(1, o1);
    for (int chunk = 0; chunk < p.nchunks; chunk += 3) {
      link(chunk, o0, o2);
      if (chunk + 1 < p.nchunks) link(chunk + 1, o1, o0);
      if (chunk + 2 < p.nchunks) link(chunk + 2, o2, o1);
    }
  }
}

}  // namespace

// Returns -1 when the shapes are outside the chunked form (the caller keeps its other kernel).
int gdn_chunked_recurrence(ornith_ctx* ctx, const void* d_q, const void* d_k, const void* d_v, const float* d_g,
                           const void* d_beta, const float* d_state_in, int T, int Hk, int Hv, int Dk, int Dv,
                           void* d_y, float* d_state_out) {
  if (Dk != DK || Dv % 16 != 0 || Dv > 128 || Hv % Hk != 0) return -1;
  // Long calls go block by block (the state handed on in d_state_out): what the prep kernel
  // writes for a block and the scan reads back should still be in the last-level cache, which
  // about 64 chunks of 32 heads fill (116 KB a chunk and head); past that the scan, which asks
  // for its operands one chunk ahead, waits for HBM every chunk (2.4 us a chunk against 1.7).
  const int block_rows = max(1, ornith_option_gdn_block_chunks()) * C;
  const int nmax = (min(T, block_rows) + C - 1) / C;
  const size_t per = (size_t)nmax * Hv;
  void* base = nullptr;
  const size_t need = per * ((size_t)C * DK * 2 * 2 + (size_t)C * Dv * 4 + (size_t)C * C * 2 * 2 + C * 4) +
                      (size_t)nmax * Hk * DK * C * 2 * 2 + 10 * 256;
  int rc = ornith_scratch(ctx, need, &base);
  if (rc) return rc;
  ScratchCursor sc(base);
  ChunkArgs a{};
  a.wh = sc.take<bf16_t>(per * C * DK);
  a.wl = sc.take<bf16_t>(per * C * DK);
  a.u = sc.take<float>(per * C * Dv);
  a.pm = sc.take<bf16_t>(per * C * C);
  a.pl = sc.take<bf16_t>(per * C * C);
  a.ell = sc.take<float>(per * C);
  a.kt = sc.take<bf16_t>((size_t)nmax * Hk * DK * C);
  a.qf = sc.take<bf16_t>((size_t)nmax * Hk * C * DK);
  a.Hk = Hk;
  a.Hv = Hv;
  a.Dv = Dv;
  a.state_out = d_state_out;
  for (int t0 = 0; t0 < T; t0 += block_rows) {
    const int rows = min(block_rows, T - t0), n = (rows + C - 1) / C;
    a.q = (const bf16_t*)d_q + (size_t)t0 * Hk * DK;
    a.k = (const bf16_t*)d_k + (size_t)t0 * Hk * DK;
    a.v = (const bf16_t*)d_v + (size_t)t0 * Hv * Dv;
    a.g = d_g + (size_t)t0 * Hv;
    a.beta = (const bf16_t*)d_beta + (size_t)t0 * Hv;
    a.y = (bf16_t*)d_y + (size_t)t0 * Hv * Dv;
    a.state_in = t0 == 0 ? d_state_in : d_state_out;
    a.T = rows;
    a.nchunks = n;
    hipLaunchKernelGGL(gdn_chunk_prep_kernel, dim3(Hv, n), dim3(256), 0, ctx->stream, a);
    ORN_LAUNCH_CHECK("gdn_chunk_prep_kernel");
    hipLaunchKernelGGL(gdn_chunk_scan_kernel, dim3(8 * ((Hv + 7) / 8) * (Dv / 16)), dim3(512), 0, ctx->stream, a);
    ORN_LAUNCH_CHECK("gdn_chunk_scan_kernel");
  }
  return ORNITH_OK;
}
