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

// ---- first kernel: everything of a chunk that does not depend on the state --------------
// grid (nchunks, Hv), 256 threads. Operand layout of v_mfma_f32_16x16x32_bf16: lane (l16, lg)
// holds A[m = l16][k = 8 lg ..+8], B^T[n = l16][k = 8 lg ..+8] of a 32-wide k slab and
// D[m = 4 lg + r][n = l16], r < 4.
__global__ __launch_bounds__(256) void gdn_chunk_prep_kernel(ChunkArgs p) {
  __shared__ float lg_s[C], ell_s[C], bet_s[C];
  __shared__ __attribute__((aligned(16))) bf16_t Kt[DK][LDT];
  __shared__ __attribute__((aligned(16))) bf16_t Vt[DK][LDT];  // Dv <= 128 rows used
  __shared__ __attribute__((aligned(16))) float Am[C][C + 8];  // A, later T in two bf16 parts
  bf16_t(*Th)[LDT] = reinterpret_cast<bf16_t(*)[LDT]>(&Am[0][0]);
  bf16_t(*Tl)[LDT] = Th + C;
  static_assert(sizeof(float) * C * (C + 8) >= sizeof(bf16_t) * 2 * C * LDT, "T fits where A was");

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, lg = lane >> 4;
  const int chunk = blockIdx.x, hv = blockIdx.y, hk = hv / (p.Hv / p.Hk);
  const int t0 = chunk * C, Dv = p.Dv;
  const size_t ch = (size_t)chunk * p.Hv + hv;

  // decay logs and beta of the chunk's tokens; tokens past the end leave the state alone
  if (tid < C) {
    const int t = t0 + tid;
    const bool live = t < p.T;
    const float gv = live ? p.g[(size_t)t * p.Hv + hv] : 1.f;
    lg_s[tid] = live ? fmaxf(__logf(gv), -100.f) : 0.f;
    bet_s[tid] = live ? dm_bf2f(p.beta[(size_t)t * p.Hv + hv]) : 0.f;
  }
  // K and V of the chunk, transposed into LDS: thread = (token tid / 4 + 64 pass.., 8-wide piece)
  for (int idx = tid; idx < C * (DK / 8); idx += 256) {
    const int tok = idx / (DK / 8), pc = idx % (DK / 8);
    const int t = min(t0 + tok, p.T - 1);
    const uint4 kv8 = *reinterpret_cast<const uint4*>(p.k + ((size_t)t * p.Hk + hk) * DK + 8 * pc);
    const uint32_t kw[4] = {kv8.x, kv8.y, kv8.z, kv8.w};
#pragma unroll
    for (int e = 0; e < 8; ++e) Kt[8 * pc + e][tok] = (bf16_t)(kw[e >> 1] >> (16 * (e & 1)));
  }
  for (int idx = tid; idx < C * (Dv / 8); idx += 256) {
    const int tok = idx / (Dv / 8), pc = idx % (Dv / 8);
    const int t = min(t0 + tok, p.T - 1);
    const uint4 vv8 = *reinterpret_cast<const uint4*>(p.v + ((size_t)t * p.Hv + hv) * Dv + 8 * pc);
    const uint32_t vw[4] = {vv8.x, vv8.y, vv8.z, vv8.w};
#pragma unroll
    for (int e = 0; e < 8; ++e) Vt[8 * pc + e][tok] = (bf16_t)(vw[e >> 1] >> (16 * (e & 1)));
  }
  __syncthreads();
  if (tid < C) {
    float s = 0.f;
    for (int j = 0; j <= tid; ++j) s += lg_s[j];
    ell_s[tid] = s;
    p.ell[ch * C + tid] = s;
  }
  // K^T for the second kernel, once per key head
  if (hv % (p.Hv / p.Hk) == 0) {
    bf16_t* dst = p.kt + ((size_t)chunk * p.Hk + hk) * DK * C;
    for (int idx = tid; idx < DK * (C / 8); idx += 256) {
      const int r = idx / (C / 8), pc = idx % (C / 8);
      *reinterpret_cast<bf16x8_t*>(dst + (size_t)r * C + 8 * pc) = ld8(&Kt[r][8 * pc]);
    }
  }
  __syncthreads();

  // ---- K K^T and Q K^T, rows 16 wave .. of the chunk; only the lower triangle is needed
  {
    const int ti = min(t0 + 16 * wave + l16, p.T - 1);
    bf16x8_t ak[4], aq[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      ak[ks] = ld8(p.k + ((size_t)ti * p.Hk + hk) * DK + 32 * ks + 8 * lg);
      aq[ks] = ld8(p.q + ((size_t)ti * p.Hk + hk) * DK + 32 * ks + 8 * lg);
    }
    bf16_t* pdst = p.pm + ch * C * C;
    bf16_t* pdst_lo = p.pl + ch * C * C;
    for (int nt = 0; nt < 4; ++nt) {
      f32x4_t kk = {0.f, 0.f, 0.f, 0.f}, qk = {0.f, 0.f, 0.f, 0.f};
      if (nt <= wave) {
        const int tj = min(t0 + 16 * nt + l16, p.T - 1);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          const bf16x8_t bk = ld8(p.k + ((size_t)tj * p.Hk + hk) * DK + 32 * ks + 8 * lg);
          kk = mfma(ak[ks], bk, kk);
          qk = mfma(aq[ks], bk, qk);
        }
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = 16 * wave + 4 * lg + r, j = 16 * nt + l16;
        const float e = j <= i ? __expf(ell_s[i] - ell_s[j]) : 0.f;
        Am[i][j] = j < i ? bet_s[i] * e * kk[r] : 0.f;
        split_bf16(e * qk[r], &pdst[(size_t)i * C + j], &pdst_lo[(size_t)i * C + j]);
      }
    }
  }
  __syncthreads();

  // ---- T = (I + A)^-1 by forward substitution, one column a lane (first wavefront)
  float t[C];
  if (wave == 0) {
#pragma unroll
    for (int i = 0; i < C; ++i) {
      float acc = i == lane ? 1.f : 0.f;
#pragma unroll
      for (int j = 0; j < i; ++j) acc = dm_fma(-Am[i][j], t[j], acc);
      t[i] = acc;
    }
  }
  __syncthreads();  // A has been read; its memory becomes T

  // two passes over T with its columns scaled: by beta e_j0 against K (W), by beta against V (U)
  for (int pass = 0; pass < 2; ++pass) {
    if (wave == 0) {
      const float sc = pass == 0 ? bet_s[lane] * __expf(ell_s[lane]) : bet_s[lane];
#pragma unroll
      for (int i = 0; i < C; ++i) split_bf16(t[i] * sc, &Th[i][lane], &Tl[i][lane]);
    }
    __syncthreads();
    bf16x8_t ah[2], al[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      ah[ks] = ld8(&Th[16 * wave + l16][32 * ks + 8 * lg]);
      al[ks] = ld8(&Tl[16 * wave + l16][32 * ks + 8 * lg]);
    }
    const int ntiles = pass == 0 ? DK / 16 : Dv / 16;
    for (int nt = 0; nt < ntiles; ++nt) {
      f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const bf16x8_t b = pass == 0 ? ld8(&Kt[16 * nt + l16][32 * ks + 8 * lg]) : ld8(&Vt[16 * nt + l16][32 * ks + 8 * lg]);
        acc = mfma(ah[ks], b, acc);
        acc = mfma(al[ks], b, acc);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = 16 * wave + 4 * lg + r, n = 16 * nt + l16;
        if (pass == 0) {
          bf16_t hi, lo;
          split_bf16(-acc[r], &hi, &lo);
          p.wh[(ch * C + i) * DK + n] = hi;
          p.wl[(ch * C + i) * DK + n] = lo;
        } else {
          p.u[(ch * C + i) * Dv + n] = acc[r];
        }
      }
    }
    __syncthreads();  // T's first scaling has been read before the second is written
  }
}

// ---- second kernel: the chunks of a head in order ------------------------------------------
// grid (Dv / 16, Hv), 256 threads: a workgroup owns 16 rows of a head's state. Wavefront w owns
// the chunk's tokens 16 w .. for D and Y, and the state columns 32 w .. for S.
__global__ __launch_bounds__(256) void gdn_chunk_scan_kernel(ChunkArgs p) {
  __shared__ __attribute__((aligned(16))) bf16_t S0h[16][LDS0], S0l[16][LDS0];
  __shared__ __attribute__((aligned(16))) bf16_t Dh[16][LDT], Dl[16][LDT], Fh[16][LDT], Fl[16][LDT];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, lg = lane >> 4;
  const int dvb = blockIdx.x, hv = blockIdx.y, hk = hv / (p.Hv / p.Hk);
  const int Dv = p.Dv, dv0 = dvb * 16;

  f32x4_t s[2];
#pragma unroll
  for (int n2 = 0; n2 < 2; ++n2)
#pragma unroll
    for (int r = 0; r < 4; ++r)
      s[n2][r] = p.state_in[((size_t)hv * Dv + dv0 + 4 * lg + r) * DK + 16 * (2 * wave + n2) + l16];

  for (int chunk = 0; chunk < p.nchunks; ++chunk) {
    const int t0 = chunk * C;
    const size_t ch = (size_t)chunk * p.Hv + hv;
    const int row = 16 * wave + l16;  // this lane's token as an A-operand row
    // operands that come straight from memory, asked for before anything waits
    bf16x8_t awh[4], awl[4], aq[4], ap[2], apl[2], bk[2][2];
    const int tq = min(t0 + row, p.T - 1);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      awh[ks] = ld8(p.wh + (ch * C + row) * DK + 32 * ks + 8 * lg);
      awl[ks] = ld8(p.wl + (ch * C + row) * DK + 32 * ks + 8 * lg);
      aq[ks] = ld8(p.q + ((size_t)tq * p.Hk + hk) * DK + 32 * ks + 8 * lg);
    }
#pragma unroll
    for (int k2 = 0; k2 < 2; ++k2) {
      ap[k2] = ld8(p.pm + (ch * C + row) * C + 32 * k2 + 8 * lg);
      apl[k2] = ld8(p.pl + (ch * C + row) * C + 32 * k2 + 8 * lg);
#pragma unroll
      for (int n2 = 0; n2 < 2; ++n2)
        bk[n2][k2] = ld8(p.kt + (((size_t)chunk * p.Hk + hk) * DK + 16 * (2 * wave + n2) + l16) * C + 32 * k2 + 8 * lg);
    }
    f32x4_t d, ellr;
    const float ell_c = p.ell[ch * C + C - 1];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i = 16 * wave + 4 * lg + r;
      d[r] = p.u[(ch * C + i) * Dv + dv0 + l16];
      ellr[r] = p.ell[ch * C + i];
    }

    // 1. the state as two bf16 parts
#pragma unroll
    for (int n2 = 0; n2 < 2; ++n2)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        split_bf16(s[n2][r], &S0h[4 * lg + r][16 * (2 * wave + n2) + l16], &S0l[4 * lg + r][16 * (2 * wave + n2) + l16]);
    __syncthreads();

    // 2. D = U + W S_0^T and the start of Y = diag(e_i0) Q S_0^T
    f32x4_t yv = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const bf16x8_t bh = ld8(&S0h[l16][32 * ks + 8 * lg]), bl = ld8(&S0l[l16][32 * ks + 8 * lg]);
      d = mfma(awh[ks], bh, d);
      d = mfma(awh[ks], bl, d);
      d = mfma(awl[ks], bh, d);
      yv = mfma(aq[ks], bh, yv);
      yv = mfma(aq[ks], bl, yv);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i = 16 * wave + 4 * lg + r;
      split_bf16(d[r], &Dh[l16][i], &Dl[l16][i]);
      split_bf16(d[r] * __expf(ell_c - ellr[r]), &Fh[l16][i], &Fl[l16][i]);
      yv[r] *= __expf(ellr[r]);
    }
    __syncthreads();

    // 3. Y += P D
#pragma unroll
    for (int k2 = 0; k2 < 2; ++k2) {
      const bf16x8_t dh = ld8(&Dh[l16][32 * k2 + 8 * lg]);
      yv = mfma(ap[k2], dh, yv);
      yv = mfma(ap[k2], ld8(&Dl[l16][32 * k2 + 8 * lg]), yv);
      yv = mfma(apl[k2], dh, yv);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int tk = t0 + 16 * wave + 4 * lg + r;
      if (tk < p.T) p.y[((size_t)tk * p.Hv + hv) * Dv + dv0 + l16] = dm_f2bf(yv[r]);
    }

    // 4. S = e_C0 S + (diag(e_Cj) D)^T K
    const float gc = __expf(ell_c);
#pragma unroll
    for (int n2 = 0; n2 < 2; ++n2) {
#pragma unroll
      for (int r = 0; r < 4; ++r) s[n2][r] *= gc;
#pragma unroll
      for (int k2 = 0; k2 < 2; ++k2) {
        s[n2] = mfma(ld8(&Fh[l16][32 * k2 + 8 * lg]), bk[n2][k2], s[n2]);
        s[n2] = mfma(ld8(&Fl[l16][32 * k2 + 8 * lg]), bk[n2][k2], s[n2]);
      }
    }
    __syncthreads();  // the tiles are rewritten by the next chunk
  }
#pragma unroll
  for (int n2 = 0; n2 < 2; ++n2)
#pragma unroll
    for (int r = 0; r < 4; ++r)
      p.state_out[((size_t)hv * Dv + dv0 + 4 * lg + r) * DK + 16 * (2 * wave + n2) + l16] = s[n2][r];
}

}  // namespace

// Returns -1 when the shapes are outside the chunked form (the caller keeps its other kernel).
int gdn_chunked_recurrence(ornith_ctx* ctx, const void* d_q, const void* d_k, const void* d_v, const float* d_g,
                           const void* d_beta, const float* d_state_in, int T, int Hk, int Hv, int Dk, int Dv,
                           void* d_y, float* d_state_out) {
  if (Dk != DK || Dv % 16 != 0 || Dv > 128 || Hv % Hk != 0) return -1;
  const int n = (T + C - 1) / C;
  const size_t per = (size_t)n * Hv;
  void* base = nullptr;
  const size_t need = per * ((size_t)C * DK * 2 * 2 + (size_t)C * Dv * 4 + (size_t)C * C * 2 * 2 + C * 4) +
                      (size_t)n * Hk * DK * C * 2 + 8 * 256;
  int rc = ornith_scratch(ctx, need, &base);
  if (rc) return rc;
  ScratchCursor sc(base);
  ChunkArgs a{};
  a.q = (const bf16_t*)d_q;
  a.k = (const bf16_t*)d_k;
  a.v = (const bf16_t*)d_v;
  a.g = d_g;
  a.beta = (const bf16_t*)d_beta;
  a.state_in = d_state_in;
  a.state_out = d_state_out;
  a.y = (bf16_t*)d_y;
  a.wh = sc.take<bf16_t>(per * C * DK);
  a.wl = sc.take<bf16_t>(per * C * DK);
  a.u = sc.take<float>(per * C * Dv);
  a.pm = sc.take<bf16_t>(per * C * C);
  a.pl = sc.take<bf16_t>(per * C * C);
  a.ell = sc.take<float>(per * C);
  a.kt = sc.take<bf16_t>((size_t)n * Hk * DK * C);
  a.T = T;
  a.Hk = Hk;
  a.Hv = Hv;
  a.Dv = Dv;
  a.nchunks = n;
  hipLaunchKernelGGL(gdn_chunk_prep_kernel, dim3(n, Hv), dim3(256), 0, ctx->stream, a);
  ORN_LAUNCH_CHECK("gdn_chunk_prep_kernel");
  hipLaunchKernelGGL(gdn_chunk_scan_kernel, dim3(Dv / 16, Hv), dim3(256), 0, ctx->stream, a);
  ORN_LAUNCH_CHECK("gdn_chunk_scan_kernel");
  return ORNITH_OK;
}
