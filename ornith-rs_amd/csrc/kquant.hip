// Q4_K / Q6_K dequantize, mat-vec and expert gather mat-vec for gfx950.
//
// Replaces kquant::{dequantize,qmv,gather_qmv}
// (/root/reference/src/ops/kquant.rs:418-433,539-595,741-770) and the kernels
// they dispatch (/root/reference/kernels/q4k.metal:64-249,628-656,
// /root/reference/kernels/q6k.metal:47-169,365-393). The storage format is the
// reference's three tensors per matrix, untouched.
//
// Schedule (this build's own, for 64-lane wavefronts; bandwidth bound, no MFMA):
//
//   A row of K weights is cut into chunks, one per lane:
//     Q4_K  16 code bytes = 32 weights: low nibbles are weights 64g+16h+i, high
//           nibbles the same +32 (g = 64-weight group, h = half, i < 16).
//           One 16-byte load per lane; a 2048-wide row is exactly 64 chunks, so
//           a wavefront reads a row's codes as one contiguous 1 KiB burst.
//     Q6_K  16 positions of one 128-half: ql[l], ql[l+32], qh[l] -> 64 weights
//           (l, l+32, l+64, l+96). Three 16-byte loads per lane.
//   chunk j belongs to lane j % 64; rows narrower than 64 chunks pack 64/LPR
//   rows into one wavefront (LPR lanes per row); rows wider than 64 chunks are
//   split over KS wavefronts whose lane partials are added through LDS in
//   ascending chunk order. Each lane keeps the activations of its chunk in
//   registers (they do not depend on the output row) and walks down the rows,
//   so the weight stream is the only traffic that scales with O.
//
//   The sum of a row is then: lane partials (ascending chunk), butterfly
//   v += v[l ^ s] for s = 32..1. Rows of a multi-token call are independent
//   accumulators over the same weights in the same order, which is what makes
//   row r of an M-row call bit-identical to that row alone (the property
//   /root/reference/src/ops/invariant.rs:88-116 buys with its exact window).
#include "dmath.h"
#include "rt.h"

namespace {

struct KqArgs {
  const uint8_t* qs;
  const uint8_t* scales;
  const uint16_t* dm;
  const void* x;
  void* y;
  const uint32_t* lhs;  // gather only
  const uint32_t* rhs;  // gather only
  int O, K;
  int E, x_rows;  // gather only: bounds for rhs / lhs (out-of-range ids are clamped)
  int iters;    // row iterations per wavefront
  int y_bf16;   // 1: round outputs to bf16, 0: fp32
};

// 16 consecutive activations -> fp32 registers
template <bool XF32>
__device__ __forceinline__ void load_x16(const void* xrow, int off, float (&v)[16]) {
  if constexpr (XF32) {
    const float4* p = reinterpret_cast<const float4*>(static_cast<const float*>(xrow) + off);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float4 f = p[i];
      v[4 * i + 0] = f.x;
      v[4 * i + 1] = f.y;
      v[4 * i + 2] = f.z;
      v[4 * i + 3] = f.w;
    }
  } else {
    const uint4* p = reinterpret_cast<const uint4*>(static_cast<const bf16_t*>(xrow) + off);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      uint4 w = p[i];
      v[8 * i + 0] = dm_bf2f_lo(w.x);
      v[8 * i + 1] = dm_bf2f_hi(w.x);
      v[8 * i + 2] = dm_bf2f_lo(w.y);
      v[8 * i + 3] = dm_bf2f_hi(w.y);
      v[8 * i + 4] = dm_bf2f_lo(w.z);
      v[8 * i + 5] = dm_bf2f_hi(w.z);
      v[8 * i + 6] = dm_bf2f_lo(w.w);
      v[8 * i + 7] = dm_bf2f_hi(w.w);
    }
  }
}

__device__ __forceinline__ float ub(uint32_t w, int k) { return (float)((w >> (8 * k)) & 0xffu); }

// ---- Q4_K ---------------------------------------------------------------
template <int M>
struct Q4Lane {
  float xl[M][16], xh[M][16], sl[M], sh[M];
  int b, g, h;  // block, 64-group, half

  template <bool XF32>
  __device__ __forceinline__ void load_x(const void* const (&xrow)[M], int chunk) {
    b = chunk >> 3;
    g = (chunk & 7) >> 1;
    h = chunk & 1;
    const int off = 256 * b + 64 * g + 16 * h;
#pragma unroll
    for (int t = 0; t < M; ++t) {
      load_x16<XF32>(xrow[t], off, xl[t]);
      load_x16<XF32>(xrow[t], off + 32, xh[t]);
      float a = 0.f, c = 0.f;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        a = a + xl[t][i];
        c = c + xh[t][i];
      }
      sl[t] = a;
      sh[t] = c;
    }
  }
};

struct Q4Row {
  uint4 q;
  uint32_t s0, s1, s2, dmw;
};

template <int M>
__device__ __forceinline__ Q4Row q4_load(const KqArgs& a, int64_t row, int nb, const Q4Lane<M>& L) {
  Q4Row r;
  const uint8_t* qrow = a.qs + row * (int64_t)nb * 128;
  r.q = *reinterpret_cast<const uint4*>(qrow + L.b * 128 + 32 * L.g + 16 * L.h);
  const uint32_t* sc = reinterpret_cast<const uint32_t*>(a.scales + (row * nb + L.b) * 12);
  r.s0 = sc[0];
  r.s1 = sc[1];
  r.s2 = sc[2];
  r.dmw = *reinterpret_cast<const uint32_t*>(a.dm + (row * nb + L.b) * 2);
  return r;
}

template <int M>
__device__ __forceinline__ void q4_accumulate(const Q4Row& r, const Q4Lane<M>& L, float (&acc)[M]) {
  const int sh16 = (L.g & 1) * 16;
  const uint32_t a = (r.s0 >> sh16) & 0xffffu, b = (r.s1 >> sh16) & 0xffffu,
                 c = (r.s2 >> sh16) & 0xffffu;
  uint32_t sc16, m16;
  if (L.g < 2) {
    sc16 = a & 0x3f3fu;
    m16 = b & 0x3f3fu;
  } else {
    sc16 = (c & 0x0f0fu) | ((a & 0xc0c0u) >> 2);
    m16 = ((c >> 4) & 0x0f0fu) | ((b & 0xc0c0u) >> 2);
  }
  const float s1 = (float)(sc16 & 0xffu), s2 = (float)(sc16 >> 8);
  const float m1 = (float)(m16 & 0xffu), m2 = (float)(m16 >> 8);
  const float d = dm_h2f((f16_t)(r.dmw & 0xffffu)), dmin = dm_h2f((f16_t)(r.dmw >> 16));

  const uint32_t w[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
  float lo[M], hi[M];
#pragma unroll
  for (int t = 0; t < M; ++t) lo[t] = hi[t] = 0.f;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const uint32_t wl = w[k] & 0x0f0f0f0fu;
    // high nibbles left in place: 16*n. Scaling by a power of two commutes with
    // every rounding below, so 16*sum == sum of 16*terms bit for bit.
    const uint32_t wh = w[k] & 0xf0f0f0f0u;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float fl = ub(wl, i), fh = ub(wh, i);
#pragma unroll
      for (int t = 0; t < M; ++t) {
        lo[t] = dm_fma(L.xl[t][4 * k + i], fl, lo[t]);
        hi[t] = dm_fma(L.xh[t][4 * k + i], fh, hi[t]);
      }
    }
  }
#pragma unroll
  for (int t = 0; t < M; ++t) {
    float t1 = lo[t] * s1;
    t1 = dm_fma(hi[t] * 0.0625f, s2, t1);
    float t2 = L.sl[t] * m1;
    t2 = dm_fma(L.sh[t], m2, t2);
    float p = d * t1;
    p = dm_fma(-dmin, t2, p);
    acc[t] = acc[t] + p;
  }
}

// ---- Q6_K ---------------------------------------------------------------
template <int M>
struct Q6Lane {
  float x[M][4][16];
  int b, n, u;

  template <bool XF32>
  __device__ __forceinline__ void load_x(const void* const (&xrow)[M], int chunk) {
    b = chunk >> 2;
    n = (chunk & 3) >> 1;
    u = chunk & 1;
    const int off = 256 * b + 128 * n + 16 * u;
#pragma unroll
    for (int t = 0; t < M; ++t)
#pragma unroll
      for (int g = 0; g < 4; ++g) load_x16<XF32>(xrow[t], off + 32 * g, x[t][g]);
  }
};

struct Q6Row {
  uint4 qa, qb, qh;  // ql[l], ql[l+32], qh[l]
  uint2 sc;
  uint16_t d;
};

template <int M>
__device__ __forceinline__ Q6Row q6_load(const KqArgs& a, int64_t row, int nb, const Q6Lane<M>& L) {
  Q6Row r;
  const uint8_t* blk = a.qs + (row * nb + L.b) * 192;
  r.qa = *reinterpret_cast<const uint4*>(blk + 64 * L.n + 16 * L.u);
  r.qb = *reinterpret_cast<const uint4*>(blk + 64 * L.n + 32 + 16 * L.u);
  r.qh = *reinterpret_cast<const uint4*>(blk + 128 + 32 * L.n + 16 * L.u);
  r.sc = *reinterpret_cast<const uint2*>(a.scales + (row * nb + L.b) * 16 + 8 * L.n);
  r.d = a.dm[row * nb + L.b];
  return r;
}

__device__ __forceinline__ float sb(uint32_t w, int k) { return (float)(int)(int8_t)((w >> (8 * k)) & 0xffu); }

template <int M>
__device__ __forceinline__ void q6_accumulate(const Q6Row& r, const Q6Lane<M>& L, float (&acc)[M]) {
  const uint32_t A[4] = {r.qa.x, r.qa.y, r.qa.z, r.qa.w};
  const uint32_t B[4] = {r.qb.x, r.qb.y, r.qb.z, r.qb.w};
  const uint32_t H[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
  float s[M][4];
#pragma unroll
  for (int t = 0; t < M; ++t)
#pragma unroll
    for (int g = 0; g < 4; ++g) s[t][g] = 0.f;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    uint32_t c[4];
    c[0] = (A[k] & 0x0f0f0f0fu) | ((H[k] << 4) & 0x30303030u);
    c[1] = (B[k] & 0x0f0f0f0fu) | ((H[k] << 2) & 0x30303030u);
    c[2] = ((A[k] >> 4) & 0x0f0f0f0fu) | (H[k] & 0x30303030u);
    c[3] = ((B[k] >> 4) & 0x0f0f0f0fu) | ((H[k] >> 2) & 0x30303030u);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        // code - 32, exact either as an integer or (as here) as a float subtract
        const float q = ub(c[g], i) - 32.0f;
#pragma unroll
        for (int t = 0; t < M; ++t) s[t][g] = dm_fma(L.x[t][g][4 * k + i], q, s[t][g]);
      }
    }
  }
  // scales: bytes u, u+2, u+4, u+6 of the half's eight
  const uint32_t lo = r.sc.x >> (8 * L.u), hi = r.sc.y >> (8 * L.u);
  const float c0 = sb(lo, 0), c1 = sb(lo, 2), c2 = sb(hi, 0), c3 = sb(hi, 2);
  const float d = dm_h2f(r.d);
#pragma unroll
  for (int t = 0; t < M; ++t) {
    float v = s[t][0] * c0;
    v = dm_fma(s[t][1], c1, v);
    v = dm_fma(s[t][2], c2, v);
    v = dm_fma(s[t][3], c3, v);
    acc[t] = acc[t] + d * v;
  }
}

template <int KIND, int M>
struct LaneOf;
template <int M>
struct LaneOf<ORNITH_Q4K, M> {
  using type = Q4Lane<M>;
};
template <int M>
struct LaneOf<ORNITH_Q6K, M> {
  using type = Q6Lane<M>;
};

// One kernel for plain and gathered mat-vecs.
//   KIND  format; LPR lanes per row (4,8,16,32,64); KS wavefronts per row (1,2)
//   M     activation rows sharing each weight read (1..4); gather uses M == 1
//   grid.x covers output rows, grid.y is the gather row (1 for plain)
template <int KIND, int LPR, int KS, int M, bool XF32, bool GATHER>
__global__ __launch_bounds__(256) void kq_qmv_kernel(KqArgs a) {
  constexpr int RPW = 64 / LPR;   // rows in flight per wavefront
  constexpr int WPB = 4 / KS;     // row-wavefronts per block
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int slot = lane / LPR, c = lane % LPR;
  const int ks = (KS == 1) ? 0 : (wave & 1);
  const int rw = (KS == 1) ? wave : (wave >> 1);
  const int nb = a.K >> 8;

  const size_t xsz = XF32 ? 4 : 2;
  const void* xrow[M];
  int64_t row0 = 0;  // first weight row of this matrix (expert offset)
  int64_t yrow0 = 0;
  if constexpr (GATHER) {
    const int r = blockIdx.y;
    const uint32_t xi = min(a.lhs[r], (uint32_t)(a.x_rows - 1));
    const uint32_t ei = min(a.rhs[r], (uint32_t)(a.E - 1));
    xrow[0] = static_cast<const char*>(a.x) + (size_t)xi * a.K * xsz;
    row0 = (int64_t)ei * a.O;
    yrow0 = (int64_t)r * a.O;
  } else {
#pragma unroll
    for (int t = 0; t < M; ++t) xrow[t] = static_cast<const char*>(a.x) + (size_t)t * a.K * xsz;
  }

  typename LaneOf<KIND, M>::type L;
  L.template load_x<XF32>(xrow, c + 64 * ks);

  __shared__ float part[(KS == 2) ? 2 * M * 64 : 1];

  const int rows_per_wave = RPW * a.iters;
  const int base = (blockIdx.x * WPB + rw) * rows_per_wave;
  for (int it = 0; it < a.iters; ++it) {
    const int o = base + it * RPW + slot;
    const bool valid = o < a.O;
    const int64_t row = row0 + (valid ? o : a.O - 1);
    float acc[M];
#pragma unroll
    for (int t = 0; t < M; ++t) acc[t] = 0.f;
    if constexpr (KIND == ORNITH_Q4K) {
      Q4Row r = q4_load(a, row, nb, L);
      q4_accumulate(r, L, acc);
    } else {
      Q6Row r = q6_load(a, row, nb, L);
      q6_accumulate(r, L, acc);
    }
    if constexpr (KS == 2) {
      // lane partial = (chunk l) + (chunk l + 64), in that order
      float* mine = part + rw * M * 64;
      __syncthreads();
      if (ks == 1) {
#pragma unroll
        for (int t = 0; t < M; ++t) mine[t * 64 + lane] = acc[t];
      }
      __syncthreads();
      if (ks == 0) {
#pragma unroll
        for (int t = 0; t < M; ++t) acc[t] = acc[t] + mine[t * 64 + lane];
      }
    }
#pragma unroll
    for (int t = 0; t < M; ++t) {
      const float v = dm_wave_sum<LPR>(acc[t]);
      if (c == 0 && ks == 0 && valid) {
        const int64_t yi = (GATHER ? yrow0 : (int64_t)t * a.O) + o;
        if (a.y_bf16)
          static_cast<bf16_t*>(a.y)[yi] = dm_f2bf(v);
        else
          static_cast<float*>(a.y)[yi] = v;
      }
    }
  }
}

// one thread per 256-weight block, the shape of the reference loop
template <int KIND>
__global__ void kq_dequant_kernel(const uint8_t* qs, const uint8_t* scales, const uint16_t* dm,
                                  int64_t nblocks, void* out, int out_bf16) {
  const int64_t ib = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (ib >= nblocks) return;
  auto put = [&](int i, float v) {
    if (out_bf16)
      static_cast<bf16_t*>(out)[ib * 256 + i] = dm_f2bf(v);
    else
      static_cast<float*>(out)[ib * 256 + i] = v;
  };
  if constexpr (KIND == ORNITH_Q4K) {
    const uint8_t* q = qs + ib * 128;
    const uint8_t* sc = scales + ib * 12;
    const float d = dm_h2f(dm[ib * 2]), dmin = dm_h2f(dm[ib * 2 + 1]);
    for (int cch = 0; cch < 4; ++cch) {
      float dd[2], mm[2];
      for (int k = 0; k < 2; ++k) {
        const int j = 2 * cch + k;
        uint32_t s, m;
        if (j < 4) {
          s = sc[j] & 63;
          m = sc[j + 4] & 63;
        } else {
          s = (sc[j + 4] & 0xF) | ((sc[j - 4] >> 6) << 4);
          m = (sc[j + 4] >> 4) | ((sc[j] >> 6) << 4);
        }
        dd[k] = d * (float)s;
        mm[k] = dmin * (float)m;
      }
      for (int l = 0; l < 32; ++l) {
        put(64 * cch + l, dd[0] * (float)(q[32 * cch + l] & 0xF) - mm[0]);
        put(64 * cch + 32 + l, dd[1] * (float)(q[32 * cch + l] >> 4) - mm[1]);
      }
    }
  } else {
    const float d = dm_h2f(dm[ib]);
    for (int n = 0; n < 2; ++n) {
      const uint8_t* ql = qs + ib * 192 + 64 * n;
      const uint8_t* qh = qs + ib * 192 + 128 + 32 * n;
      const int8_t* sc = reinterpret_cast<const int8_t*>(scales + ib * 16) + 8 * n;
      for (int l = 0; l < 32; ++l) {
        const int is = l / 16;
        const int q1 = (int)((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
        const int q2 = (int)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
        const int q3 = (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
        const int q4 = (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
        put(128 * n + l, d * (float)sc[is] * (float)q1);
        put(128 * n + l + 32, d * (float)sc[is + 2] * (float)q2);
        put(128 * n + l + 64, d * (float)sc[is + 4] * (float)q3);
        put(128 * n + l + 96, d * (float)sc[is + 6] * (float)q4);
      }
    }
  }
}

template <int KIND, int LPR, int KS, int M, bool XF32, bool GATHER>
int launch_one(ornith_ctx* ctx, const KqArgs& a, int grid_y) {
  constexpr int RPW = 64 / LPR, WPB = 4 / KS;
  const int rows_per_block = RPW * WPB * a.iters;
  dim3 grid((a.O + rows_per_block - 1) / rows_per_block, grid_y, 1);
  hipLaunchKernelGGL((kq_qmv_kernel<KIND, LPR, KS, M, XF32, GATHER>), grid, dim3(256), 0,
                     ctx->stream, a);
  ORN_LAUNCH_CHECK("kq_qmv_kernel");
  return ORNITH_OK;
}

template <int KIND, int M, bool XF32, bool GATHER>
int launch_shape(ornith_ctx* ctx, const KqArgs& a, int grid_y) {
  const int nch = (a.K >> 8) * (KIND == ORNITH_Q4K ? 8 : 4);
  switch (nch) {
    case 4: return launch_one<KIND, 4, 1, M, XF32, GATHER>(ctx, a, grid_y);
    case 8: return launch_one<KIND, 8, 1, M, XF32, GATHER>(ctx, a, grid_y);
    case 16: return launch_one<KIND, 16, 1, M, XF32, GATHER>(ctx, a, grid_y);
    case 32: return launch_one<KIND, 32, 1, M, XF32, GATHER>(ctx, a, grid_y);
    case 64: return launch_one<KIND, 64, 1, M, XF32, GATHER>(ctx, a, grid_y);
    case 128: return launch_one<KIND, 64, 2, M, XF32, GATHER>(ctx, a, grid_y);
    default:
      return ornith_fail(ORNITH_ERR_UNSUPPORTED,
                         "k-quant mat-vec: K=%d is not one of the supported widths "
                         "(Q4_K: 256,512,1024,2048,4096; Q6_K: 256,512,1024,2048,4096,8192)",
                         a.K);
  }
}

template <int KIND, bool XF32>
int launch_m(ornith_ctx* ctx, const KqArgs& a, int M) {
  switch (M) {
    case 1: return launch_shape<KIND, 1, XF32, false>(ctx, a, 1);
    case 2: return launch_shape<KIND, 2, XF32, false>(ctx, a, 1);
    case 3: return launch_shape<KIND, 3, XF32, false>(ctx, a, 1);
    default: return launch_shape<KIND, 4, XF32, false>(ctx, a, 1);
  }
}

// rows each wavefront walks: enough blocks to cover the chip several times over
// while keeping the activation registers amortised.
int pick_iters(const ornith_ctx* ctx, int kind, int K, int O, int grid_y) {
  const int nch = (K >> 8) * (kind == ORNITH_Q4K ? 8 : 4);
  const int lpr = nch >= 64 ? 64 : nch;
  const int ks = nch > 64 ? 2 : 1;
  const int rows_per_pass = (64 / lpr) * (4 / ks);  // rows a block covers per iteration
  const long blocks_at_1 = ((long)O + rows_per_pass - 1) / rows_per_pass * grid_y;
  const long want = (long)ctx->compute_units * 8;
  int iters = (int)(blocks_at_1 / want);
  if (iters < 1) iters = 1;
  if (iters > 8) iters = 8;
  return iters;
}

int check_matrix(const ornith_kmatrix* w, const char* who) {
  ORN_REQUIRE(w, "%s: null matrix", who);
  ORN_REQUIRE(w->kind == ORNITH_Q4K || w->kind == ORNITH_Q6K, "%s: unknown k-quant kind %d", who,
              w->kind);
  ORN_REQUIRE(w->E >= 1 && w->O >= 1 && w->K >= 256, "%s: bad dims E=%d O=%d K=%d", who, w->E,
              w->O, w->K);
  ORN_REQUIRE(w->K % 256 == 0, "%s: %d is not a multiple of 256", who, w->K);
  ORN_REQUIRE(w->d_qs && w->d_scales && w->d_dm, "%s: null tensor", who);
  return ORNITH_OK;
}

}  // namespace

extern "C" {

int ornith_kmatrix_check(const ornith_kmatrix* w, size_t qs_bytes, size_t scales_bytes,
                         size_t dm_bytes) {
  int rc = check_matrix(w, "KMatrix");
  if (rc) return rc;
  const size_t blocks = (size_t)w->E * w->O * (w->K / 256);
  const size_t cb = w->kind == ORNITH_Q4K ? 128 : 192, sb_ = w->kind == ORNITH_Q4K ? 12 : 16,
               db = w->kind == ORNITH_Q4K ? 4 : 2;
  const char* name = w->kind == ORNITH_Q4K ? "q4k" : "q6k";
  ORN_REQUIRE(qs_bytes == blocks * cb, "%s qs size: %zu bytes, %zu blocks want %zu", name, qs_bytes,
              blocks, blocks * cb);
  ORN_REQUIRE(scales_bytes == blocks * sb_, "%s scales size: %zu bytes, want %zu", name,
              scales_bytes, blocks * sb_);
  ORN_REQUIRE(dm_bytes == blocks * db, "%s dm size: %zu bytes, want %zu", name, dm_bytes,
              blocks * db);
  return ORNITH_OK;
}

int ornith_kq_dequantize(ornith_ctx* ctx, const ornith_kmatrix* w, void* d_out, int out_dtype) {
  ORN_REQUIRE(ctx && d_out, "kq_dequantize: null argument");
  int rc = check_matrix(w, "kq_dequantize");
  if (rc) return rc;
  const int64_t blocks = (int64_t)w->E * w->O * (w->K / 256);
  dim3 grid((unsigned)((blocks + 63) / 64));
  if (w->kind == ORNITH_Q4K)
    hipLaunchKernelGGL(kq_dequant_kernel<ORNITH_Q4K>, grid, dim3(64), 0, ctx->stream,
                       (const uint8_t*)w->d_qs, (const uint8_t*)w->d_scales,
                       (const uint16_t*)w->d_dm, blocks, d_out, out_dtype == ORNITH_BF16);
  else
    hipLaunchKernelGGL(kq_dequant_kernel<ORNITH_Q6K>, grid, dim3(64), 0, ctx->stream,
                       (const uint8_t*)w->d_qs, (const uint8_t*)w->d_scales,
                       (const uint16_t*)w->d_dm, blocks, d_out, out_dtype == ORNITH_BF16);
  ORN_LAUNCH_CHECK("kq_dequant_kernel");
  return ORNITH_OK;
}

int ornith_kq_qmv(ornith_ctx* ctx, const ornith_kmatrix* w, const void* d_x, int x_dtype, int M,
                  void* d_y, int y_dtype) {
  ORN_REQUIRE(ctx && d_x && d_y, "kq_qmv: null argument");
  int rc = check_matrix(w, "kq_qmv");
  if (rc) return rc;
  ORN_REQUIRE(w->E == 1, "kq_qmv: matrix has %d experts; use gather_qmv", w->E);
  ORN_REQUIRE(M >= 1, "kq_qmv: M=%d", M);
  ORN_REQUIRE(((uintptr_t)d_x & 15) == 0, "kq_qmv: x must be 16-byte aligned");
  const size_t xs = ornith_dtype_size(x_dtype), ys = ornith_dtype_size(y_dtype);
  KqArgs a{};
  a.qs = (const uint8_t*)w->d_qs;
  a.scales = (const uint8_t*)w->d_scales;
  a.dm = (const uint16_t*)w->d_dm;
  a.O = w->O;
  a.K = w->K;
  a.y_bf16 = y_dtype == ORNITH_BF16;
  a.iters = pick_iters(ctx, w->kind, w->K, w->O, 1);
  for (int m0 = 0; m0 < M; m0 += 4) {
    const int mw = M - m0 < 4 ? M - m0 : 4;
    a.x = (const char*)d_x + (size_t)m0 * w->K * xs;
    a.y = (char*)d_y + (size_t)m0 * w->O * ys;
    if (w->kind == ORNITH_Q4K)
      rc = x_dtype == ORNITH_F32 ? launch_m<ORNITH_Q4K, true>(ctx, a, mw)
                                 : launch_m<ORNITH_Q4K, false>(ctx, a, mw);
    else
      rc = x_dtype == ORNITH_F32 ? launch_m<ORNITH_Q6K, true>(ctx, a, mw)
                                 : launch_m<ORNITH_Q6K, false>(ctx, a, mw);
    if (rc) return rc;
  }
  return ORNITH_OK;
}

int ornith_kq_gather_qmv(ornith_ctx* ctx, const ornith_kmatrix* w, const void* d_x, int x_dtype,
                         int x_rows, const uint32_t* d_lhs, const uint32_t* d_rhs, int rows,
                         void* d_y, int y_dtype) {
  ORN_REQUIRE(ctx && d_x && d_y && d_lhs && d_rhs, "kq_gather_qmv: null argument");
  int rc = check_matrix(w, "kq_gather_qmv");
  if (rc) return rc;
  ORN_REQUIRE(rows >= 0 && rows <= 65535, "kq_gather_qmv: rows=%d", rows);
  ORN_REQUIRE(x_rows >= 1, "kq_gather_qmv: x_rows=%d", x_rows);
  ORN_REQUIRE(((uintptr_t)d_x & 15) == 0, "kq_gather_qmv: x must be 16-byte aligned");
  if (rows == 0) return ORNITH_OK;
  KqArgs a{};
  a.qs = (const uint8_t*)w->d_qs;
  a.scales = (const uint8_t*)w->d_scales;
  a.dm = (const uint16_t*)w->d_dm;
  a.x = d_x;
  a.y = d_y;
  a.lhs = d_lhs;
  a.rhs = d_rhs;
  a.E = w->E;
  a.x_rows = x_rows;
  a.O = w->O;
  a.K = w->K;
  a.y_bf16 = y_dtype == ORNITH_BF16;
  a.iters = pick_iters(ctx, w->kind, w->K, w->O, rows);
  if (w->kind == ORNITH_Q4K)
    return x_dtype == ORNITH_F32 ? launch_shape<ORNITH_Q4K, 1, true, true>(ctx, a, rows)
                                 : launch_shape<ORNITH_Q4K, 1, false, true>(ctx, a, rows);
  return x_dtype == ORNITH_F32 ? launch_shape<ORNITH_Q6K, 1, true, true>(ctx, a, rows)
                               : launch_shape<ORNITH_Q6K, 1, false, true>(ctx, a, rows);
}

}  // extern "C"
