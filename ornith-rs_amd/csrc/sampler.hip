// The sampled-token path: log-softmax, top-p, top-k, inverse-CDF draw, threefry keys.
//
// Replaces TopSampler / apply_top_p / apply_top_k / categorical_sampling
// (/root/reference/src/sample.rs:79-225) and what they are built from: argsort_last_axis,
// cumsum_last_axis, take / put_along_last_axis, searchsorted, all_reduce
// (/root/reference/src/ops/{sort,scan,indexing,searchsorted,reduce}.rs), the elementwise
// steps of /root/reference/kernels/sampler_ops.metal:36-140 and the key sequence of
// /root/reference/src/ops/random.rs:16-67 (threefry2x32, vendored random.metal:5-66).
//
// Everything is in the logits' dtype, bf16, except the CDF (fp32), as in the reference.
//
// Sort: bf16 has 65536 values, so the stable argsort is an LSD radix sort of the 16-bit
// order-preserving key in two 8-bit passes (histogram per 1024-element block, one
// exclusive scan over the digit-major table, scatter with ranks from wavefront ballots).
// It is integer work: the result is THE stable argsort, no order of evaluation involved.
//
// Cumulative sums: a row is cut into chunks of 1024 and a chunk into 16 segments of 64
// (one wavefront each). Inside a segment the inclusive scan is Hillis-Steele
// (v[l] += v[l-s], s = 1..32); segment totals are added left to right inside the chunk,
// chunk totals left to right over the row; cum_i = (base_chunk + off_segment) + v_i.
// In bf16 every add rounds. The draw takes the first index whose inclusive cdf exceeds
// u, which is what searchsorted(exclusive cdf, u, right) - 1 selects.
//
// The key sequence lives on the host (64 bits of integer state per sampler); the raw
// random word is passed to the draw kernel as an argument.
#include <cstring>
#include <utility>

#include "dmath.h"
#include "rt.h"

namespace {

constexpr int RB = 1024;  // elements per workgroup in every kernel here
constexpr uint16_t kNegInf = 0xFF80u;

// ---- threefry (host) ---------------------------------------------------------------
inline uint32_t rotl32(uint32_t v, int r) { return (v << r) | (v >> (32 - r)); }

void threefry2x32(const uint32_t key[2], uint32_t c0, uint32_t c1, uint32_t out[2]) {
  static const int rot[2][4] = {{13, 15, 26, 6}, {17, 29, 16, 24}};
  const uint32_t ks[3] = {key[0], key[1], key[0] ^ key[1] ^ 0x1BD11BDAu};
  uint32_t x = c0 + ks[0], y = c1 + ks[1];
  for (int i = 0; i < 5; ++i) {
    for (int j = 0; j < 4; ++j) {
      x += y;
      y = rotl32(y, rot[i % 2][j]);
      y ^= x;
    }
    x += ks[(i + 1) % 3];
    y += ks[(i + 2) % 3] + (uint32_t)i + 1u;
  }
  out[0] = x;
  out[1] = y;
}

// ---- Philox4x32-10 (host): Salmon, Moraes, Dror, Shaw, "Parallel random numbers: as easy as
// 1, 2, 3" (SC'11); Random123's philox4x32 at 10 rounds ---------------------------------
void philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3], k0 = key[0], k1 = key[1];
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1, n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

// ---- radix sort ----------------------------------------------------------------------
__device__ __forceinline__ uint32_t sort_key(uint32_t b) {
  return (b & 0x8000u) ? (0xFFFFu - b) : (b | 0x8000u);
}

template <int PASS>
__device__ __forceinline__ uint32_t load_key(const bf16_t* x, int negate, const uint16_t* keys_in, int i) {
  if constexpr (PASS == 0)
    return sort_key(negate ? (uint32_t)(x[i] ^ 0x8000u) : (uint32_t)x[i]);
  else
    return keys_in[i];
}

// table is digit-major: table[d * nblk + block]
template <int PASS>
__global__ __launch_bounds__(RB) void radix_hist_kernel(const bf16_t* x, int negate,
                                                        const uint16_t* keys_in, int n, int nblk,
                                                        uint32_t* table) {
  __shared__ uint32_t h[256];
  const int tid = threadIdx.x, i = blockIdx.x * RB + tid;
  if (tid < 256) h[tid] = 0;
  __syncthreads();
  if (i < n) {
    const uint32_t key = load_key<PASS>(x, negate, keys_in, i);
    atomicAdd(&h[PASS == 0 ? (key & 255u) : (key >> 8)], 1u);
  }
  __syncthreads();
  if (tid < 256) table[(size_t)tid * nblk + blockIdx.x] = h[tid];
}

// in-place exclusive scan of m counters (a multiple of 4, 16-byte aligned) by one workgroup, in
// tiles of 4096 consecutive counters: a thread takes four neighbours as one 16-byte load, so a
// 62 k table is 16 tiles (a barrier and a wavefront scan each; with a counter a thread it was
// 61). All tiles are fetched into registers before the first is scanned, so the walk never
// waits on memory. One barrier a tile: the wavefront totals of consecutive tiles alternate
// between two LDS rows, and every thread keeps the running total itself. Integer sums: the
// result does not depend on the grouping.
__global__ __launch_bounds__(RB) void radix_scan_kernel(uint32_t* table, int m) {
  constexpr int NW = RB / 64, TILE = 4 * RB;
  __shared__ uint32_t wtot[2][NW];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  constexpr int G = 16;
  uint32_t carry = 0;
  for (int t0 = 0; t0 * TILE < m; t0 += G) {
    uint4 v[G];
#pragma unroll
    for (int t = 0; t < G; ++t) {
      const int j = (t0 + t) * TILE + 4 * tid;
      v[t] = j < m ? *reinterpret_cast<const uint4*>(table + j) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < G; ++t) {
      if ((t0 + t) * TILE >= m) break;
      // the thread's four, inclusive scan of the sums inside the wavefront, then across the 16
      // wavefront totals
      const uint32_t p1 = v[t].x, p2 = p1 + v[t].y, p3 = p2 + v[t].z, own = p3 + v[t].w;
      uint32_t x = own;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const uint32_t o = __shfl_up(x, d, 64);
        if (lane >= d) x += o;
      }
      if (lane == 63) wtot[t & 1][wave] = x;
      __syncthreads();
      uint32_t before = carry, total = 0;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const uint32_t c = wtot[t & 1][w];
        before += w < wave ? c : 0u;
        total += c;
      }
      const int j = (t0 + t) * TILE + 4 * tid;
      const uint32_t b = before + x - own;
      if (j < m) *reinterpret_cast<uint4*>(table + j) = make_uint4(b, b + p1, b + p2, b + p3);
      carry += total;
    }
    __syncthreads();  // (G is even: the next round starts on row 0 again, which tile G - 2 used)
  }
}

template <int PASS>
__global__ __launch_bounds__(RB) void radix_scatter_kernel(const bf16_t* x, int negate,
                                                           const uint16_t* keys_in,
                                                           const uint32_t* idx_in, int n, int nblk,
                                                           const uint32_t* table, uint16_t* keys_out,
                                                           uint32_t* idx_out) {
  __shared__ uint32_t wcount[RB / 64][256];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, i = blockIdx.x * RB + tid;
  for (int j = tid; j < (RB / 64) * 256; j += RB) (&wcount[0][0])[j] = 0;
  __syncthreads();
  const bool valid = i < n;
  const uint32_t key = valid ? load_key<PASS>(x, negate, keys_in, i) : 0u;
  const uint32_t d = PASS == 0 ? (key & 255u) : (key >> 8);
  // lanes of this wavefront holding the same digit
  unsigned long long same = __ballot(valid);
#pragma unroll
  for (int bit = 0; bit < 8; ++bit) {
    const bool set = (d >> bit) & 1u;
    const unsigned long long b = __ballot(valid && set);
    same &= set ? b : ~b;
  }
  const uint32_t rank = __popcll(same & ((1ull << lane) - 1ull));
  if (valid && rank == 0) wcount[wave][d] = __popcll(same);
  __syncthreads();
  if (tid < 256) {
    uint32_t acc = 0;
#pragma unroll
    for (int w = 0; w < RB / 64; ++w) {
      const uint32_t c = wcount[w][tid];
      wcount[w][tid] = acc;
      acc += c;
    }
  }
  __syncthreads();
  if (valid) {
    const uint32_t pos = table[(size_t)d * nblk + blockIdx.x] + wcount[wave][d] + rank;
    idx_out[pos] = PASS == 0 ? (uint32_t)i : idx_in[i];
    if constexpr (PASS == 0) keys_out[pos] = (uint16_t)key;
  }
}

size_t argsort_workspace(int n) {
  const int nblk = (n + RB - 1) / RB;
  return (size_t)n * (2 + 4) + (size_t)256 * nblk * 4 + 3 * 256;
}

int argsort_impl(ornith_ctx* ctx, const bf16_t* x, int n, int negate, uint32_t* idx_out,
                 ScratchCursor& sc) {
  const int nblk = (n + RB - 1) / RB;
  uint16_t* keys = sc.take<uint16_t>(n);
  uint32_t* idx1 = sc.take<uint32_t>(n);
  uint32_t* table = sc.take<uint32_t>((size_t)256 * nblk);
  hipLaunchKernelGGL(radix_hist_kernel<0>, dim3(nblk), dim3(RB), 0, ctx->stream, x, negate,
                     (const uint16_t*)nullptr, n, nblk, table);
  hipLaunchKernelGGL(radix_scan_kernel, dim3(1), dim3(RB), 0, ctx->stream, table, 256 * nblk);
  hipLaunchKernelGGL(radix_scatter_kernel<0>, dim3(nblk), dim3(RB), 0, ctx->stream, x, negate,
                     (const uint16_t*)nullptr, (const uint32_t*)nullptr, n, nblk, table, keys, idx1);
  hipLaunchKernelGGL(radix_hist_kernel<1>, dim3(nblk), dim3(RB), 0, ctx->stream, x, negate, keys, n,
                     nblk, table);
  hipLaunchKernelGGL(radix_scan_kernel, dim3(1), dim3(RB), 0, ctx->stream, table, 256 * nblk);
  hipLaunchKernelGGL(radix_scatter_kernel<1>, dim3(nblk), dim3(RB), 0, ctx->stream, x, negate, keys,
                     idx1, n, nblk, table, (uint16_t*)nullptr, idx_out);
  ORN_LAUNCH_CHECK("radix sort kernels");
  return ORNITH_OK;
}

// ---- scans ---------------------------------------------------------------------------
template <bool BF16>
__device__ __forceinline__ float add_r(float a, float b) {
  const float r = a + b;
  return BF16 ? dm_rb(r) : r;
}

// stage 1: segment-local inclusive scans, segment offsets inside the chunk, chunk totals.
// `v` is the calling thread's element (0 past the end); every thread of the workgroup calls.
template <bool BF16>
__device__ __forceinline__ void scan_local_body(float v, int n, float* vloc, float* segoff, float* chunk_tot) {
  __shared__ float seg[RB / 64], so[RB / 64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, i = blockIdx.x * RB + tid;
#pragma unroll
  for (int s = 1; s < 64; s <<= 1) {
    const float o = __shfl_up(v, s, 64);
    if (lane >= s) v = add_r<BF16>(v, o);
  }
  if (lane == 63) seg[wave] = v;
  __syncthreads();
  if (tid == 0) {
    float off = 0.f;
    for (int g = 0; g < RB / 64; ++g) {
      so[g] = off;
      off = add_r<BF16>(off, seg[g]);
    }
    chunk_tot[blockIdx.x] = off;
  }
  __syncthreads();
  if (i < n) vloc[i] = v;
  if (lane == 0) segoff[blockIdx.x * (RB / 64) + wave] = so[wave];
}
template <bool BF16>
__global__ __launch_bounds__(RB) void scan_local_kernel(const float* in, int n, float* vloc,
                                                        float* segoff, float* chunk_tot) {
  const int i = blockIdx.x * RB + threadIdx.x;
  scan_local_body<BF16>(i < n ? in[i] : 0.f, n, vloc, segoff, chunk_tot);
}
// the same over out[j] = bf16(exp(lp[S[j]])) made on the way in (the sorted probabilities of top-p)
__global__ __launch_bounds__(RB) void gather_exp_scan_kernel(const bf16_t* lp, const uint32_t* S, int n,
                                                             float* vloc, float* segoff, float* chunk_tot) {
  const int j = blockIdx.x * RB + threadIdx.x;
  scan_local_body<true>(j < n ? dm_rb(dm_exp(dm_bf2f(lp[S[j]]))) : 0.f, n, vloc, segoff, chunk_tot);
}

// base of this chunk (sum of the chunk totals before it, left to right) and the row total
template <bool BF16>
__device__ __forceinline__ void chunk_base(const float* chunk_tot, int nch, float& base, float& total) {
  __shared__ float s_base, s_total;
  __shared__ float s_tot[RB];
  // the totals come in with one coalesced load per 1024 chunks; the left-to-right sum over
  // them is the only sequential part
  float acc = 0.f, b = 0.f;
  for (int c0 = 0; c0 < nch; c0 += RB) {
    if (c0 + (int)threadIdx.x < nch) s_tot[threadIdx.x] = chunk_tot[c0 + threadIdx.x];
    __syncthreads();
    if (threadIdx.x == 0) {
      const int n = min(RB, nch - c0);
      for (int c = 0; c < n; ++c) {
        if (c0 + c == (int)blockIdx.x) b = acc;
        acc = add_r<BF16>(acc, s_tot[c]);
      }
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    s_base = b;
    s_total = acc;
  }
  __syncthreads();
  base = s_base;
  total = s_total;
}

template <bool BF16>
__device__ __forceinline__ float cum_at(const float* vloc, const float* segoff, float base, int i) {
  const float pre = add_r<BF16>(base, segoff[i >> 6]);
  return add_r<BF16>(pre, vloc[i]);
}

// stage 2 variants
template <bool BF16>
__global__ __launch_bounds__(RB) void scan_out_kernel(const float* vloc, const float* segoff,
                                                      const float* chunk_tot, int n, int nch,
                                                      void* out) {
  float base, total;
  chunk_base<BF16>(chunk_tot, nch, base, total);
  const int i = blockIdx.x * RB + threadIdx.x;
  if (i >= n) return;
  const float c = cum_at<BF16>(vloc, segoff, base, i);
  if (BF16)
    static_cast<bf16_t*>(out)[i] = dm_f2bf(c);
  else
    static_cast<float*>(out)[i] = c;
}

// top-p: keep[S[j]] = cum_j > thresh; out = keep ? lp : -inf
__global__ __launch_bounds__(RB) void top_p_apply_kernel(const float* vloc, const float* segoff,
                                                         const float* chunk_tot, int n, int nch,
                                                         const uint32_t* S, const bf16_t* lp,
                                                         float thresh, bf16_t* out) {
  float base, total;
  chunk_base<true>(chunk_tot, nch, base, total);
  const int j = blockIdx.x * RB + threadIdx.x;
  if (j >= n) return;
  const float c = cum_at<true>(vloc, segoff, base, j);
  const uint32_t t = S[j];
  out[t] = c > thresh ? lp[t] : kNegInf;
}

__global__ void widen_bf16_kernel(const bf16_t* in, int n, float* out) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = dm_bf2f(in[i]);
}
__global__ void fill_u16_kernel(uint16_t* p, int n, uint16_t v) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}
// out[order[j]] = lp[order[j]] for j < k
__global__ void top_k_keep_kernel(const bf16_t* lp, const uint32_t* order, int k, bf16_t* out) {
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j < k) out[order[j]] = lp[order[j]];
}

// ---- the draw --------------------------------------------------------------------------
// x = float(bf16(lp * scale)); per-chunk maxima
__global__ __launch_bounds__(RB) void cat_scale_kernel(const bf16_t* lp, int n, float scale, float* x,
                                                       float* pmax) {
  __shared__ float red[RB / 64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, i = blockIdx.x * RB + tid;
  float v = -DM_INF;
  if (i < n) {
    v = dm_rb(dm_bf2f(lp[i]) * scale);
    x[i] = v;
  }
  float m = dm_wave_max<64>(v);
  if (lane == 0) red[wave] = m;
  __syncthreads();
  if (tid == 0) {
    for (int w = 1; w < RB / 64; ++w) m = red[w] > m ? red[w] : m;
    pmax[blockIdx.x] = m;
  }
}

// w = isinf(m) ? (x == m) : exp(x - m), in place over x (m: the row maximum from the chunk
// maxima), and in the same launch the chunk's scan_local_kernel<false> over those weights (the
// weight is scanned from the register it was made in: same values, same order as a launch of
// its own). `init`, when given, is the search's (first, last) pair, reset here by one thread.
__global__ __launch_bounds__(RB) void cat_weights_scan_kernel(float* x, int n, const float* pmax, int nch,
                                                              float* vloc, float* segoff, float* chunk_tot,
                                                              uint32_t* init) {
  __shared__ float red[RB / 64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, i = blockIdx.x * RB + tid;
  if (init && blockIdx.x == 0 && tid == 0) {
    init[0] = 0xffffffffu;
    init[1] = 0u;
  }
  float m = -DM_INF;
  for (int c = tid; c < nch; c += RB) m = pmax[c] > m ? pmax[c] : m;
  m = dm_wave_max<64>(m);
  if (lane == 0) red[wave] = m;
  __syncthreads();
  m = red[0];
#pragma unroll
  for (int w = 1; w < RB / 64; ++w) m = red[w] > m ? red[w] : m;
  const bool inf = m == DM_INF || m == -DM_INF;
  float v = 0.f;
  if (i < n) {
    const float xv = x[i];
    v = inf ? (xv == m ? 1.f : 0.f) : dm_exp(xv - m);
    x[i] = v;
  }
  scan_local_body<false>(v, n, vloc, segoff, chunk_tot);
}

// u = min(float(bits) / 2^32, nextafter(1, 0)) * total; first index with cdf > u, last with w > 0
// (first_last[2], when asked for, receives the bits of the row total)
__global__ __launch_bounds__(RB) void cat_search_kernel(const float* vloc, const float* segoff,
                                                        const float* chunk_tot, const float* w, int n,
                                                        int nch, uint32_t bits, uint32_t* first_last,
                                                        bool store_total) {
  float base, total;
  chunk_base<false>(chunk_tot, nch, base, total);
  if (store_total && blockIdx.x == 0 && threadIdx.x == 0) first_last[2] = __float_as_uint(total);
  const int i = blockIdx.x * RB + threadIdx.x;
  float u = (float)bits / 4294967296.0f;
  const float upper = __uint_as_float(0x3f7fffffu);
  u = u < upper ? u : upper;
  u = 1.0f * u + 0.0f;
  u = u * total;
  uint32_t first = 0xffffffffu, last = 0u;
  if (i < n) {
    if (cum_at<false>(vloc, segoff, base, i) > u) first = (uint32_t)i;
    if (w[i] > 0.f) last = (uint32_t)i;
  }
  // one atomic per workgroup, not per element: half the vocabulary lies above u
  __shared__ uint32_t s_first[RB / 64], s_last[RB / 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    first = min(first, (uint32_t)__shfl_xor((int)first, d, 64));
    last = max(last, (uint32_t)__shfl_xor((int)last, d, 64));
  }
  if (lane == 0) {
    s_first[wave] = first;
    s_last[wave] = last;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w2 = 1; w2 < RB / 64; ++w2) {
      first = min(first, s_first[w2]);
      last = max(last, s_last[w2]);
    }
    if (first != 0xffffffffu) atomicMin(&first_last[0], first);
    if (last != 0u) atomicMax(&first_last[1], last);
  }
}

__global__ void cat_init_kernel(uint32_t* first_last) {
  first_last[0] = 0xffffffffu;
  first_last[1] = 0u;
}
__global__ void cat_pick_kernel(const uint32_t* first_last, uint32_t* token) {
  token[0] = first_last[0] != 0xffffffffu ? first_last[0] : first_last[1];
}

// lp = bf16(x - lse) for one row
__global__ __launch_bounds__(RB) void logprob_kernel(const bf16_t* logits, const bf16_t* lse, int n,
                                                     bf16_t* lp) {
  const int i = blockIdx.x * RB + threadIdx.x;
  if (i < n) lp[i] = dm_f2bf(dm_bf2f(logits[i]) - dm_bf2f(lse[0]));
}

int nchunks(int n) { return (n + RB - 1) / RB; }

struct ScanBufs {
  float* vloc;
  float* segoff;
  float* chunk_tot;
};
ScanBufs scan_bufs(ScratchCursor& sc, int n) {
  const int nch = nchunks(n);
  return ScanBufs{sc.take<float>(n), sc.take<float>((size_t)nch * (RB / 64)), sc.take<float>(nch)};
}
size_t scan_workspace(int n) { return (size_t)n * 4 + (size_t)nchunks(n) * (RB / 64 + 1) * 4 + 3 * 256; }

int top_p_impl(ornith_ctx* ctx, const bf16_t* lp, int V, double top_p, bf16_t* out, ScratchCursor& sc) {
  const int nch = nchunks(V);
  uint32_t* S = sc.take<uint32_t>(V);
  (void)sc.take<float>(V);  // (kept: the workspace layout callers size for)
  ScanBufs b = scan_bufs(sc, V);
  int rc = argsort_impl(ctx, lp, V, 0, S, sc);
  if (rc) return rc;
  hipLaunchKernelGGL(gather_exp_scan_kernel, dim3(nch), dim3(RB), 0, ctx->stream, lp, S, V, b.vloc, b.segoff,
                     b.chunk_tot);
  // weak-typed scalar: 1 - top_p rounded to the array's dtype
  const float t32 = (float)(1.0 - top_p);
  uint32_t u;
  memcpy(&u, &t32, 4);
  u = (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u;
  float thresh;
  memcpy(&thresh, &u, 4);
  hipLaunchKernelGGL(top_p_apply_kernel, dim3(nch), dim3(RB), 0, ctx->stream, b.vloc, b.segoff,
                     b.chunk_tot, V, nch, S, lp, thresh, out);
  ORN_LAUNCH_CHECK("top-p kernels");
  return ORNITH_OK;
}

int top_k_impl(ornith_ctx* ctx, const bf16_t* lp, int V, int top_k, bf16_t* out, ScratchCursor& sc) {
  uint32_t* order = sc.take<uint32_t>(V);
  int rc = argsort_impl(ctx, lp, V, 1, order, sc);
  if (rc) return rc;
  hipLaunchKernelGGL(fill_u16_kernel, dim3(nchunks(V)), dim3(RB), 0, ctx->stream, out, V, kNegInf);
  hipLaunchKernelGGL(top_k_keep_kernel, dim3((top_k + 255) / 256), dim3(256), 0, ctx->stream, lp,
                     order, top_k, out);
  ORN_LAUNCH_CHECK("top-k kernels");
  return ORNITH_OK;
}

int categorical_impl(ornith_ctx* ctx, const bf16_t* lp, int V, double temp, uint32_t bits,
                     uint32_t* token, ScratchCursor& sc) {
  const int nch = nchunks(V);
  float* x = sc.take<float>(V);
  float* pmax = sc.take<float>(nch);
  uint32_t* fl = sc.take<uint32_t>(2);
  ScanBufs b = scan_bufs(sc, V);
  const float s32 = (float)(1.0 / temp);
  uint32_t u;
  memcpy(&u, &s32, 4);
  u = (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u;
  float scale;
  memcpy(&scale, &u, 4);
  hipLaunchKernelGGL(cat_scale_kernel, dim3(nch), dim3(RB), 0, ctx->stream, lp, V, scale, x, pmax);
  hipLaunchKernelGGL(cat_weights_scan_kernel, dim3(nch), dim3(RB), 0, ctx->stream, x, V, pmax, nch, b.vloc,
                     b.segoff, b.chunk_tot, fl);
  hipLaunchKernelGGL(cat_search_kernel, dim3(nch), dim3(RB), 0, ctx->stream, b.vloc, b.segoff,
                     b.chunk_tot, x, V, nch, bits, fl, false);
  hipLaunchKernelGGL(cat_pick_kernel, dim3(1), dim3(1), 0, ctx->stream, fl, token);
  ORN_LAUNCH_CHECK("categorical kernels");
  return ORNITH_OK;
}

// ---- distributions as weights, speculative sampling ----------------------------------------
// w[n] = the row total of w[0..n) in the scan's order
__global__ __launch_bounds__(RB) void weights_total_kernel(const float* chunk_tot, int nch, float* w, int n) {
  float base, total;
  chunk_base<false>(chunk_tot, nch, base, total);
  if (threadIdx.x == 0) w[n] = total;
}

// the categorical weights of filtered log-probabilities: w[0..V) and their total in w[V]
int weights_impl(ornith_ctx* ctx, const bf16_t* lp, int V, double temp, float* w, ScratchCursor& sc) {
  const int nch = nchunks(V);
  float* pmax = sc.take<float>(nch);
  ScanBufs b = scan_bufs(sc, V);
  const float s32 = (float)(1.0 / temp);
  uint32_t u;
  memcpy(&u, &s32, 4);
  u = (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u;
  float scale;
  memcpy(&scale, &u, 4);
  hipLaunchKernelGGL(cat_scale_kernel, dim3(nch), dim3(RB), 0, ctx->stream, lp, V, scale, w, pmax);
  hipLaunchKernelGGL(cat_weights_scan_kernel, dim3(nch), dim3(RB), 0, ctx->stream, w, V, pmax, nch, b.vloc,
                     b.segoff, b.chunk_tot, (uint32_t*)nullptr);
  hipLaunchKernelGGL(weights_total_kernel, dim3(1), dim3(RB), 0, ctx->stream, b.chunk_tot, nch, w, V);
  ORN_LAUNCH_CHECK("sampler weights kernels");
  return ORNITH_OK;
}

// scan + search of one weight vector; leaves (first, last[, total bits]) in fl
int search_weights(ornith_ctx* ctx, const float* w, int V, uint32_t bits, uint32_t* fl, bool store_total,
                   ScratchCursor& sc) {
  const int nch = nchunks(V);
  ScanBufs b = scan_bufs(sc, V);
  hipLaunchKernelGGL(scan_local_kernel<false>, dim3(nch), dim3(RB), 0, ctx->stream, w, V, b.vloc, b.segoff,
                     b.chunk_tot);
  hipLaunchKernelGGL(cat_init_kernel, dim3(1), dim3(1), 0, ctx->stream, fl);
  hipLaunchKernelGGL(cat_search_kernel, dim3(nch), dim3(RB), 0, ctx->stream, b.vloc, b.segoff, b.chunk_tot, w, V,
                     nch, bits, fl, store_total);
  return ORNITH_OK;
}

__global__ void spec_zero_kernel(float* w, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) w[i] = 0.f;
}
// full[ids[l]] = local[l]; full[V] = local[n]
__global__ void spec_scatter_kernel(const float* local, const uint32_t* ids, int n, int V, float* full) {
  const int l = blockIdx.x * blockDim.x + threadIdx.x;
  if (l < n) {
    const uint32_t id = ids[l];
    if (id < (uint32_t)V) full[id] = local[l];
  }
  if (l == 0) full[V] = local[n];
}
// accept iff u * q(x) < p(x)
__global__ void spec_accept_kernel(const float* wp, const float* wq, int V, const uint32_t* x_ptr, uint32_t bits,
                                   uint32_t* accept) {
  const uint32_t x = min(x_ptr[0], (uint32_t)(V - 1));
  const float px = wp[x] / wp[V], qx = wq[x] / wq[V];
  float u = (float)bits / 4294967296.0f;
  const float upper = __uint_as_float(0x3f7fffffu);
  u = u < upper ? u : upper;
  u = 1.0f * u + 0.0f;
  u = u * 1.0f;
  accept[0] = u * qx < px ? 1u : 0u;
}
// r = max(0, p - q)
__global__ void spec_residual_kernel(const float* wp, const float* wq, int V, float* r) {
  const int y = blockIdx.x * blockDim.x + threadIdx.x;
  if (y < V) {
    const float d = wp[y] / wp[V] - wq[y] / wq[V];
    r[y] = d > 0.f ? d : 0.f;
  }
}
// the residual's draw if it has any mass, the target's otherwise
__global__ void spec_pick_kernel(const uint32_t* fl_r, const uint32_t* fl_p, uint32_t* token) {
  const uint32_t* fl = __uint_as_float(fl_r[2]) > 0.f ? fl_r : fl_p;
  token[0] = fl[0] != 0xffffffffu ? fl[0] : fl[1];
}

size_t sampler_workspace(int V) {
  // two bf16 rows + top-p (S, sp, scan, sort) + top-k / draw reuse the same space
  return (size_t)V * (2 * 2 + 4 + 4 + 4) + scan_workspace(V) + argsort_workspace(V) +
         (size_t)nchunks(V) * 16 + 64 * 256;
}

}  // namespace

struct ornith_top_sampler {
  ornith_ctx* ctx;
  double temp, top_p;
  int top_k, vocab;
  uint32_t key[2];
  int rng = ORNITH_RNG_THREEFRY;
  uint64_t seed = 0, philox_n = 0;
};

namespace {
// the filtered log-probabilities of one row (log-softmax, top-p, top-k): returns the buffer
// holding them (one of two taken from sc); sc.off is left past both rows
int filtered_logprobs(ornith_top_sampler* s, const void* d_logits_row, int V, ScratchCursor& sc,
                      const bf16_t** out) {
  ornith_ctx* ctx = s->ctx;
  bf16_t* a = sc.take<bf16_t>(V);
  bf16_t* b = sc.take<bf16_t>(V);
  bf16_t* lse = sc.take<bf16_t>(1);
  uint32_t* tok_tmp = sc.take<uint32_t>(1);
  const size_t mark = sc.off;
  // lse through the greedy selector's kernels (its token output is not used)
  int rc = ornith_greedy_rows_ws(ctx, d_logits_row, 1, V, tok_tmp, lse, sc);
  if (rc) return rc;
  hipLaunchKernelGGL(logprob_kernel, dim3(nchunks(V)), dim3(RB), 0, ctx->stream,
                     (const bf16_t*)d_logits_row, lse, V, a);
  bf16_t *cur = a, *nxt = b;
  if (s->top_p > 0.0 && s->top_p < 1.0) {
    sc.off = mark;
    rc = top_p_impl(ctx, cur, V, s->top_p, nxt, sc);
    if (rc) return rc;
    std::swap(cur, nxt);
  }
  if (s->top_k > 0 && s->top_k < V) {
    sc.off = mark;
    rc = top_k_impl(ctx, cur, V, s->top_k, nxt, sc);
    if (rc) return rc;
    std::swap(cur, nxt);
  }
  sc.off = mark;
  *out = cur;
  return ORNITH_OK;
}
}  // namespace

extern "C" {

void ornith_random_key(uint64_t seed, uint32_t key_out[2]) {
  key_out[0] = (uint32_t)(seed >> 32);
  key_out[1] = (uint32_t)seed;
}

int ornith_random_bits(const uint32_t key[2], int n, uint32_t* out) {
  ORN_REQUIRE(key && out && n >= 1, "random_bits: bad argument");
  const int half = n / 2, odd = n & 1, gy = half + odd;
  for (int t = 0; t < gy; ++t) {
    const bool drop_last = odd && t == half;
    uint32_t h[2];
    threefry2x32(key, (uint32_t)t, drop_last ? 0u : (uint32_t)(t + gy), h);
    out[t] = h[0];
    if (!drop_last) out[t + gy] = h[1];
  }
  return ORNITH_OK;
}

int ornith_random_split(uint32_t key_state[2], uint32_t sub_out[2]) {
  ORN_REQUIRE(key_state && sub_out, "random_split: null argument");
  uint32_t b[4];
  ornith_random_bits(key_state, 4, b);
  key_state[0] = b[0];
  key_state[1] = b[1];
  sub_out[0] = b[2];
  sub_out[1] = b[3];
  return ORNITH_OK;
}

int ornith_argsort_bf16(ornith_ctx* ctx, const void* d_x, int n, int negate, uint32_t* d_idx_out) {
  ORN_REQUIRE(ctx && d_x && d_idx_out, "argsort: null argument");
  ORN_REQUIRE(n >= 1 && n <= (1 << 24), "argsort: n=%d", n);
  void* base = nullptr;
  int rc = ornith_scratch(ctx, argsort_workspace(n), &base);
  if (rc) return rc;
  ScratchCursor sc(base);
  return argsort_impl(ctx, (const bf16_t*)d_x, n, negate, d_idx_out, sc);
}

int ornith_cumsum(ornith_ctx* ctx, const void* d_x, int dtype, int n, void* d_out) {
  ORN_REQUIRE(ctx && d_x && d_out, "cumsum: null argument");
  ORN_REQUIRE(n >= 1 && (dtype == ORNITH_F32 || dtype == ORNITH_BF16), "cumsum: n=%d dtype=%d", n, dtype);
  void* base = nullptr;
  int rc = ornith_scratch(ctx, scan_workspace(n) + (size_t)n * 4 + 256, &base);
  if (rc) return rc;
  ScratchCursor sc(base);
  ScanBufs b = scan_bufs(sc, n);
  const int nch = nchunks(n);
  if (dtype == ORNITH_BF16) {
    // widen once; the scan itself rounds every add to bf16
    float* f = sc.take<float>(n);
    hipLaunchKernelGGL(widen_bf16_kernel, dim3(nch), dim3(RB), 0, ctx->stream, (const bf16_t*)d_x, n, f);
    hipLaunchKernelGGL(scan_local_kernel<true>, dim3(nch), dim3(RB), 0, ctx->stream, f, n, b.vloc,
                       b.segoff, b.chunk_tot);
    hipLaunchKernelGGL(scan_out_kernel<true>, dim3(nch), dim3(RB), 0, ctx->stream, b.vloc, b.segoff,
                       b.chunk_tot, n, nch, d_out);
  } else {
    hipLaunchKernelGGL(scan_local_kernel<false>, dim3(nch), dim3(RB), 0, ctx->stream,
                       (const float*)d_x, n, b.vloc, b.segoff, b.chunk_tot);
    hipLaunchKernelGGL(scan_out_kernel<false>, dim3(nch), dim3(RB), 0, ctx->stream, b.vloc, b.segoff,
                       b.chunk_tot, n, nch, d_out);
  }
  ORN_LAUNCH_CHECK("cumsum kernels");
  return ORNITH_OK;
}

int ornith_apply_top_p(ornith_ctx* ctx, const void* d_logprobs, int V, double top_p, void* d_out) {
  ORN_REQUIRE(ctx && d_logprobs && d_out && d_out != d_logprobs, "apply_top_p: bad argument");
  ORN_REQUIRE(V >= 1 && top_p > 0.0 && top_p < 1.0, "apply_top_p: V=%d top_p=%g", V, top_p);
  void* base = nullptr;
  int rc = ornith_scratch(ctx, sampler_workspace(V), &base);
  if (rc) return rc;
  ScratchCursor sc(base);
  return top_p_impl(ctx, (const bf16_t*)d_logprobs, V, top_p, (bf16_t*)d_out, sc);
}

int ornith_apply_top_k(ornith_ctx* ctx, const void* d_logprobs, int V, int top_k, void* d_out) {
  ORN_REQUIRE(ctx && d_logprobs && d_out && d_out != d_logprobs, "apply_top_k: bad argument");
  ORN_REQUIRE(V >= 2 && top_k > 0 && top_k < V, "apply_top_k: top_k=%d must be in (0, %d)", top_k, V);
  void* base = nullptr;
  int rc = ornith_scratch(ctx, sampler_workspace(V), &base);
  if (rc) return rc;
  ScratchCursor sc(base);
  return top_k_impl(ctx, (const bf16_t*)d_logprobs, V, top_k, (bf16_t*)d_out, sc);
}

int ornith_categorical(ornith_ctx* ctx, const void* d_logprobs, int V, double temp, uint32_t raw_bits,
                       uint32_t* d_token_out) {
  ORN_REQUIRE(ctx && d_logprobs && d_token_out, "categorical: null argument");
  ORN_REQUIRE(V >= 1 && temp > 0.0, "categorical: V=%d temp=%g", V, temp);
  void* base = nullptr;
  int rc = ornith_scratch(ctx, sampler_workspace(V), &base);
  if (rc) return rc;
  ScratchCursor sc(base);
  return categorical_impl(ctx, (const bf16_t*)d_logprobs, V, temp, raw_bits, d_token_out, sc);
}

int ornith_top_sampler_create(ornith_ctx* ctx, double temp, double top_p, int top_k, uint64_t seed,
                              int vocab, ornith_top_sampler** out) {
  ORN_REQUIRE(ctx && out, "top_sampler_create: null argument");
  ORN_REQUIRE(temp > 0.0 && vocab >= 2 && top_k >= 0 && top_k < vocab,
              "top_sampler_create: temp=%g top_k=%d vocab=%d", temp, top_k, vocab);
  void* base = nullptr;
  int rc = ornith_scratch(ctx, sampler_workspace(vocab), &base);  // sized once, here
  if (rc) return rc;
  auto* s = new ornith_top_sampler{ctx, temp, top_p, top_k, vocab, {0, 0}};
  ornith_random_key(seed, s->key);
  s->seed = seed;
  *out = s;
  return ORNITH_OK;
}

int ornith_top_sampler_destroy(ornith_top_sampler* s) {
  delete s;
  return ORNITH_OK;
}

int ornith_top_sampler_set_rng(ornith_top_sampler* s, int rng) {
  ORN_REQUIRE(s, "top_sampler_set_rng: null sampler");
  ORN_REQUIRE(rng == ORNITH_RNG_THREEFRY || rng == ORNITH_RNG_PHILOX, "top_sampler_set_rng: unknown generator %d", rng);
  s->rng = rng;
  return ORNITH_OK;
}

int ornith_top_sampler_next_bits(ornith_top_sampler* s, uint32_t* bits_out) {
  ORN_REQUIRE(s && bits_out, "top_sampler_next_bits: null argument");
  if (s->rng == ORNITH_RNG_PHILOX) {
    const uint64_t n = s->philox_n++;
    const uint32_t ctr[4] = {(uint32_t)n, (uint32_t)(n >> 32), 0u, 0u};
    const uint32_t key[2] = {(uint32_t)s->seed, (uint32_t)(s->seed >> 32)};
    uint32_t out[4];
    philox4x32_10(ctr, key, out);
    *bits_out = out[0];
    return ORNITH_OK;
  }
  uint32_t sub[2];
  ornith_random_split(s->key, sub);
  return ornith_random_bits(sub, 1, bits_out);
}

void ornith_philox4x32_10(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4]) {
  philox4x32_10(counter, key, out);
}

int ornith_top_sampler_sample(ornith_top_sampler* s, const void* d_logits_row, uint32_t* d_token_out) {
  ORN_REQUIRE(s && d_logits_row && d_token_out, "top_sampler_sample: null argument");
  ornith_ctx* ctx = s->ctx;
  const int V = s->vocab;
  void* base = nullptr;
  int rc = ornith_scratch(ctx, sampler_workspace(V), &base);
  if (rc) return rc;
  ScratchCursor sc(base);
  const bf16_t* cur = nullptr;
  rc = filtered_logprobs(s, d_logits_row, V, sc, &cur);
  if (rc) return rc;
  uint32_t raw;
  rc = ornith_top_sampler_next_bits(s, &raw);
  if (rc) return rc;
  return categorical_impl(ctx, cur, V, s->temp, raw, d_token_out, sc);
}

int ornith_sampler_weights(ornith_top_sampler* s, const void* d_logits_row, int V, float* d_w) {
  ORN_REQUIRE(s && d_logits_row && d_w, "sampler_weights: null argument");
  ORN_REQUIRE(V >= 2 && V <= s->vocab, "sampler_weights: V=%d outside the sampler's vocabulary of %d", V, s->vocab);
  ornith_ctx* ctx = s->ctx;
  void* base = nullptr;
  int rc = ornith_scratch(ctx, sampler_workspace(s->vocab), &base);
  if (rc) return rc;
  ScratchCursor sc(base);
  const bf16_t* cur = nullptr;
  rc = filtered_logprobs(s, d_logits_row, V, sc, &cur);
  if (rc) return rc;
  return weights_impl(ctx, cur, V, s->temp, d_w, sc);
}

int ornith_draw_weights(ornith_ctx* ctx, const float* d_w, int V, uint32_t raw_bits, uint32_t* d_token_out) {
  ORN_REQUIRE(ctx && d_w && d_token_out && V >= 1, "draw_weights: bad argument");
  void* base = nullptr;
  int rc = ornith_scratch(ctx, scan_workspace(V) + 1024, &base);
  if (rc) return rc;
  ScratchCursor sc(base);
  uint32_t* fl = sc.take<uint32_t>(4);
  rc = search_weights(ctx, d_w, V, raw_bits, fl, false, sc);
  if (rc) return rc;
  hipLaunchKernelGGL(cat_pick_kernel, dim3(1), dim3(1), 0, ctx->stream, fl, d_token_out);
  ORN_LAUNCH_CHECK("draw_weights kernels");
  return ORNITH_OK;
}

int ornith_spec_scatter(ornith_ctx* ctx, const float* d_w_local, const uint32_t* d_ids, int n, int V,
                        float* d_w_full) {
  ORN_REQUIRE(ctx && d_w_local && d_ids && d_w_full && n >= 1 && n <= V, "spec_scatter: bad argument");
  hipLaunchKernelGGL(spec_zero_kernel, dim3((V + 255) / 256), dim3(256), 0, ctx->stream, d_w_full, V);
  hipLaunchKernelGGL(spec_scatter_kernel, dim3((n + 255) / 256), dim3(256), 0, ctx->stream, d_w_local, d_ids, n, V,
                     d_w_full);
  ORN_LAUNCH_CHECK("spec_scatter kernels");
  return ORNITH_OK;
}

int ornith_spec_accept(ornith_ctx* ctx, const float* d_wp, const float* d_wq, int V, const uint32_t* d_x,
                       uint32_t raw_bits, uint32_t* d_accept_out) {
  ORN_REQUIRE(ctx && d_wp && d_wq && d_x && d_accept_out && V >= 1, "spec_accept: bad argument");
  hipLaunchKernelGGL(spec_accept_kernel, dim3(1), dim3(1), 0, ctx->stream, d_wp, d_wq, V, d_x, raw_bits,
                     d_accept_out);
  ORN_LAUNCH_CHECK("spec_accept_kernel");
  return ORNITH_OK;
}

int ornith_spec_resample(ornith_ctx* ctx, const float* d_wp, const float* d_wq, int V, uint32_t raw_bits,
                         uint32_t* d_token_out) {
  ORN_REQUIRE(ctx && d_wp && d_wq && d_token_out && V >= 1, "spec_resample: bad argument");
  void* base = nullptr;
  int rc = ornith_scratch(ctx, (size_t)V * 4 + 2 * scan_workspace(V) + 2048, &base);
  if (rc) return rc;
  ScratchCursor sc(base);
  float* r = sc.take<float>(V);
  uint32_t* fl_r = sc.take<uint32_t>(4);
  uint32_t* fl_p = sc.take<uint32_t>(4);
  hipLaunchKernelGGL(spec_residual_kernel, dim3((V + 255) / 256), dim3(256), 0, ctx->stream, d_wp, d_wq, V, r);
  rc = search_weights(ctx, r, V, raw_bits, fl_r, true, sc);
  if (rc) return rc;
  rc = search_weights(ctx, d_wp, V, raw_bits, fl_p, false, sc);
  if (rc) return rc;
  hipLaunchKernelGGL(spec_pick_kernel, dim3(1), dim3(1), 0, ctx->stream, fl_r, fl_p, d_token_out);
  ORN_LAUNCH_CHECK("spec_resample kernels");
  return ORNITH_OK;
}

}  // extern "C"
