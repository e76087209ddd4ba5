// Greedy token selection over the vocabulary.
//
// Replaces ops::sample::{greedy_token, greedy_argmax_into, logsumexp_last_axis,
// argmax_last_axis_into} (/root/reference/src/ops/sample.rs:1-19,37-147,174-191):
// target rows take argmax(logits - logsumexp(logits)) with the subtraction done in
// bf16, draft rows take argmax of the raw logits; ties go to the lowest index
// (vendored arg_reduce.metal:54-64).
//
// The vocabulary is cut into chunks of 1024, one workgroup each: pass 1 leaves
// (max, sum exp) per chunk, pass 2 merges them in ascending chunk order into the
// row's logsumexp and finds each chunk's best (value, lowest index), pass 3 picks
// the winner. All of it is wavefront shuffles plus one LDS hop.
#include "dmath.h"
#include "rt.h"

#include <mutex>

namespace {

constexpr int CH = 1024;

// ---- the no-allocation variant's scratch --------------------------------------------
// ornith_greedy_rows_noalloc keeps its per-chunk partials (maximum, sum of exponentials,
// best value, best index) in this fixed device array instead of the context's grow-only
// scratch block, so the call never reaches hipMalloc. Limits: 8 rows of at most 262144
// logits -> 4 arrays x 8 rows x 256 chunks x 4 bytes = 32 KiB, held by every GPU the
// library runs on until the process ends.
constexpr int NA_MAX_ROWS = 8;
constexpr int NA_MAX_V = 262144;
constexpr int NA_MAX_NCH = NA_MAX_V / CH;
constexpr size_t NA_ARRAY_BYTES = (size_t)NA_MAX_ROWS * NA_MAX_NCH * 4;  // a multiple of 256
constexpr size_t NA_BYTES = 4 * NA_ARRAY_BYTES;
static __device__ __align__(256) unsigned char scratch[NA_BYTES];

// `scratch` names a host-side stand-in here; the array's device address differs per GPU
// and is asked for once per device (ornith_sample_init_device, under the lock) and kept in this
// table; a context carries its device's address, so no call reads the table afterwards.
constexpr int NA_MAX_DEVICES = 64;
void* g_scratch_ptr[NA_MAX_DEVICES] = {};
std::mutex g_scratch_mu;

__global__ __launch_bounds__(CH) void lse_chunk_kernel(const bf16_t* logits, int V, int nch,
                                                       float* mc, float* lc) {
  const int c = blockIdx.x, r = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  __shared__ float red[16];
  const int i = c * CH + tid;
  const bool ok = i < V;
  const float x = ok ? dm_bf2f(logits[(size_t)r * V + i]) : -DM_INF;
  float m = dm_wave_max<64>(x);
  if (lane == 0) red[wave] = m;
  __syncthreads();
  m = red[0];
#pragma unroll
  for (int w = 1; w < 16; ++w) m = red[w] > m ? red[w] : m;
  __syncthreads();
  const float e = ok ? dm_exp(x - m) : 0.f;
  const float ws = dm_wave_sum<64>(e);
  if (lane == 0) red[wave] = ws;
  __syncthreads();
  if (tid == 0) {
    float l = red[0];
#pragma unroll
    for (int w = 1; w < 16; ++w) l = l + red[w];
    mc[(size_t)r * nch + c] = m;
    lc[(size_t)r * nch + c] = l;
  }
}

// (value, index) max with lowest index on ties
__device__ __forceinline__ void best_merge(float& v, int& i, float ov, int oi) {
  if (ov > v || (ov == v && oi < i)) {
    v = ov;
    i = oi;
  }
}

// pass 2: per chunk. USE_LSE: value = bf16(x - lse), else raw x.
template <bool USE_LSE>
__global__ __launch_bounds__(CH) void argmax_chunk_kernel(const bf16_t* logits, int V, int nch,
                                                          const float* mc, const float* lc,
                                                          float* bv, int* bi, bf16_t* lse_out) {
  const int c = blockIdx.x, r = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  __shared__ float sv[16];
  __shared__ int si[16];
  __shared__ float s_lse;
  float lse = 0.f;
  if constexpr (USE_LSE) {
    // every workgroup repeats the short merge: cheaper than another launch
    __shared__ float smax[16];
    float m = -DM_INF;
    for (int k = tid; k < nch; k += CH) m = mc[(size_t)r * nch + k] > m ? mc[(size_t)r * nch + k] : m;
    m = dm_wave_max<64>(m);
    if (lane == 0) smax[wave] = m;
    __syncthreads();
    float M = smax[0];
#pragma unroll
    for (int w = 1; w < 16; ++w) M = smax[w] > M ? smax[w] : M;
    // the chunk terms are independent and computed by all threads; only the fma chain
    // over them (ascending chunk order) is sequential
    __shared__ float s_l[CH], s_e[CH];
    float L = 0.f;
    for (int k0 = 0; k0 < nch; k0 += CH) {
      const int k = k0 + tid;
      if (k < nch) {
        s_l[tid] = lc[(size_t)r * nch + k];
        s_e[tid] = dm_exp(mc[(size_t)r * nch + k] - M);
      }
      __syncthreads();
      if (tid == 0) {
        const int n = min(CH, nch - k0);
        for (int q = 0; q < n; ++q) L = dm_fma(s_l[q], s_e[q], L);
      }
      __syncthreads();
    }
    if (tid == 0) {
      s_lse = dm_rb(dm_log(L) + M);
      if (c == 0 && lse_out) lse_out[r] = dm_f2bf(s_lse);
    }
    __syncthreads();
    lse = s_lse;
  }
  const int i = c * CH + tid;
  float v = -DM_INF;
  int idx = 0x7fffffff;
  if (i < V) {
    const float x = dm_bf2f(logits[(size_t)r * V + i]);
    v = USE_LSE ? dm_rb(x - lse) : x;
    idx = i;
    if (v != v) v = -DM_INF;  // NaN never wins
  }
#pragma unroll
  for (int s = 32; s >= 1; s >>= 1) {
    const float ov = __shfl_xor(v, s, 64);
    const int oi = __shfl_xor(idx, s, 64);
    best_merge(v, idx, ov, oi);
  }
  if (lane == 0) {
    sv[wave] = v;
    si[wave] = idx;
  }
  __syncthreads();
  if (tid == 0) {
    for (int w = 1; w < 16; ++w) best_merge(v, idx, sv[w], si[w]);
    bv[(size_t)r * nch + c] = v;
    bi[(size_t)r * nch + c] = idx;
  }
}

// pass 3: one wavefront per row over the chunk winners
// With id_map the winner is stored as id_map[winner]: a pruned head's row number turned into
// the vocabulary id (FrSpec::map_id, /root/reference/src/frspec.rs:134-142) without a launch.
__global__ __launch_bounds__(64) void argmax_final_kernel(const float* bv, const int* bi, int nch,
                                                          int V, uint32_t* out, const uint32_t* id_map) {
  const int r = blockIdx.x, lane = threadIdx.x;
  float v = -DM_INF;
  int idx = 0x7fffffff;
  for (int k = lane; k < nch; k += 64) best_merge(v, idx, bv[(size_t)r * nch + k], bi[(size_t)r * nch + k]);
#pragma unroll
  for (int s = 32; s >= 1; s >>= 1) {
    const float ov = __shfl_xor(v, s, 64);
    const int oi = __shfl_xor(idx, s, 64);
    best_merge(v, idx, ov, oi);
  }
  if (lane == 0) {
    const uint32_t t = (idx >= 0 && idx < V) ? (uint32_t)idx : 0u;
    out[r] = id_map ? id_map[t] : t;
  }
}

int run(ornith_ctx* ctx, const void* d_logits, int rows, int V, uint32_t* d_tokens, void* d_lse,
        bool use_lse, const char* who, ScratchCursor* ws = nullptr, const uint32_t* d_id_map = nullptr) {
  ORN_REQUIRE(ctx && d_logits && d_tokens, "%s: null argument", who);
  ORN_REQUIRE(rows >= 1 && rows <= 65535 && V >= 1, "%s: rows=%d V=%d", who, rows, V);
  const int nch = (V + CH - 1) / CH;
  void* base = nullptr;
  if (!ws) {
    int rc = ornith_scratch(ctx, (size_t)rows * nch * 16 + 2048, &base);
    if (rc) return rc;
  }
  ScratchCursor own(base);
  ScratchCursor& sc = ws ? *ws : own;
  float* mc = sc.take<float>((size_t)rows * nch);
  float* lc = sc.take<float>((size_t)rows * nch);
  float* bv = sc.take<float>((size_t)rows * nch);
  int* bi = sc.take<int>((size_t)rows * nch);
  const bf16_t* lg = (const bf16_t*)d_logits;
  if (use_lse) {
    hipLaunchKernelGGL(lse_chunk_kernel, dim3(nch, rows), dim3(CH), 0, ctx->stream, lg, V, nch, mc, lc);
    ORN_LAUNCH_CHECK("lse_chunk_kernel");
    hipLaunchKernelGGL(argmax_chunk_kernel<true>, dim3(nch, rows), dim3(CH), 0, ctx->stream, lg, V,
                       nch, mc, lc, bv, bi, (bf16_t*)d_lse);
  } else {
    hipLaunchKernelGGL(argmax_chunk_kernel<false>, dim3(nch, rows), dim3(CH), 0, ctx->stream, lg, V,
                       nch, mc, lc, bv, bi, (bf16_t*)nullptr);
  }
  ORN_LAUNCH_CHECK("argmax_chunk_kernel");
  hipLaunchKernelGGL(argmax_final_kernel, dim3(rows), dim3(64), 0, ctx->stream, bv, bi, nch, V,
                     d_tokens, d_id_map);
  ORN_LAUNCH_CHECK("argmax_final_kernel");
  return ORNITH_OK;
}

}  // namespace

// Called by ornith_ctx_create with `device` current: resolves this GPU's copy of `scratch`.
int ornith_sample_init_device(int device, void** ptr_out) {
  ORN_REQUIRE(device >= 0 && device < NA_MAX_DEVICES, "device %d is beyond the %d this library tracks", device,
              NA_MAX_DEVICES);
  ORN_REQUIRE(ptr_out, "sample_init_device: null argument");
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[device]) {
    void* ptr = nullptr;
    ORN_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    ORN_REQUIRE(ptr != nullptr, "hipGetSymbolAddress returned a null address for the fixed scratch array");
    g_scratch_ptr[device] = ptr;
  }
  *ptr_out = g_scratch_ptr[device];
  return ORNITH_OK;
}

int ornith_greedy_rows_ws(ornith_ctx* ctx, const void* d_logits, int rows, int V, uint32_t* d_tokens,
                          void* d_lse, ScratchCursor& sc) {
  return run(ctx, d_logits, rows, V, d_tokens, d_lse, true, "greedy_rows", &sc);
}

// argmax over the V rows of a pruned head, stored as vocabulary ids: d_id_map holds V entries
int argmax_rows_mapped(ornith_ctx* ctx, const void* d_logits, int rows, int V, const uint32_t* d_id_map,
                       uint32_t* d_out) {
  ORN_REQUIRE(d_id_map, "argmax_rows_mapped: null id map");
  return run(ctx, d_logits, rows, V, d_out, nullptr, false, "argmax_rows", nullptr, d_id_map);
}

extern "C" {

int ornith_greedy_rows(ornith_ctx* ctx, const void* d_logits, int rows, int V, uint32_t* d_tokens,
                       void* d_lse) {
  return run(ctx, d_logits, rows, V, d_tokens, d_lse, true, "greedy_rows");
}

int ornith_argmax_rows(ornith_ctx* ctx, const void* d_logits, int rows, int V, uint32_t* d_out) {
  return run(ctx, d_logits, rows, V, d_out, nullptr, false, "argmax_rows");
}

int ornith_greedy_rows_noalloc(ornith_ctx* ctx, const void* d_logits, int rows, int V,
                               uint32_t* d_tokens, void* d_lse) {
  ORN_REQUIRE(ctx && d_logits && d_tokens, "greedy_rows_noalloc: null argument");
  ORN_REQUIRE(rows >= 1 && rows <= NA_MAX_ROWS,
              "greedy_rows_noalloc: %d rows; the fixed scratch array holds at most %d (use ornith_greedy_rows)",
              rows, NA_MAX_ROWS);
  ORN_REQUIRE(V >= 1 && V <= NA_MAX_V,
              "greedy_rows_noalloc: %d logits a row; the fixed scratch array holds at most %d (use "
              "ornith_greedy_rows)", V, NA_MAX_V);
  void* ptr = ctx->na_scratch;  // resolved for this context's device when the context was made
  ORN_REQUIRE(ptr != nullptr, "greedy_rows_noalloc: the fixed scratch array of device %d was never resolved",
              ctx->device);
  // every partial is written by the pass before the one that reads it, for exactly the
  // rows x chunks of this call, so nothing left by an earlier call is ever read
  ScratchCursor sc(ptr);
  return run(ctx, d_logits, rows, V, d_tokens, d_lse, true, "greedy_rows_noalloc", &sc);
}

}  // extern "C"
