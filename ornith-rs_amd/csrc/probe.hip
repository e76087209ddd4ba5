// Machine probes behind `bench.py --ceiling`: what a launch costs when it does nothing, what a
// launch of the expert kernel's shape costs when it only streams its bytes, what a long read
// sustains, where workgroups land, and how long a word written by one workgroup takes to be
// seen by another. They price the decode kernels against the machine instead of against the
// 8 TB/s figure alone. No reference counterpart; nothing in the decode path calls them.
#include "rt.h"

namespace {

__global__ void probe_empty_kernel() {}

struct ProbeArgs {
  const void* p[12];
  int n[8];
};
// the same nothing, with an argument block of the expert kernel's size (never read)
__global__ void probe_empty_args_kernel(ProbeArgs a) {
  if (threadIdx.x == 4095 && a.n[0] == 0x7fffffff) *(int*)a.p[0] = 1;
}

// Every thread reads `per_thread` 16-byte pieces; a wavefront's piece i is 1 KB contiguous and
// its pieces are `stride` bytes apart (stride = 1024: one contiguous run a wavefront). The
// values are folded into a word that is stored only if it has an impossible value.
__global__ __launch_bounds__(256) void probe_stream_kernel(const uint4* __restrict__ src, int per_thread,
                                                           size_t stride16, uint32_t* sink) {
  const size_t wave = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const uint4* p = src + wave * (size_t)per_thread * stride16 + (threadIdx.x & 63);
  uint4 v[16];
#pragma unroll
  for (int i = 0; i < 16; ++i)
    if (i < per_thread) v[i] = p[(size_t)i * stride16];
  uint32_t acc = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i)
    if (i < per_thread) acc ^= v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
  if (acc == 0x13579bdfu) *sink = acc;
}

// grid-stride read of the whole buffer, 16 bytes a lane, four loads in flight a thread
__global__ __launch_bounds__(256) void probe_read_kernel(const uint4* __restrict__ src, size_t n16, uint32_t* sink) {
  const size_t step = (size_t)gridDim.x * 256;
  uint32_t acc = 0;
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  for (; i + 3 * step < n16; i += 4 * step) {
    const uint4 a = src[i], b = src[i + step], c = src[i + 2 * step], d = src[i + 3 * step];
    acc ^= a.x ^ b.y ^ c.z ^ d.w;
  }
  for (; i < n16; i += step) acc ^= src[i].x;
  if (acc == 0x13579bdfu) *sink = acc;
}

__device__ __forceinline__ uint32_t probe_xcc_id() {
  uint32_t v;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v));
  return v & 0xf;
}

__global__ void probe_xcc_kernel(uint32_t* out) {
  if (threadIdx.x == 0) out[blockIdx.x] = probe_xcc_id();
}

// Workgroup `prod` waits 4 us and writes one word; workgroup `cons` polls it. out[0] = the
// 100 MHz clock at the store, out[1] = at the observation (0: the bounded poll ran out),
// out[2], out[3] = the two workgroups' XCC ids.
// mode 0: plain store, agent-scope (sc1) load; 1: sc1 store, sc1 load; 2: plain store and plain
// load (the stale line in the consumer's L1 is never refreshed: expected to run out).
__global__ __launch_bounds__(64) void probe_handoff_kernel(uint32_t* flag, long long* out, int prod, int cons,
                                                           int mode, int max_polls) {
  const int wg = blockIdx.x;
  if ((wg != prod && wg != cons) || threadIdx.x != 0) return;
  uint32_t old;
  asm volatile("global_load_dword %0, %1, off\n\ts_waitcnt vmcnt(0)" : "=v"(old) : "v"(flag) : "memory");
  const long long t0 = wall_clock64();
  if (wg == prod) {
    while (wall_clock64() - t0 < 400) __builtin_amdgcn_s_sleep(8);
    out[0] = wall_clock64();
    if (mode == 1)
      asm volatile("global_store_dword %0, %1, off sc1" ::"v"(flag), "v"(old + 1) : "memory");
    else
      asm volatile("global_store_dword %0, %1, off" ::"v"(flag), "v"(old + 1) : "memory");
    out[2] = probe_xcc_id();
  } else {
    long long seen = 0;
    for (int i = 0; i < max_polls; ++i) {
      uint32_t v;
      if (mode == 2)
        asm volatile("global_load_dword %0, %1, off\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(flag) : "memory");
      else
        asm volatile("global_load_dword %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(flag) : "memory");
      if (v != old) {
        seen = wall_clock64();
        break;
      }
    }
    out[1] = seen;
    out[3] = probe_xcc_id();
  }
}

}  // namespace

extern "C" {

int ornith_probe_empty(ornith_ctx* ctx, int workgroups, int threads, int with_args, int launches) {
  ORN_REQUIRE(ctx && workgroups >= 1 && threads >= 1 && threads <= 1024 && launches >= 1, "probe_empty: bad argument");
  ProbeArgs a{};
  for (int i = 0; i < launches; ++i) {
    if (with_args)
      hipLaunchKernelGGL(probe_empty_args_kernel, dim3(workgroups), dim3(threads), 0, ctx->stream, a);
    else
      hipLaunchKernelGGL(probe_empty_kernel, dim3(workgroups), dim3(threads), 0, ctx->stream);
  }
  ORN_LAUNCH_CHECK("probe_empty_kernel");
  return ORNITH_OK;
}

// The same launches recorded into a graph and replayed as one submission: the device's own
// rate of taking one launch after another, with the host's enqueue cost out of the picture.
int ornith_probe_empty_graph(ornith_ctx* ctx, int workgroups, int threads, int with_args, int launches, float* ms_out) {
  ORN_REQUIRE(ctx && ms_out && workgroups >= 1 && threads >= 1 && threads <= 1024 && launches >= 1,
              "probe_empty_graph: bad argument");
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  ORN_HIP(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
  ProbeArgs a{};
  for (int i = 0; i < launches; ++i) {
    if (with_args)
      hipLaunchKernelGGL(probe_empty_args_kernel, dim3(workgroups), dim3(threads), 0, ctx->stream, a);
    else
      hipLaunchKernelGGL(probe_empty_kernel, dim3(workgroups), dim3(threads), 0, ctx->stream);
  }
  ORN_HIP(hipStreamEndCapture(ctx->stream, &graph));
  hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  if (e != hipSuccess) {
    (void)hipGraphDestroy(graph);
    return ornith_fail(ORNITH_ERR_HIP, "probe_empty_graph: hipGraphInstantiate failed: %s", hipGetErrorString(e));
  }
  int rc = ORNITH_OK;
  do {
    if ((e = hipGraphLaunch(exec, ctx->stream)) != hipSuccess) break;  // warm-up replay
    if ((e = hipStreamSynchronize(ctx->stream)) != hipSuccess) break;
    if ((e = hipEventRecord(ctx->ev0, ctx->stream)) != hipSuccess) break;
    if ((e = hipGraphLaunch(exec, ctx->stream)) != hipSuccess) break;
    if ((e = hipEventRecord(ctx->ev1, ctx->stream)) != hipSuccess) break;
    if ((e = hipEventSynchronize(ctx->ev1)) != hipSuccess) break;
    e = hipEventElapsedTime(ms_out, ctx->ev0, ctx->ev1);
  } while (0);
  if (e != hipSuccess) rc = ornith_fail(ORNITH_ERR_HIP, "probe_empty_graph: %s", hipGetErrorString(e));
  (void)hipGraphExecDestroy(exec);
  (void)hipGraphDestroy(graph);
  return rc;
}

int ornith_probe_stream(ornith_ctx* ctx, const void* d_src, size_t bytes, int workgroups, int per_thread,
                        size_t stride_bytes, void* d_sink, int launches) {
  ORN_REQUIRE(ctx && d_src && d_sink && workgroups >= 1 && per_thread >= 1 && per_thread <= 16 && launches >= 1,
              "probe_stream: bad argument");
  ORN_REQUIRE(stride_bytes >= 1024 && stride_bytes % 16 == 0, "probe_stream: stride of %zu bytes", stride_bytes);
  // one launch reads `span` bytes; launch i starts (i mod slots) spans into the buffer, so that
  // no launch finds its bytes in a cache when the buffer holds many spans
  const size_t span = ((((size_t)workgroups * 4 * per_thread - 1) * stride_bytes + 1024) + 4095) & ~size_t(4095);
  ORN_REQUIRE(span <= bytes, "probe_stream: a launch reads %zu bytes, the buffer has %zu", span, bytes);
  const size_t slots = bytes / span;
  for (int i = 0; i < launches; ++i)
    hipLaunchKernelGGL(probe_stream_kernel, dim3(workgroups), dim3(256), 0, ctx->stream,
                       (const uint4*)(static_cast<const char*>(d_src) + (i % slots) * span), per_thread,
                       stride_bytes / 16, (uint32_t*)d_sink);
  ORN_LAUNCH_CHECK("probe_stream_kernel");
  return ORNITH_OK;
}

int ornith_probe_read(ornith_ctx* ctx, const void* d_src, size_t bytes, void* d_sink) {
  ORN_REQUIRE(ctx && d_src && d_sink && bytes >= 16, "probe_read: bad argument");
  hipLaunchKernelGGL(probe_read_kernel, dim3(ctx->compute_units * 8), dim3(256), 0, ctx->stream,
                     (const uint4*)d_src, bytes / 16, (uint32_t*)d_sink);
  ORN_LAUNCH_CHECK("probe_read_kernel");
  return ORNITH_OK;
}

int ornith_probe_xcc(ornith_ctx* ctx, int workgroups, uint32_t* d_out) {
  ORN_REQUIRE(ctx && d_out && workgroups >= 1, "probe_xcc: bad argument");
  hipLaunchKernelGGL(probe_xcc_kernel, dim3(workgroups), dim3(64), 0, ctx->stream, d_out);
  ORN_LAUNCH_CHECK("probe_xcc_kernel");
  return ORNITH_OK;
}

int ornith_probe_handoff(ornith_ctx* ctx, void* d_flag, void* d_out4, int producer, int consumer, int mode) {
  ORN_REQUIRE(ctx && d_flag && d_out4 && producer >= 0 && consumer >= 0 && producer != consumer && mode >= 0 && mode <= 2,
              "probe_handoff: bad argument");
  const int n = (producer > consumer ? producer : consumer) + 1;
  ORN_HIP(hipMemsetAsync(d_out4, 0, 32, ctx->stream));
  hipLaunchKernelGGL(probe_handoff_kernel, dim3(n), dim3(64), 0, ctx->stream, (uint32_t*)d_flag, (long long*)d_out4,
                     producer, consumer, mode, 4000);
  ORN_LAUNCH_CHECK("probe_handoff_kernel");
  return ORNITH_OK;
}

}  // extern "C"
