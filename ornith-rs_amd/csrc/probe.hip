// Machine probes behind `bench.py --ceiling`: what a launch costs when it does nothing, what a
// launch of the expert kernel's shape costs when it only streams its bytes, what a long read
// sustains, where workgroups land, and how long a word written by one workgroup takes to be
// seen by another. They price the decode kernels against the machine instead of against the
// 8 TB/s figure alone; what single vector instructions and kernel arguments cost. No reference
// counterpart; nothing in the decode path calls them.
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

// ---- what one vector instruction costs: eight independent chains of the same instruction per
// thread, 256 threads a workgroup. The instruction is a template parameter so that the loop
// holds nothing else; the operands are harmless for every instruction in the list.
#define ORN_PROBE_OPS(X)                                                                \
  X(0, "v_fmac_f32 %0, %1, %2")                                                         \
  X(1, "v_mul_f32 %0, %1, %0")                                                          \
  X(2, "v_add_f32 %0, %1, %0")                                                          \
  X(3, "v_and_b32 %0, %2, %0")                                                          \
  X(4, "v_lshrrev_b32 %0, 1, %0")                                                       \
  X(5, "v_cvt_f32_ubyte1 %0, %0")                                                       \
  X(6, "v_cvt_f32_f16 %0, %0")                                                          \
  X(7, "v_and_or_b32 %0, %0, %2, %2")                                                   \
  X(8, "v_perm_b32 %0, %0, %2, %2")                                                     \
  X(9, "v_bfe_u32 %0, %0, 4, 4")                                                        \
  X(10, "v_pk_add_f16 %0, %0, %2")                                                      \
  X(11, "v_fma_mix_f32 %0, %1, %2, %0 op_sel:[0,0,0] op_sel_hi:[0,1,0]")                \
  X(12, "v_cvt_f32_ubyte1 %0, %2\n\tv_fmac_f32 %0, %1, %0")

template <int OP>
__global__ __launch_bounds__(256) void probe_valu_kernel(const float* xin, const uint32_t* pin, float* out, int iters) {
  const float x = xin[threadIdx.x & 3];
  const uint32_t p = pin[threadIdx.x & 3];
  float a0 = 0.f, a1 = 1.f, a2 = 2.f, a3 = 3.f, a4 = 4.f, a5 = 5.f, a6 = 6.f, a7 = 7.f;
  for (int i = 0; i < iters; ++i) {
#define X(N, S)                                          \
  if constexpr (OP == N) {                               \
    asm volatile(S : "+v"(a0) : "v"(x), "v"(p));         \
    asm volatile(S : "+v"(a1) : "v"(x), "v"(p));         \
    asm volatile(S : "+v"(a2) : "v"(x), "v"(p));         \
    asm volatile(S : "+v"(a3) : "v"(x), "v"(p));         \
    asm volatile(S : "+v"(a4) : "v"(x), "v"(p));         \
    asm volatile(S : "+v"(a5) : "v"(x), "v"(p));         \
    asm volatile(S : "+v"(a6) : "v"(x), "v"(p));         \
    asm volatile(S : "+v"(a7) : "v"(x), "v"(p));         \
  }
    ORN_PROBE_OPS(X)
#undef X
  }
  out[blockIdx.x * 256 + threadIdx.x] = a0 + a1 + a2 + a3 + a4 + a5 + a6 + a7;
}
constexpr int kProbeOps = 13;
#define X(N, S) S,
const char* const kProbeOpNames[kProbeOps] = {ORN_PROBE_OPS(X)};
#undef X

// ---- what a kernel argument costs. The same kernel twice: its arguments as one struct (read
// through a scalar load when the wavefront starts, as most kernels of this library take theirs)
// and as leading flat arguments (preloaded into scalar registers with the wavefront). Each
// workgroup stamps the 100 MHz clock at entry, when the argument is in a register, after a scalar
// load that depends on it and after a vector load that depends on that.
struct ProbeArgPack {
  const uint32_t* p[6];
  int n[4];
};
__device__ __forceinline__ void probe_kernarg_body(const uint32_t* idx, const uint32_t* data, long long* out,
                                                   long long t0) {
  uint64_t v = (uint64_t)idx;
  asm volatile("" : "+s"(v));
  const long long t1 = wall_clock64();
  uint32_t i2 = __builtin_amdgcn_readfirstlane(*reinterpret_cast<const uint32_t*>(v));
  asm volatile("" : "+s"(i2));
  const long long t2 = wall_clock64();
  uint32_t w = data[(i2 & 255u) * 64 + threadIdx.x];
  asm volatile("" : "+v"(w));
  const long long t3 = wall_clock64();
  if (threadIdx.x == 0) {
    long long* o = out + blockIdx.x * 4;
    o[0] = t0;
    o[1] = t1;
    o[2] = t2;
    o[3] = t3 + (w == 0x12345u);
  }
}
__global__ __launch_bounds__(256) void probe_kernarg_struct_kernel(ProbeArgPack a, long long* out) {
  const long long t0 = wall_clock64();
  probe_kernarg_body(a.p[1], a.p[2], out, t0);
}
__global__ __launch_bounds__(256) void probe_kernarg_flat_kernel(const uint32_t* idx, const uint32_t* data, long long* out) {
  const long long t0 = wall_clock64();
  probe_kernarg_body(idx, data, out, t0);
}

}  // namespace

extern "C" {

// One launch of `workgroups` x 256 threads, each thread running 8 x `iters` of instruction `op`
// (ornith_probe_valu_name(op) names it; ops 0 .. ornith_probe_valu_count() - 1). d_x: 4 floats,
// d_p: 4 words (a word whose halves are small f16 values keeps every instruction finite),
// d_out: workgroups * 256 floats.
int ornith_probe_valu_count(void) { return kProbeOps; }
const char* ornith_probe_valu_name(int op) { return op >= 0 && op < kProbeOps ? kProbeOpNames[op] : ""; }
int ornith_probe_valu(ornith_ctx* ctx, int op, int workgroups, int iters, const void* d_x, const void* d_p, void* d_out) {
  ORN_REQUIRE(ctx && d_x && d_p && d_out && op >= 0 && op < kProbeOps && workgroups >= 1 && iters >= 1,
              "probe_valu: bad argument");
  switch (op) {
#define X(N, S)                                                                                                   \
  case N:                                                                                                         \
    hipLaunchKernelGGL(probe_valu_kernel<N>, dim3(workgroups), dim3(256), 0, ctx->stream, (const float*)d_x,      \
                       (const uint32_t*)d_p, (float*)d_out, iters);                                               \
    break;
    ORN_PROBE_OPS(X)
#undef X
  }
  ORN_LAUNCH_CHECK("probe_valu_kernel");
  return ORNITH_OK;
}

// flat = 0: the arguments in a struct; 1: as leading flat arguments. d_idx: one word (an index
// below 256), d_data: 64 KB, d_out: workgroups x 4 x int64 (the four stamps).
int ornith_probe_kernarg(ornith_ctx* ctx, int flat, int workgroups, const void* d_idx, const void* d_data, void* d_out) {
  ORN_REQUIRE(ctx && d_idx && d_data && d_out && workgroups >= 1, "probe_kernarg: bad argument");
  if (flat) {
    hipLaunchKernelGGL(probe_kernarg_flat_kernel, dim3(workgroups), dim3(256), 0, ctx->stream, (const uint32_t*)d_idx,
                       (const uint32_t*)d_data, (long long*)d_out);
  } else {
    ProbeArgPack a{};
    a.p[1] = (const uint32_t*)d_idx;
    a.p[2] = (const uint32_t*)d_data;
    hipLaunchKernelGGL(probe_kernarg_struct_kernel, dim3(workgroups), dim3(256), 0, ctx->stream, a, (long long*)d_out);
  }
  ORN_LAUNCH_CHECK("probe_kernarg_kernel");
  return ORNITH_OK;
}

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
