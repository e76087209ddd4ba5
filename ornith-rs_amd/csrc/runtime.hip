// Context, memory and timing: the part of metal::Context
// (/root/reference/src/metal/mod.rs:433-519) a HIP stream does not already give.
// A stream orders every kernel after the previous one, so the reference's hazard
// tracker, barrier epochs and command-buffer batching have no counterpart here.
#include "rt.h"

#include <cstdlib>

static thread_local char g_err[512] = "";

int ornith_fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof g_err, fmt, ap);
  va_end(ap);
  return code;
}

int ornith_scratch(ornith_ctx* ctx, size_t bytes, void** out) {
  if (bytes > ctx->scratch_cap) {
    ORN_HIP(hipStreamSynchronize(ctx->stream));
    if (ctx->scratch) ORN_HIP(hipFree(ctx->scratch));
    ctx->scratch = nullptr;
    ctx->scratch_cap = 0;
    size_t cap = (bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
    ORN_HIP(hipMalloc(&ctx->scratch, cap));
    ctx->scratch_cap = cap;
  }
  *out = ctx->scratch;
  return ORNITH_OK;
}

namespace {
struct Option {
  const char* name;
  const char* env;
  int dflt;
  int value;  // -1: not read yet
};
Option g_options[] = {{"fuse_moe", "ORNITH_FUSE_MOE", 1, -1},
                      {"fuse_proj", "ORNITH_FUSE_PROJ", 1, -1},
                      {"moe_up_iters", "ORNITH_MOE_UP_ITERS", 0, -1},
                      {"kq_iters", "ORNITH_KQ_ITERS", 0, -1},
                      {"gemm_rows", "ORNITH_GEMM_ROWS", 32, -1},
                      {"fuse_gdn", "ORNITH_FUSE_GDN", 1, -1},
                      {"fuse_norm", "ORNITH_FUSE_NORM", 1, -1},
                      {"gemm_duo", "ORNITH_GEMM_DUO", 1, -1},
                      {"fuse_moe_one", "ORNITH_FUSE_MOE_ONE", 0, -1},
                      {"ho_spins", "ORNITH_HO_SPINS", 1 << 20, -1},
                      {"moe_down_iters", "ORNITH_MOE_DOWN_ITERS", 0, -1},
                      {"gdn_chunked", "ORNITH_GDN_CHUNKED", 1, -1},
                      {"gemm_reg", "ORNITH_GEMM_REG", 1, -1},
                      {"gdn_block_chunks", "ORNITH_GDN_BLOCK_CHUNKS", 64, -1},
                      {"fuse_attn_prep", "ORNITH_FUSE_ATTN_PREP", 1, -1}};
int option_value(int i) {
  Option& o = g_options[i];
  if (o.value < 0) {
    const char* e = getenv(o.env);
    o.value = (e && e[0] >= '0' && e[0] <= '9') ? atoi(e) : o.dflt;
  }
  return o.value;
}
}  // namespace

int ornith_option_fuse_moe() { return option_value(0); }
int ornith_option_fuse_proj() { return option_value(1); }
int ornith_option_moe_up_iters() { return option_value(2); }
int ornith_option_kq_iters() { return option_value(3); }
int ornith_option_fuse_gdn() { return option_value(5); }
int ornith_option_fuse_norm() { return option_value(6); }
int ornith_option_gemm_duo() { return option_value(7); }
int ornith_option_fuse_moe_one() { return option_value(8); }
int ornith_option_moe_down_iters() { return option_value(10); }
int ornith_option_gdn_chunked() { return option_value(11); }
int ornith_option_gemm_reg() { return option_value(12); }
int ornith_option_gdn_block_chunks() { return option_value(13); }
int ornith_option_fuse_attn_prep() { return option_value(14); }
int ornith_option_ho_spins() { return option_value(9) < 1 ? 1 : option_value(9); }

int ornith_check_handoffs(ornith_ctx* ctx) {
  if (ctx->ho_err && *ctx->ho_err) {
    *ctx->ho_err = 0;
    return ornith_fail(ORNITH_ERR_HIP,
                       "a wait between workgroups inside a launch ran out of its bound (ho_spins = %d): "
                       "the results of that launch are invalid", ornith_option_ho_spins());
  }
  return ORNITH_OK;
}
int ornith_option_gemm_rows() {
  const int v = option_value(4);
  return v <= 0 ? 1 << 30 : v;
}

namespace {
// one workgroup per gathered row, 4-byte words
__global__ __launch_bounds__(256) void gather_rows_kernel(const uint32_t* __restrict__ src, size_t row_words,
                                                          const uint32_t* __restrict__ ids,
                                                          uint32_t* __restrict__ dst) {
  const uint32_t* s = src + (size_t)ids[blockIdx.x] * row_words;
  uint32_t* d = dst + (size_t)blockIdx.x * row_words;
  for (size_t i = threadIdx.x; i < row_words; i += 256) d[i] = s[i];
}
}  // namespace

int ornith_gather_rows(ornith_ctx* ctx, const void* d_src, size_t row_bytes, const uint32_t* d_ids,
                       int n, void* d_dst) {
  ORN_REQUIRE(ctx && d_src && d_ids && d_dst && n >= 1, "gather_rows: null argument");
  ORN_REQUIRE(row_bytes >= 4 && row_bytes % 4 == 0, "gather_rows: rows of %zu bytes", row_bytes);
  hipLaunchKernelGGL(gather_rows_kernel, dim3(n), dim3(256), 0, ctx->stream, (const uint32_t*)d_src,
                     row_bytes / 4, d_ids, (uint32_t*)d_dst);
  ORN_LAUNCH_CHECK("gather_rows_kernel");
  return ORNITH_OK;
}

extern "C" {

int ornith_set_option(const char* name, int value) {
  ORN_REQUIRE(name, "set_option: null name");
  for (auto& o : g_options)
    if (!strcmp(o.name, name)) {
      o.value = value < 0 ? 0 : value;
      return ORNITH_OK;
    }
  return ornith_fail(ORNITH_ERR_INVALID, "set_option: unknown option '%s'", name);
}

const char* ornith_last_error(void) { return g_err; }

int ornith_ctx_create(int device, ornith_ctx** out) {
  ORN_REQUIRE(out != nullptr, "ornith_ctx_create: out is null");
  int n = 0;
  ORN_HIP(hipGetDeviceCount(&n));
  ORN_REQUIRE(device >= 0 && device < n, "ornith_ctx_create: device %d of %d", device, n);
  ORN_HIP(hipSetDevice(device));
  hipDeviceProp_t prop;
  ORN_HIP(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return ornith_fail(ORNITH_ERR_UNSUPPORTED,
                       "ornith_ctx_create: device %d is %s; this library is built for gfx950 only",
                       device, prop.gcnArchName);
  void* na_scratch = nullptr;
  if (int rc = ornith_sample_init_device(device, &na_scratch)) return rc;
  ornith_ctx* c = new ornith_ctx();
  c->device = device;
  c->na_scratch = na_scratch;
  c->compute_units = prop.multiProcessorCount;
  // every step below can fail: one way out, which releases whatever the steps before it made
  const int rc = [&]() -> int {
    ORN_HIP(hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking));
    ORN_HIP(hipEventCreate(&c->ev0));
    ORN_HIP(hipEventCreate(&c->ev1));
    ORN_HIP(hipHostMalloc(&c->pinned, ornith_ctx::kPinnedBytes, hipHostMallocDefault));
    ORN_HIP(hipMalloc((void**)&c->ho_flags, sizeof(uint32_t) * ornith_ctx::kHoFlagWords));
    ORN_HIP(hipMemset(c->ho_flags, 0, sizeof(uint32_t) * ornith_ctx::kHoFlagWords));
    void* err_host = nullptr;
    ORN_HIP(hipHostMalloc(&err_host, 256, hipHostMallocDefault));
    memset(err_host, 0, 256);
    c->ho_err = static_cast<volatile uint32_t*>(err_host);
    ORN_HIP(hipHostGetDevicePointer((void**)&c->ho_err_dev, err_host, 0));
    return ORNITH_OK;
  }();
  if (rc) {
    ornith_ctx_destroy(c);
    return rc;
  }
  *out = c;
  return ORNITH_OK;
}

int ornith_ctx_destroy(ornith_ctx* ctx) {
  if (!ctx) return ORNITH_OK;
  // also the way out of a context that was only partly made: every member is checked
  if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
  if (ctx->scratch) (void)hipFree(ctx->scratch);
  if (ctx->pinned) (void)hipHostFree(ctx->pinned);
  if (ctx->ho_flags) (void)hipFree(ctx->ho_flags);
  if (ctx->ho_err) (void)hipHostFree(const_cast<uint32_t*>(ctx->ho_err));
  if (ctx->ev0) (void)hipEventDestroy(ctx->ev0);
  if (ctx->ev1) (void)hipEventDestroy(ctx->ev1);
  if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
  delete ctx;
  return ORNITH_OK;
}

int ornith_sync(ornith_ctx* ctx) {
  ORN_REQUIRE(ctx, "ornith_sync: null ctx");
  ORN_HIP(hipStreamSynchronize(ctx->stream));
  return ornith_check_handoffs(ctx);
}

int ornith_alloc(ornith_ctx* ctx, size_t bytes, void** d_out) {
  ORN_REQUIRE(ctx && d_out, "ornith_alloc: null argument");
  if (bytes == 0) bytes = 256;
  ORN_HIP(hipSetDevice(ctx->device));
  ORN_HIP(hipMalloc(d_out, bytes));
  return ORNITH_OK;
}

int ornith_free(ornith_ctx* ctx, void* d_ptr) {
  ORN_REQUIRE(ctx, "ornith_free: null ctx");
  if (!d_ptr) return ORNITH_OK;
  ORN_HIP(hipStreamSynchronize(ctx->stream));
  ORN_HIP(hipFree(d_ptr));
  return ORNITH_OK;
}

int ornith_upload(ornith_ctx* ctx, void* d_dst, const void* host, size_t bytes) {
  ORN_REQUIRE(ctx && (bytes == 0 || (d_dst && host)), "ornith_upload: null argument");
  if (bytes == 0) return ORNITH_OK;
  ORN_HIP(hipMemcpyAsync(d_dst, host, bytes, hipMemcpyHostToDevice, ctx->stream));
  // pageable source: the copy may still be staging from `host`; wait so the
  // caller is free to reuse it, which is what the reference's from_slice gives.
  ORN_HIP(hipStreamSynchronize(ctx->stream));
  return ORNITH_OK;
}

int ornith_download(ornith_ctx* ctx, void* host, const void* d_src, size_t bytes) {
  ORN_REQUIRE(ctx && (bytes == 0 || (d_src && host)), "ornith_download: null argument");
  if (bytes == 0) return ORNITH_OK;
  if (bytes <= ornith_ctx::kPinnedBytes && ctx->pinned) {
    ORN_HIP(hipMemcpyAsync(ctx->pinned, d_src, bytes, hipMemcpyDeviceToHost, ctx->stream));
    ORN_HIP(hipStreamSynchronize(ctx->stream));
    memcpy(host, ctx->pinned, bytes);
    return ornith_check_handoffs(ctx);
  }
  ORN_HIP(hipMemcpyAsync(host, d_src, bytes, hipMemcpyDeviceToHost, ctx->stream));
  ORN_HIP(hipStreamSynchronize(ctx->stream));
  return ornith_check_handoffs(ctx);
}

int ornith_memset(ornith_ctx* ctx, void* d_dst, int byte, size_t bytes) {
  ORN_REQUIRE(ctx && (bytes == 0 || d_dst), "ornith_memset: null argument");
  if (bytes == 0) return ORNITH_OK;
  ORN_HIP(hipMemsetAsync(d_dst, byte, bytes, ctx->stream));
  return ORNITH_OK;
}

int ornith_copy(ornith_ctx* ctx, void* d_dst, const void* d_src, size_t bytes) {
  ORN_REQUIRE(ctx && (bytes == 0 || (d_dst && d_src)), "ornith_copy: null argument");
  if (bytes == 0) return ORNITH_OK;
  ORN_HIP(hipMemcpyAsync(d_dst, d_src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
  return ORNITH_OK;
}

int ornith_device_info(ornith_ctx* ctx, char* name, size_t name_len, int* compute_units,
                       size_t* total_mem) {
  ORN_REQUIRE(ctx, "ornith_device_info: null ctx");
  hipDeviceProp_t prop;
  ORN_HIP(hipGetDeviceProperties(&prop, ctx->device));
  if (name && name_len) snprintf(name, name_len, "%s (%s)", prop.name, prop.gcnArchName);
  if (compute_units) *compute_units = prop.multiProcessorCount;
  if (total_mem) *total_mem = prop.totalGlobalMem;
  return ORNITH_OK;
}

int ornith_timer_begin(ornith_ctx* ctx) {
  ORN_REQUIRE(ctx, "ornith_timer_begin: null ctx");
  ORN_HIP(hipEventRecord(ctx->ev0, ctx->stream));
  return ORNITH_OK;
}

int ornith_timer_end(ornith_ctx* ctx, float* ms_out) {
  ORN_REQUIRE(ctx && ms_out, "ornith_timer_end: null argument");
  ORN_HIP(hipEventRecord(ctx->ev1, ctx->stream));
  ORN_HIP(hipEventSynchronize(ctx->ev1));
  ORN_HIP(hipEventElapsedTime(ms_out, ctx->ev0, ctx->ev1));
  return ORNITH_OK;
}

}  // extern "C"
