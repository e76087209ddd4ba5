// Internal runtime declarations shared by the HIP translation units.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "../../include/ornith_hip.h"

struct ornith_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  int compute_units = 0;
  // grow-only scratch for operators that need temporaries between their kernels;
  // stream order makes reuse by the next operator safe.
  void* scratch = nullptr;
  size_t scratch_cap = 0;
  // pinned host staging for the few bytes a decode loop reads back per step (token ids):
  // a copy into pinned memory completes without the runtime's pageable detour
  void* pinned = nullptr;
  static constexpr size_t kPinnedBytes = 4096;
  // hand-offs inside a launch (handoff.h): the flag words, the epoch handed to the next such
  // launch, and the word a wait that ran out of its bound reports through (pinned host
  // memory the kernels write directly; checked after every synchronisation)
  uint32_t* ho_flags = nullptr;
  static constexpr size_t kHoFlagWords = 16384;
  uint32_t ho_epoch = 0;
  volatile uint32_t* ho_err = nullptr;
  uint32_t* ho_err_dev = nullptr;
  // kernels whose dynamic LDS limit has been raised for this context's device (a function
  // attribute is per device; a context is used from one thread at a time)
  unsigned lds_attr_set = 0;
  // this device's copy of the greedy selection's fixed scratch array (sample.hip)
  void* na_scratch = nullptr;
};

// After the stream has been synchronised: fails if a hand-off wait inside a launch gave up.
int ornith_check_handoffs(ornith_ctx* ctx);

// Returns at least `bytes` of device scratch (256-byte aligned). Growing it
// synchronises the stream; callers that must not allocate size it once up front.
int ornith_scratch(ornith_ctx* ctx, size_t bytes, void** out);

// d_dst[r] = d_src[d_ids[r]] for n rows of row_bytes (a multiple of 4) each, one launch.
int ornith_gather_rows(ornith_ctx* ctx, const void* d_src, size_t row_bytes, const uint32_t* d_ids,
                       int n, void* d_dst);

// bump allocator over a scratch block
struct ScratchCursor {
  char* base;
  size_t off = 0;
  explicit ScratchCursor(void* p) : base(static_cast<char*>(p)) {}
  template <typename T>
  T* take(size_t count) {
    T* r = reinterpret_cast<T*>(base + off);
    off += (count * sizeof(T) + 255) & ~size_t(255);
    return r;
  }
};

// Activation rows from which the k-quant projections and the MoE block switch from the
// exact mat-vec path (every row as if alone) to the matrix-core GEMM path. The reference
// draws the same line at its EXACT_WINDOW (src/ops/invariant.rs:88-116).
int ornith_option_gemm_rows();  // default 32; 0 = never (everything through the exact path)
#define kPrefillRows (ornith_option_gemm_rows())

// ornith_greedy_rows with its temporaries taken from the caller's cursor (for operators
// that hold other scratch buffers at the same time). Needs rows * ceil(V/1024) * 16 + 2048 bytes.
int ornith_greedy_rows_ws(ornith_ctx* ctx, const void* d_logits, int rows, int V, uint32_t* d_tokens,
                          void* d_lse, ScratchCursor& sc);

// Resolves the device address of the greedy selection's fixed scratch array on `device`
// (which must be current) once per device; ornith_ctx_create keeps it in the context.
int ornith_sample_init_device(int device, void** ptr_out);

// Records the message for ornith_last_error() and returns `code`.
int ornith_fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

#define ORN_HIP(expr)                                                                   \
  do {                                                                                  \
    hipError_t e__ = (expr);                                                            \
    if (e__ != hipSuccess)                                                              \
      return ornith_fail(ORNITH_ERR_HIP, "%s failed: %s (%s:%d)", #expr,                \
                         hipGetErrorString(e__), __FILE__, __LINE__);                   \
  } while (0)

#define ORN_REQUIRE(cond, ...)                                  \
  do {                                                          \
    if (!(cond)) return ornith_fail(ORNITH_ERR_INVALID, __VA_ARGS__); \
  } while (0)

// After a kernel launch: report a launch failure (bad grid, missing code object).
#define ORN_LAUNCH_CHECK(name)                                                         \
  do {                                                                                  \
    hipError_t e__ = hipGetLastError();                                                 \
    if (e__ != hipSuccess)                                                              \
      return ornith_fail(ORNITH_ERR_HIP, "launch of %s failed: %s", name,               \
                         hipGetErrorString(e__));                                       \
  } while (0)

// Behaviour switches, read once from the environment (ORNITH_FUSE_MOE=0 ...) and
// settable at run time through ornith_set_option so A/B runs share a process, the way
// the reference's ORNITH_* flags work (/root/reference/src/ops/moe.rs:397-414).
int ornith_option_fuse_moe();
int ornith_option_fuse_proj();
int ornith_option_fuse_gdn();
int ornith_option_fuse_norm();
extern "C" int ornith_kq_matmul_multi(ornith_ctx* ctx, const ornith_kmatrix* const* ws, int n, const void* d_x, int M,
                                      void* const* d_ys);
int ornith_option_gemm_reg();  // 1: expert-gathered prefill GEMM with the weights dequantized into MFMA operand registers; 0: through LDS
int ornith_option_gdn_block_chunks();  // 64-token chunks a launch pair of the chunked gated-delta recurrence takes
int ornith_option_gemm_duo();  // 1: prefill GEMM with producer and consumer wavefronts; 0: every wavefront does both in turn
int ornith_option_fuse_attn_prep();  // 1: the attention launch does its own prep at decode widths
int ornith_option_kq_iters();      // output rows per wavefront pass of the mat-vec kernels; 0 = by shape
int ornith_option_moe_up_iters();  // rows per wavefront of the fused gate+up kernel; 0 = by shape
int ornith_option_moe_down_iters();  // column groups per workgroup of the expert down kernel; 0 = by shape
int ornith_option_gdn_chunked();  // 1: the gated-delta recurrence of calls of 128 rows or more runs chunked on the matrix cores
int ornith_option_fuse_moe_one();  // 1: the MoE block's router, up and down phases in one launch
int ornith_option_ho_spins();      // polling rounds a hand-off wait inside a launch may take

static inline size_t ornith_dtype_size(int dt) { return dt == ORNITH_F32 ? 4 : 2; }
