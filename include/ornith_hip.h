/*
 * ornith_hip.h -- C ABI of the MI355X (gfx950) speculative-decode path.
 *
 * Every entry point takes plain pointers and sizes, returns an int status
 * (ORNITH_OK == 0) and never aborts; the message for the last failure on the
 * calling thread is available from ornith_last_error(). Pointers named d_* are
 * device pointers obtained from ornith_alloc(); everything else is host memory.
 * A context owns one HIP stream; all work of a context is ordered on it and a
 * context must be used from one thread at a time (the reference's Context is
 * !Send for the same reason, /root/reference/src/metal/mod.rs:433-519).
 *
 * Each declaration cites the reference interface it stands in for.
 */
#ifndef ORNITH_HIP_H
#define ORNITH_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* exported from the shared library (everything else is hidden) */
#define ORNITH_API __attribute__((visibility("default")))

#define ORNITH_OK 0
#define ORNITH_ERR_INVALID 1 /* shape / mode / argument mismatch (the reference asserts) */
#define ORNITH_ERR_HIP 2     /* a HIP call or kernel launch failed */
#define ORNITH_ERR_IO 3      /* file could not be read / parsed */
#define ORNITH_ERR_UNSUPPORTED 4

/* activation / output element types */
#define ORNITH_F32 0
#define ORNITH_BF16 1

/* k-quant kinds (src/ops/kquant.rs KQuant) */
#define ORNITH_Q4K 0
#define ORNITH_Q6K 1
/* a third kind a stacked-expert descriptor may carry (the MoE block only; the k-quant
 * operators refuse it): mlx 4-bit affine, group 32 - the published artifact's switch_mlp */
#define ORNITH_AFFINE4_G32 2

typedef struct ornith_ctx ornith_ctx;

/* ---- runtime: replaces metal::Context (src/metal/mod.rs:433-519, 521-646, 833-879) */
ORNITH_API int ornith_ctx_create(int device, ornith_ctx** out);
ORNITH_API int ornith_ctx_destroy(ornith_ctx* ctx);
/* Context::sync (src/metal/mod.rs:833-879): block until the stream is idle. */
ORNITH_API int ornith_sync(ornith_ctx* ctx);
/* Array::empty / alloc_exact (src/metal/mod.rs:636-646). 256-byte aligned. */
ORNITH_API int ornith_alloc(ornith_ctx* ctx, size_t bytes, void** d_out);
ORNITH_API int ornith_free(ornith_ctx* ctx, void* d_ptr);
/* Array::from_slice / to_vec (src/array.rs:132-197). Both are stream ordered;
 * download synchronises before returning, upload does not outlive `host`. */
ORNITH_API int ornith_upload(ornith_ctx* ctx, void* d_dst, const void* host, size_t bytes);
ORNITH_API int ornith_download(ornith_ctx* ctx, void* host, const void* d_src, size_t bytes);
ORNITH_API int ornith_memset(ornith_ctx* ctx, void* d_dst, int byte, size_t bytes);
ORNITH_API int ornith_copy(ornith_ctx* ctx, void* d_dst, const void* d_src, size_t bytes);
ORNITH_API const char* ornith_last_error(void);
/* device facts for reports: name into buf, CU count, bytes of device memory */
ORNITH_API int ornith_device_info(ornith_ctx* ctx, char* name, size_t name_len, int* compute_units,
                       size_t* total_mem);
/* Event timing on the context's stream (the reference sums GPUEndTime -
 * GPUStartTime per command buffer, src/metal/mod.rs:197-285). begin/end record
 * events; elapsed synchronises on the end event and returns milliseconds. */
/* Behaviour switches (the reference's ORNITH_* flags with their runtime set_* twins,
 * src/ops/moe.rs:397-414, src/ops/gdn.rs:416-426). Each is also read once from the
 * environment variable named here; every value gives bit-identical results.
 *   "fuse_moe"  (ORNITH_FUSE_MOE, default 1): the two fused expert kernels vs. one
 *               launch per operator
 *   "fuse_proj" (ORNITH_FUSE_PROJ, default 1): projections sharing an input in one launch
 *   "moe_up_iters" (ORNITH_MOE_UP_ITERS, default 0 = chosen by shape; 2 or 4): output
 *               rows per wavefront of the fused gate+up expert kernel, a tuning knob
 *   "fuse_gdn"  (ORNITH_FUSE_GDN, default 1): the gated-delta mixer core (a / b projections,
 *               front, recurrence, gated norm) in one launch at decode / verify widths
 *   "fuse_norm" (ORNITH_FUSE_NORM, default 1): the residual add + RMS norm in front of a
 *               group of k-quant projections / the router is computed inside their launch
 *   "gemm_rows" (ORNITH_GEMM_ROWS, default 32; 0 = never): activation rows from which the
 *               k-quant projections and the MoE experts run as matrix-core GEMMs instead of
 *               exact mat-vecs. The one switch that changes results (to bf16 rounding of the
 *               weights): prefill is outside the exact window in the reference as well.
 *   "kq_iters"  (ORNITH_KQ_ITERS, default 0 = chosen by the launch from its shape and from how
 *               many of its workgroups a compute unit holds; 1..8): output rows each
 *               wavefront of the k-quant mat-vec walks, a tuning knob
 *   "gemm_duo"  (ORNITH_GEMM_DUO, default 1): the 256-row tile of the prefill GEMM runs with
 *               producer and consumer wavefronts (0: every wavefront dequantizes, then
 *               multiplies); same results either way
 *   "gemm_reg"  (ORNITH_GEMM_REG, default 1): the expert-gathered prefill GEMM dequantizes the
 *               weights into MFMA operand registers where the shape suits it (48 rows an expert
 *               or more: a workgroup a tile for K >= 1024, 64-row workgroups for fewer K slabs;
 *               0: always through LDS); results agree to the order of the fp32 sums
 *   "gdn_chunked" (ORNITH_GDN_CHUNKED, default 1): the gated-delta recurrence of calls of 128
 *               rows or more (without per-token snapshots) runs in 64-token chunks on the
 *               matrix cores (0: token by token); results agree to rounding
 *   "gdn_block_chunks" (ORNITH_GDN_BLOCK_CHUNKS, default 64): chunks one prepare / scan launch
 *               pair of that recurrence covers (longer calls go block by block so that the
 *               block's operands stay in the last-level cache); same results for any value
 *   "fuse_attn_prep" (ORNITH_FUSE_ATTN_PREP, default 1): ornith_attn_decode lets the attention
 *               launch do the prep of its own rows (norm, RoPE, KV append) at decode widths
 *               (0: a prep launch first); bit-identical
 *   "fuse_moe_one" (ORNITH_FUSE_MOE_ONE, default 0): the MoE block's phases as ranges of
 *               workgroups of ONE launch that hand their intermediates over through memory
 *               (1: router + up + down, 2: up + down after a router launch). Bit-identical,
 *               measured slower than the separate launches on this part, kept for that
 *               measurement (hidden size 2048, expert width 512, T <= 4 only)
 *   "ho_spins"  (ORNITH_HO_SPINS, default 2^20): polling rounds a wait between workgroups of
 *               such a launch may take before it gives up; the failure is reported by the next
 *               ornith_sync / ornith_download (ORNITH_ERR_HIP) */
ORNITH_API int ornith_set_option(const char* name, int value);
ORNITH_API int ornith_timer_begin(ornith_ctx* ctx);
ORNITH_API int ornith_timer_end(ornith_ctx* ctx, float* ms_out);

/* ---- k-quant matrices: KMatrix (src/ops/kquant.rs:349-411) ------------------
 * Three device tensors in the reference's layout:
 *   Q4_K qs u32[E,O,K/8]     scales u8[E,O,K/256,12]  dm f16[E,O,K/256,2]
 *   Q6_K qs u32[E,O,3K/16]   scales u8[E,O,K/256,16]  dm f16[E,O,K/256,1]
 * E == 1 for a plain matrix. For routed experts in the 4-bit affine format
 * (src/ops/quantized.rs:531-589) the same three slots carry kind ORNITH_AFFINE4_G32:
 *   qs u32[E,O,K/8] (eight codes a word)   scales bf16[E,O,K/32]   dm = biases bf16[E,O,K/32] */
typedef struct ornith_kmatrix {
  int kind; /* ORNITH_Q4K / ORNITH_Q6K (/ ORNITH_AFFINE4_G32: expert stacks of a MoE block) */
  int E, O, K;
  const void* d_qs;
  const void* d_scales;
  const void* d_dm;
} ornith_kmatrix;

/* KMatrix::check: validates kind, K % 256, and the three byte sizes. */
ORNITH_API int ornith_kmatrix_check(const ornith_kmatrix* w, size_t qs_bytes, size_t scales_bytes,
                         size_t dm_bytes);

/* kquant::dequantize (src/ops/kquant.rs:418-433; kernels q4k.metal:64-96,
 * q6k.metal:47-77): all E*O*K weights to out_dtype. */
ORNITH_API int ornith_kq_dequantize(ornith_ctx* ctx, const ornith_kmatrix* w, void* d_out, int out_dtype);

/* kquant::qmv (src/ops/kquant.rs:539-595): y[M,O] = x[M,K] . W^T, fp32
 * accumulate, each row computed exactly as it would be alone. M <= 4 is the
 * decode/verify shape; larger M loops in groups of four. */
ORNITH_API int ornith_kq_qmv(ornith_ctx* ctx, const ornith_kmatrix* w, const void* d_x, int x_dtype, int M,
                  void* d_y, int y_dtype);

/* n <= 4 kquant::qmv calls over the same activations in one launch (the reference issues
 * them back to back, src/model/qwen3_5.rs:441-447,493-494). All matrices must share
 * format and width; d_ys[i] receives [M, ws[i]->O]. Bit-identical to separate calls. */
ORNITH_API int ornith_kq_qmv_multi(ornith_ctx* ctx, const ornith_kmatrix* const* ws, int n,
                                   const void* d_x, int x_dtype, int M, void* const* d_ys,
                                   int y_dtype);

/* kquant::gather_qmv (src/ops/kquant.rs:741-770): out[r] = x[lhs[r]] . W[rhs[r]]^T,
 * r < rows; lhs/rhs are device u32 arrays; x has x_rows rows. Indices live on the
 * device, so they cannot be validated here: an id past the end is clamped to the
 * last row / expert instead of reading out of bounds. */
ORNITH_API int ornith_kq_gather_qmv(ornith_ctx* ctx, const ornith_kmatrix* w, const void* d_x, int x_dtype,
                         int x_rows, const uint32_t* d_lhs, const uint32_t* d_rhs, int rows,
                         void* d_y, int y_dtype);

/* kquant::matmul / qmm_t (src/ops/kquant.rs:783-905; kernels/kquant_mm.h): the prefill-width
 * GEMM y[M,O] = x[M,K] . W^T, bf16 in and out, on the matrix cores: weight tiles are
 * dequantized to bf16 on the way into LDS (HBM traffic stays at the quantized size), fp32
 * accumulate. Agrees with kq_qmv to bf16 rounding of the weights, not bit for bit (prefill
 * is outside the reference's exact window as well, src/ops/invariant.rs:140-168). */
ORNITH_API int ornith_kq_matmul(ornith_ctx* ctx, const ornith_kmatrix* w, const void* d_x, int M,
                                void* d_y);
/* kquant::gather_matmul / gather_qmm_t (src/ops/kquant.rs:907-1027): the same GEMM over an
 * expert-stacked matrix, rows grouped by routed expert. d_inds[p] is the expert of pair
 * p = token * top_k + slot. is_up != 0: pair p reads row p / top_k of x (the token) and
 * writes row p of y (gate / up projections); is_up == 0: reads row p of x and writes row p
 * (down projection). d_plan: ornith_kq_gather_plan_bytes(pairs, E) bytes of device memory
 * holding the expert-sorted pair list; rebuild_plan != 0 recomputes it from d_inds (one
 * launch), 0 reuses what an earlier call with the same inds left there (gate, up and down
 * of one MoE block share one plan). */
ORNITH_API size_t ornith_kq_gather_plan_bytes(int pairs, int E);
ORNITH_API int ornith_kq_gather_matmul(ornith_ctx* ctx, const ornith_kmatrix* w, const void* d_x,
                                       const uint32_t* d_inds, int pairs, int top_k, int is_up,
                                       void* d_plan, int rebuild_plan, void* d_y);

/* ---- Linear: ops::linear::Linear (src/ops/linear.rs:23-28), one polymorphic
 * projection. Activations in and out are bf16. -------------------------------- */
#define ORNITH_LIN_KQUANT 0  /* Linear::K(KMatrix) */
#define ORNITH_LIN_AFFINE8 1 /* Linear::Mlx, mlx affine 8-bit group 64 (quantized.rs:311-333) */
#define ORNITH_LIN_DENSE 2   /* bf16 [O,K], ops::matmul::gemv (matmul.rs:334-438) */
#define ORNITH_LIN_AFFINE4 3 /* Linear::Mlx, mlx affine 4-bit group 32, the published artifact's format
                                (quantized.rs:311-333; vendored quantized.h:235-244) */
typedef struct ornith_linear {
  int mode;
  int O, K;
  ornith_kmatrix km;    /* KQUANT */
  const void* d_w;      /* AFFINE8: u8[O,K] (the reference's u32[O,K/4] bytes); DENSE: bf16[O,K];
                           AFFINE4: u8[O,K/2] (the reference's u32[O,K/8] bytes, lowest nibble first) */
  const void* d_scales; /* AFFINE8: bf16[O,K/64]; AFFINE4: bf16[O,K/32] */
  const void* d_biases; /* as d_scales */
} ornith_linear;

/* Linear::matmul (src/ops/linear.rs:60-110): y[M,O] = x[M,K] . W^T, bf16 in/out. */
ORNITH_API int ornith_linear_matmul(ornith_ctx* ctx, const ornith_linear* w, const void* d_x, int M,
                                    void* d_y);

/* n Linear::matmul calls over the same activations (in_proj_qkv + in_proj_z, in_proj_a +
 * in_proj_b, q/k/v projections: src/model/qwen3_5.rs:441-447,493-499). Fused into one
 * launch where the formats allow (same mode, width and k-quant kind; n <= 4), issued
 * one by one otherwise. Results are bit-identical either way. */
ORNITH_API int ornith_linear_matmul_multi(ornith_ctx* ctx, const ornith_linear* const* ws, int n,
                                          const void* d_x, int M, void* const* d_ys);

/* norm::add_rms_norm followed by the projections that read its output (the closing add of a
 * decoder layer, the next layer's input norm and its in_proj_qkv + in_proj_z or q/k/v
 * projections: src/model/qwen3_5.rs:374-396, 441-447, 493-499): h = res + y (bf16),
 * normed = rms_norm(h, w_norm), ys[i] = normed . W_i^T. For k-quant projections of width 2048
 * at M <= 4 the norm is made inside the projections' launch (every workgroup computes it while
 * its weight loads are in flight; one of them stores h and normed); otherwise add_rms_norm and
 * linear_matmul_multi are issued. Bit-identical either way. */
ORNITH_API int ornith_add_rms_linear_multi(ornith_ctx* ctx, const ornith_linear* const* ws, int n,
                                           const void* d_res, const void* d_y, const void* d_wnorm,
                                           float eps, int M, void* d_h_out, void* d_normed_out,
                                           void* const* d_ys);

/* ops::matmul::gather_mv (src/ops/matmul.rs:649-): stacked dense bf16 experts
 * W[E,O,K]; out[r] = x[lhs[r]] . W[rhs[r]]^T. Used by the MTP head's MoE. */
ORNITH_API int ornith_dense_gather_mv(ornith_ctx* ctx, const void* d_w, int E, int O, int K,
                                      const void* d_x, int x_rows, const uint32_t* d_lhs,
                                      const uint32_t* d_rhs, int rows, void* d_y);

/* quantized::gather_qmv for the 4-bit affine format (src/ops/quantized.rs:531-589): stacked
 * experts w u8[E,O,K/2], scales / biases bf16[E,O,K/32]; out[r] = x[lhs[r]] . W[rhs[r]]^T, bf16 in
 * and out. Ids past the end are clamped to the last row / expert. */
ORNITH_API int ornith_affine4_gather_qmv(ornith_ctx* ctx, const void* d_w, const void* d_scales,
                                         const void* d_biases, int E, int O, int K, const void* d_x,
                                         int x_rows, const uint32_t* d_lhs, const uint32_t* d_rhs, int rows,
                                         void* d_y);

/* ops::embedding::embedding (src/ops/embedding.rs:18-46): affine table rows (8-bit group 64 or
 * 4-bit group 32) -> bf16; ids are device u32, clamped to the table. */
ORNITH_API int ornith_embedding(ornith_ctx* ctx, const ornith_linear* table, const uint32_t* d_ids,
                                int n, void* d_out);

/* ---- MoE block -------------------------------------------------------------- */
/* softmax::softmax(precise) + moe::top_k -> router_top_k (src/ops/moe.rs:113-134,
 * 688-697; kernels/moe.metal:568-614): gates bf16 [T,E] -> probabilities (bf16) ->
 * the k winners by (value, then larger index), slots ascending; scores are the
 * winners' probabilities. d_probs may be null. E % 64 == 0, E <= 1024, k <= 16. */
ORNITH_API int ornith_router_topk(ornith_ctx* ctx, const void* d_gates, int T, int E, int k,
                                  uint32_t* d_inds, void* d_scores, void* d_probs);

/* elementwise::swiglu (kernels/ornith_elementwise.metal:97-105), bf16. */
ORNITH_API int ornith_swiglu(ornith_ctx* ctx, const void* d_gate, const void* d_up, int64_t n,
                             void* d_out);

/* moe::combine -> moe_combine (src/ops/moe.rs:548-596; kernels/moe.metal:207-258). */
ORNITH_API int ornith_moe_combine(ornith_ctx* ctx, const void* d_scores, const void* d_y,
                                  const void* d_gate, const void* d_shared, int T, int k, int dim,
                                  int normalize, void* d_out);

typedef struct ornith_moe_weights {
  ornith_linear router;                    /* mlp.gate [E,H] */
  ornith_kmatrix ex_gate, ex_up, ex_down;  /* mlp.switch_mlp.{gate,up,down}_proj */
  ornith_linear sh_gate, sh_up, sh_down;   /* mlp.shared_expert.* */
  ornith_linear sh_egate;                  /* mlp.shared_expert_gate [1,H] */
  int top_k;
  int norm_topk_prob;
  /* the MTP head's block (sparse_moe_block_dense, src/ops/moe.rs:863-937): experts are
   * stacked dense bf16 [E,O,K]; ex_* above then carry the dims only. */
  int ex_dense;
  const void* d_ex_gate;
  const void* d_ex_up;
  const void* d_ex_down;
} ornith_moe_weights;

/* moe::sparse_moe_block (src/ops/moe.rs:662-741): x bf16 [T,H] -> out bf16 [T,H].
 * d_inds_out (u32 [T,k]) and d_scores_out (bf16 [T,k]) may be null. T <= 64. */
ORNITH_API int ornith_moe_block(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_x, int T,
                                void* d_out, uint32_t* d_inds_out, void* d_scores_out);

/* norm::add_rms_norm followed by sparse_moe_block on its output (the post-attention norm and
 * the MLP of a decoder layer, src/model/qwen3_5.rs:384-392): h = res + y, normed =
 * rms_norm(h, w_norm), out = moe(normed). With the fused expert kernels, hidden size 2048 and
 * T <= 4 the norm is made inside the router's launch; otherwise add_rms_norm is issued first.
 * Bit-identical either way. */
ORNITH_API int ornith_add_rms_moe_block(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_res,
                                        const void* d_y, const void* d_wnorm, float eps, int T,
                                        void* d_h_out, void* d_normed_out, void* d_out);


/* moe::switch_glu_rows + the shared expert + moe::combine (src/ops/moe.rs:256-338,548-596)
 * given the router's picks: the expert gather-GEMV proper, as two kernels.
 *   phases & 1: act[(t*k+j)] = swiglu(gate_e(x_t), up_e(x_t)) for every routed pair, and
 *               act[T*k + t] for the shared expert; act is bf16 [(T*k + T), I] scratch
 *   phases & 2: out[t] = sum_j w_j * down_e(act) + sigmoid(egate_t) * down_shared(act)
 * d_inds u32 [T,k], d_scores bf16 [T,k] (router_topk outputs), d_egate bf16 [T]
 * (shared_expert_gate's output). Needs k-quant routed and shared experts of matching
 * formats and top_k <= 8 (ORNITH_ERR_UNSUPPORTED otherwise; ornith_moe_block falls back
 * to one launch per operator by itself). The ids live on the device and are not validated:
 * an id >= num_experts is read as the last expert (clamped for memory safety), so a corrupt
 * routing buffer gives plausible output, not an error. */
ORNITH_API int ornith_moe_experts(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_x, int T,
                                  const uint32_t* d_inds, const void* d_scores, const void* d_egate,
                                  void* d_act, void* d_out, int phases);

/* The same two launches as ornith_moe_block issues them after its router launch: the routing
 * (softmax + top-k, src/ops/moe.rs:688-697) is made from the router's gates (d_gates bf16
 * [T,E]) in the head of the up launch and stored to d_inds_out / d_scores_out, then the down
 * launch. What a caller times to see the expert gather-GEMV as the model runs it. */
ORNITH_API int ornith_moe_experts_from_gates(ornith_ctx* ctx, const ornith_moe_weights* w, const void* d_x,
                                             int T, const void* d_gates, const void* d_egate,
                                             uint32_t* d_inds_out, void* d_scores_out, void* d_act,
                                             void* d_out);

/* ---- norms: src/ops/norm.rs:19-220 (vendored rms_norm.metal:12-81,
 * kernels/ornith_norm.metal:28-183). Rows of n bf16 values, n = 64 * 2^j <= 4096. */
/* norm::rms_norm: out = w * (x * rsqrt(mean(x^2) + eps)); d_w may be null (weight 1). */
ORNITH_API int ornith_rms_norm(ornith_ctx* ctx, const void* d_x, const void* d_w, int rows, int n,
                               float eps, void* d_out);
/* norm::add_rms_norm: h = a + b (rounded, written to d_h_out), out = rms_norm(h). */
ORNITH_API int ornith_add_rms_norm(ornith_ctx* ctx, const void* d_a, const void* d_b, const void* d_w,
                                   int rows, int n, float eps, void* d_h_out, void* d_out);
/* norm::rms_norm_gated (Qwen3NextRMSNormGated): out = silu_f32(z) * rms_norm(y, w). */
ORNITH_API int ornith_rms_norm_gated(ornith_ctx* ctx, const void* d_y, const void* d_w,
                                     const void* d_z, int rows, int n, float eps, void* d_out);

/* ---- gated-delta layer --------------------------------------------------------- */
/* gdn::gdn_front (src/ops/gdn.rs:331-413, kernels/gdn_front.metal:65-190), batch 1:
 *   conv_state bf16[K-1,D], qkv bf16[T,D], cw bf16[D,K], a,b bf16[T,Hv], a_log,dt_bias bf16[Hv]
 *   -> q,k bf16[T,Hk,Dk], v bf16[T,Hv,Dv], beta bf16[T,Hv], g f32[T,Hv],
 *      conv_input bf16[K-1+T,D] (the concatenated window, keep_conv_input = true).
 * D = 2*Hk*Dk + Hv*Dv, Dk = Dv = 128. The next conv state is rows [T, T+K-1) of
 * conv_input, or rows [keep, keep+K-1) after a rollback (qwen3_5.rs:324-348). */
ORNITH_API int ornith_gdn_front(ornith_ctx* ctx, const void* d_conv_state, const void* d_qkv,
                                const void* d_cw, const void* d_a, const void* d_b,
                                const void* d_a_log, const void* d_dt_bias, int T, int K, int Hk,
                                int Dk, int Hv, int Dv, float eps, void* d_q, void* d_k, void* d_v,
                                void* d_beta, float* d_g, void* d_conv_input);
/* gdn::gated_delta_kernel_into stepped per token as GatedDeltaNet::forward_capture does
 * (src/ops/gdn.rs:131-271, kernels/gated_delta.metal:36-142, qwen3_5.rs:650-677):
 * state_in f32[Hv,Dv,Dk] -> y bf16[T,Hv,Dv] and one state snapshot per token,
 * d_snapshots f32[T][Hv,Dv,Dk]; snapshot T-1 is the new state, snapshot keep-1 is
 * the state to continue from after accepting keep tokens. With snapshot_every_token == 0
 * (plain forward, no rollback wanted) only the final state is written, to slot 0.
 * d_snapshots may alias d_state_in: a lane reads its state elements before it writes. */
ORNITH_API int ornith_gdn_recurrence(ornith_ctx* ctx, const void* d_q, const void* d_k,
                                     const void* d_v, const float* d_g, const void* d_beta,
                                     const float* d_state_in, int T, int Hk, int Hv, int Dk, int Dv,
                                     void* d_y, float* d_snapshots, int snapshot_every_token);

/* The core of GatedDeltaNet::forward / forward_capture between the big projections
 * (src/model/qwen3_5.rs:493-560, 650-677) in one launch, T <= 16: in_proj_a / in_proj_b
 * (dense bf16 weights d_wa / d_wb [Hv, H] applied to d_xn [T, H]; or pass the projections
 * d_a / d_b [T, Hv] and null weights), gdn_front, the recurrence with its per-token state
 * snapshots, and rms_norm_gated against d_z -> d_gated_out [T, Hv*Dv]. One workgroup per
 * value head keeps q, k, v, g, beta and y in LDS. Bit-identical to the separate calls. */
ORNITH_API int ornith_gdn_step(ornith_ctx* ctx, const void* d_conv_state, const void* d_qkv,
                               const void* d_cw, const void* d_a, const void* d_b, const void* d_wa,
                               const void* d_wb, const void* d_xn, int H, const void* d_a_log,
                               const void* d_dt_bias, int T, int K, int Hk, int Dk, int Hv, int Dv,
                               float eps, const float* d_state_in, float* d_snapshots,
                               int snapshot_every_token, const void* d_norm_w, const void* d_z,
                               float norm_eps, void* d_conv_input, void* d_gated_out);

/* ---- full-attention layer at decode / verify width ------------------------------ */
/* ops::rope tables (src/ops/rope.rs:6-60): cos/sin f32 [npos, dims/2] for
 * inv_freq_i = theta^(-i/(dims/2)), computed in double on the host and uploaded. */
ORNITH_API int ornith_rope_table(ornith_ctx* ctx, int npos, int dims, double theta, float* d_cos,
                                 float* d_sin);
/* Attention::forward up to the cache write (src/model/qwen3_5.rs:439-463): per-head
 * rms_norm of q and k (weights [hd]), partial RoPE at position offset + t, append of
 * K and V at rows [offset, offset+T) of the caches bf16 [Hkv, cap, hd]
 * (KvCache::update_and_fetch, src/model/cache.rs:38-79). qg is q_proj's output
 * [T, Hq, 2*hd] (query | gate), kx / vx are k_proj / v_proj outputs [T, Hkv, hd].
 * If d_offset is non-null the offset is read from device memory at run time. */
ORNITH_API int ornith_attn_prep(ornith_ctx* ctx, const void* d_qg, const void* d_kx, const void* d_vx,
                                const void* d_q_norm_w, const void* d_k_norm_w, int T, int Hq, int Hkv,
                                int hd, int rope_dims, float eps, const float* d_cos,
                                const float* d_sin, int table_npos, int offset, const int* d_offset,
                                int cap, void* d_q_rot, void* d_k_cache, void* d_v_cache);
/* sdpa::attention_with_cache + sigmoid_gate (src/ops/sdpa.rs:61-83, qwen3_5.rs:465-472):
 * query row t sees keys [0, offset + t]; out bf16 [T, Hq*hd] = sigmoid(gate) * attn. */
ORNITH_API int ornith_sdpa_decode_gated(ornith_ctx* ctx, const void* d_q_rot, const void* d_k_cache,
                                        const void* d_v_cache, const void* d_qg, int T, int Hq,
                                        int Hkv, int hd, int offset, const int* d_offset, int cap,
                                        float scale, void* d_out);
/* ornith_attn_prep followed by ornith_sdpa_decode_gated on the same rows, as Attention::forward
 * runs them (src/model/qwen3_5.rs:430-474), host-side offset: the same results and the same
 * cache contents; at decode widths (T <= 8, a context short enough for the one-workgroup-per-
 * block form) one launch does both -- every workgroup makes its query row and the call's new
 * key rows itself, and the caches are written as a side effect. d_q_rot is only written when
 * the prep runs as its own launch. */
ORNITH_API int ornith_attn_decode(ornith_ctx* ctx, const void* d_qg, const void* d_kx, const void* d_vx,
                                  const void* d_q_norm_w, const void* d_k_norm_w, int T, int Hq, int Hkv,
                                  int hd, int rope_dims, float eps, const float* d_cos, const float* d_sin,
                                  int table_npos, int offset, int cap, float scale, void* d_q_rot,
                                  void* d_k_cache, void* d_v_cache, void* d_out);
/* sdpa_unfused (src/ops/sdpa.rs:386-461) for the rows of a prompt chunk, with the same output
 * gate: causal flash attention on the matrix cores, head_dim 256. Same arguments as
 * sdpa_decode_gated (host-side offset only), which forwards to it from 32 rows up; agrees
 * with the exact kernel to rounding, not bit for bit. */
ORNITH_API int ornith_sdpa_prefill_gated(ornith_ctx* ctx, const void* d_q_rot, const void* d_k_cache,
                                         const void* d_v_cache, const void* d_qg, int T, int Hq, int Hkv,
                                         int hd, int offset, int cap, float scale, void* d_out);

/* ---- greedy selection: src/ops/sample.rs ------------------------------------------ */
/* greedy_token / the verify rows of generate_step_mtp (src/ops/sample.rs:134-147,
 * src/mtp_generate.rs:237-250): tokens[r] = argmax_i bf16(logits[r,i] - lse_r), lowest
 * index on ties; logits bf16 [rows, V]; d_lse (bf16 [rows]) may be null. */
ORNITH_API int ornith_greedy_rows(ornith_ctx* ctx, const void* d_logits, int rows, int V,
                                  uint32_t* d_tokens, void* d_lse);
/* ornith_greedy_rows for callers that cannot allocate (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc). No counterpart in the reference. Same
 * arguments and same results, bit for bit; its per-chunk partials live in a fixed 32 KiB
 * device array inside the library instead of the context's grow-only scratch block, so the
 * call reaches no hipMalloc / hipFree. Limits: rows <= 8, V <= 262144 (ORNITH_ERR_INVALID
 * beyond). Every call on one GPU shares that GPU's array: calls that overlap on one GPU
 * (two contexts, two streams) race; calls on one context are stream ordered and safe. */
ORNITH_API int ornith_greedy_rows_noalloc(ornith_ctx* ctx, const void* d_logits, int rows, int V,
                                          uint32_t* d_tokens, void* d_lse);
/* greedy_argmax_into (src/ops/sample.rs:174-191): argmax of the raw logits, the draft
 * chain's choice. */
ORNITH_API int ornith_argmax_rows(ornith_ctx* ctx, const void* d_logits, int rows, int V,
                                  uint32_t* d_out);

/* ---- weights: WeightStore (src/weights.rs:41-279) -------------------------------
 * A named-tensor store on the device. Names are the reference's
 * (language_model.model.layers.N.linear_attn.in_proj_qkv.weight, ...). A module
 * <path> is k-quant if it has <path>.dm (Q4_K when scales are 12 bytes a block,
 * Q6_K when 16; .weight may be u32 or u8, same bytes), 8-bit affine if it has
 * <path>.biases, dense bf16 otherwise -- the same three-way dispatch as
 * WeightStore::linear (src/weights.rs:179-184). */
#define ORNITH_DT_F32 0
#define ORNITH_DT_BF16 1
#define ORNITH_DT_F16 2
#define ORNITH_DT_U8 3
#define ORNITH_DT_U32 4
#define ORNITH_DT_I32 5
/* dtypes a safetensors header may name besides those above; no kernel consumes them */
#define ORNITH_DT_I8 6
#define ORNITH_DT_I16 7
#define ORNITH_DT_U16 8
#define ORNITH_DT_I64 9
#define ORNITH_DT_U64 10
#define ORNITH_DT_F64 11
#define ORNITH_DT_BOOL 12
typedef struct ornith_weights ornith_weights;
ORNITH_API int ornith_weights_create(ornith_ctx* ctx, ornith_weights** out);
/* WeightStore::tensor: copies host_data to the device and records it under `name`. */
ORNITH_API int ornith_weights_put(ornith_weights* ws, const char* name, int dtype,
                                  const int64_t* shape, int ndim, const void* host_data);
ORNITH_API int ornith_weights_destroy(ornith_weights* ws);
/* number of tensors held and their total bytes (the loader's report, src/main.rs:483-488) */
ORNITH_API int ornith_weights_stats(const ornith_weights* ws, int64_t* n_tensors, int64_t* bytes);

/* ---- artifact files: SafeTensors (src/safetensors.rs:196-310) ---------------------
 * Host only: maps each shard read-only, parses and validates its JSON header (dtype,
 * shape, data_offsets against the file length). `data` pointers stay valid until close. */
typedef struct ornith_safetensors ornith_safetensors;
/* SafeTensors::open_many (src/safetensors.rs:204-210): later files win a repeated name. */
ORNITH_API int ornith_safetensors_open(const char* const* paths, int n_paths,
                                       ornith_safetensors** out);
/* shards_from_index (src/safetensors.rs:296-310): the shards model.safetensors.index.json's
 * weight_map names, sorted and de-duplicated, then `extra` (the MTP sidecar file). */
ORNITH_API int ornith_safetensors_open_model(const char* model_dir, const char* const* extra,
                                             int n_extra, ornith_safetensors** out);
ORNITH_API int ornith_safetensors_close(ornith_safetensors* st);
ORNITH_API int ornith_safetensors_count(const ornith_safetensors* st, int64_t* n_tensors,
                                        int64_t* n_files);
/* SafeTensors::names (src/safetensors.rs:283-285), in sorted order */
ORNITH_API int ornith_safetensors_name(const ornith_safetensors* st, int64_t i, const char** name);
/* SafeTensors::{get, bytes} (src/safetensors.rs:275-281); shape has room for 8 dims */
ORNITH_API int ornith_safetensors_info(const ornith_safetensors* st, const char* name, int* dtype,
                                       int64_t* shape, int* ndim, const void** data,
                                       size_t* nbytes);

/* config.json's `quantization` block (src/weights.rs:46-80): top-level group_size / bits /
 * mode (absent mode = affine) with per-module overrides; mode strings as
 * QuantMode::from_config (src/ops/quantized.rs:60-75). nvfp4 / mxfp4 / mxfp8 are
 * ORNITH_ERR_UNSUPPORTED. */
#define ORNITH_QM_AFFINE 0
#define ORNITH_QM_Q4K 1
#define ORNITH_QM_Q6K 2
/* WeightStore::quant_config (src/weights.rs:96-98) straight from <model_dir>/config.json */
ORNITH_API int ornith_quant_config_load(const char* model_dir, const char* module_path,
                                        int* group_size, int* bits, int* mode);
/* WeightStore::open (src/weights.rs:41-80): the indexed shards plus `extra` files and the
 * quantization block. Tensors are copied to the device the first time a loader asks for
 * them (WeightStore::tensor, src/weights.rs:101-108), so only what the model uses is
 * resident. With a quantization block present, ornith_model_load / ornith_mtp_load check
 * each module's tensors against its configured mode (src/weights.rs:132-150, 199-220). The
 * MTP head's numbered experts.N.* tensors are stacked on load (stacked_experts,
 * src/weights.rs:237-279). */
ORNITH_API int ornith_weights_open(ornith_ctx* ctx, const char* model_dir,
                                   const char* const* extra, int n_extra, ornith_weights** out);
ORNITH_API int ornith_weights_quant_config(const ornith_weights* ws, const char* module_path,
                                           int* group_size, int* bits, int* mode);
/* WeightStore::has (src/weights.rs:82-84): 1 if resident or in a mapped shard, else 0 */
ORNITH_API int ornith_weights_has(const ornith_weights* ws, const char* name);
/* WeightStore::tensor followed by a copy back: dtype / shape of `name` and, when host_out is
 * not NULL, its bytes (host_bytes must equal the tensor's size). */
ORNITH_API int ornith_weights_fetch(const ornith_weights* ws, const char* name, int* dtype,
                                    int64_t* shape, int* ndim, void* host_out, size_t host_bytes);

/* TextConfig (src/model/config.rs:46-134), the fields this path reads. */
typedef struct ornith_text_config {
  int hidden_size, num_hidden_layers, vocab_size;
  int num_experts, num_experts_per_tok, moe_intermediate_size, shared_expert_intermediate_size;
  int linear_num_key_heads, linear_num_value_heads, linear_key_head_dim, linear_value_head_dim;
  int linear_conv_kernel_dim;
  int num_attention_heads, num_key_value_heads, head_dim, rope_dims;
  int full_attention_interval; /* layer i is full attention iff (i+1) % interval == 0 */
  int norm_topk_prob;
  float rms_norm_eps;
  double rope_theta;
} ornith_text_config;

/* ---- model: TextModel (src/model/qwen3_5.rs:102-279), caches (src/model/cache.rs) */
typedef struct ornith_model ornith_model;
typedef struct ornith_caches ornith_caches;
/* TextModel::load: resolves every tensor by name; the store must outlive the model. */
ORNITH_API int ornith_model_load(ornith_ctx* ctx, const ornith_weights* ws,
                                 const ornith_text_config* cfg, ornith_model** out);
/* TextConfig::load (src/model/config.rs:46-133): <model_dir>/config.json, keys under
 * `text_config` when present; rope settings from `rope_parameters`; mtp_layers (may be NULL)
 * receives num_nextn_predict_layers. Host only. */
ORNITH_API int ornith_text_config_load(const char* model_dir, ornith_text_config* out,
                                       int* mtp_layers);
ORNITH_API int ornith_model_destroy(ornith_model* m);
/* Rows one forward call may carry (default 16: decode, verify, short prompt chunks). The
 * reference prefills in chunks of prefill_step_size (2048, src/generate.rs:90-136); raise
 * this before creating caches to prefill in chunks that wide (16 .. 8192 rows). From 32
 * rows up the k-quant projections and the MoE experts run as matrix-core GEMMs. */
ORNITH_API int ornith_model_set_max_rows(ornith_model* m, int rows);
/* The MoE block of decoder layer `layer` as the model holds it (pointers into the weight
 * store, valid while the model lives): lets a caller run or time ornith_moe_block /
 * ornith_moe_experts on the resident weights (the reference reaches them as
 * model.layers[i].mlp, src/model/qwen3_5.rs:261-283). */
ORNITH_API int ornith_model_moe_weights(const ornith_model* m, int layer, ornith_moe_weights* out);
/* make_cache: one KvCache (bf16 [Hkv, capacity, hd] x2) or GdnCache (conv window +
 * fp32 state with max_window snapshot slots) per layer. `capacity` is where the KV tensors
 * start; a forward that needs more rows grows them, as KvCache::update_and_fetch does
 * (src/model/cache.rs:38-79): to a multiple of 256 rows, at least half as large again as
 * before, rows [0, offset) carried over (the stream is synchronised and device memory is
 * allocated and freed at that moment). A caller that must not allocate inside its loop
 * reserves up front (ornith_caches_reserve) or fixes the capacity
 * (ornith_caches_set_growable(c, 0)): ornith_generate / ornith_mtp_generate then refuse, before
 * any token is handed out, a run whose prompt + max_tokens (+ depth) rows cannot fit, and a
 * forward past the capacity is an error. */
ORNITH_API int ornith_caches_create(ornith_model* m, int capacity, int max_window,
                                    ornith_caches** out);
ORNITH_API int ornith_caches_reserve(ornith_caches* c, int rows);
ORNITH_API int ornith_caches_set_growable(ornith_caches* c, int growable);
ORNITH_API int ornith_caches_capacity(const ornith_caches* c, int* capacity_out);
ORNITH_API int ornith_caches_reset(ornith_caches* c);
ORNITH_API int ornith_caches_destroy(ornith_caches* c);
ORNITH_API int ornith_caches_offset(const ornith_caches* c, int* offset_out);
/* TextModel::forward_hidden (capture = 0) / forward_capture (capture = 1): T tokens
 * (device u32) through the trunk; writes the post-norm hidden rows bf16 [T, H] and
 * advances the caches by T. With capture, T <= max_window and every gated-delta layer
 * keeps a state snapshot per token so ornith_model_rewind can take rows back. */
ORNITH_API int ornith_model_forward(ornith_model* m, ornith_caches* c, const uint32_t* d_tokens, int T,
                                    int capture, void* d_hidden_out);
/* TrunkCapture::rewind (src/model/qwen3_5.rs:324-348): after a captured forward of T
 * tokens keep only the first `keep` (1 <= keep <= T). Pointer moves only. */
ORNITH_API int ornith_model_rewind(ornith_model* m, ornith_caches* c, int keep);
/* lm_head.matmul: hidden bf16 [T, H] -> logits bf16 [T, vocab]. */
ORNITH_API int ornith_model_logits(ornith_model* m, const void* d_hidden, int T, void* d_logits);

/* ---- FR-Spec: FrSpec (src/frspec.rs:38-158) ----------------------------------------- */
typedef struct ornith_frspec ornith_frspec;
/* FrSpec::load: file = u32 n, then n x u32 LE; rejects n == 0, n >= vocab, ids out of
 * range, duplicates. FrSpec::prune: row-gathers lm_head's tensors into an n-row head. */
ORNITH_API int ornith_frspec_load(ornith_model* m, const char* path, ornith_frspec** out);
/* frspec::default_path (src/frspec.rs:153-158): $ORNITH_FRSPEC, else
 * <$ORNITH_REFS or "refs">/frspec/ids_64k.bin. ornith_frspec_load(m, NULL, ..) reads from there. */
ORNITH_API int ornith_frspec_default_path(char* buf, size_t len);
/* The list file on the host (src/frspec.rs:101-117; tools/merge_frspec.py:74-92). read: ids in
 * file order, *n_out their number (ids_out == NULL only asks for it); write: sorted and
 * de-duplicated, refusing an empty list, one that is not a strict pruning of `vocab`, or an id
 * outside it. */
ORNITH_API int ornith_frspec_read_ids(const char* path, uint32_t* ids_out, size_t cap, size_t* n_out);
ORNITH_API int ornith_frspec_write_ids(const char* path, const uint32_t* ids, size_t n, uint32_t vocab,
                                       size_t* n_written);
/* The superset merge of tools/merge_frspec.py:176-204 on token ids: merged = base + every id the
 * corpus (a token-id stream) used at least min_count times and base lacks + `extra` (e.g. every
 * id of one script), sorted and de-duplicated. It only adds, so coverage of what the base list
 * covered is unchanged by construction. out == NULL only computes the statistics. */
typedef struct ornith_frspec_merge_stats {
  size_t n_merged;         /* ids in the merged list */
  size_t corpus_tokens;    /* tokens in the corpus */
  size_t covered_before;   /* of them inside the base list */
  size_t covered_after;    /* inside the merged list, corpus additions only (the script's count apart) */
  size_t missing_distinct; /* distinct corpus ids the base lacks */
  size_t missing_kept;     /* of them seen >= min_count times */
  size_t extra_new;        /* distinct extra ids the base lacks */
} ornith_frspec_merge_stats;
ORNITH_API int ornith_frspec_merge(const uint32_t* base, size_t n_base, const uint32_t* corpus, size_t n_corpus,
                                   uint32_t min_count, const uint32_t* extra, size_t n_extra, uint32_t vocab,
                                   uint32_t* out, size_t out_cap, ornith_frspec_merge_stats* stats);
ORNITH_API int ornith_frspec_from_ids(ornith_model* m, const uint32_t* ids, int n, ornith_frspec** out);
ORNITH_API int ornith_frspec_destroy(ornith_frspec* f);
/* the pruned head as a Linear (for tests: pruned row == original row) and its size */
ORNITH_API int ornith_frspec_head(const ornith_frspec* f, ornith_linear* head_out, int* n_out);

/* ---- MTP head: MtpHead (src/model/mtp.rs:96-268) ----------------------------------- */
typedef struct ornith_mtp_head ornith_mtp_head;
/* MtpHead::load from the mtp.* tensors (dense bf16); owns a one-layer KV cache. */
ORNITH_API int ornith_mtp_load(ornith_model* m, const ornith_weights* ws, int capacity,
                               ornith_mtp_head** out);
ORNITH_API int ornith_mtp_destroy(ornith_mtp_head* h);
/* MtpHead::hidden / forward: T rows of trunk hidden + the T token ids that follow them
 * -> post-norm hidden bf16 [T, H] (and, if d_logits != null, logits through the pruned
 * head when `frspec` != null, else through lm_head). Appends T rows to the head's cache. */
ORNITH_API int ornith_mtp_forward(ornith_mtp_head* h, const ornith_frspec* frspec,
                                  const void* d_trunk_hidden, const uint32_t* d_next_ids, int T,
                                  void* d_hidden_out, void* d_logits);
ORNITH_API int ornith_mtp_cache_set_offset(ornith_mtp_head* h, int offset);
/* the head's one-layer KV cache grows like the trunk's (see ornith_caches_create) */
ORNITH_API int ornith_mtp_cache_reserve(ornith_mtp_head* h, int rows);
ORNITH_API int ornith_mtp_cache_set_growable(ornith_mtp_head* h, int growable);
ORNITH_API int ornith_mtp_cache_offset(const ornith_mtp_head* h, int* offset_out);
/* Measurement aid, no counterpart in the reference: a host list g[0..n) of the tokens a run
 * is known to produce (g[0] = the first token after the prompt, e.g. the plain greedy output).
 * While set, ornith_mtp_generate still runs the head for every draft but then replaces the
 * draft for output position p with g[p], so every draft inside the list is accepted and a
 * cycle yields depth + 1 tokens: the throughput ceiling of the loop at that depth. n = 0
 * clears the list. Positions past the list keep the head's own drafts. */
ORNITH_API int ornith_mtp_force_drafts(ornith_mtp_head* h, const uint32_t* tokens, size_t n);

/* ---- the sampled-token path: TopSampler (src/sample.rs:79-225) -------------------------
 * bf16 throughout except the CDF, as in the reference. Cumulative sums associate in
 * chunks of 1024 / segments of 64 (see csrc/sampler.hip); sorts are stable. */
/* random::key / KeySequence::next / random::bits (src/ops/random.rs:16-67; threefry2x32 of
 * vendored random.metal:5-66). Host functions: the key sequence is 64 bits of integer state. */
ORNITH_API void ornith_random_key(uint64_t seed, uint32_t key_out[2]);
ORNITH_API int ornith_random_split(uint32_t key_state[2], uint32_t sub_out[2]);
ORNITH_API int ornith_random_bits(const uint32_t key[2], int n, uint32_t* out);
/* ops::sort::argsort_last_axis over one row of bf16 (negate != 0: of the negated values,
 * as apply_top_k asks): the stable ascending order as u32 indices. */
ORNITH_API int ornith_argsort_bf16(ornith_ctx* ctx, const void* d_x, int n, int negate,
                                   uint32_t* d_idx_out);
/* ops::scan::cumsum_last_axis, inclusive, one row; dtype ORNITH_BF16 accumulates in bf16. */
ORNITH_API int ornith_cumsum(ornith_ctx* ctx, const void* d_x, int dtype, int n, void* d_out);
/* apply_top_p (src/sample.rs:79-115), apply_top_k (:117-136): bf16 logprobs [V] -> bf16 [V]
 * with the dropped entries at -inf. d_out must not alias the input. */
ORNITH_API int ornith_apply_top_p(ornith_ctx* ctx, const void* d_logprobs, int V, double top_p,
                                  void* d_out);
ORNITH_API int ornith_apply_top_k(ornith_ctx* ctx, const void* d_logprobs, int V, int top_k,
                                  void* d_out);
/* categorical_sampling (src/sample.rs:138-190) with the raw 32-bit random word given:
 * writes the drawn index to d_token_out. */
ORNITH_API int ornith_categorical(ornith_ctx* ctx, const void* d_logprobs, int V, double temp,
                                  uint32_t raw_bits, uint32_t* d_token_out);
/* TopSampler (src/sample.rs:192-225): log-softmax of one row of logits, top-p if
 * 0 < top_p < 1, top-k if top_k > 0, one draw; every sample consumes one split of the key. */
typedef struct ornith_top_sampler ornith_top_sampler;
ORNITH_API int ornith_top_sampler_create(ornith_ctx* ctx, double temp, double top_p, int top_k,
                                         uint64_t seed, int vocab, ornith_top_sampler** out);
ORNITH_API int ornith_top_sampler_destroy(ornith_top_sampler* s);
ORNITH_API int ornith_top_sampler_sample(ornith_top_sampler* s, const void* d_logits_row,
                                         uint32_t* d_token_out);

/* Which generator a TopSampler draws its random words from (default ORNITH_RNG_THREEFRY), and
 * the next raw word of its stream (one key split, or one Philox counter value, per word). */
ORNITH_API int ornith_top_sampler_set_rng(ornith_top_sampler* s, int rng);
ORNITH_API int ornith_top_sampler_next_bits(ornith_top_sampler* s, uint32_t* bits_out);
/* Philox4x32-10 (Salmon et al., SC'11; Random123's philox4x32 at 10 rounds): host function. */
ORNITH_API void ornith_philox4x32_10(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4]);

/* ---- speculative sampling: no counterpart in the reference, which accepts drafts by token
 * equality only and says so (src/mtp_generate.rs:27-35). A distribution is carried as
 * unnormalised fp32 weights w[0..V) with their total in w[V] (V + 1 floats on the device);
 * the probabilities are w[i] / w[V]. ---------------------------------------------------- */
/* The distribution TopSampler draws from for one row of logits (log-softmax, top-p, top-k,
 * temperature: src/sample.rs:79-190) as such weights. Consumes no random word. */
ORNITH_API int ornith_sampler_weights(ornith_top_sampler* s, const void* d_logits_row, int V, float* d_w);
/* inverse-CDF draw from such weights with the raw random word given (the draw of
 * categorical_sampling, src/sample.rs:138-190, on weights already made) */
ORNITH_API int ornith_draw_weights(ornith_ctx* ctx, const float* d_w, int V, uint32_t raw_bits,
                                   uint32_t* d_token_out);
/* weights over a pruned draft vocabulary (n entries, d_ids their vocabulary ids) placed in
 * vocabulary space: zero off the list */
ORNITH_API int ornith_spec_scatter(ornith_ctx* ctx, const float* d_w_local, const uint32_t* d_ids, int n,
                                   int V, float* d_w_full);
/* the draft token *d_x was drawn from q: *d_accept_out = (u * q(x) < p(x)), u uniform in [0, 1)
 * from raw_bits, i.e. acceptance with probability min(1, p(x) / q(x)) */
ORNITH_API int ornith_spec_accept(ornith_ctx* ctx, const float* d_wp, const float* d_wq, int V,
                                  const uint32_t* d_x, uint32_t raw_bits, uint32_t* d_accept_out);
/* the token for a rejected position: a draw from norm(max(0, p - q)); from p if that is empty */
ORNITH_API int ornith_spec_resample(ornith_ctx* ctx, const float* d_wp, const float* d_wq, int V,
                                    uint32_t raw_bits, uint32_t* d_token_out);

/* ---- generation loops ---------------------------------------------------------------- */
/* Sampler (src/generate.rs:36-64, src/sample.rs:205-225). rows_are_independent is
 * true for GREEDY. */
#define ORNITH_SAMPLER_GREEDY 0
#define ORNITH_SAMPLER_TOP_P 1
/* how generate_step_mtp decides on a draft under a sampling sampler */
#define ORNITH_ACCEPT_EQUALITY 0 /* the reference's rule: the target's own sample must equal the draft
                                    (src/mtp_generate.rs:27-35, 255-279); drafts are the head's argmax */
#define ORNITH_ACCEPT_RATIO 1    /* speculative sampling, which the reference names as not carried
                                    (src/mtp_generate.rs:27-30): drafts are drawn from the head's
                                    distribution q, accepted with probability min(1, p/q), and a
                                    rejected position is redrawn from norm(max(0, p - q)) */
/* where the sampler's random words come from */
#define ORNITH_RNG_THREEFRY 0 /* the reference's key sequence (src/ops/random.rs:16-67) */
#define ORNITH_RNG_PHILOX 1   /* Philox4x32-10: draw n of a seed is word 0 of
                                 philox(counter = (n, 0, 0, 0) as 64 + 64 bits, key = seed) */
typedef struct ornith_sampler {
  int kind;
  double temperature, top_p; /* as TopSampler::new(f64, f64, ..) takes them (src/sample.rs:205-225) */
  int top_k;
  uint64_t seed;
  int accept; /* ORNITH_ACCEPT_*; ignored by GREEDY and by generate_step */
  int rng;    /* ORNITH_RNG_* */
} ornith_sampler;
/* on_token: return 0 to stop (FnMut(u32) -> bool); progress: (done, total) prompt tokens */
typedef int (*ornith_token_cb)(uint32_t token, void* user);
typedef void (*ornith_progress_cb)(size_t done, size_t total, void* user);

/* generate::generate_step (src/generate.rs:162-206): prefill all but the last prompt
 * token in chunks of prefill_step, then one step per token; the caches end holding the
 * prompt plus exactly the tokens shown to on_token. */
ORNITH_API int ornith_generate(ornith_model* m, ornith_caches* c, const uint32_t* prompt, size_t n_prompt,
                               const ornith_sampler* sampler, size_t max_tokens, size_t prefill_step,
                               ornith_progress_cb progress, ornith_token_cb on_token, void* user);

#define ORNITH_HISTORY_CYCLE 0     /* HistoryPolicy::Cycle */
#define ORNITH_HISTORY_COMMITTED 1 /* HistoryPolicy::Committed (the CLI default) */
#define ORNITH_MAX_DEPTH 8
typedef struct ornith_mtp_stats { /* MtpStats (src/mtp_generate.rs:66-84) */
  size_t cycles, drafted, accepted;
  size_t reached_by_depth[ORNITH_MAX_DEPTH], accepted_by_depth[ORNITH_MAX_DEPTH];
} ornith_mtp_stats;
/* mtp_generate::generate_step_mtp (src/mtp_generate.rs:150-317): draft `depth` tokens
 * with the MTP head (through the FR-Spec head if frspec != null), verify depth+1 rows in
 * one trunk forward, accept the leading run of equal tokens, rewind, repeat. */
ORNITH_API int ornith_mtp_generate(ornith_model* m, ornith_mtp_head* head, const ornith_frspec* frspec,
                                   ornith_caches* c, const uint32_t* prompt, size_t n_prompt,
                                   const ornith_sampler* sampler, int depth, size_t max_tokens,
                                   size_t prefill_step, int policy, ornith_progress_cb progress,
                                   ornith_token_cb on_token, void* user, ornith_mtp_stats* stats_out);

/* ---- text in, text out: tokenizer, streaming detokenizer, chat template (host only) ----
 * The callers' side of the loops (src/main.rs:651-741): a prompt is rendered by the chat
 * template, encoded, generated from, and the tokens handed to on_token go through the
 * detokenizer. Nothing here touches the GPU. Strings are UTF-8 with explicit lengths (no
 * terminator needed or written). Every function that returns text or a list takes a buffer,
 * its capacity and a count pointer: with a NULL buffer it only reports the size needed. */
typedef struct ornith_tokenizer ornith_tokenizer;
typedef struct ornith_detokenizer ornith_detokenizer;
/* split::Dialect (src/tokenizer/split.rs:55-78): which of the two split patterns runs */
#define ORNITH_DIALECT_TOKENIZER_JSON 0 /* the pattern tokenizer.json carries, \p{M} beside \p{L} */
#define ORNITH_DIALECT_TRANSFORMERS 1   /* transformers' PRETOKENIZE_REGEX, without \p{M} */
/* Tokenizer::load / load_as (src/tokenizer/mod.rs:78-259): reads tokenizer.json,
 * tokenizer_config.json (added tokens only the config knows, eos_token) and, when present,
 * generation_config.json (eos_token_id). A file that asks for a pipeline other than
 * NFC -> Split(the pattern, Isolated) + ByteLevel -> BPE without dropout / unk / fallback is
 * refused (ORNITH_ERR_UNSUPPORTED) where the reference asserts. */
ORNITH_API int ornith_tokenizer_load(const char* model_dir, int dialect, ornith_tokenizer** out);
ORNITH_API int ornith_tokenizer_destroy(ornith_tokenizer* tk);
/* Tokenizer::vocab_size (mod.rs:261-263): ids the tokenizer has a string for, added ones included */
ORNITH_API int ornith_tokenizer_vocab_size(const ornith_tokenizer* tk, size_t* n_out);
/* Tokenizer::encode (mod.rs:279-308): tokenizer.encode(text, add_special_tokens=False).
 * The text must be valid UTF-8 (ORNITH_ERR_INVALID otherwise; the reference takes &str). */
ORNITH_API int ornith_tokenizer_encode(const ornith_tokenizer* tk, const char* text, size_t text_len,
                                       uint32_t* ids_out, size_t cap, size_t* n_out);
/* Tokenizer::decode (mod.rs:330-346): ByteLevel decoding, ill-formed bytes as U+FFFD */
ORNITH_API int ornith_tokenizer_decode(const ornith_tokenizer* tk, const uint32_t* ids, size_t n, char* out,
                                       size_t cap, size_t* n_out);
/* Tokenizer::token (mod.rs:349-355): the token string of an id; "!" for an id past the entries */
ORNITH_API int ornith_tokenizer_token(const ornith_tokenizer* tk, uint32_t id, char* out, size_t cap,
                                      size_t* n_out);
/* Tokenizer::id (mod.rs:265-271): token is NUL-terminated; ORNITH_ERR_INVALID when absent */
ORNITH_API int ornith_tokenizer_id(const ornith_tokenizer* tk, const char* token, uint32_t* id_out);
/* Tokenizer::is_special (mod.rs:273-275): 1 / 0 */
ORNITH_API int ornith_tokenizer_is_special(const ornith_tokenizer* tk, uint32_t id);
/* Tokenizer::eos_ids (mod.rs:230-247) */
ORNITH_API int ornith_tokenizer_eos_ids(const ornith_tokenizer* tk, uint32_t* ids_out, size_t cap,
                                        size_t* n_out);
/* The pattern string a dialect spells (Dialect::TOKENIZER_JSON_PATTERN / TRANSFORMERS_PATTERN) */
ORNITH_API const char* ornith_tokenizer_split_pattern(int dialect);
/* Detokenizer (mod.rs:352-417, mlx-lm's BPEStreamingDetokenizer with its two quirks: the single
 * leading space of a generation is dropped; the character standing for byte 0 is emitted as
 * itself while streaming). add_token holds back an unfinished UTF-8 sequence and a lone space;
 * last_segment returns (and, with a buffer, consumes) the text made since its last call. */
ORNITH_API int ornith_detokenizer_create(const ornith_tokenizer* tk, ornith_detokenizer** out);
ORNITH_API int ornith_detokenizer_destroy(ornith_detokenizer* d);
ORNITH_API int ornith_detokenizer_add_token(ornith_detokenizer* d, uint32_t token);
ORNITH_API int ornith_detokenizer_finalize(ornith_detokenizer* d);
ORNITH_API int ornith_detokenizer_last_segment(ornith_detokenizer* d, char* out, size_t cap, size_t* n_out);
ORNITH_API int ornith_detokenizer_text(const ornith_detokenizer* d, char* out, size_t cap, size_t* n_out);
/* The tokenizer's layers one by one, as the reference's tests reach them (tests/tokenizer.rs):
 * nfc::nfc (src/tokenizer/nfc.rs:121-170); split::pre_split (split.rs:134-153: the byte offset
 * at which each piece ends); the class the split pattern puts a code point in (1 letter or
 * mark, 2 number, 3 white space, 0 other; split.rs:100-118). */
ORNITH_API int ornith_text_nfc(const char* text, size_t n, char* out, size_t cap, size_t* n_out);
ORNITH_API int ornith_text_pre_split(const char* text, size_t n, int dialect, size_t* ends_out, size_t cap,
                                     size_t* n_out);
ORNITH_API int ornith_text_char_class(uint32_t code_point);
/* chat::apply_chat_template (src/chat.rs:196-352): the artifact's chat template written out as
 * code. messages_json: the list tokenizer.apply_chat_template takes, [{"role": "system" |
 * "user" | "assistant" | "tool", "content": string | [{"type": "text" | "image" | "video", ...}]
 * | null, "reasoning_content"?, "tool_calls"?: [{"function"?: {"name", "arguments": {...}}}]}];
 * tools_json: a list of tool schemas, or NULL / empty for none. The template's own errors
 * ("No messages provided.", "No user query found in messages.", "System message must be at
 * the beginning.", "System message cannot contain images." / "videos.") come back as
 * ORNITH_ERR_INVALID with that text. */
ORNITH_API int ornith_chat_apply_template(const char* messages_json, size_t messages_len, const char* tools_json,
                                          size_t tools_len, int add_generation_prompt, int enable_thinking,
                                          char* out, size_t cap, size_t* n_out);
/* json::Value::to_json (src/json.rs): json.dumps(value, ensure_ascii=False) of a JSON text,
 * keys in their written order - what the template's tojson filter produces. */
ORNITH_API int ornith_json_dumps(const char* json, size_t len, char* out, size_t cap, size_t* n_out);

/* ---- self test ------------------------------------------------------------------
 * Evaluates one of the library's scalar device functions element-wise (fp32 in,
 * fp32 out) so their bits can be compared with a CPU evaluation. No reference
 * counterpart: the reference calls Metal's math library
 * (kernels/ornith_sigmoid.h:27-31, ornith_logaddexp.h:12-23), whose last bits are not
 * reproducible off its device; this library carries its own. WAVE_SUM returns, in
 * every element, the 64-lane butterfly sum of its wavefront (n must be a multiple of 64). */
#define ORNITH_FN_EXP 0
#define ORNITH_FN_LOG 1
#define ORNITH_FN_LOG1P 2
#define ORNITH_FN_SIGMOID_BF16 3
#define ORNITH_FN_SIGMOID_F32 4
#define ORNITH_FN_RSQRT 5
#define ORNITH_FN_RECIP 6
#define ORNITH_FN_ROUND_BF16 7
#define ORNITH_FN_WAVE_SUM 8
/* 9 + i: the value of lane (l xor 2^i) of the 64-lane wavefront, i = 0..5 (n a multiple of 64) */
#define ORNITH_FN_XOR_LANE 9
ORNITH_API int ornith_selftest_unary(ornith_ctx* ctx, int fn, const float* d_in, float* d_out, int64_t n);

/* ---- machine probes (`bench.py --ceiling`) ------------------------------------------
 * No reference counterpart (the reference times its own dispatches from the host,
 * src/bin/dispatch.rs, Q4K.md:479-484); nothing on the decode path calls these. They price a
 * decode launch against the machine: all are enqueued on the context's stream and timed by
 * the caller with ornith_timer_begin / ornith_timer_end.
 * probe_empty: `launches` launches of a kernel that does nothing (with_args: it carries an
 * argument block the size of the expert kernel's). probe_stream: `launches` launches of
 * `workgroups` x 256 threads in which every thread reads `per_thread` (1..16) 16-byte pieces, a
 * wavefront's pieces 1 KB contiguous each and `stride_bytes` apart, all requested before any is
 * used: the expert launch's shape with none of its arithmetic; successive launches walk through
 * the buffer so that none finds its bytes cached. probe_read: one grid-stride read of the
 * whole buffer. probe_xcc: the XCC (die) id each of `workgroups` workgroups ran on, in launch
 * order. probe_handoff: workgroup `producer` writes a word 4 us into the launch, workgroup
 * `consumer` polls it (mode 0: plain store, agent-scope loads; 1: agent-scope store and loads;
 * 2: plain store and plain loads, which never see it); d_out4 receives four 64-bit words:
 * the 100 MHz clock at the store, at the observation (0: the bounded poll ran out), and the
 * two workgroups' XCC ids. d_flag must be zeroed by the caller. */
ORNITH_API int ornith_probe_empty(ornith_ctx* ctx, int workgroups, int threads, int with_args, int launches);
/* the same launches recorded into a HIP graph and replayed as one submission; *ms_out = the
 * replay's duration (the device's own launch-after-launch rate, no host enqueue in it) */
ORNITH_API int ornith_probe_empty_graph(ornith_ctx* ctx, int workgroups, int threads, int with_args, int launches,
                                        float* ms_out);
ORNITH_API int ornith_probe_stream(ornith_ctx* ctx, const void* d_src, size_t bytes, int workgroups, int per_thread,
                                   size_t stride_bytes, void* d_sink, int launches);
ORNITH_API int ornith_probe_read(ornith_ctx* ctx, const void* d_src, size_t bytes, void* d_sink);
ORNITH_API int ornith_probe_xcc(ornith_ctx* ctx, int workgroups, uint32_t* d_out);
ORNITH_API int ornith_probe_handoff(ornith_ctx* ctx, void* d_flag, void* d_out4, int producer, int consumer, int mode);
/* probe_valu: one launch of `workgroups` x 256 threads, every thread running 8 x `iters` of one
 * vector instruction (op 0 .. ornith_probe_valu_count() - 1, named by ornith_probe_valu_name):
 * what the instructions of the dequantizing mat-vecs cost each. d_x: 4 floats, d_p: 4 words,
 * d_out: workgroups x 256 floats. probe_kernarg: the same small kernel with its arguments in a
 * struct (flat = 0: read through a scalar load when the wavefront starts) or as leading flat
 * arguments (flat = 1: preloaded into scalar registers with the wavefront); every workgroup
 * stores four 64-bit stamps of the 100 MHz clock: entry, argument in a register, after a
 * dependent scalar load, after a dependent vector load. d_idx: one word below 256, d_data:
 * 64 KB, d_out: workgroups x 4 x int64. */
ORNITH_API int ornith_probe_valu_count(void);
ORNITH_API const char* ornith_probe_valu_name(int op);
ORNITH_API int ornith_probe_valu(ornith_ctx* ctx, int op, int workgroups, int iters, const void* d_x, const void* d_p,
                                 void* d_out);
ORNITH_API int ornith_probe_kernarg(ornith_ctx* ctx, int flat, int workgroups, const void* d_idx, const void* d_data,
                                    void* d_out);

#ifdef __cplusplus
}
#endif
#endif /* ORNITH_HIP_H */
