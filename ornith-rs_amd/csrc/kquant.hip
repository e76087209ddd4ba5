// Q4_K / Q6_K dequantize, mat-vec and expert gather mat-vec for gfx950.
//
// Replaces kquant::{dequantize,qmv,gather_qmv}
// (/root/reference/src/ops/kquant.rs:418-433,539-595,741-770) and the kernels
// they dispatch (/root/reference/kernels/q4k.metal:64-249,628-656,
// /root/reference/kernels/q6k.metal:47-169,365-393). The storage format is the
// reference's three tensors per matrix, untouched.
//
// Schedule (this build's own, for 64-lane wavefronts; bandwidth bound, no MFMA):
//   chunk j of a row belongs to lane j % 64 (see kq_device.h); rows narrower than
//   64 chunks pack 64/LPR rows into one wavefront (LPR lanes per row); rows wider
//   than 64 chunks are split over KS wavefronts whose lane partials are added
//   through LDS in ascending chunk order. Each lane keeps the activations of its
//   chunk in registers (they do not depend on the output row) and walks down the
//   rows, so the weight stream is the only traffic that scales with O.
//
//   The sum of a row is then: lane partials (ascending chunk), butterfly
//   v += v[l ^ s] for s = 32..1. Rows of a multi-token call are independent
//   accumulators over the same weights in the same order, which is what makes
//   row r of an M-row call bit-identical to that row alone (the property
//   /root/reference/src/ops/invariant.rs:88-116 buys with its exact window).
//
//   One launch can cover up to four matrices of the same format and width that
//   read the same activations (q/k/v projections, in_proj_qkv + in_proj_z): the
//   grid is the concatenation of their row ranges.
#include "kq_device.h"
#include "norm_device.h"
#include "rt.h"

namespace {

constexpr int kMaxSeg = 4;

struct KqSeg {
  const uint8_t* qs;
  const uint8_t* scales;
  const uint16_t* dm;
  void* y;
  int O;
  int first_block;
};

struct KqArgs {
  KqSeg seg[kMaxSeg];
  int nseg;
  const void* x;
  const uint32_t* lhs;  // gather only
  const uint32_t* rhs;  // gather only
  int K;
  int E, x_rows;  // gather only: bounds for rhs / lhs (out-of-range ids are clamped)
  int iters;      // row iterations per wavefront
  int y_bf16;     // 1: round outputs to bf16, 0: fp32
  PreNorm pre;    // PRE kernels: the activations are rms_norm(res + y) computed by every workgroup
};

#ifdef ORN_TIMING
// debug build only: per-workgroup phase time stamps (100 MHz wall clock) of the last launch
__device__ long long g_marks[4096][8];
#define ORN_MARK(i) do { if (threadIdx.x == 0 && blockIdx.x < 4096 && blockIdx.y == 0) g_marks[blockIdx.x][i] = wall_clock64(); } while (0)
extern "C" __attribute__((visibility("default"))) int ornith_debug_marks(long long* out, int blocks) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_marks), sizeof(long long) * 8 * blocks);
}
#else
#define ORN_MARK(i)
#endif

// One kernel for plain and gathered mat-vecs.
//   KIND  format; LPR lanes per row (4,8,16,32,64); KS wavefronts per row (1,2)
//   M     activation rows sharing each weight read (1..4); gather uses M == 1
//   grid.x covers output rows (of all segments), grid.y is the gather row
//   PRE   the activation rows are not read but made: every workgroup computes
//         h = res + y, x = rms_norm(h) of the M rows (K == 2048) into LDS while its weight
//         loads are in flight; workgroup 0 also stores h and x for later consumers
template <int KIND, int LPR, int KS, int M, bool XF32, bool GATHER, bool PRE = false>
__global__ __launch_bounds__(256) void kq_qmv_kernel(KqArgs a) {
  ORN_MARK(0);
  using KL = KqLane<KIND, M>;
  constexpr int RPW = 64 / LPR;  // rows in flight per wavefront
  constexpr int WPB = 4 / KS;    // row-wavefronts per block
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int slot = lane / LPR, c = lane % LPR;
  const int ks = (KS == 1) ? 0 : (wave & 1);
  const int rw = (KS == 1) ? wave : (wave >> 1);
  const int nb = a.K >> 8;

  // every segment's fields are fetched at once and one is selected: indexing the argument
  // array with a computed value would put a second scalar memory trip ahead of the first
  // weight load
  KqSeg sg = a.seg[0];
  {
    KqSeg all[kMaxSeg];
    int nseg = a.nseg;
    static_assert(kMaxSeg == 4, "the one statement below names every field");
    // pins the values (not their addresses) in scalar registers in ONE statement, so that all
    // the argument loads are issued together and waited for once (a statement per segment
    // made the compiler wait for each segment's loads before issuing the next's)
    uint64_t q[kMaxSeg], sc[kMaxSeg], d[kMaxSeg], y[kMaxSeg];
    int so[kMaxSeg], fb[kMaxSeg];
#pragma unroll
    for (int i = 0; i < kMaxSeg; ++i) {
      q[i] = (uint64_t)a.seg[i].qs;
      sc[i] = (uint64_t)a.seg[i].scales;
      d[i] = (uint64_t)a.seg[i].dm;
      y[i] = (uint64_t)a.seg[i].y;
      so[i] = a.seg[i].O;
      fb[i] = a.seg[i].first_block;
    }
    if constexpr (PRE) {
      // the norm's three input pointers ride along with the same batch of argument loads
      uint64_t pr = (uint64_t)a.pre.res, py = (uint64_t)a.pre.y, pw = (uint64_t)a.pre.w;
      asm volatile("" : "+s"(pr), "+s"(py), "+s"(pw));
      a.pre.res = dm_global_ptr<const bf16_t>(pr);
      a.pre.y = dm_global_ptr<const bf16_t>(py);
      a.pre.w = dm_global_ptr<const bf16_t>(pw);
    }
    asm volatile(""
                 : "+s"(q[0]), "+s"(sc[0]), "+s"(d[0]), "+s"(y[0]), "+s"(so[0]), "+s"(fb[0]), "+s"(q[1]), "+s"(sc[1]),
                   "+s"(d[1]), "+s"(y[1]), "+s"(so[1]), "+s"(fb[1]), "+s"(q[2]), "+s"(sc[2]), "+s"(d[2]), "+s"(y[2]),
                   "+s"(so[2]), "+s"(fb[2]), "+s"(q[3]), "+s"(sc[3]), "+s"(d[3]), "+s"(y[3]), "+s"(so[3]), "+s"(fb[3]),
                   "+s"(nseg), "+s"(a.K), "+s"(a.iters), "+s"(a.y_bf16));
#pragma unroll
    for (int i = 0; i < kMaxSeg; ++i) {
      all[i] = a.seg[i];
      all[i].qs = dm_global_ptr<const uint8_t>(q[i]);
      all[i].scales = dm_global_ptr<const uint8_t>(sc[i]);
      all[i].dm = dm_global_ptr<const uint16_t>(d[i]);
      all[i].y = dm_global_ptr<void>(y[i]);
      all[i].O = so[i];
      all[i].first_block = fb[i];
    }
    sg = all[0];
#pragma unroll
    for (int i = 1; i < kMaxSeg; ++i)
      if (i < nseg && (int)blockIdx.x >= all[i].first_block) sg = all[i];
  }
  const int O = sg.O;

  const size_t xsz = XF32 ? 4 : 2;
  const void* xrow[M];
  int64_t row0 = 0;  // first weight row of this matrix (expert offset)
  int64_t yrow0 = 0;
  if constexpr (GATHER) {
    const int r = blockIdx.y;
    const uint32_t xi = min(a.lhs[r], (uint32_t)(a.x_rows - 1));
    const uint32_t ei = min(a.rhs[r], (uint32_t)(a.E - 1));
    xrow[0] = static_cast<const char*>(a.x) + (size_t)xi * a.K * xsz;
    row0 = (int64_t)ei * O;
    yrow0 = (int64_t)r * O;
  } else {
#pragma unroll
    for (int t = 0; t < M; ++t) xrow[t] = static_cast<const char*>(a.x) + (size_t)t * a.K * xsz;
  }

  // Rows kept in flight per wavefront. Cold weights come from HBM with a latency many
  // times the arithmetic of one row, so every wavefront issues the loads of its first PF
  // rows at once (they depend on nothing), behind only the few cached operands named
  // below, and refills a slot as soon as that row's registers are consumed.
  constexpr int PF = (KIND == ORNITH_Q4K) ? (M <= 2 ? 4 : 2) : (M <= 2 ? 2 : 1);
  typename KL::Lane L;
  L.set_chunk(c + 64 * ks);

  __shared__ float part[(KS == 2) ? 2 * M * 64 : 1];

  const int rows_per_wave = RPW * a.iters;
  const int base = (((int)blockIdx.x - sg.first_block) * WPB + rw) * rows_per_wave;
  auto row_of = [&](int it) {
    const int o = base + it * RPW + slot;
    return row0 + (o < O ? o : O - 1);
  };
  // The rows the norm is made from are a few KB that sit in cache; their loads go out first
  // because loads return in issue order: behind the cold weight rows they would hold the
  // norm back until the weights had arrived.
  PreNormRegs<PRE ? M : 1> pg;
  if constexpr (PRE) {
    prenorm_issue<M>(a.pre, pg);
    __builtin_amdgcn_sched_barrier(0);
  }
  // activations from memory go first: loads return in issue order, so behind the weight rows the
  // (cached) activation rows and their conversion would wait for the last weight byte
  if constexpr (!PRE) {
    L.template load_x<XF32>(xrow, c + 64 * ks);
    __builtin_amdgcn_sched_barrier(0);
  }
  typename KL::Row pf[PF];
#pragma unroll
  for (int i = 0; i < PF; ++i) pf[i] = KL::load(sg.qs, sg.scales, sg.dm, row_of(i), nb, L);
  __builtin_amdgcn_sched_barrier(0);  // keep the weight loads ahead of everything that follows
  ORN_MARK(1);
  if constexpr (PRE) {
    __shared__ PreNormLds<M> pn;
    prenorm_finish<M>(a.pre, pg, blockIdx.x == 0, pn);
#pragma unroll
    for (int t = 0; t < M; ++t) xrow[t] = &pn.xn[t][0];
  }
  ORN_MARK(2);
  if constexpr (PRE) L.template load_x<XF32>(xrow, c + 64 * ks);  // from the normed rows in LDS
  ORN_MARK(3);

  for (int it0 = 0; it0 < a.iters; it0 += PF) {
#pragma unroll
   for (int i = 0; i < PF; ++i) {
    const int it = it0 + i;
    if (it >= a.iters) break;
    const int o = base + it * RPW + slot;
    const bool valid = o < O;
    float acc[M];
#pragma unroll
    for (int t = 0; t < M; ++t) acc[t] = 0.f;
    const typename KL::Row r = pf[i];
    if (it + PF < a.iters) pf[i] = KL::load(sg.qs, sg.scales, sg.dm, row_of(it + PF), nb, L);
    KL::accumulate(r, L, acc);
    if (it == 0) ORN_MARK(4);
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
        const int64_t yi = (GATHER ? yrow0 : (int64_t)t * O) + o;
        if (a.y_bf16)
          static_cast<bf16_t*>(sg.y)[yi] = dm_f2bf(v);
        else
          static_cast<float*>(sg.y)[yi] = v;
      }
    }
   }
  }
  ORN_MARK(5);
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

// fills first_block for every segment and returns the grid width
template <int LPR, int KS>
int layout_segments(KqArgs& a) {
  constexpr int RPW = 64 / LPR, WPB = 4 / KS;
  const int rows_per_block = RPW * WPB * a.iters;
  int blocks = 0;
  for (int s = 0; s < a.nseg; ++s) {
    a.seg[s].first_block = blocks;
    blocks += (a.seg[s].O + rows_per_block - 1) / rows_per_block;
  }
  return blocks;
}

// Workgroups of a kernel that one compute unit holds at once (its registers and LDS decide:
// from five for one Q4_K activation row down to one for three or four Q6_K rows, whose lanes
// keep 64 activations a row in registers). Asked of the runtime once per kernel.
template <typename Kernel>
int resident_workgroups(Kernel kernel) {
  int n = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, 256, 0) != hipSuccess || n < 1) {
    (void)hipGetLastError();
    n = 2;
  }
  return n;
}

// Rows each wavefront walks when the caller leaves it open (a.iters == 0): the fewest with
// which the whole grid is resident at once, counting at most three workgroups a compute unit.
// The kernels are bound by latency and vector-ALU issue, not by HBM: a grid larger than the
// chip holds runs as two rounds of the same chain of latencies (a 9216 x 2048 Q6_K projection
// of two rows: 9.9 us as 1152 workgroups where 512 fit, 8.6 us as 384; one workgroup too many
// costs the same second round: 8192 + 4096 Q4_K rows of four activation rows take 19.0 us as
// 342 + 171 workgroups where 512 fit, 15.8 us as 384), while rows beyond that only lengthen the
// one round; and beyond three workgroups a compute unit the activations' conversion (and a norm
// made in the head) is repeated for nothing.
template <int LPR, int KS>
int auto_iters(const ornith_ctx* ctx, const KqArgs& a, int grid_y, int resident, int most = 3) {
  constexpr int rows_per_pass = (64 / LPR) * (4 / KS);
  const long room = (long)ctx->compute_units * (resident < most ? resident : most);
  for (int iters = 1; iters < 8; ++iters) {
    long blocks = 0;
    for (int s = 0; s < a.nseg; ++s) blocks += (a.seg[s].O + rows_per_pass * iters - 1) / (rows_per_pass * iters);
    if (blocks * grid_y <= room) return iters;
  }
  return 8;
}

template <int KIND, int LPR, int KS, int M, bool XF32, bool GATHER>
int launch_one(ornith_ctx* ctx, KqArgs& a, int grid_y) {
  static const int resident = resident_workgroups(kq_qmv_kernel<KIND, LPR, KS, M, XF32, GATHER>);
  const int asked = a.iters;
  if (!asked) a.iters = auto_iters<LPR, KS>(ctx, a, grid_y, resident);
  dim3 grid(layout_segments<LPR, KS>(a), grid_y, 1);
  hipLaunchKernelGGL((kq_qmv_kernel<KIND, LPR, KS, M, XF32, GATHER>), grid, dim3(256), 0,
                     ctx->stream, a);
  a.iters = asked;
  ORN_LAUNCH_CHECK("kq_qmv_kernel");
  return ORNITH_OK;
}

template <int KIND, int M, bool XF32, bool GATHER>
int launch_shape(ornith_ctx* ctx, KqArgs& a, int grid_y) {
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

template <int KIND, int LPR, int M>
int launch_pre(ornith_ctx* ctx, KqArgs& a) {
  static const int resident = resident_workgroups(kq_qmv_kernel<KIND, LPR, 1, M, false, false, true>);
  // (with the norm in its head a Q6_K launch, whose lanes take 64 weights a pass, measures best
  // at no more than two workgroups a compute unit: 9216 rows of one activation row 8.0 -> 7.4 us)
  if (!a.iters) a.iters = auto_iters<LPR, 1>(ctx, a, 1, resident, KIND == ORNITH_Q6K ? 2 : 3);
  dim3 grid(layout_segments<LPR, 1>(a), 1, 1);
  hipLaunchKernelGGL((kq_qmv_kernel<KIND, LPR, 1, M, false, false, true>), grid, dim3(256), 0, ctx->stream, a);
  ORN_LAUNCH_CHECK("kq_qmv_kernel<pre-norm>");
  return ORNITH_OK;
}
template <int KIND, int LPR>
int launch_pre_m(ornith_ctx* ctx, KqArgs& a, int M) {
  switch (M) {
    case 1: return launch_pre<KIND, LPR, 1>(ctx, a);
    case 2: return launch_pre<KIND, LPR, 2>(ctx, a);
    case 3: return launch_pre<KIND, LPR, 3>(ctx, a);
    default: return launch_pre<KIND, LPR, 4>(ctx, a);
  }
}

template <int KIND, bool XF32>
int launch_m(ornith_ctx* ctx, KqArgs& a, int M) {
  switch (M) {
    case 1: return launch_shape<KIND, 1, XF32, false>(ctx, a, 1);
    case 2: return launch_shape<KIND, 2, XF32, false>(ctx, a, 1);
    case 3: return launch_shape<KIND, 3, XF32, false>(ctx, a, 1);
    default: return launch_shape<KIND, 4, XF32, false>(ctx, a, 1);
  }
}

// rows each wavefront walks: the option's value when it is set, else 0 = left to the launch,
// which knows its kernel (auto_iters)
int pick_iters() {
  const int forced = ornith_option_kq_iters();
  return forced > 8 ? 8 : forced;
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
  if (w && w->kind == ORNITH_AFFINE4_G32) {
    ORN_REQUIRE(w->E >= 1 && w->O >= 1 && w->K >= 32 && w->K % 32 == 0, "KMatrix: bad dims E=%d O=%d K=%d", w->E,
                w->O, w->K);
    ORN_REQUIRE(w->d_qs && w->d_scales && w->d_dm, "KMatrix: null tensor");
    const size_t groups = (size_t)w->E * w->O * (w->K / 32);
    ORN_REQUIRE(qs_bytes == groups * 16 && scales_bytes == groups * 2 && dm_bytes == groups * 2,
                "affine4 sizes: %zu / %zu / %zu bytes, %zu groups want %zu / %zu / %zu", qs_bytes, scales_bytes,
                dm_bytes, groups, groups * 16, groups * 2, groups * 2);
    return ORNITH_OK;
  }
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

// ys[i] = rms_norm(res + y, w_norm) . W_i^T with the norm made inside the launch.
// Returns -1 (nothing launched) when the shapes are outside what the kernel covers.
int kq_qmv_multi_prenorm(ornith_ctx* ctx, const ornith_kmatrix* const* ws, int n, const void* d_res,
                         const void* d_y, const void* d_wnorm, float eps, int M, void* d_h_out,
                         void* d_normed_out, void* const* d_ys) {
  if (n < 1 || n > kMaxSeg || M < 1 || M > 4 || ws[0]->K != kPreN) return -1;
  // (Q6_K lanes hold 64 activations a row in registers, and the M >= 2 kernels once lost their
  // occupancy to the norm's own registers on top; they no longer do -- the prologue's registers
  // are dead before the row loop's peak -- and the launch saved is worth 0.4 % at depth 1 and 1.7 %
  // at depth 3 in same-box A/B runs, so every width takes the norm in its head now.)
  for (int s = 0; s < n; ++s) {
    if (check_matrix(ws[s], "kq_qmv_prenorm")) return -1;
    if (ws[s]->E != 1 || ws[s]->kind != ws[0]->kind || ws[s]->K != ws[0]->K || !d_ys[s]) return -1;
  }
  KqArgs a{};
  a.nseg = n;
  a.K = kPreN;
  a.y_bf16 = 1;
  a.iters = pick_iters();
  for (int s = 0; s < n; ++s) {
    a.seg[s].qs = (const uint8_t*)ws[s]->d_qs;
    a.seg[s].scales = (const uint8_t*)ws[s]->d_scales;
    a.seg[s].dm = (const uint16_t*)ws[s]->d_dm;
    a.seg[s].O = ws[s]->O;
    a.seg[s].y = d_ys[s];
  }
  a.pre = PreNorm{(const bf16_t*)d_res, (const bf16_t*)d_y, (const bf16_t*)d_wnorm, (bf16_t*)d_h_out,
                  (bf16_t*)d_normed_out, eps};
  return ws[0]->kind == ORNITH_Q4K ? launch_pre_m<ORNITH_Q4K, 64>(ctx, a, M)
                                   : launch_pre_m<ORNITH_Q6K, 32>(ctx, a, M);
}

int ornith_kq_qmv_multi(ornith_ctx* ctx, const ornith_kmatrix* const* ws, int n, const void* d_x,
                        int x_dtype, int M, void* const* d_ys, int y_dtype) {
  ORN_REQUIRE(ctx && ws && d_x && d_ys, "kq_qmv: null argument");
  ORN_REQUIRE(n >= 1 && n <= kMaxSeg, "kq_qmv: %d matrices in one launch (1..%d)", n, kMaxSeg);
  ORN_REQUIRE(M >= 1, "kq_qmv: M=%d", M);
  ORN_REQUIRE(((uintptr_t)d_x & 15) == 0, "kq_qmv: x must be 16-byte aligned");
  for (int s = 0; s < n; ++s) {
    int rc = check_matrix(ws[s], "kq_qmv");
    if (rc) return rc;
    ORN_REQUIRE(ws[s]->E == 1, "kq_qmv: matrix has %d experts; use gather_qmv", ws[s]->E);
    ORN_REQUIRE(ws[s]->kind == ws[0]->kind && ws[s]->K == ws[0]->K,
                "kq_qmv: matrices fused into one launch must share format and width");
    ORN_REQUIRE(d_ys[s], "kq_qmv: null output");
  }
  const int kind = ws[0]->kind, K = ws[0]->K;
  const size_t xs = ornith_dtype_size(x_dtype), ys = ornith_dtype_size(y_dtype);
  KqArgs a{};
  a.nseg = n;
  a.K = K;
  a.y_bf16 = y_dtype == ORNITH_BF16;
  a.iters = pick_iters();
  for (int m0 = 0; m0 < M; m0 += 4) {
    const int mw = M - m0 < 4 ? M - m0 : 4;
    a.x = (const char*)d_x + (size_t)m0 * K * xs;
    for (int s = 0; s < n; ++s) {
      a.seg[s].qs = (const uint8_t*)ws[s]->d_qs;
      a.seg[s].scales = (const uint8_t*)ws[s]->d_scales;
      a.seg[s].dm = (const uint16_t*)ws[s]->d_dm;
      a.seg[s].O = ws[s]->O;
      a.seg[s].y = (char*)d_ys[s] + (size_t)m0 * ws[s]->O * ys;
    }
    int rc;
    if (kind == ORNITH_Q4K)
      rc = x_dtype == ORNITH_F32 ? launch_m<ORNITH_Q4K, true>(ctx, a, mw)
                                 : launch_m<ORNITH_Q4K, false>(ctx, a, mw);
    else
      rc = x_dtype == ORNITH_F32 ? launch_m<ORNITH_Q6K, true>(ctx, a, mw)
                                 : launch_m<ORNITH_Q6K, false>(ctx, a, mw);
    if (rc) return rc;
  }
  return ORNITH_OK;
}

int ornith_kq_qmv(ornith_ctx* ctx, const ornith_kmatrix* w, const void* d_x, int x_dtype, int M,
                  void* d_y, int y_dtype) {
  ORN_REQUIRE(d_y, "kq_qmv: null argument");
  return ornith_kq_qmv_multi(ctx, &w, 1, d_x, x_dtype, M, &d_y, y_dtype);
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
  a.nseg = 1;
  a.seg[0].qs = (const uint8_t*)w->d_qs;
  a.seg[0].scales = (const uint8_t*)w->d_scales;
  a.seg[0].dm = (const uint16_t*)w->d_dm;
  a.seg[0].y = d_y;
  a.seg[0].O = w->O;
  a.x = d_x;
  a.lhs = d_lhs;
  a.rhs = d_rhs;
  a.E = w->E;
  a.x_rows = x_rows;
  a.K = w->K;
  a.y_bf16 = y_dtype == ORNITH_BF16;
  a.iters = pick_iters();
  if (w->kind == ORNITH_Q4K)
    return x_dtype == ORNITH_F32 ? launch_shape<ORNITH_Q4K, 1, true, true>(ctx, a, rows)
                                 : launch_shape<ORNITH_Q4K, 1, false, true>(ctx, a, rows);
  return x_dtype == ORNITH_F32 ? launch_shape<ORNITH_Q6K, 1, true, true>(ctx, a, rows)
                               : launch_shape<ORNITH_Q6K, 1, false, true>(ctx, a, rows);
}

}  // extern "C"
