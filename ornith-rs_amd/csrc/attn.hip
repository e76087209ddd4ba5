// Full-attention layer at decode / verify width: per-head RMS + partial RoPE +
// KV append in one kernel, split-K attention over the cache, merge + output gate.
//
// Replaces the middle of Attention::forward
// (/root/reference/src/model/qwen3_5.rs:430-474): rms_norm on q/k heads,
// rope (/root/reference/src/ops/rope.rs:6-60, vendored rope.metal:11-67),
// KvCache::update_and_fetch (/root/reference/src/model/cache.rs:38-79),
// attention_with_cache -> sdpa_vector[_2pass]
// (/root/reference/src/ops/sdpa.rs:33-83,166-264, vendored sdpa_vector.h:15-318)
// and sigmoid_gate (kernels/ornith_elementwise.metal).
//
// Attention is split over keys in blocks of 256 by absolute position, one
// workgroup per (block, query head, query row): a key's score is one fma chain per
// 64 channels with the chains added pairwise, a channel's output one fma chain per
// 64 keys of the block added the same way, so neither needs a cross-lane reduction
// per key. The partial (max, sum, values) of each block go to scratch and a second
// kernel merges them in ascending block order and applies the sigmoid output gate;
// when every row has a single block the partial kernel does that itself.
// A query row only ever sees keys at or before its own position, and blocks are
// aligned to absolute positions, so row r of a T-row verify call is bit-identical
// to a one-row call at that position.
#include <type_traits>

#include "dmath.h"
#include "rt.h"

namespace {

constexpr int ATT_KB = 256;

struct PrepArgs {
  const bf16_t* qg;  // [T, Hq, 2*hd]
  const bf16_t* kx;  // [T, Hkv, hd]
  const bf16_t* vx;  // [T, Hkv, hd]
  const bf16_t* qw;  // [hd]
  const bf16_t* kw;  // [hd]
  const float* cos_t;  // [npos, half]
  const float* sin_t;
  const int* d_offset;  // optional: position of the first new row, read on the device
  bf16_t* q_rot;      // [T, Hq, hd]
  bf16_t* k_cache;    // [Hkv, cap, hd]
  bf16_t* v_cache;
  int T, Hq, Hkv, offset, cap, npos, half;
  float eps;
};

// The per-head prep of one row by one wavefront (PER = hd / 64 contiguous channels a lane), in
// two steps so that a caller can put other loads between the request and the arithmetic:
// prep_issue asks for the row, the norm weight and the lane's cos / sin entries; prep_finish
// returns the normed, rotated values (rounded to bf16 by whoever stores them).
template <int PER>
struct PrepRegs {
  bf16_t x[PER], w[PER];
  float c[PER], s[PER];
};

template <int PER>
__device__ __forceinline__ void prep_issue(const bf16_t* src, const bf16_t* w, const float* cos_t, const float* sin_t,
                                           int pos, int half, int lane, PrepRegs<PER>& g) {
#pragma unroll
  for (int i = 0; i < PER; ++i) g.x[i] = src[lane * PER + i];
  if (w) {
#pragma unroll
    for (int i = 0; i < PER; ++i) g.w[i] = w[lane * PER + i];
    const int hl = half / PER;
    const bool lowg = lane < hl, rot = lane < 2 * hl;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int e = (lowg ? lane : lane - hl) * PER + i;
      g.c[i] = rot ? cos_t[(size_t)pos * half + e] : 0.f;
      g.s[i] = rot ? sin_t[(size_t)pos * half + e] : 0.f;
    }
  }
}

template <int PER>
__device__ __forceinline__ void prep_finish(const PrepRegs<PER>& g, bool normed, int half, float eps, int lane,
                                            float (&x)[PER]) {
  constexpr int HD = 64 * PER;
#pragma unroll
  for (int i = 0; i < PER; ++i) x[i] = dm_bf2f(g.x[i]);
  if (!normed) return;
  float a = 0.f;
#pragma unroll
  for (int i = 0; i < PER; ++i) a = dm_fma(x[i], x[i], a);
  const float inv = dm_rsqrt(dm_wave_sum<64>(a) / (float)HD + eps);
#pragma unroll
  for (int i = 0; i < PER; ++i) x[i] = dm_rb(dm_bf2f(g.w[i]) * dm_rb(x[i] * inv));
  // rotate pairs (e, e + half), e < half; the partner channel lives hl lanes away
  const int hl = half / PER;
  const bool lowg = lane < hl, rot = lane < 2 * hl;
  const int partner = lowg ? lane + hl : lane - hl;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const float other = __shfl(x[i], partner & 63, 64);
    if (rot) {
      float r;
      if (lowg) {
        r = x[i] * g.c[i];
        r = dm_fma(-other, g.s[i], r);
      } else {
        r = other * g.s[i];
        r = dm_fma(x[i], g.c[i], r);
      }
      x[i] = r;  // rounded on store
    }
  }
}

// one wavefront per (head, token)
template <int PER>
__global__ __launch_bounds__(64) void attn_prep_kernel(PrepArgs p) {
  constexpr int HD = 64 * PER;
  const int hidx = blockIdx.x, t = blockIdx.y, lane = threadIdx.x;
  const int offset = p.d_offset ? *p.d_offset : p.offset;
  const int pos = offset + t;
  if (pos >= p.cap || pos >= p.npos) return;  // host checks the static case; device offset guarded here
  const bf16_t* src;
  bf16_t* dst;
  const bf16_t* w = nullptr;
  if (hidx < p.Hq) {
    src = p.qg + ((size_t)t * p.Hq + hidx) * 2 * HD;
    dst = p.q_rot + ((size_t)t * p.Hq + hidx) * HD;
    w = p.qw;
  } else if (hidx < p.Hq + p.Hkv) {
    const int h = hidx - p.Hq;
    src = p.kx + ((size_t)t * p.Hkv + h) * HD;
    dst = p.k_cache + ((size_t)h * p.cap + pos) * HD;
    w = p.kw;
  } else {
    const int h = hidx - p.Hq - p.Hkv;
    src = p.vx + ((size_t)t * p.Hkv + h) * HD;
    dst = p.v_cache + ((size_t)h * p.cap + pos) * HD;
  }
  PrepRegs<PER> g;
  prep_issue<PER>(src, w, p.cos_t, p.sin_t, pos, p.half, lane, g);
  float x[PER];
  prep_finish<PER>(g, w != nullptr, p.half, p.eps, lane, x);
#pragma unroll
  for (int i = 0; i < PER; ++i) dst[lane * PER + i] = dm_f2bf(x[i]);
}

struct SdpaArgs {
  const bf16_t* q_rot;   // [T, Hq, HD]
  const bf16_t* k_cache; // [Hkv, cap, HD]
  const bf16_t* v_cache;
  const bf16_t* qg;      // [T, Hq, 2*HD] (gate half read by the merge)
  const int* d_offset;
  float* part_m;         // [T, Hq, nblk]
  float* part_l;         // [T, Hq, nblk]
  float* part_o;         // [T, Hq, nblk, HD]
  bf16_t* out;           // [T, Hq*HD]
  int T, Hq, Hkv, offset, cap, nblk;
  float scale;
  int finish;  // 1: every row has a single key block, the partial kernel applies the merge's
               //    arithmetic itself and writes `out` (no merge launch follows)
};

// grid (nblk, Hq, T), 1024 threads: one query head against one block of ATT_KB keys.
//
// The sums: a key's score is one fma chain per 64 channels, the chains added pairwise
// ((c0 + c1) + (c2 + c3)); a channel's output over the block is one chain per 64 keys, added
// the same way. That gives every one of the 1024 threads a chain of 64 in both phases.
//
// The arithmetic is small and a trip to memory is long, so the whole block -- every key row
// and every value row -- is requested by the 16 wavefronts at once, in 16-byte pieces with
// eight lanes to a 128-byte line, before anything is computed. The rows then pass through
// LDS (keys as 64-channel panels with rows padded by 16 bytes to spread the banks; the values
// take the same memory over once the scores are done). Rows past the last valid key are not
// read, and the chains that would hold only such rows are not run.
constexpr int SDPA_NT = 1024;
constexpr int SDPA_KROW = 64 * 2 + 16;  // bytes of a staged 64-channel key row

// A native vector, not HIP's uint4 struct: arrays of the struct copied to LDS through casts are
// left in scratch memory by the compiler, arrays of this type stay in registers.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <int HD>
constexpr int sdpa_stage_bytes() {
  constexpr int k = (HD / 64) * ATT_KB * SDPA_KROW, v = ATT_KB * HD * 2;
  return k > v ? k : v;
}

// (p0 + p1) + (p2 + p3) for N = 4, p0 + p1 for N = 2
template <int N>
__device__ __forceinline__ float sdpa_pair_tree(const float* p, int stride) {
  float t[N];
#pragma unroll
  for (int i = 0; i < N; ++i) t[i] = p[i * stride];
#pragma unroll
  for (int w = N; w > 1; w /= 2)
#pragma unroll
    for (int i = 0; i < w / 2; ++i) t[i] = t[2 * i] + t[2 * i + 1];
  return t[0];
}

//
// PREP: the launch also does attn_prep's work (the per-head norm, RoPE and the KV append), so
// that no prep launch precedes it: wavefront 0 makes the query row of this (row, head) from the
// raw projection, wavefronts 1 .. t + 1 the key rows of the call's new positions that lie in this
// block (they go into the staged block in place of the cache's rows, which are not yet written),
// the new value rows are read from the raw projection, and the workgroup of a KV group's first
// head stores its own row's key and value to the cache. Static offset, T <= 8.
template <int HD, bool PREP>
__global__ __launch_bounds__(SDPA_NT) __attribute__((amdgpu_waves_per_eu(4, 4))) void sdpa_partial_kernel(SdpaArgs p,
                                                                                                           PrepArgs q) {
  const int b = blockIdx.x, hq = blockIdx.y, t = blockIdx.z, tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int offset = PREP ? p.offset : (p.d_offset ? *p.d_offset : p.offset);
  const int last = min(offset + t, p.cap - 1);
  if (b * ATT_KB > last) return;
  const int hk = hq / (p.Hq / p.Hkv);

  constexpr int PPR = HD / 8;                    // 16-byte pieces per row
  constexpr int RPU = SDPA_NT / PPR;             // value rows covered by one load per thread
  constexpr int NLD = ATT_KB / RPU;              // loads per thread for the block (keys: same count)
  constexpr int KC = 64, NKC = HD / KC, KROW = SDPA_KROW;
  constexpr int KPC = ATT_KB * (KC / 8) / SDPA_NT, KRS = SDPA_NT / (KC / 8);
  constexpr int VB = 64, NVB = ATT_KB / VB;
  static_assert(SDPA_NT % PPR == 0 && ATT_KB % RPU == 0 && KPC * NKC == NLD, "piece mapping");
  static_assert(ATT_KB == 256 && NKC <= 4 && NVB == 4 && HD <= 256, "chains of 64, four wavefronts a chain group");
  extern __shared__ __align__(16) unsigned char stage[];
  __shared__ __align__(16) float qs[HD];
  __shared__ float pr[ATT_KB];
  __shared__ float red[4];
  __shared__ float part[4 * 256];  // chain results: [panel][key], later [key group][channel]

  const int nvalid = min(ATT_KB, last - b * ATT_KB + 1);
  const int row0 = tid / PPR, piece = tid - row0 * PPR;    // values: rows row0 + RPU*u, piece column
  const int krow0 = tid / (KC / 8), kpc = tid % (KC / 8);  // keys: rows krow0 + KRS*i of every panel
  const bf16_t* kbase = p.k_cache + ((size_t)hk * p.cap + (size_t)b * ATT_KB) * HD;
  const bf16_t* vblk = p.v_cache + ((size_t)hk * p.cap + (size_t)b * ATT_KB) * HD + 8 * piece;
  u32x4 kreg[NLD], vreg[NLD];
  // PREP: this wavefront's row of the prep (0: none, 1: the query, 2: a new key row at kpos);
  // its few loads go out ahead of the block's, so that they are back first
  constexpr int PER = HD / 64;
  PrepRegs<PER> pg;
  int task = 0, kpos = 0;
  const bool first_of_group = hq % (p.Hq / p.Hkv) == 0;
  if constexpr (PREP) {
    if (wave == 0) {
      task = 1;
      prep_issue<PER>(q.qg + ((size_t)t * p.Hq + hq) * 2 * HD, q.qw, q.cos_t, q.sin_t, offset + t, q.half, lane, pg);
    } else if (wave <= t + 1 && (offset + wave - 1) / ATT_KB == b) {
      task = 2;
      kpos = offset + wave - 1;
      prep_issue<PER>(q.kx + ((size_t)(wave - 1) * p.Hkv + hk) * HD, q.kw, q.cos_t, q.sin_t, kpos, q.half, lane, pg);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  // Rows past the last valid key are neither requested nor staged (a short context leaves most
  // of the block empty, and a request costs its slot in the compute unit's load path whether or
  // not the line is cached); what LDS holds in their place is never added to anything.
  // PREP: nor are the key rows of this call's positions, which come from their wavefronts.
  auto key_row_staged = [&](int r) { return r < nvalid && !(PREP && b * ATT_KB + r >= offset); };
#pragma unroll
  for (int c = 0; c < NKC; ++c)
#pragma unroll
    for (int i = 0; i < KPC; ++i) {
      const int r = krow0 + KRS * i;
      if (key_row_staged(r)) kreg[c * KPC + i] = *reinterpret_cast<const u32x4*>(kbase + (size_t)r * HD + c * KC + 8 * kpc);
    }
#pragma unroll
  for (int u = 0; u < NLD; ++u) {
    const int vr = row0 + RPU * u;
    if (vr >= nvalid) continue;
    const bf16_t* src = vblk + (size_t)vr * HD;
    // a position of this call: its value row is still in the projection's output
    if (PREP && b * ATT_KB + vr >= offset)
      src = q.vx + ((size_t)(b * ATT_KB + vr - offset) * p.Hkv + hk) * HD + 8 * piece;
    vreg[u] = *reinterpret_cast<const u32x4*>(src);
  }
  // the output gate of a finishing block is requested with everything else
  bf16_t gate_pre = 0;
  if (p.finish && tid < HD) gate_pre = p.qg[((size_t)t * p.Hq + hq) * 2 * HD + HD + tid];
  if constexpr (!PREP)
    if (tid < HD) qs[tid] = p.scale * dm_bf2f(p.q_rot[((size_t)t * p.Hq + hq) * HD + tid]);

  // scores: thread (key, panel) runs the chain over the panel's 64 channels
#pragma unroll
  for (int c = 0; c < NKC; ++c)
#pragma unroll
    for (int i = 0; i < KPC; ++i) {
      const int dest = krow0 + KRS * i;
      if (!key_row_staged(dest)) continue;
      *reinterpret_cast<u32x4*>(stage + c * (ATT_KB * KROW) + dest * KROW + 16 * kpc) = kreg[c * KPC + i];
    }
  if constexpr (PREP) {
    if (task) {
      float x[PER];
      prep_finish<PER>(pg, true, q.half, q.eps, lane, x);
      if (task == 1) {
#pragma unroll
        for (int i = 0; i < PER; ++i) qs[lane * PER + i] = p.scale * dm_bf2f(dm_f2bf(x[i]));  // q_rot is bf16
      } else {
        const int dest = kpos - b * ATT_KB, ch = lane * PER;
        bf16_t* row = reinterpret_cast<bf16_t*>(stage + (ch / KC) * (ATT_KB * KROW) + dest * KROW) + ch % KC;
        bf16_t* crow = q.k_cache + ((size_t)hk * p.cap + kpos) * HD + ch;
        const bool append = first_of_group && wave - 1 == t;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
          const bf16_t v = dm_f2bf(x[i]);
          row[i] = v;
          if (append) crow[i] = v;
        }
      }
    }
    // this row's value row to the cache (the thread that holds its piece unclamped)
    if (first_of_group && b == (offset + t) / ATT_KB) {
#pragma unroll
      for (int u = 0; u < NLD; ++u)
        if (b * ATT_KB + row0 + RPU * u == offset + t)
          *reinterpret_cast<u32x4*>(q.v_cache + ((size_t)hk * p.cap + offset + t) * HD + 8 * piece) = vreg[u];
    }
  }
  __syncthreads();
  // wavefront w takes panel w % 4 of keys [64 (w / 4), +64): a SIMD (wavefronts go round the four
  // in order) then holds one panel of every key group, and the groups past the last valid key
  // drop out of all four SIMDs alike
  const int grp = wave & 3, key = (wave >> 2) * 64 + lane;
  if (grp < NKC && (wave >> 2) * 64 < nvalid) {
    u32x4 kws[KC / 8];
#pragma unroll
    for (int i = 0; i < KC / 8; ++i)
      kws[i] = *reinterpret_cast<const u32x4*>(stage + grp * (ATT_KB * KROW) + key * KROW + 16 * i);
    // the panel's 64 query values: one per lane, handed out through scalar registers
    const int qv = __float_as_int(qs[grp * KC + lane]);
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < KC / 8; ++i) {
      const u32x4 kw = kws[i];
      const float kf[8] = {dm_bf2f_lo(kw.x), dm_bf2f_hi(kw.x), dm_bf2f_lo(kw.y), dm_bf2f_hi(kw.y),
                           dm_bf2f_lo(kw.z), dm_bf2f_hi(kw.z), dm_bf2f_lo(kw.w), dm_bf2f_hi(kw.w)};
#pragma unroll
      for (int e = 0; e < 8; ++e)
        acc = dm_fma(__int_as_float(__builtin_amdgcn_readlane(qv, 8 * i + e)), kf[e], acc);
    }
    part[grp * ATT_KB + key] = acc;
  }
  __syncthreads();
  // block max, probabilities, their sum (the first four wavefronts hold the keys)
  const bool valid = tid < nvalid;
  float sc = 0.f;
  if (tid < ATT_KB) {
    sc = sdpa_pair_tree<NKC>(part + tid, ATT_KB);
    const float m = dm_wave_max<64>(valid ? sc : -DM_INF);
    if (lane == 0) red[wave] = m;
  }
  __syncthreads();
  float mg = red[0];
  mg = red[1] > mg ? red[1] : mg;
  mg = red[2] > mg ? red[2] : mg;
  mg = red[3] > mg ? red[3] : mg;
  __syncthreads();
  if (tid < ATT_KB) {
    const float pv = valid ? dm_exp(sc - mg) : 0.f;
    pr[tid] = pv;
    const float ws = dm_wave_sum<64>(pv);
    if (lane == 0) red[wave] = ws;
  }
  // values: thread (channel, group of 64 keys) runs the chain over the group's valid keys
  bf16_t (*vst)[HD] = reinterpret_cast<bf16_t (*)[HD]>(stage);
#pragma unroll
  for (int u = 0; u < NLD; ++u)
    if (row0 + RPU * u < nvalid) *reinterpret_cast<u32x4*>(&vst[row0 + RPU * u][8 * piece]) = vreg[u];
  __syncthreads();  // probabilities and value rows in place (the key panels were last read two barriers ago)
  const int ch = tid % HD, vg = tid / HD;
  if (vg < NVB && VB * vg >= nvalid) part[vg * HD + ch] = 0.f;  // a chain with no valid key
  if (vg < NVB && VB * vg < nvalid) {
    const int prv = __float_as_int(pr[VB * vg + lane]);
    bf16_t vv[VB];
#pragma unroll
    for (int j = 0; j < VB; ++j) vv[j] = vst[VB * vg + j][ch];
    float o = 0.f;
#pragma unroll
    for (int j = 0; j < VB; ++j) {
      const float next = dm_fma(__int_as_float(__builtin_amdgcn_readlane(prv, j)), dm_bf2f(vv[j]), o);
      o = VB * vg + j < nvalid ? next : o;
    }
    part[vg * HD + ch] = o;
  }
  __syncthreads();
  const size_t pi = ((size_t)t * p.Hq + hq) * p.nblk + b;
  float l = red[0] + red[1];
  l = l + red[2];
  l = l + red[3];
  if (p.finish) {
    // the merge over one block, operation for operation (sdpa_merge_kernel with nb == 1)
    if (tid < HD) {
      const float w = dm_exp(mg - mg);
      const float L = dm_fma(l, w, 0.f);
      const float O = dm_fma(sdpa_pair_tree<NVB>(part + tid, HD), w, 0.f);
      const float att = dm_rb(O / L);
      const float g = dm_sigmoid_bf16(dm_bf2f(gate_pre));
      p.out[((size_t)t * p.Hq + hq) * HD + tid] = dm_f2bf(g * att);
    }
    return;
  }
  if (tid < HD) p.part_o[pi * HD + tid] = sdpa_pair_tree<NVB>(part + tid, HD);
  if (tid == 0) {
    p.part_m[pi] = mg;
    p.part_l[pi] = l;
  }
}

// The same partial sums when there are many blocks to work through (long contexts): 256
// threads a block, several blocks resident per compute unit. A workgroup takes NH query heads
// of one KV group (four when the group allows it): the key and value block is then read once
// for the four instead of once a head (with one head a workgroup the L2 delivered every block
// 32 times for 8 heads a group and 4 rows, 440 MB a call at a 6.6 k context, and that, not
// HBM or the arithmetic, set the time). Thread `tid` owns key `tid` for the scores and runs
// the chains of 64 channels one after the other; the key block reaches it through LDS, 64
// channels at a time, so that the global loads are whole 128-byte pieces of a row. For the
// values a thread owns four channels of one 64-key chain (8-byte loads, a wavefront reads 512
// contiguous bytes a key); the four chains of a channel meet in LDS. Every sum of every head
// keeps its order. grid (nblk, Hq / NH, T), 256 threads.
template <int HD, int NH>
__global__ __launch_bounds__(256) void sdpa_partial_many_kernel(SdpaArgs p) {
  const int b = blockIdx.x, hq0 = blockIdx.y * NH, t = blockIdx.z, tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int offset = p.d_offset ? *p.d_offset : p.offset;
  const int last = min(offset + t, p.cap - 1);
  if (b * ATT_KB > last) return;
  const int hk = hq0 / (p.Hq / p.Hkv);  // the NH heads share it
  constexpr int NKC = HD / 64, NVB = ATT_KB / 64, KLD = 64 + 8;
  static_assert(ATT_KB == 256, "one key per thread");
  static_assert(NKC == 2 || NKC == 4, "head widths of 128 and 256");

  __shared__ __align__(16) bf16_t ks[ATT_KB][KLD];
  __shared__ __align__(16) float qs[NH][HD];
  __shared__ float pr[NH][ATT_KB];
  __shared__ float red[NH][4];
  __shared__ float part[NH][NVB * HD];

  const int key = b * ATT_KB + tid;
  const bool valid = key <= last;
  const int nvalid = min(ATT_KB, last - b * ATT_KB + 1);
  const bf16_t* kblk = p.k_cache + ((size_t)hk * p.cap + (size_t)b * ATT_KB) * HD;

  // 64-channel panel c of the key block: 2048 16-byte pieces, eight a thread (rows past the
  // last key read the last key's: their scores are masked). Two panels travel in registers
  // ahead of their use, and so do the first 32 keys of this thread's value chain: a block is a
  // chain of memory latencies otherwise.
  u32x4 kreg[2][8];
  auto fetch_panel = [&](auto set, int c) {
    constexpr int S = decltype(set)::value;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int idx = tid + 256 * u, r = min(idx >> 3, nvalid - 1), part8 = idx & 7;
      kreg[S][u] = *reinterpret_cast<const u32x4*>(kblk + (size_t)r * HD + 64 * c + 8 * part8);
    }
  };
  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;
  fetch_panel(S0{}, 0);
  fetch_panel(S1{}, 1);
  constexpr int TPC = HD / 4;  // threads a value chain
  const int vg = tid / TPC, vcg = tid % TPC;
  const bf16_t* vcol = p.v_cache + ((size_t)hk * p.cap + (size_t)b * ATT_KB + 64 * vg) * HD + 4 * vcg;
  const int vn = min(64, nvalid - 64 * vg);  // keys of this thread's chain that exist (may be <= 0)
  uint2 vreg[2][16];
  auto fetch_values = [&](auto set, int i0) {
    constexpr int S = decltype(set)::value;
    if (tid < HD) {
#pragma unroll
      for (int u = 0; u < 16; ++u)
        vreg[S][u] = *reinterpret_cast<const uint2*>(vcol + (size_t)min(i0 + u, max(vn - 1, 0)) * HD);
    }
  };
  fetch_values(S0{}, 0);
  fetch_values(S1{}, 16);
  for (int i = tid; i < NH * HD; i += 256)
    qs[i / HD][i % HD] = p.scale * dm_bf2f(p.q_rot[((size_t)t * p.Hq + hq0 + i / HD) * HD + i % HD]);
  float cpart[NH][NKC];
  auto panel = [&](auto set, auto cc) {
    constexpr int S = decltype(set)::value, c = decltype(cc)::value;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int idx = tid + 256 * u;
      *reinterpret_cast<u32x4*>(&ks[idx >> 3][8 * (idx & 7)]) = kreg[S][u];
    }
    __syncthreads();
    if constexpr (c + 2 < NKC) fetch_panel(set, c + 2);
    float a[NH];
#pragma unroll
    for (int j = 0; j < NH; ++j) a[j] = 0.f;
#pragma unroll
    for (int dc = 0; dc < 8; ++dc) {
      const uint4 kw = *reinterpret_cast<const uint4*>(&ks[tid][8 * dc]);
      const float k0 = dm_bf2f_lo(kw.x), k1 = dm_bf2f_hi(kw.x), k2 = dm_bf2f_lo(kw.y), k3 = dm_bf2f_hi(kw.y);
      const float k4 = dm_bf2f_lo(kw.z), k5 = dm_bf2f_hi(kw.z), k6 = dm_bf2f_lo(kw.w), k7 = dm_bf2f_hi(kw.w);
#pragma unroll
      for (int j = 0; j < NH; ++j) {
        const float4 q0 = *reinterpret_cast<const float4*>(&qs[j][64 * c + 8 * dc]);
        const float4 q1 = *reinterpret_cast<const float4*>(&qs[j][64 * c + 8 * dc + 4]);
        a[j] = dm_fma(q0.x, k0, a[j]);
        a[j] = dm_fma(q0.y, k1, a[j]);
        a[j] = dm_fma(q0.z, k2, a[j]);
        a[j] = dm_fma(q0.w, k3, a[j]);
        a[j] = dm_fma(q1.x, k4, a[j]);
        a[j] = dm_fma(q1.y, k5, a[j]);
        a[j] = dm_fma(q1.z, k6, a[j]);
        a[j] = dm_fma(q1.w, k7, a[j]);
      }
    }
#pragma unroll
    for (int j = 0; j < NH; ++j) cpart[j][c] = a[j];
    __syncthreads();
  };
  panel(S0{}, std::integral_constant<int, 0>{});
  panel(S1{}, std::integral_constant<int, 1>{});
  if constexpr (NKC > 2) {
    panel(S0{}, std::integral_constant<int, 2>{});
    panel(S1{}, std::integral_constant<int, 3>{});
  }
  float sc[NH], mg[NH];
#pragma unroll
  for (int j = 0; j < NH; ++j) {
    sc[j] = sdpa_pair_tree<NKC>(cpart[j], 1);
    const float m = dm_wave_max<64>(valid ? sc[j] : -DM_INF);  // block max
    if (lane == 0) red[j][wave] = m;
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < NH; ++j) {
    float m = red[j][0];
    m = red[j][1] > m ? red[j][1] : m;
    m = red[j][2] > m ? red[j][2] : m;
    m = red[j][3] > m ? red[j][3] : m;
    mg[j] = m;
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < NH; ++j) {
    const float pv = valid ? dm_exp(sc[j] - mg[j]) : 0.f;
    pr[j][tid] = pv;
    const float ws = dm_wave_sum<64>(pv);
    if (lane == 0) red[j][wave] = ws;
  }
  __syncthreads();
  // values: chain vg = keys 64 * vg .. + 64, channels 4 * vcg .. + 4, for every head
  if (tid < HD) {
    float o[NH][4];
#pragma unroll
    for (int j = 0; j < NH; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) o[j][e] = 0.f;
    auto batch = [&](auto set, int i0) {
      constexpr int S = decltype(set)::value;
#pragma unroll
      for (int u = 0; u < 16; ++u)
        if (i0 + u < vn) {
          const float v0 = dm_bf2f_lo(vreg[S][u].x), v1 = dm_bf2f_hi(vreg[S][u].x);
          const float v2 = dm_bf2f_lo(vreg[S][u].y), v3 = dm_bf2f_hi(vreg[S][u].y);
#pragma unroll
          for (int j = 0; j < NH; ++j) {
            const float pw = pr[j][64 * vg + i0 + u];
            o[j][0] = dm_fma(pw, v0, o[j][0]);
            o[j][1] = dm_fma(pw, v1, o[j][1]);
            o[j][2] = dm_fma(pw, v2, o[j][2]);
            o[j][3] = dm_fma(pw, v3, o[j][3]);
          }
        }
    };
    batch(S0{}, 0);
    fetch_values(S0{}, 32);
    batch(S1{}, 16);
    fetch_values(S1{}, 48);
    batch(S0{}, 32);
    batch(S1{}, 48);
#pragma unroll
    for (int j = 0; j < NH; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) part[j][vg * HD + 4 * vcg + e] = o[j][e];
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < NH; ++j) {
    const size_t pi = ((size_t)t * p.Hq + hq0 + j) * p.nblk + b;
    if (tid < HD) p.part_o[pi * HD + tid] = sdpa_pair_tree<NVB>(part[j] + tid, HD);
    if (tid == 0) {
      float l = red[j][0] + red[j][1];
      l = l + red[j][2];
      l = l + red[j][3];
      p.part_m[pi] = mg[j];
      p.part_l[pi] = l;
    }
  }
}

// grid (Hq, T), HD threads: merge blocks ascending, divide, gate.
// Thread b fetches block b's maximum and sum (one load each for the whole row), every thread
// asks for its channel's partial outputs of up to kMergeAhead blocks at once, and the block
// weights exp(m_b - M) are made once (thread b) and shared through LDS; the sums over the blocks
// stay one ascending fma chain per thread. (A loop that fetched the maxima one by one and then
// eight blocks at a time was a dozen trips to memory for a 27-block row.)
constexpr int kMergeAhead = 32;
template <int HD>
__global__ __launch_bounds__(HD) void sdpa_merge_kernel(SdpaArgs p) {
  const int h = blockIdx.x, t = blockIdx.y, d = threadIdx.x;
  const int lane = d & 63, wave = d >> 6;
  const int offset = p.d_offset ? *p.d_offset : p.offset;
  const int last = min(offset + t, p.cap - 1);
  const int nb = last / ATT_KB + 1;
  const size_t pi = ((size_t)t * p.Hq + h) * p.nblk;
  __shared__ float sw[kMergeAhead], sl[kMergeAhead];
  __shared__ float red[HD / 64];
  const bf16_t gate_bits = p.qg[((size_t)t * p.Hq + h) * 2 * HD + HD + d];
  // the row's maximum: every thread over its blocks d, d + HD, ..., then over the workgroup
  float M = -DM_INF;
  for (int b = d; b < nb; b += HD) {
    const float m = p.part_m[pi + b];
    M = m > M ? m : M;
  }
  M = dm_wave_max<64>(M);
  if (lane == 0) red[wave] = M;
  __syncthreads();
  M = red[0];
#pragma unroll
  for (int w = 1; w < HD / 64; ++w) M = red[w] > M ? red[w] : M;
  float L = 0.f, O = 0.f;
  for (int b0 = 0; b0 < nb; b0 += kMergeAhead) {
    const int n = min(kMergeAhead, nb - b0);
    float po[kMergeAhead];
#pragma unroll
    for (int u = 0; u < kMergeAhead; ++u) po[u] = p.part_o[(pi + b0 + min(u, n - 1)) * HD + d];
    __syncthreads();  // the previous round's weights have been read
    if (d < n) {
      sw[d] = dm_exp(p.part_m[pi + b0 + d] - M);
      sl[d] = p.part_l[pi + b0 + d];
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < kMergeAhead; ++u)
      if (u < n) {
        const float w = sw[u];
        L = dm_fma(sl[u], w, L);
        O = dm_fma(po[u], w, O);
      }
  }
  const float att = dm_rb(O / L);
  const float g = dm_sigmoid_bf16(dm_bf2f(gate_bits));
  p.out[((size_t)t * p.Hq + h) * HD + d] = dm_f2bf(g * att);
}

}  // namespace

extern "C" {

int ornith_rope_table(ornith_ctx* ctx, int npos, int dims, double theta, float* d_cos,
                      float* d_sin) {
  ORN_REQUIRE(ctx && d_cos && d_sin, "rope_table: null argument");
  ORN_REQUIRE(npos >= 1 && dims >= 2 && dims % 2 == 0 && theta > 0, "rope_table: npos=%d dims=%d",
              npos, dims);
  const int half = dims / 2;
  float* hc = (float*)malloc(sizeof(float) * (size_t)npos * half * 2);
  if (!hc) return ornith_fail(ORNITH_ERR_INVALID, "rope_table: out of host memory");
  float* hs = hc + (size_t)npos * half;
  for (int i = 0; i < half; ++i) {
    const double inv_freq = pow(theta, -(double)i / (double)half);
    for (int pos = 0; pos < npos; ++pos) {
      const double ang = (double)pos * inv_freq;
      hc[(size_t)pos * half + i] = (float)cos(ang);
      hs[(size_t)pos * half + i] = (float)sin(ang);
    }
  }
  int rc = ornith_upload(ctx, d_cos, hc, sizeof(float) * (size_t)npos * half);
  if (!rc) rc = ornith_upload(ctx, d_sin, hs, sizeof(float) * (size_t)npos * half);
  free(hc);
  return rc;
}

static int prep_args(ornith_ctx* ctx, const void* d_qg, const void* d_kx, const void* d_vx, const void* d_q_norm_w,
                     const void* d_k_norm_w, int T, int Hq, int Hkv, int hd, int rope_dims, float eps,
                     const float* d_cos, const float* d_sin, int table_npos, int offset, const int* d_offset, int cap,
                     void* d_q_rot, void* d_k_cache, void* d_v_cache, PrepArgs* out) {
  ORN_REQUIRE(ctx && d_qg && d_kx && d_vx && d_q_norm_w && d_k_norm_w && d_cos && d_sin && d_q_rot &&
                  d_k_cache && d_v_cache,
              "attn_prep: null argument");
  ORN_REQUIRE(hd == 256 || hd == 128, "attn_prep: head_dim %d (128 or 256)", hd);
  const int per = hd / 64, half = rope_dims / 2;
  ORN_REQUIRE(rope_dims >= 2 * per && rope_dims <= hd && half % per == 0 &&
                  ((half / per) & (half / per - 1)) == 0,
              "attn_prep: rope_dims=%d does not tile head_dim %d", rope_dims, hd);
  ORN_REQUIRE(T >= 1 && T <= 65535 && Hq >= 1 && Hkv >= 1 && Hq % Hkv == 0, "attn_prep: T=%d Hq=%d Hkv=%d",
              T, Hq, Hkv);
  ORN_REQUIRE(offset >= 0 && offset + T <= cap && offset + T <= table_npos,
              "attn_prep: rows [%d,%d) do not fit cache capacity %d / rope table %d", offset,
              offset + T, cap, table_npos);
  PrepArgs p{};
  p.qg = (const bf16_t*)d_qg;
  p.kx = (const bf16_t*)d_kx;
  p.vx = (const bf16_t*)d_vx;
  p.qw = (const bf16_t*)d_q_norm_w;
  p.kw = (const bf16_t*)d_k_norm_w;
  p.cos_t = d_cos;
  p.sin_t = d_sin;
  p.d_offset = d_offset;
  p.q_rot = (bf16_t*)d_q_rot;
  p.k_cache = (bf16_t*)d_k_cache;
  p.v_cache = (bf16_t*)d_v_cache;
  p.T = T;
  p.Hq = Hq;
  p.Hkv = Hkv;
  p.offset = offset;
  p.cap = cap;
  p.npos = table_npos;
  p.half = half;
  p.eps = eps;
  *out = p;
  return ORNITH_OK;
}

static int prep_launch(ornith_ctx* ctx, const PrepArgs& p, int hd) {
  dim3 grid(p.Hq + 2 * p.Hkv, p.T);
  if (hd == 256)
    hipLaunchKernelGGL(attn_prep_kernel<4>, grid, dim3(64), 0, ctx->stream, p);
  else
    hipLaunchKernelGGL(attn_prep_kernel<2>, grid, dim3(64), 0, ctx->stream, p);
  ORN_LAUNCH_CHECK("attn_prep_kernel");
  return ORNITH_OK;
}

int ornith_attn_prep(ornith_ctx* ctx, const void* d_qg, const void* d_kx, const void* d_vx,
                     const void* d_q_norm_w, const void* d_k_norm_w, int T, int Hq, int Hkv, int hd,
                     int rope_dims, float eps, const float* d_cos, const float* d_sin, int table_npos,
                     int offset, const int* d_offset, int cap, void* d_q_rot, void* d_k_cache,
                     void* d_v_cache) {
  PrepArgs p;
  int rc = prep_args(ctx, d_qg, d_kx, d_vx, d_q_norm_w, d_k_norm_w, T, Hq, Hkv, hd, rope_dims, eps, d_cos, d_sin,
                     table_npos, offset, d_offset, cap, d_q_rot, d_k_cache, d_v_cache, &p);
  if (rc) return rc;
  return prep_launch(ctx, p, hd);
}

// prep != null: the prep of the same rows has not been launched yet; it is done inside the
// attention launch where that launch's form can (the 1024-thread form, T <= 8, static offset), by
// its own launch first otherwise
static int sdpa_decode(ornith_ctx* ctx, const void* d_q_rot, const void* d_k_cache, const void* d_v_cache,
                       const void* d_qg, int T, int Hq, int Hkv, int hd, int offset, const int* d_offset, int cap,
                       float scale, void* d_out, const PrepArgs* prep) {
  ORN_REQUIRE(ctx && d_q_rot && d_k_cache && d_v_cache && d_qg && d_out, "sdpa_decode: null argument");
  ORN_REQUIRE(hd == 256 || hd == 128, "sdpa_decode: head_dim %d (128 or 256)", hd);
  // prompt chunks: the matrix-core kernel (outside the exact window, like the projections)
  if (T >= kPrefillRows && hd == 256 && !d_offset) {
    if (prep) {
      int rc = prep_launch(ctx, *prep, hd);
      if (rc) return rc;
    }
    return ornith_sdpa_prefill_gated(ctx, d_q_rot, d_k_cache, d_v_cache, d_qg, T, Hq, Hkv, hd, offset, cap,
                                     scale, d_out);
  }
  ORN_REQUIRE(T >= 1 && T <= 64 && Hq >= 1 && Hkv >= 1 && Hq % Hkv == 0, "sdpa_decode: T=%d Hq=%d Hkv=%d",
              T, Hq, Hkv);
  ORN_REQUIRE(offset >= 0 && offset + T <= cap, "sdpa_decode: rows [%d,%d) exceed capacity %d", offset,
              offset + T, cap);
  // with a device-side offset the grid must cover the whole cache
  const int nblk = d_offset ? (cap + ATT_KB - 1) / ATT_KB : (offset + T - 1) / ATT_KB + 1;
  const size_t per = (size_t)T * Hq * nblk;
  void* base = nullptr;
  int rc = ornith_scratch(ctx, (per * (hd + 2)) * 4 + 1024, &base);
  if (rc) return rc;
  ScratchCursor sc(base);
  SdpaArgs p{};
  p.q_rot = (const bf16_t*)d_q_rot;
  p.k_cache = (const bf16_t*)d_k_cache;
  p.v_cache = (const bf16_t*)d_v_cache;
  p.qg = (const bf16_t*)d_qg;
  p.d_offset = d_offset;
  p.part_m = sc.take<float>(per);
  p.part_l = sc.take<float>(per);
  p.part_o = sc.take<float>(per * hd);
  p.out = (bf16_t*)d_out;
  p.T = T;
  p.Hq = Hq;
  p.Hkv = Hkv;
  p.offset = offset;
  p.cap = cap;
  p.nblk = nblk;
  p.scale = scale;
  // one query head per workgroup: the arithmetic (256 keys x head_dim fmas per head) is what
  // bounds a block, so spreading heads over workgroups beats sharing the key loads
  dim3 grid(nblk, Hq, T);
  // few live blocks (short contexts): one 1024-thread block per (key block, head) finishes
  // soonest; many: the 256-thread form keeps more blocks in flight. Same sums either way.
  const int last_max = (d_offset ? cap - 1 : (offset + T - 1 < cap - 1 ? offset + T - 1 : cap - 1));
  const long live = (long)(last_max / ATT_KB + 1) * Hq * T;
  // four heads of a KV group a workgroup (the key / value block read once for the four) from a
  // workgroup for every fourth compute unit on: 25.6 us against 35.4 for one row at a 6.6 k
  // context (108 workgroups), 22.4 against 14.3 at 3 k (48)
  // (inside the first key block the finishing form is one launch instead of two)
  const bool four = (Hq / Hkv) % 4 == 0 && live / 4 >= ctx->compute_units / 4 && last_max >= ATT_KB;
  const bool many = live > 2L * ctx->compute_units || four;
  // one key block for every row, in the kernel form that knows how to finish: no merge launch
  p.finish = (last_max < ATT_KB && !many) ? 1 : 0;
  const bool fold = prep && !many && !d_offset && T <= 8 && ornith_option_fuse_attn_prep();
  PrepArgs pq{};
  if (prep) {
    pq = *prep;
    if (!fold) {
      const int rcp = prep_launch(ctx, pq, hd);
      if (rcp) return rcp;
    }
  }
  if (many) {
    const dim3 g4(nblk, Hq / 4, T);
    if (hd == 256) {
      if (four) hipLaunchKernelGGL((sdpa_partial_many_kernel<256, 4>), g4, dim3(256), 0, ctx->stream, p);
      else hipLaunchKernelGGL((sdpa_partial_many_kernel<256, 1>), grid, dim3(256), 0, ctx->stream, p);
    } else {
      if (four) hipLaunchKernelGGL((sdpa_partial_many_kernel<128, 4>), g4, dim3(256), 0, ctx->stream, p);
      else hipLaunchKernelGGL((sdpa_partial_many_kernel<128, 1>), grid, dim3(256), 0, ctx->stream, p);
    }
  } else if (hd == 256) {
    // 150 KB of LDS a block (the whole key block staged at once): asked for once per kernel
    if (!(ctx->lds_attr_set & 1)) {
      ORN_HIP(hipFuncSetAttribute((const void*)sdpa_partial_kernel<256, false>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, sdpa_stage_bytes<256>()));
      ORN_HIP(hipFuncSetAttribute((const void*)sdpa_partial_kernel<256, true>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, sdpa_stage_bytes<256>()));
      ctx->lds_attr_set |= 1;
    }
    if (fold)
      hipLaunchKernelGGL((sdpa_partial_kernel<256, true>), grid, dim3(SDPA_NT), sdpa_stage_bytes<256>(), ctx->stream, p, pq);
    else
      hipLaunchKernelGGL((sdpa_partial_kernel<256, false>), grid, dim3(SDPA_NT), sdpa_stage_bytes<256>(), ctx->stream, p, pq);
  } else {
    if (!(ctx->lds_attr_set & 2)) {
      ORN_HIP(hipFuncSetAttribute((const void*)sdpa_partial_kernel<128, false>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, sdpa_stage_bytes<128>()));
      ORN_HIP(hipFuncSetAttribute((const void*)sdpa_partial_kernel<128, true>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, sdpa_stage_bytes<128>()));
      ctx->lds_attr_set |= 2;
    }
    if (fold)
      hipLaunchKernelGGL((sdpa_partial_kernel<128, true>), grid, dim3(SDPA_NT), sdpa_stage_bytes<128>(), ctx->stream, p, pq);
    else
      hipLaunchKernelGGL((sdpa_partial_kernel<128, false>), grid, dim3(SDPA_NT), sdpa_stage_bytes<128>(), ctx->stream, p, pq);
  }
  ORN_LAUNCH_CHECK("sdpa_partial_kernel");
  if (p.finish) return ORNITH_OK;
  if (hd == 256)
    hipLaunchKernelGGL(sdpa_merge_kernel<256>, dim3(Hq, T), dim3(256), 0, ctx->stream, p);
  else
    hipLaunchKernelGGL(sdpa_merge_kernel<128>, dim3(Hq, T), dim3(128), 0, ctx->stream, p);
  ORN_LAUNCH_CHECK("sdpa_merge_kernel");
  return ORNITH_OK;
}

int ornith_sdpa_decode_gated(ornith_ctx* ctx, const void* d_q_rot, const void* d_k_cache,
                             const void* d_v_cache, const void* d_qg, int T, int Hq, int Hkv, int hd,
                             int offset, const int* d_offset, int cap, float scale, void* d_out) {
  return sdpa_decode(ctx, d_q_rot, d_k_cache, d_v_cache, d_qg, T, Hq, Hkv, hd, offset, d_offset, cap, scale, d_out,
                     nullptr);
}

int ornith_attn_decode(ornith_ctx* ctx, const void* d_qg, const void* d_kx, const void* d_vx,
                       const void* d_q_norm_w, const void* d_k_norm_w, int T, int Hq, int Hkv, int hd,
                       int rope_dims, float eps, const float* d_cos, const float* d_sin, int table_npos,
                       int offset, int cap, float scale, void* d_q_rot, void* d_k_cache, void* d_v_cache,
                       void* d_out) {
  PrepArgs p;
  int rc = prep_args(ctx, d_qg, d_kx, d_vx, d_q_norm_w, d_k_norm_w, T, Hq, Hkv, hd, rope_dims, eps, d_cos, d_sin,
                     table_npos, offset, nullptr, cap, d_q_rot, d_k_cache, d_v_cache, &p);
  if (rc) return rc;
  return sdpa_decode(ctx, d_q_rot, d_k_cache, d_v_cache, d_qg, T, Hq, Hkv, hd, offset, nullptr, cap, scale, d_out, &p);
}

}  // extern "C"
