// Q4_K / Q6_K tiled GEMM on the matrix cores, for prefill widths.
//
// Replaces kquant::{qmm_t, gather_qmm_t, matmul, gather_matmul}
// (/root/reference/src/ops/kquant.rs:783-1027; kernels/kquant_mm.h): Y[M,O] = X[M,K] . W^T
// with the weight tile dequantized to bf16 on the way into LDS and fp32 accumulation, and
// the expert-gathered form where each tile's rows belong to one routed expert.
//
// This is the one GEMM-shaped piece of the path (81 % of a prefill chunk in the
// reference, /root/reference/src/bin/arithmetic.rs:4-7), so it runs on MFMA
// (v_mfma_f32_32x32x16_bf16). Three forms, all reading the weights as k-quant codes (the 144 /
// 210 bytes per 256 weights that HBM holds) and dequantizing them with the arithmetic of
// kquant::dequantize (d*sc*q - dmin*m, resp. d*sc*q), rounded to bf16:
//   * kq_mm_kernel: a workgroup tile of BM x 128 outputs over K slabs of 128; activations go
//     global -> LDS as they are, weights are dequantized on the way into LDS; LDS rows padded by
//     8 elements so the 16-byte fragment reads of 32 consecutive rows spread over the banks;
//     four wavefronts: 2 x 2 of 64 x 64 outputs each for BM = 128, 1 x 4 of 64 x 32 for BM = 64.
//   * kq_mm_duo_kernel: the 256-row tile with producer and consumer wavefronts.
//   * kq_mm_reg_kernel: expert-gathered tiles of up to 192 rows with the weights dequantized
//     straight into MFMA operand registers (only activations through LDS).
// Up to four matrices of one kind and K over the same activations share a launch.
//
// Prefill is exempt from the "row r of a batch == row r alone" rule in the reference too
// (src/ops/invariant.rs:140-168): results agree with the mat-vec path to bf16 rounding of
// the weights and the order of the fp32 sums, not bit for bit.
#include <type_traits>

#include "dmath.h"
#include "rt.h"

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
// (a native vector: arrays of HIP's uint4 struct that are stored to LDS through casts are left in scratch memory)
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

constexpr int BN = 128, BK = 128, LDK = BK + 8;

struct MmArgs {
  const uint8_t* qs;
  const uint8_t* scales;
  const uint16_t* dm;
  const bf16_t* x;   // [x_rows, K]
  bf16_t* y;         // [y_rows, O]
  int M, O, K;
  // gathered form: tiles over (expert, row range) of an expert-sorted pair list
  const uint32_t* pair;        // [pairs] expert-sorted pair ids (row of y; row of x is pair / up_div)
  int up_div;                  // top_k for the gate / up projections (x row = token), 1 for down
  const uint32_t* tile_expert; // [tiles]
  const uint32_t* tile_start;  // [tiles] first pair
  const uint32_t* tile_count;  // [tiles] pairs in the tile (<= BM)
  const uint32_t* n_tiles;     // device scalar
  int sub;                     // workgroups a plan tile takes (plan tiles may be taller than the kernel's)
  int vec;                     // rows of y can be stored 16 bytes at a time
  // further matrices of the same kind and K over the same activations (plain form): the
  // workgroups from column block bx0 on belong to segment i
  struct Seg {
    const uint8_t* qs;
    const uint8_t* scales;
    const uint16_t* dm;
    bf16_t* y;
    int O, bx0, kind;
  } seg[3];
  int nseg;
  int kind;  // of the first matrix (read by the kernel instance for matrices of both kinds)
};

// the matrix a workgroup of the plain form works on; returns its column block there
__device__ __forceinline__ int pick_segment(MmArgs& a) {
  int bx = blockIdx.x;
#pragma unroll
  for (int i = 0; i < 3; ++i)
    if (i < a.nseg && (int)blockIdx.x >= a.seg[i].bx0) {
      a.qs = a.seg[i].qs;
      a.scales = a.seg[i].scales;
      a.dm = a.seg[i].dm;
      a.y = a.seg[i].y;
      a.O = a.seg[i].O;
      a.kind = a.seg[i].kind;
      bx = (int)blockIdx.x - a.seg[i].bx0;
    }
  return bx;
}

__device__ __forceinline__ uint32_t pack2(float a, float b) { return dm_f2bf2(a, b); }

// ---- weight slab pieces: loaded as codes into registers (so the loads of the next slab can
// be in flight while the matrix cores work on this one), dequantized on the way into LDS ----
struct BRegsQ4 {
  uint4 q0, q1;
  uint32_t s0, s1, s2, dmw;
};
struct BRegsQ6 {
  uint4 qa, qb, qh;
  uint2 sc;
  uint32_t d;
};

// 64-group `grp` of super-block `ib` of weight row `row`
__device__ __forceinline__ BRegsQ4 load_q4k(const MmArgs& a, int64_t row, int nb, int ib, int grp) {
  const int64_t blk = row * nb + ib;
  BRegsQ4 r;
  const uint4* q = reinterpret_cast<const uint4*>(a.qs + blk * 128 + grp * 32);
  r.q0 = q[0];
  r.q1 = q[1];
  const uint32_t* sc = reinterpret_cast<const uint32_t*>(a.scales + blk * 12);
  r.s0 = sc[0];
  r.s1 = sc[1];
  r.s2 = sc[2];
  r.dmw = *reinterpret_cast<const uint32_t*>(a.dm + blk * 2);
  return r;
}

// 64 weights as bf16 into dst[0..64): d*sc*q - dmin*m (kquant::dequantize, q4k.metal:64-96).
// Two and a half vector instructions a weight (byte -> float, one fma, half a two-value bf16
// conversion): the dequantization shares the wavefront with the MFMAs it feeds, so its length
// is GEMM time.
__device__ __forceinline__ void dequant_q4k(const BRegsQ4& r, int grp, bf16_t* dst) {
  // the 6-bit scale and min of sub-blocks 2*grp and 2*grp + 1, two bytes each way
  const int sh16 = (grp & 1) * 16;
  const uint32_t a = r.s0 >> sh16, b = r.s1 >> sh16, c = r.s2 >> sh16;
  const bool low = grp < 2;
  const uint32_t sc16 = low ? (a & 0x3f3fu) : ((c & 0x0f0fu) | ((a & 0xc0c0u) >> 2));
  const uint32_t m16 = low ? (b & 0x3f3fu) : (((c >> 4) & 0x0f0fu) | ((b & 0xc0c0u) >> 2));
  const float d = dm_h2f((f16_t)(r.dmw & 0xffffu)), dmin = dm_h2f((f16_t)(r.dmw >> 16));
  const float dd0 = d * dm_ubyte<0>(sc16), dd1 = d * dm_ubyte<1>(sc16);
  const float mm0 = -(dmin * dm_ubyte<0>(m16)), mm1 = -(dmin * dm_ubyte<1>(m16));
  uint32_t* out = reinterpret_cast<uint32_t*>(dst);
  const uint32_t w[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t lo = w[i] & 0x0f0f0f0fu, hi = (w[i] >> 4) & 0x0f0f0f0fu;
    out[2 * i] = pack2(dm_fma(dd0, dm_ubyte<0>(lo), mm0), dm_fma(dd0, dm_ubyte<1>(lo), mm0));  // low nibbles: weights 4i .. 4i+3
    out[2 * i + 1] = pack2(dm_fma(dd0, dm_ubyte<2>(lo), mm0), dm_fma(dd0, dm_ubyte<3>(lo), mm0));
    out[16 + 2 * i] = pack2(dm_fma(dd1, dm_ubyte<0>(hi), mm1), dm_fma(dd1, dm_ubyte<1>(hi), mm1));  // high nibbles: the same + 32
    out[16 + 2 * i + 1] = pack2(dm_fma(dd1, dm_ubyte<2>(hi), mm1), dm_fma(dd1, dm_ubyte<3>(hi), mm1));
  }
}

// positions l in [16*j, 16*j + 16) of the 128-half `hh` of super-block `ib`
__device__ __forceinline__ BRegsQ6 load_q6k(const MmArgs& a, int64_t row, int nb, int ib, int hh, int j) {
  const int64_t blk = row * nb + ib;
  const uint8_t* base = a.qs + blk * 192;
  BRegsQ6 r;
  r.qa = *reinterpret_cast<const uint4*>(base + 64 * hh + 16 * j);
  r.qb = *reinterpret_cast<const uint4*>(base + 64 * hh + 32 + 16 * j);
  r.qh = *reinterpret_cast<const uint4*>(base + 128 + 32 * hh + 16 * j);
  r.sc = *reinterpret_cast<const uint2*>(a.scales + blk * 16 + 8 * hh);
  r.d = a.dm[blk];
  return r;
}

// the four weights l, l+32, l+64, l+96 of each position, d*sc*(q - 32) (q6k.metal:47-77), as
// bf16 into dst[0..128) (dst = start of the half). The 6-bit codes are put together four at a
// time in a word; (q - 32) * s is one fma with -32 s.
__device__ __forceinline__ void dequant_q6k(const BRegsQ6& r, int j, bf16_t* dst) {
  const float d = dm_h2f((f16_t)r.d);
  const uint32_t scw[2] = {r.sc.x, r.sc.y};
  auto scale = [&](int i) { return (float)(int)(int8_t)((scw[i >> 2] >> (8 * (i & 3))) & 0xffu); };
  const float sv[4] = {d * scale(j), d * scale(j + 2), d * scale(j + 4), d * scale(j + 6)};
  const float off[4] = {-32.f * sv[0], -32.f * sv[1], -32.f * sv[2], -32.f * sv[3]};
  const uint32_t la[4] = {r.qa.x, r.qa.y, r.qa.z, r.qa.w}, lb[4] = {r.qb.x, r.qb.y, r.qb.z, r.qb.w},
                 hv[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
  uint32_t* out = reinterpret_cast<uint32_t*>(dst);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t A = la[i], B = lb[i], H = hv[i];
    const uint32_t c[4] = {(A & 0x0f0f0f0fu) | ((H << 4) & 0x30303030u), (B & 0x0f0f0f0fu) | ((H << 2) & 0x30303030u),
                           ((A >> 4) & 0x0f0f0f0fu) | (H & 0x30303030u), ((B >> 4) & 0x0f0f0f0fu) | ((H >> 2) & 0x30303030u)};
    const int e = (16 * j + 4 * i) >> 1;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      out[16 * g + e] = pack2(dm_fma(sv[g], dm_ubyte<0>(c[g]), off[g]), dm_fma(sv[g], dm_ubyte<1>(c[g]), off[g]));
      out[16 * g + e + 1] = pack2(dm_fma(sv[g], dm_ubyte<2>(c[g]), off[g]), dm_fma(sv[g], dm_ubyte<3>(c[g]), off[g]));
    }
  }
}

template <int KIND>
struct BRegsOf { typedef BRegsQ4 type; };
template <>
struct BRegsOf<ORNITH_Q6K> { typedef BRegsQ6 type; };

#ifdef ORN_TIMING
__device__ long long g_mm_marks[1024][8];
#define MM_MARK(i, cond) do { if (threadIdx.x == 0 && blockIdx.x == 0 && blockIdx.y < 1024 && (cond)) g_mm_marks[blockIdx.y][i] = wall_clock64(); } while (0)
#define MM_MARK_P(i, cond) do { if (threadIdx.x == 256 && blockIdx.x == 0 && blockIdx.y < 1024 && (cond)) g_mm_marks[blockIdx.y][i] = wall_clock64(); } while (0)
extern "C" __attribute__((visibility("default"))) int ornith_debug_marks_mm(long long* out) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_mm_marks), sizeof(g_mm_marks));
}
#else
#define MM_MARK(i, cond)
#define MM_MARK_P(i, cond)
#endif

// ---- epilogue ------------------------------------------------------------------------------
// The MFMA result has one output column per lane (D[row = 8*b + 4*(lane/32) + r][col = lane%32]
// = acc[4*b + r]): stored from there, a tile row leaves in 2-byte pieces, 64 store instructions
// per 32 x 32 tile. Each wavefront instead turns its own window of the tile around in LDS (the
// slab buffers are free after the last barrier; no other wavefront touches the window, so no
// barrier is needed) and stores 16 bytes a lane, eight lanes a 128-byte row piece. `vec`: the
// rows of y are 16-byte aligned (O a multiple of 8); otherwise the direct 2-byte stores.
template <int TM, int TN, bool GATHER>
__device__ __forceinline__ void store_tile(const MmArgs& a, const f32x16_t (&acc)[TM][TN], bf16_t* cs, int row0,
                                           int col0, int lane, int n0, int m0, int rows_here, const uint32_t* s_dst,
                                           bool vec, int ld = LDK) {
  constexpr int WTM = TM * 32, WTN = TN * 32, PPR = WTN / 8;
  if (!vec) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int o = n0 + col0 + j * 32 + (lane & 31);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int r = row0 + i * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
          if (r < rows_here && o < a.O) {
            const int64_t dst = GATHER ? (int64_t)s_dst[r] : (int64_t)(m0 + r);
            a.y[dst * a.O + o] = dm_f2bf(acc[i][j][e]);
          }
        }
      }
    return;
  }
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      bf16_t* w = cs + (row0 + i * 32 + 4 * (lane >> 5)) * ld + col0 + j * 32 + (lane & 31);
#pragma unroll
      for (int e = 0; e < 16; e += 2) {
        const uint32_t pk = dm_f2bf2(acc[i][j][e], acc[i][j][e + 1]);
        w[(8 * (e >> 2) + (e & 3)) * ld] = (bf16_t)(pk & 0xffffu);
        w[(8 * (e >> 2) + (e & 3) + 1) * ld] = (bf16_t)(pk >> 16);
      }
    }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
  for (int p0 = 0; p0 < WTM * PPR; p0 += 64) {
    const int p = p0 + lane, r = row0 + p / PPR, c = col0 + (p % PPR) * 8;
    if (r < rows_here && n0 + c < a.O) {
      const int64_t dst = GATHER ? (int64_t)s_dst[r] : (int64_t)(m0 + r);
      *reinterpret_cast<u32x4_t*>(a.y + dst * a.O + n0 + c) = *reinterpret_cast<const u32x4_t*>(cs + r * ld + c);
    }
  }
}

// BM = 256: 2 x 2 wavefronts of 128 x 64; BM = 128: 2 x 2 of 64 x 64; BM = 64: 1 x 4 of 64 x 32.
// KIND = kMixed: the matrices of the launch differ in kind (a workgroup asks its own).
constexpr int kMixed = 2;
template <int KIND, int BM, bool GATHER>
__global__ __launch_bounds__(256) void kq_mm_kernel(MmArgs a) {
  constexpr int WM = BM >= 128 ? 2 : 1, WN = 4 / WM;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int NA = BM * 16 / 256;  // 16-byte pieces of the activation slab per thread
  __shared__ __attribute__((aligned(16))) bf16_t As[BM][LDK];
  __shared__ __attribute__((aligned(16))) bf16_t Bs[BN][LDK];
  __shared__ uint32_t s_src[BM], s_dst[BM];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int n0 = (GATHER ? (int)blockIdx.x : pick_segment(a)) * BN;
  const int nb = a.K >> 8;

  int rows_here, m0 = 0;
  int64_t wrow0 = 0;  // first weight row of this tile's matrix
  if constexpr (GATHER) {
    // a plan tile of more rows than BM is worked on by a.sub workgroups, BM rows each
    const uint32_t tile = blockIdx.y / (uint32_t)a.sub, part = blockIdx.y % (uint32_t)a.sub;
    if (tile >= *a.n_tiles) return;
    const uint32_t e = a.tile_expert[tile], st = a.tile_start[tile] + part * BM;
    rows_here = min((int)a.tile_count[tile] - (int)(part * BM), BM);
    if (rows_here <= 0) return;
    wrow0 = (int64_t)e * a.O;
    for (int r = tid; r < BM; r += 256) {
      const uint32_t p = r < rows_here ? a.pair[st + r] : 0u;
      s_src[r] = p / (uint32_t)a.up_div;
      s_dst[r] = p;
    }
    __syncthreads();
  } else {
    m0 = blockIdx.y * BM;
    rows_here = min(BM, a.M - m0);
  }

  // this thread's pieces of a slab: NA activation pieces and one weight piece
  const int br = tid >> 1, bpart = tid & 1;
  const int64_t brow = wrow0 + min(n0 + br, a.O - 1);
  const bf16_t* asrc[NA];
#pragma unroll
  for (int i = 0; i < NA; ++i) {
    const int idx = tid + 256 * i, r = idx >> 4, c8 = idx & 15;
    // rows past the end of the tile read a valid row instead (pair 0's, or the last one): what
    // they produce lands in output rows the epilogue does not store, and no load needs a branch
    const int64_t src = GATHER ? (int64_t)s_src[r] : (int64_t)min(m0 + r, a.M - 1);
    asrc[i] = a.x + src * a.K + 8 * c8;
  }
  u32x4_t areg[NA];
  BRegsQ4 breg4;
  BRegsQ6 breg6;
  const bool q4 = KIND == kMixed ? a.kind == ORNITH_Q4K : KIND == ORNITH_Q4K;
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < NA; ++i)
      areg[i] = *reinterpret_cast<const u32x4_t*>(asrc[i] + k0);
    if (q4)
      breg4 = load_q4k(a, brow, nb, k0 >> 8, ((k0 & 255) >> 6) + bpart);
    else
      breg6 = load_q6k(a, brow, nb, k0 >> 8, (k0 & 255) >> 7, bpart);
  };

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  fetch(0);
  for (int k0 = 0; k0 < a.K; k0 += BK) {
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const int idx = tid + 256 * i;
      *reinterpret_cast<u32x4_t*>(&As[idx >> 4][8 * (idx & 15)]) = areg[i];
    }
    if (q4)
      dequant_q4k(breg4, ((k0 & 255) >> 6) + bpart, &Bs[br][64 * bpart]);
    else
      dequant_q6k(breg6, bpart, &Bs[br][0]);
    __syncthreads();
    if (k0 + BK < a.K) fetch(k0 + BK);  // in flight while the matrix cores run
    // fragments of step kk + 1 leave LDS while the matrix cores work on step kk
    bf16x8_t af[2][TM], bfr[2][TN];
    auto frags = [&](int kk, bf16x8_t (&fa)[TM], bf16x8_t (&fb)[TN]) {
      const int kc = kk * 16 + 8 * (lane >> 5);
#pragma unroll
      for (int i = 0; i < TM; ++i)
        fa[i] = *reinterpret_cast<const bf16x8_t*>(&As[wm * WTM + i * 32 + (lane & 31)][kc]);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        fb[j] = *reinterpret_cast<const bf16x8_t*>(&Bs[wn * WTN + j * 32 + (lane & 31)][kc]);
    };
    frags(0, af[0], bfr[0]);
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      if (kk + 1 < BK / 16) frags(kk + 1, af[(kk + 1) & 1], bfr[(kk + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);  // or the reads are sunk to just before their use
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[kk & 1][i], bfr[kk & 1][j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
  }

  store_tile<TM, TN, GATHER>(a, acc, &As[0][0], wm * WTM, wn * WTN, lane, n0, m0, rows_here, s_dst, a.vec != 0);
}

// ---- the same GEMM with producers and consumers --------------------------------------------
// Eight wavefronts a workgroup. Four (one a SIMD) run the MFMAs of K slab s out of one LDS
// buffer; the other four meanwhile write slab s + 1 into the other buffer (activations as they
// are, weights dequantized, from registers loaded two slabs ahead): the vector work of the
// dequantization and the matrix cores then run side by side on every SIMD instead of one after
// the other in one wavefront. K slabs of 64, one barrier a slab.
constexpr int BK2 = 64, LD2 = BK2 + 8;

struct PipeQ4 {
  float dd, mm;
  uint32_t w[8];  // this thread's nibble of each of the 32 code bytes, 4 to a word
};
struct PipeQ6 {
  float sa, sb, oa, ob;
  uint32_t ca[4], cb[4];  // the 6-bit codes of the positions' two weights, 4 to a word
};

// what a thread needs of its 32 weights before the quarters: scale, offset, codes
__device__ __forceinline__ PipeQ4 pipe_prepare(const BRegsQ4& r, int grp, int half) {
  const int sh16 = (grp & 1) * 16;
  const uint32_t a = r.s0 >> sh16, b = r.s1 >> sh16, c = r.s2 >> sh16;
  const bool low = grp < 2;
  const uint32_t sc16 = low ? (a & 0x3f3fu) : ((c & 0x0f0fu) | ((a & 0xc0c0u) >> 2));
  const uint32_t m16 = low ? (b & 0x3f3fu) : (((c >> 4) & 0x0f0fu) | ((b & 0xc0c0u) >> 2));
  const float d = dm_h2f((f16_t)(r.dmw & 0xffffu)), dmin = dm_h2f((f16_t)(r.dmw >> 16));
  PipeQ4 p;
  p.dd = d * dm_ubyte<0>(sc16 >> (8 * half));
  p.mm = -(dmin * dm_ubyte<0>(m16 >> (8 * half)));
  const uint32_t w[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
#pragma unroll
  for (int i = 0; i < 8; ++i) p.w[i] = (w[i] >> (4 * half)) & 0x0f0f0f0fu;
  return p;
}
// quarter q: weights 8q .. 8q + 8 of the thread's 32, to dst[8q ..]
__device__ __forceinline__ void pipe_quarter(const PipeQ4& p, int q, bf16_t* dst) {
  u32x4_t o;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const uint32_t c = p.w[2 * q + h];
    o[2 * h] = pack2(dm_fma(p.dd, dm_ubyte<0>(c), p.mm), dm_fma(p.dd, dm_ubyte<1>(c), p.mm));
    o[2 * h + 1] = pack2(dm_fma(p.dd, dm_ubyte<2>(c), p.mm), dm_fma(p.dd, dm_ubyte<3>(c), p.mm));
  }
  *reinterpret_cast<u32x4_t*>(dst + 8 * q) = o;
}

// Q6_K: the 64-slab `sub` of a 128-half holds weights l and l + 32 (sub 0: low nibbles) or
// l + 64 and l + 96 (sub 1: high nibbles) of positions l; a thread has positions 16j .. 16j + 16
__device__ __forceinline__ PipeQ6 pipe_prepare(const BRegsQ6& r, int j, int sub) {
  const float d = dm_h2f((f16_t)r.d);
  const uint32_t scw[2] = {r.sc.x, r.sc.y};
  auto scale = [&](int i) { return (float)(int)(int8_t)((scw[i >> 2] >> (8 * (i & 3))) & 0xffu); };
  PipeQ6 p;
  p.sa = d * scale(j + 4 * sub);
  p.sb = d * scale(j + 2 + 4 * sub);
  p.oa = -32.f * p.sa;
  p.ob = -32.f * p.sb;
  const uint32_t la[4] = {r.qa.x, r.qa.y, r.qa.z, r.qa.w}, lb[4] = {r.qb.x, r.qb.y, r.qb.z, r.qb.w},
                 hv[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t H = hv[i] >> (4 * sub);  // bits 0-1: the A-side weight's, bits 2-3: the B-side's
    p.ca[i] = ((la[i] >> (4 * sub)) & 0x0f0f0f0fu) | ((H << 4) & 0x30303030u);
    p.cb[i] = ((lb[i] >> (4 * sub)) & 0x0f0f0f0fu) | ((H << 2) & 0x30303030u);
  }
  return p;
}
// quarter q: positions 16j + 4q .. + 4: A-side weights to dst[16j + 4q ..], B-side 32 further on
__device__ __forceinline__ void pipe_quarter(const PipeQ6& p, int q, int j, bf16_t* dst) {
  uint2 oa, ob;
  oa.x = pack2(dm_fma(p.sa, dm_ubyte<0>(p.ca[q]), p.oa), dm_fma(p.sa, dm_ubyte<1>(p.ca[q]), p.oa));
  oa.y = pack2(dm_fma(p.sa, dm_ubyte<2>(p.ca[q]), p.oa), dm_fma(p.sa, dm_ubyte<3>(p.ca[q]), p.oa));
  ob.x = pack2(dm_fma(p.sb, dm_ubyte<0>(p.cb[q]), p.ob), dm_fma(p.sb, dm_ubyte<1>(p.cb[q]), p.ob));
  ob.y = pack2(dm_fma(p.sb, dm_ubyte<2>(p.cb[q]), p.ob), dm_fma(p.sb, dm_ubyte<3>(p.cb[q]), p.ob));
  *reinterpret_cast<uint2*>(dst + 16 * j + 4 * q) = oa;
  *reinterpret_cast<uint2*>(dst + 32 + 16 * j + 4 * q) = ob;
}

template <int KIND>
struct PipeOf { typedef PipeQ4 type; };
template <>
struct PipeOf<ORNITH_Q6K> { typedef PipeQ6 type; };


template <int KIND, int BM, bool GATHER>
__global__ __launch_bounds__(512) void kq_mm_duo_kernel(MmArgs a) {
  constexpr int WM = BM >= 128 ? 2 : 1, WN = 4 / WM;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int NA = BM * 8 / 256;  // 16-byte pieces of an activation slab per thread of one role
  // The producers set the pace (activations and weights into LDS, the loads asked for), the
  // consumers wait a third of a slab at its barrier: the consumers carry the upper half of the
  // activation rows into LDS themselves (asked for two slabs ahead, written before the slab's MFMAs).
  constexpr int NAP = NA / 2, NAC = NA - NAP;
  __shared__ __attribute__((aligned(16))) bf16_t As[2][BM][LD2];
  __shared__ __attribute__((aligned(16))) bf16_t Bs[2][BN][LD2];
  __shared__ uint32_t s_src[BM], s_dst[BM];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = (GATHER ? (int)blockIdx.x : pick_segment(a)) * BN;
  const int nb = a.K >> 8;
  const int nslab = a.K / BK2;  // K is a multiple of 256: a multiple of four slabs

  int rows_here, m0 = 0;
  int64_t wrow0 = 0;
  if constexpr (GATHER) {
    if (blockIdx.y >= *a.n_tiles) return;
    const uint32_t e = a.tile_expert[blockIdx.y], st = a.tile_start[blockIdx.y];
    rows_here = (int)a.tile_count[blockIdx.y];
    wrow0 = (int64_t)e * a.O;
    for (int r = tid; r < BM; r += 512) {
      const uint32_t p = r < rows_here ? a.pair[st + r] : 0u;
      s_src[r] = p / (uint32_t)a.up_div;
      s_dst[r] = p;
    }
    __syncthreads();
  } else {
    m0 = blockIdx.y * BM;
    rows_here = min(BM, a.M - m0);
  }
  using Set0 = std::integral_constant<int, 0>;
  using Set1 = std::integral_constant<int, 1>;

  if (wave >= 4) {
    // ---- producers ----
    const int ptid = tid - 256;
    const int br = ptid >> 1, bpart = ptid & 1;
    const int64_t brow = wrow0 + min(n0 + br, a.O - 1);
    const bf16_t* asrc[NAP];
#pragma unroll
    for (int i = 0; i < NAP; ++i) {
      const int idx = ptid + 256 * i, r = idx >> 3, c8 = idx & 7;
      // rows past the end of the tile read a valid row: what they produce is never stored
      const int64_t src = GATHER ? (int64_t)s_src[r] : (int64_t)min(m0 + r, a.M - 1);
      asrc[i] = a.x + src * a.K + 8 * c8;
    }
    // Four register sets: slab k travels in set k & 3 and is asked for four slabs before it is
    // written to LDS buffer k & 1, so a load has about four slab times to arrive. (Sets and
    // buffers are picked by constants: an index known only at run time would put the arrays
    // in scratch memory.)
    u32x4_t areg[4][NAP];
    typename BRegsOf<KIND>::type breg[4];
    auto fetch = [&](auto set, int k0) {
      constexpr int SET = decltype(set)::value;
#pragma unroll
      for (int i = 0; i < NAP; ++i) areg[SET][i] = *reinterpret_cast<const u32x4_t*>(asrc[i] + k0);
      if constexpr (KIND == ORNITH_Q4K)
        breg[SET] = load_q4k(a, brow, nb, k0 >> 8, (k0 & 255) >> 6);
      else
        breg[SET] = load_q6k(a, brow, nb, k0 >> 8, (k0 & 255) >> 7, bpart);
    };
    auto write = [&](auto set, int k0) {
      constexpr int SET = decltype(set)::value, BUF = SET & 1;
#pragma unroll
      for (int i = 0; i < NAP; ++i) {
        const int idx = ptid + 256 * i;
        *reinterpret_cast<u32x4_t*>(&As[BUF][idx >> 3][8 * (idx & 7)]) = areg[SET][i];
      }
      MM_MARK_P(7, k0 == 9 * BK2);
      if constexpr (KIND == ORNITH_Q4K) {
        const PipeQ4 pp = pipe_prepare(breg[SET], (k0 & 255) >> 6, bpart);
#pragma unroll
        for (int q = 0; q < 4; ++q) pipe_quarter(pp, q, &Bs[BUF][br][32 * bpart]);
      } else {
        const PipeQ6 pp = pipe_prepare(breg[SET], bpart, (k0 & 127) >> 6);
#pragma unroll
        for (int q = 0; q < 4; ++q) pipe_quarter(pp, q, bpart, &Bs[BUF][br][0]);
      }
    };
    using Set2 = std::integral_constant<int, 2>;
    using Set3 = std::integral_constant<int, 3>;
    fetch(Set0{}, 0);
    fetch(Set1{}, BK2);
    fetch(Set2{}, 2 * BK2);
    fetch(Set3{}, 3 * BK2);
    write(Set0{}, 0);
    if (4 < nslab) fetch(Set0{}, 4 * BK2);
    __syncthreads();
    // while the consumers work on slab s + u: slab s + u + 1 into the other buffer, then its
    // register set asks for the slab four further on
    auto step = [&](auto set, int k) {
      MM_MARK_P(3, k == 9);
      if (k < nslab) write(set, k * BK2);
      MM_MARK_P(4, k == 9);
      if (k + 4 < nslab) fetch(set, (k + 4) * BK2);
      MM_MARK_P(5, k == 9);
      __syncthreads();
      MM_MARK_P(6, k == 9);
    };
    for (int s = 0; s < nslab; s += 4) {
      step(Set1{}, s + 1);
      step(Set2{}, s + 2);
      step(Set3{}, s + 3);
      step(Set0{}, s + 4);
    }
    return;
  }

  // ---- consumers ----
  const int wm = wave / WN, wn = wave % WN;
  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  // the consumers' share of the activation slab: pieces NAP .. NA of the same index scheme; slab
  // k travels in register set k & 1 into LDS buffer k & 1
  const bf16_t* csrc[NAC];
#pragma unroll
  for (int i = 0; i < NAC; ++i) {
    const int idx = tid + 256 * (NAP + i), r = idx >> 3, c8 = idx & 7;
    const int64_t src = GATHER ? (int64_t)s_src[r] : (int64_t)min(m0 + r, a.M - 1);
    csrc[i] = a.x + src * a.K + 8 * c8;
  }
  u32x4_t creg[2][NAC];
  auto cfetch = [&](auto set, int k) {
    constexpr int SET = decltype(set)::value;
    if (k < nslab) {
#pragma unroll
      for (int i = 0; i < NAC; ++i) creg[SET][i] = *reinterpret_cast<const u32x4_t*>(csrc[i] + k * BK2);
    }
  };
  auto cwrite = [&](auto set, int k) {
    constexpr int SET = decltype(set)::value;
    if (k < nslab) {
#pragma unroll
      for (int i = 0; i < NAC; ++i) {
        const int idx = tid + 256 * (NAP + i);
        *reinterpret_cast<u32x4_t*>(&As[SET][idx >> 3][8 * (idx & 7)]) = creg[SET][i];
      }
    }
  };
  auto frags = [&](int buf, int kk, bf16x8_t (&fa)[TM], bf16x8_t (&fb)[TN]) {
    const int kc = kk * 16 + 8 * (lane >> 5);
#pragma unroll
    for (int i = 0; i < TM; ++i)
      fa[i] = *reinterpret_cast<const bf16x8_t*>(&As[buf][wm * WTM + i * 32 + (lane & 31)][kc]);
#pragma unroll
    for (int j = 0; j < TN; ++j)
      fb[j] = *reinterpret_cast<const bf16x8_t*>(&Bs[buf][wn * WTN + j * 32 + (lane & 31)][kc]);
  };
  auto slab = [&](int buf) {
    bf16x8_t af[2][TM], bfr[2][TN];
    frags(buf, 0, af[0], bfr[0]);
#pragma unroll
    for (int kk = 0; kk < BK2 / 16; ++kk) {
      if (kk + 1 < BK2 / 16) frags(buf, kk + 1, af[(kk + 1) & 1], bfr[(kk + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);  // or the reads are sunk to just before their use
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[kk & 1][i], bfr[kk & 1][j], acc[i][j], 0, 0, 0);
    }
  };
  cfetch(Set0{}, 0);
  cfetch(Set1{}, 1);
  cwrite(Set0{}, 0);
  cfetch(Set0{}, 2);
  __syncthreads();  // slab 0 is in buffer 0
  for (int s = 0; s < nslab; s += 2) {  // (the producers count the same barriers, four a turn)
    MM_MARK(0, s == 8);
    cwrite(Set1{}, s + 1);  // into the buffer the MFMAs below do not read
    cfetch(Set1{}, s + 3);
    slab(0);
    MM_MARK(1, s == 8);
    __syncthreads();
    MM_MARK(2, s == 8);
    cwrite(Set0{}, s + 2);
    cfetch(Set0{}, s + 4);
    slab(1);
    __syncthreads();
  }

  static_assert(2 * LD2 >= LDK, "the tile does not fit over the slab buffers");
  store_tile<TM, TN, GATHER>(a, acc, &As[0][0][0], wm * WTM, wn * WTN, lane, n0, m0, rows_here, s_dst, a.vec != 0);
}

// ---- the gathered GEMM with the weights kept out of LDS -------------------------------------
// A 64 x 64 wavefront tile reads 4 KB of fragments out of LDS for every four MFMAs: at the
// matrix cores' full rate that is all the LDS bandwidth a compute unit has, so the kernels
// above cannot pass half of the peak. Here a wavefront owns 64 output columns over ALL rows of
// the tile (32 * TM, up to 192: an expert's whole share of a 4096-token chunk in one tile, so
// its weights are dequantized once), and dequantizes the weights of its columns straight into
// MFMA operand registers: a lane of v_mfma_f32_32x32x16_bf16 supplies 8 consecutive k of one
// weight row, which is 4 bytes of Q4_K nibbles / Q6_K codes, and the order of the k steps
// inside a slab is free as long as the activation fragments follow it. Only the activations go
// through LDS (written once a slab, read by the four wavefronts: 32 * TM * 32 bytes per
// 2 * TM MFMAs), and the vector work of the dequantization sits between the MFMAs of the same
// wavefront. One wavefront a SIMD (the accumulators take 32 * TM registers), K slabs of 128.
//
// k step t (0..7) of a slab, lane half h: k = 32 * (t >> 1) + 16 * h + 8 * (t & 1) .. + 8.
//   Q4_K: the slab is two 64-groups; the lane holds bytes 16h .. 16h + 16 of each (low nibbles:
//         weights 16h + i, high nibbles: 32 + 16h + i).
//   Q6_K: the slab is a 128-half; the lane holds positions 16h .. 16h + 16 (their weights l,
//         l + 32, l + 64, l + 96 are quarters t >> 1 of the slab).
struct RawQ4 {
  u32x4_t q[2];
  uint32_t s0, s1, s2, dmw;
};
struct RawQ6 {
  u32x4_t qa, qb, qh;
  uint32_t sc0, sc1, d;
};
template <int KIND>
struct RawOf { typedef RawQ4 type; };
template <>
struct RawOf<ORNITH_Q6K> { typedef RawQ6 type; };

// Every load of the main loop is a base the whole workgroup shares, moved from slab to slab by
// scalar arithmetic, plus a 32-bit byte offset a lane computes once: no vector instruction is
// spent on addresses between the MFMAs.
struct RawOff {
  uint32_t q, s, d;  // byte offsets of the lane's weight row in qs / scales / dm (+ 16 * h in q)
};
__device__ __forceinline__ RawOff raw_offsets(int kind, int64_t row, int nb, int h) {
  RawOff o;
  o.q = (uint32_t)(row * nb * (kind == ORNITH_Q4K ? 128 : 192) + 16 * h);
  o.s = (uint32_t)(row * nb * (kind == ORNITH_Q4K ? 12 : 16));
  o.d = (uint32_t)(row * nb * (kind == ORNITH_Q4K ? 4 : 2));
  return o;
}
template <class V>
__device__ __forceinline__ V ld_off(const uint8_t* base, uint32_t off) {
  return *reinterpret_cast<const V*>(base + off);
}
__device__ __forceinline__ void raw_load(RawQ4& r, const MmArgs& a, const RawOff& o, int slab) {
  const uint8_t* q = a.qs + slab * 64;
  r.q[0] = ld_off<u32x4_t>(q, o.q);
  r.q[1] = ld_off<u32x4_t>(q + 32, o.q);
  const uint8_t* sc = a.scales + (slab >> 1) * 12;
  r.s0 = ld_off<uint32_t>(sc, o.s);
  r.s1 = ld_off<uint32_t>(sc + 4, o.s);
  r.s2 = ld_off<uint32_t>(sc + 8, o.s);
  r.dmw = ld_off<uint32_t>(reinterpret_cast<const uint8_t*>(a.dm) + (slab >> 1) * 4, o.d);
}
__device__ __forceinline__ void raw_load(RawQ6& r, const MmArgs& a, const RawOff& o, int slab) {
  const int hh = slab & 1;
  const uint8_t* base = a.qs + (slab >> 1) * 192;
  r.qa = ld_off<u32x4_t>(base + 64 * hh, o.q);
  r.qb = ld_off<u32x4_t>(base + 64 * hh + 32, o.q);
  r.qh = ld_off<u32x4_t>(base + 128 + 32 * hh, o.q);
  const uint8_t* sc = a.scales + slab * 8;
  r.sc0 = ld_off<uint32_t>(sc, o.s);
  r.sc1 = ld_off<uint32_t>(sc + 4, o.s);
  r.d = ld_off<uint16_t>(reinterpret_cast<const uint8_t*>(a.dm) + (slab >> 1) * 2, o.d);
}

// scale and offset of the slab's four quarters (w = s * code + o)
template <int HH>
__device__ __forceinline__ void raw_scales(const RawQ4& r, int, float (&s)[4], float (&o)[4]) {
  const float d = dm_h2f((f16_t)(r.dmw & 0xffffu)), dmin = dm_h2f((f16_t)(r.dmw >> 16));
  // sub-blocks 4 * HH .. + 4: the 6-bit scales and mins, four to a word
  uint32_t sc4, m4;
  if constexpr (HH == 0) {
    sc4 = r.s0 & 0x3f3f3f3fu;
    m4 = r.s1 & 0x3f3f3f3fu;
  } else {
    sc4 = (r.s2 & 0x0f0f0f0fu) | ((r.s0 & 0xc0c0c0c0u) >> 2);
    m4 = ((r.s2 >> 4) & 0x0f0f0f0fu) | ((r.s1 & 0xc0c0c0c0u) >> 2);
  }
  s[0] = d * dm_ubyte<0>(sc4);
  s[1] = d * dm_ubyte<1>(sc4);
  s[2] = d * dm_ubyte<2>(sc4);
  s[3] = d * dm_ubyte<3>(sc4);
  o[0] = -(dmin * dm_ubyte<0>(m4));
  o[1] = -(dmin * dm_ubyte<1>(m4));
  o[2] = -(dmin * dm_ubyte<2>(m4));
  o[3] = -(dmin * dm_ubyte<3>(m4));
}
template <int HH>
__device__ __forceinline__ void raw_scales(const RawQ6& r, int h, float (&s)[4], float (&o)[4]) {
  const float d = dm_h2f((f16_t)r.d);
  // the scale of quarter qd and lane half h is byte 2 * qd + h of the half's eight
  const uint32_t w0 = r.sc0 >> (8 * h), w1 = r.sc1 >> (8 * h);
  s[0] = d * (float)(int)(int8_t)(w0 & 0xffu);
  s[1] = d * (float)(int)(int8_t)((w0 >> 16) & 0xffu);
  s[2] = d * (float)(int)(int8_t)(w1 & 0xffu);
  s[3] = d * (float)(int)(int8_t)((w1 >> 16) & 0xffu);
#pragma unroll
  for (int i = 0; i < 4; ++i) o[i] = -32.f * s[i];
}

// the two code words (four codes each) of k step T and the quarter they are scaled by
template <int T>
__device__ __forceinline__ void raw_codes(const RawQ4& r, uint32_t& c0, uint32_t& c1, int& quarter) {
  constexpr int G = T >> 2, NIB = (T >> 1) & 1, W = 2 * (T & 1);
  c0 = (r.q[G][W] >> (4 * NIB)) & 0x0f0f0f0fu;
  c1 = (r.q[G][W + 1] >> (4 * NIB)) & 0x0f0f0f0fu;
  quarter = 2 * G + NIB;
}
template <int T>
__device__ __forceinline__ void raw_codes(const RawQ6& r, uint32_t& c0, uint32_t& c1, int& quarter) {
  constexpr int QD = T >> 1, NIB = QD >> 1, W = 2 * (T & 1);
  const u32x4_t& lo = (QD & 1) ? r.qb : r.qa;
  c0 = ((lo[W] >> (4 * NIB)) & 0x0f0f0f0fu) | (((r.qh[W] >> (2 * QD)) & 0x03030303u) << 4);
  c1 = ((lo[W + 1] >> (4 * NIB)) & 0x0f0f0f0fu) | (((r.qh[W + 1] >> (2 * QD)) & 0x03030303u) << 4);
  quarter = QD;
}
template <int T, class Raw>
__device__ __forceinline__ bf16x8_t raw_fragment(const Raw& r, const float (&s)[4], const float (&o)[4]) {
  uint32_t c0, c1;
  int qd;
  raw_codes<T>(r, c0, c1, qd);
  u32x4_t f;
  f[0] = pack2(dm_fma(s[qd], dm_ubyte<0>(c0), o[qd]), dm_fma(s[qd], dm_ubyte<1>(c0), o[qd]));
  f[1] = pack2(dm_fma(s[qd], dm_ubyte<2>(c0), o[qd]), dm_fma(s[qd], dm_ubyte<3>(c0), o[qd]));
  f[2] = pack2(dm_fma(s[qd], dm_ubyte<0>(c1), o[qd]), dm_fma(s[qd], dm_ubyte<1>(c1), o[qd]));
  f[3] = pack2(dm_fma(s[qd], dm_ubyte<2>(c1), o[qd]), dm_fma(s[qd], dm_ubyte<3>(c1), o[qd]));
  return __builtin_bit_cast(bf16x8_t, f);
}

constexpr int RN = 256;  // output columns of a workgroup of the register form

constexpr int RM = 192;  // most rows of a tile of the register form

// the main loop and the epilogue for a tile of up to 32 * TM rows
template <int KIND, int TM, bool GATHER, int ROWS>
__device__ __forceinline__ void reg_tile(const MmArgs& a, bf16_t (*As)[ROWS][LDK], const uint32_t* s_src,
                                         const uint32_t* s_dst, int rows_here, int m0, int64_t wrow0) {
  constexpr int BM = 32 * TM, TN = 2;
  constexpr int NA = BM * 16 / 256;  // 16-byte pieces of an activation slab per thread
  typedef typename RawOf<KIND>::type Raw;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, h = lane >> 5;
  const int n0 = blockIdx.x * RN;
  const int nb = a.K >> 8, nslab = a.K / BK;  // an even number of slabs
  MM_MARK(5, true);

  RawOff boff[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) boff[j] = raw_offsets(KIND, wrow0 + min(n0 + wave * 64 + j * 32 + l32, a.O - 1), nb, h);
  uint32_t aoff[NA];
#pragma unroll
  for (int i = 0; i < NA; ++i) {
    const int idx = tid + 256 * i, r = idx >> 4, c8 = idx & 15;
    // rows past the end of the tile read a valid row: what they produce is never stored
    const int64_t src = GATHER ? (int64_t)s_src[r] : (int64_t)min(m0 + r, a.M - 1);
    aoff[i] = (uint32_t)((src * a.K + 8 * c8) * 2);
  }
  // Registers of a slab's way in: activations of slab k travel in areg[k & 1] (asked for two
  // slabs ahead, written to LDS buffer k & 1 one slab ahead), codes in raw[k & 1] (asked for one
  // slab ahead), scales in sc / of [k & 1].
  u32x4_t areg[2][NA];
  Raw raw[2][TN];
  float sc[2][TN][4], of[2][TN][4];
  auto fetch_a1 = [&](auto set, auto piece, int slab) {
    constexpr int S = decltype(set)::value, I = decltype(piece)::value;
    areg[S][I] = ld_off<u32x4_t>(reinterpret_cast<const uint8_t*>(a.x) + slab * (BK * 2), aoff[I]);
  };
  auto fetch_a = [&](auto set, int slab) {
#define ORN_FETCH_A(I) if constexpr (NA > I) fetch_a1(set, std::integral_constant<int, (I < NA ? I : 0)>{}, slab)
    ORN_FETCH_A(0); ORN_FETCH_A(1); ORN_FETCH_A(2); ORN_FETCH_A(3); ORN_FETCH_A(4); ORN_FETCH_A(5);
    ORN_FETCH_A(6); ORN_FETCH_A(7); ORN_FETCH_A(8); ORN_FETCH_A(9); ORN_FETCH_A(10); ORN_FETCH_A(11);
#undef ORN_FETCH_A
  };
  auto write_a = [&](auto set, auto piece) {
    constexpr int S = decltype(set)::value, I = decltype(piece)::value;
    const int idx = tid + 256 * I;
    *reinterpret_cast<u32x4_t*>(&As[S][idx >> 4][8 * (idx & 15)]) = areg[S][I];
  };
  auto fetch_b = [&](auto set, int slab) {
    constexpr int S = decltype(set)::value;
#pragma unroll
    for (int j = 0; j < TN; ++j) raw_load(raw[S][j], a, boff[j], slab);
  };
  auto scales = [&](auto set) {
    constexpr int S = decltype(set)::value;
#pragma unroll
    for (int j = 0; j < TN; ++j) raw_scales<S>(raw[S][j], h, sc[S][j], of[S][j]);
  };

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  bf16x8_t af[2][TM], bfr[2][TN];
  // operands of k step T of the slab in set S into fragment set T & 1
  auto frags = [&](auto set, auto tc) {
    constexpr int S = decltype(set)::value, T = decltype(tc)::value;
    const int kc = 32 * (T >> 1) + 16 * h + 8 * (T & 1);
#pragma unroll
    for (int i = 0; i < TM; ++i) af[T & 1][i] = *reinterpret_cast<const bf16x8_t*>(&As[S][i * 32 + l32][kc]);
#pragma unroll
    for (int j = 0; j < TN; ++j) bfr[T & 1][j] = raw_fragment<T>(raw[S][j], sc[S][j], of[S][j]);
  };
  auto mfmas = [&](auto tc) {
    constexpr int T = decltype(tc)::value;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[T & 1][i], bfr[T & 1][j], acc[i][j], 0, 0, 0);
  };
  // issue order of a step: the LDS reads first, then every MFMA followed by its share of the
  // step's other work (VALU: dequantization; LDS writes; global loads), which then runs in the
  // shadow of the matrix core
  auto order = [&](auto valu, auto dsw, auto vmem) {
    __builtin_amdgcn_sched_group_barrier(0x100, TM, 0);
#pragma unroll
    for (int m = 0; m < TM * TN; ++m) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, decltype(valu)::value, 0);
      if (m < decltype(dsw)::value) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
      if (m < decltype(vmem)::value) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;
  constexpr int VQ = (52 + TM * TN - 1) / (TM * TN);  // vector instructions of a step's dequantization per MFMA

  // slab s (parity: its LDS buffer and register sets). On entry fragment set 0 holds step 0.
  auto slab = [&](auto par, int s) {
    constexpr int HH = decltype(par)::value;
    using Other = std::integral_constant<int, HH ^ 1>;
    // (past the last slab the last one is asked for and written again, to no effect: loads and
    // stores under a condition would make the compiler wait for everything in flight)
    MM_MARK(0, s == 2);
    // step 0: ask for the codes of slab s + 1
    fetch_b(Other{}, min(s + 1, nslab - 1));
    frags(par, std::integral_constant<int, 1>{});
    mfmas(std::integral_constant<int, 0>{});
    order(std::integral_constant<int, VQ>{}, std::integral_constant<int, 0>{}, std::integral_constant<int, TM * TN>{});
    MM_MARK(1, s == 2);
    // steps 1 .. 6: the activations of slab s + 1 go from their registers to the other buffer,
    // and those of slab s + 2 are asked for, a few pieces a step (all loads of a slab in one
    // step fill the memory pipe's queue, and the wavefront stands still until it has drained)
    const int s2 = min(s + 2, nslab - 1);
    auto mid = [&](auto tc) {
      constexpr int T = decltype(tc)::value;
      constexpr int W0 = (T - 1) * NA / 6, W1 = T * NA / 6;
      frags(par, std::integral_constant<int, T + 1>{});
      mfmas(tc);
      if constexpr (W1 - W0 >= 1) write_a(Other{}, std::integral_constant<int, W0>{});
      if constexpr (W1 - W0 >= 2) write_a(Other{}, std::integral_constant<int, W0 + 1>{});
      if constexpr (W1 - W0 >= 3) write_a(Other{}, std::integral_constant<int, W0 + 2>{});
      if constexpr (W1 - W0 >= 1) fetch_a1(par, std::integral_constant<int, W0>{}, s2);
      if constexpr (W1 - W0 >= 2) fetch_a1(par, std::integral_constant<int, W0 + 1>{}, s2);
      if constexpr (W1 - W0 >= 3) fetch_a1(par, std::integral_constant<int, W0 + 2>{}, s2);
      static_assert(W1 - W0 <= 3, "more activation pieces a step than written");
      order(std::integral_constant<int, VQ>{}, std::integral_constant<int, W1 - W0>{}, std::integral_constant<int, W1 - W0>{});
    };
    mid(std::integral_constant<int, 1>{});
    mid(std::integral_constant<int, 2>{});
    mid(std::integral_constant<int, 3>{});
    mid(std::integral_constant<int, 4>{});
    mid(std::integral_constant<int, 5>{});
    mid(std::integral_constant<int, 6>{});
    MM_MARK(2, s == 2);
    // every read of this slab's buffer has been issued, slab s + 1 is in the other one
    __syncthreads();
    MM_MARK(3, s == 2);
    // step 7: scales and step 0 of slab s + 1
    scales(Other{});
    frags(Other{}, std::integral_constant<int, 0>{});
    mfmas(std::integral_constant<int, 7>{});
    order(std::integral_constant<int, (52 + 40 + TM * TN - 1) / (TM * TN)>{}, std::integral_constant<int, 0>{},
          std::integral_constant<int, 0>{});
    MM_MARK(4, s == 2);
  };

  fetch_a(P0{}, 0);
  fetch_b(P0{}, 0);
  fetch_a(P1{}, 1);
#define ORN_WRITE_A(I) if constexpr (NA > I) write_a(P0{}, std::integral_constant<int, (I < NA ? I : 0)>{})
  ORN_WRITE_A(0); ORN_WRITE_A(1); ORN_WRITE_A(2); ORN_WRITE_A(3); ORN_WRITE_A(4); ORN_WRITE_A(5);
  ORN_WRITE_A(6); ORN_WRITE_A(7); ORN_WRITE_A(8); ORN_WRITE_A(9); ORN_WRITE_A(10); ORN_WRITE_A(11);
#undef ORN_WRITE_A
  static_assert(NA <= 12, "more activation pieces a thread than written");
  __syncthreads();
  scales(P0{});
  frags(P0{}, std::integral_constant<int, 0>{});
  __builtin_amdgcn_sched_barrier(0);
  for (int s = 0; s < nslab; s += 2) {
    slab(P0{}, s);
    slab(P1{}, s + 1);
  }
  __syncthreads();  // the fragments of a slab past the end were read out of the buffers the output tile goes over
  MM_MARK(6, true);
  store_tile<TM, TN, GATHER>(a, acc, &As[0][0][0], 0, wave * 64, lane, n0, m0, rows_here, s_dst, a.vec != 0, RN + 8);
  MM_MARK(7, true);
}

// One kernel for every tile height: a tile runs the loop compiled for the number of 32-row
// MFMA tiles it really has (an expert with few pairs does not pay for the widest tile).
template <int KIND, bool GATHER, int ROWS>
__device__ __forceinline__ void reg_body(const MmArgs& a) {
  __shared__ __attribute__((aligned(16))) bf16_t As[2][ROWS][LDK];
  __shared__ uint32_t s_src[ROWS], s_dst[ROWS];
  static_assert(2 * LDK >= RN + 8 && ROWS % 32 == 0 && ROWS <= RM, "the output tile does not fit over the slab buffers");
  const int tid = threadIdx.x;
  int rows_here, m0 = 0;
  int64_t wrow0 = 0;
  if constexpr (GATHER) {
    // a plan tile of more rows than ROWS is worked on by a.sub workgroups, ROWS rows each
    const uint32_t tile = blockIdx.y / (uint32_t)a.sub, part = blockIdx.y % (uint32_t)a.sub;
    if (tile >= *a.n_tiles) return;
    const uint32_t e = a.tile_expert[tile], st = a.tile_start[tile] + part * ROWS;
    rows_here = min((int)a.tile_count[tile] - (int)(part * ROWS), ROWS);
    if (rows_here <= 0) return;
    wrow0 = (int64_t)e * a.O;
    for (int r = tid; r < ROWS; r += 256) {
      const uint32_t p = r < rows_here ? a.pair[st + r] : 0u;
      s_src[r] = p / (uint32_t)a.up_div;
      s_dst[r] = p;
    }
    __syncthreads();
  } else {
    m0 = blockIdx.y * ROWS;
    rows_here = min(ROWS, a.M - m0);
  }
  // a tile runs the loop compiled for the number of 32-row MFMA tiles it really has (an expert
  // with few pairs does not pay for the widest tile)
  const int groups = (rows_here + 31) >> 5;
#define ORN_REG_TILE(N) reg_tile<KIND, (N <= ROWS / 32 ? N : 1), GATHER, ROWS>(a, As, s_src, s_dst, rows_here, m0, wrow0)
  if (groups <= 1) ORN_REG_TILE(1);
  else if (groups == 2 || ROWS / 32 == 2) ORN_REG_TILE(2);
  else if (groups == 3 || ROWS / 32 == 3) ORN_REG_TILE(3);
  else if (groups == 4 || ROWS / 32 == 4) ORN_REG_TILE(4);
  else if (groups == 5 || ROWS / 32 == 5) ORN_REG_TILE(5);
  else ORN_REG_TILE(6);
#undef ORN_REG_TILE
}

template <int KIND, bool GATHER>
__global__ __launch_bounds__(256) void kq_mm_reg_kernel(MmArgs a) {
  reg_body<KIND, GATHER, RM>(a);
}
// 64 rows a workgroup, two workgroups a compute unit: one's way in and out runs beside the
// other's main loop (matrices of few K slabs)
template <int KIND, bool GATHER>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void kq_mm_reg64_kernel(MmArgs a) {
  reg_body<KIND, GATHER, 64>(a);
}

// BM == 64 has two 32-row MFMA tiles per wavefront as well (TM = 2), one wavefront column
static_assert(BN == 128 && BK == 128, "tile constants are baked into the index arithmetic");

// ---- expert-sorted pair list for the gathered form -----------------------------------
// inds [pairs] (expert of pair p; pair p = token * k + slot). One workgroup: counts per expert,
// exclusive scan, scatter, then the tile list, fullest tiles first (the GEMM's workgroups start
// in the order of the list, and one that starts late with many rows would be the tail).
constexpr int kSortTilesMax = 2048;  // tile lists up to this length are ordered

// Writes the tile list fullest first: a counting sort over the tile heights (a tile has 1 .. bm
// <= 256 rows; tiles of one height land in the order their atomics are served, which changes
// the order workgroups start in and nothing else). All 1024 threads of the workgroup call it.
__device__ __forceinline__ void order_tiles(uint32_t total_tiles, int bm, const uint32_t* t_expert, const uint32_t* t_start,
                                            const uint32_t* t_count, uint32_t* tile_expert, uint32_t* tile_start,
                                            uint32_t* tile_count) {
  __shared__ uint32_t bin[257];
  const int tid = threadIdx.x;
  if (tid < 257) bin[tid] = 0;
  __syncthreads();
  for (uint32_t i = tid; i < total_tiles; i += 1024) atomicAdd(&bin[min(t_count[i], 256u)], 1u);
  __syncthreads();
  if (tid == 0) {  // places of the heights, tallest first
    uint32_t at = 0;
    for (int c = min(bm, 256); c >= 0; --c) {
      const uint32_t n = bin[c];
      bin[c] = at;
      at += n;
    }
  }
  __syncthreads();
  for (uint32_t i = tid; i < total_tiles; i += 1024) {
    const uint32_t c = t_count[i], at = atomicAdd(&bin[min(c, 256u)], 1u);
    tile_expert[at] = t_expert[i];
    tile_start[at] = t_start[i];
    tile_count[at] = c;
  }
}


__global__ __launch_bounds__(1024) void moe_sort_pairs_kernel(const uint32_t* inds, int pairs, int E,
                                                              int bm, uint32_t* pair, uint32_t* tile_expert,
                                                              uint32_t* tile_start, uint32_t* tile_count,
                                                              uint32_t* n_tiles) {
  __shared__ uint32_t cnt[1024], fill[1024];
  __shared__ unsigned long long scan[2][1024];  // pairs before an expert (low 40 bits) and tiles before it
  __shared__ uint32_t t_expert[kSortTilesMax], t_start[kSortTilesMax], t_count[kSortTilesMax];
  const int tid = threadIdx.x;
  cnt[tid] = 0;
  fill[tid] = 0;
  __syncthreads();
  // (eight loads in flight a thread: one after the other, each pass over the pairs is 32 memory
  // latencies long for a 4096-token chunk)
  for (int p0 = tid; p0 < pairs; p0 += 8 * 1024) {
    uint32_t e[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) e[u] = p0 + 1024 * u < pairs ? inds[p0 + 1024 * u] : 0u;
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (p0 + 1024 * u < pairs) atomicAdd(&cnt[min(e[u], (uint32_t)(E - 1))], 1u);
  }
  __syncthreads();
  // inclusive scan over the 1024 slots (experts past E hold zero), ten doubling steps
  const uint32_t mine = cnt[tid];
  scan[0][tid] = (unsigned long long)mine | ((unsigned long long)((mine + bm - 1) / bm) << 40);
  __syncthreads();
  int cur = 0;
  for (int d = 1; d < 1024; d <<= 1) {
    const unsigned long long v = scan[cur][tid] + (tid >= d ? scan[cur][tid - d] : 0ull);
    scan[cur ^ 1][tid] = v;
    cur ^= 1;
    __syncthreads();
  }
  const unsigned long long incl = scan[cur][tid];
  const uint32_t my_tiles = (mine + bm - 1) / bm;
  const uint32_t start = (uint32_t)(incl & ((1ull << 40) - 1)) - mine;
  const uint32_t tiles_before = (uint32_t)(incl >> 40) - my_tiles;
  const uint32_t total_tiles = (uint32_t)(scan[cur][1023] >> 40);
  if (tid == 0) *n_tiles = total_tiles;
  __syncthreads();
  scan[0][tid] = start;  // (reused: where an expert's run of pairs begins)
  __syncthreads();
  // placement: a pair takes the next free place of its expert. The order inside an expert's
  // run depends on the scheduling of the atomics, the results do not: every output row is one
  // dot product over k in a fixed order, whichever tile row computes it.
  for (int p0 = tid; p0 < pairs; p0 += 8 * 1024) {
    uint32_t e[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) e[u] = p0 + 1024 * u < pairs ? min(inds[p0 + 1024 * u], (uint32_t)(E - 1)) : 0u;
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (p0 + 1024 * u < pairs) pair[(uint32_t)scan[0][e[u]] + atomicAdd(&fill[e[u]], 1u)] = (uint32_t)(p0 + 1024 * u);
  }
  const bool ordered = total_tiles <= (uint32_t)kSortTilesMax;
  if (tid < E)
    for (uint32_t t = 0; t < my_tiles; ++t) {
      const uint32_t i = tiles_before + t, st = start + t * bm, c = min((uint32_t)bm, mine - t * bm);
      if (ordered) {
        t_expert[i] = tid;
        t_start[i] = st;
        t_count[i] = c;
      } else {
        tile_expert[i] = tid;
        tile_start[i] = st;
        tile_count[i] = c;
      }
    }
  __syncthreads();
  if (!ordered) return;
  order_tiles(total_tiles, bm, t_expert, t_start, t_count, tile_expert, tile_start, tile_count);
}

// ---- the same plan from many workgroups -----------------------------------------------
// A pass over the pairs is one LDS atomic a pair, about a cycle each in one workgroup: 33 us
// for the 32768 pairs of a 4096-token chunk. From 8192 pairs on, kSortParts workgroups count
// their slices of the pairs side by side, one workgroup turns the counts into places (per
// expert, then per slice inside an expert's run) and writes the tile list, and the slices
// scatter side by side.
constexpr int kSortParts = 32;

__global__ __launch_bounds__(256) void moe_sort_count_kernel(const uint32_t* inds, int pairs, int E, uint32_t* part_cnt) {
  __shared__ uint32_t cnt[1024];
  for (int e = threadIdx.x; e < E; e += 256) cnt[e] = 0;
  __syncthreads();
  const int per = (pairs + kSortParts - 1) / kSortParts, a = blockIdx.x * per, b = min(pairs, a + per);
  for (int p = a + threadIdx.x; p < b; p += 256) atomicAdd(&cnt[min(inds[p], (uint32_t)(E - 1))], 1u);
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += 256) part_cnt[blockIdx.x * E + e] = cnt[e];
}

// part_cnt [parts, E] in: pairs of expert e in slice b; out: where slice b's pairs of expert e begin
__global__ __launch_bounds__(1024) void moe_sort_plan_kernel(int E, int bm, uint32_t* part_cnt, uint32_t* tile_expert,
                                                             uint32_t* tile_start, uint32_t* tile_count,
                                                             uint32_t* n_tiles) {
  __shared__ unsigned long long scan[2][1024];
  __shared__ uint32_t t_expert[kSortTilesMax], t_start[kSortTilesMax], t_count[kSortTilesMax];
  const int tid = threadIdx.x;
  uint32_t mine = 0;
  if (tid < E)
    for (int b = 0; b < kSortParts; ++b) mine += part_cnt[b * E + tid];
  const uint32_t my_tiles = (mine + bm - 1) / bm;
  scan[0][tid] = (unsigned long long)mine | ((unsigned long long)my_tiles << 40);
  __syncthreads();
  int cur = 0;
  for (int d = 1; d < 1024; d <<= 1) {
    const unsigned long long v = scan[cur][tid] + (tid >= d ? scan[cur][tid - d] : 0ull);
    scan[cur ^ 1][tid] = v;
    cur ^= 1;
    __syncthreads();
  }
  const unsigned long long incl = scan[cur][tid];
  const uint32_t start = (uint32_t)(incl & ((1ull << 40) - 1)) - mine;
  const uint32_t tiles_before = (uint32_t)(incl >> 40) - my_tiles;
  const uint32_t total_tiles = (uint32_t)(scan[cur][1023] >> 40);
  if (tid == 0) *n_tiles = total_tiles;
  if (tid < E) {
    uint32_t at = start;
    for (int b = 0; b < kSortParts; ++b) {
      const uint32_t c = part_cnt[b * E + tid];
      part_cnt[b * E + tid] = at;
      at += c;
    }
  }
  const bool ordered = total_tiles <= (uint32_t)kSortTilesMax;
  if (tid < E)
    for (uint32_t t = 0; t < my_tiles; ++t) {
      const uint32_t i = tiles_before + t, st = start + t * bm, c = min((uint32_t)bm, mine - t * bm);
      if (ordered) {
        t_expert[i] = tid;
        t_start[i] = st;
        t_count[i] = c;
      } else {
        tile_expert[i] = tid;
        tile_start[i] = st;
        tile_count[i] = c;
      }
    }
  __syncthreads();
  if (!ordered) return;
  order_tiles(total_tiles, bm, t_expert, t_start, t_count, tile_expert, tile_start, tile_count);
}

__global__ __launch_bounds__(256) void moe_sort_scatter_kernel(const uint32_t* inds, int pairs, int E,
                                                               const uint32_t* part_at, uint32_t* pair) {
  __shared__ uint32_t at[1024];
  for (int e = threadIdx.x; e < E; e += 256) at[e] = part_at[blockIdx.x * E + e];
  __syncthreads();
  const int per = (pairs + kSortParts - 1) / kSortParts, a = blockIdx.x * per, b = min(pairs, a + per);
  for (int p = a + threadIdx.x; p < b; p += 256) pair[atomicAdd(&at[min(inds[p], (uint32_t)(E - 1))], 1u)] = (uint32_t)p;
}

int check(const ornith_kmatrix* w, const char* who) {
  ORN_REQUIRE(w && (w->kind == ORNITH_Q4K || w->kind == ORNITH_Q6K), "%s: bad matrix", who);
  ORN_REQUIRE(w->K >= 256 && w->K % 256 == 0 && w->O >= 1 && w->E >= 1, "%s: bad dims E=%d O=%d K=%d", who,
              w->E, w->O, w->K);
  ORN_REQUIRE(w->d_qs && w->d_scales && w->d_dm, "%s: null tensor", who);
  return ORNITH_OK;
}

}  // namespace

extern "C" {

// Up to four matrices of one K over the same activations in one launch (the projections that
// share an input: narrow ones alone leave compute units without a workgroup). Matrices of one
// kind take the tile the whole launch's size calls for; a mix of kinds takes 128-row tiles.
int ornith_kq_matmul_multi(ornith_ctx* ctx, const ornith_kmatrix* const* ws, int n, const void* d_x, int M,
                           void* const* d_ys) {
  ORN_REQUIRE(ctx && ws && d_x && d_ys && n >= 1 && n <= 4, "kq_matmul: bad argument");
  ORN_REQUIRE(M >= 1, "kq_matmul: M=%d", M);
  ORN_REQUIRE(((uintptr_t)d_x & 15) == 0, "kq_matmul: x must be 16-byte aligned");
  MmArgs a{};
  int nx = 0;
  bool mixed = false;
  a.vec = 1;
  for (int i = 0; i < n; ++i) {
    ORN_REQUIRE(ws[i] && d_ys[i], "kq_matmul: null entry %d", i);
    int rc = check(ws[i], "kq_matmul");
    if (rc) return rc;
    ORN_REQUIRE(ws[i]->E == 1, "kq_matmul: stacked matrix (use kq_gather_matmul)");
    ORN_REQUIRE(ws[i]->K == ws[0]->K, "kq_matmul: matrices of one launch differ in K");
    mixed = mixed || ws[i]->kind != ws[0]->kind;
    a.vec = a.vec && ws[i]->O % 8 == 0 && ((uintptr_t)d_ys[i] & 15) == 0;
    if (i == 0) {
      a.qs = (const uint8_t*)ws[0]->d_qs;
      a.scales = (const uint8_t*)ws[0]->d_scales;
      a.dm = (const uint16_t*)ws[0]->d_dm;
      a.y = (bf16_t*)d_ys[0];
      a.O = ws[0]->O;
    } else {
      a.seg[i - 1] = {(const uint8_t*)ws[i]->d_qs, (const uint8_t*)ws[i]->d_scales, (const uint16_t*)ws[i]->d_dm,
                      (bf16_t*)d_ys[i], ws[i]->O, nx, ws[i]->kind};
    }
    nx += (ws[i]->O + BN - 1) / BN;
  }
  a.nseg = n - 1;
  a.x = (const bf16_t*)d_x;
  a.M = M;
  a.K = ws[0]->K;
  const int kind = ws[0]->kind;
  a.kind = kind;
  if (mixed) {  // matrices of both kinds: the 128-row tile, every workgroup asking its matrix's kind
    hipLaunchKernelGGL((kq_mm_kernel<kMixed, 128, false>), dim3(nx, (M + 127) / 128), dim3(256), 0, ctx->stream, a);
    ORN_LAUNCH_CHECK("kq_mm_kernel<mixed>");
    return ORNITH_OK;
  }
  // 256-row tiles dequantize every weight tile half as often; 128-row tiles when that is what
  // it takes to give every compute unit a workgroup
  const bool big = M >= 256 && (long)nx * ((M + 255) / 256) >= ctx->compute_units;
  const dim3 grid(nx, big ? (M + 255) / 256 : (M + 127) / 128);
  // the 256-row tile runs in its producer / consumer form (the smaller tiles measured no
  // faster that way: they have too few MFMAs a slab)
  if (big && ornith_option_gemm_duo()) {
    if (kind == ORNITH_Q4K)
      hipLaunchKernelGGL((kq_mm_duo_kernel<ORNITH_Q4K, 256, false>), grid, dim3(512), 0, ctx->stream, a);
    else
      hipLaunchKernelGGL((kq_mm_duo_kernel<ORNITH_Q6K, 256, false>), grid, dim3(512), 0, ctx->stream, a);
  } else if (kind == ORNITH_Q4K) {
    if (big)
      hipLaunchKernelGGL((kq_mm_kernel<ORNITH_Q4K, 256, false>), grid, dim3(256), 0, ctx->stream, a);
    else
      hipLaunchKernelGGL((kq_mm_kernel<ORNITH_Q4K, 128, false>), grid, dim3(256), 0, ctx->stream, a);
  } else {
    if (big)
      hipLaunchKernelGGL((kq_mm_kernel<ORNITH_Q6K, 256, false>), grid, dim3(256), 0, ctx->stream, a);
    else
      hipLaunchKernelGGL((kq_mm_kernel<ORNITH_Q6K, 128, false>), grid, dim3(256), 0, ctx->stream, a);
  }
  ORN_LAUNCH_CHECK("kq_mm_kernel");
  return ORNITH_OK;
}

int ornith_kq_matmul(ornith_ctx* ctx, const ornith_kmatrix* w, const void* d_x, int M, void* d_y) {
  ORN_REQUIRE(w && d_y, "kq_matmul: null argument");
  return ornith_kq_matmul_multi(ctx, &w, 1, d_x, M, &d_y);
}

// gather plan: expert-sorted pairs and the tile list, in caller-provided device memory
// (ornith_kq_gather_plan_bytes(pairs, E) bytes)
size_t ornith_kq_gather_plan_bytes(int pairs, int E) {
  const size_t tiles = (size_t)pairs / 64 + (size_t)E + 1;
  return ((size_t)pairs + tiles * 3 + 1 + (size_t)kSortParts * E) * 4 + 6 * 256;
}

int ornith_kq_gather_matmul(ornith_ctx* ctx, const ornith_kmatrix* w, const void* d_x,
                            const uint32_t* d_inds, int pairs, int top_k, int is_up, void* d_plan,
                            int rebuild_plan, void* d_y) {
  ORN_REQUIRE(ctx && d_x && d_inds && d_plan && d_y, "kq_gather_matmul: null argument");
  int rc = check(w, "kq_gather_matmul");
  if (rc) return rc;
  ORN_REQUIRE(pairs >= 1 && top_k >= 1 && pairs % top_k == 0 && w->E <= 1024,
              "kq_gather_matmul: pairs=%d top_k=%d E=%d", pairs, top_k, w->E);
  const size_t tiles_max = (size_t)pairs / 64 + (size_t)w->E + 1;
  ScratchCursor pc(d_plan);
  uint32_t* pair = pc.take<uint32_t>(pairs);
  uint32_t* te = pc.take<uint32_t>(tiles_max);
  uint32_t* ts = pc.take<uint32_t>(tiles_max);
  uint32_t* tc = pc.take<uint32_t>(tiles_max);
  uint32_t* nt = pc.take<uint32_t>(1);
  uint32_t* parts = pc.take<uint32_t>((size_t)kSortParts * w->E);
  // Rows per plan tile: the choice depends only on pairs and E (and the option), so the calls
  // sharing a plan agree on it. With 48 rows an expert or more: the smallest of 96 / 128 / 160 /
  // 192 rows that holds an expert's share of the pairs with 2.5 standard deviations to spare, so
  // that nearly every expert is one tile (the register form dequantizes its weights once).
  // Otherwise 128-row tiles from 96 rows an expert on average, else 64.
  const int avg = pairs / w->E;
  int spare = 0;
  while (4 * spare * spare < 25 * avg) ++spare;
  const int need = avg + spare;
  const bool tall = ornith_option_gemm_reg() && avg >= 48;
  const int tile_rows = tall ? (need <= 96 ? 96 : need <= 128 ? 128 : need <= 160 ? 160 : 192) : avg >= 96 ? 128 : 64;
  // The kernel for this matrix. Tall plans take the register form when its 32-bit offsets reach:
  // for K >= 1024 a workgroup a plan tile (one a compute unit), for fewer K slabs 64-row
  // workgroups, two a compute unit (a workgroup's way in and out, which weighs more the fewer
  // slabs there are, then runs beside the other's main loop; the weights still bypass LDS, which
  // is what bounds the LDS form at 64 rows). Otherwise the LDS form: 128 rows a workgroup from 96
  // rows an expert on and K >= 1024, else 64. A plan tile taller than its kernel's workgroups is
  // split over several of them.
  const size_t x_bytes = (size_t)(is_up ? pairs / top_k : pairs) * w->K * 2;
  const size_t q_bytes = (size_t)w->E * w->O * (w->K / 256) * (w->kind == ORNITH_Q4K ? 128 : 192);
  const bool reg = tall && w->K >= 1024 && x_bytes < (size_t(1) << 32) && q_bytes < (size_t(1) << 32);
  const int lds_rows = (avg >= 96 && w->K >= 1024) ? 128 : 64;
  if (rebuild_plan && pairs >= 8192) {
    hipLaunchKernelGGL(moe_sort_count_kernel, dim3(kSortParts), dim3(256), 0, ctx->stream, d_inds, pairs, w->E, parts);
    hipLaunchKernelGGL(moe_sort_plan_kernel, dim3(1), dim3(1024), 0, ctx->stream, w->E, tile_rows, parts, te, ts, tc, nt);
    hipLaunchKernelGGL(moe_sort_scatter_kernel, dim3(kSortParts), dim3(256), 0, ctx->stream, d_inds, pairs, w->E,
                       parts, pair);
    ORN_LAUNCH_CHECK("moe_sort_*_kernel");
  } else if (rebuild_plan) {
    hipLaunchKernelGGL(moe_sort_pairs_kernel, dim3(1), dim3(1024), 0, ctx->stream, d_inds, pairs, w->E,
                       tile_rows, pair, te, ts, tc, nt);
    ORN_LAUNCH_CHECK("moe_sort_pairs_kernel");
  }
  MmArgs a{};
  a.qs = (const uint8_t*)w->d_qs;
  a.scales = (const uint8_t*)w->d_scales;
  a.dm = (const uint16_t*)w->d_dm;
  a.x = (const bf16_t*)d_x;
  a.y = (bf16_t*)d_y;
  a.M = pairs;
  a.O = w->O;
  a.K = w->K;
  a.vec = w->O % 8 == 0 && ((uintptr_t)d_y & 15) == 0;
  a.pair = pair;
  a.up_div = is_up ? top_k : 1;
  a.tile_expert = te;
  a.tile_start = ts;
  a.tile_count = tc;
  a.n_tiles = nt;
  if (reg) {
    a.sub = 1;
    const dim3 rgrid((w->O + RN - 1) / RN, (unsigned)tiles_max);
    if (w->kind == ORNITH_Q4K)
      hipLaunchKernelGGL((kq_mm_reg_kernel<ORNITH_Q4K, true>), rgrid, dim3(256), 0, ctx->stream, a);
    else
      hipLaunchKernelGGL((kq_mm_reg_kernel<ORNITH_Q6K, true>), rgrid, dim3(256), 0, ctx->stream, a);
    ORN_LAUNCH_CHECK("kq_mm_reg_kernel<gather>");
    return ORNITH_OK;
  }
  if (tall && w->K % 256 == 0 && x_bytes < (size_t(1) << 32) && q_bytes < (size_t(1) << 32)) {
    a.sub = (tile_rows + 63) / 64;
    const dim3 rgrid((w->O + RN - 1) / RN, (unsigned)(tiles_max * a.sub));
    if (w->kind == ORNITH_Q4K)
      hipLaunchKernelGGL((kq_mm_reg64_kernel<ORNITH_Q4K, true>), rgrid, dim3(256), 0, ctx->stream, a);
    else
      hipLaunchKernelGGL((kq_mm_reg64_kernel<ORNITH_Q6K, true>), rgrid, dim3(256), 0, ctx->stream, a);
    ORN_LAUNCH_CHECK("kq_mm_reg64_kernel<gather>");
    return ORNITH_OK;
  }
  a.sub = (tile_rows + lds_rows - 1) / lds_rows;
  const dim3 grid((w->O + BN - 1) / BN, (unsigned)(tiles_max * a.sub));
  if (lds_rows == 128) {
    if (w->kind == ORNITH_Q4K)
      hipLaunchKernelGGL((kq_mm_kernel<ORNITH_Q4K, 128, true>), grid, dim3(256), 0, ctx->stream, a);
    else
      hipLaunchKernelGGL((kq_mm_kernel<ORNITH_Q6K, 128, true>), grid, dim3(256), 0, ctx->stream, a);
  } else if (w->kind == ORNITH_Q4K)
    hipLaunchKernelGGL((kq_mm_kernel<ORNITH_Q4K, 64, true>), grid, dim3(256), 0, ctx->stream, a);
  else
    hipLaunchKernelGGL((kq_mm_kernel<ORNITH_Q6K, 64, true>), grid, dim3(256), 0, ctx->stream, a);
  ORN_LAUNCH_CHECK("kq_mm_kernel<gather>");
  return ORNITH_OK;
}

}  // extern "C"
