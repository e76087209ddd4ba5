/*
 * CPU oracle -- TEST INFRASTRUCTURE (see orc_common.h). The sampled-token path.
 *
 * Restates /root/reference/src/sample.rs:79-225 (make_sampler of mlx-lm: top-p, then
 * top-k over what top-p left, then an inverse-CDF draw; everything in the logits' own
 * dtype, bf16, except the CDF which is fp32), /root/reference/src/ops/random.rs:16-67
 * and the vendored threefry2x32 (kernels/mlx/.../random.metal:5-33,35-66).
 *
 *   logprobs   lp_i = bf16(x_i - lse), lse as in orc_sample.c
 *   top-p      probs = bf16(exp(lp)); S = stable ascending argsort of lp;
 *              cum = inclusive bf16 cumulative sum of probs[S]; keep[S[j]] = cum_j > bf16(1-p);
 *              lp' = keep ? lp : -inf                                   (sample.rs:79-115)
 *   top-k      order = stable ascending argsort of -lp'; lp'[order[k:]] = -inf   (:117-136)
 *   draw       x = float(bf16(lp' * bf16(1/temp))); m = max x;
 *              w = isinf(m) ? (x == m) : exp(x - m); cdf = exclusive fp32 cumulative sum;
 *              u = min(float(bits) / 2^32, nextafter(1,0)) * sum(w);
 *              token = searchsorted(cdf, u, right) - 1                     (:138-190)
 *   keys       key(seed) = [hi, lo]; next(): bits([2,2]) of the key, first row becomes
 *              the state, second is handed out; the draw uses bits([1]) of that sub-key
 *
 * Association orders the reference leaves to its scan kernels are fixed here (this
 * build's own; the HIP path implements the same): a row is cut into chunks of 1024 and a
 * chunk into 16 segments of 64. Inside a segment the inclusive scan is Hillis-Steele
 * (for s = 1,2,4,..,32: v[l] = v[l] + v[l-s], l >= s); segment totals are added left to
 * right inside the chunk, chunk totals left to right over the row;
 * cum_i = (base_chunk + off_segment) + v_i. In bf16 every one of those adds rounds.
 * The draw takes the first index whose INCLUSIVE cdf exceeds u, which is what
 * "searchsorted(exclusive cdf, u, right) - 1" selects on a non-decreasing cdf, and is
 * still defined where rounding makes two neighbouring partial sums swap order.
 *
 * Parity note: the reference's own sort / scan kernels associate differently (tiles of
 * its Metal block size); its fixtures for this path (refs/, tests/sampler.rs:29-170) are
 * not in the repository, so the last-bit behaviour of the two cumulative sums against
 * the reference is "parity unpinned". What is pinned: threefry against the published
 * Random123 vectors, key splitting and the uniform scaling by closed forms, argsort /
 * top-k / the draw against numpy on the same inputs, the cumulative sums against float64.
 */
#include "orc_common.h"

/* ---- threefry2x32, 20 rounds --------------------------------------------------- */
static inline uint32_t rotl32(uint32_t v, int r) { return (v << r) | (v >> (32 - r)); }

ORC_API void orc_threefry2x32(const uint32_t key[2], const uint32_t count[2], uint32_t out[2]) {
  static const int rot[2][4] = {{13, 15, 26, 6}, {17, 29, 16, 24}};
  const uint32_t ks[3] = {key[0], key[1], key[0] ^ key[1] ^ 0x1BD11BDAu};
  uint32_t x = count[0] + ks[0], y = count[1] + ks[1];
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

/* random::bits(shape = n words, key): word w < half comes from x of hash(w, w + half'),
 * word w + half' from its y; an odd count drops the last y (random.metal:35-66). */
ORC_API void orc_random_bits(const uint32_t key[2], int n, uint32_t* out) {
  const int half = n / 2, odd = n & 1, gy = half + odd;
  for (int t = 0; t < gy; ++t) {
    const int drop_last = odd && t == half;
    const uint32_t cnt[2] = {(uint32_t)t, drop_last ? 0u : (uint32_t)(t + gy)};
    uint32_t h[2];
    orc_threefry2x32(key, cnt, h);
    out[t] = h[0];
    if (!drop_last) out[t + gy] = h[1];
  }
}

ORC_API void orc_key_from_seed(uint64_t seed, uint32_t key[2]) {
  key[0] = (uint32_t)(seed >> 32);
  key[1] = (uint32_t)seed;
}

/* KeySequence::next: state <- first row of bits([2,2]), returns the second */
ORC_API void orc_key_next(uint32_t state[2], uint32_t sub[2]) {
  uint32_t b[4];
  orc_random_bits(state, 4, b);
  state[0] = b[0];
  state[1] = b[1];
  sub[0] = b[2];
  sub[1] = b[3];
}

/* uniform in [0,1) from raw bits, then times total (sampler_ops.metal:122-133) */
ORC_API float orc_uniform_scaled(uint32_t bits, float total) {
  float u = (float)bits / 4294967296.0f;
  const float upper = orc_u2f(0x3f7fffffu);
  u = u < upper ? u : upper;
  u = 1.0f * u + 0.0f;
  return u * total;
}

/* ---- sort ------------------------------------------------------------------------ */
/* bf16 bits -> unsigned key whose order is the float order (-inf < ... < -0 < +0 < ... < +inf) */
static inline uint32_t sort_key(bf16_t b) { return (b & 0x8000u) ? (uint32_t)(0xFFFFu - b) : (uint32_t)(b | 0x8000u); }

/* stable ascending argsort of bf16 values (negate: of their negation) */
ORC_API void orc_argsort_bf16(const bf16_t* x, int n, int negate, uint32_t* idx) {
  /* counting sort over the 65536 keys: stable by construction */
  uint32_t* count = (uint32_t*)calloc(65537, sizeof(uint32_t));
  for (int i = 0; i < n; ++i) {
    const bf16_t b = negate ? (bf16_t)(x[i] ^ 0x8000u) : x[i];
    count[sort_key(b) + 1]++;
  }
  for (int k = 0; k < 65536; ++k) count[k + 1] += count[k];
  for (int i = 0; i < n; ++i) {
    const bf16_t b = negate ? (bf16_t)(x[i] ^ 0x8000u) : x[i];
    idx[count[sort_key(b)]++] = (uint32_t)i;
  }
  free(count);
}

/* ---- scans ----------------------------------------------------------------------- */
#define SCAN_CHUNK 1024

/* inclusive cumulative sum in the order of the header; bf16 != 0 rounds every add */
static void scan_row(const float* in, int n, int bf16, float* out, float* total_out) {
  float base = 0.f;
  for (int c0 = 0; c0 < n; c0 += SCAN_CHUNK) {
    float off = 0.f;
    for (int g0 = c0; g0 < c0 + SCAN_CHUNK; g0 += 64) {
      float v[64];
      for (int l = 0; l < 64; ++l) v[l] = g0 + l < n ? in[g0 + l] : 0.f;
      for (int s = 1; s < 64; s <<= 1) {
        float t[64];
        for (int l = 0; l < 64; ++l) {
          t[l] = l >= s ? v[l] + v[l - s] : v[l];
          if (bf16 && l >= s) t[l] = orc_rb(t[l]);
        }
        memcpy(v, t, sizeof(v));
      }
      float pre = base + off;
      if (bf16) pre = orc_rb(pre);
      for (int l = 0; l < 64 && g0 + l < n; ++l) {
        float r = pre + v[l];
        out[g0 + l] = bf16 ? orc_rb(r) : r;
      }
      off = off + v[63];
      if (bf16) off = orc_rb(off);
    }
    base = base + off;
    if (bf16) base = orc_rb(base);
  }
  if (total_out) *total_out = base;
}

ORC_API void orc_cumsum_bf16(const bf16_t* x, int n, bf16_t* out) {
  if (n <= 0) return;
  float* f = (float*)malloc(sizeof(float) * (size_t)n * 2);
  for (int i = 0; i < n; ++i) f[i] = orc_bf16_to_f32(x[i]);
  scan_row(f, n, 1, f + n, NULL);
  for (int i = 0; i < n; ++i) out[i] = orc_f32_to_bf16(f[n + i]);
  free(f);
}

ORC_API float orc_cumsum_f32(const float* x, int n, float* out) {
  float total;
  scan_row(x, n, 0, out, &total);
  return total;
}

/* ---- the sampler's stages ---------------------------------------------------------- */
ORC_API void orc_logprobs_row(const bf16_t* logits, int V, bf16_t* lp) {
  extern float orc_logsumexp_bf16(const bf16_t* x, int V);
  const float lse = orc_logsumexp_bf16(logits, V);
  for (int i = 0; i < V; ++i) lp[i] = orc_f32_to_bf16(orc_bf16_to_f32(logits[i]) - lse);
}

ORC_API void orc_apply_top_p(const bf16_t* lp, int V, double top_p, bf16_t* out) {
  uint32_t* S = (uint32_t*)malloc(sizeof(uint32_t) * (size_t)V);
  bf16_t* sp = (bf16_t*)malloc(sizeof(bf16_t) * (size_t)V * 2);
  bf16_t* cum = sp + V;
  orc_argsort_bf16(lp, V, 0, S);
  for (int j = 0; j < V; ++j) sp[j] = orc_f32_to_bf16(orc_expf(orc_bf16_to_f32(lp[S[j]])));
  orc_cumsum_bf16(sp, V, cum);
  const float thresh = orc_bf16_to_f32(orc_f32_to_bf16((float)(1.0 - top_p)));
  for (int j = 0; j < V; ++j) {
    const int keep = orc_bf16_to_f32(cum[j]) > thresh;
    out[S[j]] = keep ? lp[S[j]] : (bf16_t)0xFF80u;
  }
  free(S);
  free(sp);
}

ORC_API void orc_apply_top_k(const bf16_t* lp, int V, int top_k, bf16_t* out) {
  uint32_t* order = (uint32_t*)malloc(sizeof(uint32_t) * (size_t)V);
  orc_argsort_bf16(lp, V, 1, order);
  memcpy(out, lp, sizeof(bf16_t) * (size_t)V);
  for (int j = top_k; j < V; ++j) out[order[j]] = (bf16_t)0xFF80u;
  free(order);
}

/* weights of mx.random.categorical(lp * (1/temp)): x = float(bf16(lp * bf16(1/temp))), m = max x,
 * w = isinf(m) ? (x == m) : exp(x - m); returns their sum in the scan's order */
ORC_API float orc_categorical_weights(const bf16_t* lp, int V, double temp, float* w) {
  const float scale = orc_bf16_to_f32(orc_f32_to_bf16((float)(1.0 / temp)));
  float m = -INFINITY;
  for (int i = 0; i < V; ++i) {
    w[i] = orc_rb(orc_bf16_to_f32(lp[i]) * scale);
    m = w[i] > m ? w[i] : m;
  }
  const int inf = (m == INFINITY) || (m == -INFINITY);
  for (int i = 0; i < V; ++i) w[i] = inf ? (w[i] == m ? 1.f : 0.f) : orc_expf(w[i] - m);
  float* cdf = (float*)malloc(sizeof(float) * (size_t)V);
  const float total = orc_cumsum_f32(w, V, cdf);
  free(cdf);
  return total;
}

/* inverse-CDF draw from unnormalised weights with the given raw random word: the first index
 * whose inclusive cumulative sum exceeds u * total, else the last index of positive weight */
ORC_API uint32_t orc_draw_weights(const float* w, int V, uint32_t bits) {
  float* cdf = (float*)malloc(sizeof(float) * (size_t)V);
  const float total = orc_cumsum_f32(w, V, cdf);
  const float u = orc_uniform_scaled(bits, total);
  uint32_t tok = 0xffffffffu, last = 0;
  for (int i = 0; i < V; ++i) {
    if (w[i] > 0.f) last = (uint32_t)i;
    if (tok == 0xffffffffu && cdf[i] > u) tok = (uint32_t)i;
  }
  free(cdf);
  return tok == 0xffffffffu ? last : tok;
}

/* mx.random.categorical(logits * (1/temp)) with the given raw random word */
ORC_API uint32_t orc_categorical(const bf16_t* lp, int V, double temp, uint32_t bits) {
  float* w = (float*)malloc(sizeof(float) * (size_t)V);
  orc_categorical_weights(lp, V, temp, w);
  const uint32_t tok = orc_draw_weights(w, V, bits);
  free(w);
  return tok;
}

/* log-softmax, then top-p / top-k as configured: the filtered log-probabilities the draw sees */
static void filtered_logprobs(const bf16_t* logits, int V, double top_p, int top_k, bf16_t* a) {
  bf16_t* b = (bf16_t*)malloc(sizeof(bf16_t) * (size_t)V);
  orc_logprobs_row(logits, V, a);
  if (top_p > 0.0 && top_p < 1.0) {
    orc_apply_top_p(a, V, top_p, b);
    memcpy(a, b, sizeof(bf16_t) * (size_t)V);
  }
  if (top_k > 0) {
    orc_apply_top_k(a, V, top_k, b);
    memcpy(a, b, sizeof(bf16_t) * (size_t)V);
  }
  free(b);
}

/* The sampler's distribution over one row of logits as unnormalised weights (the probabilities
 * TopSampler draws with are w / total); returns the total. */
ORC_API float orc_sampler_weights(const bf16_t* logits, int V, double temp, double top_p, int top_k, float* w) {
  bf16_t* a = (bf16_t*)malloc(sizeof(bf16_t) * (size_t)V);
  filtered_logprobs(logits, V, top_p, top_k, a);
  const float total = orc_categorical_weights(a, V, temp, w);
  free(a);
  return total;
}

/* TopSampler::sample with the raw random word given (sample.rs:205-225) */
ORC_API uint32_t orc_top_sample_bits(const bf16_t* logits, int V, double temp, double top_p, int top_k,
                                     uint32_t raw) {
  bf16_t* a = (bf16_t*)malloc(sizeof(bf16_t) * (size_t)V);
  filtered_logprobs(logits, V, top_p, top_k, a);
  const uint32_t tok = orc_categorical(a, V, temp, raw);
  free(a);
  return tok;
}

/* TopSampler::sample (sample.rs:205-225): one token from one row of logits; advances the key */
ORC_API uint32_t orc_top_sample(const bf16_t* logits, int V, double temp, double top_p, int top_k,
                                uint32_t key_state[2]) {
  uint32_t sub[2], raw;
  orc_key_next(key_state, sub);
  orc_random_bits(sub, 1, &raw);
  return orc_top_sample_bits(logits, V, temp, top_p, top_k, raw);
}

/* ---- Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3",
 * SC'11; the Random123 library's philox4x32 with 10 rounds). Not in the reference, whose
 * sampler draws from threefry keys; the counter-based generator the sampled speculative
 * configuration asks for. ctr: 128-bit counter, key: 64-bit key. ------------------------- */
ORC_API void orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
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

/* the sampler's stream under Philox: draw number n of seed s is word 0 of
 * philox(counter = (n_lo, n_hi, 0, 0), key = (s_lo, s_hi)) */
ORC_API uint32_t orc_philox_draw(uint64_t seed, uint64_t n) {
  const uint32_t ctr[4] = {(uint32_t)n, (uint32_t)(n >> 32), 0u, 0u};
  const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  uint32_t out[4];
  orc_philox4x32_10(ctr, key, out);
  return out[0];
}

/* ---- speculative sampling (Leviathan, Kalman, Matias 2023; Chen et al. 2023). Not carried by
 * the reference, which accepts a draft by token equality only and says so
 * (src/mtp_generate.rs:27-35). The draft token x was drawn from q; it is accepted with
 * probability min(1, p(x) / q(x)); on rejection the token is drawn from norm(max(0, p - q)).
 * The committed token is then distributed exactly as p whatever q is.
 *   wp / wq: unnormalised weights over the vocabulary, sp / sq their totals (q lives in
 *   vocabulary space: zero outside a pruned draft vocabulary).
 * orc_spec_accept: u = uniform(bits); accept iff u * q(x) < p(x), p(x) = wp[x] / sp,
 *   q(x) = wq[x] / sq (so p(x) >= q(x) always accepts, since u < 1).
 * orc_spec_resample: r_y = max(0, wp[y] / sp - wq[y] / sq), inverse-CDF draw over r with
 *   fresh bits; if every r_y is zero (p == q to the last bit) the draw is over wp instead. */
ORC_API int orc_spec_accept(const float* wp, float sp, const float* wq, float sq, uint32_t x, uint32_t bits) {
  const float px = wp[x] / sp, qx = wq[x] / sq;
  const float u = orc_uniform_scaled(bits, 1.0f);
  return u * qx < px;
}

ORC_API uint32_t orc_spec_resample(const float* wp, float sp, const float* wq, float sq, int V, uint32_t bits) {
  float* r = (float*)malloc(sizeof(float) * (size_t)V * 2);
  float* cdf = r + V;
  for (int y = 0; y < V; ++y) {
    const float d = wp[y] / sp - wq[y] / sq;
    r[y] = d > 0.f ? d : 0.f;
  }
  const float total = orc_cumsum_f32(r, V, cdf);
  const uint32_t tok = total > 0.f ? orc_draw_weights(r, V, bits) : orc_draw_weights(wp, V, bits);
  free(r);
  return tok;
}
