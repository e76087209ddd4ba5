// The two generation loops.
//
// Mirrors generate::{prefill, step, generate_step}
// (/root/reference/src/generate.rs:86-206) and mtp_generate::{draft,
// generate_step_mtp} (/root/reference/src/mtp_generate.rs:99-317): same order of
// model calls, same points at which a token is handed to the caller, same cache
// contract (on return the caches hold the prompt plus exactly the tokens shown to
// on_token), same statistics. One blocking read-back per speculative cycle.
#include <algorithm>
#include <vector>

#include "model.h"

#define TRY(e)             \
  do {                     \
    int rc__ = (e);        \
    if (rc__) return rc__; \
  } while (0)

// sample.hip: argmax over a pruned head's rows stored as vocabulary ids (FrSpec::map_id,
// src/frspec.rs:140-142, inside the argmax's last launch)
int argmax_rows_mapped(ornith_ctx* ctx, const void* d_logits, int rows, int V, const uint32_t* d_id_map,
                       uint32_t* d_out);

namespace {

// device buffers a generation call needs, freed on scope exit
struct Bufs {
  ornith_ctx* ctx;
  std::vector<void*> all;
  explicit Bufs(ornith_ctx* c) : ctx(c) {}
  ~Bufs() {
    for (void* p : all) ornith_free(ctx, p);
  }
  int get(size_t bytes, void** out) {
    int rc = ornith_alloc(ctx, bytes, out);
    if (!rc) all.push_back(*out);
    return rc;
  }
};

// The `Sampler` a loop drives (src/generate.rs:36-64): Greedy, or TopSampler built from
// the tagged struct. rows_are_independent() is true for Greedy only: every draw of the
// other advances its key, so rows are sampled one by one and only when asked for.
struct LoopSampler {
  ornith_ctx* ctx = nullptr;
  ornith_top_sampler* top = nullptr;
  int V = 0;
  bool ratio = false;  // drafts drawn from the head's distribution and accepted by probability ratio
  ~LoopSampler() {
    if (top) ornith_top_sampler_destroy(top);
  }
  int init(ornith_ctx* c, const ornith_sampler* s, int vocab) {
    ORN_REQUIRE(s, "sampler is null");
    ctx = c;
    V = vocab;
    if (s->kind == ORNITH_SAMPLER_GREEDY) return ORNITH_OK;
    ORN_REQUIRE(s->kind == ORNITH_SAMPLER_TOP_P, "unknown sampler kind %d", s->kind);
    ORN_REQUIRE(s->accept == ORNITH_ACCEPT_EQUALITY || s->accept == ORNITH_ACCEPT_RATIO,
                "unknown acceptance rule %d", s->accept);
    ORN_REQUIRE(s->rng == ORNITH_RNG_THREEFRY || s->rng == ORNITH_RNG_PHILOX, "unknown generator %d", s->rng);
    TRY(ornith_top_sampler_create(c, s->temperature, s->top_p, s->top_k, s->seed, vocab, &top));
    ratio = s->accept == ORNITH_ACCEPT_RATIO;
    return ornith_top_sampler_set_rng(top, s->rng);
  }
  int next_bits(uint32_t* bits) { return ornith_top_sampler_next_bits(top, bits); }
  bool rows_are_independent() const { return top == nullptr; }
  // one row of logits -> token on the device
  int sample(const void* d_logits_row, uint32_t* d_token) {
    if (top) return ornith_top_sampler_sample(top, d_logits_row, d_token);
    return ornith_greedy_rows(ctx, d_logits_row, 1, V, d_token, nullptr);
  }
};

// prefill (src/generate.rs:90-136): everything but the last token, in chunks
int prefill(ornith_model* m, ornith_caches* c, const uint32_t* prompt, size_t total, size_t step,
            uint32_t* d_tok, void* d_hidden, ornith_progress_cb progress, void* user,
            size_t* processed_out) {
  size_t processed = 0;
  if (progress) progress(0, total, user);
  const size_t chunk = std::max<size_t>(1, std::min<size_t>(step, (size_t)m->max_rows));
  while (total - processed > 1) {
    const size_t n = std::min(chunk, total - processed - 1);
    TRY(ornith_upload(m->ctx, d_tok, prompt + processed, n * 4));
    TRY(ornith_model_forward(m, c, d_tok, (int)n, 0, d_hidden));
    TRY(ornith_sync(m->ctx));
    processed += n;
    if (progress) progress(processed, total, user);
  }
  *processed_out = processed;
  return ORNITH_OK;
}

}  // namespace

extern "C" {

int ornith_generate(ornith_model* m, ornith_caches* c, const uint32_t* prompt, size_t n_prompt,
                    const ornith_sampler* sampler, size_t max_tokens, size_t prefill_step,
                    ornith_progress_cb progress, ornith_token_cb on_token, void* user) {
  ORN_REQUIRE(m && c && prompt && on_token, "generate: null argument");
  ORN_REQUIRE(n_prompt >= 1, "generate_step needs a prompt");
  // caches whose capacity has been fixed (ornith_caches_set_growable(c, 0)): refuse a run that
  // cannot finish before any token has been handed out; growable ones grow as the rows arrive
  ORN_REQUIRE(caches_fit(c, (size_t)c->offset + n_prompt + max_tokens),
              "generate: %d cached + %zu prompt + %zu new tokens exceed cache capacity %d", c->offset, n_prompt,
              max_tokens, c->capacity);
  ornith_ctx* ctx = m->ctx;
  const size_t H = m->cfg.hidden_size, V = m->cfg.vocab_size, R = m->max_rows;
  LoopSampler smp;
  TRY(smp.init(ctx, sampler, (int)V));
  Bufs b(ctx);
  uint32_t *d_tok, *d_out;
  void *d_hidden, *d_logits;
  TRY(b.get(R * 4, (void**)&d_tok));
  TRY(b.get(4, (void**)&d_out));
  TRY(b.get(R * H * 2, &d_hidden));
  TRY(b.get(V * 2, &d_logits));

  size_t processed = 0;
  TRY(prefill(m, c, prompt, n_prompt, prefill_step, d_tok, d_hidden, progress, user, &processed));
  // step(): run the n tokens in d_tok and sample from the last position; the one wait of the
  // step is the read-back of the sampled id
  auto step = [&](const uint32_t* d_in, size_t n, uint32_t* y) -> int {
    TRY(ornith_model_forward(m, c, d_in, (int)n, 0, d_hidden));
    TRY(ornith_model_logits(m, (char*)d_hidden + (n - 1) * H * 2, 1, d_logits));
    TRY(smp.sample(d_logits, d_out));
    return ornith_download(ctx, y, d_out, 4);
  };
  uint32_t y = 0;
  TRY(ornith_upload(ctx, d_tok, prompt + processed, (n_prompt - processed) * 4));
  TRY(step(d_tok, n_prompt - processed, &y));
  if (progress) progress(n_prompt, n_prompt, user);
  size_t n = 0;
  for (;;) {
    if (n == max_tokens) return ORNITH_OK;
    uint32_t next = 0;
    // the token just sampled is fed back from where it lies on the device: the forward
    // reads it in its first launch, the sampler overwrites it in the step's last
    TRY(step(d_out, 1, &next));
    if (!on_token(y, user)) return ORNITH_OK;
    y = next;
    ++n;
  }
}

int ornith_mtp_generate(ornith_model* m, ornith_mtp_head* head, const ornith_frspec* frspec,
                        ornith_caches* c, const uint32_t* prompt, size_t n_prompt,
                        const ornith_sampler* sampler, int depth, size_t max_tokens,
                        size_t prefill_step, int policy, ornith_progress_cb progress,
                        ornith_token_cb on_token, void* user, ornith_mtp_stats* stats_out) {
  ORN_REQUIRE(m && head && c && prompt && on_token, "mtp_generate: null argument");
  ORN_REQUIRE(depth >= 1, "MTP depth must be at least 1");
  ORN_REQUIRE(depth <= ORNITH_MAX_DEPTH && depth + 1 <= c->max_window,
              "mtp_generate: depth %d needs a capture window of %d rows (caches have %d)", depth,
              depth + 1, c->max_window);
  ORN_REQUIRE(n_prompt >= 1, "generate_step_mtp needs a prompt");
  ORN_REQUIRE(max_tokens >= 1, "mtp_generate: max_tokens must be at least 1");
  ORN_REQUIRE(policy == ORNITH_HISTORY_CYCLE || policy == ORNITH_HISTORY_COMMITTED,
              "mtp_generate: unknown history policy %d", policy);
  ORN_REQUIRE(head->m == m && (!frspec || frspec->m == m), "mtp_generate: head / frspec of another model");
  if (stats_out) *stats_out = ornith_mtp_stats{};  // defined on every return, error returns included
  // a verify window holds up to `depth` rows beyond the committed ones; the head's own cache
  // holds one row per committed token under Committed, a cycle's rows under Cycle. With caches
  // of fixed capacity a run that cannot fit is refused up front rather than failing between two
  // tokens already handed out; growable caches grow as the rows arrive.
  ORN_REQUIRE(caches_fit(c, (size_t)c->offset + n_prompt + max_tokens + (size_t)depth),
              "mtp_generate: %d cached + %zu prompt + %zu new tokens + a %d-row window exceed cache capacity %d",
              c->offset, n_prompt, max_tokens, depth, c->capacity);
  ORN_REQUIRE(mtp_cache_fits(head, policy == ORNITH_HISTORY_COMMITTED ? max_tokens + (size_t)depth : (size_t)depth),
              "mtp_generate: the head's cache of %d rows is too small for %zu tokens at depth %d under this "
              "history policy", head->capacity, max_tokens, depth);
  ornith_ctx* ctx = m->ctx;
  const size_t H = m->cfg.hidden_size, V = m->cfg.vocab_size, R = m->max_rows;
  LoopSampler smp;
  TRY(smp.init(ctx, sampler, (int)V));
  ornith_mtp_stats stats{};
  // an error return below still reports the cycles counted so far
  struct StatsOut {
    ornith_mtp_stats* out;
    const ornith_mtp_stats* cur;
    ~StatsOut() {
      if (out) *out = *cur;
    }
  } stats_guard{stats_out, &stats};

  Bufs b(ctx);
  uint32_t *d_tok, *d_window, *d_targets;
  void *d_hidden, *d_vlogits, *d_dlogits, *d_mh, *d_scratch_h;
  const size_t W = (size_t)depth + 1;
  TRY(b.get(R * 4, (void**)&d_tok));
  TRY(b.get(2 * W * 4, (void**)&d_window));  // window, then the targets: one read-back a cycle
  d_targets = d_window + W;
  TRY(b.get(R * H * 2, &d_hidden));
  TRY(b.get(W * V * 2, &d_vlogits));
  TRY(b.get(V * 2, &d_dlogits));
  TRY(b.get(W * H * 2, &d_mh));
  TRY(b.get(W * H * 2, &d_scratch_h));
  // probability-ratio acceptance keeps every draft level's distribution q (vocabulary space)
  // for the verify pass, the target's p of the row in hand, and a flag word
  float *d_wq = nullptr, *d_wp = nullptr, *d_wloc = nullptr;
  uint32_t* d_flag = nullptr;
  if (smp.ratio) {
    TRY(b.get((size_t)depth * (V + 1) * 4, (void**)&d_wq));
    TRY(b.get((V + 1) * 4, (void**)&d_wp));
    TRY(b.get((V + 1) * 4, (void**)&d_wloc));
    TRY(b.get(4, (void**)&d_flag));
  }

  size_t processed = 0;
  TRY(prefill(m, c, prompt, n_prompt, prefill_step, d_tok, d_hidden, progress, user, &processed));
  const size_t rows = n_prompt - processed;
  TRY(ornith_upload(ctx, d_tok, prompt + processed, rows * 4));
  TRY(ornith_model_forward(m, c, d_tok, (int)rows, 0, d_hidden));
  TRY(ornith_model_logits(m, (char*)d_hidden + (rows - 1) * H * 2, 1, d_vlogits));
  TRY(smp.sample(d_vlogits, d_targets));
  uint32_t primary = 0;
  TRY(ornith_download(ctx, &primary, d_targets, 4));
  // the prompt is consumed once its last position has been sampled from, as in generate_step
  if (progress) progress(n_prompt, n_prompt, user);
  // the trunk hidden a cycle drafts from is read where the last forward left it: the next
  // write to d_hidden is the cycle's verify pass, after the drafts
  const void* d_h = (char*)d_hidden + (rows - 1) * H * 2;

  size_t emitted = 0;
  TRY(ornith_mtp_cache_set_offset(head, 0));  // make_mtp_cache()
  const int draft_vocab = frspec ? frspec->n : (int)V;
  std::vector<uint32_t> wt(2 * W);
  uint32_t* const win = wt.data();
  uint32_t* const targets = wt.data() + W;
  // the token every cycle starts from lies on the device where it was sampled
  TRY(ornith_copy(ctx, d_window, d_targets, 4));
  for (;;) {
    if (policy == ORNITH_HISTORY_CYCLE) TRY(ornith_mtp_cache_set_offset(head, 0));
    const int cycle_mtp_offset = head->offset;
    const size_t left = max_tokens > emitted + 1 ? max_tokens - (emitted + 1) : 0;
    const int want = (int)std::min<size_t>((size_t)depth, left);

    // draft(): `want` chained head forwards, entirely on the device (d_window[0] holds the
    // primary token; the chain fills the entries after it)
    const void* hcur = d_h;
    for (int i = 0; i < want; ++i) {
      void* hid = (char*)d_mh + (size_t)i * H * 2;
      TRY(ornith_mtp_forward(head, frspec, hcur, d_window + i, 1, hid, d_dlogits));
      if (smp.ratio) {
        // the draft is DRAWN from the head's distribution under the sampler's own settings
        float* q = d_wq + (size_t)i * (V + 1);
        uint32_t bits = 0;
        TRY(smp.next_bits(&bits));
        if (frspec) {
          TRY(ornith_sampler_weights(smp.top, d_dlogits, draft_vocab, d_wloc));
          TRY(ornith_draw_weights(ctx, d_wloc, draft_vocab, bits, d_flag));
          TRY(ornith_gather_rows(ctx, frspec->d_ids, 4, d_flag, 1, d_window + i + 1));  // map_id
          TRY(ornith_spec_scatter(ctx, d_wloc, frspec->d_ids, draft_vocab, (int)V, q));
        } else {
          TRY(ornith_sampler_weights(smp.top, d_dlogits, (int)V, q));
          TRY(ornith_draw_weights(ctx, q, (int)V, bits, d_window + i + 1));
        }
      } else if (frspec) {
        // FrSpec::map_id rides in the argmax's last launch
        TRY(argmax_rows_mapped(ctx, d_dlogits, 1, draft_vocab, frspec->d_ids, d_window + i + 1));
      } else {
        TRY(ornith_argmax_rows(ctx, d_dlogits, 1, draft_vocab, d_window + i + 1));
      }
      // a forced draft (measurement aid) takes the place of the head's own
      const size_t pos = emitted + 1 + (size_t)i;
      if (pos < head->n_forced) TRY(ornith_copy(ctx, d_window + i + 1, head->d_forced + pos, 4));
      hcur = hid;
    }
    if (want > 0) {
      stats.cycles += 1;
      stats.drafted += want;
    }

    // verify: one trunk forward over [primary] + drafts, every row's target at once
    const int n_rows = want + 1;
    TRY(ornith_model_forward(m, c, d_window, n_rows, 1, d_hidden));
    TRY(ornith_model_logits(m, d_hidden, n_rows, d_vlogits));
    const bool independent = smp.rows_are_independent();
    if (independent) {
      TRY(ornith_greedy_rows(ctx, d_vlogits, n_rows, (int)V, d_targets, nullptr));
      TRY(ornith_download(ctx, wt.data(), d_window, 2 * W * 4));  // the cycle's one wait
    } else {
      TRY(ornith_download(ctx, win, d_window, (size_t)n_rows * 4));
    }
    // a dependent sampler draws row by row, as far as the accept loop asks
    auto take = [&](int row, uint32_t* t) -> int {
      if (independent) {
        *t = targets[row];
        return ORNITH_OK;
      }
      TRY(smp.sample((const char*)d_vlogits + (size_t)row * V * 2, d_targets + row));
      return ornith_download(ctx, t, d_targets + row, 4);
    };

    // accept the leading run of agreements
    int k = 0;
    bool have_next = false;
    uint32_t next_primary = 0;
    while (k < want) {
      if (smp.ratio) {
        // accept with probability min(1, p(x) / q(x)); a rejected position is redrawn from
        // norm(max(0, p - q)) and ends the cycle
        const float* q = d_wq + (size_t)k * (V + 1);
        uint32_t bits = 0, ok = 0;
        TRY(ornith_sampler_weights(smp.top, (const char*)d_vlogits + (size_t)k * V * 2, (int)V, d_wp));
        TRY(smp.next_bits(&bits));
        TRY(ornith_spec_accept(ctx, d_wp, q, (int)V, d_window + 1 + k, bits, d_flag));
        TRY(ornith_download(ctx, &ok, d_flag, 4));
        stats.reached_by_depth[k] += 1;
        if (!ok) {
          TRY(smp.next_bits(&bits));
          TRY(ornith_spec_resample(ctx, d_wp, q, (int)V, bits, d_targets + k));
          TRY(ornith_download(ctx, &next_primary, d_targets + k, 4));
          have_next = true;
          break;
        }
      } else {
        uint32_t target = 0;
        TRY(take(k, &target));
        stats.reached_by_depth[k] += 1;
        if (target != win[1 + k]) {
          next_primary = target;
          have_next = true;
          break;
        }
      }
      stats.accepted_by_depth[k] += 1;
      stats.accepted += 1;
      ++k;
    }
    if (!have_next) TRY(take(k, &next_primary));  // the bonus token

    // the window put want+1 tokens into the caches; k+1 of them are committed
    TRY(ornith_model_rewind(m, c, k + 1));
    if (policy == ORNITH_HISTORY_COMMITTED) {
      // keep the level-1 row (it drafted from the trunk's hidden), rebuild the rest
      // from what the verify pass actually saw
      TRY(ornith_mtp_cache_reserve(head, cycle_mtp_offset + 1 + k));
      TRY(ornith_mtp_cache_set_offset(head, std::min(cycle_mtp_offset + 1, head->capacity)));
      if (k > 0) TRY(ornith_mtp_forward(head, nullptr, d_hidden, d_window + 1, k, d_scratch_h, nullptr));
    }
    d_h = (char*)d_hidden + (size_t)k * H * 2;
    // next cycle's primary token: row k's target (the correction or the bonus token)
    TRY(ornith_copy(ctx, d_window, d_targets + k, 4));

    for (int i = 0; i <= k; ++i) {
      const uint32_t t = i == 0 ? primary : win[i];
      if (!on_token(t, user)) {
        if (stats_out) *stats_out = stats;
        return ORNITH_OK;
      }
      ++emitted;
      if (emitted == max_tokens) {
        if (stats_out) *stats_out = stats;
        return ORNITH_OK;
      }
    }
    primary = next_primary;
  }
}

}  // extern "C"
