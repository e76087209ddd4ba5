"""Pins for the parts of the sampled speculative configuration the reference does not carry
(it accepts a draft by token equality only, src/mtp_generate.rs:27-35): the Philox4x32-10
stream and probability-ratio acceptance (speculative sampling). CPU only.

  Philox            the published Random123 known-answer vectors (kat_vectors: philox4x32 10)
  acceptance        q == p accepts every draft; the acceptance rate is sum_y min(p_y, q_y);
                    the committed token follows p exactly whatever q is: a chi-square test on a
                    16-token vocabulary, with q pruned to a sub-vocabulary as FR-Spec does
  loop              sampled depth-1..3 generation under ratio acceptance on a tiny model:
                    deterministic per seed, counts consistent, some drafts accepted and some
                    rejected, and the two generators give different streams
"""
import ctypes as C

import numpy as np

import synth
import util
from util import oracle, p


def _philox(ctr, key):
    c, k, out = (C.c_uint32 * 4)(*ctr), (C.c_uint32 * 2)(*key), (C.c_uint32 * 4)()
    oracle().orc_philox4x32_10(c, k, out)
    return list(out)


def test_philox_known_answers():
    # Random123 kat_vectors, "philox4x32 10": counter, key -> output
    assert _philox([0, 0, 0, 0], [0, 0]) == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]
    assert _philox([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2) == [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]
    assert _philox([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0]) == \
        [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]
    # the sampler's stream: draw n of seed s = word 0 of philox((n_lo, n_hi, 0, 0), (s_lo, s_hi))
    f = oracle().orc_philox_draw
    f.restype = C.c_uint32
    seed, n = 0x299F31D0A4093822, 0x85A308D3243F6A88
    assert f(C.c_uint64(seed), C.c_uint64(n)) == _philox([0x243F6A88, 0x85A308D3, 0, 0], [0xA4093822, 0x299F31D0])[0]
    assert f(C.c_uint64(0), C.c_uint64(0)) == 0x6627E8D5


def _accept(wp, wq, x, bits):
    o = oracle()
    return bool(o.orc_spec_accept(p(wp), C.c_float(wp.sum(dtype=np.float32)), p(wq), C.c_float(wq.sum(dtype=np.float32)),
                                  C.c_uint32(x), C.c_uint32(bits)))


def test_equal_distributions_accept_every_draft():
    rng = np.random.default_rng(0)
    w = rng.random(16).astype(np.float32)
    w[3] = 0.0
    for x in np.flatnonzero(w):
        for bits in (0, 1, 0x7FFFFFFF, 0xFFFFFFFF, 12345):
            assert _accept(w, w.copy(), int(x), bits)
    # a scaled copy is the same distribution
    assert all(_accept(w, (w * 4).astype(np.float32), int(x), 0xFFFFFFFF) for x in np.flatnonzero(w))


def test_committed_tokens_follow_the_target_distribution():
    o = oracle()
    draw = o.orc_draw_weights
    draw.restype = C.c_uint32
    res = o.orc_spec_resample
    res.restype = C.c_uint32
    ph = o.orc_philox_draw
    ph.restype = C.c_uint32
    rng = np.random.default_rng(1)
    V, N = 16, 40000
    wp = rng.random(V).astype(np.float32) ** 2
    wq = rng.random(V).astype(np.float32)
    wq[[1, 5, 6, 11, 12, 13]] = 0.0            # a pruned draft vocabulary: q is zero off the list
    wp[2] = 0.0                                 # and a token the target never emits
    sp, sq = C.c_float(wp.sum(dtype=np.float32)), C.c_float(wq.sum(dtype=np.float32))
    # totals as the oracle's own scan gives them (the sums the loop would pass)
    cs = o.orc_cumsum_f32
    cs.restype = C.c_float
    tmp = np.empty(V, np.float32)
    sp, sq = C.c_float(cs(p(wp), V, p(tmp))), C.c_float(cs(p(wq), V, p(tmp)))
    pn, qn = wp.astype(np.float64) / sp.value, wq.astype(np.float64) / sq.value
    counts, accepted, n = np.zeros(V), 0, 0
    for t in range(N):
        x = draw(p(wq), V, C.c_uint32(ph(C.c_uint64(7), C.c_uint64(n)))); n += 1
        if o.orc_spec_accept(p(wp), sp, p(wq), sq, C.c_uint32(x), C.c_uint32(ph(C.c_uint64(7), C.c_uint64(n)))):
            accepted += 1
            tok = x
        else:
            tok = res(p(wp), sp, p(wq), sq, V, C.c_uint32(ph(C.c_uint64(7), C.c_uint64(n + 1))))
            n += 1
        n += 1
        counts[tok] += 1
    assert counts[2] == 0
    live = pn > 0
    chi2 = float((((counts - N * pn) ** 2)[live] / (N * pn[live])).sum())
    assert chi2 < 45.0, chi2          # 14 degrees of freedom: P(chi2 > 45) < 1e-4
    want_rate = np.minimum(pn, qn).sum()
    assert abs(accepted / N - want_rate) < 4 * np.sqrt(want_rate * (1 - want_rate) / N), (accepted / N, want_rate)
    # a wrong rule is caught: accepting by equality with an independent draw from p does not give p
    counts2 = np.zeros(V)
    for t in range(N):
        x = draw(p(wq), V, C.c_uint32(ph(C.c_uint64(8), C.c_uint64(2 * t))))
        counts2[x] += 1                                       # "always accept": committed ~ q
    chi2_bad = float((((counts2 - N * pn) ** 2)[live] / (N * pn[live])).sum())
    assert chi2_bad > 1000.0


def test_resample_falls_back_to_the_target_when_the_residual_is_empty():
    res = oracle().orc_spec_resample
    res.restype = C.c_uint32
    draw = oracle().orc_draw_weights
    draw.restype = C.c_uint32
    w = np.array([0.0, 1.0, 2.0, 0.0, 5.0], np.float32)
    for bits in (0, 0x40000000, 0xFFFFFFFF):
        assert res(p(w), C.c_float(8.0), p(w), C.c_float(8.0), 5, C.c_uint32(bits)) == draw(p(w), 5, C.c_uint32(bits))
    # residual mass only where p exceeds q
    wq = np.array([0.0, 4.0, 0.0, 0.0, 4.0], np.float32)
    assert {res(p(w), C.c_float(8.0), p(wq), C.c_float(8.0), 5, C.c_uint32(b)) for b in range(0, 2 ** 32, 2 ** 27)} == {2, 4}


def test_sampled_loop_with_ratio_acceptance():
    V = 32
    s = synth.SynthModel(dict(synth.TINY, vocab_size=V), seed=12)
    prompt = np.random.default_rng(7).integers(0, V, 11).astype(np.uint32)
    n = 30
    fr_ids = synth.zipf_frspec_ids(V, 24, seed=1)
    fr_host = synth.prune_head(s.lm_head, fr_ids)
    runs = {}
    try:
        for rng_kind in (0, 1):
            for depth in (1, 3):
                for use_fr in (False, True):
                    out = []
                    for rep in range(2):
                        r = synth.OracleRun(s, 64)
                        r.set_sampler(1, 0.8, 0.95, 0, seed=99, accept=1, rng=rng_kind)
                        toks, st = r.mtp_generate(prompt, depth, n, fr_ids if use_fr else None,
                                                  fr_host if use_fr else None, policy=1, prefill_step=4)
                        assert r.o.orc_state_offset(r.st) == len(prompt) + n
                        r.close()
                        assert len(toks) == n and all(0 <= t < V for t in toks)
                        assert st.accepted <= st.drafted and st.cycles >= 1
                        assert sum(st.accepted_by) == st.accepted and st.reached[0] == st.cycles
                        out.append((toks, st.cycles, st.drafted, st.accepted))
                    assert out[0] == out[1]                      # deterministic per seed
                    runs[(rng_kind, depth, use_fr)] = out[0]
        acc = sum(v[3] for v in runs.values())
        dr = sum(v[2] for v in runs.values())
        assert 0 < acc < dr                                      # both branches of the rule ran
        assert runs[(0, 1, False)][0] != runs[(1, 1, False)][0]  # the generators differ
    finally:
        synth.util.oracle().orc_set_sampler(0, C.c_double(1.0), C.c_double(1.0), 0, C.c_uint64(0))


def test_sampler_weights_against_float64():
    """orc_sampler_weights (the unnormalised distribution both sides of the acceptance ratio
    use): w_i = exp((lp_i - max) / T) over the filtered log-probabilities, 0 for a filtered-out
    token, and the returned total is their sum. Checked against float64 on the surviving set
    the oracle's own (separately pinned) top-p / top-k stages name; the temperature enters as
    the bf16-rounded 1/T and the scaled log-probability is rounded to bf16 before the exponential,
    as the reference's categorical draw does, so the comparison allows that rounding."""
    f = oracle().orc_sampler_weights
    f.restype = C.c_float
    rng = np.random.default_rng(4)
    V = 300
    for temp, top_p, top_k in ((0.8, 0.95, 0), (1.0, 1.0, 0), (0.6, 0.9, 20), (1.3, 0.5, 0)):
        logits = util.bf16_normal(rng, (V,), 2.5)
        w = np.empty(V, np.float32)
        total = f(p(logits), V, C.c_double(temp), C.c_double(top_p), top_k, p(w))
        # the filtered log-probabilities, from the stages pinned in test_oracle_sampler.py
        lp = np.empty(V, np.uint16)
        oracle().orc_logprobs_row(p(logits), V, p(lp))
        if 0.0 < top_p < 1.0:
            b = np.empty(V, np.uint16)
            oracle().orc_apply_top_p(p(lp), V, C.c_double(top_p), p(b))
            lp = b
        if top_k > 0:
            b = np.empty(V, np.uint16)
            oracle().orc_apply_top_k(p(lp), V, top_k, p(b))
            lp = b
        lpf = util.bf16_to_f32(lp).astype(np.float64)
        keep = np.isfinite(lpf)
        assert 0 < keep.sum() <= V and (top_k == 0 or keep.sum() <= top_k)
        assert np.all(w[~keep] == 0.0) and np.all(w[keep] > 0.0)
        inv_t = float(util.bf16_to_f32(util.f32_to_bf16(np.array([1.0 / temp], np.float32)))[0])
        z = lpf[keep] * inv_t
        want = np.exp(z - z.max())
        # z is rounded to bf16 (relative 2^-9 of |z|) before the exponential: an absolute error of
        # up to 2^-9 |z| in the exponent, i.e. that much relative error in w
        tol = 2.0 ** -8 * np.maximum(np.abs(z), np.abs(z.max())) + 1e-6
        assert np.all(np.abs(w[keep] / want - 1.0) <= tol), float(np.max(np.abs(w[keep] / want - 1.0) / tol))
        assert w[keep].max() == 1.0            # the most likely token has weight exp(0)
        assert abs(float(total) - float(np.sum(w.astype(np.float64)))) <= 1e-5 * float(total)
