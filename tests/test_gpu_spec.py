"""GPU parity for the sampled speculative configuration: the distribution-as-weights operators,
probability-ratio acceptance and the Philox stream, bit for bit against the oracle, and the
sampled depth-1..3 loop under ratio acceptance (tokens, counts, cache length) against the
oracle's loop."""
import ctypes as C

import numpy as np
import pytest

import synth
import util
from util import oracle, p

pytestmark = pytest.mark.gpu


def _orc_weights(logits, temp, top_p, top_k):
    V = logits.size
    w = np.empty(V + 1, np.float32)
    f = oracle().orc_sampler_weights
    f.restype = C.c_float
    w[V] = f(p(logits), V, C.c_double(temp), C.c_double(top_p), top_k, p(w))
    return w


@pytest.mark.parametrize("V,temp,top_p,top_k", [(248320, 0.8, 0.95, 0), (32768, 0.6, 0.95, 20), (5000, 1.0, 1.0, 0),
                                                (1000, 0.8, 0.5, 0)])
def test_weights_draw_accept_resample_bit_exact(orn, ctx, V, temp, top_p, top_k):
    rng = np.random.default_rng(V)
    o = oracle()
    draw = o.orc_draw_weights; draw.restype = C.c_uint32
    res = o.orc_spec_resample; res.restype = C.c_uint32
    lp_, lq_ = util.bf16_normal(rng, (V,), 3.0), util.bf16_normal(rng, (V,), 3.0)
    # a draft distribution close to the target's (so both branches of the rule occur)
    lq_ = util.f32_to_bf16(util.bf16_to_f32(lp_) + 0.5 * util.bf16_to_f32(lq_))
    s = orn.TopSampler(ctx, temp, top_p, top_k, seed=5, vocab=V)
    dlp, dlq = ctx.to_device(lp_), ctx.to_device(lq_)
    dwp, dwq = ctx.alloc((V + 1) * 4), ctx.alloc((V + 1) * 4)
    tok, flag = ctx.alloc(4), ctx.alloc(4)
    try:
        s.weights(dlp, V, dwp); s.weights(dlq, V, dwq)
        wp, wq = _orc_weights(lp_, temp, top_p, top_k), _orc_weights(lq_, temp, top_p, top_k)
        assert np.array_equal(dwp.download(np.uint32, (V + 1,)), wp.view(np.uint32))
        assert np.array_equal(dwq.download(np.uint32, (V + 1,)), wq.view(np.uint32))
        n_acc = 0
        for i, bits in enumerate([0, 1, 0x3FFFFFFF, 0x7FFFFFFF, 0xBFFFFFFF, 0xFFFFFFFF] + list(rng.integers(0, 2 ** 32, 10))):
            bits = int(bits)
            orn.draw_weights(ctx, dwq, V, bits, tok)
            x = int(tok.download(np.uint32, (1,))[0])
            assert x == draw(p(wq), V, C.c_uint32(bits))
            b2 = int(rng.integers(0, 2 ** 32))
            orn.spec_accept(ctx, dwp, dwq, V, tok, b2, flag)
            got = int(flag.download(np.uint32, (1,))[0])
            want = o.orc_spec_accept(p(wp), C.c_float(wp[V]), p(wq), C.c_float(wq[V]), C.c_uint32(x), C.c_uint32(b2))
            assert got == want
            n_acc += got
            orn.spec_resample(ctx, dwp, dwq, V, bits, tok)
            assert int(tok.download(np.uint32, (1,))[0]) == res(p(wp), C.c_float(wp[V]), p(wq), C.c_float(wq[V]), V,
                                                                 C.c_uint32(bits))
        assert 0 < n_acc < 16
        # an empty residual falls back to the target
        orn.spec_resample(ctx, dwp, dwp, V, 0x12345678, tok)
        assert int(tok.download(np.uint32, (1,))[0]) == draw(p(wp), V, C.c_uint32(0x12345678))
        orn.spec_accept(ctx, dwp, dwp, V, tok, 0xFFFFFFFF, flag)
        assert int(flag.download(np.uint32, (1,))[0]) == 1
    finally:
        for b in (dlp, dlq, dwp, dwq, tok, flag): b.free()
        s.close()


def test_scatter_places_pruned_weights_in_vocabulary_space(orn, ctx):
    rng = np.random.default_rng(2)
    V, n = 4096, 600
    ids = rng.permutation(V)[:n].astype(np.uint32)
    wl = np.append(rng.random(n).astype(np.float32), np.float32(123.5))
    dwl, did, dwf = ctx.to_device(wl), ctx.to_device(ids), ctx.alloc((V + 1) * 4)
    orn.spec_scatter(ctx, dwl, did, n, V, dwf)
    got = dwf.download(np.float32, (V + 1,))
    want = np.zeros(V + 1, np.float32); want[ids] = wl[:n]; want[V] = 123.5
    assert np.array_equal(got, want)
    for b in (dwl, did, dwf): b.free()


def test_sampler_streams(orn, ctx):
    """next_bits: the threefry key sequence as before, the Philox counter stream on request."""
    ph = oracle().orc_philox_draw; ph.restype = C.c_uint32
    s = orn.TopSampler(ctx, 0.8, 0.95, 0, seed=0x0123456789ABCDEF, vocab=64)
    st = orn.random_key(0x0123456789ABCDEF)
    for _ in range(3):
        st, sub = util.orc_key_next(st)
        assert s.next_bits() == int(util.orc_random_bits(sub, 1)[0])
    s.set_rng(orn.RNG_PHILOX)
    assert [s.next_bits() for _ in range(4)] == [ph(C.c_uint64(0x0123456789ABCDEF), C.c_uint64(n)) for n in range(4)]
    s.close()


@pytest.fixture(scope="module")
def tiny_small_vocab(orn, ctx):
    s = synth.SynthModel(dict(synth.TINY, vocab_size=32), seed=12)
    ws = s.upload(orn, ctx)
    model = orn.TextModel(ctx, ws, s.text_config(orn))
    yield s, ws, model
    model.close()
    ws.close()


@pytest.mark.parametrize("rng_kind", [0, 1])
def test_sampled_loop_with_ratio_acceptance_matches_oracle(orn, ctx, tiny_small_vocab, rng_kind):
    s, ws, model = tiny_small_vocab
    V = s.cfg["vocab_size"]
    prompt = np.random.default_rng(7).integers(0, V, 11).astype(np.uint32)
    n_tok, cap = 30, 11 + 30 + 8
    fr_ids = synth.zipf_frspec_ids(V, 24, seed=1)
    fr_host = synth.prune_head(s.lm_head, fr_ids)
    fr = orn.FrSpec(model, ids=fr_ids)
    caches = model.make_cache(cap, 4)
    head = orn.MtpHead(model, ws, cap)
    smp = orn.Sampler(1, 0.8, 0.95, 0, 99, orn.ACCEPT_RATIO, rng_kind)
    acc = dr = 0
    try:
        for depth in (1, 3):
            for use_fr in (False, True):
                caches.reset()
                toks, st = orn.generate_step_mtp(model, head, fr if use_fr else None, caches, prompt, depth, n_tok,
                                                 sampler=smp, prefill_step=4, policy=orn.HISTORY_COMMITTED)
                r = synth.OracleRun(s, cap)
                r.set_sampler(1, 0.8, 0.95, 0, seed=99, accept=1, rng=rng_kind)
                otoks, ost = r.mtp_generate(prompt, depth, n_tok, fr_ids if use_fr else None, fr_host if use_fr else None,
                                            policy=1, prefill_step=4)
                r.close()
                assert toks == otoks, (depth, use_fr)
                assert (st.cycles, st.drafted, st.accepted) == (ost.cycles, ost.drafted, ost.accepted)
                assert list(st.reached_by_depth) == list(ost.reached) and caches.offset == 11 + n_tok
                acc, dr = acc + st.accepted, dr + st.drafted
        assert 0 < acc < dr
    finally:
        oracle().orc_set_sampler(0, C.c_double(1.0), C.c_double(1.0), 0, C.c_uint64(0))
        fr.close(); head.close(); caches.close()


def test_config5_sequence_on_the_tiny_model(orn, ctx):
    """The sampled configuration end to end at its cache size: a 700-token prompt through the
    matrix-core prefill path (256-row calls), then sampled depth-3 decode with probability-ratio
    acceptance and the Philox stream into a 16384-row cache. The prefill path is a tolerance
    path (its sums run in another order than the oracle's), so what is pinned here is what the
    configuration promises: the same seed gives the same tokens and counts on every run, another
    seed gives another sequence, the counts are consistent and the caches end where the loop's
    contract says (prompt + tokens shown)."""
    s = synth.SynthModel(dict(synth.TINY, vocab_size=512), seed=21)
    ws = s.upload(orn, ctx)
    model = orn.TextModel(ctx, ws, s.text_config(orn))
    model.set_max_rows(256)
    V = s.cfg["vocab_size"]
    n_prompt, n_tok, cap, depth = 700, 48, 16384, 3
    prompt = np.random.default_rng(3).integers(0, V, n_prompt).astype(np.uint32)
    fr = orn.FrSpec(model, ids=synth.zipf_frspec_ids(V, 128, seed=1))
    caches = model.make_cache(cap, depth + 1)
    head = orn.MtpHead(model, ws, cap)
    runs = []
    try:
        for seed in (2025, 2025, 7):
            caches.reset()
            smp = orn.Sampler(1, 0.8, 0.95, 0, seed, orn.ACCEPT_RATIO, orn.RNG_PHILOX)
            toks, st = orn.generate_step_mtp(model, head, fr, caches, prompt, depth, n_tok, sampler=smp,
                                             prefill_step=256, policy=orn.HISTORY_COMMITTED)
            assert len(toks) == n_tok and caches.offset == n_prompt + n_tok
            assert 0 <= st.accepted <= st.drafted <= depth * st.cycles and st.cycles >= n_tok // (depth + 1)
            assert st.accepted + st.cycles >= n_tok - 1
            runs.append((toks, (int(st.cycles), int(st.drafted), int(st.accepted))))
        assert runs[0] == runs[1], "same seed, different sampled sequence"
        assert runs[0][0] != runs[2][0], "another seed gave the same 48 sampled tokens"
    finally:
        for o in (fr, head, caches, model, ws):
            o.close()
