"""GPU parity at model level on reduced configurations: trunk forward / capture / rewind,
MTP head, FR-Spec, and both generation loops vs the CPU oracle. Hidden states and logits
are compared by bf16 bits, tokens and acceptance counters exactly. The reference's own
release check -- greedy speculative output identical to plain greedy
(/root/reference/README.md:193-197, tests/mtp.rs:246-349) -- is asserted on both sides."""
import os
import struct

import numpy as np
import pytest

import synth
import util

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tiny(orn, ctx):
    s = synth.SynthModel(synth.TINY, seed=11)
    ws = s.upload(orn, ctx)
    model = orn.TextModel(ctx, ws, s.text_config(orn))
    yield s, ws, model
    model.close()
    ws.close()


@pytest.fixture(scope="module")
def tiny_small_vocab(orn, ctx):
    """vocab 32: random drafts agree often enough to exercise acceptance and history repair"""
    s = synth.SynthModel(dict(synth.TINY, vocab_size=32), seed=12)
    ws = s.upload(orn, ctx)
    model = orn.TextModel(ctx, ws, s.text_config(orn))
    yield s, ws, model
    model.close()
    ws.close()


def test_forward_capture_rewind_bit_exact(orn, ctx, tiny):
    s, ws, model = tiny
    rng = np.random.default_rng(0)
    toks = rng.integers(0, s.cfg["vocab_size"], 12).astype(np.uint32)
    caches = model.make_cache(64, 4)
    orc = synth.OracleRun(s, 64)
    # a 5-token chunk (prefill width), then single steps, then a captured window
    for chunk, cap in ((toks[:5], False), (toks[5:6], False), (toks[6:7], False), (toks[7:10], True)):
        got = model.forward(caches, chunk, capture=cap)
        want = orc.forward(chunk, capture=cap)
        assert np.array_equal(got, want), (len(chunk), cap)
    assert caches.offset == 10 == util.oracle().orc_state_offset(orc.st)
    # reject two of the three window tokens, then continue: must equal the oracle doing the same,
    # and must equal a run that never saw the rejected tokens
    model.rewind(caches, 1)
    orc.rewind(1)
    assert caches.offset == 8
    nxt = model.forward(caches, toks[10:12])
    assert np.array_equal(nxt, orc.forward(toks[10:12]))
    fresh = model.make_cache(64, 4)
    model.forward(fresh, toks[:5]); model.forward(fresh, toks[5:8])
    assert np.array_equal(model.forward(fresh, toks[10:12]), nxt)
    # logits and the greedy choice
    lg = model.logits(nxt)
    assert np.array_equal(lg, orc.logits(nxt))
    for c in (caches, fresh): c.close()
    orc.close()


def test_batch_invariance_chunking_does_not_matter(orn, ctx, tiny):
    """row r of a T-row forward == that row run alone (src/ops/invariant.rs:88-116)."""
    s, ws, model = tiny
    toks = np.random.default_rng(1).integers(0, s.cfg["vocab_size"], 9).astype(np.uint32)
    a, b = model.make_cache(32, 4), model.make_cache(32, 4)
    whole = np.concatenate([model.forward(a, toks[:4]), model.forward(a, toks[4:9])])
    single = np.concatenate([model.forward(b, toks[i:i + 1]) for i in range(9)])
    assert np.array_equal(whole, single)
    a.close(); b.close()


def test_mtp_head_forward_bit_exact(orn, ctx, tiny):
    s, ws, model = tiny
    # the head's dense-expert MoE block as two fused expert launches (fuse_moe 1) and as one
    # launch per operator (0): both the oracle's bits
    for fuse in (1, 0):
        orn.set_option("fuse_moe", fuse)
        rng = np.random.default_rng(2)
        head = orn.MtpHead(model, ws, 64)
        orc = synth.OracleRun(s, 64)
        hid = util.bf16_normal(rng, (3, s.cfg["hidden_size"]))
        ids = rng.integers(0, s.cfg["vocab_size"], 3).astype(np.uint32)
        lg, h1 = head.forward(hid[:1], ids[:1])
        w1 = orc.mtp_hidden(hid[:1], ids[:1])
        assert np.array_equal(h1, w1) and np.array_equal(lg, orc.logits(w1)), fuse
        _, h2 = head.forward(hid[1:], ids[1:], want_logits=False)   # two rows at once, cache offset 1
        assert np.array_equal(h2, orc.mtp_hidden(hid[1:], ids[1:])), fuse
        assert head.offset == 3
        head.close(); orc.close()
    orn.set_option("fuse_moe", 1)


def test_frspec_prune_map_and_file_format(orn, ctx, tiny, tmp_path):
    s, ws, model = tiny
    V = s.cfg["vocab_size"]
    ids = synth.zipf_frspec_ids(V, 256, seed=5)
    fr = orn.FrSpec(model, ids=ids)
    head, n = fr.head()
    assert n == 256
    # pruned row == original row, exact (tests/q4k.rs:739-767)
    x = util.bf16_normal(np.random.default_rng(3), (2, s.cfg["hidden_size"]))
    full = model.logits(x)
    dx, dy = ctx.to_device(x), ctx.alloc(2 * 256 * 2)
    lin = orn.Linear(head, [])
    ctx.linear_matmul(lin, dx, 2, dy)
    assert np.array_equal(dy.download(np.uint16, (2, 256)), full[:, ids.astype(np.int64)])
    dx.free(); dy.free(); fr.close()
    # the file format: u32 n, then n x u32 little endian (src/frspec.rs:101-117)
    path = tmp_path / "ids.bin"
    path.write_bytes(struct.pack("<I", len(ids)) + ids.astype("<u4").tobytes())
    fr = orn.FrSpec(model, path=path)
    assert fr.head()[1] == 256
    fr.close()
    # no path at all: the default location (frspec::default_path, src/frspec.rs:153-158)
    os.environ["ORNITH_FRSPEC"] = str(path)
    try:
        fr = orn.FrSpec(model)
        assert fr.head()[1] == 256
        fr.close()
    finally:
        del os.environ["ORNITH_FRSPEC"]
    bad = {
        "empty": struct.pack("<I", 0),
        "too many": struct.pack("<I", V) + np.arange(V, dtype="<u4").tobytes(),
        "out of range": struct.pack("<I", 2) + np.array([1, V], "<u4").tobytes(),
        "listed twice": struct.pack("<I", 3) + np.array([4, 9, 4], "<u4").tobytes(),
        "holds": struct.pack("<I", 5) + np.array([1, 2], "<u4").tobytes(),
    }
    msgs = {"empty": "empty", "too many": "nothing to prune", "out of range": "outside the vocabulary",
            "listed twice": "listed twice", "holds": "says 5 ids"}
    for k, blob in bad.items():
        path.write_bytes(blob)
        with pytest.raises(orn.OrnithError, match=msgs[k]):
            orn.FrSpec(model, path=path)
    with pytest.raises(orn.OrnithError, match="cannot open"):
        orn.FrSpec(model, path=tmp_path / "missing.bin")


def _run_loops(orn, ctx, s, ws, model, max_tokens, depths, fr_n):
    rng = np.random.default_rng(7)
    V = s.cfg["vocab_size"]
    prompt = rng.integers(0, V, 11).astype(np.uint32)
    cap = 11 + max_tokens + 8
    caches = model.make_cache(cap, 4)
    ar = orn.generate_step(model, caches, prompt, max_tokens, prefill_step=4)
    assert len(ar) == max_tokens and caches.offset == 11 + max_tokens
    orc = synth.OracleRun(s, cap)
    assert ar == orc.generate(prompt, max_tokens, prefill_step=4), "AR tokens differ from the oracle"
    orc.close()
    head = orn.MtpHead(model, ws, cap)
    fr_ids = synth.zipf_frspec_ids(V, fr_n, seed=1)
    fr = orn.FrSpec(model, ids=fr_ids)
    fr_host = synth.prune_head(s.lm_head, fr_ids)
    total_acc = 0
    for depth in depths:
        for policy in (orn.HISTORY_CYCLE, orn.HISTORY_COMMITTED):
            for use_fr in (False, True):
                caches.reset()
                toks, st = orn.generate_step_mtp(model, head, fr if use_fr else None, caches, prompt, depth,
                                                 max_tokens, prefill_step=4, policy=policy)
                assert toks == ar, f"depth {depth} policy {policy} frspec {use_fr}: not identical to greedy"
                assert st.accepted <= st.drafted and len(toks) == max_tokens
                assert caches.offset == 11 + max_tokens
                orc = synth.OracleRun(s, cap)
                otoks, ost = orc.mtp_generate(prompt, depth, max_tokens, fr_ids if use_fr else None,
                                              fr_host if use_fr else None, policy=policy, prefill_step=4)
                orc.close()
                assert otoks == ar
                assert (st.cycles, st.drafted, st.accepted) == (ost.cycles, ost.drafted, ost.accepted)
                assert list(st.accepted_by_depth[:depth]) == list(ost.accepted_by[:depth])
                assert list(st.reached_by_depth[:depth]) == list(ost.reached[:depth])
                total_acc += st.accepted
    for o in (fr, head, caches): o.close()
    return total_acc


def test_generation_loops_tiny(orn, ctx, tiny):
    s, ws, model = tiny
    _run_loops(orn, ctx, s, ws, model, max_tokens=12, depths=(1, 3), fr_n=512)


def test_generation_loops_small_vocab_exercise_acceptance(orn, ctx, tiny_small_vocab):
    s, ws, model = tiny_small_vocab
    acc = _run_loops(orn, ctx, s, ws, model, max_tokens=40, depths=(1, 2), fr_n=24)
    assert acc > 0, "no draft was ever accepted: the acceptance path went untested"


def test_forced_drafts_accept_everything(orn, ctx, tiny):
    """The measurement aid: with the run's own output as the forced drafts every draft is
    accepted (depth + 1 tokens a cycle), the output stays the greedy one under both history
    policies, a short list forces only the positions it covers, and clearing it brings the
    head's own drafts back."""
    s, ws, model = tiny
    rng = np.random.default_rng(9)
    prompt = rng.integers(0, s.cfg["vocab_size"], 9).astype(np.uint32)
    n = 25
    cap = 9 + n + 8
    caches = model.make_cache(cap, 4)
    ar = orn.generate_step(model, caches, prompt, n, prefill_step=4)
    head = orn.MtpHead(model, ws, cap)
    caches.reset()
    base, base_st = orn.generate_step_mtp(model, head, None, caches, prompt, 2, n, prefill_step=4)
    assert base == ar
    head.force_drafts(ar)
    for depth in (1, 2, 3):
        for policy in (orn.HISTORY_CYCLE, orn.HISTORY_COMMITTED):
            caches.reset()
            toks, st = orn.generate_step_mtp(model, head, None, caches, prompt, depth, n, prefill_step=4,
                                             policy=policy)
            assert toks == ar and caches.offset == 9 + n
            assert st.accepted == st.drafted, (depth, policy, st.accepted, st.drafted)
            emitted = cycles = drafted = 0
            while emitted < n:   # every cycle yields its drafts and one more token
                want = min(depth, n - (emitted + 1))
                cycles, drafted, emitted = cycles + (want > 0), drafted + want, emitted + want + 1
            assert (st.cycles, st.drafted) == (cycles, drafted)
    # a list that ends early: positions past it fall back to the head
    head.force_drafts(ar[:7])
    caches.reset()
    toks, st = orn.generate_step_mtp(model, head, None, caches, prompt, 2, n, prefill_step=4)
    assert toks == ar and 4 <= st.accepted < st.drafted
    head.force_drafts([])
    caches.reset()
    toks, st = orn.generate_step_mtp(model, head, None, caches, prompt, 2, n, prefill_step=4)
    assert toks == ar and (st.cycles, st.drafted, st.accepted) == (base_st.cycles, base_st.drafted, base_st.accepted)
    head.close(); caches.close()


def test_stop_callback_and_errors(orn, ctx, tiny):
    s, ws, model = tiny
    prompt = np.arange(5, dtype=np.uint32)
    caches = model.make_cache(32, 2)
    seen = []
    orn.generate_step(model, caches, prompt, 10, on_token=lambda t: (seen.append(t), len(seen) < 3)[1])
    assert len(seen) == 3 and caches.offset == 5 + 3   # the stopping token is in the caches too
    head = orn.MtpHead(model, ws, 32)
    caches.reset()
    caches.set_growable(False)      # fixed capacity: what cannot fit is refused
    with pytest.raises(orn.OrnithError, match="capture window"):
        orn.generate_step_mtp(model, head, None, caches, prompt, 3, 5)
    with pytest.raises(orn.OrnithError, match="exceed cache capacity"):
        model.forward(caches, np.zeros(16, np.uint32)); model.forward(caches, np.zeros(16, np.uint32)); model.forward(caches, np.zeros(1, np.uint32))
    # a run that cannot fit is refused before any token is handed out, and leaves defined stats
    seen.clear()
    with pytest.raises(orn.OrnithError, match="exceed cache capacity"):
        orn.generate_step(model, caches, prompt, 2, on_token=lambda t: (seen.append(t), True)[1])
    caches.reset()
    with pytest.raises(orn.OrnithError, match="exceed cache capacity"):
        orn.generate_step_mtp(model, head, None, caches, prompt, 1, 27, on_token=lambda t: (seen.append(t), True)[1])
    small_head = orn.MtpHead(model, ws, 4)
    small_head.set_growable(False)
    with pytest.raises(orn.OrnithError, match="head's cache"):
        orn.generate_step_mtp(model, small_head, None, caches, prompt, 1, 10, on_token=lambda t: (seen.append(t), True)[1])
    toks, _ = orn.generate_step_mtp(model, small_head, None, caches, prompt, 1, 10, policy=orn.HISTORY_CYCLE)
    assert len(toks) == 10 and not seen
    small_head.close()
    caches.reset()
    with pytest.raises(orn.OrnithError, match="sampler kind"):
        orn.generate_step(model, caches, prompt, 2, sampler=orn.Sampler(7, 0.8, 0.95, 0, 1))
    with pytest.raises(orn.OrnithError, match="temp"):
        orn.generate_step(model, caches, prompt, 2, sampler=orn.Sampler(1, 0.0, 0.95, 0, 1))
    head.close(); caches.close()


def test_caches_grow_like_the_reference_and_change_nothing(orn, ctx, tiny):
    """KvCache::update_and_fetch grows its tensors when a step does not fit
    (/root/reference/src/model/cache.rs:38-79). Caches that start at 8 rows and grow under both
    loops give the tokens, the counts and the hidden rows of caches that were large from the
    start; the capacity moves in multiples of 256 rows; reserve() grows ahead of time."""
    s, ws, model = tiny
    rng = np.random.default_rng(17)
    prompt = rng.integers(0, s.cfg["vocab_size"], 300).astype(np.uint32)   # past one 256-row step in the prefill
    n = 40
    big, small = model.make_cache(1024, 3), model.make_cache(8, 3)
    hb, hs = orn.MtpHead(model, ws, 1024), orn.MtpHead(model, ws, 2)
    try:
        want = orn.generate_step(model, big, prompt, n, prefill_step=16)
        got = orn.generate_step(model, small, prompt, n, prefill_step=16)
        assert got == want and small.offset == big.offset == 300 + n
        assert small.capacity % 256 == 0 and 300 + n <= small.capacity < 1024
        # the rows a grown cache holds are the rows a large one holds: continue from both
        nxt = rng.integers(0, s.cfg["vocab_size"], 5).astype(np.uint32)
        assert np.array_equal(model.forward(small, nxt), model.forward(big, nxt))
        big.reset(); small.close()
        small = model.make_cache(8, 3)
        wt, wst = orn.generate_step_mtp(model, hb, None, big, prompt, 2, n, prefill_step=16, policy=orn.HISTORY_COMMITTED)
        gt, gst = orn.generate_step_mtp(model, hs, None, small, prompt, 2, n, prefill_step=16, policy=orn.HISTORY_COMMITTED)
        assert gt == wt == want
        assert (gst.cycles, gst.drafted, gst.accepted) == (wst.cycles, wst.drafted, wst.accepted)
        assert hs.offset == hb.offset
        small.reserve(5000)
        assert small.capacity >= 5000 and small.capacity % 256 == 0 and small.offset == 300 + n
        assert np.array_equal(model.forward(small, nxt), model.forward(big, nxt))
    finally:
        for o in (hb, hs, big, small): o.close()


@pytest.mark.parametrize("temp,top_p,top_k", [(0.8, 0.95, 0), (0.6, 0.95, 20), (1.0, 1.0, 0)])
def test_sampled_loops_match_oracle(orn, ctx, tiny_small_vocab, temp, top_p, top_k):
    """Sampled decode (temperature / top-p / top-k, seeded threefry keys): the AR loop and
    the depth-1..3 MTP loop draw the same tokens, accept the same drafts and leave the caches
    at the same length as the oracle. Rows are sampled one by one, only as far as the accept
    loop asks, so the key sequence is part of what is compared."""
    s, ws, model = tiny_small_vocab
    V = s.cfg["vocab_size"]
    rng = np.random.default_rng(3)
    prompt = rng.integers(0, V, 9).astype(np.uint32)
    n_tok, cap = 24, 9 + 24 + 8
    smp = orn.Sampler(1, temp, top_p, top_k, 4242)
    caches = model.make_cache(cap, 4)
    head = orn.MtpHead(model, ws, cap)
    orc = synth.OracleRun(s, cap)
    try:
        orc.set_sampler(1, temp, top_p, top_k, 4242)
        got = orn.generate_step(model, caches, prompt, n_tok, sampler=smp, prefill_step=4)
        want = orc.generate(prompt, n_tok, prefill_step=4)
        assert got == want
        greedy = orn.generate_step(model, model.make_cache(cap, 4), prompt, n_tok, prefill_step=4)
        assert got != greedy, "the sampled run never left the greedy path: nothing was tested"
        for depth in (1, 3):
            caches.reset()
            toks, st = orn.generate_step_mtp(model, head, None, caches, prompt, depth, n_tok, sampler=smp,
                                             prefill_step=4, policy=orn.HISTORY_COMMITTED)
            o2 = synth.OracleRun(s, cap)
            otoks, ost = o2.mtp_generate(prompt, depth, n_tok, policy=1, prefill_step=4)
            o2.close()
            assert toks == otoks, depth
            assert (st.cycles, st.drafted, st.accepted) == (ost.cycles, ost.drafted, ost.accepted)
            assert caches.offset == 9 + n_tok
    finally:
        orc.set_sampler(0)
        orc.close(); head.close(); caches.close()
