"""Pins for the oracle's model-level code (CPU only), through properties the reference
itself tests: capture + rewind leaves the caches as a forward over the kept tokens would
(tests/mtp.rs:177-234), rows are independent of how they are batched
(tests/batch_invariance.rs:85-151), and greedy speculative output equals plain greedy
for every depth, policy and draft vocabulary (tests/mtp.rs:246-349)."""
import numpy as np

import synth


def test_oracle_capture_rewind_and_batch_invariance():
    s = synth.SynthModel(synth.TINY, seed=3, with_mtp=False)
    toks = np.random.default_rng(0).integers(0, 2048, 10).astype(np.uint32)
    a, b = synth.OracleRun(s, 32), synth.OracleRun(s, 32)
    ha = np.concatenate([a.forward(toks[:4]), a.forward(toks[4:7], capture=True)])
    hb = np.concatenate([b.forward(toks[i:i + 1]) for i in range(7)])
    assert np.array_equal(ha, hb)
    a.rewind(2)  # keep toks[4], toks[5]
    c = synth.OracleRun(s, 32)
    c.forward(toks[:6])
    assert np.array_equal(a.forward(toks[7:9]), c.forward(toks[7:9]))
    for r in (a, b, c): r.close()


def test_oracle_speculative_equals_greedy():
    s = synth.SynthModel(dict(synth.TINY, vocab_size=32), seed=12)
    prompt = np.random.default_rng(7).integers(0, 32, 11).astype(np.uint32)
    r = synth.OracleRun(s, 64)
    ar = r.generate(prompt, 24, prefill_step=4)
    r.close()
    fr_ids = synth.zipf_frspec_ids(32, 24, seed=1)
    fr_host = synth.prune_head(s.lm_head, fr_ids)
    accepted = 0
    for depth in (1, 2, 3):
        for policy in (0, 1):
            for use_fr in (False, True):
                r = synth.OracleRun(s, 64)
                toks, st = r.mtp_generate(prompt, depth, 24, fr_ids if use_fr else None, fr_host if use_fr else None,
                                          policy=policy, prefill_step=4)
                r.close()
                assert toks == ar, (depth, policy, use_fr)
                assert st.accepted <= st.drafted
                accepted += st.accepted
    assert accepted > 0


def _scripted_counts(ar, drafts, depth, n):
    """What the accept loop must report when the drafts are scripted and the targets are the
    greedy tokens `ar`: a plain walk over two token lists (src/mtp_generate.rs:205-315)."""
    emitted = cycles = drafted = accepted = 0
    reached, acc_by = [0] * 8, [0] * 8
    while emitted < n:
        want = min(depth, n - (emitted + 1))
        cycles += want > 0
        drafted += want
        k = 0
        while k < want:
            reached[k] += 1
            if drafts[emitted + 1 + k] != ar[emitted + 1 + k]:
                break
            acc_by[k] += 1
            accepted += 1
            k += 1
        emitted += k + 1
    return cycles, drafted, accepted, reached, acc_by


def test_oracle_scripted_drafts_give_closed_form_counts():
    """With the drafts scripted, cycles / drafted / accepted / reached-by-depth are a closed
    form of the script: every draft right -> depth + 1 tokens a cycle; a wrong draft at every
    third position -> the walk above. Output stays the greedy one throughout."""
    V = 32
    s = synth.SynthModel(dict(synth.TINY, vocab_size=V), seed=12)
    prompt = np.random.default_rng(7).integers(0, V, 11).astype(np.uint32)
    n = 22
    r = synth.OracleRun(s, 64)
    ar = r.generate(prompt, n, prefill_step=4)
    r.close()
    wrong = [(t + 1) % V if i % 3 == 2 else t for i, t in enumerate(ar)]
    try:
        for script in (ar, wrong, ar[:7]):
            for depth in (1, 2, 3):
                for policy in (0, 1):
                    r = synth.OracleRun(s, 64)
                    r.force_drafts(script)
                    toks, st = r.mtp_generate(prompt, depth, n, policy=policy, prefill_step=4)
                    r.close()
                    assert toks == ar
                    if len(script) < n:
                        continue      # past the script the head drafts by itself: no closed form
                    cyc, dr, acc, reached, acc_by = _scripted_counts(ar, script, depth, n)
                    assert (st.cycles, st.drafted, st.accepted) == (cyc, dr, acc), (depth, policy)
                    assert list(st.reached) == reached and list(st.accepted_by) == acc_by
                    if script is ar:
                        assert st.accepted == st.drafted     # every draft right: depth + 1 tokens a cycle
    finally:
        util_o = synth.util.oracle()
        util_o.orc_mtp_force_drafts(None, 0)
