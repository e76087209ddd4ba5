"""CPU: the sampled-token oracle against what pins it without the reference's fixtures
(tests/sampler.rs reads refs/, which the repository does not hold): the published
Random123 known-answer vectors for threefry2x32-20, closed forms for key splitting and the
uniform scaling, numpy for the sort / top-k / draw, float64 for the cumulative sums."""
import numpy as np

import util


def test_threefry_known_answers():
    # Random123 kat_vectors, threefry2x32 20 rounds (also the vectors JAX checks its PRNG with)
    assert util.orc_threefry((0, 0), (0, 0)) == (0x6B200159, 0x99BA4EFE)
    assert util.orc_threefry((0xFFFFFFFF, 0xFFFFFFFF), (0xFFFFFFFF, 0xFFFFFFFF)) == (0x1CB996FC, 0xBB002BE7)
    assert util.orc_threefry((0x13198A2E, 0x03707344), (0x243F6A88, 0x85A308D3)) == (0xC4923A9C, 0x483DF7A0)


def test_bits_layout_and_key_split():
    key = (0x01234567, 0x89ABCDEF)
    # n words: word t and word t + ceil(n/2) are the x and y of hash(t, t + ceil(n/2)); odd n drops the last y
    for n in (1, 2, 3, 4, 7, 8):
        got = util.orc_random_bits(key, n)
        gy = (n + 1) // 2
        for t in range(gy):
            last = (n % 2 == 1) and t == n // 2
            x, y = util.orc_threefry(key, (t, 0 if last else t + gy))
            assert got[t] == x
            if not last:
                assert got[t + gy] == y
    # KeySequence::next = split: bits([2,2]); first row is the new state, second the sub key
    b = util.orc_random_bits(key, 4)
    st, sub = util.orc_key_next(key)
    assert st == [b[0], b[1]] and sub == [b[2], b[3]]
    # two sequences from the same seed agree, different seeds differ
    a, _ = util.orc_key_next((0, 7)); c, _ = util.orc_key_next((0, 8))
    assert a != c


def test_uniform_scaling_closed_forms():
    assert util.orc_uniform_scaled(0, 3.0) == 0.0
    assert util.orc_uniform_scaled(1 << 31, 1.0) == np.float32(0.5)
    assert util.orc_uniform_scaled(1 << 30, 8.0) == np.float32(2.0)
    upper = np.array([0x3F7FFFFF], np.uint32).view(np.float32)[0]
    # 2^32 - 1 rounds to 2^32 as a float: the quotient 1.0 is clamped to nextafter(1, 0)
    assert util.orc_uniform_scaled(0xFFFFFFFF, 1.0) == upper
    assert util.orc_uniform_scaled(0xFFFFFFFF, 5.0) < np.float32(5.0)


def test_argsort_is_numpy_stable_argsort():
    rng = np.random.default_rng(0)
    for n in (1, 63, 64, 1000, 1025, 5000):
        # few distinct values -> many ties; both signs, zeros, infinities
        vals = rng.choice(np.array([-np.inf, -3.5, -1.0, -0.0, 0.0, 0.5, 2.0, np.inf], np.float32), n)
        vals = np.where(rng.random(n) < 0.5, vals, rng.standard_normal(n).astype(np.float32))
        xb = util.f32_to_bf16(vals)
        xf = util.bf16_to_f32(xb)
        got = util.orc_argsort_bf16(xb)
        # -0.0 sorts before +0.0 in the key order; numpy treats them equal: compare on a key that separates them
        key = xf.astype(np.float64) - np.where((xb == 0x8000), 1e-300, 0.0)
        want = np.argsort(key, kind="stable")
        assert np.array_equal(got, want.astype(np.uint32)), n
        gotn = util.orc_argsort_bf16(xb, negate=True)
        keyn = (-xf).astype(np.float64) - np.where((xb == 0x0000), 1e-300, 0.0)
        assert np.array_equal(gotn, np.argsort(keyn, kind="stable").astype(np.uint32)), n


def test_cumsum_against_float64():
    rng = np.random.default_rng(1)
    for n in (1, 64, 65, 1024, 1025, 5000):
        x = rng.random(n).astype(np.float32)
        got, total = util.orc_cumsum_f32(x)
        want = np.cumsum(x.astype(np.float64))
        assert np.max(np.abs(got - want) / want) < 2e-6
        assert total == got[-1] or abs(float(total) - want[-1]) / want[-1] < 2e-6
        # exactly representable sums: any association gives the exact integers
        xi = rng.integers(0, 4, n).astype(np.float32)
        g, t = util.orc_cumsum_f32(xi)
        assert np.array_equal(g, np.cumsum(xi)) and t == xi.sum()
    # bf16 accumulation: exact on small integers, within bf16 resolution of float64 otherwise
    xi = util.f32_to_bf16(rng.integers(0, 2, 200).astype(np.float32))
    assert np.array_equal(util.bf16_to_f32(util.orc_cumsum_bf16(xi)), np.cumsum(util.bf16_to_f32(xi)))
    xb = util.f32_to_bf16((rng.random(3000) * 1e-3).astype(np.float32))
    got = util.bf16_to_f32(util.orc_cumsum_bf16(xb)).astype(np.float64)
    want = np.cumsum(util.bf16_to_f32(xb).astype(np.float64))
    assert np.max(np.abs(got - want) / want) < 0.05     # bf16 adds: 2^-9 each, they do not pile up over 3 levels


def _lp(rng, V, spread):
    logits = util.f32_to_bf16((rng.standard_normal(V) * spread).astype(np.float32))
    return logits, util.orc_logprobs_row(logits)


def test_logprobs_normalise():
    rng = np.random.default_rng(2)
    logits, lp = _lp(rng, 5000, 3.0)
    pr = np.exp(util.bf16_to_f32(lp).astype(np.float64))
    assert abs(pr.sum() - 1.0) < 0.02          # bf16 logprobs
    x = util.bf16_to_f32(logits).astype(np.float64)
    ref = x - np.log(np.exp(x - x.max()).sum()) - x.max()
    assert np.max(np.abs(util.bf16_to_f32(lp) - ref)) < 0.1   # half a bf16 step at |lp| < 32 plus the rounded lse


def test_top_k_keeps_exactly_the_k_largest_lowest_index_on_ties():
    rng = np.random.default_rng(3)
    logits, lp = _lp(rng, 4000, 1.0)
    lpf = util.bf16_to_f32(lp)
    for k in (1, 5, 20, 399):
        out = util.orc_apply_top_k(lp, k)
        kept = np.nonzero(out != 0xFF80)[0]
        order = np.lexsort((np.arange(lp.size), -lpf.astype(np.float64)))   # by value desc, then index asc
        assert np.array_equal(np.sort(kept), np.sort(order[:k]))
        assert np.array_equal(out[kept], lp[kept])
    # heavy ties: constant row keeps ids 0..k-1
    const = np.full(100, util.f32_to_bf16(np.float32(-4.5)), np.uint16)
    out = util.orc_apply_top_k(const, 7)
    assert np.array_equal(np.nonzero(out != 0xFF80)[0], np.arange(7))


def test_top_p_drops_a_low_tail_of_at_most_one_minus_p():
    rng = np.random.default_rng(4)
    for spread, top_p in ((3.0, 0.95), (6.0, 0.9), (1.0, 0.5)):
        logits, lp = _lp(rng, 6000, spread)
        out = util.orc_apply_top_p(lp, top_p)
        kept = out != 0xFF80
        assert np.array_equal(out[kept], lp[kept])
        pr = np.exp(util.bf16_to_f32(lp).astype(np.float64))
        pr /= pr.sum()
        # what is dropped is a set of the least likely tokens ...
        assert pr[~kept].max(initial=0.0) <= pr[kept].min() * (1 + 2 ** -7)
        # ... whose mass is about 1 - p (bf16 running sum: a few percent of slack), and the best token stays
        assert pr[~kept].sum() <= (1 - top_p) * 1.08 + 0.01
        assert kept[np.argmax(pr)]
        # maximality: adding the next token would cross the threshold (again up to bf16 slack)
        if (~kept).any() and kept.any():
            nxt = pr[kept].min()
            assert pr[~kept].sum() + nxt >= (1 - top_p) * 0.9 - 0.01


def test_categorical_is_the_inverse_cdf_and_follows_the_distribution():
    rng = np.random.default_rng(5)
    logits, lp = _lp(rng, 300, 2.0)
    lp = util.orc_apply_top_k(lp, 12)
    temp = 0.8
    scale = util.bf16_to_f32(util.f32_to_bf16(np.float32(1 / temp)))
    x = util.bf16_to_f32(util.f32_to_bf16(util.bf16_to_f32(lp) * scale)).astype(np.float64)
    w = np.exp(x - x.max()); w[np.isneginf(x)] = 0
    cdf = np.cumsum(w) / w.sum()
    counts = np.zeros(300)
    for bits in np.linspace(0, 2 ** 32 - 1, 4001).astype(np.uint64):
        tok = util.orc_categorical(lp, temp, int(bits))
        counts[tok] += 1
        u = min(float(np.float32(bits)) / 2 ** 32, 1 - 2 ** -24)
        lo = cdf[tok - 1] if tok > 0 else 0.0
        assert w[tok] > 0 and lo - 1e-5 <= u <= cdf[tok] + 1e-5
    # an evenly spaced sweep of u reproduces the probabilities
    assert np.max(np.abs(counts / counts.sum() - w / w.sum())) < 2e-3
    # a single surviving token is always drawn; -inf everywhere else
    one = np.full(50, 0xFF80, np.uint16); one[17] = util.f32_to_bf16(np.array([-0.25], np.float32))[0]
    assert util.orc_categorical(one, 1.0, 123456789) == 17


def test_top_sample_composes_the_stages_and_advances_the_key():
    rng = np.random.default_rng(6)
    logits, lp = _lp(rng, 3000, 2.5)
    st = [0, 42]
    tok, st2 = util.orc_top_sample(logits, 0.8, 0.95, 20, st)
    a = util.orc_apply_top_k(util.orc_apply_top_p(lp, 0.95), 20)
    st_ref, sub = util.orc_key_next(st)
    raw = util.orc_random_bits(sub, 1)[0]
    assert st2 == st_ref and tok == util.orc_categorical(a, 0.8, int(raw))
    tok_b, _ = util.orc_top_sample(logits, 0.8, 0.95, 20, st)
    assert tok_b == tok                       # same key, same draw
    toks = set()
    s = st
    for _ in range(30):
        t, s = util.orc_top_sample(logits, 0.8, 0.95, 20, s)
        toks.add(t)
    assert len(toks) > 3                      # the sequence moves
