"""Pins for the oracle's attention pieces (CPU only)."""
import numpy as np

import util


def test_rope_table_and_offset_zero_identity():
    c, s = util.orc_rope_table(8, 64, 1e7)
    assert np.all(c[0] == 1.0) and np.all(s[0] == 0.0)
    i = np.arange(32)
    ang = 5 * (1e7 ** (-i / 32.0))
    assert np.allclose(c[5], np.cos(ang), atol=1e-7) and np.allclose(s[5], np.sin(ang), atol=1e-7)


def _mk(rng, T, Hq, Hkv, hd, cap, offset):
    qg = util.bf16_normal(rng, (T, Hq, 2 * hd)); kx = util.bf16_normal(rng, (T, Hkv, hd)); vx = util.bf16_normal(rng, (T, Hkv, hd))
    qw = util.bf16_normal(rng, (hd,)); kw = util.bf16_normal(rng, (hd,))
    kc = np.zeros((Hkv, cap, hd), np.uint16); vc = np.zeros((Hkv, cap, hd), np.uint16)
    kc[:, :offset] = util.bf16_normal(rng, (Hkv, offset, hd)); vc[:, :offset] = util.bf16_normal(rng, (Hkv, offset, hd))
    return qg, kx, vx, qw, kw, kc, vc


def test_prep_and_sdpa_vs_double():
    rng = np.random.default_rng(0)
    T, Hq, Hkv, hd, cap, offset = 3, 4, 2, 256, 1024, 300
    qg, kx, vx, qw, kw, kc, vc = _mk(rng, T, Hq, Hkv, hd, cap, offset)
    c, s = util.orc_rope_table(cap, 64, 1e7)
    q_rot, gate = util.orc_attn_prep(qg, kx, vx, qw, kw, 64, c, s, offset, kc, vc)
    f = lambda a: util.bf16_to_f32(a).astype(np.float64)

    def ref_head(x, w, pos):
        x = f(x); n = f(w) * x / np.sqrt((x ** 2).mean() + 1e-6)
        o = n.copy()
        o[:32] = n[:32] * c[pos] - n[32:64] * s[pos]
        o[32:64] = n[:32] * s[pos] + n[32:64] * c[pos]
        return o

    for t in range(T):
        for h in range(Hq):
            want = ref_head(qg[t, h, :hd], qw, offset + t)
            assert np.all(np.abs(f(q_rot[t, h]) - want) <= 0.02 * np.abs(want) + 0.02)
        for h in range(Hkv):
            want = ref_head(kx[t, h], kw, offset + t)
            assert np.all(np.abs(f(kc[h, offset + t]) - want) <= 0.02 * np.abs(want) + 0.02)
            assert np.array_equal(vc[h, offset + t], vx[t, h])
    assert np.array_equal(gate, qg[:, :, hd:])
    out = util.orc_sdpa(q_rot, kc, vc, gate, offset, hd ** -0.5)
    for t in range(T):
        n = offset + t + 1
        for h in range(Hq):
            hk = h // (Hq // Hkv)
            sc = (f(kc[hk, :n]) @ f(q_rot[t, h])) * hd ** -0.5
            pr = np.exp(sc - sc.max()); pr /= pr.sum()
            att = pr @ f(vc[hk, :n])
            want = att / (1 + np.exp(-f(gate[t, h])))
            got = f(out[t].reshape(Hq, hd)[h])
            assert np.all(np.abs(got - want) <= 0.03 * np.abs(want) + 0.01 * np.max(np.abs(want)))


def test_causal_row_equals_single_row_call():
    """Row r of a T-row call == a 1-row call at that position (truncated cache), bit for bit."""
    rng = np.random.default_rng(1)
    T, Hq, Hkv, hd, cap, offset = 4, 4, 1, 256, 1024, 509  # crosses a 256-key block boundary
    qg, kx, vx, qw, kw, kc, vc = _mk(rng, T, Hq, Hkv, hd, cap, offset)
    c, s = util.orc_rope_table(cap, 64, 1e7)
    kc1, vc1 = kc.copy(), vc.copy()
    q_rot, gate = util.orc_attn_prep(qg, kx, vx, qw, kw, 64, c, s, offset, kc, vc)
    out = util.orc_sdpa(q_rot, kc, vc, gate, offset, hd ** -0.5)
    for t in range(T):
        q1, g1 = util.orc_attn_prep(qg[t:t + 1], kx[t:t + 1], vx[t:t + 1], qw, kw, 64, c, s, offset + t, kc1, vc1)
        o1 = util.orc_sdpa(q1, kc1, vc1, g1, offset + t, hd ** -0.5)
        assert np.array_equal(o1[0], out[t]), t
    assert np.array_equal(kc1, kc)
