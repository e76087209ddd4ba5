"""Pins for the oracle's norms and gated-delta pieces (CPU only), each against an
independent float64 statement or a closed form."""
import numpy as np

import util


def test_rms_variants_vs_double_and_fused_add_equals_unfused():
    rng = np.random.default_rng(0)
    for n in (128, 256, 2048):
        x = util.bf16_normal(rng, (3, n), 2.0)
        w = util.bf16_normal(rng, (n,), 1.0)
        xd = util.bf16_to_f32(x).astype(np.float64)
        want = util.bf16_to_f32(w) * (xd / np.sqrt((xd ** 2).mean(1, keepdims=True) + 1e-6))
        got = util.bf16_to_f32(util.orc_rms_norm(x, w)).astype(np.float64)
        assert np.all(np.abs(got - want) <= 2.0 ** -7 * np.abs(want) + 1e-30)
        # weightless == weight of ones (1*x is exact)
        ones = util.f32_to_bf16(np.ones(n, np.float32))
        assert np.array_equal(util.orc_rms_norm(x, None), util.orc_rms_norm(x, ones))
        b = util.bf16_normal(rng, (3, n), 1.0)
        h, out = util.orc_add_rms_norm(x, b, w)
        h2 = util.f32_to_bf16(util.bf16_to_f32(x) + util.bf16_to_f32(b))
        assert np.array_equal(h, h2) and np.array_equal(out, util.orc_rms_norm(h2, w))
    y = util.bf16_normal(rng, (5, 128)); z = util.bf16_normal(rng, (5, 128), 2.0); w = util.bf16_normal(rng, (128,))
    got = util.bf16_to_f32(util.orc_rms_norm_gated(y, w, z)).astype(np.float64)
    yd, zd = util.bf16_to_f32(y).astype(np.float64), util.bf16_to_f32(z).astype(np.float64)
    want = zd / (1 + np.exp(-zd)) * util.bf16_to_f32(w) * yd / np.sqrt((yd ** 2).mean(1, keepdims=True) + 1e-6)
    assert np.all(np.abs(got - want) <= 3 * 2.0 ** -8 * np.abs(want) + 1e-30)


def _front_inputs(rng, T, Hk, Hv):
    D = 2 * Hk * 128 + Hv * 128
    return dict(conv_state=util.bf16_normal(rng, (3, D)), qkv=util.bf16_normal(rng, (T, D)),
                cw=util.bf16_normal(rng, (D, 4), 0.5), a=util.bf16_normal(rng, (T, Hv)),
                b=util.bf16_normal(rng, (T, Hv)), a_log=util.bf16_normal(rng, (Hv,), 0.5),
                dt_bias=util.bf16_normal(rng, (Hv,), 0.5))


def test_gdn_front_vs_double_composition():
    rng = np.random.default_rng(1)
    T, Hk, Hv = 3, 2, 4
    i = _front_inputs(rng, T, Hk, Hv)
    q, k, v, beta, g, ci = util.orc_gdn_front(i["conv_state"], i["qkv"], i["cw"], i["a"], i["b"], i["a_log"], i["dt_bias"], Hk, Hv)
    f = lambda a: util.bf16_to_f32(a).astype(np.float64)
    cat = np.concatenate([f(i["conv_state"]), f(i["qkv"])])
    assert np.array_equal(ci, np.concatenate([i["conv_state"], i["qkv"]]))
    conv = np.stack([(cat[t:t + 4] * f(i["cw"]).T).sum(0) for t in range(T)])  # taps ascending, causal
    s = conv / (1 + np.exp(-conv))
    kd = Hk * 128
    qd = s[:, :kd].reshape(T, Hk, 128); kk = s[:, kd:2 * kd].reshape(T, Hk, 128)
    nrm = lambda a: a / np.sqrt((a ** 2).mean(-1, keepdims=True) + 1e-6)
    tol = lambda want: 0.02 * np.abs(want) + 0.02 * np.max(np.abs(want))
    assert np.all(np.abs(f(q) - nrm(qd) / 128) <= tol(nrm(qd) / 128))
    assert np.all(np.abs(f(k) - nrm(kk) / np.sqrt(128)) <= tol(nrm(kk) / np.sqrt(128)))
    assert np.all(np.abs(f(v) - s[:, 2 * kd:].reshape(T, Hv, 128)) <= tol(s[:, 2 * kd:].reshape(T, Hv, 128)))
    assert np.all(np.abs(f(beta) - 1 / (1 + np.exp(-f(i["b"])))) <= 2.0 ** -7)
    sp = np.log1p(np.exp(f(i["a"]) + f(i["dt_bias"])))
    want_g = np.exp(-np.exp(f(i["a_log"])) * sp)
    assert np.all(np.abs(g - want_g) <= 0.02)


def test_recurrence_vs_double_bruteforce_and_special_cases():
    rng = np.random.default_rng(2)
    T, Hk, Hv = 3, 2, 4
    q = util.bf16_normal(rng, (T, Hk, 128), 0.1); k = util.bf16_normal(rng, (T, Hk, 128), 0.1)
    v = util.bf16_normal(rng, (T, Hv, 128)); beta = util.f32_to_bf16(rng.random((T, Hv)).astype(np.float32))
    g = rng.random((T, Hv)).astype(np.float32)
    S0 = (rng.standard_normal((Hv, 128, 128)) * 0.1).astype(np.float32)
    y, snaps = util.orc_gdn_recurrence(q, k, v, g, beta, S0)
    f = lambda a: util.bf16_to_f32(a).astype(np.float64)
    S = S0.astype(np.float64)
    for t in range(T):
        for hv in range(Hv):
            hk = hv // (Hv // Hk)
            S[hv] *= g[t, hv]
            kv = S[hv] @ f(k)[t, hk]
            delta = (f(v)[t, hv] - kv) * f(beta)[t, hv]
            S[hv] += np.outer(delta, f(k)[t, hk])
            want = S[hv] @ f(q)[t, hk]
            assert np.all(np.abs(f(y)[t, hv] - want) <= 2.0 ** -7 * np.abs(want) + 1e-4)
        assert np.allclose(snaps[t], S, rtol=1e-5, atol=1e-6)
    # T-step call == T one-step calls, bit for bit (tests/gdn.rs:113-120, qwen3_5.rs:590-598)
    st = S0
    for t in range(T):
        y1, s1 = util.orc_gdn_recurrence(q[t:t + 1], k[t:t + 1], v[t:t + 1], g[t:t + 1], beta[t:t + 1], st)
        assert np.array_equal(y1[0], y[t]) and np.array_equal(s1[0].view(np.uint32), snaps[t].view(np.uint32))
        st = s1[0]
    # S = 0, g = beta = 1  ->  y = (k.q) v
    one = util.f32_to_bf16(np.ones((1, Hv), np.float32))
    y0, _ = util.orc_gdn_recurrence(q[:1], k[:1], v[:1], np.ones((1, Hv), np.float32), one, np.zeros_like(S0))
    kq = (f(k)[0] * f(q)[0]).sum(-1)
    want = f(v)[0] * np.repeat(kq, Hv // Hk)[:, None]
    assert np.all(np.abs(f(y0)[0] - want) <= 2.0 ** -7 * np.abs(want) + 1e-6)
