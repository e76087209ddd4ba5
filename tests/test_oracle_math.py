"""Pins for the oracle's deterministic scalar functions against libm in double."""
import ctypes as C

import numpy as np

import util
from util import oracle, p


def _ulp_err(got, want64):
    got = got.astype(np.float64)
    ulp = np.spacing(np.abs(want64).astype(np.float32)).astype(np.float64)
    return np.abs(got - want64) / ulp


def _apply(fn, x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    fn(p(x), p(out), C.c_int64(x.size))
    return out


def test_expf_within_2ulp_and_limits():
    o = oracle()
    x = np.concatenate([np.linspace(-87, 88, 400001), np.random.default_rng(0).normal(0, 8, 200000)]).astype(np.float32)
    x = x[(x >= -87) & (x <= 88)]
    got = _apply(o.orc_expf_n, x)
    assert _ulp_err(got, np.exp(x.astype(np.float64))).max() <= 2.0
    edge = _apply(o.orc_expf_n, np.array([0.0, -100.0, 100.0, -87.5, 88.5], np.float32))
    assert edge[0] == 1.0 and edge[1] == 0.0 and np.isinf(edge[2]) and edge[3] == 0.0 and np.isinf(edge[4])


def test_logf_and_log1pf_within_2ulp():
    o = oracle()
    rng = np.random.default_rng(1)
    x = np.exp(rng.uniform(-80, 80, 400000)).astype(np.float32)
    got = _apply(o.orc_logf_n, x)
    assert _ulp_err(got, np.log(x.astype(np.float64))).max() <= 2.0
    assert _apply(o.orc_logf_n, np.array([1.0], np.float32))[0] == 0.0
    u = np.exp(rng.uniform(-40, 3, 400000)).astype(np.float32)
    got = _apply(o.orc_log1pf_n, u)
    assert _ulp_err(got, np.log1p(u.astype(np.float64))).max() <= 3.0


def test_bf16_rne_and_f16_conversions():
    o = oracle()
    # bf16: exhaustive over the upper 16 bits is the identity; ties go to even
    bits = np.arange(65536, dtype=np.uint32)
    f = (bits << 16).view(np.float32)
    got = util.orc_f32_to_bf16(f)
    nan = np.isnan(f)
    assert np.array_equal(got[~nan], bits[~nan].astype(np.uint16))
    tie = np.array([0x3F808000, 0x3F818000, 0x3F808001, 0x3F807FFF], np.uint32).view(np.float32)
    assert list(util.orc_f32_to_bf16(tie)) == [0x3F80, 0x3F82, 0x3F81, 0x3F80]
    # the numpy conversion the tests build their inputs with is the same function, bit for bit,
    # NaN and infinities included
    rnd = np.random.default_rng(0).integers(0, 2 ** 32, 2_000_000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    for v in (f, tie, rnd):
        assert np.array_equal(util.f32_to_bf16(v), util.orc_f32_to_bf16(v))
    # f16 -> f32 exhaustive vs numpy; f32 -> f16 on random values vs numpy (RNE)
    h = np.arange(65536, dtype=np.uint16)
    out = np.empty(65536, np.float32)
    o.orc_f16_to_f32_n(p(h), p(out), C.c_int64(65536))
    want = h.view(np.float16).astype(np.float32)
    ok = ~np.isnan(want)
    assert np.array_equal(out[ok], want[ok])
    x = np.random.default_rng(2).normal(0, 1, 100000).astype(np.float32) * np.float32(10.0) ** np.random.default_rng(3).integers(-9, 5, 100000).astype(np.float32)
    back = np.empty(x.size, np.uint16)
    o.orc_f32_to_f16_n(p(x), p(back), C.c_int64(x.size))
    assert np.array_equal(back, x.astype(np.float16).view(np.uint16))


def test_sigmoid_bf16_all_inputs_within_1ulp_of_double():
    """Exhaustive over bf16 (the reference does the same against mlx, tests/activations.rs)."""
    o = oracle()
    bits = np.arange(65536, dtype=np.uint16)
    x = util.bf16_to_f32(bits)
    fin = np.isfinite(x)
    out = np.empty(65536, np.uint16)
    o.orc_sigmoid_bf16_n(p(bits), p(out), C.c_int64(65536))
    got = util.bf16_to_f32(out)[fin].astype(np.float64)
    xd = x[fin].astype(np.float64)
    want = np.where(xd >= 0, 1 / (1 + np.exp(-np.abs(xd))), np.exp(-np.abs(xd)) / (1 + np.exp(-np.abs(xd))))
    # three bf16 roundings on the way: 3 bf16 ulps of the result for x < 0 (plus the
    # flush of results below exp(-87)); for x >= 0 the subtraction 1 - y lands in
    # [0.5, 1] where a bf16 ulp is 2^-8 (y itself carries up to 1.5 ulps of [0.25, 0.5))
    ulp_bf16 = np.spacing(want.astype(np.float32)).astype(np.float64) * 65536
    tol = np.where(xd < 0, 3 * ulp_bf16 + 2e-38, 1.5 * 2.0 ** -8)
    assert np.all(np.abs(got - want) <= tol)
    assert np.all((got >= 0) & (got <= 1))


def test_tree64_is_butterfly_order():
    o = oracle()
    rng = np.random.default_rng(5)
    v = (rng.standard_normal(64) * 10.0 ** rng.integers(-3, 4, 64)).astype(np.float32)
    w = v.copy()
    for s in (32, 16, 8, 4, 2, 1):
        w = (w + w[np.arange(64) ^ s]).astype(np.float32)
    assert np.all(w == w[0])
    assert o.orc_tree64_export(p(v)) == w[0]
    # narrower rows: upper lanes zero => same as a tree over the low lanes only
    for width in (8, 16, 32):
        z = np.zeros(64, np.float32)
        z[:width] = v[:width]
        t = z[:width].copy()
        s = width // 2
        while s >= 1:
            t = (t + t[np.arange(width) ^ s]).astype(np.float32)
            s //= 2
        assert o.orc_tree64_export(p(z)) == t[0]
