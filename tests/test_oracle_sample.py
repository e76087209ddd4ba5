"""Pins for the oracle's greedy selection (CPU only)."""
import ctypes as C

import numpy as np

import util
from util import oracle, p


def test_logsumexp_vs_double_and_argmax_rules():
    rng = np.random.default_rng(0)
    o = oracle()
    o.orc_logsumexp_bf16.restype = C.c_float
    for V in (1000, 1024, 5000, 248320):
        x = util.bf16_normal(rng, (V,), 3.0)
        got = o.orc_logsumexp_bf16(p(x), V)
        xd = util.bf16_to_f32(x).astype(np.float64)
        want = np.log(np.exp(xd - xd.max()).sum()) + xd.max()
        assert abs(got - want) <= 2.0 ** -8 * abs(want) + 1e-6
    # lowest index wins ties, both for raw logits and after the bf16 subtraction merges values
    x = util.f32_to_bf16(np.array([[1.0, 5.0, 5.0, 2.0], [3.0, 3.0, 3.0, 3.0]], np.float32))
    out = np.empty(2, np.uint32)
    o.orc_argmax_rows(p(x), 2, 4, p(out))
    assert list(out) == [1, 0]
    # 100 and 100.5 are distinct bf16 values, but (x - lse) rounds both to the same bf16
    x = util.f32_to_bf16(np.array([[100.0, 100.5] + [0.0] * 62], np.float32))
    xf = util.bf16_to_f32(x)
    assert xf[0, 0] != xf[0, 1]
    tok = np.empty(1, np.uint32); lse = np.empty(1, np.uint16)
    o.orc_greedy_rows(p(x), 1, 64, p(tok), p(lse))
    l = util.bf16_to_f32(lse)[0]
    lp = util.bf16_to_f32(util.f32_to_bf16((xf[0] - l).astype(np.float32)))
    assert tok[0] == int(np.flatnonzero(lp == lp.max())[0])
    raw = np.empty(1, np.uint32)
    o.orc_argmax_rows(p(x), 1, 64, p(raw))
    assert raw[0] == 1
