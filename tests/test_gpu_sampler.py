"""GPU: the sampled-token path bit for bit against the oracle: stable argsort, cumulative
sums (bf16 and fp32), top-p, top-k, the inverse-CDF draw, and whole TopSampler sequences
(the reference checks the same stages against mlx dumps, tests/sampler.rs:29-170)."""
import importlib

import numpy as np
import pytest

import util

pytestmark = pytest.mark.gpu

V_FULL = 248320


def _logits(rng, V, spread):
    return util.f32_to_bf16((rng.standard_normal(V) * spread).astype(np.float32))


@pytest.mark.parametrize("n", [1, 63, 1024, 1025, 5000, V_FULL])
def test_argsort_stable_bit_exact(orn, ctx, n):
    rng = np.random.default_rng(n)
    xb = _logits(rng, n, 2.0)
    if n > 100:     # ties, zeros of both signs, infinities
        xb[rng.integers(0, n, n // 3)] = util.f32_to_bf16(np.array([-2.5], np.float32))[0]
        xb[rng.integers(0, n, 5)] = [0x0000, 0x8000, 0x7F80, 0xFF80, 0x8000]
    dx, di = ctx.to_device(xb), ctx.alloc(n * 4)
    for neg in (False, True):
        orn.argsort_bf16(ctx, dx, n, neg, di)
        assert np.array_equal(di.download(np.uint32, (n,)), util.orc_argsort_bf16(xb, neg)), (n, neg)
    dx.free(); di.free()


@pytest.mark.parametrize("n", [1, 64, 65, 1024, 1025, 40000, V_FULL])
def test_cumsum_bit_exact(orn, ctx, n):
    rng = np.random.default_rng(n + 7)
    x = (rng.random(n) * np.exp(rng.normal(0, 3, n))).astype(np.float32)
    dx, do = ctx.to_device(x), ctx.alloc(n * 4)
    orn.cumsum(ctx, dx, orn.F32, n, do)
    want, _ = util.orc_cumsum_f32(x)
    assert np.array_equal(do.download(np.float32, (n,)).view(np.uint32), want.view(np.uint32))
    xb = util.f32_to_bf16(x * 1e-3)
    dxb, dob = ctx.to_device(xb), ctx.alloc(n * 2)
    orn.cumsum(ctx, dxb, orn.BF16, n, dob)
    assert np.array_equal(dob.download(np.uint16, (n,)), util.orc_cumsum_bf16(xb))
    for b in (dx, do, dxb, dob): b.free()


@pytest.mark.parametrize("V,spread", [(300, 2.0), (5000, 3.0), (V_FULL, 1.0), (V_FULL, 4.0)])
def test_top_p_top_k_and_draw_bit_exact(orn, ctx, V, spread):
    rng = np.random.default_rng(V + int(spread))
    lp = util.orc_logprobs_row(_logits(rng, V, spread))
    dlp, dout, dout2, dtok = ctx.to_device(lp), ctx.alloc(V * 2), ctx.alloc(V * 2), ctx.alloc(4)
    for top_p in (0.95, 0.5):
        orn.apply_top_p(ctx, dlp, V, top_p, dout)
        want_p = util.orc_apply_top_p(lp, top_p)
        assert np.array_equal(dout.download(np.uint16, (V,)), want_p), top_p
    for k in (1, 20, 257):
        orn.apply_top_k(ctx, dlp, V, k, dout)
        assert np.array_equal(dout.download(np.uint16, (V,)), util.orc_apply_top_k(lp, k)), k
    # top-k over what top-p left, then draws with many raw words (including the extremes)
    orn.apply_top_p(ctx, dlp, V, 0.95, dout)
    orn.apply_top_k(ctx, dout, V, 20, dout2)
    a = util.orc_apply_top_k(util.orc_apply_top_p(lp, 0.95), 20)
    assert np.array_equal(dout2.download(np.uint16, (V,)), a)
    raws = [0, 1, 0xFFFFFFFF, 0x80000000] + [int(v) for v in rng.integers(0, 2 ** 32, 12)]
    for src, host in ((dout2, a), (dlp, lp)):     # after the filters, and temperature only
        for raw in raws[: (16 if V < 10000 else 6)]:
            orn.categorical(ctx, src, V, 0.8, raw, dtok)
            assert int(dtok.download(np.uint32, (1,))[0]) == util.orc_categorical(host, 0.8, raw), raw
    for b in (dlp, dout, dout2, dtok): b.free()


def test_degenerate_rows(orn, ctx):
    V = 2000
    dtok, dout = ctx.alloc(4), ctx.alloc(V * 2)
    # one finite entry: always drawn; constant row: top-k keeps the lowest ids
    one = np.full(V, 0xFF80, np.uint16); one[1234] = util.f32_to_bf16(np.array([-0.5], np.float32))[0]
    d1 = ctx.to_device(one)
    orn.categorical(ctx, d1, V, 1.0, 987654321, dtok)
    assert int(dtok.download(np.uint32, (1,))[0]) == 1234 == util.orc_categorical(one, 1.0, 987654321)
    const = np.full(V, util.f32_to_bf16(np.array([-7.625], np.float32))[0], np.uint16)
    dc = ctx.to_device(const)
    orn.apply_top_k(ctx, dc, V, 9, dout)
    got = dout.download(np.uint16, (V,))
    assert np.array_equal(np.nonzero(got != 0xFF80)[0], np.arange(9))
    orn.apply_top_p(ctx, dc, V, 0.9, dout)
    assert np.array_equal(dout.download(np.uint16, (V,)), util.orc_apply_top_p(const, 0.9))
    with pytest.raises(orn.OrnithError):
        orn.apply_top_k(ctx, dc, V, V, dout)          # the reference asserts 0 < top_k < n
    for b in (dtok, dout, d1, dc): b.free()


@pytest.mark.parametrize("V,temp,top_p,top_k", [(3000, 0.6, 0.95, 20), (V_FULL, 0.8, 0.95, 0), (V_FULL, 0.6, 0.95, 20),
                                                 (5000, 1.0, 1.0, 0), (5000, 0.7, 0.0, 5)])
def test_top_sampler_sequences_match_oracle(orn, ctx, V, temp, top_p, top_k):
    rng = np.random.default_rng(V + top_k)
    s = orn.TopSampler(ctx, temp, top_p, top_k, seed=1234, vocab=V)
    key = orn.random_key(1234)
    for step in range(4 if V > 10000 else 10):
        logits = _logits(rng, V, 3.0)
        dl = ctx.to_device(logits)
        got = s.sample(dl)
        want, key = util.orc_top_sample(logits, temp, top_p, top_k, key)
        assert got == want, step
        dl.free()
    s.close()
