"""GPU parity: attention prep (q/k norm + RoPE + KV append) and split-K decode attention
with the output gate vs the oracle, bit for bit."""
import numpy as np
import pytest

import util

pytestmark = pytest.mark.gpu


def _mk(rng, T, Hq, Hkv, hd, cap, offset):
    qg = util.bf16_normal(rng, (T, Hq, 2 * hd)); kx = util.bf16_normal(rng, (T, Hkv, hd)); vx = util.bf16_normal(rng, (T, Hkv, hd))
    qw = util.bf16_normal(rng, (hd,)); kw = util.bf16_normal(rng, (hd,))
    kc = np.zeros((Hkv, cap, hd), np.uint16); vc = np.zeros((Hkv, cap, hd), np.uint16)
    kc[:, :offset] = util.bf16_normal(rng, (Hkv, offset, hd)); vc[:, :offset] = util.bf16_normal(rng, (Hkv, offset, hd))
    # rows past the end hold NaN patterns: nothing may read them
    kc[:, offset + T:] = 0x7FC0; vc[:, offset + T:] = 0x7FC0
    return qg, kx, vx, qw, kw, kc, vc


@pytest.mark.parametrize("T,Hq,Hkv,hd,cap,offset", [
    (1, 16, 2, 256, 4096, 4000), (2, 16, 2, 256, 4096, 255), (4, 16, 2, 256, 4096, 1021),
    # decode widths in short contexts (prep folded into the attention launch): first rows of a
    # cache, new rows across the end of a key block, the widest folded call, head_dim 128
    (1, 16, 2, 256, 4096, 0), (2, 16, 2, 256, 4096, 51), (4, 16, 2, 256, 4096, 254), (8, 16, 2, 256, 4096, 250),
    (8, 16, 2, 256, 4096, 100), (3, 8, 2, 128, 1024, 255), (5, 4, 4, 256, 512, 300),
    (3, 4, 1, 256, 512, 0), (2, 4, 2, 128, 768, 300), (1, 2, 2, 256, 256, 7),
    # many live key blocks: the launch switches to its 256-thread form (same sums)
    (4, 16, 2, 256, 4096, 4000), (4, 16, 2, 128, 4096, 3000),
    # ... with one head a workgroup (KV groups of three heads) and four (groups of eight, ragged last block)
    (8, 6, 2, 256, 8192, 8000), (3, 16, 2, 256, 8192, 7000),
    # 16-row prompt chunks inside the first key block (one finishing launch) and across its end
    # (enough rows for the four-head form, which leaves the finishing to the merge launch)
    (16, 16, 2, 256, 4096, 35), (16, 16, 2, 128, 4096, 0), (16, 16, 2, 256, 4096, 250),
    # the long-context configuration: a depth-3 verify window at the end of a 16384-row cache
    (4, 16, 2, 256, 16384, 16380), (1, 16, 2, 256, 16384, 6621)])
def test_attention_bit_exact(orn, ctx, T, Hq, Hkv, hd, cap, offset):
    rng = np.random.default_rng(T * 1000 + offset)
    qg, kx, vx, qw, kw, kc, vc = _mk(rng, T, Hq, Hkv, hd, cap, offset)
    rd = 64 if hd == 256 else 32
    c, s = util.orc_rope_table(cap, rd, 1e7)
    dc, ds = ctx.rope_table(cap, rd, 1e7)
    assert np.array_equal(dc.download(np.float32, c.shape), c) and np.array_equal(ds.download(np.float32, s.shape), s)
    d = [ctx.to_device(a) for a in (qg, kx, vx, qw, kw)]
    dkc, dvc = ctx.to_device(kc), ctx.to_device(vc)
    dq, dout = ctx.alloc(T * Hq * hd * 2), ctx.alloc(T * Hq * hd * 2)
    wkc, wvc = kc.copy(), vc.copy()
    wq, wgate = util.orc_attn_prep(qg, kx, vx, qw, kw, rd, c, s, offset, wkc, wvc)
    want = util.orc_sdpa(wq, wkc, wvc, wgate, offset, hd ** -0.5)
    for use_dev_offset in (False, True):
        doff = ctx.to_device(np.array([offset], np.int32)) if use_dev_offset else None
        dkc.upload(kc); dvc.upload(vc)
        ctx.attn_prep(*d, T, Hq, Hkv, hd, rd, 1e-6, dc, ds, cap, 0 if use_dev_offset else offset, cap, dq, dkc, dvc, d_offset=doff)
        assert np.array_equal(dq.download(np.uint16, wq.shape), wq)
        assert np.array_equal(dkc.download(np.uint16, kc.shape), wkc) and np.array_equal(dvc.download(np.uint16, vc.shape), wvc)
        ctx.sdpa_decode_gated(dq, dkc, dvc, d[0], T, Hq, Hkv, hd, 0 if use_dev_offset else offset, cap, hd ** -0.5, dout, d_offset=doff)
        assert np.array_equal(dout.download(np.uint16, want.shape), want), use_dev_offset
        if doff: doff.free()
    # prep + attention as one call (one launch at decode widths in short contexts, a prep launch
    # first otherwise; with the fold switched off it is always two): same output, same caches
    for fold in (1, 0):
        orn.set_option("fuse_attn_prep", fold)
        dkc.upload(kc); dvc.upload(vc); dout.zero()
        ctx.attn_decode(*d, T, Hq, Hkv, hd, rd, 1e-6, dc, ds, cap, offset, cap, hd ** -0.5, dq, dkc, dvc, dout)
        assert np.array_equal(dout.download(np.uint16, want.shape), want), ("attn_decode", fold)
        assert np.array_equal(dkc.download(np.uint16, kc.shape), wkc) and np.array_equal(dvc.download(np.uint16, vc.shape), wvc), fold
    orn.set_option("fuse_attn_prep", 1)
    for b in d + [dkc, dvc, dq, dout, dc, ds]: b.free()
