"""GPU: the prefill-width kernels (matrix-core GEMM over k-quant weights, gathered per expert).
Prefill is outside the exact window in the reference too, so these are tolerance tests: the
reference of record is a float64 GEMM over the bf16-rounded dequantized weights (what the
kernel feeds the matrix cores); the tolerance is stated in _check."""
import numpy as np
import pytest

import util
from util import Q4K, Q6K

pytestmark = pytest.mark.gpu


def _deq_bf16(kind, t, E, O, K):
    w = util.orc_dequant(kind, *t, E * O * K // 256).reshape(E, O, K)
    return util.bf16_to_f32(util.f32_to_bf16(w)).astype(np.float64)


def _check(got_bits, want64, K, what):
    """|got - want| <= 2^-8 |want| (bf16 output rounding, one ulp) + 2e-3 * sqrt(K) * rms-product:
    fp32 accumulation order on the matrix cores is not the oracle's; both terms are ~10x what
    is observed."""
    got = util.bf16_to_f32(got_bits).astype(np.float64)
    scale = np.sqrt(np.mean(want64 ** 2))
    err = np.abs(got - want64)
    bound = 2.0 ** -8 * np.abs(want64) + 2e-3 * scale
    assert np.all(err <= bound), (what, float(err.max()), float(scale))
    return float((err / (np.abs(want64) + scale)).max())


@pytest.mark.parametrize("kind,O,K,M", [(Q4K, 256, 512, 128), (Q4K, 512, 2048, 300), (Q6K, 256, 512, 128),
                                         (Q6K, 384, 2048, 77), (Q4K, 8192, 2048, 256), (Q6K, 2048, 4096, 129),
                                         (Q4K, 200, 256, 16),
                                         # enough 256-row tiles to fill the device: the producer / consumer kernel,
                                         # ragged in rows (1061 = 4 tiles + 37) and a whole number of tiles
                                         (Q4K, 8192, 512, 1061), (Q6K, 8192, 1024, 1024),
                                         # a 4096-row prompt chunk through the widest projection of a gated-delta
                                         # layer and through q_proj: the sampled configuration's prefill call
                                         (Q4K, 8192, 2048, 4096), (Q6K, 8192, 2048, 4096)])
def test_kq_matmul_vs_float64(orn, ctx, kind, O, K, M):
    rng = np.random.default_rng(O + K + M + kind)
    t = util.make_kq(kind, rng, 1, O, K)
    w = orn.KMatrix(ctx, kind, *t, 1, O, K)
    xb = util.bf16_normal(rng, (M, K))
    dx, dy = ctx.to_device(xb), ctx.alloc(M * O * 2)
    orn.kq_matmul(ctx, w, dx, M, dy)
    got = dy.download(np.uint16, (M, O))
    want = util.bf16_to_f32(xb).astype(np.float64) @ _deq_bf16(kind, t, 1, O, K)[0].T
    _check(got, want, K, (kind, O, K, M))
    # and against the exact mat-vec path on a few rows: same numbers up to the weights' bf16 rounding
    dy1 = ctx.alloc(4 * O * 2)
    ctx.kq_qmv(w, dx, orn.BF16, 4, dy1, orn.BF16)
    mv = util.bf16_to_f32(dy1.download(np.uint16, (4, O))).astype(np.float64)
    g4 = util.bf16_to_f32(got[:4]).astype(np.float64)
    assert np.max(np.abs(mv - g4)) <= 0.02 * np.sqrt(np.mean(mv ** 2)) + 2.0 ** -7 * np.abs(mv).max()
    for b in (dx, dy, dy1): b.free()
    w.free()


@pytest.mark.parametrize("kind,O,K,M", [(Q4K, 512, 2048, 256), (Q6K, 2048, 512, 256), (Q4K, 8192, 2048, 512),
                                         (Q6K, 2048, 4096, 300)])
def test_kq_matmul_error_against_the_true_weights(orn, ctx, kind, O, K, M):
    """The stated numerical contract of the matrix-core GEMM. The reference dequantizes into a
    float tile (kernels/kquant_mm.h:88-118); this kernel rounds every dequantized weight to bf16
    on its way to the matrix cores, so against a float64 product over the TRUE dequantized
    weights it carries that rounding on top of the bf16 rounding of its output. Measured and
    bounded here: global relative error ||got - want|| / ||want|| <= 3.5e-3 (observed 2.3e-3 to
    2.4e-3) and every element error <= 2 % of the output's rms + one bf16 ulp of the element;
    the exact mat-vec path on the same rows, which rounds only its output: <= 2.5e-3 (observed
    1.7e-3). So the weight rounding adds about as much again as the output rounding.
    `pytest -s` prints the figures."""
    rng = np.random.default_rng(O * 7 + K + M + kind)
    t = util.make_kq(kind, rng, 1, O, K)
    w = orn.KMatrix(ctx, kind, *t, 1, O, K)
    xb = util.bf16_normal(rng, (M, K))
    true64 = util.orc_dequant(kind, *t, O * K // 256).reshape(O, K).astype(np.float64)
    want = util.bf16_to_f32(xb).astype(np.float64) @ true64.T
    dx, dy = ctx.to_device(xb), ctx.alloc(M * O * 2)
    orn.kq_matmul(ctx, w, dx, M, dy)
    got = util.bf16_to_f32(dy.download(np.uint16, (M, O))).astype(np.float64)
    rms = float(np.sqrt(np.mean(want ** 2)))
    g_rel = float(np.linalg.norm(got - want) / np.linalg.norm(want))
    g_abs = float(np.abs(got - want).max())
    # the exact path on the first rows (four rows a call)
    rows = min(M, 32)
    ex = np.empty((rows, O), np.float64)
    dy1 = ctx.alloc(4 * O * 2)
    for r in range(0, rows, 4):
        ctx.kq_qmv(w, ctx_off(dx, r * K * 2), orn.BF16, 4, dy1, orn.BF16)
        ex[r:r + 4] = util.bf16_to_f32(dy1.download(np.uint16, (4, O)))
    e_rel = float(np.linalg.norm(ex - want[:rows]) / np.linalg.norm(want[:rows]))
    e_abs = float(np.abs(ex - want[:rows]).max())
    print("%s %dx%d M=%d vs float64 of the true weights: GEMM global-rel %.3e max-abs %.3e (%.2f %% of rms); "
          "exact path global-rel %.3e max-abs %.3e" % ("Q4_K" if kind == Q4K else "Q6_K", O, K, M, g_rel, g_abs,
                                                       100 * g_abs / rms, e_rel, e_abs))
    assert g_rel <= 3.5e-3, g_rel
    assert np.all(np.abs(got - want) <= 0.02 * rms + 2.0 ** -8 * np.abs(want)), g_abs / rms
    assert e_rel <= 2.5e-3, e_rel
    for b in (dx, dy, dy1): b.free()
    w.free()


class _Off:
    """A device pointer `bytes` into a DeviceBuffer, for calls that take a buffer object."""

    def __init__(self, buf, nbytes):
        import ctypes as C
        self.ptr = C.c_void_p(buf.ptr.value + nbytes)


def ctx_off(buf, nbytes):
    return _Off(buf, nbytes)


@pytest.mark.parametrize("kind,E,O,K,T,k", [(Q4K, 8, 256, 512, 40, 2), (Q4K, 256, 512, 2048, 300, 8),
                                             (Q6K, 256, 2048, 512, 300, 8), (Q6K, 16, 128, 256, 5, 4),
                                             # about 100 rows an expert and more: 128-row tiles
                                             (Q4K, 8, 256, 512, 400, 2), (Q6K, 16, 128, 256, 500, 4),
                                             # more than 8192 pairs (the plan made by three launches), a few
                                             # hundred rows an expert and one crowded expert: tall tiles, the
                                             # register form for K >= 1024 and its split over shorter workgroups
                                             (Q4K, 32, 512, 2048, 1100, 8), (Q6K, 32, 256, 1024, 1100, 8),
                                             (Q6K, 32, 1024, 512, 1100, 8)])
def test_kq_gather_matmul_vs_float64(orn, ctx, kind, E, O, K, T, k):
    rng = np.random.default_rng(E + O + K + T)
    t = util.make_kq(kind, rng, E, O, K)
    w = orn.KMatrix(ctx, kind, *t, E, O, K)
    inds = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.uint32)
    if T > 20:
        inds[: T // 2, 0] = 3        # one crowded expert: several tiles, one of them ragged
    pairs = T * k
    deq = _deq_bf16(kind, t, E, O, K)
    plan = ctx.alloc(orn.kq_gather_plan_bytes(pairs, E))
    di = ctx.to_device(inds.reshape(-1))
    # gate / up form: pair p reads token p // k
    xb = util.bf16_normal(rng, (T, K))
    dx, dy = ctx.to_device(xb), ctx.alloc(pairs * O * 2)
    ctx.memset(dy, 0xFF, pairs * O * 2)
    orn.kq_gather_matmul(ctx, w, dx, di, pairs, k, True, plan, True, dy)
    got = dy.download(np.uint16, (pairs, O))
    xf = util.bf16_to_f32(xb).astype(np.float64)
    flat = inds.reshape(-1)

    def by_expert(rows_in):       # want[p] = rows_in[p] @ deq[flat[p]].T, one product an expert
        out = np.empty((pairs, O))
        for e in np.unique(flat):
            sel = np.nonzero(flat == e)[0]
            out[sel] = rows_in[sel] @ deq[e].T
        return out

    want = by_expert(xf[np.arange(pairs) // k])
    _check(got, want, K, "up")
    # down form on the same plan: pair p reads row p
    ab = util.bf16_normal(rng, (pairs, K))
    da = ctx.to_device(ab)
    orn.kq_gather_matmul(ctx, w, da, di, pairs, k, False, plan, False, dy)
    got = dy.download(np.uint16, (pairs, O))
    af = util.bf16_to_f32(ab).astype(np.float64)
    want = by_expert(af)
    _check(got, want, K, "down")
    for b in (plan, di, dx, dy, da): b.free()
    w.free()


def _rows_close(got_bits, want_bits, tol):
    """per-row relative L2 error of two bf16 [T, n] arrays"""
    g = util.bf16_to_f32(got_bits).astype(np.float64)
    w = util.bf16_to_f32(want_bits).astype(np.float64)
    return np.linalg.norm(g - w, axis=1) / (np.linalg.norm(w, axis=1) + 1e-30) <= tol


@pytest.mark.parametrize("H,E,I,T", [(512, 64, 256, 48), (2048, 256, 512, 160),
                                     # 64 and 150 rows an expert: tall plan tiles, split over 64-row workgroups
                                     (512, 64, 256, 512), (512, 64, 256, 1200),
                                     # gate / up in the register form (K = 1024), down on the same plan in 64-row workgroups
                                     (1024, 64, 256, 512), (1024, 64, 256, 1300)])
def test_moe_block_prefill_width_close_to_exact_path(orn, ctx, H, E, I, T):
    """At prefill width the block runs as GEMMs. Against the oracle's exact path the rows agree
    to 2 % relative L2 (bf16 weights on the matrix cores, fp32 sums in another order); a row
    whose router logits tie within that noise may route one expert differently, so up to 3 % of
    the rows are allowed to differ more."""
    rng = np.random.default_rng(H + T)
    moe = util.HostMoe(rng, H=H, E=E, I=I, top_k=8, gate_kind=Q4K, down_kind=Q6K, router_kind=Q6K)
    dw = moe.dev(orn, ctx)
    xb = util.bf16_normal(rng, (T, H))
    dx, dout = ctx.to_device(xb), ctx.alloc(T * H * 2)
    ctx.moe_block(dw, dx, T, dout)
    got = dout.download(np.uint16, (T, H))
    want = np.concatenate([util.orc_moe_block(moe, xb[t:t + 1], 1)[0] for t in range(T)])
    ok = _rows_close(got, want, 0.02)
    assert ok.mean() >= 0.97, float(ok.mean())
    dx.free(); dout.free(); moe.free()


def _make_weights_bf16_exact(s):
    """Rewrites the k-quant fields of a SynthModel in place so that every dequantized weight is
    exactly a bf16 number: d a power of two, Q4_K scale / min codes <= 7 with dmin = 7.5 d
    (|d*sc*q - dmin*m| <= 210 half-units of d), Q6_K scales in [-4, 3] (|sc*q| <= 128). The GEMM
    path then differs from the exact path by the order of its fp32 sums alone."""
    for name, (arr, _) in s.tensors.items():
        if not name.endswith(".dm"):
            continue
        sc = s.tensors[name[:-3] + ".scales"][0]
        d = arr.view(np.float16)
        if arr.shape[-1] == 2:      # Q4_K
            p2 = np.exp2(np.floor(np.log2(np.maximum(d[..., 0].astype(np.float32), 2.0 ** -14)))).astype(np.float16)
            d[..., 0] = p2
            d[..., 1] = (p2.astype(np.float32) * 7.5).astype(np.float16)
            sc[..., 0:8] &= 0x07
            sc[..., 8:12] &= 0x77
        else:                        # Q6_K
            d[..., 0] = np.exp2(np.floor(np.log2(np.maximum(d[..., 0].astype(np.float32), 2.0 ** -14)))).astype(np.float16)
            sc8 = sc.view(np.int8)
            sc8[...] = sc8 >> 4


@pytest.mark.parametrize("exact_weights", [True, False])
def test_model_prefill_in_wide_chunks_close_to_exact_chunks(orn, ctx, exact_weights):
    """A 96-token prompt through the tiny model in chunks of 48 (GEMM path) and of 16 (exact
    path). With weights that are bf16 numbers already the two paths differ by fp32 summation
    order only: nearly every row agrees to 1 % relative L2 (a bf16 ulp that flips early can
    re-route an expert downstream). With ordinary weights the bf16 rounding of every weight
    tile is on top, and a random 4-layer router is chaotic: the rows stay correlated, no more
    is asserted. The caches end at the same length and decode continues from either."""
    import synth
    s = synth.SynthModel(synth.TINY, seed=5)
    if exact_weights:
        _make_weights_bf16_exact(s)
    ws = s.upload(orn, ctx)
    model = orn.TextModel(ctx, ws, s.text_config(orn))
    rng = np.random.default_rng(9)
    toks = rng.integers(0, s.cfg["vocab_size"], 96).astype(np.uint32)
    narrow = model.make_cache(128, 2)
    h16 = np.concatenate([model.forward(narrow, toks[i:i + 16]) for i in range(0, 96, 16)])
    model.set_max_rows(64)
    wide = model.make_cache(128, 2)
    h48 = np.concatenate([model.forward(wide, toks[i:i + 48]) for i in range(0, 96, 48)])
    assert wide.offset == narrow.offset == 96
    g = util.bf16_to_f32(h48).astype(np.float64); w = util.bf16_to_f32(h16).astype(np.float64)
    rel = np.linalg.norm(g - w, axis=1) / np.linalg.norm(w, axis=1)
    cos = np.sum(g * w, axis=1) / (np.linalg.norm(g, axis=1) * np.linalg.norm(w, axis=1))
    print("relative L2 per row: median %.4f max %.4f; min cosine %.4f" % (np.median(rel), rel.max(), cos.min()))
    if exact_weights:
        assert (rel <= 0.01).mean() >= 0.9 and np.median(rel) < 0.003, (float(np.median(rel)), float(rel.max()))
    else:
        assert np.median(cos) > 0.99 and cos.min() > 0.7
    nxt = np.array([7], np.uint32)
    a, b = model.forward(narrow, nxt), model.forward(wide, nxt)
    assert a.shape == b.shape
    with pytest.raises(orn.OrnithError, match="created for"):
        model.forward(narrow, toks[:48])          # caches made before the model was widened
    for o in (narrow, wide, model, ws): o.close()


@pytest.mark.parametrize("T,Hq,Hkv,cap,offset", [(64, 16, 2, 512, 0), (100, 4, 1, 1024, 37), (300, 16, 2, 2048, 1000),
                                                 (33, 2, 2, 256, 200), (512, 8, 2, 1024, 512)])
def test_prefill_attention_close_to_exact_kernel(orn, ctx, T, Hq, Hkv, cap, offset):
    """Causal flash attention on the matrix cores vs the oracle's exact attention: every row
    within 1 % relative L2 (bf16 probabilities into the second GEMM, fp32 sums in block order).
    Cache rows past the chunk hold NaN patterns: nothing may read them."""
    from test_gpu_attn import _mk
    hd, rd = 256, 64
    rng = np.random.default_rng(T + offset)
    qg, kx, vx, qw, kw, kc, vc = _mk(rng, T, Hq, Hkv, hd, cap, offset)
    c, s = util.orc_rope_table(cap, rd, 1e7)
    wkc, wvc = kc.copy(), vc.copy()
    wq, wgate = util.orc_attn_prep(qg, kx, vx, qw, kw, rd, c, s, offset, wkc, wvc)
    want = util.orc_sdpa(wq, wkc, wvc, wgate, offset, hd ** -0.5)
    dq, dk, dv, dg = ctx.to_device(wq), ctx.to_device(wkc), ctx.to_device(wvc), ctx.to_device(qg)
    dout = ctx.alloc(T * Hq * hd * 2)
    ctx.sdpa_decode_gated(dq, dk, dv, dg, T, Hq, Hkv, hd, offset, cap, hd ** -0.5, dout)
    got = dout.download(np.uint16, want.shape)
    g = util.bf16_to_f32(got).astype(np.float64).reshape(T * Hq, hd)
    w = util.bf16_to_f32(want).astype(np.float64).reshape(T * Hq, hd)
    assert np.isfinite(g).all()
    rel = np.linalg.norm(g - w, axis=1) / np.linalg.norm(w, axis=1)
    assert rel.max() < 0.01, float(rel.max())
    for b in (dq, dk, dv, dg, dout): b.free()


@pytest.mark.parametrize("T,offset", [(4096, 4096), (6621, 0)])
def test_prefill_attention_at_the_long_context_sizes(orn, ctx, T, offset):
    """The sampled configuration's sizes: a 4096-row prompt chunk behind 4096 cached rows, and
    the whole 6621-row prompt in one call, in a 16384-row cache, 16 query heads over 2 KV heads
    of 256. Checked on 96 sampled (row, head) pairs (first and last rows included) against a
    float64 softmax attention of the same bf16 operands, and for chunk invariance: the same rows
    in 512-row calls agree with the one call to rounding."""
    Hq, Hkv, hd, cap = 16, 2, 256, 16384
    rng = np.random.default_rng(55 + offset)
    q = util.bf16_normal(rng, (T, Hq, hd)); qg = util.bf16_normal(rng, (T, Hq, 2 * hd))
    kc = np.full((Hkv, cap, hd), 0x7FC0, np.uint16); vc = np.full((Hkv, cap, hd), 0x7FC0, np.uint16)
    kc[:, :offset + T] = util.bf16_normal(rng, (Hkv, offset + T, hd)); vc[:, :offset + T] = util.bf16_normal(rng, (Hkv, offset + T, hd))
    dq, dk, dv, dg = ctx.to_device(q), ctx.to_device(kc), ctx.to_device(vc), ctx.to_device(qg)
    dout = ctx.alloc(T * Hq * hd * 2)
    ctx.sdpa_decode_gated(dq, dk, dv, dg, T, Hq, Hkv, hd, offset, cap, hd ** -0.5, dout)
    got = util.bf16_to_f32(dout.download(np.uint16, (T, Hq, hd))).astype(np.float64)
    assert np.isfinite(got).all()
    K64 = util.bf16_to_f32(kc[:, :offset + T]).astype(np.float64); V64 = util.bf16_to_f32(vc[:, :offset + T]).astype(np.float64)
    rows = [0, 1, T - 1, T - 2] + list(rng.integers(2, T - 2, 20))
    worst = 0.0
    for t in rows:
        for h in rng.choice(Hq, 4, replace=False):
            n = offset + t + 1
            sc = (K64[h // (Hq // Hkv), :n] @ util.bf16_to_f32(q[t, h]).astype(np.float64)) * hd ** -0.5
            pr = np.exp(sc - sc.max()); pr /= pr.sum()
            gate = util.bf16_to_f32(qg[t, h, hd:]).astype(np.float64)
            want = (pr @ V64[h // (Hq // Hkv), :n]) / (1 + np.exp(-gate))
            worst = max(worst, np.linalg.norm(got[t, h] - want) / np.linalg.norm(want))
    assert worst < 0.01, worst
    # the same rows in 512-row calls
    dq2, dg2, dout2 = ctx.alloc(512 * Hq * hd * 2), ctx.alloc(512 * Hq * 2 * hd * 2), ctx.alloc(512 * Hq * hd * 2)
    for c0 in (0, 2048, 3584):
        dq2.upload(q[c0:c0 + 512]); dg2.upload(qg[c0:c0 + 512])
        ctx.sdpa_decode_gated(dq2, dk, dv, dg2, 512, Hq, Hkv, hd, offset + c0, cap, hd ** -0.5, dout2)
        part = util.bf16_to_f32(dout2.download(np.uint16, (512, Hq, hd))).astype(np.float64)
        rel = np.linalg.norm((part - got[c0:c0 + 512]).reshape(-1, hd), axis=1) / np.linalg.norm(got[c0:c0 + 512].reshape(-1, hd), axis=1)
        assert rel.max() < 0.01, (c0, float(rel.max()))
    for b in (dq, dk, dv, dg, dout, dq2, dg2, dout2): b.free()


def test_model_forward_at_the_reference_chunk_width(orn, ctx):
    """2048 rows in one call (the reference's prefill_step_size): the step buffers are sized by
    the layout they hold, so every row lands inside them; with bf16-exact weights the result
    agrees with four 512-row calls to summation-order noise."""
    import synth
    s = synth.SynthModel(synth.TINY, seed=8, with_mtp=False)
    _make_weights_bf16_exact(s)
    ws = s.upload(orn, ctx)
    model = orn.TextModel(ctx, ws, s.text_config(orn))
    model.set_max_rows(2048)
    toks = np.random.default_rng(1).integers(0, s.cfg["vocab_size"], 2048).astype(np.uint32)
    a, b = model.make_cache(2100, 2), model.make_cache(2100, 2)
    h1 = model.forward(a, toks)
    h4 = np.concatenate([model.forward(b, toks[i:i + 512]) for i in range(0, 2048, 512)])
    assert a.offset == b.offset == 2048
    g = util.bf16_to_f32(h1).astype(np.float64); w = util.bf16_to_f32(h4).astype(np.float64)
    assert np.isfinite(g).all()
    rel = np.linalg.norm(g - w, axis=1) / np.linalg.norm(w, axis=1)
    assert np.median(rel) < 0.003 and (rel <= 0.02).mean() >= 0.95, (float(np.median(rel)), float(rel.max()))
    for o in (a, b, model, ws): o.close()


def test_model_forward_of_a_whole_long_prompt_in_one_call(orn, ctx):
    """6621 rows (the sampled configuration's prompt) in one call, ragged against every tile
    (6621 = 103 * 64 + 29), against the EXACT path (16-row calls, every row as if alone: the path
    whose bits equal the oracle's). With bf16-exact weights the two differ by the order of their
    fp32 sums alone: the rows agree to summation-order noise, and the cache ends at the same
    length."""
    import synth
    s = synth.SynthModel(synth.TINY, seed=11, with_mtp=False)
    _make_weights_bf16_exact(s)
    ws = s.upload(orn, ctx)
    model = orn.TextModel(ctx, ws, s.text_config(orn))
    T = 6621
    toks = np.random.default_rng(2).integers(0, s.cfg["vocab_size"], T).astype(np.uint32)
    b = model.make_cache(6700, 2)
    hc = np.concatenate([model.forward(b, toks[i:i + 16]) for i in range(0, T, 16)])
    model.set_max_rows(8192)
    a = model.make_cache(6700, 2)
    h1 = model.forward(a, toks)
    assert a.offset == b.offset == T
    g = util.bf16_to_f32(h1).astype(np.float64); w = util.bf16_to_f32(hc).astype(np.float64)
    assert np.isfinite(g).all()
    rel = np.linalg.norm(g - w, axis=1) / np.linalg.norm(w, axis=1)
    print("6621-row call vs the exact path: relative L2 per row median %.4f, 95th percentile %.4f, max %.4f"
          % (np.median(rel), np.percentile(rel, 95), rel.max()))
    assert np.median(rel) < 0.003 and (rel <= 0.02).mean() >= 0.95, (float(np.median(rel)), float(rel.max()))
    with pytest.raises(orn.OrnithError, match="rows"):
        model.set_max_rows(8193)
    for o in (a, b, model, ws): o.close()


@pytest.mark.parametrize("O,K,M", [(32, 2048, 4096), (1, 2048, 300), (48, 256, 33), (130, 512, 77), (64, 128, 32)])
def test_dense_matmul_vs_float64(orn, ctx, O, K, M):
    """narrow dense bf16 projections at prefill widths run as a small matrix-core GEMM (rows split
    over workgroups, K over a workgroup's wavefronts); reference: float64 over the same bf16 values"""
    rng = np.random.default_rng(O + K + M)
    hl = util.HostLinear.dense(rng, O, K)
    lin = hl.dev(orn, ctx)
    xb = util.bf16_normal(rng, (M, K))
    dx, dy = ctx.to_device(xb), ctx.alloc(M * O * 2)
    ctx.memset(dy, 0xFF, M * O * 2)
    ctx.linear_matmul(lin, dx, M, dy)
    got = dy.download(np.uint16, (M, O))
    want = util.bf16_to_f32(xb).astype(np.float64) @ util.bf16_to_f32(hl.w).astype(np.float64).T
    _check(got, want, K, (O, K, M))
    # rows inside the exact window keep the mat-vec path: bit-equal to it row by row
    dy1 = ctx.alloc(4 * O * 2)
    ctx.linear_matmul(lin, dx, 4, dy1)
    mv = util.bf16_to_f32(dy1.download(np.uint16, (4, O))).astype(np.float64)
    assert np.max(np.abs(mv - util.bf16_to_f32(got[:4]).astype(np.float64))) <= 2.0 ** -7 * np.abs(mv).max() + 1e-3
    for b in (dx, dy, dy1): b.free()
    lin.free()


@pytest.mark.parametrize("kind,Os,K,M", [(Q4K, (512, 512), 2048, 4096), (Q6K, (8192, 200, 512), 512, 300),
                                         (Q4K, (256, 128, 384, 512), 256, 77),
                                         # both kinds in one launch: the MoE block's router with the shared expert's gate / up
                                         ((Q6K, Q4K, Q4K), (256, 512, 512), 2048, 4096), ((Q4K, Q6K), (100, 300), 512, 130)])
def test_projections_sharing_an_input_share_a_gemm_launch(orn, ctx, kind, Os, K, M):
    """linear_matmul_multi at prefill width: k-quant matrices of one K run as column ranges of
    one GEMM launch; every output equals the matrix's own launch bit for bit (an output element
    is one dot product in a fixed k order, whatever tile computes it)"""
    rng = np.random.default_rng(sum(Os) + K + M)
    kinds = kind if isinstance(kind, tuple) else (kind,) * len(Os)
    hls = [util.HostLinear.kq(rng, kd, O, K) for kd, O in zip(kinds, Os)]
    lins = [h.dev(orn, ctx) for h in hls]
    xb = util.bf16_normal(rng, (M, K))
    dx = ctx.to_device(xb)
    ys = [ctx.alloc(M * O * 2) for O in Os]
    for y, O in zip(ys, Os): ctx.memset(y, 0xFF, M * O * 2)
    ctx.linear_matmul_multi(lins, dx, M, ys)
    y1 = ctx.alloc(M * max(Os) * 2)
    for lin, y, O in zip(lins, ys, Os):
        ctx.linear_matmul(lin, dx, M, y1)
        assert np.array_equal(y.download(np.uint16, (M, O)), y1.download(np.uint16, (M, O))), O
    for b in [dx, y1] + ys: b.free()
    for l in lins: l.free()


@pytest.mark.parametrize("Os,K,M", [((32, 32), 2048, 4096), ((1, 40, 16), 256, 77)])
def test_dense_projections_sharing_an_input_share_a_launch(orn, ctx, Os, K, M):
    """linear_matmul_multi over dense matrices at prefill width: their 16-output tiles laid end to
    end in one launch; every output equals the matrix's own launch bit for bit"""
    rng = np.random.default_rng(sum(Os) + K + M)
    hls = [util.HostLinear.dense(rng, O, K) for O in Os]
    lins = [h.dev(orn, ctx) for h in hls]
    xb = util.bf16_normal(rng, (M, K))
    dx = ctx.to_device(xb)
    ys = [ctx.alloc(M * O * 2) for O in Os]
    for y, O in zip(ys, Os): ctx.memset(y, 0xFF, M * O * 2)
    ctx.linear_matmul_multi(lins, dx, M, ys)
    y1 = ctx.alloc(M * max(Os) * 2)
    for lin, y, O in zip(lins, ys, Os):
        ctx.linear_matmul(lin, dx, M, y1)
        assert np.array_equal(y.download(np.uint16, (M, O)), y1.download(np.uint16, (M, O))), O
    for b in [dx, y1] + ys: b.free()
    for l in lins: l.free()


def test_gathered_matmuls_of_different_depth_share_a_plan(orn, ctx):
    """The MoE block builds the pair plan with its gate projection (K = 1024 here: tall tiles,
    register form) and runs the down projection (K = 256: 64-row workgroups) on the same plan
    without rebuilding it: every pair's row must be computed, whatever the kernel's own tile
    height (outputs poisoned beforehand)."""
    rng = np.random.default_rng(12)
    E, T, k, Kg, Og, Kd, Od = 64, 700, 8, 1024, 256, 256, 384
    pairs = T * k
    tg, td = util.make_kq(Q4K, rng, E, Og, Kg), util.make_kq(Q6K, rng, E, Od, Kd)
    wg, wd = orn.KMatrix(ctx, Q4K, *tg, E, Og, Kg), orn.KMatrix(ctx, Q6K, *td, E, Od, Kd)
    inds = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.uint32)
    plan = ctx.alloc(orn.kq_gather_plan_bytes(pairs, E)); di = ctx.to_device(inds.reshape(-1))
    xb = util.bf16_normal(rng, (T, Kg)); ab = util.bf16_normal(rng, (pairs, Kd))
    dx, da = ctx.to_device(xb), ctx.to_device(ab)
    dyg, dyd = ctx.alloc(pairs * Og * 2), ctx.alloc(pairs * Od * 2)
    ctx.memset(dyg, 0xFF, pairs * Og * 2); ctx.memset(dyd, 0xFF, pairs * Od * 2)
    orn.kq_gather_matmul(ctx, wg, dx, di, pairs, k, True, plan, True, dyg)
    orn.kq_gather_matmul(ctx, wd, da, di, pairs, k, False, plan, False, dyd)
    flat = inds.reshape(-1)
    dg, dd = _deq_bf16(Q4K, tg, E, Og, Kg), _deq_bf16(Q6K, td, E, Od, Kd)
    xf, af = util.bf16_to_f32(xb).astype(np.float64), util.bf16_to_f32(ab).astype(np.float64)
    _check(dyg.download(np.uint16, (pairs, Og)), np.stack([xf[p // k] @ dg[flat[p]].T for p in range(pairs)]), Kg, "gate")
    _check(dyd.download(np.uint16, (pairs, Od)), np.stack([af[p] @ dd[flat[p]].T for p in range(pairs)]), Kd, "down")
    for b in (plan, di, dx, da, dyg, dyd): b.free()
    wg.free(); wd.free()


def test_prefill_paths_are_repeatable(orn, ctx):
    """The same MoE block call and the same model forward twice give the same bits: the expert
    plan is built with atomics (the order of an expert's pairs changes from run to run), so a row
    that depended on its place in a tile, or a tile row left uncomputed, shows up here as a
    difference between runs."""
    import synth
    rng = np.random.default_rng(21)
    moe = util.HostMoe(rng, H=1024, E=64, I=256, top_k=8, gate_kind=Q4K, down_kind=Q6K, router_kind=Q6K)
    dw = moe.dev(orn, ctx)
    T = 1300
    xb = util.bf16_normal(rng, (T, 1024))
    dx, dout = ctx.to_device(xb), ctx.alloc(T * 1024 * 2)
    outs = []
    for fill in (0x00, 0xFF, 0x5A):
        ctx.memset(dout, fill, T * 1024 * 2)
        ctx.moe_block(dw, dx, T, dout)
        outs.append(dout.download(np.uint16, (T, 1024)))
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])
    dx.free(); dout.free(); moe.free()
    s = synth.SynthModel(synth.TINY, seed=13, with_mtp=False)
    ws = s.upload(orn, ctx)
    model = orn.TextModel(ctx, ws, s.text_config(orn))
    model.set_max_rows(2048)
    toks = np.random.default_rng(3).integers(0, s.cfg["vocab_size"], 1500).astype(np.uint32)
    cache = model.make_cache(1600, 2)
    hs = []
    for _ in range(3):
        cache.reset()
        hs.append(model.forward(cache, toks))
    assert np.array_equal(hs[0], hs[1]) and np.array_equal(hs[0], hs[2])
    for o in (cache, model, ws): o.close()


@pytest.mark.parametrize("kind,E,O,K,T", [(Q4K, 8, 256, 1024, 3000), (Q6K, 8, 256, 512, 700)])
def test_kq_gather_matmul_every_pair_on_one_expert(orn, ctx, kind, E, O, K, T):
    """The other experts have no rows and no tiles; the one expert's rows fill tile after tile
    (the last one ragged). k = 1: a pair is a token."""
    rng = np.random.default_rng(T)
    t = util.make_kq(kind, rng, E, O, K)
    w = orn.KMatrix(ctx, kind, *t, E, O, K)
    inds = np.full(T, 5, np.uint32)
    deq = _deq_bf16(kind, t, E, O, K)
    plan = ctx.alloc(orn.kq_gather_plan_bytes(T, E))
    di = ctx.to_device(inds)
    xb = util.bf16_normal(rng, (T, K))
    dx, dy = ctx.to_device(xb), ctx.alloc(T * O * 2)
    want = util.bf16_to_f32(xb).astype(np.float64) @ deq[5].T
    for make_plan, gate_form in ((True, True), (False, False)):
        ctx.memset(dy, 0xFF, T * O * 2)
        orn.kq_gather_matmul(ctx, w, dx, di, T, 1, gate_form, plan, make_plan, dy)
        _check(dy.download(np.uint16, (T, O)), want, K, "one expert")
    for b in (plan, di, dx, dy): b.free()
    w.free()
