"""GPU parity of the 4-bit affine (group 32) format against the oracle, bit for bit: Linear
mat-vec at decode widths, the gathered form over stacked experts, the table lookup, and a
small model whose affine modules (embed_tokens, shared_expert_gate) are in that format through
both generation loops."""
import numpy as np
import pytest

import synth
import util
from util import oracle, p

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("O,K", [(512, 2048), (7, 32), (2048, 4096), (33, 96), (1, 2048)])
def test_affine4_linear_bit_exact(orn, ctx, O, K):
    rng = np.random.default_rng(O + K)
    lin = util.HostLinear.affine4(rng, O, K)
    dl = lin.dev(orn, ctx)
    for M in (1, 2, 4, 5):
        xb = util.bf16_normal(rng, (M, K))
        want = np.empty((M, O), np.uint16)
        oracle().orc_affine4_gather_qmv(p(lin.w), p(lin.scales), p(lin.biases), 1, O, K, p(xb), None, None, M, p(want))
        dx, dy = ctx.to_device(xb), ctx.alloc(M * O * 2)
        ctx.linear_matmul(dl, dx, M, dy)
        assert np.array_equal(dy.download(np.uint16, (M, O)), want), M
        dx.free(); dy.free()
    dl.free()


def test_affine4_gather_and_lookup_bit_exact(orn, ctx):
    rng = np.random.default_rng(3)
    E, O, K, T, k = 16, 256, 512, 3, 4
    lin = util.HostLinear.affine4(rng, E * O, K)
    xb = util.bf16_normal(rng, (T, K))
    lhs = np.repeat(np.arange(T, dtype=np.uint32), k)
    rhs = np.concatenate([rng.permutation(E)[:k] for _ in range(T)]).astype(np.uint32)
    want = np.empty((T * k, O), np.uint16)
    oracle().orc_affine4_gather_qmv(p(lin.w), p(lin.scales), p(lin.biases), E, O, K, p(xb), p(lhs), p(rhs), T * k, p(want))
    d = [ctx.to_device(a) for a in (lin.w, lin.scales, lin.biases, xb, lhs, rhs)]
    dy = ctx.alloc(T * k * O * 2)
    ctx.affine4_gather_qmv(d[0], d[1], d[2], E, O, K, d[3], T, d[4], d[5], T * k, dy)
    assert np.array_equal(dy.download(np.uint16, (T * k, O)), want)
    # the lookup: rows of the same tensors seen as a [E*O, K] table
    table = orn.Linear(orn.LinearStruct(orn.LIN_AFFINE4, E * O, K, orn.KMatrixStruct(), d[0].ptr, d[1].ptr, d[2].ptr), [])
    ids = np.array([0, E * O - 1, 77], np.uint32)
    wout = np.empty((3, K), np.uint16)
    oracle().orc_embedding4(p(lin.w), p(lin.scales), p(lin.biases), K, p(ids), 3, p(wout))
    di, do = ctx.to_device(ids), ctx.alloc(3 * K * 2)
    ctx.embedding(table, di, 3, do)
    assert np.array_equal(do.download(np.uint16, (3, K)), wout)
    for b in d + [dy, di, do]: b.free()


def test_model_with_4bit_affine_modules_matches_oracle(orn, ctx):
    s = synth.SynthModel(dict(synth.TINY, vocab_size=256), seed=31, affine="affine4")
    ws = s.upload(orn, ctx)
    model = orn.TextModel(ctx, ws, s.text_config(orn))
    prompt = np.random.default_rng(1).integers(0, 256, 9).astype(np.uint32)
    caches = model.make_cache(48, 3)
    head = orn.MtpHead(model, ws, 48)
    try:
        ar = orn.generate_step(model, caches, prompt, 14, prefill_step=4)
        caches.reset()
        spec, st = orn.generate_step_mtp(model, head, None, caches, prompt, 2, 14, prefill_step=4)
        o = synth.OracleRun(s, 48)
        want = o.generate(prompt, 14, prefill_step=4)
        o.close()
        assert ar == want and spec == ar
    finally:
        head.close(); caches.close(); model.close(); ws.close()


@pytest.mark.parametrize("T", [1, 2, 4, 9, 150])
def test_moe_block_with_4bit_affine_experts_bit_exact(orn, ctx, T):
    """The published artifact's block: routed and shared experts 4-bit affine group 32, router and
    shared gate 8-bit. Expert ids, scores and output by bits against the oracle. 150 rows: a
    prompt chunk wider than the operator path's 64 rows, taken in blocks."""
    rng = np.random.default_rng(40 + T)
    moe = util.HostMoe(rng, H=1024, E=64, I=256, top_k=8, gate_kind=util.AFFINE4)
    xb = util.bf16_normal(rng, (T, 1024))
    want, winds, wscores, _ = util.orc_moe_block(moe, xb, T)
    w = moe.dev(orn, ctx)
    dx = ctx.to_device(xb)
    out, inds, scores = ctx.alloc(T * 1024 * 2), ctx.alloc(T * 8 * 4), ctx.alloc(T * 8 * 2)
    try:
        # the two fused expert launches (the default), then one launch per operator
        for fuse in (1, 0):
            orn.set_option("fuse_moe", fuse)
            for b in (out, inds, scores): b.zero()
            ctx.moe_block(w, dx, T, out, inds, scores)
            assert np.array_equal(inds.download(np.uint32, (T, 8)), winds), fuse
            assert np.array_equal(scores.download(np.uint16, (T, 8)), wscores), fuse
            assert np.array_equal(out.download(np.uint16, (T, 1024)), want), fuse
    finally:
        orn.set_option("fuse_moe", 1)
        for b in (dx, out, inds, scores): b.free()
        moe.free()


def test_model_in_the_published_artifacts_format_matches_oracle(orn, ctx):
    """Every projection, the routed and shared experts, embed_tokens and lm_head 4-bit affine
    group 32 (routers 8-bit), as the published mlx artifact stores them: both loops, with and
    without a pruned draft head, token for token against the oracle."""
    s = synth.SynthModel(dict(synth.TINY, vocab_size=256), seed=33, affine="affine4", trunk="affine4")
    ws = s.upload(orn, ctx)
    model = orn.TextModel(ctx, ws, s.text_config(orn))
    prompt = np.random.default_rng(2).integers(0, 256, 9).astype(np.uint32)
    caches = model.make_cache(48, 3)
    head = orn.MtpHead(model, ws, 48)
    fr_ids = synth.zipf_frspec_ids(256, 96, seed=3)
    fr = orn.FrSpec(model, ids=fr_ids)
    try:
        ar = orn.generate_step(model, caches, prompt, 14, prefill_step=4)
        o = synth.OracleRun(s, 48)
        want = o.generate(prompt, 14, prefill_step=4)
        o.close()
        assert ar == want
        for frs, frh in ((None, None), (fr, synth.prune_head(s.lm_head, fr_ids))):
            caches.reset()
            head.set_offset(0)
            spec, st = orn.generate_step_mtp(model, head, frs, caches, prompt, 2, 14, prefill_step=4)
            o = synth.OracleRun(s, 48)
            wspec, wst = o.mtp_generate(prompt, 2, 14, fr_ids if frs else None, frh, prefill_step=4)
            o.close()
            assert spec == ar == wspec
            assert (st.cycles, st.drafted, st.accepted) == (wst.cycles, wst.drafted, wst.accepted)
    finally:
        fr.close(); head.close(); caches.close(); model.close(); ws.close()
