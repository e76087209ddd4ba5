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
