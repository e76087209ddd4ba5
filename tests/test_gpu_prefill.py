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
                                         (Q4K, 200, 256, 16)])
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


@pytest.mark.parametrize("kind,E,O,K,T,k", [(Q4K, 8, 256, 512, 40, 2), (Q4K, 256, 512, 2048, 300, 8),
                                             (Q6K, 256, 2048, 512, 300, 8), (Q6K, 16, 128, 256, 5, 4)])
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
    want = np.stack([xf[p // k] @ deq[inds.reshape(-1)[p]].T for p in range(pairs)])
    _check(got, want, K, "up")
    # down form on the same plan: pair p reads row p
    ab = util.bf16_normal(rng, (pairs, K))
    da = ctx.to_device(ab)
    orn.kq_gather_matmul(ctx, w, da, di, pairs, k, False, plan, False, dy)
    got = dy.download(np.uint16, (pairs, O))
    af = util.bf16_to_f32(ab).astype(np.float64)
    want = np.stack([af[p] @ deq[inds.reshape(-1)[p]].T for p in range(pairs)])
    _check(got, want, K, "down")
    for b in (plan, di, dx, dy, da): b.free()
    w.free()
