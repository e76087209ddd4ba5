"""GPU parity: MoE pieces and the whole block (BASELINE config 2) vs the oracle, bit-exact.
Expert indices are integers and must match exactly; every activation is bf16 and is
compared by bits."""
import ctypes as C

import numpy as np
import pytest

import util
from util import Q4K, Q6K, oracle, p

pytestmark = pytest.mark.gpu


def test_linear_modes_bit_exact(orn, ctx):
    rng = np.random.default_rng(0)
    for lin in (util.HostLinear.affine8(rng, 5, 2048), util.HostLinear.affine8(rng, 1, 512),
                util.HostLinear.dense(rng, 33, 2048), util.HostLinear.dense(rng, 64, 512),
                util.HostLinear.dense(rng, 7, 4096), util.HostLinear.kq(rng, Q6K, 256, 2048)):
        M = 3
        xb = util.f32_to_bf16(rng.standard_normal((M, lin.K)).astype(np.float32))
        want = np.empty((M, lin.O), np.uint16)
        if lin.mode == "affine8":
            oracle().orc_affine8_qmv(p(lin.w), p(lin.scales), p(lin.biases), lin.O, lin.K, p(xb), M, p(want))
        elif lin.mode == "dense":
            oracle().orc_dense_gemv(p(lin.w), lin.O, lin.K, p(xb), M, p(want))
        else:
            want = util.f32_to_bf16(util.orc_qmv(lin.km.kind, lin.km.qs, lin.km.scales, lin.km.dm, lin.O, lin.K, util.bf16_to_f32(xb)))
        d = lin.dev(orn, ctx)
        dx, dy = ctx.to_device(xb), ctx.alloc(M * lin.O * 2)
        ctx.linear_matmul(d, dx, M, dy)
        assert np.array_equal(dy.download(np.uint16, (M, lin.O)), want), lin.mode
        for b in (dx, dy): b.free()
        d.free()


@pytest.mark.parametrize("sizes", [(33, 5), (33, 5, 1), (7, 64, 1, 130), (1, 1, 1, 1)])
def test_dense_multi_equals_single_launches(orn, ctx, sizes):
    """Dense projections of the same activations in one launch: every output row is the
    oracle's (and so the single launch's), whatever the row counts of the segments."""
    rng = np.random.default_rng(len(sizes))
    K, M = 2048, 3
    lins = [util.HostLinear.dense(rng, O, K) for O in sizes]
    xb = util.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    devs = [l.dev(orn, ctx) for l in lins]
    dx = ctx.to_device(xb)
    # canaries after each output: a segment must not write past its own rows
    ys = [ctx.to_device(np.full(M * l.O + 8, 0xabcd, np.uint16)) for l in lins]
    ctx.linear_matmul_multi(devs, dx, M, ys)
    for l, y in zip(lins, ys):
        want = np.empty((M, l.O), np.uint16)
        oracle().orc_dense_gemv(p(l.w), l.O, l.K, p(xb), M, p(want))
        got = y.download(np.uint16, (M * l.O + 8,))
        assert np.array_equal(got[:M * l.O].reshape(M, l.O), want), sizes
        assert (got[M * l.O:] == 0xabcd).all()
    for b in ys + [dx]: b.free()
    for d in devs: d.free()


def test_embedding_and_dense_gather_bit_exact(orn, ctx):
    rng = np.random.default_rng(1)
    tab = util.HostLinear.affine8(rng, 300, 2048)
    ids = np.array([0, 299, 17, 17], np.uint32)
    want = np.empty((4, 2048), np.uint16)
    oracle().orc_embedding(p(tab.w), p(tab.scales), p(tab.biases), 2048, p(ids), 4, p(want))
    d = tab.dev(orn, ctx)
    di, do = ctx.to_device(ids), ctx.alloc(4 * 2048 * 2)
    ctx.embedding(d, di, 4, do)
    assert np.array_equal(do.download(np.uint16, (4, 2048)), want)
    E, O, K = 6, 40, 512
    w = util.f32_to_bf16((rng.standard_normal((E, O, K)) / np.sqrt(K)).astype(np.float32))
    xb = util.f32_to_bf16(rng.standard_normal((2, K)).astype(np.float32))
    lhs = np.array([0, 1, 1, 0, 1], np.uint32); rhs = np.array([5, 0, 3, 3, 2], np.uint32)
    want = np.empty((5, O), np.uint16)
    oracle().orc_dense_gather_mv(p(w), O, K, p(xb), p(lhs), p(rhs), 5, p(want))
    dw, dx, dl, dr, dy = ctx.to_device(w), ctx.to_device(xb), ctx.to_device(lhs), ctx.to_device(rhs), ctx.alloc(5 * O * 2)
    ctx.dense_gather_mv(dw, E, O, K, dx, 2, dl, dr, 5, dy)
    assert np.array_equal(dy.download(np.uint16, (5, O)), want)
    for b in (di, do, dw, dx, dl, dr, dy): b.free()
    d.free()


@pytest.mark.parametrize("E", [64, 128, 256, 512, 1024])
def test_router_softmax_topk_bit_exact_with_ties(orn, ctx, E):
    rng = np.random.default_rng(2 + E)
    T, k = 6, 8
    g = (rng.standard_normal((T, E)) * 2).astype(np.float32)
    g[1] = np.round(g[1])            # many equal gates -> equal probabilities
    g[2] = 0.0                       # all tied: picks are the k largest indices
    g[3, :] = -50.0; g[3, 5] = 50.0  # one-hot softmax: exact zeros tie everywhere else
    gb = util.f32_to_bf16(g)
    probs = np.empty((T, E), np.uint16); inds = np.empty((T, k), np.uint32); sc = np.empty((T, k), np.uint16)
    oracle().orc_softmax_bf16(p(gb), T, E, p(probs))
    oracle().orc_router_topk(p(probs), T, E, k, p(inds), p(sc))
    dg, di, ds, dp = ctx.to_device(gb), ctx.alloc(T * k * 4), ctx.alloc(T * k * 2), ctx.alloc(T * E * 2)
    ctx.router_topk(dg, T, E, k, di, ds, dp)
    assert np.array_equal(dp.download(np.uint16, (T, E)), probs)
    assert np.array_equal(di.download(np.uint32, (T, k)), inds)
    assert np.array_equal(ds.download(np.uint16, (T, k)), sc)
    assert list(inds[2]) == list(range(E - k, E))
    for b in (dg, di, ds, dp): b.free()


def test_swiglu_and_combine_bit_exact(orn, ctx):
    rng = np.random.default_rng(3)
    bits = np.arange(65536, dtype=np.uint16)
    fin = np.isfinite(util.bf16_to_f32(bits))
    up = util.f32_to_bf16(rng.standard_normal(65536).astype(np.float32))
    want = np.empty(65536, np.uint16)
    oracle().orc_swiglu_bf16(p(bits), p(up), C.c_int64(65536), p(want))
    dg, du, do = ctx.to_device(bits), ctx.to_device(up), ctx.alloc(65536 * 2)
    ctx.swiglu(dg, du, 65536, do)
    assert np.array_equal(do.download(np.uint16, (65536,))[fin], want[fin])
    # a length that is not a multiple of 8 takes the one-element-a-thread form
    ctx.swiglu(dg, du, 65531, do)
    assert np.array_equal(do.download(np.uint16, (65536,))[:65531][fin[:65531]], want[:65531][fin[:65531]])
    for T, k, dim in ((3, 8, 2048), (5, 4, 100)):  # 100: not a multiple of 8 either
        scores = util.f32_to_bf16(rng.random((T, k)).astype(np.float32) * 0.1)
        y = util.f32_to_bf16(rng.standard_normal((T, k, dim)).astype(np.float32))
        gate = util.f32_to_bf16(rng.standard_normal(T).astype(np.float32) * 3)
        shared = util.f32_to_bf16(rng.standard_normal((T, dim)).astype(np.float32))
        for norm in (1, 0):
            want_c = np.empty((T, dim), np.uint16)
            oracle().orc_moe_combine(p(scores), p(y), p(gate), p(shared), T, k, dim, norm, p(want_c))
            bufs = [ctx.to_device(a) for a in (scores, y, gate, shared)]
            out = ctx.alloc(T * dim * 2)
            ctx.moe_combine(*bufs, T, k, dim, norm, out)
            assert np.array_equal(out.download(np.uint16, (T, dim)), want_c)
            for b in bufs + [out]: b.free()
    for b in (dg, du, do): b.free()


def _run_block(orn, ctx, moe, dw, xb, T):
    dx, dout = ctx.to_device(xb), ctx.alloc(T * moe.H * 2)
    di, ds = ctx.alloc(T * moe.top_k * 4), ctx.alloc(T * moe.top_k * 2)
    ctx.moe_block(dw, dx, T, dout, di, ds)
    r = (dout.download(np.uint16, (T, moe.H)), di.download(np.uint32, (T, moe.top_k)), ds.download(np.uint16, (T, moe.top_k)))
    for b in (dx, dout, di, ds): b.free()
    return r


def test_moe_block_config2_full_size(orn, ctx):
    """hidden 2048, 256 experts top-8, inter 512; gate/up Q4_K, down Q6_K; T in {1,2,4}."""
    rng = np.random.default_rng(42)
    moe = util.HostMoe(rng)
    dw = moe.dev(orn, ctx)
    x4 = util.f32_to_bf16(rng.standard_normal((4, 2048)).astype(np.float32))
    rows = {}
    for T in (1, 2, 4):
        xb = np.ascontiguousarray(x4[:T])
        want_out, want_inds, want_sc, _ = util.orc_moe_block(moe, xb, T)
        out, inds, sc = _run_block(orn, ctx, moe, dw, xb, T)
        assert np.array_equal(inds, want_inds), f"T={T}: expert indices differ"
        assert np.array_equal(sc, want_sc)
        assert np.array_equal(out, want_out), f"T={T}: output differs"
        rows[T] = out
        print(f"T={T}: distinct routed experts U={len(np.unique(inds))}")
    # batch invariance: row r of a wider call is that row alone
    assert np.array_equal(rows[4][:2], rows[2]) and np.array_equal(rows[2][:1], rows[1])
    moe.free()


def test_moe_block_small_all_q4k_and_all_q6k(orn, ctx):
    rng = np.random.default_rng(43)
    for gk, dk in ((Q4K, Q4K), (Q6K, Q6K)):
        moe = util.HostMoe(rng, H=512, E=64, I=256, top_k=8, gate_kind=gk, down_kind=dk, router_kind=gk)
        dw = moe.dev(orn, ctx)
        xb = util.f32_to_bf16(rng.standard_normal((3, 512)).astype(np.float32))
        want_out, want_inds, want_sc, _ = util.orc_moe_block(moe, xb, 3)
        out, inds, sc = _run_block(orn, ctx, moe, dw, xb, 3)
        assert np.array_equal(inds, want_inds) and np.array_equal(sc, want_sc) and np.array_equal(out, want_out)
        moe.free()
