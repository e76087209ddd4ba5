"""GPU parity: norms and the gated-delta pieces vs the oracle, bit for bit (bf16
activations by bits, fp32 state and decay by bits)."""
import numpy as np
import pytest

import util

pytestmark = pytest.mark.gpu


def test_norms_bit_exact(orn, ctx):
    rng = np.random.default_rng(0)
    for n in (64, 128, 256, 512, 1024, 2048, 4096):
        rows = 5
        x = util.bf16_normal(rng, (rows, n), 3.0); b = util.bf16_normal(rng, (rows, n)); w = util.bf16_normal(rng, (n,))
        z = util.bf16_normal(rng, (rows, n), 2.0)
        dx, db, dw, dz = (ctx.to_device(a) for a in (x, b, w, z))
        dh, do = ctx.alloc(x.nbytes), ctx.alloc(x.nbytes)
        ctx.rms_norm(dx, dw, rows, n, 1e-6, do)
        assert np.array_equal(do.download(np.uint16, x.shape), util.orc_rms_norm(x, w)), n
        ctx.rms_norm(dx, None, rows, n, 1e-6, do)
        assert np.array_equal(do.download(np.uint16, x.shape), util.orc_rms_norm(x, None)), n
        ctx.add_rms_norm(dx, db, dw, rows, n, 1e-6, dh, do)
        h, out = util.orc_add_rms_norm(x, b, w)
        assert np.array_equal(dh.download(np.uint16, x.shape), h) and np.array_equal(do.download(np.uint16, x.shape), out), n
        ctx.rms_norm_gated(dx, dw, dz, rows, n, 1e-6, do)
        assert np.array_equal(do.download(np.uint16, x.shape), util.orc_rms_norm_gated(x, w, z)), n
        for d in (dx, db, dw, dz, dh, do): d.free()


def _front(orn, ctx, i, T, Hk, Hv):
    D = 2 * Hk * 128 + Hv * 128
    names = ("conv_state", "qkv", "cw", "a", "b", "a_log", "dt_bias")
    d = {n: ctx.to_device(i[n]) for n in names}
    q, k = ctx.alloc(T * Hk * 256), ctx.alloc(T * Hk * 256)
    v, beta, g, ci = ctx.alloc(T * Hv * 256), ctx.alloc(T * Hv * 2), ctx.alloc(T * Hv * 4), ctx.alloc((3 + T) * D * 2)
    ctx.gdn_front(*(d[n] for n in names), T, 4, Hk, 128, Hv, 128, 1e-6, q, k, v, beta, g, ci)
    out = (q.download(np.uint16, (T, Hk, 128)), k.download(np.uint16, (T, Hk, 128)), v.download(np.uint16, (T, Hv, 128)),
           beta.download(np.uint16, (T, Hv)), g.download(np.float32, (T, Hv)), ci.download(np.uint16, (3 + T, D)))
    for b in list(d.values()) + [q, k, v, beta, g, ci]: b.free()
    return out


def _inputs(rng, T, Hk, Hv):
    D = 2 * Hk * 128 + Hv * 128
    return dict(conv_state=util.bf16_normal(rng, (3, D)), qkv=util.bf16_normal(rng, (T, D)),
                cw=util.bf16_normal(rng, (D, 4), 0.5), a=util.bf16_normal(rng, (T, Hv), 2.0),
                b=util.bf16_normal(rng, (T, Hv), 2.0), a_log=util.bf16_normal(rng, (Hv,), 0.5),
                dt_bias=util.bf16_normal(rng, (Hv,), 0.5))


# from 32 rows a call a workgroup takes a run of 16 tokens (same arithmetic): 32, a ragged 45, 100
@pytest.mark.parametrize("T,Hk,Hv", [(1, 16, 32), (2, 16, 32), (4, 16, 32), (3, 2, 4), (7, 1, 1), (32, 2, 4), (45, 2, 4),
                                     (100, 16, 32)])
def test_gdn_front_bit_exact(orn, ctx, T, Hk, Hv):
    rng = np.random.default_rng(10 + T + Hv)
    i = _inputs(rng, T, Hk, Hv)
    want = util.orc_gdn_front(i["conv_state"], i["qkv"], i["cw"], i["a"], i["b"], i["a_log"], i["dt_bias"], Hk, Hv)
    got = _front(orn, ctx, i, T, Hk, Hv)
    for name, gq, wq in zip(("q", "k", "v", "beta", "g", "conv_input"), got, want):
        assert np.array_equal(gq.view(np.uint32) if gq.dtype == np.float32 else gq,
                              wq.view(np.uint32) if wq.dtype == np.float32 else wq), name


def _rec(ctx, q, k, v, g, beta, state):
    T, Hk, _ = q.shape
    _, Hv, Dv = v.shape
    d = [ctx.to_device(a) for a in (q, k, v, g, beta, state)]
    y, snaps = ctx.alloc(T * Hv * Dv * 2), ctx.alloc(T * Hv * Dv * 128 * 4)
    ctx.gdn_recurrence(*d, T, Hk, Hv, 128, Dv, y, snaps)
    out = y.download(np.uint16, (T, Hv, Dv)), snaps.download(np.float32, (T, Hv, Dv, 128))
    for b in d + [y, snaps]: b.free()
    return out


def test_config3_verify_snapshots_and_rollback(orn, ctx):
    """BASELINE config 3: 16 key x 128 / 32 value x 128 heads, conv kernel 4, fp32 state
    [32,128,128] ~ N(0,0.1); T=2 verify tokens with per-token snapshots, then rollback of the
    rejected token must equal a forward over the one accepted token, bit for bit."""
    rng = np.random.default_rng(3)
    T, Hk, Hv = 2, 16, 32
    i = _inputs(rng, T, Hk, Hv)
    S0 = (rng.standard_normal((Hv, 128, 128)) * 0.1).astype(np.float32)
    q, k, v, beta, g, ci = _front(orn, ctx, i, T, Hk, Hv)
    y, snaps = _rec(ctx, q, k, v, g, beta, S0)
    wq, wk, wv, wbeta, wg, wci = util.orc_gdn_front(i["conv_state"], i["qkv"], i["cw"], i["a"], i["b"], i["a_log"], i["dt_bias"], Hk, Hv)
    wy, wsnaps = util.orc_gdn_recurrence(wq, wk, wv, wg, wbeta, S0)
    assert np.array_equal(y, wy) and np.array_equal(snaps.view(np.uint32), wsnaps.view(np.uint32))
    # rollback to keep = 1: conv state = rows [1, 4) of the window, state = snapshot 0
    keep = 1
    conv_after, state_after = ci[keep:keep + 3], snaps[keep - 1]
    # forward over the accepted token alone from the same start
    i1 = dict(i, qkv=i["qkv"][:1], a=i["a"][:1], b=i["b"][:1])
    q1, k1, v1, beta1, g1, ci1 = _front(orn, ctx, i1, 1, Hk, Hv)
    y1, snaps1 = _rec(ctx, q1, k1, v1, g1, beta1, S0)
    assert np.array_equal(y1[0], y[0])
    assert np.array_equal(ci1[1:4], conv_after)
    assert np.array_equal(snaps1[0].view(np.uint32), state_after.view(np.uint32))
    # and continuing from the rolled-back caches reproduces a fresh step on token 2
    i2 = dict(i, conv_state=np.ascontiguousarray(conv_after), qkv=i["qkv"][1:2], a=i["a"][1:2], b=i["b"][1:2])
    q2, k2, v2, beta2, g2, _ = _front(orn, ctx, i2, 1, Hk, Hv)
    y2, snaps2 = _rec(ctx, q2, k2, v2, g2, beta2, np.ascontiguousarray(state_after))
    assert np.array_equal(y2[0], y[1]) and np.array_equal(snaps2[0].view(np.uint32), snaps[1].view(np.uint32))


def test_recurrence_small_heads_and_in_place(orn, ctx):
    rng = np.random.default_rng(4)
    T, Hk, Hv = 4, 2, 4
    q = util.bf16_normal(rng, (T, Hk, 128), 0.1); k = util.bf16_normal(rng, (T, Hk, 128), 0.1)
    v = util.bf16_normal(rng, (T, Hv, 128)); beta = util.f32_to_bf16(rng.random((T, Hv)).astype(np.float32))
    g = rng.random((T, Hv)).astype(np.float32)
    S0 = (rng.standard_normal((Hv, 128, 128)) * 0.1).astype(np.float32)
    y, snaps = _rec(ctx, q, k, v, g, beta, S0)
    wy, wsnaps = util.orc_gdn_recurrence(q, k, v, g, beta, S0)
    assert np.array_equal(y, wy) and np.array_equal(snaps.view(np.uint32), wsnaps.view(np.uint32))
    # T == 1 with the snapshot written over the input state
    d = [ctx.to_device(a) for a in (q[:1], k[:1], v[:1], g[:1], beta[:1], S0)]
    yb = ctx.alloc(Hv * 128 * 2)
    ctx.gdn_recurrence(*d, 1, Hk, Hv, 128, 128, yb, d[5])
    assert np.array_equal(d[5].download(np.float32, S0.shape).view(np.uint32), wsnaps[0].view(np.uint32))
    for b in d + [yb]: b.free()


@pytest.mark.parametrize("T,Hk,Hv", [(32, 2, 4), (77, 2, 4), (130, 16, 32), (128, 2, 4), (257, 2, 4), (1000, 4, 8)])
def test_recurrence_at_prefill_width_close_to_exact(orn, ctx, T, Hk, Hv):
    """From 32 rows a call (only the final state wanted) the recurrence runs in its
    short-dependent-chain form, which sums in another order, and from 128 rows in 64-token
    chunks on the matrix cores: outputs within 0.5 % relative L2 of the oracle's exact
    recurrence per token, final state within 1e-4 relative L2."""
    rng = np.random.default_rng(T + Hv)
    q = util.bf16_normal(rng, (T, Hk, 128), 0.1); k = util.bf16_normal(rng, (T, Hk, 128), 0.1)
    v = util.bf16_normal(rng, (T, Hv, 128)); beta = util.f32_to_bf16(rng.random((T, Hv)).astype(np.float32))
    g = (0.9 + 0.1 * rng.random((T, Hv))).astype(np.float32)
    S0 = (rng.standard_normal((Hv, 128, 128)) * 0.1).astype(np.float32)
    wy, wsnaps = util.orc_gdn_recurrence(q, k, v, g, beta, S0)
    d = [ctx.to_device(a) for a in (q, k, v, g, beta, S0)]
    y, fin = ctx.alloc(T * Hv * 128 * 2), ctx.alloc(Hv * 128 * 128 * 4)
    ctx.gdn_recurrence(*d, T, Hk, Hv, 128, 128, y, fin, snap_all=False)
    gy = util.bf16_to_f32(y.download(np.uint16, (T, Hv, 128)))
    gs = fin.download(np.float32, (Hv, 128, 128))
    for b in d + [y, fin]: b.free()
    ry = util.bf16_to_f32(wy)
    err = np.linalg.norm((gy - ry).reshape(T, -1), axis=1) / (np.linalg.norm(ry.reshape(T, -1), axis=1) + 1e-30)
    assert err.max() < 5e-3, err.max()
    serr = np.linalg.norm(gs - wsnaps[-1]) / np.linalg.norm(wsnaps[-1])
    assert serr < 1e-4, serr


@pytest.mark.parametrize("T,decay", [(192, "wide"), (300, "tiny"), (500, "mixed")])
def test_chunked_recurrence_over_hard_decays(orn, ctx, T, decay):
    """The chunked form keeps its decays as differences of running log sums: decays far from one,
    decays that underflow to nothing (the state is forgotten mid-chunk) and beta = 0 / 1 rows
    must come out like the exact walk. Same bounds as above; and with the chunked form switched
    off the same call (the other prefill kernel) agrees with it too."""
    rng = np.random.default_rng(T)
    Hk, Hv = 2, 4
    q = util.bf16_normal(rng, (T, Hk, 128), 0.1); k = util.bf16_normal(rng, (T, Hk, 128), 0.1)
    v = util.bf16_normal(rng, (T, Hv, 128))
    beta = rng.random((T, Hv)).astype(np.float32)
    beta[rng.random((T, Hv)) < 0.1] = 0.0
    beta[rng.random((T, Hv)) < 0.1] = 1.0
    beta = util.f32_to_bf16(beta)
    if decay == "wide":
        g = (0.3 + 0.7 * rng.random((T, Hv))).astype(np.float32)
    elif decay == "tiny":
        g = (0.9 + 0.1 * rng.random((T, Hv))).astype(np.float32)
        g[rng.random((T, Hv)) < 0.03] = 1e-30
        g[7, 0] = 0.0
    else:
        g = np.exp(-np.exp(rng.normal(-3.0, 2.0, (T, Hv)))).astype(np.float32)
    S0 = (rng.standard_normal((Hv, 128, 128)) * 0.1).astype(np.float32)
    wy, wsnaps = util.orc_gdn_recurrence(q, k, v, g, beta, S0)
    ry = util.bf16_to_f32(wy)
    outs = {}
    for chunked in (1, 0):
        orn.set_option("gdn_chunked", chunked)
        d = [ctx.to_device(a) for a in (q, k, v, g, beta, S0)]
        y, fin = ctx.alloc(T * Hv * 128 * 2), ctx.alloc(Hv * 128 * 128 * 4)
        ctx.gdn_recurrence(*d, T, Hk, Hv, 128, 128, y, fin, snap_all=False)
        gy = util.bf16_to_f32(y.download(np.uint16, (T, Hv, 128)))
        gs = fin.download(np.float32, (Hv, 128, 128))
        for b in d + [y, fin]: b.free()
        assert np.all(np.isfinite(gy)) and np.all(np.isfinite(gs))
        err = np.linalg.norm((gy - ry).reshape(T, -1), axis=1) / (np.linalg.norm(ry.reshape(T, -1), axis=1) + 1e-30)
        assert err.max() < 5e-3, (chunked, err.max())
        serr = np.linalg.norm(gs - wsnaps[-1]) / np.linalg.norm(wsnaps[-1])
        assert serr < 1e-4, (chunked, serr)
        outs[chunked] = gy
    orn.set_option("gdn_chunked", 1)
    assert not np.array_equal(outs[0], outs[1])        # two different kernels did run


def test_chunked_recurrence_block_by_block_is_the_same_recurrence(orn, ctx):
    """Long calls of the chunked form go through the prepare / scan kernels in blocks of chunks
    with the state handed on: blocks of 2 chunks, of 3 (a ragged last block) and one block give
    the same outputs and final state bit for bit (a chunk's arithmetic does not depend on the
    block it is launched in)."""
    rng = np.random.default_rng(77)
    T, Hk, Hv = 531, 2, 4
    q = util.bf16_normal(rng, (T, Hk, 128), 0.1); k = util.bf16_normal(rng, (T, Hk, 128), 0.1)
    v = util.bf16_normal(rng, (T, Hv, 128))
    beta = util.f32_to_bf16(rng.random((T, Hv)).astype(np.float32))
    g = (0.9 + 0.1 * rng.random((T, Hv))).astype(np.float32)
    S0 = (rng.standard_normal((Hv, 128, 128)) * 0.1).astype(np.float32)
    outs = []
    try:
        for blk in (64, 2, 3):
            orn.set_option("gdn_block_chunks", blk)
            d = [ctx.to_device(a) for a in (q, k, v, g, beta, S0)]
            y, fin = ctx.alloc(T * Hv * 128 * 2), ctx.alloc(Hv * 128 * 128 * 4)
            ctx.gdn_recurrence(*d, T, Hk, Hv, 128, 128, y, fin, snap_all=False)
            outs.append((y.download(np.uint16, (T, Hv, 128)), fin.download(np.float32, (Hv, 128, 128))))
            for b in d + [y, fin]: b.free()
    finally:
        orn.set_option("gdn_block_chunks", 64)
    for gy, gs in outs[1:]:
        assert np.array_equal(gy, outs[0][0]) and np.array_equal(gs, outs[0][1])
