"""GPU: every fused launch structure gives the same bits as the one-launch-per-operator
path (the reference holds its own fusions to the same standard, e.g. tests/gdn.rs:176-230,
tests/q4k.rs:778-822), and as the oracle."""
import numpy as np
import pytest

import util
from util import Q4K, Q6K

pytestmark = pytest.mark.gpu


def _block(orn, ctx, moe, dw, xb, T):
    dx, dout = ctx.to_device(xb), ctx.alloc(T * moe.H * 2)
    di, ds = ctx.alloc(T * moe.top_k * 4), ctx.alloc(T * moe.top_k * 2)
    ctx.moe_block(dw, dx, T, dout, di, ds)
    r = (dout.download(np.uint16, (T, moe.H)), di.download(np.uint32, (T, moe.top_k)), ds.download(np.uint16, (T, moe.top_k)))
    for b in (dx, dout, di, ds): b.free()
    return r


@pytest.mark.parametrize("H,E,I,gk,dk", [(2048, 256, 512, Q4K, Q6K), (512, 64, 256, Q4K, Q6K),
                                          (512, 64, 256, Q6K, Q4K), (1024, 64, 512, Q4K, Q4K)])
def test_moe_fused_equals_unfused_and_oracle(orn, ctx, H, E, I, gk, dk):
    rng = np.random.default_rng(H + E + I + gk)
    moe = util.HostMoe(rng, H=H, E=E, I=I, top_k=8, gate_kind=gk, down_kind=dk, router_kind=Q6K)
    dw = moe.dev(orn, ctx)
    try:
        for T in (1, 2, 4, 7):
            xb = util.bf16_normal(rng, (T, H))
            orn.set_option("fuse_moe", 1)
            fused = _block(orn, ctx, moe, dw, xb, T)
            orn.set_option("fuse_moe", 0)
            plain = _block(orn, ctx, moe, dw, xb, T)
            for a, b in zip(fused, plain):
                assert np.array_equal(a, b), T
            if T <= 2:
                want_out, want_inds, want_sc, _ = util.orc_moe_block(moe, xb, T)
                assert np.array_equal(fused[1], want_inds) and np.array_equal(fused[0], want_out)
    finally:
        orn.set_option("fuse_moe", 1)
        moe.free()


@pytest.mark.parametrize("gk,dk,rk", [(Q4K, Q6K, Q6K), (Q4K, Q4K, Q4K), (Q6K, Q6K, Q6K)])
def test_moe_block_in_one_launch_equals_separate_launches(orn, ctx, gk, dk, rk):
    """The block's phases as workgroup ranges of one launch, handing gates / routing / expert
    activations over through memory inside the launch (option fuse_moe_one = 1: router + up +
    down, 2: up + down): same bits as the separate launches and as the oracle, T = 1..4, on the
    three format mixes the launch is instantiated for; repeated so that every call meets the
    flag words its predecessors left."""
    rng = np.random.default_rng(77 + gk + 2 * dk)
    moe = util.HostMoe(rng, H=2048, E=256, I=512, top_k=8, gate_kind=gk, down_kind=dk, router_kind=rk)
    dw = moe.dev(orn, ctx)
    try:
        for T in (1, 2, 3, 4, 2):
            xb = util.bf16_normal(rng, (T, 2048))
            orn.set_option("fuse_moe_one", 0)
            want = _block(orn, ctx, moe, dw, xb, T)
            for how in (1, 2, 1):
                orn.set_option("fuse_moe_one", how)
                got = _block(orn, ctx, moe, dw, xb, T)
                for a, b in zip(got, want):
                    assert np.array_equal(a, b), (T, how)
            if T == 2:
                want_out, want_inds, _, _ = util.orc_moe_block(moe, xb, T)
                assert np.array_equal(want[1], want_inds) and np.array_equal(want[0], want_out)
    finally:
        orn.set_option("fuse_moe_one", 0)
        moe.free()


def test_wait_inside_a_launch_gives_up_and_reports(orn, ctx):
    """A wait between workgroups is bounded: with the bound forced to one polling round from the
    host the consumers give up at once, every wavefront still exits, and the next
    synchronisation reports the failure; the following call (bound restored) is right again."""
    rng = np.random.default_rng(5)
    moe = util.HostMoe(rng, H=2048, E=256, I=512, top_k=8)
    dw = moe.dev(orn, ctx)
    T = 2
    xb = util.bf16_normal(rng, (T, 2048))
    try:
        orn.set_option("fuse_moe_one", 0)
        want = _block(orn, ctx, moe, dw, xb, T)
        orn.set_option("fuse_moe_one", 1)
        orn.set_option("ho_spins", 1)
        with pytest.raises(orn.OrnithError, match="ran out of its bound"):
            for _ in range(4):       # a single polling round can succeed by luck; four launches do not
                _block(orn, ctx, moe, dw, xb, T)
        orn.set_option("ho_spins", 1 << 20)
        got = _block(orn, ctx, moe, dw, xb, T)
        for a, b in zip(got, want):
            assert np.array_equal(a, b)
    finally:
        orn.set_option("ho_spins", 1 << 20)
        orn.set_option("fuse_moe_one", 0)
        moe.free()


# shapes that take the other lane-per-row widths of the two expert kernels: K = 256 (8 Q4_K / 4 Q6_K
# chunks a row), 1024, 2048 in either format, and the four-rows-a-wavefront form of the up kernel
@pytest.mark.parametrize("H,E,I,gk,dk,iters", [(2048, 256, 512, Q4K, Q6K, 0), (2048, 256, 512, Q4K, Q6K, 4),
                                                (256, 64, 256, Q4K, Q6K, 0), (256, 64, 256, Q6K, Q4K, 4),
                                                (1024, 64, 1024, Q6K, Q4K, 0), (2048, 64, 2048, Q6K, Q4K, 0),
                                                (512, 64, 256, Q4K, Q4K, 4), (4096, 64, 256, Q6K, Q4K, 0)])
def test_moe_experts_entry_equals_block(orn, ctx, H, E, I, gk, dk, iters):
    """ornith_moe_experts (the expert ids given: the launch bench.py times) gives the bits of
    ornith_moe_block, which makes the routing itself, and of the oracle."""
    rng = np.random.default_rng(H + E + I + gk + iters)
    moe = util.HostMoe(rng, H=H, E=E, I=I, top_k=8, gate_kind=gk, down_kind=dk, router_kind=gk)
    dw = moe.dev(orn, ctx)
    k = moe.top_k
    try:
        orn.set_option("moe_up_iters", iters)
        for T in (1, 2, 3, 4):
            xb = util.bf16_normal(rng, (T, H))
            want_out, want_inds, want_sc = _block(orn, ctx, moe, dw, xb, T)
            dx = ctx.to_device(xb)
            di, ds, de = ctx.to_device(want_inds), ctx.to_device(want_sc), ctx.alloc(T * 2)
            ctx.linear_matmul(moe._dev[7], dx, T, de)  # the shared expert's scalar gate
            act, out = ctx.alloc((T * k + T) * I * 2), ctx.alloc(T * H * 2)
            orn.moe_experts(ctx, dw, dx, T, di, ds, de, act, out, 1)
            orn.moe_experts(ctx, dw, dx, T, di, ds, de, act, out, 2)
            assert np.array_equal(out.download(np.uint16, (T, H)), want_out), T
            if T <= 2:
                assert np.array_equal(want_out, util.orc_moe_block(moe, xb, T)[0])
            for b in (dx, di, ds, de, act, out): b.free()
    finally:
        orn.set_option("moe_up_iters", 0)
        moe.free()


def test_multi_matrix_launch_equals_separate(orn, ctx):
    rng = np.random.default_rng(5)
    for kind, K in ((Q4K, 2048), (Q6K, 2048), (Q4K, 512), (Q4K, 4096)):
        Os = (8192, 4096, 40)
        ts = [util.make_kq(kind, rng, 1, O, K) for O in Os]
        ws = [orn.KMatrix(ctx, kind, *t, 1, O, K) for t, O in zip(ts, Os)]
        for M in (1, 2, 4):
            xb = util.bf16_normal(rng, (M, K))
            dx = ctx.to_device(xb)
            ys = [ctx.alloc(M * O * 2) for O in Os]
            orn.kq_qmv_multi(ctx, ws, dx, orn.BF16, M, ys, orn.BF16)
            for w, y, O in zip(ws, ys, Os):
                y1 = ctx.alloc(M * O * 2)
                ctx.kq_qmv(w, dx, orn.BF16, M, y1, orn.BF16)
                assert np.array_equal(y.download(np.uint16, (M, O)), y1.download(np.uint16, (M, O))), (kind, K, M, O)
                y1.free()
            for b in ys + [dx]: b.free()
        for w in ws: w.free()



def test_gdn_step_fused_equals_separate_launches(orn, ctx):
    """The gated-delta mixer core in one launch (a / b projections, front, recurrence with
    snapshots, gated norm) against the four separate launches: same hidden rows, and after a
    rewind the same continuation, for verify widths 1..4 and a 16-row prompt chunk."""
    import synth
    s = synth.SynthModel(synth.TINY, seed=21, with_mtp=False)
    ws = s.upload(orn, ctx)
    model = orn.TextModel(ctx, ws, s.text_config(orn))
    rng = np.random.default_rng(2)
    toks = rng.integers(0, s.cfg["vocab_size"], 40).astype(np.uint32)

    def run(fuse):
        orn.set_option("fuse_gdn", fuse)
        c = model.make_cache(64, 4)
        out = [model.forward(c, toks[:16])]
        pos = 16
        for T, keep in ((4, 2), (1, 1), (3, 3), (2, 1), (4, 4)):
            out.append(model.forward(c, toks[pos:pos + T], capture=True))
            model.rewind(c, keep)
            pos += keep
        out.append(model.forward(c, toks[pos:pos + 5]))
        c.close()
        return out

    try:
        a, b = run(1), run(0)
        for x, y in zip(a, b):
            assert np.array_equal(x, y)
    finally:
        orn.set_option("fuse_gdn", 1)
        model.close(); ws.close()


@pytest.mark.parametrize("kind,Os", [(Q4K, (8192, 4096)), (Q6K, (8192, 512, 512)), (Q4K, (40,))])
def test_norm_inside_projection_launch_equals_separate(orn, ctx, kind, Os):
    """add_rms_norm made inside the launch of the projections that read it (every workgroup
    recomputes it, one stores it) == add_rms_norm, then the projections: h, normed and every
    projection output, at M = 1..4, plus the M = 6 and fuse_norm = 0 fall-backs."""
    rng = np.random.default_rng(sum(Os) + kind)
    H = 2048
    lins = [orn.Linear.kquant(ctx, kind, *util.make_kq(kind, rng, 1, O, H), O, H) for O in Os]
    wn = ctx.to_device(util.bf16_normal(rng, (H,)))
    try:
        for M, fuse in ((1, 1), (2, 1), (3, 1), (4, 1), (6, 1), (2, 0), (2, 1)):
            orn.set_option("fuse_norm", fuse)
            res, y = ctx.to_device(util.bf16_normal(rng, (M, H))), ctx.to_device(util.bf16_normal(rng, (M, H)))
            h1, n1, h2, n2 = (ctx.alloc(M * H * 2) for _ in range(4))
            ys1 = [ctx.alloc(M * O * 2) for O in Os]
            ys2 = [ctx.alloc(M * O * 2) for O in Os]
            orn.add_rms_linear_multi(ctx, lins, res, y, wn, 1e-6, M, h1, n1, ys1)
            ctx.add_rms_norm(res, y, wn, M, H, 1e-6, h2, n2)
            for l, yy in zip(lins, ys2):
                ctx.linear_matmul(l, n2, M, yy)
            assert np.array_equal(h1.download(np.uint16, (M, H)), h2.download(np.uint16, (M, H))), (M, fuse)
            assert np.array_equal(n1.download(np.uint16, (M, H)), n2.download(np.uint16, (M, H))), (M, fuse)
            for a, b, O in zip(ys1, ys2, Os):
                assert np.array_equal(a.download(np.uint16, (M, O)), b.download(np.uint16, (M, O))), (M, fuse, O)
            for b in [res, y, h1, n1, h2, n2] + ys1 + ys2: b.free()
    finally:
        orn.set_option("fuse_norm", 1)
        wn.free()
        for l in lins: l.free()


def test_norm_inside_router_launch_equals_separate(orn, ctx):
    rng = np.random.default_rng(77)
    H = 2048
    moe = util.HostMoe(rng, H=H, E=256, I=512, top_k=8, gate_kind=Q4K, down_kind=Q6K, router_kind=Q6K)
    dw = moe.dev(orn, ctx)
    wn = ctx.to_device(util.bf16_normal(rng, (H,)))
    try:
        for T, fuse in ((1, 1), (2, 1), (4, 1), (7, 1), (2, 0)):
            orn.set_option("fuse_norm", fuse)
            res, y = ctx.to_device(util.bf16_normal(rng, (T, H))), ctx.to_device(util.bf16_normal(rng, (T, H)))
            h1, n1, o1, h2, n2, o2 = (ctx.alloc(T * H * 2) for _ in range(6))
            orn.add_rms_moe_block(ctx, dw, res, y, wn, 1e-6, T, h1, n1, o1)
            ctx.add_rms_norm(res, y, wn, T, H, 1e-6, h2, n2)
            ctx.moe_block(dw, n2, T, o2)
            for a, b in ((h1, h2), (n1, n2), (o1, o2)):
                assert np.array_equal(a.download(np.uint16, (T, H)), b.download(np.uint16, (T, H))), (T, fuse)
            for b in (res, y, h1, n1, o1, h2, n2, o2): b.free()
    finally:
        orn.set_option("fuse_norm", 1)
        wn.free(); moe.free()


@pytest.mark.parametrize("H,E,I,gk,dk", [(2048, 256, 512, Q4K, Q6K), (512, 64, 256, Q6K, Q4K)])
def test_expert_kernels_under_overlapping_routing(orn, ctx, H, E, I, gk, dk):
    """Verify rows of real text share experts. With routing that overlaps fully (every token on
    the same 8 experts), with the same experts in other slots, partly, and not at all: every
    (token, slot) row of the up launch equals that row computed alone (T = 1 with that expert),
    the block's output equals the per-token outputs, rows of one input on the same experts
    equal each other, and whole blocks (routing made in the launch) on duplicated input rows
    equal the oracle."""
    rng = np.random.default_rng(H + I)
    moe = util.HostMoe(rng, H=H, E=E, I=I, top_k=8, gate_kind=gk, down_kind=dk, router_kind=Q6K)
    dw = moe.dev(orn, ctx)
    k = 8
    try:
        for T in (2, 3, 4):
            base = rng.permutation(E)[:k].astype(np.uint32)
            others = [rng.permutation(E)[:k].astype(np.uint32) for _ in range(T)]
            part = np.stack(others)
            for t in range(1, T):       # tokens 1.. take three of token 0's experts, in other slots
                take = part[0, [5, 6, 7]]
                rest = np.array([e for e in part[t] if e not in set(take.tolist())], np.uint32)[:k - 3]
                part[t] = np.concatenate([take[::-1], rest]) if t % 2 else np.concatenate([rest, take])
            cases = {"none": np.stack(others), "full": np.stack([base] * T),
                     "rotated": np.stack([np.roll(base, t) for t in range(T)]), "partial": part}
            for inds in cases.values():
                for t in range(T):
                    assert len(set(inds[t].tolist())) == k
            xb = util.bf16_normal(rng, (T, H))
            xb[1] = xb[0]              # tokens 0 and 1 are the same input row
            scores = util.f32_to_bf16(rng.random((T, k)).astype(np.float32) + 0.1)
            eg = util.bf16_normal(rng, (T,))
            dx, ds, de = ctx.to_device(xb), ctx.to_device(scores), ctx.to_device(eg)
            act, out = ctx.alloc((T * k + T) * I * 2), ctx.alloc(T * H * 2)
            act1, out1 = ctx.alloc((k + 1) * I * 2), ctx.alloc(H * 2)
            for name, inds in cases.items():
                di = ctx.to_device(np.ascontiguousarray(inds, dtype=np.uint32))
                orn.moe_experts(ctx, dw, dx, T, di, ds, de, act, out, 3)
                a, o = act.download(np.uint16, (T * k + T, I)), out.download(np.uint16, (T, H))
                for t in range(T):     # the same token alone
                    d1 = [ctx.to_device(np.ascontiguousarray(v)) for v in (xb[t:t + 1], inds[t], scores[t], eg[t:t + 1])]
                    orn.moe_experts(ctx, dw, d1[0], 1, d1[1], d1[2], d1[3], act1, out1, 3)
                    a1 = act1.download(np.uint16, (k + 1, I))
                    assert np.array_equal(a[t * k:(t + 1) * k], a1[:k]) and np.array_equal(a[T * k + t], a1[k]), (T, name, t)
                    assert np.array_equal(o[t], out1.download(np.uint16, (H,))), (T, name, t)
                    for b in d1: b.free()
                if name == "full":
                    assert np.array_equal(a[0:k], a[k:2 * k]) and np.array_equal(a[T * k], a[T * k + 1])
                di.free()
            for b in (dx, ds, de, act, out, act1, out1): b.free()
            # whole blocks on duplicated rows (identical routing by construction) against the oracle
            xd = util.bf16_normal(rng, (T, H))
            xd[T - 1] = xd[0]
            want_out, want_inds, _, _ = util.orc_moe_block(moe, xd, T)
            got_out, got_inds, _ = _block(orn, ctx, moe, dw, xd, T)
            assert np.array_equal(got_inds, want_inds) and np.array_equal(got_inds[0], got_inds[T - 1])
            assert np.array_equal(got_out, want_out)
    finally:
        moe.free()
