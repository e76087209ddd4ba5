"""GPU parity: k-quant dequantize / mat-vec / gather mat-vec through the C ABI vs the oracle.

Integer and layout work is bit-exact; the fp32 mat-vec is bit-exact against the
oracle's canonical order and within 1e-5 global-rel of the float64 product (the
reference's own bound, tests/q4k.rs:43)."""
import numpy as np
import pytest

import util
from util import Q4K, Q6K

pytestmark = pytest.mark.gpu


def _dev_matrix(orn, ctx, kind, t, E, O, K):
    return orn.KMatrix(ctx, kind, t[0], t[1], t[2], E, O, K)


def test_device_scalar_functions_bit_exact(orn, ctx):
    import ctypes as C
    o = util.oracle()
    rng = np.random.default_rng(0)

    def host(fn, x):
        out = np.empty_like(x)
        fn(util.p(x), util.p(out), C.c_int64(x.size))
        return out

    x = np.concatenate([np.linspace(-90, 90, 200001), rng.normal(0, 5, 100000)]).astype(np.float32)
    assert np.array_equal(ctx.selftest_unary(orn.FN_EXP, x).view(np.uint32), host(o.orc_expf_n, x).view(np.uint32))
    xp = np.exp(rng.uniform(-80, 80, 300000)).astype(np.float32)
    assert np.array_equal(ctx.selftest_unary(orn.FN_LOG, xp).view(np.uint32), host(o.orc_logf_n, xp).view(np.uint32))
    u = np.exp(rng.uniform(-40, 3, 300000)).astype(np.float32)
    assert np.array_equal(ctx.selftest_unary(orn.FN_LOG1P, u).view(np.uint32), host(o.orc_log1pf_n, u).view(np.uint32))
    # division and sqrt are the correctly rounded IEEE ones
    assert np.array_equal(ctx.selftest_unary(orn.FN_RECIP, xp), (np.float32(1) / xp).astype(np.float32))
    assert np.array_equal(ctx.selftest_unary(orn.FN_RSQRT, xp), (np.float32(1) / np.sqrt(xp)).astype(np.float32))
    # bf16 sigmoid over every bf16 input
    bits = np.arange(65536, dtype=np.uint16)
    xb = util.bf16_to_f32(bits)
    fin = np.isfinite(xb)
    want = np.empty(65536, np.uint16)
    o.orc_sigmoid_bf16_n(util.p(bits), util.p(want), C.c_int64(65536))
    got = ctx.selftest_unary(orn.FN_SIGMOID_BF16, xb)
    assert np.array_equal(util.f32_to_bf16(got[fin]), want[fin])
    # rounding and the wavefront butterfly
    assert np.array_equal(util.f32_to_bf16(ctx.selftest_unary(orn.FN_ROUND_BF16, x)), util.f32_to_bf16(x))
    # ... over every exponent and upper mantissa, with the lower halves that decide rounding
    # (ties, just above / below, zero) and random ones: subnormals, infinities, both signs
    lows = np.concatenate([np.array([0, 1, 0x7fff, 0x8000, 0x8001, 0xffff], np.uint32),
                           rng.integers(0, 65536, 26).astype(np.uint32)])
    pat = ((np.arange(65536, dtype=np.uint32)[:, None] << 16) | lows[None, :]).reshape(-1)
    xf = pat.view(np.float32)
    ok = ~np.isnan(xf)
    got = ctx.selftest_unary(orn.FN_ROUND_BF16, xf)
    assert np.array_equal(got[ok].view(np.uint32) >> 16, util.f32_to_bf16(xf[ok]).astype(np.uint32))
    assert np.all((got[ok].view(np.uint32) & 0xffff) == 0) and np.all(np.isnan(got[~ok]))
    v = (rng.standard_normal(64 * 52) * 10.0 ** rng.integers(-3, 4, 64 * 52)).astype(np.float32)
    # the lane exchanges every reduction is built from: out[l] = in[l ^ 2**i]
    for i in range(6):
        got = ctx.selftest_unary(orn.FN_XOR_LANE + i, v).reshape(52, 64)
        assert np.array_equal(got.view(np.uint32), v.reshape(52, 64)[:, np.arange(64) ^ (1 << i)].view(np.uint32)), i
    got = ctx.selftest_unary(orn.FN_WAVE_SUM, v).reshape(52, 64)
    for i in range(52):
        want_s = o.orc_tree64_export(util.p(np.ascontiguousarray(v[64 * i:64 * i + 64])))
        assert np.all(got[i] == np.float32(want_s))


@pytest.mark.parametrize("kind", [Q4K, Q6K])
def test_dequantize_bit_exact(orn, ctx, kind):
    rng = np.random.default_rng(100 + kind)
    E, O, K = 2, 48, 1024
    t = util.make_kq(kind, rng, E, O, K)
    w = _dev_matrix(orn, ctx, kind, t, E, O, K)
    out = ctx.alloc(E * O * K * 4)
    ctx.kq_dequantize(w, out, orn.F32)
    got = out.download(np.float32, (E * O * K,))
    want = util.orc_dequant(kind, *t, E * O * K // 256)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    ctx.kq_dequantize(w, out, orn.BF16)
    assert np.array_equal(out.download(np.uint16, (E * O * K,)), util.f32_to_bf16(want))
    w.free(); out.free()


SHAPES = [(Q4K, 2048, 512), (Q4K, 512, 96), (Q4K, 4096, 200), (Q4K, 1024, 64), (Q4K, 256, 40),
          (Q6K, 2048, 256), (Q6K, 512, 2048), (Q6K, 4096, 130), (Q6K, 1024, 64), (Q6K, 8192, 32), (Q6K, 256, 24)]


@pytest.mark.parametrize("kind,K,O", SHAPES)
def test_qmv_bit_exact_vs_oracle_all_widths(orn, ctx, kind, K, O):
    rng = np.random.default_rng(200 + kind + K + O)
    t = util.make_kq(kind, rng, 1, O, K)
    w = _dev_matrix(orn, ctx, kind, t, 1, O, K)
    for M in (1, 2, 3, 4, 5, 8):
        x = rng.standard_normal((M, K)).astype(np.float32)
        want = util.orc_qmv(kind, *t, O, K, x)
        dx, dy = ctx.to_device(x), ctx.alloc(M * O * 4)
        ctx.kq_qmv(w, dx, orn.F32, M, dy, orn.F32)
        got = dy.download(np.float32, (M, O))
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (M,)
        assert util.global_rel(got, util.orc_matvec_f64(kind, *t, O, K, x)) <= 1e-5
        # bf16 activations in, bf16 out (the model's dtype)
        xb = util.f32_to_bf16(x)
        wantb = util.f32_to_bf16(util.orc_qmv(kind, *t, O, K, util.bf16_to_f32(xb)))
        dxb, dyb = ctx.to_device(xb), ctx.alloc(M * O * 2)
        ctx.kq_qmv(w, dxb, orn.BF16, M, dyb, orn.BF16)
        assert np.array_equal(dyb.download(np.uint16, (M, O)), wantb), (M, "bf16")
        for b in (dx, dy, dxb, dyb):
            b.free()
    w.free()


def test_config1_q4k_gemv_512x2048(orn, ctx):
    """BASELINE config 1 exactly: Q4_K 512x2048, x fp32 N(0,1) [1,2048] -> fp32 [1,512]."""
    rng = np.random.default_rng(2025)
    t = util.make_q4k(rng, 1, 512, 2048)
    x = rng.standard_normal((1, 2048)).astype(np.float32)
    w = _dev_matrix(orn, ctx, Q4K, t, 1, 512, 2048)
    dx, dy = ctx.to_device(x), ctx.alloc(512 * 4)
    ctx.kq_qmv(w, dx, orn.F32, 1, dy, orn.F32)
    got = dy.download(np.float32, (1, 512))
    y64 = util.orc_matvec_f64(Q4K, *t, 512, 2048, x)
    rel = util.global_rel(got, y64)
    print(f"config1: max_abs={np.max(np.abs(got - y64)):.3e} global_rel={rel:.3e}")
    assert rel <= 1e-5
    assert np.array_equal(got, util.orc_qmv(Q4K, *t, 512, 2048, x))
    # one-hot -> dequantized column exactly; zero row -> exact zeros
    deq = util.orc_dequant(Q4K, *t, 512 * 8).reshape(512, 2048)
    for k in (0, 33, 2047):
        e = np.zeros((1, 2048), np.float32); e[0, k] = 1.0
        dx.upload(e)
        ctx.kq_qmv(w, dx, orn.F32, 1, dy, orn.F32)
        assert np.array_equal(dy.download(np.float32, (512,)), deq[:, k])
    dx.upload(np.zeros((1, 2048), np.float32))
    ctx.kq_qmv(w, dx, orn.F32, 1, dy, orn.F32)
    assert np.all(dy.download(np.float32, (512,)) == 0.0)
    for b in (dx, dy): b.free()
    w.free()


@pytest.mark.parametrize("kind,K,O", [(Q4K, 2048, 512), (Q6K, 512, 2048), (Q6K, 2048, 64), (Q4K, 512, 128),
                                       (Q4K, 256, 64), (Q6K, 256, 64), (Q4K, 1024, 96), (Q6K, 1024, 96),
                                       (Q4K, 4096, 64), (Q6K, 4096, 64)])
def test_gather_qmv_bit_exact(orn, ctx, kind, K, O):
    rng = np.random.default_rng(300 + kind + K)
    E = 16
    t = util.make_kq(kind, rng, E, O, K)
    w = _dev_matrix(orn, ctx, kind, t, E, O, K)
    for T in (1, 2, 4):
        rows = 8 * T
        xb = util.f32_to_bf16(rng.standard_normal((T, K)).astype(np.float32))
        lhs = np.repeat(np.arange(T, dtype=np.uint32), 8)
        rhs = np.concatenate([rng.permutation(E)[:8] for _ in range(T)]).astype(np.uint32)
        want = util.orc_gather_qmv(kind, *t, E, O, K, util.bf16_to_f32(xb), lhs, rhs, round_bf16=True)
        dx, dl, dr, dy = ctx.to_device(xb), ctx.to_device(lhs), ctx.to_device(rhs), ctx.alloc(rows * O * 2)
        ctx.kq_gather_qmv(w, dx, orn.BF16, T, dl, dr, rows, dy, orn.BF16)
        got = dy.download(np.uint16, (rows, O))
        assert np.array_equal(got, util.f32_to_bf16(want)), T
        # indexed == plain mat-vec on the expert's slice (tests/q4k.rs:610-651)
        e = int(rhs[3]); sl = slice(e * O, (e + 1) * O)
        we = _dev_matrix(orn, ctx, kind, (t[0][sl], t[1][sl], t[2][sl]), 1, O, K)
        dy1 = ctx.alloc(O * 2)
        dx1 = ctx.to_device(xb[lhs[3]])
        ctx.kq_qmv(we, dx1, orn.BF16, 1, dy1, orn.BF16)
        assert np.array_equal(dy1.download(np.uint16, (O,)), got[3])
        # fp32 activations and fp32 outputs through the same gather
        xf = util.bf16_to_f32(xb)
        dxf, dyf = ctx.to_device(xf), ctx.alloc(rows * O * 4)
        ctx.kq_gather_qmv(w, dxf, orn.F32, T, dl, dr, rows, dyf, orn.F32)
        want32 = util.orc_gather_qmv(kind, *t, E, O, K, xf, lhs, rhs, round_bf16=False)
        assert np.array_equal(dyf.download(np.float32, (rows, O)).view(np.uint32), want32.view(np.uint32)), T
        for b in (dx, dl, dr, dy, dy1, dx1, dxf, dyf): b.free()
        we.free()
    w.free()


def test_errors_are_reported_not_fatal(orn, ctx):
    rng = np.random.default_rng(1)
    t = util.make_q4k(rng, 1, 8, 768)
    w = _dev_matrix(orn, ctx, Q4K, t, 1, 8, 768)  # 24 chunks: not a supported width
    dx, dy = ctx.alloc(768 * 4), ctx.alloc(8 * 4)
    with pytest.raises(orn.OrnithError, match="supported widths"):
        ctx.kq_qmv(w, dx, orn.F32, 1, dy, orn.F32)
    for b in (dx, dy): b.free()
    w.free()


def test_launch_sizing_never_changes_bits(orn, ctx):
    """The rows a wavefront walks (chosen by the launch from its kernel's residency, or forced
    through the kq_iters option) only shape the grid: every output bit stays the same, for the
    plain mat-vec and for the one that makes the layer's norm in its head, ragged row counts and
    several matrices a launch included."""
    import ctypes as C
    rng = np.random.default_rng(77)
    lib = orn.lib()
    try:
        for kind, K, Os in ((Q4K, 2048, (1000,)), (Q6K, 2048, (520, 36)), (Q4K, 4096, (300,)), (Q6K, 4096, (130,))):
            ts = [util.make_kq(kind, rng, 1, O, K) for O in Os]
            lins = [orn.Linear.kquant(ctx, kind, *t, O, K) for t, O in zip(ts, Os)]
            for M in (1, 2, 3, 4):
                x = util.bf16_normal(rng, (M, K))
                dx = ctx.to_device(x)
                ys = [ctx.alloc(M * O * 2) for O in Os]
                got = {}
                for it in (0, 1, 3, 8):
                    orn.set_option("kq_iters", it)
                    ctx.linear_matmul_multi(lins, dx, M, ys)
                    got[it] = [y.download(np.uint16, (M * O,)) for y, O in zip(ys, Os)]
                for it in (1, 3, 8):
                    for a, b in zip(got[0], got[it]):
                        assert np.array_equal(a, b), (kind, K, M, it)
                if K != 2048:
                    continue
                # norm in the head of the launch
                res, yv = util.bf16_normal(rng, (M, K)), util.bf16_normal(rng, (M, K))
                wn = ctx.to_device(util.bf16_normal(rng, (K,)))
                dres, dyv = ctx.to_device(res), ctx.to_device(yv)
                h, nm = ctx.alloc(M * K * 2), ctx.alloc(M * K * 2)
                n = len(Os)
                wp = (C.c_void_p * n)(*[C.cast(C.pointer(l.s), C.c_void_p) for l in lins])
                yp = (C.c_void_p * n)(*[y.ptr for y in ys])
                got = {}
                for it in (0, 1, 2, 5, 8):
                    orn.set_option("kq_iters", it)
                    rc = lib.ornith_add_rms_linear_multi(ctx.h, wp, n, dres.ptr, dyv.ptr, wn.ptr, C.c_float(1e-6), M,
                                                         h.ptr, nm.ptr, yp)
                    assert rc == 0
                    got[it] = [y.download(np.uint16, (M * O,)) for y, O in zip(ys, Os)] + \
                              [h.download(np.uint16, (M * K,)), nm.download(np.uint16, (M * K,))]
                for it in (1, 2, 5, 8):
                    for a, b in zip(got[0], got[it]):
                        assert np.array_equal(a, b), ("prenorm", kind, M, it)
    finally:
        orn.set_option("kq_iters", 0)
