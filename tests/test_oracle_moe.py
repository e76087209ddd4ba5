"""Pins for the oracle's MoE pieces (CPU only): each against a brute-force or
closed-form statement that does not share code with it."""
import ctypes as C

import numpy as np

import util
from util import oracle, p


def test_softmax_matches_double_and_sums_to_one():
    rng = np.random.default_rng(0)
    for n in (64, 256, 1024):
        g = util.f32_to_bf16((rng.standard_normal((5, n)) * 3).astype(np.float32))
        out = np.empty_like(g)
        oracle().orc_softmax_bf16(p(g), 5, n, p(out))
        gd = util.bf16_to_f32(g).astype(np.float64)
        want = np.exp(gd - gd.max(1, keepdims=True))
        want /= want.sum(1, keepdims=True)
        got = util.bf16_to_f32(out).astype(np.float64)
        assert np.all(np.abs(got - want) <= want * 2.0 ** -8 + 1e-30)
        assert np.all(np.abs(got.sum(1) - 1) < 2e-2)


def test_topk_is_tail_of_stable_ascending_sort_with_ties():
    rng = np.random.default_rng(1)
    n, k = 256, 8
    # few distinct values -> many ties, including at the cut
    vals = util.f32_to_bf16(rng.integers(0, 6, size=(50, n)).astype(np.float32) / 8)
    inds = np.empty((50, k), np.uint32)
    sc = np.empty((50, k), np.uint16)
    oracle().orc_router_topk(p(vals), 50, n, k, p(inds), p(sc))
    v = util.bf16_to_f32(vals)
    for r in range(50):
        order = np.argsort(v[r], kind="stable")  # equal values keep input order
        assert np.array_equal(inds[r], order[-k:].astype(np.uint32))
        assert np.array_equal(sc[r], vals[r][order[-k:]])


def test_swiglu_all_gate_values_close_to_double():
    bits = np.arange(65536, dtype=np.uint16)
    g = util.bf16_to_f32(bits)
    ok = np.isfinite(g) & (np.abs(g) < 1e30)
    up = util.f32_to_bf16(np.full(65536, 1.5, np.float32))
    out = np.empty(65536, np.uint16)
    oracle().orc_swiglu_bf16(p(bits), p(up), C.c_int64(65536), p(out))
    got = util.bf16_to_f32(out)[ok].astype(np.float64)
    gd = g[ok].astype(np.float64)
    with np.errstate(over="ignore"):
        want = gd / (1 + np.exp(-gd)) * 1.5
    # five bf16 roundings: a few bf16 ulps of the result, or of |g| where silu cancels
    tol = 2.0 ** -6 * np.maximum(np.abs(want), 1e-38) + 2.0 ** -7 * np.minimum(np.abs(gd), 1.0) * 1.5
    assert np.all(np.abs(got - want) <= tol)


def test_combine_closed_form_and_order():
    # powers of two keep every bf16 step exact, so the formula can be checked exactly
    T, k, dim = 2, 8, 4
    scores = util.f32_to_bf16(np.array([[0.125] * 8, [0.25, 0.25, 0.5, 0.5, 1, 1, 2, 2]], np.float32))
    y = util.f32_to_bf16(np.arange(T * k * dim, dtype=np.float32).reshape(T, k, dim) % 8)
    gate = util.f32_to_bf16(np.array([0.0, 0.0], np.float32))  # sigmoid = 0.5
    shared = util.f32_to_bf16(np.full((T, dim), 4.0, np.float32))
    out = np.empty((T, dim), np.uint16)
    oracle().orc_moe_combine(p(scores), p(y), p(gate), p(shared), T, k, dim, 1, p(out))
    s = util.bf16_to_f32(scores)
    yy = util.bf16_to_f32(y)
    want = (yy * (s / s.sum(1, keepdims=True))[:, :, None]).sum(1) + 2.0
    got = util.bf16_to_f32(out)
    assert np.allclose(got, want, rtol=2.0 ** -7)
    # bf16 accumulation is order dependent: 256 + 1 + 1 stays 256 in bf16 if the big term is first
    scores = util.f32_to_bf16(np.ones((1, 3), np.float32))
    gate = util.f32_to_bf16(np.array([-200.0], np.float32))  # sigmoid = 0
    shared = util.f32_to_bf16(np.zeros((1, 1), np.float32))
    for ys, want in (([256, 1, 1], 256.0), ([1, 1, 256], 258.0)):
        y = util.f32_to_bf16(np.array(ys, np.float32).reshape(1, 3, 1))
        out = np.empty((1, 1), np.uint16)
        oracle().orc_moe_combine(p(scores), p(y), p(gate), p(shared), 1, 3, 1, 0, p(out))
        assert util.bf16_to_f32(out)[0, 0] == want


def test_affine8_dense_embedding_vs_double():
    rng = np.random.default_rng(3)
    O, K = 6, 2048
    lin = util.HostLinear.affine8(rng, O, K)
    xb = util.f32_to_bf16(rng.standard_normal((2, K)).astype(np.float32))
    y = np.empty((2, O), np.uint16)
    oracle().orc_affine8_qmv(p(lin.w), p(lin.scales), p(lin.biases), O, K, p(xb), 2, p(y))
    wd = (lin.w.astype(np.float64) * np.repeat(util.bf16_to_f32(lin.scales), 64, 1) + np.repeat(util.bf16_to_f32(lin.biases), 64, 1))
    want = util.bf16_to_f32(xb).astype(np.float64) @ wd.T
    assert np.all(np.abs(util.bf16_to_f32(y) - want) <= 2.0 ** -8 * np.abs(want) + 1e-5)
    d = util.HostLinear.dense(rng, 16, 512)
    xb = util.f32_to_bf16(rng.standard_normal((3, 512)).astype(np.float32))
    y = np.empty((3, 16), np.uint16)
    oracle().orc_dense_gemv(p(d.w), 16, 512, p(xb), 3, p(y))
    want = util.bf16_to_f32(xb).astype(np.float64) @ util.bf16_to_f32(d.w).astype(np.float64).T
    assert np.all(np.abs(util.bf16_to_f32(y) - want) <= 2.0 ** -8 * np.abs(want) + 1e-5)
    ids = np.array([3, 0, 5], np.uint32)
    out = np.empty((3, K), np.uint16)
    oracle().orc_embedding(p(lin.w), p(lin.scales), p(lin.biases), K, p(ids), 3, p(out))
    assert np.all(np.abs(util.bf16_to_f32(out) - wd[ids]) <= 2.0 ** -7 * np.abs(wd[ids]) + 2.0 ** -8 * np.abs(np.repeat(util.bf16_to_f32(lin.biases), 64, 1)[ids]))


def test_moe_block_matches_numpy_float64_composition():
    """The whole block against a float64 restatement built from dequantized weights:
    same experts chosen (probabilities well separated), output within bf16 tolerance."""
    rng = np.random.default_rng(4)
    moe = util.HostMoe(rng, H=512, E=64, I=256, top_k=8)
    T = 3
    xb = util.f32_to_bf16(rng.standard_normal((T, 512)).astype(np.float32))
    out, inds, scores, probs = util.orc_moe_block(moe, xb, T)
    x = util.bf16_to_f32(xb).astype(np.float64)

    def deq(km):
        return util.orc_dequant(km.kind, km.qs, km.scales, km.dm, km.E * km.O * km.K // 256).reshape(km.E, km.O, km.K).astype(np.float64)

    Wr = deq(moe.router.km)[0]
    g = x @ Wr.T
    pr = np.exp(g - g.max(1, keepdims=True)); pr /= pr.sum(1, keepdims=True)
    Wg, Wu, Wd = deq(moe.ex_gate), deq(moe.ex_up), deq(moe.ex_down)
    Sg, Su, Sd = deq(moe.sh_gate.km)[0], deq(moe.sh_up.km)[0], deq(moe.sh_down.km)[0]
    we = (moe.sh_egate.w.astype(np.float64) * np.repeat(util.bf16_to_f32(moe.sh_egate.scales), 64, 1) + np.repeat(util.bf16_to_f32(moe.sh_egate.biases), 64, 1))[0]
    silu = lambda v: v / (1 + np.exp(-v))
    for t in range(T):
        top = np.argsort(pr[t], kind="stable")[-8:]
        # the bf16 rounding of probabilities can reorder near-equal ones; compare as sets
        # unless the k-th and (k+1)-th are within a bf16 ulp
        srt = np.sort(pr[t])
        if srt[-8] - srt[-9] > 2.0 ** -7 * srt[-8]:
            assert set(top) == set(int(i) for i in inds[t])
        w = pr[t][inds[t].astype(int)]; w = w / w.sum()
        acc = np.zeros(512)
        for j, e in enumerate(inds[t].astype(int)):
            a = silu(Wg[e] @ x[t]) * (Wu[e] @ x[t])
            acc += w[j] * (Wd[e] @ a)
        sh = Sd @ (silu(Sg @ x[t]) * (Su @ x[t]))
        want = acc + sh / (1 + np.exp(-(we @ x[t])))
        got = util.bf16_to_f32(out[t]).astype(np.float64)
        scale = np.max(np.abs(want))
        assert np.max(np.abs(got - want)) <= 0.03 * scale, (t, np.max(np.abs(got - want)), scale)


def test_dense_gather_mv_against_float64_and_its_index_roles():
    """out[r] = x[lhs[r]] . W[rhs[r]]^T over stacked bf16 experts: every row within one bf16 ulp
    of the float64 product of the row lhs names with the expert rhs names; with the two index
    lists exchanged (a transposed-operand mistake) the result must be far off."""
    rng = np.random.default_rng(11)
    E, O, K, X, R = 6, 24, 256, 4, 9
    w = util.f32_to_bf16(rng.standard_normal((E, O, K)).astype(np.float32))
    xb = util.f32_to_bf16(rng.standard_normal((X, K)).astype(np.float32))
    lhs = np.array([0, 1, 2, 3, 3, 2, 1, 0, 2], np.uint32)
    rhs = np.array([5, 4, 3, 2, 1, 0, 5, 3, 4], np.uint32)
    y = np.empty((R, O), np.uint16)
    oracle().orc_dense_gather_mv(p(w), O, K, p(xb), p(lhs), p(rhs), R, p(y))
    w64, x64 = util.bf16_to_f32(w).astype(np.float64), util.bf16_to_f32(xb).astype(np.float64)
    want = np.stack([w64[rhs[r]] @ x64[lhs[r]] for r in range(R)])
    got = util.bf16_to_f32(y).astype(np.float64)
    assert np.all(np.abs(got - want) <= 2.0 ** -8 * np.abs(want) + 1e-5)
    # the roles of the lists: lhs indexes activation rows (< X), rhs experts (< E)
    swapped = np.stack([w64[lhs[r]] @ x64[rhs[r] % X] for r in range(R)])
    assert np.max(np.abs(got - swapped)) > 1.0
    # and a gathered row is the plain mat-vec of that expert's slice on that activation row
    y1 = np.empty((1, O), np.uint16)
    oracle().orc_dense_gemv(p(np.ascontiguousarray(w[rhs[4]])), O, K, p(np.ascontiguousarray(xb[lhs[4]:lhs[4] + 1])), 1, p(y1))
    assert np.array_equal(y1[0], y[4])
