"""Pins for the oracle's 4-bit affine (group 32) mat-vec and lookup, the published artifact's
format (src/ops/quantized.rs:311-333, vendored quantized.h:235-244): the nibble order against
mlx's packing stated as `(word >> 4*(i % 8)) & 15` on the u32 words, the product against
float64, and the gathered form against the plain one. CPU only."""
import ctypes as C

import numpy as np

import util
from util import oracle, p


def _dequant(lin):
    words = lin.w.view(np.uint32)                                    # [O, K/8], as the artifact stores it
    i = np.arange(lin.K)
    q = (words[:, i // 8] >> (4 * (i % 8)).astype(np.uint32)) & 15   # mlx: eight codes a word, lowest first
    s = np.repeat(util.bf16_to_f32(lin.scales).astype(np.float64), 32, 1)
    b = np.repeat(util.bf16_to_f32(lin.biases).astype(np.float64), 32, 1)
    return q.astype(np.float64) * s + b


def _qmv(lin, xb, lhs=None, rhs=None, E=1):
    rows = len(rhs) if rhs is not None else xb.shape[0]
    O = lin.O // E
    y = np.empty((rows, O), np.uint16)
    oracle().orc_affine4_gather_qmv(p(lin.w), p(lin.scales), p(lin.biases), E, O, lin.K, p(xb),
                                    p(lhs) if lhs is not None else None, p(rhs) if rhs is not None else None, rows, p(y))
    return y


def test_affine4_matvec_vs_float64_and_nibble_order():
    rng = np.random.default_rng(0)
    for O, K in ((6, 2048), (3, 32), (5, 4096), (2, 96)):
        lin = util.HostLinear.affine4(rng, O, K)
        W = _dequant(lin)
        xb = util.bf16_normal(rng, (3, K))
        want = util.bf16_to_f32(xb).astype(np.float64) @ W.T
        got = util.bf16_to_f32(_qmv(lin, xb)).astype(np.float64)
        assert np.all(np.abs(got - want) <= 2.0 ** -8 * np.abs(want) + 1e-5 * np.abs(want).max()), (O, K)
        # one-hot activations pick out single weights: every nibble position, both ends of a group
        for col in sorted(set(list(rng.integers(0, K, 24)) + [0, 1, 7, 8, 15, 16, 31, K - 1])):
            e = np.zeros((1, K), np.float32); e[0, col] = 1.0
            y = util.bf16_to_f32(_qmv(lin, util.f32_to_bf16(e)))[0].astype(np.float64)
            assert np.all(np.abs(y - W[:, col]) <= 2.0 ** -8 * np.abs(W[:, col]) + 1e-12), (K, col)


def test_affine4_gather_equals_plain_rows_and_embedding_vs_double():
    rng = np.random.default_rng(1)
    E, O, K = 5, 12, 256
    lin = util.HostLinear.affine4(rng, E * O, K)
    xb = util.bf16_normal(rng, (4, K))
    lhs = np.array([0, 3, 3, 1, 2, 0], np.uint32); rhs = np.array([4, 0, 2, 2, 1, 3], np.uint32)
    got = _qmv(lin, xb, lhs, rhs, E)
    full = _qmv(lin, xb)                                             # every expert's rows for every x row
    for r in range(len(rhs)):
        assert np.array_equal(got[r], full[lhs[r], rhs[r] * O:(rhs[r] + 1) * O])
    ids = np.array([7, 0, 59], np.uint32)
    out = np.empty((3, K), np.uint16)
    oracle().orc_embedding4(p(lin.w), p(lin.scales), p(lin.biases), K, p(ids), 3, p(out))
    W = _dequant(lin)
    bias = np.repeat(util.bf16_to_f32(lin.biases).astype(np.float64), 32, 1)
    assert np.all(np.abs(util.bf16_to_f32(out) - W[ids]) <= 2.0 ** -7 * np.abs(W[ids]) + 2.0 ** -8 * np.abs(bias[ids]))


def test_moe_block_with_4bit_affine_experts_matches_float64_composition():
    """The published artifact's MoE block (4-bit affine group-32 routed and shared experts, 8-bit
    router and shared gate; src/ops/moe.rs:662-741 over quantized::gather_qmv) against a float64
    restatement built from dequantized weights: same experts chosen where the cut is clear,
    output within bf16 tolerance."""
    rng = np.random.default_rng(6)
    H, E, I, k, T = 512, 64, 256, 8, 3
    moe = util.HostMoe(rng, H=H, E=E, I=I, top_k=k, gate_kind=util.AFFINE4)
    xb = util.f32_to_bf16(rng.standard_normal((T, H)).astype(np.float32))
    out, inds, scores, probs = util.orc_moe_block(moe, xb, T)
    x = util.bf16_to_f32(xb).astype(np.float64)

    def deq4(w, s, b, K):
        w = np.ascontiguousarray(w)
        words = w.view(np.uint32).reshape(-1, K // 8)
        i = np.arange(K)
        q = (words[:, i // 8] >> (4 * (i % 8)).astype(np.uint32)) & 15
        sc = np.repeat(util.bf16_to_f32(s).astype(np.float64).reshape(-1, K // 32), 32, 1)
        bi = np.repeat(util.bf16_to_f32(b).astype(np.float64).reshape(-1, K // 32), 32, 1)
        return q.astype(np.float64) * sc + bi

    def deq8(lin):
        return lin.w.astype(np.float64) * np.repeat(util.bf16_to_f32(lin.scales), 64, 1) + np.repeat(util.bf16_to_f32(lin.biases), 64, 1)

    Wg = deq4(moe.ex_gate.qs, moe.ex_gate.scales, moe.ex_gate.dm, H).reshape(E, I, H)
    Wu = deq4(moe.ex_up.qs, moe.ex_up.scales, moe.ex_up.dm, H).reshape(E, I, H)
    Wd = deq4(moe.ex_down.qs, moe.ex_down.scales, moe.ex_down.dm, I).reshape(E, H, I)
    Sg, Su, Sd = (deq4(l.w, l.scales, l.biases, l.K) for l in (moe.sh_gate, moe.sh_up, moe.sh_down))
    g = x @ deq8(moe.router).T
    pr = np.exp(g - g.max(1, keepdims=True)); pr /= pr.sum(1, keepdims=True)
    we = deq8(moe.sh_egate)[0]
    silu = lambda v: v / (1 + np.exp(-v))
    for t in range(T):
        srt = np.sort(pr[t])
        if srt[-k] - srt[-k - 1] > 2.0 ** -7 * srt[-k]:
            assert set(np.argsort(pr[t], kind="stable")[-k:]) == set(int(i) for i in inds[t])
        w = pr[t][inds[t].astype(int)]; w = w / w.sum()
        acc = np.zeros(H)
        for j, e in enumerate(inds[t].astype(int)):
            acc += w[j] * (Wd[e] @ (silu(Wg[e] @ x[t]) * (Wu[e] @ x[t])))
        want = acc + (Sd @ (silu(Sg @ x[t]) * (Su @ x[t]))) / (1 + np.exp(-(we @ x[t])))
        got = util.bf16_to_f32(out[t]).astype(np.float64)
        assert np.max(np.abs(got - want)) <= 0.03 * np.max(np.abs(want)), t
