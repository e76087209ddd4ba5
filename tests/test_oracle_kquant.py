"""Pins for the oracle's k-quant formats and mat-vecs (CPU only).

The reference's golden tensors (refs/) are not in its repository, so the oracle is
pinned by what the format and the mathematics fix -- each check below is chosen so
that one plausible mistake fails it (field packing, nibble interleave, the
subtracted minimum, the -32 bias, the signed scale, a transposed operand):
  * put/get of the 6-bit fields is the identity over all 64x64 values, and the
    oracle's loop packer agrees with a vectorised restatement;
  * a Q4_K block with every code equal to c dequantizes to d*sc*c - dmin*m
    (/root/reference/kernels/q4k.metal:24-26, 64-96);
  * elements i and i+32 of each 64 share a byte (low / high nibble);
  * Q6_K: codes packed by an independently written packer dequantize to
    d*sc*(code-32) with the scale of their 16-group (kernels/q6k.metal:15-17,47-77);
  * mat-vec vs float64 product <= 1e-5 global-rel (tests/q4k.rs:43,165-198),
    one-hot activation returns a dequantized column exactly (tests/q4k.rs:85-107),
    zero activations give exact zeros (:238-269), halving x halves y exactly,
    multi-row equals single-row bit for bit (:120-163), gather row equals the plain
    mat-vec on that expert's slice (:610-651).
"""
import ctypes as C

import numpy as np
import pytest

import util
from util import Q4K, Q6K, oracle, p


def test_scale_min_put_get_identity_all_values():
    o = oracle()
    sc = np.zeros(8, np.uint8)
    mn = np.zeros(8, np.uint8)
    q = np.zeros(12, np.uint8)
    s, m = C.c_uint8(), C.c_uint8()
    rng = np.random.default_rng(1)
    for a in range(64):
        for b in range(64):
            sc[:] = rng.integers(0, 64, 8)
            mn[:] = rng.integers(0, 64, 8)
            j = (a * 64 + b) % 8
            sc[j], mn[j] = a, b
            o.orc_q4k_put_scale_min(p(sc), p(mn), p(q))
            for jj in range(8):
                o.orc_q4k_get_scale_min(jj, p(q), C.byref(s), C.byref(m))
                assert (s.value, m.value) == (sc[jj], mn[jj])
            assert np.array_equal(util.put_scale_min_np(sc, mn), q)


def test_scale_min_layout_known_bytes():
    # hand-built: low four fields are plain 6-bit, high four split 4+2
    q = np.zeros(12, np.uint8)
    q[0] = 0b11_000001  # sc0 = 1, top bits of sc4 = 3
    q[4] = 0b10_000010  # m0 = 2, top bits of m4 = 2
    q[8] = 0x5A         # sc4 low = 0xA, m4 low = 0x5
    s, m = C.c_uint8(), C.c_uint8()
    oracle().orc_q4k_get_scale_min(0, p(q), C.byref(s), C.byref(m))
    assert (s.value, m.value) == (1, 2)
    oracle().orc_q4k_get_scale_min(4, p(q), C.byref(s), C.byref(m))
    assert (s.value, m.value) == (0xA | (3 << 4), 0x5 | (2 << 4))


def test_q4k_dequant_closed_form_constant_codes():
    rng = np.random.default_rng(2)
    for c in (0, 1, 7, 15):
        sc = rng.integers(0, 64, (1, 8)).astype(np.uint8)
        mn = rng.integers(0, 64, (1, 8)).astype(np.uint8)
        scales = util.put_scale_min(sc, mn)
        qs = np.full((1, 128), c | (c << 4), np.uint8)
        dm = np.array([[0.0123, 0.0456]], np.float16).view(np.uint16)
        got = util.orc_dequant(Q4K, qs, scales, dm, 1).reshape(8, 32)
        d, dmin = util.f16_to_f32(dm)[0]
        for j in range(8):
            want = np.float32(np.float32(d * np.float32(sc[0, j])) * np.float32(c)) - np.float32(dmin * np.float32(mn[0, j]))
            assert np.all(got[j] == np.float32(want)), (c, j)


def test_q4k_nibble_interleave_and_subtraction():
    # one byte set: low nibble lands at i, high nibble at i+32 of the same 64-group
    sc = np.full((1, 8), 1, np.uint8)
    mn = np.zeros((1, 8), np.uint8)
    scales = util.put_scale_min(sc, mn)
    dm = np.array([[1.0, 1.0]], np.float16).view(np.uint16)
    for byte in (0, 5, 31, 32, 77, 127):
        qs = np.zeros((1, 128), np.uint8)
        qs[0, byte] = 0xA3
        got = util.orc_dequant(Q4K, qs, scales, dm, 1)
        want = np.zeros(256, np.float32)
        g, l = divmod(byte, 32)
        want[64 * g + l] = 3
        want[64 * g + 32 + l] = 10
        assert np.array_equal(got, want), byte
    # the minimum is subtracted
    mn[:] = 2
    scales = util.put_scale_min(sc, mn)
    got = util.orc_dequant(Q4K, np.zeros((1, 128), np.uint8), scales, dm, 1)
    assert np.all(got == -2.0)


def test_q4k_pack_codes_roundtrip_bruteforce():
    rng = np.random.default_rng(3)
    codes = rng.integers(0, 16, 256).astype(np.uint8)
    qs = np.zeros(128, np.uint8)
    oracle().orc_q4k_pack_codes(p(codes), p(qs))
    sc = rng.integers(1, 64, (1, 8)).astype(np.uint8)
    mn = rng.integers(0, 64, (1, 8)).astype(np.uint8)
    dm = np.array([[0.5, 0.25]], np.float16).view(np.uint16)
    got = util.orc_dequant(Q4K, qs.reshape(1, -1), util.put_scale_min(sc, mn), dm, 1)
    want = (0.5 * sc[0].repeat(32) * codes.astype(np.float32) - 0.25 * mn[0].repeat(32)).astype(np.float32)
    assert np.array_equal(got, want)


def test_q6k_dequant_bruteforce_inverse():
    rng = np.random.default_rng(4)
    for _ in range(8):
        codes = rng.integers(0, 64, 256).astype(np.uint8)
        w = np.zeros(192, np.uint8)
        oracle().orc_q6k_pack_codes(p(codes), p(w))
        sc = rng.integers(-128, 128, 16).astype(np.int8)
        d = np.array([0.125], np.float16).view(np.uint16)
        got = util.orc_dequant(Q6K, w.reshape(1, -1), sc.view(np.uint8).reshape(1, -1), d.reshape(1, 1), 1)
        want = (0.125 * sc.astype(np.float32).repeat(16) * (codes.astype(np.float32) - 32)).astype(np.float32)
        assert np.array_equal(got, want)


def test_q6k_bias_and_sign_single_code():
    # code 0 -> -32, code 63 -> +31; negative scale flips the sign
    w = np.zeros(192, np.uint8)
    sc = np.full(16, -3, np.int8)
    d = np.array([1.0], np.float16).view(np.uint16)
    got = util.orc_dequant(Q6K, w.reshape(1, -1), sc.view(np.uint8).reshape(1, -1), d.reshape(1, 1), 1)
    assert np.all(got == 96.0)
    codes = np.full(256, 63, np.uint8)
    oracle().orc_q6k_pack_codes(p(codes), p(w))
    got = util.orc_dequant(Q6K, w.reshape(1, -1), sc.view(np.uint8).reshape(1, -1), d.reshape(1, 1), 1)
    assert np.all(got == -93.0)


@pytest.mark.parametrize("kind,K", [(Q4K, 2048), (Q4K, 512), (Q4K, 4096), (Q6K, 2048), (Q6K, 512), (Q6K, 4096)])
def test_matvec_vs_float64_and_invariants(kind, K):
    rng = np.random.default_rng(10 + kind + K)
    O = 64
    qs, sc, dm = util.make_kq(kind, rng, 1, O, K)
    x = rng.standard_normal((1, K)).astype(np.float32)
    y64 = util.orc_matvec_f64(kind, qs, sc, dm, O, K, x)
    y = util.orc_qmv(kind, qs, sc, dm, O, K, x)
    assert util.global_rel(y, y64) <= 1e-5
    # f64 yardstick itself == dequantized matrix @ x in numpy (guards a transposed operand)
    deq = util.orc_dequant(kind, qs, sc, dm, O * K // 256).reshape(O, K)
    assert np.allclose(y64[0], deq.astype(np.float64) @ x[0].astype(np.float64), rtol=1e-12, atol=1e-12)
    # zero row -> exact zeros; halving x halves y exactly
    assert np.all(util.orc_qmv(kind, qs, sc, dm, O, K, np.zeros((1, K), np.float32)) == 0.0)
    assert np.array_equal(util.orc_qmv(kind, qs, sc, dm, O, K, x * 0.5), y * 0.5)
    # one-hot -> a dequantized column, exactly
    for k in (0, 17, 255, K - 1):
        e = np.zeros((1, K), np.float32)
        e[0, k] = 1.0
        assert np.array_equal(util.orc_qmv(kind, qs, sc, dm, O, K, e)[0], deq[:, k]), k


@pytest.mark.parametrize("kind", [Q4K, Q6K])
def test_multirow_equals_single_row_and_gather_equals_slice(kind):
    rng = np.random.default_rng(20 + kind)
    E, O, K = 4, 32, 512
    qs, sc, dm = util.make_kq(kind, rng, E, O, K)
    x = rng.standard_normal((5, K)).astype(np.float32)
    for e in range(E):
        sl = slice(e * O, (e + 1) * O)
        ym = util.orc_qmv(kind, qs[sl], sc[sl], dm[sl], O, K, x)
        for r in range(5):
            assert np.array_equal(ym[r], util.orc_qmv(kind, qs[sl], sc[sl], dm[sl], O, K, x[r:r + 1])[0])
    lhs = np.array([0, 1, 1, 4, 2], np.uint32)
    rhs = np.array([3, 0, 2, 2, 1], np.uint32)
    yg = util.orc_gather_qmv(kind, qs, sc, dm, E, O, K, x, lhs, rhs)
    for r in range(5):
        sl = slice(int(rhs[r]) * O, (int(rhs[r]) + 1) * O)
        assert np.array_equal(yg[r], util.orc_qmv(kind, qs[sl], sc[sl], dm[sl], O, K, x[lhs[r]:lhs[r] + 1])[0])


def test_config1_shape_tolerance():
    """BASELINE config 1: 512x2048 Q4_K, x fp32 N(0,1); 1e-5 rel vs the float64 product."""
    rng = np.random.default_rng(2025)
    qs, sc, dm = util.make_q4k(rng, 1, 512, 2048)
    x = rng.standard_normal((1, 2048)).astype(np.float32)
    rel = util.global_rel(util.orc_qmv(Q4K, qs, sc, dm, 512, 2048, x),
                          util.orc_matvec_f64(Q4K, qs, sc, dm, 512, 2048, x))
    assert rel <= 1e-5
