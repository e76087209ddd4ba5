"""Shared test plumbing: the CPU oracle (ctypes) and seeded synthetic inputs.

Only tests, the smoke check and the benchmark's cpu_baseline leg may load the
oracle; the shipped library never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_LIB = os.path.join(ORACLE_DIR, "liborc.so")

Q4K, Q6K = 0, 1
_orc = None


def oracle():
    global _orc
    if _orc is None:
        if not os.path.exists(ORACLE_LIB):
            subprocess.check_call(["make", "-s", "-C", ORACLE_DIR])
        _orc = C.CDLL(ORACLE_LIB)
        _orc.orc_tree64_export.restype = C.c_float
    return _orc


def p(a):
    return a.ctypes.data_as(C.c_void_p)


# ---- bf16 / f16 on the host ------------------------------------------------
def f32_to_bf16(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    out = np.empty(a.shape, dtype=np.uint16)
    oracle().orc_f32_to_bf16_n(p(a), p(out), C.c_int64(a.size))
    return out


def bf16_to_f32(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32)


def f16_to_f32(h):
    return np.ascontiguousarray(h, dtype=np.uint16).view(np.float16).astype(np.float32)


# ---- synthetic k-quant matrices -----------------------------------------------
def put_scale_min(sc, mn):
    """[...,8] scales and mins (0..63) -> [...,12] packed bytes, via the oracle's packer."""
    sc = np.ascontiguousarray(sc, dtype=np.uint8).reshape(-1, 8)
    mn = np.ascontiguousarray(mn, dtype=np.uint8).reshape(-1, 8)
    out = np.empty((sc.shape[0], 12), dtype=np.uint8)
    o = oracle()
    for i in range(sc.shape[0]):
        o.orc_q4k_put_scale_min(p(sc[i]), p(mn[i]), p(out[i]))
    return out


def put_scale_min_np(sc, mn):
    """Vectorised restatement of the 6-bit field packing (checked against the loop above)."""
    sc = np.asarray(sc, dtype=np.uint8)
    mn = np.asarray(mn, dtype=np.uint8)
    q = np.zeros(sc.shape[:-1] + (12,), dtype=np.uint8)
    q[..., 0:4] = (sc[..., 0:4] & 63) | ((sc[..., 4:8] >> 4) << 6)
    q[..., 4:8] = (mn[..., 0:4] & 63) | ((mn[..., 4:8] >> 4) << 6)
    q[..., 8:12] = (sc[..., 4:8] & 0xF) | ((mn[..., 4:8] & 0xF) << 4)
    return q


def make_q4k(rng, E, O, K, d_sigma=0.02, centered=False):
    """Q4_K tensors with fields drawn directly (BASELINE config 1):
    d, dmin = fp16(|N(0, d_sigma)|), 6-bit scale/min codes uniform, nibbles uniform.
    centered=True ties min to scale (m = sc, dmin = 7.5 d) so weights are zero-mean,
    which keeps activations of a deep random model in a sane range."""
    nb = K // 256
    n = E * O * nb
    qs = rng.integers(0, 256, size=(n, 128), dtype=np.uint8)
    sc = rng.integers(0, 64, size=(n, 8), dtype=np.uint8)
    d = np.abs(rng.normal(0.0, d_sigma, size=n)).astype(np.float32)
    if centered:
        mn = sc.copy()
        dmin = d * 7.5
    else:
        mn = rng.integers(0, 64, size=(n, 8), dtype=np.uint8)
        dmin = np.abs(rng.normal(0.0, d_sigma, size=n)).astype(np.float32)
    scales = put_scale_min_np(sc, mn)
    dm = np.stack([d, dmin], axis=1).astype(np.float16).view(np.uint16)
    return qs.reshape(E * O, nb * 128), scales.reshape(E * O, nb * 12), dm.reshape(E * O, nb * 2)


def make_q6k(rng, E, O, K, d_sigma=0.02 / 32):
    """Q6_K tensors: d = fp16(|N(0, d_sigma)|), int8 scales uniform -64..63, ql/qh bytes uniform
    (6-bit codes uniform 0..63)."""
    nb = K // 256
    n = E * O * nb
    w = rng.integers(0, 256, size=(n, 192), dtype=np.uint8)
    sc = rng.integers(-64, 64, size=(n, 16), dtype=np.int8).view(np.uint8)
    d = np.abs(rng.normal(0.0, d_sigma, size=n)).astype(np.float16).view(np.uint16)
    return w.reshape(E * O, nb * 192), sc.reshape(E * O, nb * 16), d.reshape(E * O, nb)


def make_kq(kind, rng, E, O, K, **kw):
    return make_q4k(rng, E, O, K, **kw) if kind == Q4K else make_q6k(rng, E, O, K, **kw)


# ---- oracle wrappers ---------------------------------------------------------
def orc_dequant(kind, qs, scales, dm, nblocks):
    out = np.empty(nblocks * 256, dtype=np.float32)
    f = oracle().orc_q4k_dequant if kind == Q4K else oracle().orc_q6k_dequant
    f(p(qs), p(scales), p(dm), C.c_int64(nblocks), p(out))
    return out


def orc_matvec_f64(kind, qs, scales, dm, O, K, x):
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, K)
    y = np.empty((x.shape[0], O), dtype=np.float64)
    oracle().orc_kq_matvec_f64(kind, p(qs), p(scales), p(dm), O, K, p(x), x.shape[0], p(y))
    return y


def orc_qmv(kind, qs, scales, dm, O, K, x, round_bf16=False):
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, K)
    y = np.empty((x.shape[0], O), dtype=np.float32)
    oracle().orc_kq_qmv(kind, p(qs), p(scales), p(dm), O, K, p(x), x.shape[0], p(y), int(round_bf16))
    return y


def orc_gather_qmv(kind, qs, scales, dm, E, O, K, x, lhs, rhs, round_bf16=False):
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, K)
    lhs = np.ascontiguousarray(lhs, dtype=np.uint32)
    rhs = np.ascontiguousarray(rhs, dtype=np.uint32)
    y = np.empty((len(rhs), O), dtype=np.float32)
    oracle().orc_kq_gather_qmv(kind, p(qs), p(scales), p(dm), E, O, K, p(x), p(lhs), p(rhs),
                               len(rhs), p(y), int(round_bf16))
    return y


def global_rel(got, want):
    """max|g-w| / max|w| -- the reference's compare (src/refs.rs:282-292)."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    return float(np.max(np.abs(got - want)) / max(np.max(np.abs(want)), 1e-300))
