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
AFFINE4 = 2   # stacked experts in the 4-bit affine group-32 format riding in a k-matrix descriptor
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
    """Round to nearest even, NaN -> quiet NaN (src/array.rs:229-237), in numpy: building
    inputs must not need the oracle's library (tests/test_oracle_math.py holds this against
    the oracle's own conversion)."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def orc_f32_to_bf16(a):
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


# ---- host-side model pieces: numpy tensors that feed both the oracle and the device ----
class OrcKmat(C.Structure):
    _fields_ = [("kind", C.c_int), ("E", C.c_int), ("O", C.c_int), ("K", C.c_int),
                ("qs", C.c_void_p), ("scales", C.c_void_p), ("dm", C.c_void_p)]


class OrcLinear(C.Structure):
    _fields_ = [("mode", C.c_int), ("km", OrcKmat), ("aw", C.c_void_p), ("as_", C.c_void_p),
                ("ab", C.c_void_p)]


class OrcMoeWeights(C.Structure):
    _fields_ = [("router", OrcLinear), ("ex_gate", OrcKmat), ("ex_up", OrcKmat), ("ex_down", OrcKmat),
                ("sh_gate", OrcLinear), ("sh_up", OrcLinear), ("sh_down", OrcLinear),
                ("sh_egate", OrcLinear), ("top_k", C.c_int), ("normalize", C.c_int)]


def unit_sigma(kind, K):
    """d-sigma that gives ~unit-variance outputs for N(0,1) inputs with centred weights."""
    return 1.0 / ((168.3 if kind == Q4K else 682.9) * np.sqrt(K))


class HostKMat:
    def __init__(self, kind, E, O, K, tensors):
        self.kind, self.E, self.O, self.K = kind, E, O, K
        self.qs, self.scales, self.dm = (np.ascontiguousarray(t) for t in tensors)

    @staticmethod
    def random(rng, kind, E, O, K, sigma=None):
        if kind == AFFINE4:
            # qs: codes two a byte (low nibble first); scales: bf16 scales; dm: bf16 biases, centred
            w = rng.integers(0, 256, size=(E, O, K // 2), dtype=np.uint8)
            s = (1.0 / (4.61 * np.sqrt(K))) * (0.5 + rng.random((E, O, K // 32)))
            scales = f32_to_bf16(s.astype(np.float32))
            biases = f32_to_bf16((-7.5 * bf16_to_f32(scales)).astype(np.float32))
            return HostKMat(kind, E, O, K, (w, scales, biases))
        sigma = unit_sigma(kind, K) if sigma is None else sigma
        t = make_q4k(rng, E, O, K, d_sigma=sigma, centered=True) if kind == Q4K else make_q6k(rng, E, O, K, d_sigma=sigma)
        return HostKMat(kind, E, O, K, t)

    def orc(self):
        return OrcKmat(self.kind, self.E, self.O, self.K, p(self.qs), p(self.scales), p(self.dm))

    def dev(self, orn, ctx):
        return orn.KMatrix(ctx, self.kind, self.qs, self.scales, self.dm, self.E, self.O, self.K)

    def nbytes(self):
        return self.qs.nbytes + self.scales.nbytes + self.dm.nbytes


class HostLinear:
    """mode: 'kq' (HostKMat), 'affine8' (w u8, scales bf16, biases bf16), 'dense' (w bf16)."""

    def __init__(self, mode, O, K, km=None, w=None, scales=None, biases=None):
        self.mode, self.O, self.K, self.km = mode, O, K, km
        self.w, self.scales, self.biases = w, scales, biases

    @staticmethod
    def kq(rng, kind, O, K, sigma=None):
        return HostLinear("kq", O, K, km=HostKMat.random(rng, kind, 1, O, K, sigma))

    @staticmethod
    def affine8(rng, O, K, out_std=1.0):
        w = rng.integers(0, 256, size=(O, K), dtype=np.uint8)
        # weight = s*q + b, centred: b = -127.5 s; std(q) = 73.9
        s = (out_std / (73.9 * np.sqrt(K))) * (0.5 + rng.random((O, K // 64)))
        scales = f32_to_bf16(s.astype(np.float32))
        biases = f32_to_bf16((-127.5 * bf16_to_f32(scales)).astype(np.float32))
        return HostLinear("affine8", O, K, w=w, scales=scales, biases=biases)

    @staticmethod
    def affine4(rng, O, K, out_std=1.0):
        """mlx affine 4-bit group 32: codes two a byte (low nibble first), weight = s*q + b,
        centred (b = -7.5 s; std(q) = 4.61)."""
        w = rng.integers(0, 256, size=(O, K // 2), dtype=np.uint8)
        s = (out_std / (4.61 * np.sqrt(K))) * (0.5 + rng.random((O, K // 32)))
        scales = f32_to_bf16(s.astype(np.float32))
        biases = f32_to_bf16((-7.5 * bf16_to_f32(scales)).astype(np.float32))
        return HostLinear("affine4", O, K, w=w, scales=scales, biases=biases)

    @staticmethod
    def dense(rng, O, K, out_std=1.0):
        w = f32_to_bf16((rng.standard_normal((O, K)) * (out_std / np.sqrt(K))).astype(np.float32))
        return HostLinear("dense", O, K, w=w)

    def orc(self):
        if self.mode == "kq":
            return OrcLinear(0, self.km.orc(), None, None, None)
        km = OrcKmat(0, 1, self.O, self.K, None, None, None)
        if self.mode == "affine8":
            return OrcLinear(1, km, p(self.w), p(self.scales), p(self.biases))
        if self.mode == "affine4":
            return OrcLinear(3, km, p(self.w), p(self.scales), p(self.biases))
        return OrcLinear(2, km, p(self.w), None, None)

    def dev(self, orn, ctx):
        if self.mode == "kq":
            return orn.Linear.kquant(ctx, self.km.kind, self.km.qs, self.km.scales, self.km.dm, self.O, self.K)
        if self.mode == "affine8":
            return orn.Linear.affine8(ctx, self.w, self.scales, self.biases)
        if self.mode == "affine4":
            return orn.Linear.affine4(ctx, self.w, self.scales, self.biases)
        return orn.Linear.dense(ctx, self.w)

    def nbytes(self):
        if self.mode == "kq":
            return self.km.nbytes()
        return sum(t.nbytes for t in (self.w, self.scales, self.biases) if t is not None)


class HostMoe:
    """One sparse MoE block's weights (BASELINE config 2 mix by default:
    routed gate/up Q4_K, down Q6_K, shared expert the same, router Q6_K, shared gate 8-bit)."""

    def __init__(self, rng, H=2048, E=256, I=512, top_k=8, gate_kind=Q4K, down_kind=Q6K, router_kind=Q6K):
        self.H, self.E, self.I, self.top_k = H, E, I, top_k
        if gate_kind == AFFINE4:
            # the published artifact's mix: 4-bit affine group 32 everywhere, the two gates 8-bit
            self.router = HostLinear.affine8(rng, E, H)
            self.ex_gate = HostKMat.random(rng, AFFINE4, E, I, H)
            self.ex_up = HostKMat.random(rng, AFFINE4, E, I, H)
            self.ex_down = HostKMat.random(rng, AFFINE4, E, H, I)
            self.sh_gate = HostLinear.affine4(rng, I, H)
            self.sh_up = HostLinear.affine4(rng, I, H)
            self.sh_down = HostLinear.affine4(rng, H, I)
            self.sh_egate = HostLinear.affine8(rng, 1, H)
            return
        self.router = HostLinear.kq(rng, router_kind, E, H)
        self.ex_gate = HostKMat.random(rng, gate_kind, E, I, H)
        self.ex_up = HostKMat.random(rng, gate_kind, E, I, H)
        self.ex_down = HostKMat.random(rng, down_kind, E, H, I)
        self.sh_gate = HostLinear.kq(rng, gate_kind, I, H)
        self.sh_up = HostLinear.kq(rng, gate_kind, I, H)
        self.sh_down = HostLinear.kq(rng, down_kind, H, I)
        self.sh_egate = HostLinear.affine8(rng, 1, H)

    def orc(self):
        return OrcMoeWeights(self.router.orc(), self.ex_gate.orc(), self.ex_up.orc(), self.ex_down.orc(),
                             self.sh_gate.orc(), self.sh_up.orc(), self.sh_down.orc(), self.sh_egate.orc(),
                             self.top_k, 1)

    def dev(self, orn, ctx):
        self._dev = [self.router.dev(orn, ctx), self.ex_gate.dev(orn, ctx), self.ex_up.dev(orn, ctx),
                     self.ex_down.dev(orn, ctx), self.sh_gate.dev(orn, ctx), self.sh_up.dev(orn, ctx),
                     self.sh_down.dev(orn, ctx), self.sh_egate.dev(orn, ctx)]
        d = self._dev
        return orn.MoeWeightsStruct(d[0].s, d[1].s, d[2].s, d[3].s, d[4].s, d[5].s, d[6].s, d[7].s,
                                    self.top_k, 1)

    def free(self):
        for d in getattr(self, "_dev", []):
            d.free()


def orc_moe_block(moe, xb, T):
    w = moe.orc()
    out = np.empty((T, moe.H), np.uint16)
    inds = np.empty((T, moe.top_k), np.uint32)
    scores = np.empty((T, moe.top_k), np.uint16)
    probs = np.empty((T, moe.E), np.uint16)
    oracle().orc_moe_block(C.byref(w), p(xb), T, p(out), p(inds), p(scores), p(probs))
    return out, inds, scores, probs


# ---- norms / gated-delta oracle wrappers ----------------------------------------------
def orc_rms_norm(x, w, eps=1e-6):
    rows, n = x.shape
    out = np.empty_like(x)
    oracle().orc_rms_norm(p(x), p(w) if w is not None else None, rows, n, C.c_float(eps), p(out))
    return out


def orc_add_rms_norm(a, b, w, eps=1e-6):
    rows, n = a.shape
    h, out = np.empty_like(a), np.empty_like(a)
    oracle().orc_add_rms_norm(p(a), p(b), p(w), rows, n, C.c_float(eps), p(h), p(out))
    return h, out


def orc_rms_norm_gated(y, w, z, eps=1e-6):
    rows, n = y.shape
    out = np.empty_like(y)
    oracle().orc_rms_norm_gated(p(y), p(w), p(z), rows, n, C.c_float(eps), p(out))
    return out


def orc_gdn_front(conv_state, qkv, cw, a, b, a_log, dt_bias, Hk, Hv, K=4, Dk=128, Dv=128, eps=1e-6):
    T, D = qkv.shape
    q = np.empty((T, Hk, Dk), np.uint16); k = np.empty((T, Hk, Dk), np.uint16)
    v = np.empty((T, Hv, Dv), np.uint16); beta = np.empty((T, Hv), np.uint16)
    g = np.empty((T, Hv), np.float32); ci = np.empty((K - 1 + T, D), np.uint16)
    oracle().orc_gdn_front(p(conv_state), p(qkv), p(cw), p(a), p(b), p(a_log), p(dt_bias), T, K, Hk, Dk, Hv, Dv,
                           C.c_float(eps), p(q), p(k), p(v), p(beta), p(g), p(ci))
    return q, k, v, beta, g, ci


def orc_gdn_recurrence(q, k, v, g, beta, state):
    T, Hk, Dk = q.shape
    _, Hv, Dv = v.shape
    y = np.empty((T, Hv, Dv), np.uint16)
    snaps = np.empty((T, Hv, Dv, Dk), np.float32)
    oracle().orc_gdn_recurrence(p(q), p(k), p(v), p(g), p(beta), p(np.ascontiguousarray(state)), T, Hk, Hv, Dk, Dv,
                                p(y), p(snaps))
    return y, snaps


def bf16_normal(rng, shape, std=1.0):
    return f32_to_bf16((rng.standard_normal(shape) * std).astype(np.float32))


# ---- attention oracle wrappers -------------------------------------------------------
def orc_rope_table(npos, dims, theta):
    half = dims // 2
    c = np.empty((npos, half), np.float32); s = np.empty((npos, half), np.float32)
    oracle().orc_rope_table(npos, dims, C.c_double(theta), p(c), p(s))
    return c, s


def orc_attn_prep(qg, kx, vx, qw, kw, rope_dims, cos_t, sin_t, offset, k_cache, v_cache, eps=1e-6):
    """Appends into k_cache / v_cache (numpy [Hkv, cap, hd]) in place; returns q_rot, gate."""
    T, Hq, hd2 = qg.shape
    hd = hd2 // 2
    Hkv, cap, _ = k_cache.shape
    q_rot = np.empty((T, Hq, hd), np.uint16); gate = np.empty((T, Hq, hd), np.uint16)
    oracle().orc_attn_prep(p(qg), p(kx), p(vx), p(qw), p(kw), T, Hq, Hkv, hd, rope_dims, C.c_float(eps),
                           p(cos_t), p(sin_t), offset, cap, p(q_rot), p(gate), p(k_cache), p(v_cache))
    return q_rot, gate


def orc_sdpa(q_rot, k_cache, v_cache, gate, offset, scale):
    T, Hq, hd = q_rot.shape
    Hkv, cap, _ = k_cache.shape
    out = np.empty((T, Hq * hd), np.uint16)
    oracle().orc_sdpa_decode_gated(p(q_rot), p(k_cache), p(v_cache), p(gate), T, Hq, Hkv, hd, offset, cap,
                                   C.c_float(scale), p(out))
    return out


# ---- sampler oracle wrappers -----------------------------------------------------------
def orc_threefry(key, count):
    k = (C.c_uint32 * 2)(*key); c = (C.c_uint32 * 2)(*count); o = (C.c_uint32 * 2)()
    oracle().orc_threefry2x32(k, c, o)
    return o[0], o[1]


def orc_random_bits(key, n):
    k = (C.c_uint32 * 2)(*key); out = np.empty(n, np.uint32)
    oracle().orc_random_bits(k, n, p(out))
    return out


def orc_key_next(state):
    st = (C.c_uint32 * 2)(*state); sub = (C.c_uint32 * 2)()
    oracle().orc_key_next(st, sub)
    return [st[0], st[1]], [sub[0], sub[1]]


def orc_uniform_scaled(bits, total):
    f = oracle().orc_uniform_scaled
    f.restype = C.c_float
    return np.float32(f(C.c_uint32(bits), C.c_float(total)))


def orc_argsort_bf16(x, negate=False):
    x = np.ascontiguousarray(x, np.uint16); idx = np.empty(x.size, np.uint32)
    oracle().orc_argsort_bf16(p(x), x.size, int(negate), p(idx))
    return idx


def orc_cumsum_bf16(x):
    x = np.ascontiguousarray(x, np.uint16); out = np.empty(x.size, np.uint16)
    oracle().orc_cumsum_bf16(p(x), x.size, p(out))
    return out


def orc_cumsum_f32(x):
    x = np.ascontiguousarray(x, np.float32); out = np.empty(x.size, np.float32)
    f = oracle().orc_cumsum_f32
    f.restype = C.c_float
    total = f(p(x), x.size, p(out))
    return out, np.float32(total)


def orc_logprobs_row(logits):
    logits = np.ascontiguousarray(logits, np.uint16); out = np.empty(logits.size, np.uint16)
    oracle().orc_logprobs_row(p(logits), logits.size, p(out))
    return out


def orc_apply_top_p(lp, top_p):
    lp = np.ascontiguousarray(lp, np.uint16); out = np.empty(lp.size, np.uint16)
    oracle().orc_apply_top_p(p(lp), lp.size, C.c_double(top_p), p(out))
    return out


def orc_apply_top_k(lp, k):
    lp = np.ascontiguousarray(lp, np.uint16); out = np.empty(lp.size, np.uint16)
    oracle().orc_apply_top_k(p(lp), lp.size, k, p(out))
    return out


def orc_categorical(lp, temp, bits):
    lp = np.ascontiguousarray(lp, np.uint16)
    f = oracle().orc_categorical
    f.restype = C.c_uint32
    return int(f(p(lp), lp.size, C.c_double(temp), C.c_uint32(bits)))


def orc_top_sample(logits, temp, top_p, top_k, key_state):
    logits = np.ascontiguousarray(logits, np.uint16)
    st = (C.c_uint32 * 2)(*key_state)
    f = oracle().orc_top_sample
    f.restype = C.c_uint32
    tok = int(f(p(logits), logits.size, C.c_double(temp), C.c_double(top_p), top_k, st))
    return tok, [st[0], st[1]]
