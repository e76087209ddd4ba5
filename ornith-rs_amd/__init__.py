"""ctypes binding of libornith_hip.so (the C ABI in include/ornith_hip.h).

The directory name is not a Python identifier; import it with
``importlib.import_module("ornith-rs_amd")`` (tests/conftest.py does).

There is no CPU fallback: if the shared library is missing, loading raises, and
every operator raises ``OrnithError`` with the library's own message on failure.
Arrays cross the boundary as raw host buffers (numpy) and opaque device pointers.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libornith_hip.so")

F32, BF16 = 0, 1
Q4K, Q6K = 0, 1
KIND_NAMES = {Q4K: "q4k", Q6K: "q6k"}


class OrnithError(RuntimeError):
    pass


class KMatrixStruct(C.Structure):
    _fields_ = [("kind", C.c_int), ("E", C.c_int), ("O", C.c_int), ("K", C.c_int),
                ("d_qs", C.c_void_p), ("d_scales", C.c_void_p), ("d_dm", C.c_void_p)]


_lib = None


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise OrnithError(
                f"{LIB_PATH} is missing: build it with `python ornith-rs_amd/build.py` "
                "(there is no CPU fallback)")
        _lib = C.CDLL(LIB_PATH)
        _lib.ornith_last_error.restype = C.c_char_p
    return _lib


def _check(rc, what):
    if rc != 0:
        raise OrnithError(f"{what}: [{rc}] {lib().ornith_last_error().decode()}")


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


# ---- bf16 helpers on the host (numpy has no bf16; raw uint16 bits) ----------
def f32_to_bf16(a):
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def bf16_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


class DeviceBuffer:
    """A device allocation owned by a Ctx."""

    def __init__(self, ctx, nbytes):
        self.ctx, self.nbytes = ctx, int(nbytes)
        p = C.c_void_p()
        _check(lib().ornith_alloc(ctx.h, C.c_size_t(self.nbytes), C.byref(p)), "ornith_alloc")
        self.ptr = p

    def upload(self, arr):
        arr = np.ascontiguousarray(arr)
        assert arr.nbytes <= self.nbytes, (arr.nbytes, self.nbytes)
        _check(lib().ornith_upload(self.ctx.h, self.ptr, _ptr(arr), C.c_size_t(arr.nbytes)),
               "ornith_upload")
        return self

    def download(self, dtype, shape):
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes, (out.nbytes, self.nbytes)
        _check(lib().ornith_download(self.ctx.h, _ptr(out), self.ptr, C.c_size_t(out.nbytes)),
               "ornith_download")
        return out

    def zero(self):
        _check(lib().ornith_memset(self.ctx.h, self.ptr, 0, C.c_size_t(self.nbytes)), "ornith_memset")
        return self

    def free(self):
        if self.ptr:
            lib().ornith_free(self.ctx.h, self.ptr)
            self.ptr = None


class KMatrix:
    """Device-resident k-quant matrix: ops::kquant::KMatrix of the reference."""

    def __init__(self, ctx, kind, qs, scales, dm, E, O, K):
        self.ctx, self.kind, self.E, self.O, self.K = ctx, kind, E, O, K
        qs, scales, dm = (np.ascontiguousarray(t) for t in (qs, scales, dm))
        self.bufs = [ctx.to_device(t) for t in (qs, scales, dm)]
        self.s = KMatrixStruct(kind, E, O, K, self.bufs[0].ptr, self.bufs[1].ptr, self.bufs[2].ptr)
        _check(lib().ornith_kmatrix_check(C.byref(self.s), C.c_size_t(qs.nbytes),
                                          C.c_size_t(scales.nbytes), C.c_size_t(dm.nbytes)),
               "ornith_kmatrix_check")

    def free(self):
        for b in self.bufs:
            b.free()


class Ctx:
    def __init__(self, device=0):
        h = C.c_void_p()
        _check(lib().ornith_ctx_create(device, C.byref(h)), "ornith_ctx_create")
        self.h = h

    def close(self):
        if self.h:
            lib().ornith_ctx_destroy(self.h)
            self.h = None

    def sync(self):
        _check(lib().ornith_sync(self.h), "ornith_sync")

    def alloc(self, nbytes):
        return DeviceBuffer(self, nbytes)

    def to_device(self, arr):
        arr = np.ascontiguousarray(arr)
        return DeviceBuffer(self, max(arr.nbytes, 1)).upload(arr)

    def memset(self, dst, byte, nbytes):
        _check(lib().ornith_memset(self.h, dst.ptr, byte, C.c_size_t(nbytes)), "memset")

    def copy(self, dst, src, nbytes):
        _check(lib().ornith_copy(self.h, dst.ptr, src.ptr, nbytes), "copy")

    def device_info(self):
        name = C.create_string_buffer(256)
        cus, mem = C.c_int(), C.c_size_t()
        _check(lib().ornith_device_info(self.h, name, C.c_size_t(256), C.byref(cus), C.byref(mem)),
               "ornith_device_info")
        return name.value.decode(), cus.value, mem.value

    def timer_begin(self):
        _check(lib().ornith_timer_begin(self.h), "ornith_timer_begin")

    def timer_end(self):
        ms = C.c_float()
        _check(lib().ornith_timer_end(self.h, C.byref(ms)), "ornith_timer_end")
        return ms.value

    # ---- ops on device buffers -------------------------------------------
    def kq_dequantize(self, w, out, out_dtype):
        _check(lib().ornith_kq_dequantize(self.h, C.byref(w.s), out.ptr, out_dtype), "kq_dequantize")

    def kq_qmv(self, w, x, x_dtype, M, y, y_dtype):
        _check(lib().ornith_kq_qmv(self.h, C.byref(w.s), x.ptr, x_dtype, M, y.ptr, y_dtype), "kq_qmv")

    def kq_gather_qmv(self, w, x, x_dtype, x_rows, lhs, rhs, rows, y, y_dtype):
        _check(lib().ornith_kq_gather_qmv(self.h, C.byref(w.s), x.ptr, x_dtype, x_rows, lhs.ptr,
                                          rhs.ptr, rows, y.ptr, y_dtype), "kq_gather_qmv")

    def selftest_unary(self, fn, x):
        """Element-wise device scalar function (see ORNITH_FN_* in the header)."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        din, dout = self.to_device(x), self.alloc(max(x.nbytes, 4))
        _check(lib().ornith_selftest_unary(self.h, fn, din.ptr, dout.ptr, C.c_int64(x.size)),
               "selftest_unary")
        out = dout.download(np.float32, x.shape)
        din.free()
        dout.free()
        return out


FN_EXP, FN_LOG, FN_LOG1P, FN_SIGMOID_BF16, FN_SIGMOID_F32, FN_RSQRT, FN_RECIP, FN_ROUND_BF16, FN_WAVE_SUM = range(9)
FN_XOR_LANE = 9  # + i: value of lane l ^ 2**i, i = 0..5


# ---- Linear / MoE ---------------------------------------------------------------
LIN_KQUANT, LIN_AFFINE8, LIN_DENSE, LIN_AFFINE4 = 0, 1, 2, 3


class LinearStruct(C.Structure):
    _fields_ = [("mode", C.c_int), ("O", C.c_int), ("K", C.c_int), ("km", KMatrixStruct),
                ("d_w", C.c_void_p), ("d_scales", C.c_void_p), ("d_biases", C.c_void_p)]


class MoeWeightsStruct(C.Structure):
    _fields_ = [("router", LinearStruct), ("ex_gate", KMatrixStruct), ("ex_up", KMatrixStruct),
                ("ex_down", KMatrixStruct), ("sh_gate", LinearStruct), ("sh_up", LinearStruct),
                ("sh_down", LinearStruct), ("sh_egate", LinearStruct), ("top_k", C.c_int),
                ("norm_topk_prob", C.c_int), ("ex_dense", C.c_int), ("d_ex_gate", C.c_void_p),
                ("d_ex_up", C.c_void_p), ("d_ex_down", C.c_void_p)]


class Linear:
    """ops::linear::Linear on the device, from host tensors.

    kquant: Linear.kquant(ctx, kind, qs, scales, dm, O, K)
    affine: Linear.affine8(ctx, w_u8[O,K], scales_bf16[O,K/64], biases_bf16[O,K/64])
    dense:  Linear.dense(ctx, w_bf16[O,K])
    """

    def __init__(self, s, keep):
        self.s, self.keep = s, keep

    @staticmethod
    def kquant(ctx, kind, qs, scales, dm, O, K):
        km = KMatrix(ctx, kind, qs, scales, dm, 1, O, K)
        return Linear(LinearStruct(LIN_KQUANT, O, K, km.s, None, None, None), [km])

    @staticmethod
    def affine8(ctx, w, scales, biases):
        O, K = w.shape
        bufs = [ctx.to_device(t) for t in (w, scales, biases)]
        return Linear(LinearStruct(LIN_AFFINE8, O, K, KMatrixStruct(), bufs[0].ptr, bufs[1].ptr,
                                   bufs[2].ptr), bufs)

    @staticmethod
    def affine4(ctx, w, scales, biases):
        """w: u8 [O, K/2] (two 4-bit codes a byte, low nibble first); scales / biases bf16 [O, K/32]."""
        O, K = scales.shape[0], scales.shape[1] * 32
        bufs = [ctx.to_device(t) for t in (w, scales, biases)]
        return Linear(LinearStruct(LIN_AFFINE4, O, K, KMatrixStruct(), bufs[0].ptr, bufs[1].ptr,
                                   bufs[2].ptr), bufs)

    @staticmethod
    def dense(ctx, w):
        O, K = w.shape
        buf = ctx.to_device(w)
        return Linear(LinearStruct(LIN_DENSE, O, K, KMatrixStruct(), buf.ptr, None, None), [buf])

    def free(self):
        for b in self.keep:
            b.free()


def _ctx_method(fn):
    setattr(Ctx, fn.__name__, fn)
    return fn


@_ctx_method
def linear_matmul(self, lin, x, M, y):
    _check(lib().ornith_linear_matmul(self.h, C.byref(lin.s), x.ptr, M, y.ptr), "linear_matmul")


@_ctx_method
def linear_matmul_multi(self, lins, x, M, ys):
    """Several Linear over the same activations (one launch when their formats allow)."""
    n = len(lins)
    wp = (C.c_void_p * n)(*[C.cast(C.pointer(l.s), C.c_void_p) for l in lins])
    yp = (C.c_void_p * n)(*[y.ptr for y in ys])
    _check(lib().ornith_linear_matmul_multi(self.h, wp, n, x.ptr, M, yp), "linear_matmul_multi")


@_ctx_method
def dense_gather_mv(self, w, E, O, K, x, x_rows, lhs, rhs, rows, y):
    _check(lib().ornith_dense_gather_mv(self.h, w.ptr, E, O, K, x.ptr, x_rows, lhs.ptr, rhs.ptr,
                                        rows, y.ptr), "dense_gather_mv")


@_ctx_method
def affine4_gather_qmv(self, w, scales, biases, E, O, K, x, x_rows, lhs, rhs, rows, y):
    _check(lib().ornith_affine4_gather_qmv(self.h, w.ptr, scales.ptr, biases.ptr, E, O, K, x.ptr, x_rows, lhs.ptr,
                                           rhs.ptr, rows, y.ptr), "affine4_gather_qmv")


@_ctx_method
def embedding(self, table, ids, n, out):
    _check(lib().ornith_embedding(self.h, C.byref(table.s), ids.ptr, n, out.ptr), "embedding")


@_ctx_method
def router_topk(self, gates, T, E, k, inds, scores, probs=None):
    _check(lib().ornith_router_topk(self.h, gates.ptr, T, E, k, inds.ptr, scores.ptr,
                                    probs.ptr if probs else None), "router_topk")


@_ctx_method
def swiglu(self, gate, up, n, out):
    _check(lib().ornith_swiglu(self.h, gate.ptr, up.ptr, C.c_int64(n), out.ptr), "swiglu")


@_ctx_method
def moe_combine(self, scores, y, gate, shared, T, k, dim, normalize, out):
    _check(lib().ornith_moe_combine(self.h, scores.ptr, y.ptr, gate.ptr, shared.ptr, T, k, dim,
                                    int(normalize), out.ptr), "moe_combine")


@_ctx_method
def moe_block(self, w, x, T, out, inds=None, scores=None):
    _check(lib().ornith_moe_block(self.h, C.byref(w), x.ptr, T, out.ptr,
                                  inds.ptr if inds else None, scores.ptr if scores else None),
           "moe_block")


# ---- norms / gated-delta ----------------------------------------------------------
@_ctx_method
def rms_norm(self, x, w, rows, n, eps, out):
    _check(lib().ornith_rms_norm(self.h, x.ptr, w.ptr if w else None, rows, n, C.c_float(eps), out.ptr), "rms_norm")


@_ctx_method
def add_rms_norm(self, a, b, w, rows, n, eps, h_out, out):
    _check(lib().ornith_add_rms_norm(self.h, a.ptr, b.ptr, w.ptr if w else None, rows, n, C.c_float(eps),
                                     h_out.ptr, out.ptr), "add_rms_norm")


@_ctx_method
def rms_norm_gated(self, y, w, z, rows, n, eps, out):
    _check(lib().ornith_rms_norm_gated(self.h, y.ptr, w.ptr, z.ptr, rows, n, C.c_float(eps), out.ptr),
           "rms_norm_gated")


@_ctx_method
def gdn_front(self, conv_state, qkv, cw, a, b, a_log, dt_bias, T, K, Hk, Dk, Hv, Dv, eps, q, k, v, beta, g,
              conv_input):
    _check(lib().ornith_gdn_front(self.h, conv_state.ptr, qkv.ptr, cw.ptr, a.ptr, b.ptr, a_log.ptr,
                                  dt_bias.ptr, T, K, Hk, Dk, Hv, Dv, C.c_float(eps), q.ptr, k.ptr, v.ptr,
                                  beta.ptr, g.ptr, conv_input.ptr), "gdn_front")


@_ctx_method
def gdn_recurrence(self, q, k, v, g, beta, state_in, T, Hk, Hv, Dk, Dv, y, snapshots, snap_all=True):
    _check(lib().ornith_gdn_recurrence(self.h, q.ptr, k.ptr, v.ptr, g.ptr, beta.ptr, state_in.ptr, T, Hk, Hv,
                                       Dk, Dv, y.ptr, snapshots.ptr, int(snap_all)), "gdn_recurrence")


# ---- attention ---------------------------------------------------------------------
@_ctx_method
def rope_table(self, npos, dims, theta):
    half = dims // 2
    dc, ds = self.alloc(npos * half * 4), self.alloc(npos * half * 4)
    _check(lib().ornith_rope_table(self.h, npos, dims, C.c_double(theta), dc.ptr, ds.ptr), "rope_table")
    return dc, ds


@_ctx_method
def attn_prep(self, qg, kx, vx, qw, kw, T, Hq, Hkv, hd, rope_dims, eps, cos_t, sin_t, npos, offset, cap,
              q_rot, k_cache, v_cache, d_offset=None):
    _check(lib().ornith_attn_prep(self.h, qg.ptr, kx.ptr, vx.ptr, qw.ptr, kw.ptr, T, Hq, Hkv, hd, rope_dims,
                                  C.c_float(eps), cos_t.ptr, sin_t.ptr, npos, offset,
                                  d_offset.ptr if d_offset else None, cap, q_rot.ptr, k_cache.ptr,
                                  v_cache.ptr), "attn_prep")


@_ctx_method
def sdpa_decode_gated(self, q_rot, k_cache, v_cache, qg, T, Hq, Hkv, hd, offset, cap, scale, out,
                      d_offset=None):
    _check(lib().ornith_sdpa_decode_gated(self.h, q_rot.ptr, k_cache.ptr, v_cache.ptr, qg.ptr, T, Hq, Hkv, hd,
                                          offset, d_offset.ptr if d_offset else None, cap, C.c_float(scale),
                                          out.ptr), "sdpa_decode_gated")


@_ctx_method
def attn_decode(self, qg, kx, vx, qw, kw, T, Hq, Hkv, hd, rope_dims, eps, cos_t, sin_t, npos, offset, cap, scale,
                q_rot, k_cache, v_cache, out):
    """ornith_attn_decode: prep + attention of the same rows, one launch where the shape allows."""
    _check(lib().ornith_attn_decode(self.h, qg.ptr, kx.ptr, vx.ptr, qw.ptr, kw.ptr, T, Hq, Hkv, hd, rope_dims,
                                    C.c_float(eps), cos_t.ptr, sin_t.ptr, npos, offset, cap, C.c_float(scale),
                                    q_rot.ptr, k_cache.ptr, v_cache.ptr, out.ptr), "attn_decode")


# ---- greedy selection ----------------------------------------------------------------
@_ctx_method
def greedy_rows(self, logits, rows, V, tokens, lse=None):
    _check(lib().ornith_greedy_rows(self.h, logits.ptr, rows, V, tokens.ptr, lse.ptr if lse else None),
           "greedy_rows")


@_ctx_method
def greedy_rows_noalloc(self, logits, rows, V, tokens, lse=None):
    """greedy_rows with its partials in the library's fixed device array: allocates nothing."""
    _check(lib().ornith_greedy_rows_noalloc(self.h, logits.ptr, rows, V, tokens.ptr, lse.ptr if lse else None),
           "greedy_rows_noalloc")


@_ctx_method
def argmax_rows(self, logits, rows, V, out):
    _check(lib().ornith_argmax_rows(self.h, logits.ptr, rows, V, out.ptr), "argmax_rows")


from .engine import *  # noqa: E402,F401,F403  (engine objects: WeightStore, TextModel, ...)
from .engine import TextConfig, Sampler, MtpStats, WeightStore, Caches, TextModel, FrSpec, MtpHead, generate_step, generate_step_mtp, HISTORY_CYCLE, HISTORY_COMMITTED  # noqa: E402,F401
