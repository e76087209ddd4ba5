"""Host-side mirror of the reference's engine objects over the C ABI:
WeightStore, TextModel (+ caches), FrSpec, MtpHead, generate_step, generate_step_mtp.
Names and argument meaning follow /root/reference/src/{weights,frspec,generate,
mtp_generate}.rs and src/model/{qwen3_5,mtp}.rs so tests read like the reference's."""
import ctypes as C
import os

import numpy as np

from . import (BF16, F32, LinearStruct, OrnithError, _check, _ptr, lib)

DT_F32, DT_BF16, DT_F16, DT_U8, DT_U32, DT_I32 = range(6)
DT_I8, DT_I16, DT_U16, DT_I64, DT_U64, DT_F64, DT_BOOL = range(6, 13)
DT_SIZE = {DT_F32: 4, DT_BF16: 2, DT_F16: 2, DT_U8: 1, DT_U32: 4, DT_I32: 4, DT_I8: 1, DT_I16: 2,
           DT_U16: 2, DT_I64: 8, DT_U64: 8, DT_F64: 8, DT_BOOL: 1}
QM_AFFINE, QM_Q4K, QM_Q6K = range(3)
HISTORY_CYCLE, HISTORY_COMMITTED = 0, 1
MAX_DEPTH = 8


def set_option(name, value):
    """ornith_set_option: 'fuse_moe', 'fuse_proj' (bit-identical either way)."""
    _check(lib().ornith_set_option(name.encode(), int(value)), f"set_option({name})")


def kq_qmv_multi(ctx, ws, x, x_dtype, M, ys, y_dtype):
    """Several k-quant mat-vecs over the same activations in one launch.
    ws: list of KMatrix, ys: list of DeviceBuffer."""
    n = len(ws)
    wp = (C.c_void_p * n)(*[C.cast(C.pointer(w.s), C.c_void_p) for w in ws])
    yp = (C.c_void_p * n)(*[y.ptr for y in ys])
    _check(lib().ornith_kq_qmv_multi(ctx.h, wp, n, x.ptr, x_dtype, M, yp, y_dtype), "kq_qmv_multi")


def moe_experts(ctx, w, x, T, inds, scores, egate, act, out, phases=3):
    """ornith_moe_experts: the two expert gather-GEMV kernels (1 = up, 2 = down, 3 = both)."""
    _check(lib().ornith_moe_experts(ctx.h, C.byref(w), x.ptr, T, inds.ptr, scores.ptr, egate.ptr, act.ptr,
                                    out.ptr, phases), "moe_experts")


class TextConfig(C.Structure):
    """TextConfig (src/model/config.rs); defaults are the Qwen3.5-35B-A3B shape."""
    _fields_ = [(n, C.c_int) for n in (
        "hidden_size", "num_hidden_layers", "vocab_size", "num_experts", "num_experts_per_tok",
        "moe_intermediate_size", "shared_expert_intermediate_size", "linear_num_key_heads",
        "linear_num_value_heads", "linear_key_head_dim", "linear_value_head_dim",
        "linear_conv_kernel_dim", "num_attention_heads", "num_key_value_heads", "head_dim",
        "rope_dims", "full_attention_interval", "norm_topk_prob")] + [
        ("rms_norm_eps", C.c_float), ("rope_theta", C.c_double)]

    @staticmethod
    def qwen35_35b_a3b(**over):
        d = dict(hidden_size=2048, num_hidden_layers=40, vocab_size=248320, num_experts=256,
                 num_experts_per_tok=8, moe_intermediate_size=512, shared_expert_intermediate_size=512,
                 linear_num_key_heads=16, linear_num_value_heads=32, linear_key_head_dim=128,
                 linear_value_head_dim=128, linear_conv_kernel_dim=4, num_attention_heads=16,
                 num_key_value_heads=2, head_dim=256, rope_dims=64, full_attention_interval=4,
                 norm_topk_prob=1, rms_norm_eps=1e-6, rope_theta=1e7)
        d.update(over)
        return TextConfig(**d)

    @staticmethod
    def load(model_dir):
        """TextConfig::load: (config, mtp_layers) from <model_dir>/config.json."""
        cfg, mtp = TextConfig(), C.c_int()
        _check(lib().ornith_text_config_load(os.fsencode(model_dir), C.byref(cfg), C.byref(mtp)),
               f"text_config_load({model_dir})")
        return cfg, mtp.value

    def key_dim(self):
        return self.linear_num_key_heads * self.linear_key_head_dim

    def value_dim(self):
        return self.linear_num_value_heads * self.linear_value_head_dim

    def conv_dim(self):
        return 2 * self.key_dim() + self.value_dim()

    def is_linear(self, i):
        return (i + 1) % self.full_attention_interval != 0


ACCEPT_EQUALITY, ACCEPT_RATIO = 0, 1
RNG_THREEFRY, RNG_PHILOX = 0, 1


class Sampler(C.Structure):
    """ornith_sampler: (kind, temperature, top_p, top_k, seed, accept, rng)."""
    _fields_ = [("kind", C.c_int), ("temperature", C.c_double), ("top_p", C.c_double),
                ("top_k", C.c_int), ("seed", C.c_uint64), ("accept", C.c_int), ("rng", C.c_int)]

    @staticmethod
    def greedy():
        return Sampler(0, 0.0, 1.0, 0, 0, 0, 0)


class MtpStats(C.Structure):
    _fields_ = [("cycles", C.c_size_t), ("drafted", C.c_size_t), ("accepted", C.c_size_t),
                ("reached_by_depth", C.c_size_t * MAX_DEPTH), ("accepted_by_depth", C.c_size_t * MAX_DEPTH)]


_NP_DT = {np.dtype(np.float32): DT_F32, np.dtype(np.float16): DT_F16, np.dtype(np.uint8): DT_U8,
          np.dtype(np.uint32): DT_U32, np.dtype(np.int32): DT_I32}

TOKEN_CB = C.CFUNCTYPE(C.c_int, C.c_uint32, C.c_void_p)
PROGRESS_CB = C.CFUNCTYPE(None, C.c_size_t, C.c_size_t, C.c_void_p)


class WeightStore:
    """WeightStore: named tensors on the device."""

    def put(self, name, arr, dtype=None):
        """dtype: DT_BF16 / DT_F16 for uint16 bit patterns; inferred otherwise."""
        arr = np.ascontiguousarray(arr)
        if dtype is None:
            dtype = _NP_DT[arr.dtype]
        shape = (C.c_int64 * arr.ndim)(*arr.shape)
        _check(lib().ornith_weights_put(self.h, name.encode(), dtype, shape, arr.ndim, _ptr(arr)),
               f"weights_put({name})")

    def __init__(self, ctx, _handle=None):
        self.ctx = ctx
        if _handle is None:
            _handle = C.c_void_p()
            _check(lib().ornith_weights_create(ctx.h, C.byref(_handle)), "weights_create")
        self.h = _handle

    @staticmethod
    def open(ctx, model_dir, extra=()):
        """WeightStore::open: the shards the index names plus `extra` files (the MTP sidecar)
        and config.json's quantization block; tensors reach the device on first use."""
        h = C.c_void_p()
        ex = (C.c_char_p * max(len(extra), 1))(*[os.fsencode(p) for p in extra])
        _check(lib().ornith_weights_open(ctx.h, os.fsencode(model_dir), ex, len(extra), C.byref(h)),
               f"weights_open({model_dir})")
        return WeightStore(ctx, h)

    def has(self, name):
        return bool(lib().ornith_weights_has(self.h, name.encode()))

    def quant_config(self, path):
        g, b, m = C.c_int(), C.c_int(), C.c_int()
        _check(lib().ornith_weights_quant_config(self.h, path.encode(), C.byref(g), C.byref(b),
                                                 C.byref(m)), f"quant_config({path})")
        return g.value, b.value, m.value

    def fetch(self, name):
        """(dtype code, shape, raw bytes as uint8) of a tensor, copied back from the device."""
        dt, nd = C.c_int(), C.c_int()
        shape = (C.c_int64 * 8)()
        fn = lib().ornith_weights_fetch
        fn.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                       C.c_size_t]
        _check(fn(self.h, name.encode(), C.byref(dt), shape, C.byref(nd), None, 0), f"fetch({name})")
        shp = tuple(shape[i] for i in range(nd.value))
        out = np.empty(int(np.prod(shp)) * DT_SIZE[dt.value], np.uint8)
        _check(fn(self.h, name.encode(), None, None, None, _ptr(out), out.nbytes), f"fetch({name})")
        return dt.value, shp, out

    def stats(self):
        n, b = C.c_int64(), C.c_int64()
        _check(lib().ornith_weights_stats(self.h, C.byref(n), C.byref(b)), "weights_stats")
        return n.value, b.value

    def close(self):
        if self.h:
            lib().ornith_weights_destroy(self.h)
            self.h = None


class SafeTensors:
    """SafeTensors::open_many / shards_from_index: mapped shards, host only."""

    def __init__(self, paths=None, model_dir=None, extra=()):
        h = C.c_void_p()
        if model_dir is not None:
            ex = (C.c_char_p * max(len(extra), 1))(*[os.fsencode(p) for p in extra])
            _check(lib().ornith_safetensors_open_model(os.fsencode(model_dir), ex, len(extra), C.byref(h)),
                   f"safetensors_open_model({model_dir})")
        else:
            ps = (C.c_char_p * max(len(paths), 1))(*[os.fsencode(p) for p in paths])
            _check(lib().ornith_safetensors_open(ps, len(paths), C.byref(h)), "safetensors_open")
        self.h = h

    def counts(self):
        n, f = C.c_int64(), C.c_int64()
        _check(lib().ornith_safetensors_count(self.h, C.byref(n), C.byref(f)), "safetensors_count")
        return n.value, f.value

    def names(self):
        out = []
        for i in range(self.counts()[0]):
            s = C.c_char_p()
            _check(lib().ornith_safetensors_name(self.h, C.c_int64(i), C.byref(s)), "safetensors_name")
            out.append(s.value.decode())
        return out

    def info(self, name):
        """(dtype code, shape, bytes as a uint8 copy)"""
        dt, nd, data, nb = C.c_int(), C.c_int(), C.c_void_p(), C.c_size_t()
        shape = (C.c_int64 * 8)()
        _check(lib().ornith_safetensors_info(self.h, name.encode(), C.byref(dt), shape, C.byref(nd),
                                             C.byref(data), C.byref(nb)), f"safetensors_info({name})")
        raw = np.frombuffer(C.string_at(data.value, nb.value), np.uint8) if nb.value else np.empty(0, np.uint8)
        return dt.value, tuple(shape[i] for i in range(nd.value)), raw

    def close(self):
        if self.h:
            lib().ornith_safetensors_close(self.h)
            self.h = None


def quant_config_load(model_dir, path):
    """(group_size, bits, mode) of a module from <model_dir>/config.json's quantization block."""
    g, b, m = C.c_int(), C.c_int(), C.c_int()
    _check(lib().ornith_quant_config_load(os.fsencode(model_dir), path.encode(), C.byref(g), C.byref(b),
                                          C.byref(m)), f"quant_config_load({path})")
    return g.value, b.value, m.value


class Caches:
    def __init__(self, model, capacity, max_window):
        self.model = model
        h = C.c_void_p()
        _check(lib().ornith_caches_create(model.h, capacity, max_window, C.byref(h)), "caches_create")
        self.h = h

    def reset(self):
        _check(lib().ornith_caches_reset(self.h), "caches_reset")

    def reserve(self, rows):
        """Grow the KV tensors now so that `rows` rows fit (they grow by themselves otherwise)."""
        _check(lib().ornith_caches_reserve(self.h, rows), "caches_reserve")

    def set_growable(self, growable):
        """False: the capacity is fixed; loops refuse up front what cannot fit."""
        _check(lib().ornith_caches_set_growable(self.h, int(growable)), "caches_set_growable")

    @property
    def capacity(self):
        o = C.c_int()
        _check(lib().ornith_caches_capacity(self.h, C.byref(o)), "caches_capacity")
        return o.value

    @property
    def offset(self):
        o = C.c_int()
        _check(lib().ornith_caches_offset(self.h, C.byref(o)), "caches_offset")
        return o.value

    def close(self):
        if self.h:
            lib().ornith_caches_destroy(self.h)
            self.h = None


class TextModel:
    """TextModel::load + forward_hidden / forward_capture / rewind."""

    def __init__(self, ctx, ws, cfg):
        self.ctx, self.ws, self.cfg = ctx, ws, cfg
        h = C.c_void_p()
        _check(lib().ornith_model_load(ctx.h, ws.h, C.byref(cfg), C.byref(h)), "model_load")
        self.h = h

    def make_cache(self, capacity, max_window=4):
        return Caches(self, capacity, max_window)

    def forward(self, caches, tokens, capture=False):
        """tokens: host uint32 array -> post-norm hidden rows as uint16 bf16 bits [T, H]."""
        tokens = np.ascontiguousarray(tokens, dtype=np.uint32)
        T, H = len(tokens), self.cfg.hidden_size
        dt, dh = self.ctx.to_device(tokens), self.ctx.alloc(T * H * 2)
        try:
            _check(lib().ornith_model_forward(self.h, caches.h, dt.ptr, T, int(capture), dh.ptr), "model_forward")
            return dh.download(np.uint16, (T, H))
        finally:
            dt.free()
            dh.free()

    def rewind(self, caches, keep):
        _check(lib().ornith_model_rewind(self.h, caches.h, keep), "model_rewind")

    def set_max_rows(self, rows):
        """Rows one forward call may carry (before creating caches); from 32 up the projections
        and experts run as matrix-core GEMMs."""
        _check(lib().ornith_model_set_max_rows(self.h, rows), "model_set_max_rows")

    def moe_weights(self, layer):
        """The resident MoE block of one decoder layer (valid while the model lives)."""
        from . import MoeWeightsStruct
        w = MoeWeightsStruct()
        _check(lib().ornith_model_moe_weights(self.h, layer, C.byref(w)), "model_moe_weights")
        return w

    def logits(self, hidden):
        hidden = np.ascontiguousarray(hidden, dtype=np.uint16)
        T, V = hidden.shape[0], self.cfg.vocab_size
        dh, dl = self.ctx.to_device(hidden), self.ctx.alloc(T * V * 2)
        try:
            _check(lib().ornith_model_logits(self.h, dh.ptr, T, dl.ptr), "model_logits")
            return dl.download(np.uint16, (T, V))
        finally:
            dh.free()
            dl.free()

    def close(self):
        if self.h:
            lib().ornith_model_destroy(self.h)
            self.h = None


class FrSpec:
    """FrSpec::load / from a list of ids; holds the pruned head."""

    def __init__(self, model, ids=None, path=None):
        """ids: the list itself; path: a list file; neither: the default location
        (frspec::default_path: $ORNITH_FRSPEC, else <refs>/frspec/ids_64k.bin)."""
        self.model = model
        h = C.c_void_p()
        if path is not None or ids is None:
            _check(lib().ornith_frspec_load(model.h, str(path).encode() if path is not None else None, C.byref(h)),
                   "frspec_load")
        else:
            ids = np.ascontiguousarray(ids, dtype=np.uint32)
            _check(lib().ornith_frspec_from_ids(model.h, _ptr(ids), len(ids), C.byref(h)), "frspec_from_ids")
        self.h = h

    def head(self):
        s, n = LinearStruct(), C.c_int()
        _check(lib().ornith_frspec_head(self.h, C.byref(s), C.byref(n)), "frspec_head")
        return s, n.value

    def close(self):
        if self.h:
            lib().ornith_frspec_destroy(self.h)
            self.h = None


class MtpHead:
    def __init__(self, model, ws, capacity):
        self.model = model
        h = C.c_void_p()
        _check(lib().ornith_mtp_load(model.h, ws.h, capacity, C.byref(h)), "mtp_load")
        self.h = h

    def forward(self, trunk_hidden, next_ids, frspec=None, want_logits=True):
        ctx, cfg = self.model.ctx, self.model.cfg
        trunk_hidden = np.ascontiguousarray(trunk_hidden, dtype=np.uint16)
        next_ids = np.ascontiguousarray(next_ids, dtype=np.uint32)
        T, H = len(next_ids), cfg.hidden_size
        V = frspec.head()[1] if frspec else cfg.vocab_size
        dh, di, do = ctx.to_device(trunk_hidden), ctx.to_device(next_ids), ctx.alloc(T * H * 2)
        dl = ctx.alloc(T * V * 2) if want_logits else None
        try:
            _check(lib().ornith_mtp_forward(self.h, frspec.h if frspec else None, dh.ptr, di.ptr, T, do.ptr,
                                            dl.ptr if dl else None), "mtp_forward")
            hid = do.download(np.uint16, (T, H))
            return (dl.download(np.uint16, (T, V)) if dl else None), hid
        finally:
            for b in (dh, di, do, dl):
                if b:
                    b.free()

    def set_growable(self, growable):
        """False: the head's cache keeps its capacity; a run that cannot fit is refused."""
        _check(lib().ornith_mtp_cache_set_growable(self.h, int(growable)), "mtp_cache_set_growable")

    def reserve(self, rows):
        _check(lib().ornith_mtp_cache_reserve(self.h, rows), "mtp_cache_reserve")

    def set_offset(self, off):
        _check(lib().ornith_mtp_cache_set_offset(self.h, off), "mtp_cache_set_offset")

    def force_drafts(self, tokens):
        """Measurement aid (not in the reference): the drafts of generate_step_mtp are replaced
        by tokens[p] for output position p, so every one is accepted when `tokens` is the
        run's own output. An empty list clears it."""
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        _check(lib().ornith_mtp_force_drafts(self.h, _ptr(t) if len(t) else None, C.c_size_t(len(t))),
               "mtp_force_drafts")

    @property
    def offset(self):
        o = C.c_int()
        _check(lib().ornith_mtp_cache_offset(self.h, C.byref(o)), "mtp_cache_offset")
        return o.value

    def close(self):
        if self.h:
            lib().ornith_mtp_destroy(self.h)
            self.h = None


def generate_step(model, caches, prompt, max_tokens, sampler=None, prefill_step=2048, on_token=None,
                  progress=None):
    """generate::generate_step. Returns the emitted tokens (also handed to on_token one by one;
    on_token returning False stops)."""
    prompt = np.ascontiguousarray(prompt, dtype=np.uint32)
    sampler = sampler or Sampler.greedy()
    out = []

    def _tok(t, _u):
        out.append(int(t))
        return 1 if (on_token is None or on_token(int(t))) else 0

    cb = TOKEN_CB(_tok)
    pcb = PROGRESS_CB((lambda d, t, _u: progress(d, t)) if progress else (lambda d, t, _u: None))
    _check(lib().ornith_generate(model.h, caches.h, _ptr(prompt), C.c_size_t(len(prompt)), C.byref(sampler),
                                 C.c_size_t(max_tokens), C.c_size_t(prefill_step), pcb, cb, None), "generate")
    return out


def generate_step_mtp(model, head, frspec, caches, prompt, depth, max_tokens, sampler=None,
                      prefill_step=2048, policy=HISTORY_COMMITTED, on_token=None, progress=None):
    """mtp_generate::generate_step_mtp. Returns (tokens, MtpStats)."""
    prompt = np.ascontiguousarray(prompt, dtype=np.uint32)
    sampler = sampler or Sampler.greedy()
    out, stats = [], MtpStats()

    def _tok(t, _u):
        out.append(int(t))
        return 1 if (on_token is None or on_token(int(t))) else 0

    cb = TOKEN_CB(_tok)
    pcb = PROGRESS_CB((lambda d, t, _u: progress(d, t)) if progress else (lambda d, t, _u: None))
    _check(lib().ornith_mtp_generate(model.h, head.h, frspec.h if frspec else None, caches.h, _ptr(prompt),
                                     C.c_size_t(len(prompt)), C.byref(sampler), depth, C.c_size_t(max_tokens),
                                     C.c_size_t(prefill_step), policy, pcb, cb, None, C.byref(stats)),
           "mtp_generate")
    return out, stats


# ---- the sampled-token path (src/sample.rs, src/ops/random.rs) ----------------------------
def random_key(seed):
    k = (C.c_uint32 * 2)()
    lib().ornith_random_key(C.c_uint64(seed), k)
    return [k[0], k[1]]


def random_split(state):
    """KeySequence::next: returns (new_state, sub_key)."""
    st = (C.c_uint32 * 2)(*state)
    sub = (C.c_uint32 * 2)()
    _check(lib().ornith_random_split(st, sub), "random_split")
    return [st[0], st[1]], [sub[0], sub[1]]


def random_bits(key, n):
    k = (C.c_uint32 * 2)(*key)
    out = (C.c_uint32 * n)()
    _check(lib().ornith_random_bits(k, n, out), "random_bits")
    return np.array(list(out), dtype=np.uint32)


def argsort_bf16(ctx, x, n, negate, idx_out):
    _check(lib().ornith_argsort_bf16(ctx.h, x.ptr, n, int(negate), idx_out.ptr), "argsort_bf16")


def cumsum(ctx, x, dtype, n, out):
    _check(lib().ornith_cumsum(ctx.h, x.ptr, dtype, n, out.ptr), "cumsum")


def apply_top_p(ctx, lp, V, top_p, out):
    _check(lib().ornith_apply_top_p(ctx.h, lp.ptr, V, C.c_double(top_p), out.ptr), "apply_top_p")


def apply_top_k(ctx, lp, V, top_k, out):
    _check(lib().ornith_apply_top_k(ctx.h, lp.ptr, V, top_k, out.ptr), "apply_top_k")


def categorical(ctx, lp, V, temp, raw_bits, token_out):
    _check(lib().ornith_categorical(ctx.h, lp.ptr, V, C.c_double(temp), C.c_uint32(raw_bits), token_out.ptr),
           "categorical")


class TopSampler:
    """TopSampler::new(temp, top_p, top_k, seed) over a vocabulary of `vocab` ids."""

    def __init__(self, ctx, temp, top_p, top_k, seed, vocab):
        self.ctx, self.vocab = ctx, vocab
        h = C.c_void_p()
        _check(lib().ornith_top_sampler_create(ctx.h, C.c_double(temp), C.c_double(top_p), top_k,
                                               C.c_uint64(seed), vocab, C.byref(h)), "top_sampler_create")
        self.h = h
        self._tok = ctx.alloc(4)

    def sample(self, logits_row):
        """logits_row: DeviceBuffer of bf16 [vocab] -> token id."""
        _check(lib().ornith_top_sampler_sample(self.h, logits_row.ptr, self._tok.ptr), "top_sampler_sample")
        return int(self._tok.download(np.uint32, (1,))[0])

    def set_rng(self, rng):
        _check(lib().ornith_top_sampler_set_rng(self.h, rng), "top_sampler_set_rng")

    def next_bits(self):
        b = C.c_uint32()
        _check(lib().ornith_top_sampler_next_bits(self.h, C.byref(b)), "top_sampler_next_bits")
        return b.value

    def weights(self, logits_row, V, w):
        """The sampler's distribution over bf16 logits [V] as fp32 weights [V] + their total: w is
        a DeviceBuffer of V + 1 floats."""
        _check(lib().ornith_sampler_weights(self.h, logits_row.ptr, V, w.ptr), "sampler_weights")

    def close(self):
        if self.h:
            lib().ornith_top_sampler_destroy(self.h)
            self.h = None
            self._tok.free()


def philox4x32_10(counter, key):
    c, k, out = (C.c_uint32 * 4)(*counter), (C.c_uint32 * 2)(*key), (C.c_uint32 * 4)()
    lib().ornith_philox4x32_10(c, k, out)
    return list(out)


def draw_weights(ctx, w, V, bits, tok):
    _check(lib().ornith_draw_weights(ctx.h, w.ptr, V, C.c_uint32(bits), tok.ptr), "draw_weights")


def spec_scatter(ctx, w_local, ids, n, V, w_full):
    _check(lib().ornith_spec_scatter(ctx.h, w_local.ptr, ids.ptr, n, V, w_full.ptr), "spec_scatter")


def spec_accept(ctx, wp, wq, V, x, bits, flag):
    _check(lib().ornith_spec_accept(ctx.h, wp.ptr, wq.ptr, V, x.ptr, C.c_uint32(bits), flag.ptr), "spec_accept")


def spec_resample(ctx, wp, wq, V, bits, tok):
    _check(lib().ornith_spec_resample(ctx.h, wp.ptr, wq.ptr, V, C.c_uint32(bits), tok.ptr), "spec_resample")


def moe_experts_from_gates(ctx, w, x, T, gates, egate, inds, scores, act, out):
    """The up + down launches of the MoE block with the routing made from the gates in the head
    of the up launch (what the model runs after its router launch)."""
    _check(lib().ornith_moe_experts_from_gates(ctx.h, C.byref(w), x.ptr, T, gates.ptr, egate.ptr, inds.ptr,
                                               scores.ptr, act.ptr, out.ptr), "moe_experts_from_gates")


def gdn_step(ctx, conv_state, qkv, cw, wa, wb, xn, H, a_log, dt_bias, T, K, Hk, Dk, Hv, Dv, state_in, snapshots,
             snap_all, norm_w, z, conv_input, gated_out, eps=1e-6, norm_eps=1e-6):
    """ornith_gdn_step with the a / b projections made from dense weights inside the launch."""
    _check(lib().ornith_gdn_step(ctx.h, conv_state.ptr, qkv.ptr, cw.ptr, None, None, wa.ptr, wb.ptr, xn.ptr, H,
                                 a_log.ptr, dt_bias.ptr, T, K, Hk, Dk, Hv, Dv, C.c_float(eps), state_in.ptr,
                                 snapshots.ptr, int(snap_all), norm_w.ptr, z.ptr, C.c_float(norm_eps),
                                 conv_input.ptr, gated_out.ptr), "gdn_step")


# ---- FR-Spec id lists on the host (src/frspec.rs:101-158, tools/merge_frspec.py) ------------------
class FrSpecMergeStats(C.Structure):
    _fields_ = [(n, C.c_size_t) for n in ("n_merged", "corpus_tokens", "covered_before", "covered_after",
                                           "missing_distinct", "missing_kept", "extra_new")]


def frspec_default_path():
    buf = C.create_string_buffer(4096)
    _check(lib().ornith_frspec_default_path(buf, C.c_size_t(4096)), "frspec_default_path")
    return buf.value.decode()


def frspec_read_ids(path):
    n = C.c_size_t()
    _check(lib().ornith_frspec_read_ids(str(path).encode(), None, C.c_size_t(0), C.byref(n)), "frspec_read_ids")
    out = np.empty(n.value, np.uint32)
    _check(lib().ornith_frspec_read_ids(str(path).encode(), _ptr(out), C.c_size_t(out.size), C.byref(n)), "frspec_read_ids")
    return out


def frspec_write_ids(path, ids, vocab):
    ids = np.ascontiguousarray(ids, dtype=np.uint32)
    n = C.c_size_t()
    _check(lib().ornith_frspec_write_ids(str(path).encode(), _ptr(ids), C.c_size_t(ids.size), C.c_uint32(vocab),
                                         C.byref(n)), "frspec_write_ids")
    return n.value


def frspec_merge(base, corpus, min_count, extra, vocab):
    """The superset merge on token ids: returns (merged ids, FrSpecMergeStats)."""
    base = np.ascontiguousarray(base, dtype=np.uint32)
    corpus = np.ascontiguousarray(corpus if corpus is not None else [], dtype=np.uint32)
    extra = np.ascontiguousarray(extra if extra is not None else [], dtype=np.uint32)
    st = FrSpecMergeStats()
    args = (_ptr(base), C.c_size_t(base.size), _ptr(corpus) if corpus.size else None, C.c_size_t(corpus.size),
            C.c_uint32(min_count), _ptr(extra) if extra.size else None, C.c_size_t(extra.size), C.c_uint32(vocab))
    _check(lib().ornith_frspec_merge(*args, None, C.c_size_t(0), C.byref(st)), "frspec_merge")
    out = np.empty(st.n_merged, np.uint32)
    _check(lib().ornith_frspec_merge(*args, _ptr(out), C.c_size_t(out.size), C.byref(st)), "frspec_merge")
    return out, st


# ---- prefill-width k-quant GEMM (src/ops/kquant.rs:783-1027) --------------------------------
def kq_matmul(ctx, w, x, M, y):
    _check(lib().ornith_kq_matmul(ctx.h, C.byref(w.s), x.ptr, M, y.ptr), "kq_matmul")


def kq_gather_plan_bytes(pairs, E):
    f = lib().ornith_kq_gather_plan_bytes
    f.restype = C.c_size_t
    return int(f(pairs, E))


def kq_gather_matmul(ctx, w, x, inds, pairs, top_k, is_up, plan, rebuild, y):
    _check(lib().ornith_kq_gather_matmul(ctx.h, C.byref(w.s), x.ptr, inds.ptr, pairs, top_k, int(is_up),
                                         plan.ptr, int(rebuild), y.ptr), "kq_gather_matmul")


# ---- norm folded into its consumers -----------------------------------------------------------
def add_rms_linear_multi(ctx, lins, res, y, wnorm, eps, M, h_out, normed_out, ys):
    n = len(lins)
    wp = (C.c_void_p * n)(*[C.cast(C.pointer(l.s), C.c_void_p) for l in lins])
    yp = (C.c_void_p * n)(*[b.ptr for b in ys])
    _check(lib().ornith_add_rms_linear_multi(ctx.h, wp, n, res.ptr, y.ptr, wnorm.ptr, C.c_float(eps), M,
                                             h_out.ptr, normed_out.ptr, yp), "add_rms_linear_multi")


def add_rms_moe_block(ctx, w, res, y, wnorm, eps, T, h_out, normed_out, out):
    _check(lib().ornith_add_rms_moe_block(ctx.h, C.byref(w), res.ptr, y.ptr, wnorm.ptr, C.c_float(eps), T,
                                          h_out.ptr, normed_out.ptr, out.ptr), "add_rms_moe_block")
