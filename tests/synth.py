"""Seeded synthetic Qwen3.5-MoE-shaped models for tests and the benchmark.

One generator produces numpy tensors under the reference's tensor names
(/root/reference/src/model/qwen3_5.rs:102-157, src/model/mtp.rs:96-143); the same arrays
feed the device library (through WeightStore.put) and the CPU oracle (through ctypes
structs), so both sides see identical bytes.

Format mix (BASELINE config 4, after the reference's q6k-full artifact,
tools/forge_q4k.py:138-152): gated-delta projections and routed/shared gate/up Q4_K,
attention projections, router and routed/shared down Q6_K, lm_head Q4_K, embed_tokens
and shared_expert_gate 8-bit affine, in_proj_a/b and the whole MTP head bf16.
Weights are zero-mean with unit-variance outputs so 40 random layers stay in range.
"""
import ctypes as C

import numpy as np

import util
from util import Q4K, Q6K, HostKMat, HostLinear, OrcKmat, OrcLinear, OrcMoeWeights, p

DT_F32, DT_BF16, DT_F16, DT_U8, DT_U32, DT_I32 = range(6)


class OrcConfig(C.Structure):
    _fields_ = [(n, C.c_int) for n in (
        "hidden_size", "num_hidden_layers", "vocab_size", "num_experts", "num_experts_per_tok",
        "moe_intermediate_size", "shared_expert_intermediate_size", "linear_num_key_heads",
        "linear_num_value_heads", "linear_key_head_dim", "linear_value_head_dim",
        "linear_conv_kernel_dim", "num_attention_heads", "num_key_value_heads", "head_dim",
        "rope_dims", "full_attention_interval", "norm_topk_prob")] + [
        ("rms_norm_eps", C.c_float), ("rope_theta", C.c_double)]


class OrcAttnW(C.Structure):
    _fields_ = [("q", OrcLinear), ("k", OrcLinear), ("v", OrcLinear), ("o", OrcLinear),
                ("q_norm", C.c_void_p), ("k_norm", C.c_void_p)]


class OrcGdnW(C.Structure):
    _fields_ = [("in_proj_qkv", OrcLinear), ("in_proj_z", OrcLinear), ("out_proj", OrcLinear),
                ("in_proj_a", OrcLinear), ("in_proj_b", OrcLinear), ("conv1d", C.c_void_p),
                ("dt_bias", C.c_void_p), ("a_log", C.c_void_p), ("norm", C.c_void_p)]


class OrcLayerW(C.Structure):
    _fields_ = [("linear", C.c_int), ("input_ln", C.c_void_p), ("post_ln", C.c_void_p),
                ("gdn", OrcGdnW), ("attn", OrcAttnW), ("moe", OrcMoeWeights)]


class OrcModelW(C.Structure):
    _fields_ = [("cfg", OrcConfig), ("embed", OrcLinear), ("lm_head", OrcLinear),
                ("final_norm", C.c_void_p), ("layers", C.POINTER(OrcLayerW))]


class OrcMtpW(C.Structure):
    _fields_ = [("pre_fc_norm_embedding", C.c_void_p), ("pre_fc_norm_hidden", C.c_void_p),
                ("input_ln", C.c_void_p), ("post_ln", C.c_void_p), ("norm", C.c_void_p),
                ("fc", OrcLinear), ("attn", OrcAttnW), ("moe", OrcMoeWeights),
                ("ex_gate", C.c_void_p), ("ex_up", C.c_void_p), ("ex_down", C.c_void_p)]


class OrcMtpStats(C.Structure):
    _fields_ = [("cycles", C.c_int64), ("drafted", C.c_int64), ("accepted", C.c_int64),
                ("reached", C.c_int64 * 8), ("accepted_by", C.c_int64 * 8)]


TINY = dict(hidden_size=512, num_hidden_layers=4, vocab_size=2048, num_experts=64, num_experts_per_tok=8,
            moe_intermediate_size=256, shared_expert_intermediate_size=256, linear_num_key_heads=2,
            linear_num_value_heads=4, linear_key_head_dim=128, linear_value_head_dim=128,
            linear_conv_kernel_dim=4, num_attention_heads=4, num_key_value_heads=1, head_dim=256,
            rope_dims=64, full_attention_interval=4, norm_topk_prob=1, rms_norm_eps=1e-6, rope_theta=1e7)

FULL = dict(hidden_size=2048, num_hidden_layers=40, vocab_size=248320, num_experts=256, num_experts_per_tok=8,
            moe_intermediate_size=512, shared_expert_intermediate_size=512, linear_num_key_heads=16,
            linear_num_value_heads=32, linear_key_head_dim=128, linear_value_head_dim=128,
            linear_conv_kernel_dim=4, num_attention_heads=16, num_key_value_heads=2, head_dim=256,
            rope_dims=64, full_attention_interval=4, norm_topk_prob=1, rms_norm_eps=1e-6, rope_theta=1e7)


def _norm_w(rng, n):
    return util.f32_to_bf16((1.0 + 0.1 * rng.standard_normal(n)).astype(np.float32))


class SynthModel:
    """All tensors of a trunk (+ optional MTP head) for a config dict."""

    def __init__(self, cfg, seed=0, with_mtp=True, with_oracle=True, affine="affine8", trunk="kq"):
        """affine: the format of the two affine modules (embed_tokens, shared_expert_gate):
        'affine8' (8-bit group 64, as in the k-quant artifact) or 'affine4' (4-bit group 32, the
        published artifact's format). trunk: 'kq' (the k-quant artifact: Q4_K / Q6_K
        projections and experts) or 'affine4' (the published artifact: every projection, the
        routed and shared experts and lm_head 4-bit affine group 32, the router 8-bit)."""
        self.affine = affine
        self.trunk = trunk
        t4 = (lambda kind: "affine4") if trunk == "affine4" else (lambda kind: kind)
        self._fmt = t4
        self.cfg = dict(cfg)
        self.rng = np.random.default_rng(seed)
        self.tensors = {}     # name -> (array, dtype code)
        self.keep = []        # host objects the oracle structs point into
        self.with_oracle = with_oracle
        c = self.cfg
        H, L = c["hidden_size"], c["num_hidden_layers"]
        kd = c["linear_num_key_heads"] * c["linear_key_head_dim"]
        vd = c["linear_num_value_heads"] * c["linear_value_head_dim"]
        D, Hv = 2 * kd + vd, c["linear_num_value_heads"]
        hd, Hq, Hkv = c["head_dim"], c["num_attention_heads"], c["num_key_value_heads"]
        P = "language_model.model."
        self.embed = self._linear(P + "embed_tokens", affine, c["vocab_size"], H)
        self.lm_head = self._linear("language_model.lm_head", t4(Q4K), c["vocab_size"], H)
        self.final_norm = self._plain(P + "norm.weight", _norm_w(self.rng, H))
        self.layers = []
        for i in range(L):
            lp = f"{P}layers.{i}."
            lay = dict(linear=(i + 1) % c["full_attention_interval"] != 0)
            lay["input_ln"] = self._plain(lp + "input_layernorm.weight", _norm_w(self.rng, H))
            lay["post_ln"] = self._plain(lp + "post_attention_layernorm.weight", _norm_w(self.rng, H))
            if lay["linear"]:
                g = lp + "linear_attn."
                lay["gdn"] = dict(
                    in_proj_qkv=self._linear(g + "in_proj_qkv", t4(Q4K), D, H),
                    in_proj_z=self._linear(g + "in_proj_z", t4(Q4K), vd, H),
                    out_proj=self._linear(g + "out_proj", t4(Q4K), H, vd),
                    in_proj_a=self._linear(g + "in_proj_a", "dense", Hv, H),
                    in_proj_b=self._linear(g + "in_proj_b", "dense", Hv, H),
                    conv1d=self._plain(g + "conv1d.weight", util.bf16_normal(self.rng, (D, 4, 1), 0.5)),
                    dt_bias=self._plain(g + "dt_bias", util.bf16_normal(self.rng, (Hv,), 0.5)),
                    a_log=self._plain(g + "A_log", util.bf16_normal(self.rng, (Hv,), 0.5)),
                    norm=self._plain(g + "norm.weight", _norm_w(self.rng, c["linear_value_head_dim"])))
            else:
                lay["attn"] = self._attn(lp + "self_attn.", t4(Q6K))
            lay["moe"] = self._moe(lp + "mlp.", dense=False)
            self.layers.append(lay)
        self.mtp = None
        if with_mtp:
            m = {}
            for n in ("pre_fc_norm_embedding", "pre_fc_norm_hidden", "norm"):
                m[n] = self._plain(f"mtp.{n}.weight", _norm_w(self.rng, H))
            m["input_ln"] = self._plain("mtp.layers.0.input_layernorm.weight", _norm_w(self.rng, H))
            m["post_ln"] = self._plain("mtp.layers.0.post_attention_layernorm.weight", _norm_w(self.rng, H))
            m["fc"] = self._linear("mtp.fc", "dense", H, 2 * H)
            m["attn"] = self._attn("mtp.layers.0.self_attn.", "dense")
            m["moe"] = self._moe("mtp.layers.0.mlp.", dense=True)
            self.mtp = m

    # ---- registration ---------------------------------------------------------------
    def _plain(self, name, arr_bf16):
        self.tensors[name] = (np.ascontiguousarray(arr_bf16), DT_BF16)
        return self.tensors[name][0]

    def _reg_kmat(self, path, km, routed):
        if km.kind == util.AFFINE4:
            self.tensors[path + ".weight"] = (km.qs.view(np.uint32), DT_U32)
            self.tensors[path + ".scales"] = (km.scales, DT_BF16)
            self.tensors[path + ".biases"] = (km.dm, DT_BF16)
            return
        nb = km.K // 256
        cb, sb, db = (128, 12, 2) if km.kind == Q4K else (192, 16, 1)
        lead = (km.E, km.O) if routed else (km.O,)
        self.tensors[path + ".weight"] = (km.qs.reshape(lead + (nb * cb,)).view(np.uint32), DT_U32)
        self.tensors[path + ".scales"] = (km.scales.reshape(lead + (nb, sb)), DT_U8)
        self.tensors[path + ".dm"] = (km.dm.reshape(lead + (nb, db)), DT_F16)

    def _linear(self, path, mode, O, K):
        if mode in ("affine8", "affine4"):
            lin = HostLinear.affine8(self.rng, O, K) if mode == "affine8" else HostLinear.affine4(self.rng, O, K)
            self.tensors[path + ".weight"] = (lin.w.view(np.uint32), DT_U32)
            self.tensors[path + ".scales"] = (lin.scales, DT_BF16)
            self.tensors[path + ".biases"] = (lin.biases, DT_BF16)
        elif mode == "dense":
            lin = HostLinear.dense(self.rng, O, K)
            self.tensors[path + ".weight"] = (lin.w, DT_BF16)
        else:
            lin = HostLinear.kq(self.rng, mode, O, K)
            self._reg_kmat(path, lin.km, routed=False)
        return lin

    def _attn(self, p_, mode):
        c = self.cfg
        H, hd, Hq, Hkv = c["hidden_size"], c["head_dim"], c["num_attention_heads"], c["num_key_value_heads"]
        return dict(q=self._linear(p_ + "q_proj", mode, Hq * 2 * hd, H), k=self._linear(p_ + "k_proj", mode, Hkv * hd, H),
                    v=self._linear(p_ + "v_proj", mode, Hkv * hd, H), o=self._linear(p_ + "o_proj", mode, H, Hq * hd),
                    q_norm=self._plain(p_ + "q_norm.weight", _norm_w(self.rng, hd)),
                    k_norm=self._plain(p_ + "k_norm.weight", _norm_w(self.rng, hd)))

    def _moe(self, p_, dense):
        c = self.cfg
        H, E, I, SI = c["hidden_size"], c["num_experts"], c["moe_intermediate_size"], c["shared_expert_intermediate_size"]
        m = {}
        if dense:
            m["router"] = self._linear(p_ + "gate", "dense", E, H)
            for n, (o, k) in (("gate", (I, H)), ("up", (I, H)), ("down", (H, I))):
                w = util.f32_to_bf16((self.rng.standard_normal((E, o, k)) / np.sqrt(k)).astype(np.float32))
                self.tensors[f"{p_}switch_mlp.{n}_proj.weight"] = (w, DT_BF16)
                m["ex_" + n] = w
            m["sh_gate"] = self._linear(p_ + "shared_expert.gate_proj", "dense", SI, H)
            m["sh_up"] = self._linear(p_ + "shared_expert.up_proj", "dense", SI, H)
            m["sh_down"] = self._linear(p_ + "shared_expert.down_proj", "dense", H, SI)
            m["sh_egate"] = self._linear(p_ + "shared_expert_gate", "dense", 1, H)
        else:
            a4 = self.trunk == "affine4"
            m["router"] = self._linear(p_ + "gate", "affine8" if a4 else Q6K, E, H)
            for n, kind, (o, k) in (("gate", Q4K, (I, H)), ("up", Q4K, (I, H)), ("down", Q6K, (H, I))):
                km = HostKMat.random(self.rng, util.AFFINE4 if a4 else kind, E, o, k)
                self._reg_kmat(f"{p_}switch_mlp.{n}_proj", km, routed=True)
                m["ex_" + n] = km
            m["sh_gate"] = self._linear(p_ + "shared_expert.gate_proj", self._fmt(Q4K), SI, H)
            m["sh_up"] = self._linear(p_ + "shared_expert.up_proj", self._fmt(Q4K), SI, H)
            m["sh_down"] = self._linear(p_ + "shared_expert.down_proj", self._fmt(Q6K), H, SI)
            m["sh_egate"] = self._linear(p_ + "shared_expert_gate", self.affine, 1, H)
        return m

    # ---- device side ----------------------------------------------------------------------
    def total_bytes(self):
        return sum(a.nbytes for a, _ in self.tensors.values())

    def upload(self, orn, ctx, drop_host=False):
        ws = orn.WeightStore(ctx)
        for name in list(self.tensors):
            arr, dt = self.tensors[name]
            ws.put(name, arr, dt)
            if drop_host:
                del self.tensors[name]
        return ws

    def text_config(self, orn):
        return orn.TextConfig(**self.cfg)

    # ---- oracle side ------------------------------------------------------------------------
    def _orc_attn(self, a):
        return OrcAttnW(a["q"].orc(), a["k"].orc(), a["v"].orc(), a["o"].orc(), p(a["q_norm"]), p(a["k_norm"]))

    def _orc_moe(self, m):
        c = self.cfg
        if isinstance(m["ex_gate"], HostKMat):
            eg, eu, ed = m["ex_gate"].orc(), m["ex_up"].orc(), m["ex_down"].orc()
        else:
            E, H, I = c["num_experts"], c["hidden_size"], c["moe_intermediate_size"]
            eg = OrcKmat(0, E, I, H, None, None, None); eu = OrcKmat(0, E, I, H, None, None, None)
            ed = OrcKmat(0, E, H, I, None, None, None)
        return OrcMoeWeights(m["router"].orc(), eg, eu, ed, m["sh_gate"].orc(), m["sh_up"].orc(), m["sh_down"].orc(),
                             m["sh_egate"].orc(), c["num_experts_per_tok"], c["norm_topk_prob"])

    def orc_model(self):
        L = len(self.layers)
        arr = (OrcLayerW * L)()
        for i, lay in enumerate(self.layers):
            arr[i].linear = int(lay["linear"])
            arr[i].input_ln = p(lay["input_ln"])
            arr[i].post_ln = p(lay["post_ln"])
            if lay["linear"]:
                g = lay["gdn"]
                arr[i].gdn = OrcGdnW(g["in_proj_qkv"].orc(), g["in_proj_z"].orc(), g["out_proj"].orc(),
                                     g["in_proj_a"].orc(), g["in_proj_b"].orc(), p(g["conv1d"]), p(g["dt_bias"]),
                                     p(g["a_log"]), p(g["norm"]))
            else:
                arr[i].attn = self._orc_attn(lay["attn"])
            arr[i].moe = self._orc_moe(lay["moe"])
        self.keep.append(arr)
        return OrcModelW(OrcConfig(**self.cfg), self.embed.orc(), self.lm_head.orc(), p(self.final_norm), arr)

    def orc_mtp(self):
        m = self.mtp
        return OrcMtpW(p(m["pre_fc_norm_embedding"]), p(m["pre_fc_norm_hidden"]), p(m["input_ln"]), p(m["post_ln"]),
                       p(m["norm"]), m["fc"].orc(), self._orc_attn(m["attn"]), self._orc_moe(m["moe"]),
                       p(m["moe"]["ex_gate"]), p(m["moe"]["ex_up"]), p(m["moe"]["ex_down"]))


class OracleRun:
    """A model + caches on the oracle side."""

    def __init__(self, synth, cap, max_T=16):
        self.synth = synth
        self.o = util.oracle()
        self.o.orc_state_create.restype = C.c_void_p
        self.mw = synth.orc_model()
        self.mtp = synth.orc_mtp() if synth.mtp else None
        self.st = C.c_void_p(self.o.orc_state_create(C.byref(self.mw), cap, max_T))
        self.H, self.V = synth.cfg["hidden_size"], synth.cfg["vocab_size"]

    def forward(self, tokens, capture=False):
        tokens = np.ascontiguousarray(tokens, dtype=np.uint32)
        out = np.empty((len(tokens), self.H), np.uint16)
        self.o.orc_forward(self.st, p(tokens), len(tokens), int(capture), p(out))
        return out

    def rewind(self, keep):
        self.o.orc_rewind(self.st, keep)

    def logits(self, hidden):
        hidden = np.ascontiguousarray(hidden, dtype=np.uint16)
        out = np.empty((hidden.shape[0], self.V), np.uint16)
        self.o.orc_logits(C.byref(self.mw), p(hidden), hidden.shape[0], p(out))
        return out

    def mtp_hidden(self, trunk_hidden, next_ids):
        trunk_hidden = np.ascontiguousarray(trunk_hidden, dtype=np.uint16)
        next_ids = np.ascontiguousarray(next_ids, dtype=np.uint32)
        out = np.empty((len(next_ids), self.H), np.uint16)
        self.o.orc_mtp_hidden(self.st, C.byref(self.mtp), p(trunk_hidden), p(next_ids), len(next_ids), p(out))
        return out

    def set_sampler(self, kind=0, temp=1.0, top_p=1.0, top_k=0, seed=0, accept=0, rng=0):
        """kind 0 greedy, 1 top-p/top-k/temperature; accept 0 token equality, 1 probability
        ratio; rng 0 threefry keys, 1 Philox4x32-10. Process-global in the oracle: reset to
        greedy when done."""
        self.o.orc_set_sampler2(kind, C.c_double(float(temp)), C.c_double(float(top_p)), top_k, C.c_uint64(seed),
                                accept, rng)

    def force_drafts(self, tokens):
        """Scripted drafts for mtp_generate (position p of the output is drafted as tokens[p]);
        an empty list clears them. Process-global in the oracle."""
        self._forced = np.ascontiguousarray(tokens, dtype=np.uint32)
        self.o.orc_mtp_force_drafts(p(self._forced) if len(self._forced) else None, len(self._forced))

    def generate(self, prompt, max_tokens, prefill_step=16):
        prompt = np.ascontiguousarray(prompt, dtype=np.uint32)
        out = np.empty(max_tokens, np.uint32)
        n = self.o.orc_generate(self.st, p(prompt), len(prompt), max_tokens, prefill_step, p(out))
        return [int(t) for t in out[:n]]

    def mtp_generate(self, prompt, depth, max_tokens, fr_ids=None, fr_head=None, policy=1, prefill_step=16):
        prompt = np.ascontiguousarray(prompt, dtype=np.uint32)
        out = np.empty(max_tokens, np.uint32)
        stats = OrcMtpStats()
        ids = np.ascontiguousarray(fr_ids, dtype=np.uint32) if fr_ids is not None else None
        head = fr_head.orc() if fr_head is not None else None
        n = self.o.orc_mtp_generate(self.st, C.byref(self.mtp), p(ids) if ids is not None else None,
                                    len(ids) if ids is not None else 0, C.byref(head) if head is not None else None,
                                    p(prompt), len(prompt), depth, max_tokens, prefill_step, policy, p(out),
                                    C.byref(stats))
        return [int(t) for t in out[:n]], stats

    def close(self):
        self.o.orc_state_destroy(self.st)


def prune_head(lin, ids):
    """FrSpec::prune on the host (for the oracle): row-gather of a k-quant head."""
    ids = np.asarray(ids, dtype=np.int64)
    if lin.mode in ("affine4", "affine8"):
        return HostLinear(lin.mode, len(ids), lin.K, w=np.ascontiguousarray(lin.w[ids]),
                          scales=np.ascontiguousarray(lin.scales[ids]), biases=np.ascontiguousarray(lin.biases[ids]))
    km = lin.km
    return HostLinear("kq", len(ids), lin.K, km=HostKMat(km.kind, 1, len(ids), km.K, (km.qs[ids], km.scales[ids], km.dm[ids])))


def zipf_frspec_ids(vocab, n, seed=0, a=1.1):
    """The top-n ids of a seeded Zipf(a) frequency ranking over the vocabulary (BASELINE config 4):
    a seeded permutation assigns ranks, rank r has weight r^-a; the n most frequent, in rank order."""
    rng = np.random.default_rng(seed)
    perm = rng.permutation(vocab)
    return perm[:n].astype(np.uint32)


# ---- artifact files --------------------------------------------------------------------------
_ST_NAMES = {DT_F32: "F32", DT_BF16: "BF16", DT_F16: "F16", DT_U8: "U8", DT_U32: "U32", 5: "I32"}


def write_safetensors(path, tensors, metadata=None, header_pad=0):
    """tensors: name -> (array, dtype code). Bytes are packed back to back in the given order
    behind `u64 header_len` + JSON, as the safetensors format has it; header_pad appends spaces
    to the header so the data section can start on any byte offset."""
    import json
    head, blobs, off = {}, [], 0
    if metadata is not None:
        head["__metadata__"] = metadata
    for name, (arr, dt) in tensors.items():
        raw = np.ascontiguousarray(arr).view(np.uint8).reshape(-1).tobytes()
        head[name] = {"dtype": _ST_NAMES[dt], "shape": list(arr.shape), "data_offsets": [off, off + len(raw)]}
        off += len(raw)
        blobs.append(raw)
    hj = json.dumps(head, separators=(",", ":")).encode() + b" " * header_pad
    with open(path, "wb") as f:
        f.write(len(hj).to_bytes(8, "little"))
        f.write(hj)
        for b in blobs:
            f.write(b)


def write_artifact(synth, model_dir, shards=3, nested=True):
    """The synthetic model as the files the loader reads: sharded safetensors + index,
    config.json (text config, quantization block with per-module overrides) and the MTP
    sidecar mtp/weights.safetensors with its experts as numbered tensors. Returns the
    sidecar's path (None without an MTP head)."""
    import json
    import os
    os.makedirs(model_dir, exist_ok=True)
    trunk = {n: t for n, t in synth.tensors.items() if not n.startswith("mtp.")}
    names = list(trunk)
    per = (len(names) + shards - 1) // shards
    weight_map = {}
    for s in range(shards):
        fn = f"model-{s + 1:05d}-of-{shards:05d}.safetensors"
        part = {n: trunk[n] for n in names[s * per:(s + 1) * per]}
        write_safetensors(os.path.join(model_dir, fn), part, metadata={"format": "mlx"}, header_pad=s)
        for n in part:
            weight_map[n] = fn
    with open(os.path.join(model_dir, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {"total_size": synth.total_bytes()}, "weight_map": weight_map}, f)

    a4 = getattr(synth, "trunk", "kq") == "affine4"
    quant = {"group_size": 32, "bits": 4, "mode": "affine"} if a4 else {"group_size": 64, "bits": 8, "mode": "affine"}
    for n, (arr, dt) in synth.tensors.items():
        if n.endswith(".biases"):
            # a module that departs from the artifact's default gets its own entry (mlx's per-layer overrides)
            groups, wbytes = synth.tensors[n[:-7] + ".scales"][0].size, synth.tensors[n[:-7] + ".weight"][0].nbytes
            bits = 8 if wbytes == groups * 64 else 4
            if bits != quant["bits"]:
                quant[n[:-7]] = {"group_size": 64 if bits == 8 else 32, "bits": bits, "mode": "affine"}
        if n.endswith(".dm"):
            q4 = synth.tensors[n[:-3] + ".scales"][0].shape[-1] == 12
            quant[n[:-3]] = {"group_size": 256, "bits": 4 if q4 else 6, "mode": "q4k" if q4 else "q6k"}
    c = synth.cfg
    text = {k: c[k] for k in c if k not in ("rope_dims", "rope_theta", "norm_topk_prob", "rms_norm_eps")}
    text["rms_norm_eps"] = c["rms_norm_eps"]
    text["norm_topk_prob"] = bool(c["norm_topk_prob"])
    text["rope_parameters"] = {"rope_theta": c["rope_theta"], "rope_type": "default",
                               "partial_rotary_factor": c["rope_dims"] / c["head_dim"]}
    text["model_type"] = "qwen3_5_moe_text"
    cfg = {"model_type": "qwen3_5_moe", "quantization": quant,
           "num_nextn_predict_layers": 1 if synth.mtp else 0}
    if nested:
        cfg["text_config"] = text
    else:
        cfg.update(text)
    with open(os.path.join(model_dir, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)

    if not synth.mtp:
        return None
    side = {}
    for n, (arr, dt) in synth.tensors.items():
        if not n.startswith("mtp."):
            continue
        if ".switch_mlp." in n:
            pre, suf = n.split(".switch_mlp.")
            for e in range(arr.shape[0]):
                side[f"{pre}.experts.{e}.{suf}"] = (arr[e], dt)
        else:
            side[n] = (arr, dt)
    os.makedirs(os.path.join(model_dir, "mtp"), exist_ok=True)
    sp = os.path.join(model_dir, "mtp", "weights.safetensors")
    write_safetensors(sp, side, header_pad=5)
    return sp
