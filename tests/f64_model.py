"""A float64 numpy forward of the trunk and the MTP head, written from the reference's Rust
(/root/reference/src/model/qwen3_5.rs:231-279 forward_hidden, :374-390 layer wiring,
:430-474 Attention::forward, :478-565 GatedDeltaNet::forward; src/model/mtp.rs:165-262) with
textbook formulas and dequantized weights. It shares no code with oracle/orc_model.c: it is
the independent statement the oracle's model-level composition is checked against (the
operator restatements it would otherwise lean on are replaced by plain numpy here).

Only the byte-format decoders (k-quant / 8-bit affine dequantization) come from the oracle;
those are pinned by closed forms in their own tests.
"""
import numpy as np

import util


def _deq_km(km):
    n = km.E * km.O * km.K // 256
    return util.orc_dequant(km.kind, km.qs, km.scales, km.dm, n).reshape(km.E, km.O, km.K).astype(np.float64)


def weight(lin):
    """HostLinear -> float64 [O, K]."""
    if lin.mode == "kq":
        return _deq_km(lin.km)[0]
    if lin.mode == "affine8":
        s = np.repeat(util.bf16_to_f32(lin.scales).astype(np.float64), 64, 1)
        b = np.repeat(util.bf16_to_f32(lin.biases).astype(np.float64), 64, 1)
        return lin.w.astype(np.float64) * s + b
    return util.bf16_to_f32(lin.w).astype(np.float64)


def vec(bf):
    return util.bf16_to_f32(np.asarray(bf)).astype(np.float64)


def rms(x, w, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


def silu(v):
    return v / (1.0 + np.exp(-v))


def sigmoid(v):
    return 1.0 / (1.0 + np.exp(-v))


class F64Model:
    """State-carrying float64 model over a synth.SynthModel."""

    def __init__(self, s):
        self.s, self.c = s, s.cfg
        c = self.c
        self.embed = None  # rows are dequantized on demand (the table can be large)
        self.layers = []
        for lay in s.layers:
            d = dict(linear=lay["linear"], input_ln=vec(lay["input_ln"]), post_ln=vec(lay["post_ln"]))
            if lay["linear"]:
                g = lay["gdn"]
                d["gdn"] = {k: weight(g[k]) for k in ("in_proj_qkv", "in_proj_z", "out_proj", "in_proj_a", "in_proj_b")}
                d["gdn"].update(conv1d=vec(g["conv1d"]).reshape(-1, c["linear_conv_kernel_dim"]),
                                dt_bias=vec(g["dt_bias"]), a_log=vec(g["a_log"]), norm=vec(g["norm"]))
            else:
                d["attn"] = self._attn_w(lay["attn"])
            d["moe"] = self._moe_w(lay["moe"])
            self.layers.append(d)
        self.final_norm = vec(s.final_norm)
        self.forced_picks = None
        self.reset()
        if s.mtp:
            m = s.mtp
            self.mtp = dict(pre_e=vec(m["pre_fc_norm_embedding"]), pre_h=vec(m["pre_fc_norm_hidden"]),
                            input_ln=vec(m["input_ln"]), post_ln=vec(m["post_ln"]), norm=vec(m["norm"]),
                            fc=weight(m["fc"]), attn=self._attn_w(m["attn"]), moe=self._moe_w(m["moe"]))
            self.mtp_kv = ([], [])

    def _attn_w(self, a):
        return dict(q=weight(a["q"]), k=weight(a["k"]), v=weight(a["v"]), o=weight(a["o"]),
                    q_norm=vec(a["q_norm"]), k_norm=vec(a["k_norm"]))

    def _moe_w(self, m):
        ex = {}
        for n in ("ex_gate", "ex_up", "ex_down"):
            ex[n] = _deq_km(m[n]) if isinstance(m[n], util.HostKMat) else util.bf16_to_f32(m[n]).astype(np.float64)
        ex.update({n: weight(m[n]) for n in ("router", "sh_gate", "sh_up", "sh_down", "sh_egate")})
        return ex

    def reset(self):
        c = self.c
        kd = c["linear_num_key_heads"] * c["linear_key_head_dim"]
        vd = c["linear_num_value_heads"] * c["linear_value_head_dim"]
        self.offset = 0
        self.cache = []
        for lay in self.layers:
            if lay["linear"]:
                self.cache.append(dict(conv=np.zeros((c["linear_conv_kernel_dim"] - 1, 2 * kd + vd)),
                                       state=np.zeros((c["linear_num_value_heads"], c["linear_value_head_dim"],
                                                       c["linear_key_head_dim"]))))
            else:
                self.cache.append(dict(k=[], v=[]))

    # ---- pieces --------------------------------------------------------------------------
    def embedding(self, ids):
        e = self.s.embed
        ids = np.asarray(ids, dtype=np.int64)
        s = np.repeat(util.bf16_to_f32(e.scales[ids]).astype(np.float64), 64, 1)
        b = np.repeat(util.bf16_to_f32(e.biases[ids]).astype(np.float64), 64, 1)
        return e.w[ids].astype(np.float64) * s + b

    def moe(self, w, x, margins=None):
        """margins: optional list receiving (relative gap at the top-k cut, own picks) per token.
        self.forced_picks: optional iterator of [k] expert lists, one per routed token in call
        order; when set, the experts are those (the weights are still this model's own softmax),
        so a comparison is not at the mercy of which side of a near-tie a rounding falls."""
        c = self.c
        k = c["num_experts_per_tok"]
        g = x @ w["router"].T
        p = np.exp(g - g.max(1, keepdims=True))
        p /= p.sum(1, keepdims=True)
        out = np.zeros_like(x)
        for t in range(x.shape[0]):
            order = np.argsort(p[t], kind="stable")
            top = order[-k:]
            forced = next(self.forced_picks) if self.forced_picks is not None else None
            if margins is not None:
                margins.append(((p[t][order[-k]] - p[t][order[-k - 1]]) / p[t][order[-k]], set(int(e) for e in top),
                                None if forced is None else set(int(e) for e in forced)))
            if forced is not None:
                top = np.asarray(forced, dtype=np.int64)
            wt = p[t][top]
            if c["norm_topk_prob"]:
                wt = wt / wt.sum()
            acc = np.zeros(x.shape[1])
            for j, e in enumerate(top):
                a = silu(w["ex_gate"][e] @ x[t]) * (w["ex_up"][e] @ x[t])
                acc += wt[j] * (w["ex_down"][e] @ a)
            sh = w["sh_down"] @ (silu(w["sh_gate"] @ x[t]) * (w["sh_up"] @ x[t]))
            out[t] = acc + sigmoid(w["sh_egate"][0] @ x[t]) * sh
        return out

    def attention(self, w, x, kv, offset):
        c = self.c
        T = x.shape[0]
        hd, Hq, Hkv, rd = c["head_dim"], c["num_attention_heads"], c["num_key_value_heads"], c["rope_dims"]
        qg = (x @ w["q"].T).reshape(T, Hq, 2 * hd)
        q, gate = qg[:, :, :hd], qg[:, :, hd:].reshape(T, Hq * hd)
        k = (x @ w["k"].T).reshape(T, Hkv, hd)
        v = (x @ w["v"].T).reshape(T, Hkv, hd)
        q = rms(q, w["q_norm"], c["rms_norm_eps"])
        k = rms(k, w["k_norm"], c["rms_norm_eps"])
        half = rd // 2
        inv_freq = c["rope_theta"] ** (-np.arange(half) / half)

        def rope(a):
            a = a.copy()
            for t in range(T):
                th = (offset + t) * inv_freq
                x1, x2 = a[t, :, :half].copy(), a[t, :, half:rd].copy()
                a[t, :, :half] = x1 * np.cos(th) - x2 * np.sin(th)
                a[t, :, half:rd] = x1 * np.sin(th) + x2 * np.cos(th)
            return a

        q, k = rope(q), rope(k)
        for t in range(T):
            kv[0].append(k[t])
            kv[1].append(v[t])
        K, V = np.stack(kv[0]), np.stack(kv[1])       # [N, Hkv, hd]
        out = np.zeros((T, Hq, hd))
        rep = Hq // Hkv
        for t in range(T):
            n = offset + t + 1                         # causal: keys 0..offset+t
            for h in range(Hq):
                sc = (K[:n, h // rep] @ q[t, h]) * hd ** -0.5
                pr = np.exp(sc - sc.max())
                pr /= pr.sum()
                out[t, h] = pr @ V[:n, h // rep]
        return (sigmoid(gate) * out.reshape(T, Hq * hd)) @ w["o"].T

    def gdn(self, w, x, cache):
        c = self.c
        T = x.shape[0]
        Hk, Hv, Dk, Dv, K = (c["linear_num_key_heads"], c["linear_num_value_heads"], c["linear_key_head_dim"],
                             c["linear_value_head_dim"], c["linear_conv_kernel_dim"])
        kd = Hk * Dk
        qkv = x @ w["in_proj_qkv"].T
        z = (x @ w["in_proj_z"].T).reshape(T, Hv, Dv)
        b = x @ w["in_proj_b"].T
        a = x @ w["in_proj_a"].T
        win = np.concatenate([cache["conv"], qkv])                 # [K-1+T, D]
        cache["conv"] = win[T:]
        conv = sum(win[i:i + T] * w["conv1d"][:, i] for i in range(K))
        s = silu(conv)
        q = s[:, :kd].reshape(T, Hk, Dk)
        k = s[:, kd:2 * kd].reshape(T, Hk, Dk)
        v = s[:, 2 * kd:].reshape(T, Hv, Dv)
        q = rms(q, 1.0, 1e-6) * Dk ** -1.0
        k = rms(k, 1.0, 1e-6) * Dk ** -0.5
        beta = sigmoid(b)
        g = np.exp(-np.exp(w["a_log"]) * np.logaddexp(a + w["dt_bias"], 0.0))
        S = cache["state"]
        y = np.zeros((T, Hv, Dv))
        for t in range(T):
            for hv in range(Hv):
                hk = hv // (Hv // Hk)
                S[hv] *= g[t, hv]
                kvv = S[hv] @ k[t, hk]
                delta = (v[t, hv] - kvv) * beta[t, hv]
                S[hv] += np.outer(delta, k[t, hk])
                y[t, hv] = S[hv] @ q[t, hk]
        gated = silu(z) * rms(y, w["norm"], c["rms_norm_eps"])
        return gated.reshape(T, Hv * Dv) @ w["out_proj"].T

    # ---- the trunk -----------------------------------------------------------------------
    def forward(self, ids, margins=None):
        eps = self.c["rms_norm_eps"]
        x = self.embedding(ids)
        T = x.shape[0]
        normed = rms(x, self.layers[0]["input_ln"], eps)
        for i, lay in enumerate(self.layers):
            if lay["linear"]:
                r = self.gdn(lay["gdn"], normed, self.cache[i])
            else:
                r = self.attention(lay["attn"], normed, (self.cache[i]["k"], self.cache[i]["v"]), self.offset)
            h = x + r
            m = self.moe(lay["moe"], rms(h, lay["post_ln"], eps), margins)
            x = h + m
            nw = self.layers[i + 1]["input_ln"] if i + 1 < len(self.layers) else self.final_norm
            normed = rms(x, nw, eps)
        self.offset += T
        return normed

    # ---- the MTP head ----------------------------------------------------------------------
    def mtp_hidden(self, trunk_hidden, next_ids, margins=None):
        eps = self.c["rms_norm_eps"]
        m = self.mtp
        e = rms(self.embedding(next_ids), m["pre_e"], eps)
        h = rms(np.asarray(trunk_hidden, dtype=np.float64), m["pre_h"], eps)
        x = np.concatenate([e, h], axis=1) @ m["fc"].T           # concat order: embedding, hidden
        off = len(self.mtp_kv[0])
        r = self.attention(m["attn"], rms(x, m["input_ln"], eps), self.mtp_kv, off)
        hh = x + r
        out = hh + self.moe(m["moe"], rms(hh, m["post_ln"], eps), margins)
        return rms(out, m["norm"], eps)
