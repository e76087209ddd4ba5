"""Benchmark of the speculative decode step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--tokens 200] [--depth 1]

Workload (BASELINE.json configs[3], the configuration the metric is quoted on): a seeded,
random-init Qwen3.5-35B-A3B-shaped model (40 layers = 30 gated-delta + 10 full attention,
256-expert top-8 MoE + shared expert, Q4_K/Q6_K/8-bit mix, vocab 248320, one-layer bf16
MTP head, FR-Spec draft vocabulary of 32768 ids), 51-token seeded prompt, greedy depth-1
MTP decode of 200 tokens, whose output must be byte-identical to plain greedy decode.
A "step" is one such 200-token generation; the timed region starts when the prompt has
been consumed and its last position sampled from (weights, caches and prompt state are
resident in HBM) and `value` is generated tokens per second.

`value` is a FLOOR: random-init weights accept no draft, so every cycle pays a two-row verify
plus a draft for one token. The same line carries plain greedy decode and the forced-acceptance
ceilings (every draft accepted) beside it.

Also measured in the same run and printed on the same JSON line:
  roofline      the expert gather-GEMV as the model runs it: the up launch (routing made in its
                head, gate + up + swiglu) and the down launch (down + combine) of the MoE block,
                back to back over all 40 layers' resident weights with the router's own picks, at
                verify width 2: algorithmic bytes (distinct routed experts + the shared one, three
                matrices each, + activations) over the pair's average duration from HIP events on
                the library's stream, against 8 TB/s. `by_width` repeats it at T = 1, 2, 4 with the
                number of distinct experts; `standalone_up` is the up kernel alone with the expert
                ids given (no routing head).
  per_config    BASELINE configs 1-3: the 512x2048 Q4_K mat-vec, one MoE block at T = 1, 2, 4, one
                gated-delta layer at T = 2 with per-token snapshots, each with the oracle's time on
                the host cores
  cpu_baseline  the CPU oracle running the same loop on the host cores (bounded sample); the only
                part of this script that loads anything under oracle/
"""
import argparse
import ctypes as C
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0
EXPERT_BYTES = 2 * 589_824 + 860_160       # gate + up (Q4_K 512x2048) + down (Q6_K 2048x512)

# HBM bytes per launch from two `rocprofv3 --pmc` runs of `bench.py --roofline-only` (FETCH_SIZE,
# then WRITE_SIZE, KiB per dispatch) recorded in profiles/moe_up_T2_pmc.md, each scaled by what
# the same counter reads for a 256 MiB device copy (fetch x 2.0, write x 1.0): the up + down pair
# as the model launches it at verify width 2 (the router's own picks, 15.4 distinct experts on
# average; its algorithmic bytes are the `bytes_per_pair` of that loop) and the up kernel alone
# with 17 given experts. Counters cannot be read from inside this script: the figures are
# carried from that profile and labelled so.
_KIB = 1024
PROFILE_TRAFFIC = {
    "pair": {"bytes": int(round(((9565.6 + 7095.0) * 2.0 + (36.1 + 8.0) * 1.0) * _KIB)), "algorithmic_bytes": 33_557_094,
             "kernel": "moe_up_kernel<0, 64, 2, true> + moe_down_kernel<1, 8, 2> (T = 2, the router's picks)"},
    "up_alone": {"bytes": int(round((9865.3 * 2.0 + 36.0 * 1.0) * _KIB)), "algorithmic_bytes": 20_080_704,
                 "kernel": "moe_up_kernel<0, 64, 2, false> (T = 2, 17 experts)"},
    "source": "profiles/moe_up_T2_pmc.md (rocprofv3 --pmc runs of `bench.py --roofline-only`, not read in this run)"}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


class _Lin:
    """A Linear held by the model, seen through the struct the library hands out."""

    def __init__(self, s):
        self.s = s


def _time_loop(ctx, fn, n, warm):
    for i in range(warm):
        fn(i)
    ctx.sync()
    ctx.timer_begin()
    for i in range(n):
        fn(i)
    return ctx.timer_end() * 1000.0 / n       # microseconds per call


def expert_roofline(orn, ctx, model, np, n_layers, T, pairs=400):
    """The expert gather-GEMV as the model runs it, at verify width T: per layer the router's
    gates are made once from seeded activations, then the up launch (softmax + top-8 in its head,
    gate + up + swiglu) and the down launch (down + combine) are timed back to back, cycling
    through every layer's resident weights so that no launch finds its experts in cache.
    Algorithmic bytes per pair: (distinct routed experts + 1) x 2,039,808 + the activation rows
    read and written (x, act twice, out)."""
    rng = np.random.default_rng(123)
    H, I, E, k = 2048, 512, 256, 8
    moes = [model.moe_weights(i) for i in range(n_layers)]
    x = ctx.to_device(orn.f32_to_bf16(rng.standard_normal((T, H)).astype(np.float32)))
    gates = [ctx.alloc(T * E * 2) for _ in moes]
    egate = ctx.alloc(T * 2)
    inds, scores = ctx.alloc(T * k * 4), ctx.alloc(T * k * 2)
    act, out = ctx.alloc((T * k + T) * I * 2), ctx.alloc(T * H * 2)
    U = []
    for w, g in zip(moes, gates):
        ctx.linear_matmul(_Lin(w.router), x, T, g)
        ctx.linear_matmul(_Lin(w.sh_egate), x, T, egate)
        orn.moe_experts_from_gates(ctx, w, x, T, g, egate, inds, scores, act, out)
        U.append(len(np.unique(inds.download(np.uint32, (T * k,)))))
    us = _time_loop(ctx, lambda i: orn.moe_experts_from_gates(ctx, moes[i % n_layers], x, T, gates[i % n_layers], egate,
                                                              inds, scores, act, out), pairs, n_layers)
    u_mean = float(np.mean(U))
    acts = T * H * 2 + 2 * (T * k + T) * I * 2 + T * H * 2
    nbytes = (u_mean + 1) * EXPERT_BYTES + acts
    # the up kernel alone with the ids given (no routing head): the figure earlier reports carried
    ids = np.concatenate([rng.permutation(E)[:k] for _ in range(T)]).astype(np.uint32)
    d_ids = ctx.to_device(ids)
    us_up = _time_loop(ctx, lambda i: orn.moe_experts(ctx, moes[i % n_layers], x, T, d_ids, scores, egate, act, out, 1),
                       pairs, n_layers)
    up_bytes = (len(np.unique(ids)) + 1) * 2 * 589_824 + T * H * 2 + (T * k + T) * I * 2 + T * k * 4
    for b in [x, egate, inds, scores, act, out, d_ids] + gates:
        b.free()
    ach = nbytes / (us * 1e-6) / 1e9
    return {"verify_width": T, "distinct_experts_mean": round(u_mean, 2), "us_per_pair": round(us, 3),
            "bytes_per_pair": int(nbytes), "achieved": round(ach, 1), "frac": round(ach / HBM_PEAK_GBS, 4),
            "standalone_up": {"us_per_launch": round(us_up, 3), "bytes_per_launch": int(up_bytes),
                              "achieved": round(up_bytes / (us_up * 1e-6) / 1e9, 1),
                              "frac": round(up_bytes / (us_up * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)}}


def expert_overlap(orn, ctx, model, np, n_layers, cases=("distinct", "same8"), widths=(2, 4), pairs=400):
    """Verify rows of real text share experts; random-init routing does not (U = 15.4 of 16 at
    T = 2). This leg gives the up + down pair routing in which all T tokens pick the same 8
    experts (`same8`) beside routing with 8 T distinct ones (`distinct`), ids given, cycling the
    layers' resident weights so that nothing is warm from an earlier launch. The kernels take a
    (token, expert) row per workgroup column, but a grid x of 64 puts the workgroups that read
    the same weight rows for different tokens on the same die, so the second token's reads are
    L2 hits: `bytes_distinct` is what memory has to deliver."""
    rng = np.random.default_rng(321)
    H, I, E, k = 2048, 512, 256, 8
    moes = [model.moe_weights(i) for i in range(n_layers)]
    rows = []
    for T in widths:
        x = ctx.to_device(orn.f32_to_bf16(rng.standard_normal((T, H)).astype(np.float32)))
        scores = ctx.to_device(orn.f32_to_bf16((rng.random((T, k)) + 0.1).astype(np.float32)))
        egate = ctx.to_device(orn.f32_to_bf16(rng.standard_normal((T,)).astype(np.float32)))
        act, out = ctx.alloc((T * k + T) * I * 2), ctx.alloc(T * H * 2)
        for case in cases:
            ids = []
            for _ in range(n_layers):
                if case == "same8":
                    v = np.tile(rng.permutation(E)[:k], T)
                else:
                    v = rng.permutation(E)[:k * T]
                ids.append(ctx.to_device(v.astype(np.uint32)))
            us = _time_loop(ctx, lambda i: orn.moe_experts(ctx, moes[i % n_layers], x, T, ids[i % n_layers], scores, egate,
                                                           act, out, 3), pairs, n_layers)
            U = k if case == "same8" else k * T
            nbytes = (U + 1) * EXPERT_BYTES + T * H * 2 * 2 + 2 * (T * k + T) * I * 2
            rows.append({"verify_width": T, "routing": case, "distinct_experts": U, "us_per_pair": round(us, 3),
                         "bytes_distinct": int(nbytes), "GB_s": round(nbytes / (us * 1e-6) / 1e9, 1)})
            for b in ids:
                b.free()
        for b in (x, scores, egate, act, out):
            b.free()
    return rows


def per_config(orn, ctx, np, with_cpu):
    """BASELINE configs 1-3 on their own seeded tensors: GPU time from HIP events over chained
    launches; CPU time of the oracle's restatement of the same operator (best of 5)."""
    import util
    res = {}

    def cpu_us(fn, reps=5):
        best = 1e30
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            best = min(best, time.perf_counter() - t0)
        return round(best * 1e6, 1)

    # ---- config 1: Q4_K mat-vec 512 x 2048, fp32 activations in and out
    rng = np.random.default_rng(1)
    O, K = 512, 2048
    t = util.make_q4k(rng, 1, O, K)
    w = orn.KMatrix(ctx, orn.Q4K, *t, 1, O, K)
    xf = rng.standard_normal((1, K)).astype(np.float32)
    dx, dy = ctx.to_device(xf), ctx.alloc(O * 4)
    us = _time_loop(ctx, lambda i: ctx.kq_qmv(w, dx, orn.F32, 1, dy, orn.F32), 2000, 100)
    nbytes = 589_824 + 8_192 + 2_048
    c1 = {"workload": "Q4_K dequant mat-vec 512x2048, fp32 x [1,2048] -> fp32 y [1,512], 2000 chained launches",
          "us_per_launch": round(us, 3), "algorithmic_bytes": nbytes, "GB_s": round(nbytes / (us * 1e-6) / 1e9, 1)}
    if with_cpu:
        got = dy.download(np.float32, (1, O))
        want64 = util.orc_matvec_f64(util.Q4K, *t, O, K, xf)
        c1["max_abs_err_vs_f64"] = float(np.max(np.abs(got - want64)))
        c1["global_rel_err_vs_f64"] = util.global_rel(got, want64)
        c1["bit_exact_vs_oracle"] = bool(np.array_equal(got.view(np.uint32), util.orc_qmv(util.Q4K, *t, O, K, xf).view(np.uint32)))
        c1["cpu_us"] = cpu_us(lambda: util.orc_qmv(util.Q4K, *t, O, K, xf))
    for b in (dx, dy):
        b.free()
    w.free()
    res["config1"] = c1

    # ---- config 2: one MoE block at T = 1, 2, 4 (four sets of weights cycled: 2.1 GB)
    rng = np.random.default_rng(2)
    moes = [util.HostMoe(rng) for _ in range(4)]
    devs = [m.dev(orn, ctx) for m in moes]
    c2 = {"workload": "one MoE block: hidden 2048, 256 experts top-8 (gate/up Q4_K, down Q6_K) + shared expert, "
                      "router Q6_K, bf16 activations; router + up + down launches", "by_width": []}
    for T in (1, 2, 4):
        xb = orn.f32_to_bf16(rng.standard_normal((T, 2048)).astype(np.float32))
        dxb, dout = ctx.to_device(xb), ctx.alloc(T * 2048 * 2)
        di, ds = ctx.alloc(T * 8 * 4), ctx.alloc(T * 8 * 2)
        ctx.moe_block(devs[0], dxb, T, dout, di, ds)
        inds = di.download(np.uint32, (T, 8))
        U = len(np.unique(inds))
        us = _time_loop(ctx, lambda i: ctx.moe_block(devs[i % 4], dxb, T, dout), 400, 8)
        nbytes = (U + 1) * EXPERT_BYTES + 430_080 + 2_208 + T * 2048 * 2 * 2 + 2 * 9 * T * 1024
        e = {"T": T, "distinct_experts": U, "us_per_block": round(us, 3), "algorithmic_bytes": int(nbytes),
             "GB_s": round(nbytes / (us * 1e-6) / 1e9, 1), "frac_of_hbm_peak": round(nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)}
        if with_cpu:
            _, oinds, _, _ = util.orc_moe_block(moes[0], xb, T)
            e["expert_indices_bit_exact"] = bool(np.array_equal(oinds, inds))
            e["cpu_us"] = cpu_us(lambda: util.orc_moe_block(moes[0], xb, T), reps=3)
        c2["by_width"].append(e)
        for b in (dxb, dout, di, ds):
            b.free()
    for m in moes:
        m.free()
    res["config2"] = c2

    # ---- config 3: one gated-delta layer at T = 2 with per-token snapshots (rollback is a cursor move)
    rng = np.random.default_rng(3)
    H, Hk, Hv, D = 2048, 16, 32, 8192
    T = 2
    lin = {n: util.HostLinear.kq(rng, util.Q4K, o, k) for n, (o, k) in
           (("qkv", (D, H)), ("z", (4096, H)), ("out", (H, 4096)))}
    dl = {n: l.dev(orn, ctx) for n, l in lin.items()}
    wa, wb = util.HostLinear.dense(rng, Hv, H), util.HostLinear.dense(rng, Hv, H)
    bf = lambda shape, std=1.0: orn.f32_to_bf16((rng.standard_normal(shape) * std).astype(np.float32))
    host = dict(xn=bf((T, H)), conv=bf((3, D)), cw=bf((D, 4), 0.5), a_log=bf((Hv,), 0.5), dt=bf((Hv,), 0.5),
                nw=bf((128,)), S0=(rng.standard_normal((Hv, 128, 128)) * 0.1).astype(np.float32))
    d = {n: ctx.to_device(a) for n, a in host.items()}
    d["wa"], d["wb"] = ctx.to_device(wa.w), ctx.to_device(wb.w)
    qkv, z = ctx.alloc(T * D * 2), ctx.alloc(T * 4096 * 2)
    snaps, ci, gated, r = ctx.alloc(T * Hv * 128 * 128 * 4), ctx.alloc((3 + T) * D * 2), ctx.alloc(T * 4096 * 2), ctx.alloc(T * H * 2)

    def layer(i):
        ctx.linear_matmul_multi([dl["qkv"], dl["z"]], d["xn"], T, [qkv, z])
        orn.gdn_step(ctx, d["conv"], qkv, d["cw"], d["wa"], d["wb"], d["xn"], H, d["a_log"], d["dt"], T, 4, Hk, 128, Hv,
                     128, d["S0"], snaps, True, d["nw"], z, ci, gated)
        ctx.linear_matmul(dl["out"], gated, T, r)

    us = _time_loop(ctx, layer, 400, 8)
    wbytes = 9_437_184 + 4_718_592 + 4_718_592 + 2 * 131_072 + 65_536
    state = 2_097_152 * (1 + T)
    c3 = {"workload": "one gated-delta layer, T = 2 verify rows with a state snapshot per row: in_proj qkv+z, "
                      "mixer core (a/b projections, conv, recurrence, gated norm), out_proj; 3 launches, the same "
                      "weights every call; rollback of the rejected row is a cursor move (no launch)",
          "us_per_layer": round(us, 3), "weight_bytes": wbytes, "state_bytes_moved": state,
          "GB_s": round((wbytes + state) / (us * 1e-6) / 1e9, 1)}
    if with_cpu:
        def cpu_layer():
            x32 = util.bf16_to_f32(host["xn"])
            qkv_h = util.f32_to_bf16(util.orc_qmv(util.Q4K, lin["qkv"].km.qs, lin["qkv"].km.scales, lin["qkv"].km.dm, D, H, x32, True))
            z_h = util.f32_to_bf16(util.orc_qmv(util.Q4K, lin["z"].km.qs, lin["z"].km.scales, lin["z"].km.dm, 4096, H, x32, True))
            a_h, b_h = np.empty((T, Hv), np.uint16), np.empty((T, Hv), np.uint16)
            util.oracle().orc_dense_gemv(util.p(wa.w), Hv, H, util.p(host["xn"]), T, util.p(a_h))
            util.oracle().orc_dense_gemv(util.p(wb.w), Hv, H, util.p(host["xn"]), T, util.p(b_h))
            q, k, v, beta, g, _ = util.orc_gdn_front(host["conv"], qkv_h, host["cw"], a_h, b_h, host["a_log"], host["dt"], Hk, Hv)
            y, _ = util.orc_gdn_recurrence(q, k, v, g, beta, host["S0"])
            gated_h = util.orc_rms_norm_gated(y.reshape(T * Hv, 128), host["nw"], z_h.reshape(T * Hv, 128))
            return util.f32_to_bf16(util.orc_qmv(util.Q4K, lin["out"].km.qs, lin["out"].km.scales, lin["out"].km.dm, H, 4096,
                                                 util.bf16_to_f32(gated_h.reshape(T, 4096)), True))

        want = cpu_layer()
        c3["bit_exact_vs_oracle"] = bool(np.array_equal(r.download(np.uint16, (T, H)), want))
        c3["cpu_us"] = cpu_us(cpu_layer, reps=3)
    for b in list(d.values()) + [qkv, z, snaps, ci, gated, r]:
        b.free()
    for l in dl.values():
        l.free()
    res["config3"] = c3
    return res


def cpu_baseline(synth, synth_model, np, depth, tokens, prompt):
    """The oracle's generate_step_mtp on the host cores with the benchmark's own prompt; the
    prefill (timed separately on a second state) is taken off the whole call."""
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    fr_ids = synth.zipf_frspec_ids(synth_model.cfg["vocab_size"], 32768, seed=1)
    fr_host = synth.prune_head(synth_model.lm_head, fr_ids)
    pre = synth.OracleRun(synth_model, 128)
    t0 = time.time()
    for i in range(0, len(prompt) - 1, 16):
        pre.forward(prompt[i:min(i + 16, len(prompt) - 1)])
    t_pre = time.time() - t0
    pre.close()
    run = synth.OracleRun(synth_model, 128)
    t0 = time.time()
    toks, st = run.mtp_generate(prompt, depth, tokens, fr_ids, fr_host, policy=1, prefill_step=16)
    dt = time.time() - t0
    run.close()
    dec = max(dt - t_pre, 1e-9)
    return {"value": round(len(toks) / dec, 4), "unit": "tok/s", "cores": threads, "kind": "port",
            "sample": f"oracle generate_step_mtp depth {depth} + FR-Spec on the {len(prompt)}-token prompt, first "
                      f"{len(toks)} tokens: whole call {dt:.1f} s, of which prefill {t_pre:.1f} s "
                      f"({int(st.cycles)} cycles, {int(st.accepted)} accepted)"}, toks


def moe_ab(orn, ctx, model, np, n_layers):
    """The MoE block (norm + router + up + down) as separate launches (fuse_moe_one = 0), as one
    launch with in-launch hand-offs (1), and as router + one up/down launch (2), on the resident
    weights of every layer in turn. Prints a JSON table."""
    lib = orn.lib()
    H = 2048
    rng = np.random.default_rng(5)
    moes = [model.moe_weights(i) for i in range(n_layers)]
    wn = ctx.to_device(orn.f32_to_bf16((1 + 0.1 * rng.standard_normal(H)).astype(np.float32)))
    rows = []
    for T in (1, 2, 4):
        res, y = (ctx.to_device(orn.f32_to_bf16(rng.standard_normal((T, H)).astype(np.float32))) for _ in range(2))
        h, nx, out = ctx.alloc(T * H * 2), ctx.alloc(T * H * 2), ctx.alloc(T * H * 2)
        ref = None
        for how in (0, 1, 2):
            orn.set_option("fuse_moe_one", how)

            def run(i):
                rc = lib.ornith_add_rms_moe_block(ctx.h, C.byref(moes[i % n_layers]), res.ptr, y.ptr, wn.ptr,
                                                  C.c_float(1e-6), T, h.ptr, nx.ptr, out.ptr)
                assert rc == 0, lib.ornith_last_error()

            us = _time_loop(ctx, run, 400, n_layers)
            run(0)
            o = out.download(np.uint16, (T, H))
            ref = o if ref is None else ref
            rows.append({"T": T, "fuse_moe_one": how, "us_per_block": round(us, 2), "identical": bool(np.array_equal(o, ref))})
        for b in (res, y, h, nx, out):
            b.free()
    orn.set_option("fuse_moe_one", 0)
    print(json.dumps({"moe_block_launch_structure": rows}), flush=True)


def warm_cold(orn, ctx, np):
    """What a mat-vec gains when its weights were read just before by another kernel (they then
    sit in the memory-side cache, not in the L2 of the die that needs them), against weights
    nobody read (cycling over > 600 MB of copies) and against one matrix re-used by every launch
    (warm in its own dies' L2). The read before is `ornith_copy` of the code bytes; the setting
    `other` runs the same copy on a matrix that is not used next, so `other` - `touch` is the gain
    and `none` shows what the copy itself costs in this loop. Prints a JSON table."""
    import util
    rng = np.random.default_rng(0)
    scratch = ctx.alloc(64 << 20)
    rows = []
    for name, kind, O, K in (("in_proj 12288x2048 Q4_K", util.Q4K, 12288, 2048), ("out_proj 2048x4096 Q4_K", util.Q4K, 2048, 4096),
                             ("q_proj 8192x2048 Q6_K", util.Q6K, 8192, 2048)):
        t = util.make_kq(kind, rng, 1, O, K)
        ncopy = int(600e6 // sum(a.nbytes for a in t)) + 1
        mats = [orn.KMatrix(ctx, kind, *t, 1, O, K) for _ in range(ncopy)]
        qbytes = t[0].nbytes
        for M in (1, 2):
            x = ctx.to_device(util.bf16_normal(rng, (M, K)))
            y = ctx.alloc(M * O * 2)

            def run(i, mode):
                m = mats[0] if mode == "same" else mats[i % ncopy]
                if mode == "touch":
                    ctx.copy(scratch, m.bufs[0], qbytes)
                elif mode == "other":
                    ctx.copy(scratch, mats[(i + ncopy // 2) % ncopy].bufs[0], qbytes)
                ctx.kq_qmv(m, x, orn.BF16, M, y, orn.BF16)

            row = {"matrix": name, "M": M}
            for mode in ("same", "none", "other", "touch"):
                row[mode + "_us"] = round(_time_loop(ctx, lambda i: run(i, mode), 600, 50), 2)
            rows.append(row)
            x.free(); y.free()
        for m in mats:
            m.free()
    print(json.dumps({"matvec_warm_cold": rows}), flush=True)


def ceiling(orn, ctx, np):
    """What the machine allows a decode launch, measured with the library's probe kernels
    (csrc/probe.hip): the cost of a launch that does nothing, of launches of the expert kernels'
    shapes that only stream their bytes (cold: cycling over > 1 GiB), of a long read, where
    workgroups land, and how long a word stored by one workgroup takes to reach another on the
    same die and on another. Prints one JSON object."""
    lib = orn.lib()
    res = {}
    sink = ctx.alloc(256)

    def probe(rc, what):
        if rc != 0:
            raise orn.OrnithError(f"{what}: {lib.ornith_last_error().decode()}")

    # -- launches that do nothing, back to back. The host enqueues 1000 launches per call: if
    #    the figure does not grow with the grid it is the host's enqueue rate, not the device's.
    rows = []
    for wgs, thr, args_ in ((1, 64, 0), (1152, 256, 0), (1152, 256, 1), (512, 576, 1)):
        probe(lib.ornith_probe_empty(ctx.h, wgs, thr, args_, 200), "probe_empty")
        ctx.sync()
        ctx.timer_begin()
        probe(lib.ornith_probe_empty(ctx.h, wgs, thr, args_, 2000), "probe_empty")
        us = ctx.timer_end() * 1000.0 / 2000
        ms = C.c_float()
        probe(lib.ornith_probe_empty_graph(ctx.h, wgs, thr, args_, 2000, C.byref(ms)), "probe_empty_graph")
        rows.append({"workgroups": wgs, "threads": thr, "argument_block": bool(args_), "us_per_launch": round(us, 2),
                     "us_per_launch_in_a_graph": round(ms.value * 1000.0 / 2000, 2)})
    res["empty_launch"] = rows

    # -- launches of the expert kernels' shapes with the arithmetic taken out
    big = 2 << 30
    buf = ctx.alloc(big)
    lib.ornith_memset(ctx.h, buf.ptr, 1, C.c_size_t(big))
    rows = []
    shapes = (("expert up at T=2: 1152 x 256 threads, 4 x 16 B a thread, contiguous 4 KB a wavefront (18.9 MB)", 1152, 4, 1024),
              ("expert up at T=2, a wavefront's four pieces 1152 B apart as Q4_K rows lie (18.9 MB)", 1152, 4, 1152),
              ("expert down at T=2: 512 x 256 threads, 7 x 16 B a thread (14.7 MB)", 512, 7, 1024),
              ("expert up at T=1: 576 workgroups (9.4 MB)", 576, 4, 1024),
              ("one 4 KB piece a wavefront over 4608 workgroups (75 MB)", 4608, 4, 1024),
              ("lm_head-sized: 17,460 workgroups x 16 KB (286 MB)", 17460, 4, 1024))
    for name, wgs, per, stride in shapes:
        nbytes = wgs * 256 * per * 16
        n = 400 if nbytes < (64 << 20) else 60
        best = 1e30
        for rep in range(4):   # the first pass also warms the launch path; the best of the rest is reported
            ctx.sync()
            ctx.timer_begin()
            probe(lib.ornith_probe_stream(ctx.h, buf.ptr, C.c_size_t(big), wgs, per, C.c_size_t(stride), sink.ptr, n),
                  "probe_stream")
            us = ctx.timer_end() * 1000.0 / n
            if rep:
                best = min(best, us)
        rows.append({"shape": name, "bytes": nbytes, "us_per_launch": round(best, 2),
                     "GB_s": round(nbytes / (best * 1e-6) / 1e9, 1), "frac_of_8TBs": round(nbytes / (best * 1e-6) / 8e12, 3)})
    res["stream_only_launch"] = rows

    # -- one long read
    rows = []
    for mib in (64, 256, 1024, 2048):
        n = mib << 20
        us = _time_loop(ctx, lambda i: probe(lib.ornith_probe_read(ctx.h, buf.ptr, C.c_size_t(n), sink.ptr), "probe_read"), 20, 3)
        rows.append({"MiB": mib, "us": round(us, 1), "GB_s": round(n / (us * 1e-6) / 1e9, 1), "frac_of_8TBs": round(n / (us * 1e-6) / 8e12, 3)})
    res["long_read"] = rows
    buf.free()

    # -- where workgroups land
    n = 2048
    xo = ctx.alloc(n * 4)
    agree = 0
    for rep in range(20):
        probe(lib.ornith_probe_xcc(ctx.h, n, xo.ptr), "probe_xcc")
        ids = xo.download(np.uint32, (n,))
        if rep == 0:
            first = ids[:16].tolist()
            shift = int((ids[0] - 0) % 8)
        agree += int(np.array_equal(ids, (np.arange(n) + shift) % 8))
    res["workgroup_to_xcc"] = {"first_16": first, "rule": f"xcc = (workgroup + {shift}) mod 8", "launches_following_the_rule": agree, "of": 20}
    xo.free()

    # -- a word from one workgroup to another (workgroups 0 and 8 share a die, 0 and 1 do not)
    flag, out4 = ctx.alloc(4096 * 256), ctx.alloc(64)
    flag.zero()
    rows = []
    slot = 0
    for place, cons in (("same XCC", 8), ("another XCC", 1)):
        for mode, mname in ((0, "plain store, agent-scope (sc1) loads"), (1, "sc1 store, sc1 loads"), (2, "plain store, plain loads")):
            lat, xcc = [], None
            for rep in range(9):
                probe(lib.ornith_probe_handoff(ctx.h, C.c_void_p(flag.ptr.value + 256 * slot), out4.ptr, 0, cons, mode), "probe_handoff")
                slot += 1
                o = out4.download(np.int64, (4,))
                xcc = (int(o[2]), int(o[3]))
                lat.append((o[1] - o[0]) / 100.0 if o[1] else None)
            seen = [v for v in lat if v is not None]
            rows.append({"where": place, "how": mname, "xcc_ids": xcc, "seen": len(seen), "of": len(lat),
                         "us_min": round(min(seen), 2) if seen else None, "us_median": round(float(np.median(seen)), 2) if seen else None,
                         "us_max": round(max(seen), 2) if seen else None})
    res["word_between_workgroups"] = rows
    for b in (flag, out4, sink):
        b.free()

    # -- what one vector instruction costs (2048 workgroups x 256 threads x 8 chains x 4096)
    lib.ornith_probe_valu_name.restype = C.c_char_p
    dx = ctx.to_device(np.array([1e-3, 2e-3, 3e-3, 4e-3], np.float32))
    dp = ctx.to_device(np.full(4, 0x47000007, np.uint32))   # halves: f16 7.0 and the f16 subnormal 7 * 2^-24
    wgs, iters = 2048, 4096
    dout = ctx.alloc(wgs * 256 * 4)
    rows = []
    for op in range(lib.ornith_probe_valu_count()):
        best = 1e30
        for rep in range(3):
            ctx.sync()
            ctx.timer_begin()
            probe(lib.ornith_probe_valu(ctx.h, op, wgs, iters, dx.ptr, dp.ptr, dout.ptr), "probe_valu")
            ms = ctx.timer_end()
            if rep:
                best = min(best, ms)
        text = lib.ornith_probe_valu_name(op).decode()
        name = " + ".join(part.split()[0] for part in text.split("\n\t"))   # mnemonics only; a pair counts as one
        rows.append({"instruction": name, "ms": round(best, 3),
                     "T_lane_ops_s": round(wgs * 256 * iters * 8 / (best * 1e-3) / 1e12, 1)})
    res["vector_instruction_rate"] = rows

    # -- what a kernel argument costs: a struct read by a scalar load, or preloaded flat arguments
    didx = ctx.to_device(np.array([3], np.uint32))
    ddata = ctx.alloc(64 << 10)
    ddata.zero()
    wg = 512
    dst = ctx.alloc(wg * 32)
    scrub = ctx.alloc(64 << 20)
    rows = []
    for flat in (0, 1):
        acc = []
        for rep in range(6):
            scrub.zero()   # a launch of something else between two probes, as in a decode step
            probe(lib.ornith_probe_kernarg(ctx.h, flat, wg, didx.ptr, ddata.ptr, dst.ptr), "probe_kernarg")
            st = dst.download(np.int64, (wg, 4)).astype(np.float64) / 100.0
            if rep:
                acc.append([np.mean(st[:, 1] - st[:, 0]), np.mean(st[:, 2] - st[:, 1]), np.mean(st[:, 3] - st[:, 2])])
        m = np.mean(np.array(acc), axis=0)
        rows.append({"arguments": "leading flat arguments (preloaded)" if flat else "one struct (scalar load)",
                     "us_until_the_argument_is_in_a_register": round(float(m[0]), 3),
                     "us_dependent_scalar_load": round(float(m[1]), 3), "us_dependent_vector_load": round(float(m[2]), 3)})
    res["kernel_argument"] = rows
    for b in (dx, dp, dout, didx, ddata, dst, scrub):
        b.free()
    print(json.dumps({"ceiling": res}), flush=True)


def pair_marks(orn, ctx, model, np, n_layers, T):
    """Phase time stamps of the expert up + down pair as the model launches it (one launch of a
    stamped build: `ORN_EXTRA_FLAGS=-DORN_TIMING python ornith-rs_amd/build.py`): every workgroup
    stores the 100 MHz clock at its phase boundaries; printed as percentiles over the launch's
    workgroups, in us after the launch's first workgroup started."""
    lib = orn.lib()
    if not hasattr(lib, "ornith_debug_marks_up"):
        sys.exit("bench.py --pair-marks needs the stamped build: ORN_EXTRA_FLAGS=-DORN_TIMING python ornith-rs_amd/build.py")
    rng = np.random.default_rng(123)
    H, I, E, k = 2048, 512, 256, 8
    moes = [model.moe_weights(i) for i in range(n_layers)]
    x = ctx.to_device(orn.f32_to_bf16(rng.standard_normal((T, H)).astype(np.float32)))
    gates = [ctx.alloc(T * E * 2) for _ in moes]
    egate = ctx.alloc(T * 2)
    inds, scores = ctx.alloc(T * k * 4), ctx.alloc(T * k * 2)
    act, out = ctx.alloc((T * k + T) * I * 2), ctx.alloc(T * H * 2)
    for w, g in zip(moes, gates):
        ctx.linear_matmul(_Lin(w.router), x, T, g)
        ctx.linear_matmul(_Lin(w.sh_egate), x, T, egate)
    us = _time_loop(ctx, lambda i: orn.moe_experts_from_gates(ctx, moes[i % n_layers], x, T, gates[i % n_layers], egate,
                                                              inds, scores, act, out), 200, n_layers)
    orn.moe_experts_from_gates(ctx, moes[n_layers // 2], x, T, gates[n_layers // 2], egate, inds, scores, act, out)
    ctx.sync()
    up = (C.c_longlong * (2048 * 8))()
    down = (C.c_longlong * (1024 * 8))()
    lib.ornith_debug_marks_up(up)
    lib.ornith_debug_marks_down(down)
    a = np.frombuffer(up, np.int64).reshape(2048, 8).astype(np.float64)
    a = a[a[:, 4] > 0]
    d = np.frombuffer(down, np.int64).reshape(1024, 8).astype(np.float64)
    d = d[d[:, 5] > 0]
    t0, t1 = a[:, 0].min(), d[:, 0].min()

    def row(name, v, base):
        v = (v - base) / 100.0
        return {"phase": name, "min": round(float(v.min()), 2), "p10": round(float(np.percentile(v, 10)), 2),
                "median": round(float(np.median(v)), 2), "p90": round(float(np.percentile(v, 90)), 2), "max": round(float(v.max()), 2)}

    routed = a[:, 5] > 0
    res = {"verify_width": T, "us_per_pair_stamped_build": round(us, 2),
           "up": {"workgroups": len(a), "phases": [
               row("start", a[:, 0], t0), row("gates in registers (routed workgroups)", a[routed, 6], t0),
               row("routing made (routed workgroups)", a[routed, 5], t0),
               row("weight loads issued", a[:, 1], t0), row("activations loaded", a[:, 2], t0),
               row("first two rows done", a[:, 3], t0), row("end", a[:, 4], t0),
               row("shared expert's workgroups: weight loads issued", a[~routed, 1], t0),
               row("shared expert's workgroups: end", a[~routed, 4], t0)]},
           "down": {"workgroups": len(d), "starts_us_after_the_up_launch": round(float((t1 - t0) / 100.0), 2), "phases": [
               row("start", d[:, 0], t1), row("weight loads issued", d[:, 1], t1), row("activations loaded", d[:, 2], t1),
               row("sums done (wavefront 0)", d[:, 3], t1), row("after the barrier", d[:, 4], t1), row("end", d[:, 5], t1)]}}
    if hasattr(lib, "ornith_debug_marks_down_waves"):
        # per wavefront of the down launch's workgroups (j < k: routed slot j, j >= k: the shared expert)
        wv = (C.c_longlong * (1024 * 32))()
        lib.ornith_debug_marks_down_waves(wv)
        w = np.frombuffer(wv, np.int64).reshape(1024, 32).astype(np.float64)[:len(d)]
        nw = int((w[0, :16] > 0).sum())
        res["down"]["by_wavefront_median_us"] = [
            {"wavefront": j, "rows_in_registers": round(float(np.median(w[:, j] - t1) / 100.0), 2),
             "sums_done": round(float(np.median(w[:, 16 + j] - t1) / 100.0), 2)} for j in range(nw)]
    print(json.dumps({"pair_marks": res}), flush=True)


def config5(args, orn, ctx, synth, np, model, ws, cfg, dev_name):
    """BASELINE config 5: sampled speculative decode at depth 3 after a long prefill. Runs the
    whole sequence twice (the second run is the one reported; the two must give the same tokens)
    and returns its figures."""
    depth, n_prompt, n_gen, cap = 3, 6621, (1 if args.prefill_only else 256), 16384
    model.set_max_rows(args.prefill_chunk)
    caches = model.make_cache(cap, depth + 1)
    head = orn.MtpHead(model, ws, cap)
    fr_ids = synth.zipf_frspec_ids(cfg["vocab_size"], 32768, seed=1)
    fr = orn.FrSpec(model, ids=fr_ids)
    rng = np.random.default_rng(6621)
    prompt = rng.integers(0, cfg["vocab_size"], n_prompt).astype(np.uint32)
    accept = orn.ACCEPT_RATIO if args.accept == "ratio" else orn.ACCEPT_EQUALITY
    gen = orn.RNG_PHILOX if args.rng == "philox" else orn.RNG_THREEFRY
    smp = orn.Sampler(1, 0.8, 0.95, 0, 2025, accept, gen)
    res = []
    for it in range(2):
        caches.reset()
        mark = {}

        def progress(done, total):
            ctx.sync()
            if done == 0:
                mark["p0"] = time.perf_counter()
            if done == total:
                mark["p1"] = time.perf_counter()

        toks, st = orn.generate_step_mtp(model, head, fr, caches, prompt, depth, n_gen, sampler=smp,
                                         prefill_step=args.prefill_chunk, policy=orn.HISTORY_COMMITTED,
                                         progress=progress)
        ctx.sync()
        t_end = time.perf_counter()
        res.append((toks, st, mark["p1"] - mark["p0"], t_end - mark["p1"]))
        log(f"config5 run {it}: prefill {res[-1][2]:.3f} s ({n_prompt / res[-1][2]:.0f} tok/s), decode "
            f"{n_gen / res[-1][3]:.1f} tok/s, {int(st.cycles)} cycles, {int(st.accepted)}/{int(st.drafted)} accepted")
    assert res[0][0] == res[1][0], "same seed, different tokens"
    toks, st, t_pre, t_dec = res[-1]
    # active weight bytes per prompt token are read once per chunk; the GEMM work is 2 flops per
    # active weight per token: projections + router + shared expert + 8 routed experts, 40 layers
    H, I = 2048, 512
    per_layer_gdn = H * (8192 + 4096) + 4096 * H
    per_layer_att = H * (8192 + 512 + 512) + 4096 * H
    per_layer_moe = H * 256 + 9 * 3 * H * I
    flops_tok = 2.0 * (30 * per_layer_gdn + 10 * per_layer_att + 40 * per_layer_moe)
    line = {"workload": f"config5: {n_prompt}-token prefill (chunks of {args.prefill_chunk}) into a {cap}-token context, "
                        f"then sampled MTP depth-{depth} + FR-Spec decode of {n_gen} tokens (temperature 0.8, top-p 0.95, "
                        f"{'probability-ratio (rejection-sampling)' if args.accept == 'ratio' else 'token-equality'} "
                        f"acceptance, seeded {'Philox4x32-10' if args.rng == 'philox' else 'threefry'} stream)",
            "prefill_s": round(t_pre, 4), "prefill_tok_s": round(n_prompt / t_pre, 1),
            "prefill_gemm_tflops": round(flops_tok * n_prompt / t_pre / 1e12, 2),
            "prefill_frac_of_bf16_mfma_peak": round(flops_tok * n_prompt / t_pre / 2.5e15, 4),
            "decode_tok_s": round(n_gen / t_dec, 2), "cycles": int(st.cycles), "drafted": int(st.drafted),
            "accepted": int(st.accepted), "accepted_tokens_per_verify_step": round(int(st.accepted) / max(1, int(st.cycles)), 4),
            "tokens_per_verify_step": round(n_gen / max(1, int(st.cycles)), 3),
            "repeatable": True, "device": dev_name, "data": "synthetic"}
    for o in (fr, head, caches):
        o.close()
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--tokens", type=int, default=200)
    ap.add_argument("--depth", type=int, default=1)
    ap.add_argument("--layers", type=int, default=40, help="trunk layers (40 = the named config)")
    ap.add_argument("--cpu-tokens", type=int, default=40)
    ap.add_argument("--no-cpu", action="store_true", help="skip every leg that runs the CPU oracle")
    ap.add_argument("--config5", action="store_true",
                    help="instead of the metric's workload: BASELINE config 5 (6621-token prefill into a "
                         "16384-token context through the matrix-core path, then sampled depth-3 MTP "
                         "decode of 256 tokens, temperature 0.8, top-p 0.95); prints its own JSON line")
    ap.add_argument("--accept", choices=("ratio", "equality"), default="ratio",
                    help="with --config5: probability-ratio (rejection-sampling) acceptance, or the reference's token equality")
    ap.add_argument("--rng", choices=("philox", "threefry"), default="philox",
                    help="with --config5: the sampler's random stream")
    ap.add_argument("--prefill-chunk", type=int, default=8192,
                    help="rows per prefill call with --config5 (the reference's prefill_step_size is 2048; up to 8192 "
                         "here: by default the 6621-token prompt is one call)")
    ap.add_argument("--prefill-only", action="store_true",
                    help="with --config5: stop after the first generated token (a short run for "
                         "profiling the matrix-core prefill kernels)")
    ap.add_argument("--roofline-only", action="store_true",
                    help="only the expert-kernel timing loops plus three 256 MiB device copies "
                         "(the known-size reference for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--overlap", choices=("distinct", "same8"), default=None,
                    help="only the expert pair under the named routing at T = 2 (all tokens on the same 8 experts, "
                         "or on 16 distinct ones), then three 256 MiB device copies: one rocprofv3 --pmc run a case")
    ap.add_argument("--moe-ab", action="store_true",
                    help="only the A/B of the MoE block's launch structure (option fuse_moe_one = 0, 1, 2)")
    ap.add_argument("--ceiling", action="store_true",
                    help="only the machine probes: empty launches, stream-only launches of the expert kernels' shapes, "
                         "a long read, the workgroup-to-die rule, the latency of a word between workgroups, the rate "
                         "of single vector instructions, the cost of a kernel argument")
    ap.add_argument("--pair-marks", action="store_true",
                    help="only the phase time stamps of the expert pair (needs the library built with -DORN_TIMING)")
    ap.add_argument("--warm-cold", action="store_true",
                    help="only the mat-vec timings on re-used, unread and just-read weights")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (one process, one stream); "
                 "--gpus N with N > 1 is not supported and nothing here uses a second device.")

    import numpy as np
    import synth
    orn = importlib.import_module("ornith-rs_amd")
    ctx = orn.Ctx(0)
    dev_name, cus, mem = ctx.device_info()
    log(f"device: {dev_name}, {cus} CUs, {mem / 2**30:.0f} GiB")

    if args.ceiling:
        return ceiling(orn, ctx, np)
    if args.warm_cold:
        return warm_cold(orn, ctx, np)
    cfg = dict(synth.FULL, num_hidden_layers=args.layers)
    t0 = time.time()
    sm = synth.SynthModel(cfg, seed=2025)
    log(f"synthetic weights: {sm.total_bytes() / 1e9:.2f} GB generated in {time.time() - t0:.1f} s")
    t0 = time.time()
    ws = sm.upload(orn, ctx)
    log(f"uploaded in {time.time() - t0:.1f} s")
    model = orn.TextModel(ctx, ws, sm.text_config(orn))
    if args.roofline_only:
        roof = expert_roofline(orn, ctx, model, np, args.layers, T=args.depth + 1, pairs=200)
        a, b = ctx.alloc(256 << 20), ctx.alloc(256 << 20)
        for _ in range(3):
            ctx.copy(a, b, 256 << 20)
        ctx.sync()
        print(json.dumps({"roofline": roof}), flush=True)
        return
    if args.overlap:
        rows = expert_overlap(orn, ctx, model, np, args.layers, cases=(args.overlap,), widths=(2,), pairs=200)
        a, b = ctx.alloc(256 << 20), ctx.alloc(256 << 20)
        for _ in range(3):
            ctx.copy(a, b, 256 << 20)
        ctx.sync()
        print(json.dumps({"overlapping_routing": rows}), flush=True)
        return
    if args.moe_ab:
        return moe_ab(orn, ctx, model, np, args.layers)
    if args.pair_marks:
        return pair_marks(orn, ctx, model, np, args.layers, args.depth + 1)
    if args.config5:
        print(json.dumps(config5(args, orn, ctx, synth, np, model, ws, cfg, dev_name)), flush=True)
        return
    rng = np.random.default_rng(51)
    prompt = rng.integers(0, cfg["vocab_size"], 51).astype(np.uint32)
    cap = 4096
    caches = model.make_cache(cap, args.depth + 1)
    head = orn.MtpHead(model, ws, cap)
    fr_ids = synth.zipf_frspec_ids(cfg["vocab_size"], 32768, seed=1)
    fr = orn.FrSpec(model, ids=fr_ids)

    def timed_run(fn):
        """fn(progress) -> tokens; returns (tokens, decode seconds). Both loops report the
        prompt consumed at the same point: after its last position has been sampled from."""
        mark = {}

        def progress(done, total):
            if done == total:
                ctx.sync()
                mark["t0"] = time.perf_counter()

        out = fn(progress)
        ctx.sync()
        return out, time.perf_counter() - mark["t0"]

    # plain greedy, for the byte-identity check and as the non-speculative figure
    caches.reset()
    orn.generate_step(model, caches, prompt, 8, prefill_step=16)      # warm the shapes
    caches.reset()
    ar, ar_s = timed_run(lambda pr: orn.generate_step(model, caches, prompt, args.tokens, prefill_step=16, progress=pr))
    log(f"plain greedy: {len(ar)} tokens in {ar_s * 1e3:.1f} ms = {len(ar) / ar_s:.1f} tok/s")

    times, stats, toks = [], None, None
    for it in range(args.warmup + args.steps):
        caches.reset()
        (toks, stats), dt = timed_run(lambda pr: orn.generate_step_mtp(
            model, head, fr, caches, prompt, args.depth, args.tokens, prefill_step=16,
            policy=orn.HISTORY_COMMITTED, progress=pr))
        if toks != ar:
            sys.exit("bench.py: speculative output is NOT identical to plain greedy -- result invalid")
        if it >= args.warmup:
            times.append(dt)
        log(f"mtp depth {args.depth} run {it}: {dt * 1e3:.1f} ms, {int(stats.cycles)} cycles, "
            f"{int(stats.accepted)}/{int(stats.drafted)} accepted")
    total_s = sum(times)
    tok_s = args.tokens * len(times) / total_s

    # Forced acceptance: random-init weights accept no draft, so `value` is the floor of the
    # loop. With the known output as the drafts every draft is accepted and a cycle yields
    # depth + 1 tokens: the ceiling. The head still runs for every draft.
    forced = {}
    c2 = model.make_cache(cap, 4)
    head.force_drafts(ar)
    for d in (1, 2, 3):
        for it in range(2):   # the first run warms the shapes of this depth
            c2.reset()
            (ft, fst), fdt = timed_run(lambda pr: orn.generate_step_mtp(
                model, head, fr, c2, prompt, d, args.tokens, prefill_step=16,
                policy=orn.HISTORY_COMMITTED, progress=pr))
            if ft != ar:
                sys.exit("bench.py: forced-draft output is NOT identical to plain greedy -- result invalid")
        forced[f"depth{d}"] = {"tok_s": round(args.tokens / fdt, 1), "cycles": int(fst.cycles),
                               "accepted": int(fst.accepted), "drafted": int(fst.drafted)}
        log(f"forced acceptance depth {d}: {args.tokens / fdt:.1f} tok/s, {int(fst.cycles)} cycles, "
            f"{int(fst.accepted)}/{int(fst.drafted)} accepted")
    head.force_drafts([])
    c2.close()

    by_width = [expert_roofline(orn, ctx, model, np, args.layers, T) for T in (1, 2, 4)]
    main_w = next(w for w in by_width if w["verify_width"] == 2)
    roof = {"bound": "hbm", "achieved": main_w["achieved"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": main_w["frac"],
            "traffic": PROFILE_TRAFFIC["pair"]["bytes"], "traffic_from_profile": PROFILE_TRAFFIC,
            "kernel": "moe_up_kernel<Q4_K, 64, 2, routing made in the launch> + moe_down_kernel<Q6_K, 8, 2>: the expert "
                      "gather-GEMV of one MoE block as the model launches it (gate + up + swiglu, down + combine), "
                      "verify width 2, the router's own picks",
            "us_per_launch": main_w["us_per_pair"], "launches_per_unit": 2, "bytes_per_launch": main_w["bytes_per_pair"],
            "distinct_experts": main_w["distinct_experts_mean"], "verify_width": 2, "by_width": by_width,
            "overlapping_routing": expert_overlap(orn, ctx, model, np, args.layers)}
    log("roofline:", roof)

    # Whole-step figures: the algorithmic bytes one decode step has to read (and the recurrent
    # state it writes) against the time the step takes. Dense projections of 30 gated-delta and
    # 10 attention layers, per MoE block the router + (distinct routed + 1) experts, the output
    # head (all 248,320 rows of Q4_K), 2 MiB of recurrent state a gated-delta layer read once and
    # written once per row, the KV rows of a context of about 150 tokens. The depth-1 cycle adds
    # the draft: the bf16 head layer (129 MB) and the 32,768-row pruned output head.
    dense = 30 * 19_202_048 + 10 * 22_364_160
    head_full, head_pruned, mtp_layer = 286_064_640, 37_748_736, 129_000_000
    state = 30 * 2_097_152
    kv = 10 * 2 * 2 * 150 * 256 * 2

    def step_bytes(T, U):
        return dense + 40 * ((U + 1) * EXPERT_BYTES + 430_080) + head_full + state * (1 + T) + kv

    u1 = next(w for w in by_width if w["verify_width"] == 1)["distinct_experts_mean"]
    u2 = main_w["distinct_experts_mean"]
    plain_ms = ar_s / len(ar) * 1e3
    cycle_ms = total_s / len(times) / max(1, int(stats.cycles)) * 1e3
    b_plain, b_cycle = step_bytes(1, u1), step_bytes(2, u2) + mtp_layer + head_pruned
    step_roof = {"plain_greedy": {"bytes_per_token": int(b_plain), "ms_per_token": round(plain_ms, 4),
                                  "GB_s": round(b_plain / plain_ms / 1e6, 1), "frac_of_hbm_peak": round(b_plain / plain_ms / 1e6 / HBM_PEAK_GBS, 4)},
                 "mtp_depth1_cycle": {"bytes_per_cycle": int(b_cycle), "ms_per_cycle": round(cycle_ms, 4),
                                      "GB_s": round(b_cycle / cycle_ms / 1e6, 1), "frac_of_hbm_peak": round(b_cycle / cycle_ms / 1e6 / HBM_PEAK_GBS, 4)}}
    log("step_roofline:", step_roof)

    configs = per_config(orn, ctx, np, with_cpu=not args.no_cpu)
    # config 5 (sampled depth-3 decode behind a 6621-token matrix-core prefill) on the same model
    for o in (fr, head, caches):
        o.close()
    configs["config5"] = config5(args, orn, ctx, synth, np, model, ws, cfg, dev_name)
    log("per_config:", configs)

    cpu = None
    if not args.no_cpu:
        cpu, cpu_toks = cpu_baseline(synth, sm, np, args.depth, args.cpu_tokens, prompt)
        # the same tokens must have come out of the GPU
        cpu["gpu_tokens_match"] = bool(ar[:len(cpu_toks)] == cpu_toks)
        log("cpu_baseline:", cpu)

    line = {
        "metric": "decode tok/s @MTP depth 1 (1 GPU, byte-exact); expert GEMV HBM GB/s vs peak",
        "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(total_s / len(times) * 1e3, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "value_is": "the zero-acceptance floor of the depth-1 loop (random-init weights accept no draft: one token per "
                    "two-row verify + draft); see plain_greedy_tok_s and forced_acceptance_ceiling beside it",
        "plain_greedy_tok_s": round(len(ar) / ar_s, 2),
        "forced_acceptance_ceiling": forced,
        "config": {"workload": f"config4: greedy MTP depth-{args.depth} + FR-Spec(32768) decode of {args.tokens} tokens, "
                               f"51-token prompt, Qwen3.5-35B-A3B shape, {args.layers} layers, KV capacity {cap}",
                   "arithmetic": "bf16 activations, fp32 accumulation, Q4_K/Q6_K/int8/bf16 weights",
                   "tokens_per_step": args.tokens, "byte_identical_to_greedy": True,
                   "cycles": int(stats.cycles), "accepted": int(stats.accepted), "drafted": int(stats.drafted),
                   "weights_GB": round(ws.stats()[1] / 1e9, 2), "device": dev_name},
        "roofline": roof,
        "step_roofline": step_roof,
        "per_config": configs,
        "cpu_baseline": cpu,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
