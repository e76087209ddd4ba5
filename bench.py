"""Benchmark of the speculative decode step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--tokens 200] [--depth 1]

Workload (BASELINE.json configs[3], the configuration the metric is quoted on): a seeded,
random-init Qwen3.5-35B-A3B-shaped model (40 layers = 30 gated-delta + 10 full attention,
256-expert top-8 MoE + shared expert, Q4_K/Q6_K/8-bit mix, vocab 248320, one-layer bf16
MTP head, FR-Spec draft vocabulary of 32768 ids), 51-token seeded prompt, greedy depth-1
MTP decode of 200 tokens, whose output must be byte-identical to plain greedy decode.
A "step" is one such 200-token generation; the timed region starts when the prompt has
been consumed (weights, caches and prompt state are resident in HBM) and `value` is
generated tokens per second.

Also measured in the same run and printed on the same JSON line:
  roofline      the expert gate+up gather-GEMV kernel (the largest share of the step):
                algorithmic bytes per launch (distinct routed experts + the shared one,
                two Q4_K matrices each, + activations) over the average launch duration
                from HIP events on the library's stream, against 8 TB/s
  cpu_baseline  the CPU oracle running the same loop on the host cores (bounded sample)
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

# HBM bytes per launch of the expert gate+up kernel at verify width 2 (17 distinct experts),
# from two `rocprofv3 --pmc` runs of `bench.py --roofline-only` (FETCH_SIZE, then WRITE_SIZE,
# KiB per dispatch), each scaled by what the same counter reads for the 256 MiB device copies
# that run issues: FETCH_SIZE 9866.6 x 2.0 (the copy reads 131,086 for 262,144 KiB),
# WRITE_SIZE 36.0 x 1.0. Counters cannot be read from inside this script; other widths: null.
PMC_TRAFFIC_BYTES = {2: int(round((9866.6 * 2.0 + 36.0 * 1.0) * 1024))}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def expert_gemv_roofline(orn, ctx, model, util, np, n_layers, T, launches=800):
    """Times the expert gate+up gather-GEMV kernel (Q4_K: top-8 of 256 routed experts plus the
    shared expert, gate and up projections and swiglu in one launch) at verify width T on the
    model's resident weights, cycling through every layer so no launch finds its experts in
    cache. Algorithmic bytes per launch: (distinct routed experts + 1) x 2 matrices x 512 x
    2048 weights x 144/256 bytes, plus the activations read and written."""
    rng = np.random.default_rng(123)
    H, I, E, k = 2048, 512, 256, 8
    moes = [model.moe_weights(i) for i in range(n_layers)]
    xb = util.f32_to_bf16(rng.standard_normal((T, H)).astype(np.float32))
    inds = np.concatenate([rng.permutation(E)[:k] for _ in range(T)]).astype(np.uint32)
    U = len(np.unique(inds))
    scores = util.f32_to_bf16(rng.random((T, k)).astype(np.float32))
    eg = util.f32_to_bf16(rng.standard_normal(T).astype(np.float32))
    dx, di, ds, de = ctx.to_device(xb), ctx.to_device(inds), ctx.to_device(scores), ctx.to_device(eg)
    act, out = ctx.alloc((T * k + T) * I * 2), ctx.alloc(T * H * 2)
    for w in moes:
        orn.moe_experts(ctx, w, dx, T, di, ds, de, act, out, 1)
    ctx.sync()
    ctx.timer_begin()
    for i in range(launches):
        orn.moe_experts(ctx, moes[i % len(moes)], dx, T, di, ds, de, act, out, 1)
    us = ctx.timer_end() * 1000.0 / launches
    bytes_per_launch = (U + 1) * 2 * I * (H // 256) * 144 + T * H * 2 + (T * k + T) * I * 2 + T * k * 4
    for b in (dx, di, ds, de, act, out):
        b.free()
    achieved = bytes_per_launch / (us * 1e-6) / 1e9
    return {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": PMC_TRAFFIC_BYTES.get(T) if U == 16 else None,
            "kernel": "moe_up_kernel<0, 64, 2, false> (Q4_K expert gate+up gather-GEMV + swiglu, expert ids given)",
            "us_per_launch": round(us, 3), "bytes_per_launch": int(bytes_per_launch),
            "distinct_experts": int(U), "verify_width": int(T)}


def cpu_baseline(synth, synth_model, np, depth, tokens):
    """The oracle's generate_step_mtp on the host cores, whole call timed."""
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    rng = np.random.default_rng(99)
    prompt = rng.integers(0, synth_model.cfg["vocab_size"], 2).astype(np.uint32)
    fr_ids = synth.zipf_frspec_ids(synth_model.cfg["vocab_size"], 32768, seed=1)
    fr_host = synth.prune_head(synth_model.lm_head, fr_ids)
    run = synth.OracleRun(synth_model, 64)
    t0 = time.time()
    toks, st = run.mtp_generate(prompt, depth, tokens, fr_ids, fr_host, policy=1, prefill_step=16)
    dt = time.time() - t0
    run.close()
    return {"value": round(len(toks) / dt, 4), "unit": "tok/s", "cores": threads, "kind": "port",
            "sample": f"oracle generate_step_mtp depth {depth} + FR-Spec, 2-token prompt, {len(toks)} tokens, "
                      f"whole call {dt:.1f} s ({int(st.cycles)} cycles, {int(st.accepted)} accepted)"}, toks, prompt


def config5(args, orn, ctx, synth, np, model, ws, cfg, dev_name):
    """BASELINE config 5: sampled speculative decode at depth 3 after a long prefill."""
    depth, n_prompt, n_gen, cap = 3, 6621, (1 if args.prefill_only else 256), 16384
    model.set_max_rows(args.prefill_chunk)
    caches = model.make_cache(cap, depth + 1)
    head = orn.MtpHead(model, ws, cap)
    fr_ids = synth.zipf_frspec_ids(cfg["vocab_size"], 32768, seed=1)
    fr = orn.FrSpec(model, ids=fr_ids)
    rng = np.random.default_rng(6621)
    prompt = rng.integers(0, cfg["vocab_size"], n_prompt).astype(np.uint32)
    smp = orn.Sampler(1, 0.8, 0.95, 0, 2025)
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
                        "seeded threefry keys)",
            "prefill_s": round(t_pre, 4), "prefill_tok_s": round(n_prompt / t_pre, 1),
            "prefill_gemm_tflops": round(flops_tok * n_prompt / t_pre / 1e12, 2),
            "prefill_frac_of_bf16_mfma_peak": round(flops_tok * n_prompt / t_pre / 2.5e15, 4),
            "decode_tok_s": round(n_gen / t_dec, 2), "cycles": int(st.cycles), "drafted": int(st.drafted),
            "accepted": int(st.accepted), "tokens_per_verify_step": round(n_gen / max(1, int(st.cycles)), 3),
            "repeatable": True, "device": dev_name, "data": "synthetic"}
    print(json.dumps(line), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--tokens", type=int, default=200)
    ap.add_argument("--depth", type=int, default=1)
    ap.add_argument("--layers", type=int, default=40, help="trunk layers (40 = the named config)")
    ap.add_argument("--cpu-tokens", type=int, default=48)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--config5", action="store_true",
                    help="instead of the metric's workload: BASELINE config 5 (6621-token prefill into a "
                         "16384-token context through the matrix-core path, then sampled depth-3 MTP "
                         "decode of 256 tokens, temperature 0.8, top-p 0.95); prints its own JSON line")
    ap.add_argument("--prefill-chunk", type=int, default=4096,
                    help="rows per prefill call with --config5 (the reference's prefill_step_size is 2048; up to 4096 here)")
    ap.add_argument("--prefill-only", action="store_true",
                    help="with --config5: stop after the first generated token (a short run for "
                         "profiling the matrix-core prefill kernels)")
    ap.add_argument("--roofline-only", action="store_true",
                    help="only the expert-kernel timing loop plus three 256 MiB device copies "
                         "(the known-size reference for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (one process, one stream); "
                 "--gpus N with N > 1 is not supported and nothing here uses a second device.")

    import numpy as np
    import synth
    import util
    orn = importlib.import_module("ornith-rs_amd")
    ctx = orn.Ctx(0)
    dev_name, cus, mem = ctx.device_info()
    log(f"device: {dev_name}, {cus} CUs, {mem / 2**30:.0f} GiB")

    cfg = dict(synth.FULL, num_hidden_layers=args.layers)
    t0 = time.time()
    sm = synth.SynthModel(cfg, seed=2025)
    log(f"synthetic weights: {sm.total_bytes() / 1e9:.2f} GB generated in {time.time() - t0:.1f} s")
    t0 = time.time()
    ws = sm.upload(orn, ctx)
    log(f"uploaded in {time.time() - t0:.1f} s")
    model = orn.TextModel(ctx, ws, sm.text_config(orn))
    if args.roofline_only:
        roof = expert_gemv_roofline(orn, ctx, model, util, np, args.layers, T=args.depth + 1, launches=200)
        a, b = ctx.alloc(256 << 20), ctx.alloc(256 << 20)
        for _ in range(3):
            ctx.copy(a, b, 256 << 20)
        ctx.sync()
        print(json.dumps({"roofline": roof}), flush=True)
        return
    if args.config5:
        return config5(args, orn, ctx, synth, np, model, ws, cfg, dev_name)
    rng = np.random.default_rng(51)
    prompt = rng.integers(0, cfg["vocab_size"], 51).astype(np.uint32)
    cap = 4096
    caches = model.make_cache(cap, args.depth + 1)
    head = orn.MtpHead(model, ws, cap)
    fr_ids = synth.zipf_frspec_ids(cfg["vocab_size"], 32768, seed=1)
    fr = orn.FrSpec(model, ids=fr_ids)

    def timed_run(fn):
        """fn(progress) -> tokens; returns (tokens, decode seconds, extra)."""
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

    roof = expert_gemv_roofline(orn, ctx, model, util, np, args.layers, T=args.depth + 1)
    log("roofline:", roof)

    cpu = None
    if not args.no_cpu:
        cpu, cpu_toks, cpu_prompt = cpu_baseline(synth, sm, np, args.depth, args.cpu_tokens)
        # the same short run on the GPU must give the same tokens
        caches.reset()
        g, _ = orn.generate_step_mtp(model, head, fr, caches, cpu_prompt, args.depth, args.cpu_tokens,
                                     prefill_step=16, policy=orn.HISTORY_COMMITTED)
        cpu["gpu_tokens_match"] = bool(g == cpu_toks)
        log("cpu_baseline:", cpu)

    line = {
        "metric": "decode tok/s @MTP depth 1 (1 GPU, byte-exact); expert GEMV HBM GB/s vs peak",
        "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(total_s / len(times) * 1e3, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"config4: greedy MTP depth-{args.depth} + FR-Spec(32768) decode of {args.tokens} tokens, "
                               f"51-token prompt, Qwen3.5-35B-A3B shape, {args.layers} layers, KV capacity {cap}",
                   "arithmetic": "fp32 accumulate over bf16 activations and Q4_K/Q6_K/int8/bf16 weights",
                   "tokens_per_step": args.tokens, "byte_identical_to_greedy": True,
                   "plain_greedy_tok_s": round(len(ar) / ar_s, 2),
                   "cycles": int(stats.cycles), "accepted": int(stats.accepted), "drafted": int(stats.drafted),
                   "forced_acceptance_ceiling": forced,
                   "weights_GB": round(ws.stats()[1] / 1e9, 2), "device": dev_name},
        "roofline": roof,
        "cpu_baseline": cpu,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
