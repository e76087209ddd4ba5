"""The committed fixtures of tests/golden (written by tests/golden/make_golden.py from the
pinned oracle): the oracle built from source still reproduces them (CPU), and the HIP path
reproduces them without the oracle in the loop (GPU)."""
import json
import os

import numpy as np
import pytest

import synth
import util

G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _tiny():
    j = json.load(open(os.path.join(G, "tiny_model_tokens.json")))
    return j, synth.SynthModel(synth.TINY, seed=j["model_seed"]), np.array(j["prompt"], np.uint32)


def test_oracle_reproduces_fixtures():
    f = np.load(os.path.join(G, "q4k_qmv_128x2048.npz"))
    y = util.orc_qmv(util.Q4K, f["qs"], f["scales"], f["dm"], 128, 2048, f["x"])
    assert np.array_equal(y.view(np.uint32), f["y_oracle"].view(np.uint32))
    rel = np.linalg.norm(y[0] - f["y_float64"]) / np.linalg.norm(f["y_float64"])
    assert rel <= 1e-5          # BASELINE config 1's tolerance against the float64 mat-vec
    f = np.load(os.path.join(G, "q6k_qmv_64x1024.npz"))
    y6 = util.f32_to_bf16(util.orc_qmv(util.Q6K, f["qs"], f["scales"], f["dm"], 64, 1024, util.bf16_to_f32(f["x"]), round_bf16=True))
    assert np.array_equal(y6, f["y"])
    j, s, prompt = _tiny()
    orc = synth.OracleRun(s, 64)
    assert orc.generate(prompt, 12, prefill_step=4) == j["greedy"]
    orc.close()


@pytest.mark.gpu
def test_hip_reproduces_fixtures(orn, ctx):
    f = np.load(os.path.join(G, "q4k_qmv_128x2048.npz"))
    w = orn.KMatrix(ctx, orn.Q4K, f["qs"], f["scales"], f["dm"], 1, 128, 2048)
    dx, dy = ctx.to_device(f["x"]), ctx.alloc(128 * 4)
    ctx.kq_qmv(w, dx, orn.F32, 1, dy, orn.F32)
    assert np.array_equal(dy.download(np.float32, (1, 128)).view(np.uint32), f["y_oracle"].view(np.uint32))
    w.free(); dx.free(); dy.free()
    f = np.load(os.path.join(G, "q6k_qmv_64x1024.npz"))
    w = orn.KMatrix(ctx, orn.Q6K, f["qs"], f["scales"], f["dm"], 1, 64, 1024)
    dx, dy = ctx.to_device(f["x"]), ctx.alloc(2 * 64 * 2)
    ctx.kq_qmv(w, dx, orn.BF16, 2, dy, orn.BF16)
    assert np.array_equal(dy.download(np.uint16, (2, 64)), f["y"])
    w.free(); dx.free(); dy.free()
    f = np.load(os.path.join(G, "router_topk_4x256.npz"))
    dg, di, ds, dp = ctx.to_device(f["gates"]), ctx.alloc(4 * 8 * 4), ctx.alloc(4 * 8 * 2), ctx.alloc(4 * 256 * 2)
    ctx.router_topk(dg, 4, 256, 8, di, ds, dp)
    assert np.array_equal(di.download(np.uint32, (4, 8)), f["inds"])
    assert np.array_equal(ds.download(np.uint16, (4, 8)), f["scores"])
    assert np.array_equal(dp.download(np.uint16, (4, 256)), f["probs"])
    for b in (dg, di, ds, dp): b.free()
    j, s, prompt = _tiny()
    ws = s.upload(orn, ctx)
    model = orn.TextModel(ctx, ws, s.text_config(orn))
    caches = model.make_cache(64, 4)
    assert orn.generate_step(model, caches, prompt, 12, prefill_step=4) == j["greedy"]
    head = orn.MtpHead(model, ws, 64)
    caches.reset()
    toks, st = orn.generate_step_mtp(model, head, None, caches, prompt, 2, 12, prefill_step=4)
    assert toks == j["greedy"]
    assert {"cycles": int(st.cycles), "drafted": int(st.drafted), "accepted": int(st.accepted)} == j["mtp_depth2"]
    caches.reset()
    got = orn.generate_step(model, caches, prompt, 12, sampler=orn.Sampler(1, 0.8, 0.95, 20, 99), prefill_step=4)
    assert got == j["sampled_t0.8_p0.95_k20_seed99"]
    for o in (head, caches, model, ws): o.close()
