"""A model read from artifact files (sharded safetensors + index + config.json + the MTP
sidecar) must be the model the by-name store gives: same device bytes, same tokens from both
generation loops. Follows the relation the reference's loader test asserts -- what is loaded
agrees with what config.json says about it (/root/reference/src/weights.rs:296-362)."""
import json
import os

import numpy as np
import pytest

import synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def artifact(tmp_path_factory):
    s = synth.SynthModel(synth.TINY, seed=21)
    d = str(tmp_path_factory.mktemp("artifact") / "model")
    side = synth.write_artifact(s, d, shards=3)
    return s, d, side


def test_tensors_arrive_unchanged_and_on_demand(orn, ctx, artifact):
    s, d, side = artifact
    ws = orn.WeightStore.open(ctx, d, extra=[side])
    assert ws.stats() == (0, 0)                      # nothing resident before first use
    for n in ("language_model.model.layers.1.linear_attn.in_proj_qkv.weight",
              "language_model.model.layers.2.mlp.switch_mlp.up_proj.scales",
              "language_model.model.norm.weight", "mtp.fc.weight"):
        arr, code = s.tensors[n]
        assert ws.has(n)
        dt, shape, raw = ws.fetch(n)
        assert (dt, shape) == (code, arr.shape)
        assert raw.tobytes() == arr.tobytes()
    assert ws.stats()[0] == 4
    dt, shape, raw = ws.fetch("language_model.model.norm.weight")   # cached, not copied again
    assert ws.stats()[0] == 4
    assert not ws.has("mtp.layers.0.mlp.switch_mlp.gate_proj.weight")
    assert ws.quant_config("language_model.lm_head") == (256, 4, orn.QM_Q4K)
    assert ws.quant_config("language_model.model.layers.0.mlp.switch_mlp.down_proj") == (256, 6, orn.QM_Q6K)
    assert ws.quant_config("language_model.model.embed_tokens") == (64, 8, orn.QM_AFFINE)
    with pytest.raises(orn.OrnithError, match="no tensor named"):
        ws.fetch("nope")
    ws.close()


def test_model_from_files_generates_the_same_tokens(orn, ctx, artifact):
    s, d, side = artifact
    cfg, mtp_layers = orn.TextConfig.load(d)
    assert mtp_layers == 1
    rng = np.random.default_rng(3)
    prompt = rng.integers(0, s.cfg["vocab_size"], 9).astype(np.uint32)
    fr_ids = synth.zipf_frspec_ids(s.cfg["vocab_size"], 512, seed=2)

    def run(ws, config):
        model = orn.TextModel(ctx, ws, config)
        head = orn.MtpHead(model, ws, 64)
        fr = orn.FrSpec(model, ids=fr_ids)
        caches = model.make_cache(64, 4)
        greedy = orn.generate_step(model, caches, prompt, 12, prefill_step=4)
        caches.reset()
        spec, stats = orn.generate_step_mtp(model, head, fr, caches, prompt, 2, 12, prefill_step=4)
        for o in (fr, head, caches, model):
            o.close()
        return greedy, spec, int(stats.cycles)

    ws_put = s.upload(orn, ctx)
    want = run(ws_put, s.text_config(orn))
    n_put, bytes_put = ws_put.stats()
    ws_put.close()
    ws = orn.WeightStore.open(ctx, d, extra=[side])
    got = run(ws, cfg)
    # numbered experts were stacked: three tensors stand for 3 * E of the sidecar
    n_file, bytes_file = ws.stats()
    assert (n_file, bytes_file) == (n_put, bytes_put)
    ws.close()
    assert got == want
    assert got[0] == got[1]
    orc = synth.OracleRun(s, 64)
    assert got[0] == orc.generate(prompt, 12, prefill_step=4)
    orc.close()


def test_config_and_tensors_must_agree(orn, ctx, artifact, tmp_path):
    """A module whose tensors disagree with the mode config.json claims fails at load
    (/root/reference/src/weights.rs:126-150, 199-220)."""
    s, d, side = artifact
    cfgp = os.path.join(d, "config.json")
    good = json.load(open(cfgp))
    text, _ = orn.TextConfig.load(d)

    def load_with(quant_edit):
        bad = json.loads(json.dumps(good))
        quant_edit(bad["quantization"])
        json.dump(bad, open(cfgp, "w"))
        ws = orn.WeightStore.open(ctx, d, extra=[side])
        try:
            with pytest.raises(orn.OrnithError) as e:
                orn.TextModel(ctx, ws, text)
            return str(e.value)
        finally:
            ws.close()
            json.dump(good, open(cfgp, "w"))

    lm = "language_model.lm_head"
    assert "says affine" in load_with(lambda q: q.pop(lm))
    assert "super-block is 256" in load_with(lambda q: q[lm].update(group_size=64))
    assert "laid out as q4k" in load_with(lambda q: q[lm].update(mode="q6k"))
    emb = "language_model.model.embed_tokens"
    assert "no " + emb + ".dm" in load_with(lambda q: q.update({emb: {"group_size": 256, "bits": 4, "mode": "q4k"}}))
    assert "is not carried" in load_with(lambda q: q.update({emb: {"bits": 4}}))   # 4-bit needs group 32


def test_published_artifact_format_from_files(orn, ctx, tmp_path):
    """The published mlx artifact's layout: 4-bit affine group 32 by default (projections, stacked
    experts, embed_tokens, lm_head), 8-bit group 64 for the routers, said by config.json's
    quantization block with per-module overrides. Read from files it generates the tokens of the
    same model put by name and of the oracle."""
    s = synth.SynthModel(dict(synth.TINY, vocab_size=256), seed=23, affine="affine4", trunk="affine4")
    d = str(tmp_path / "model")
    side = synth.write_artifact(s, d, shards=2)
    q = json.load(open(os.path.join(d, "config.json")))["quantization"]
    assert (q["bits"], q["group_size"]) == (4, 32)
    assert q["language_model.model.layers.0.mlp.gate"] == {"group_size": 64, "bits": 8, "mode": "affine"}
    cfg, _ = orn.TextConfig.load(d)
    prompt = np.random.default_rng(4).integers(0, 256, 7).astype(np.uint32)

    def run(ws, config):
        model = orn.TextModel(ctx, ws, config)
        head = orn.MtpHead(model, ws, 48)
        caches = model.make_cache(48, 4)
        greedy = orn.generate_step(model, caches, prompt, 10, prefill_step=4)
        caches.reset()
        spec, _ = orn.generate_step_mtp(model, head, None, caches, prompt, 2, 10, prefill_step=4)
        for o in (head, caches, model):
            o.close()
        return greedy, spec

    ws = orn.WeightStore.open(ctx, d, extra=[side])
    assert ws.quant_config("language_model.model.layers.1.mlp.switch_mlp.down_proj") == (32, 4, orn.QM_AFFINE)
    got = run(ws, cfg)
    ws.close()
    ws_put = s.upload(orn, ctx)
    want = run(ws_put, s.text_config(orn))
    ws_put.close()
    orc = synth.OracleRun(s, 48)
    assert got == want and got[0] == got[1] == orc.generate(prompt, 10, prefill_step=4)
    orc.close()
    # 8-bit stacked experts are not carried: the loader says so
    cj = json.load(open(os.path.join(d, "config.json")))
    cj["quantization"]["language_model.model.layers.0.mlp.switch_mlp.gate_proj"] = {"group_size": 64, "bits": 8, "mode": "affine"}
    json.dump(cj, open(os.path.join(d, "config.json"), "w"))
    ws = orn.WeightStore.open(ctx, d, extra=[side])
    with pytest.raises(orn.OrnithError, match="4-bit group 32 only"):
        orn.TextModel(ctx, ws, cfg)
    ws.close()
