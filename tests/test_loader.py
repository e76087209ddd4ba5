"""The artifact reader on the host: safetensors shards, the index, config.json's text and
quantization blocks. Mirrors the reference's own loader tests
(/root/reference/src/safetensors.rs:321-369, /root/reference/src/weights.rs:296-362), which
need the real model on disk; here the files are synthetic, written by an independent writer
(the `safetensors` package) and by a hand-rolled one that can place data on odd offsets."""
import importlib
import json
import os

import numpy as np
import pytest

import synth
import util

orn = importlib.import_module("ornith-rs_amd")


def _err(fn, *a, **k):
    with pytest.raises(orn.OrnithError) as e:
        fn(*a, **k)
    return str(e.value)


def test_reads_what_the_safetensors_package_wrote(tmp_path):
    from safetensors.numpy import save_file
    rng = np.random.default_rng(0)
    t = {"a.weight": rng.integers(0, 2**32, (3, 5), dtype=np.uint32),
         "a.scales": rng.integers(0, 256, (3, 2, 12), dtype=np.uint8),
         "a.dm": rng.standard_normal((3, 2, 2)).astype(np.float16),
         "f": rng.standard_normal((7,)).astype(np.float32),
         "i": rng.integers(-5, 5, (2, 2), dtype=np.int32),
         "l": rng.integers(-5, 5, (4,), dtype=np.int64),
         "d": rng.standard_normal((2, 1, 3)).astype(np.float64),
         "b": np.array([True, False, True])}
    p = str(tmp_path / "x.safetensors")
    save_file(t, p, metadata={"format": "pt", "note": "café \"quoted\" \\ \U0001F600"})
    st = orn.SafeTensors(paths=[p])
    assert st.counts() == (len(t), 1)
    assert st.names() == sorted(t)
    codes = {"a.weight": orn.DT_U32, "a.scales": orn.DT_U8, "a.dm": orn.DT_F16, "f": orn.DT_F32,
             "i": orn.DT_I32, "l": orn.DT_I64, "d": orn.DT_F64, "b": orn.DT_BOOL}
    for n, a in t.items():
        dt, shape, raw = st.info(n)
        assert (dt, shape) == (codes[n], a.shape), n
        assert raw.tobytes() == a.tobytes(), n
    assert "no tensor named" in _err(st.info, "missing")
    st.close()


def test_hand_written_file_is_what_the_package_reads(tmp_path):
    """Pins the test's own writer: the `safetensors` package must read back the same bytes."""
    from safetensors import safe_open
    rng = np.random.default_rng(1)
    t = {"x": (rng.standard_normal((4, 3)).astype(np.float32), orn.DT_F32),
         "y": (rng.integers(0, 256, (5,), dtype=np.uint8), orn.DT_U8)}
    p = str(tmp_path / "h.safetensors")
    synth.write_safetensors(p, t, metadata={"k": "v"}, header_pad=3)
    with safe_open(p, framework="np") as f:
        assert sorted(f.keys()) == ["x", "y"]
        for n, (a, _) in t.items():
            assert np.array_equal(f.get_tensor(n), a)


def test_unaligned_tensors_and_bf16(tmp_path):
    """Tensors start on odd byte offsets (/root/reference/src/safetensors.rs:359-369)."""
    rng = np.random.default_rng(2)
    t = {"odd": (rng.integers(0, 256, (3,), dtype=np.uint8), orn.DT_U8),
         "w": (util.f32_to_bf16(rng.standard_normal((6, 4)).astype(np.float32)), orn.DT_BF16),
         "h": (rng.standard_normal((5,)).astype(np.float16), orn.DT_F16)}
    p = str(tmp_path / "u.safetensors")
    synth.write_safetensors(p, t, header_pad=2)
    st = orn.SafeTensors(paths=[p])
    for n, (a, code) in t.items():
        dt, shape, raw = st.info(n)
        assert (dt, shape) == (code, a.shape)
        assert raw.tobytes() == a.tobytes()
    st.close()


def _raw_file(path, header, payload=b""):
    hj = header if isinstance(header, bytes) else json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(len(hj).to_bytes(8, "little") + hj + payload)


def test_rejects_malformed_files(tmp_path):
    p = str(tmp_path / "bad.safetensors")
    open(p, "wb").write(b"\x01\x02")
    assert "too short" in _err(orn.SafeTensors, paths=[p])
    open(p, "wb").write((1000).to_bytes(8, "little") + b"{}")
    assert "past EOF" in _err(orn.SafeTensors, paths=[p])
    _raw_file(p, b"[1,2]")
    assert "not an object" in _err(orn.SafeTensors, paths=[p])
    _raw_file(p, b'{"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]},}')
    assert "JSON" in _err(orn.SafeTensors, paths=[p])
    _raw_file(p, {"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 6]}}, b"\0" * 8)
    assert "span 6 bytes" in _err(orn.SafeTensors, paths=[p])
    _raw_file(p, {"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}, b"\0" * 7)
    assert "past EOF" in _err(orn.SafeTensors, paths=[p])
    _raw_file(p, {"a": {"dtype": "F8_E4M3", "shape": [2], "data_offsets": [0, 2]}}, b"\0" * 2)
    assert "unsupported dtype" in _err(orn.SafeTensors, paths=[p])
    _raw_file(p, {"a": {"shape": [2], "data_offsets": [0, 2]}}, b"\0" * 2)
    assert "missing dtype" in _err(orn.SafeTensors, paths=[p])
    _raw_file(p, {"a": {"dtype": "U8", "shape": [2]}}, b"\0" * 2)
    assert "missing data_offsets" in _err(orn.SafeTensors, paths=[p])
    assert "mmap" in _err(orn.SafeTensors, paths=[str(tmp_path / "absent.safetensors")])
    # empty tensors and an empty header are fine
    _raw_file(p, {"e": {"dtype": "F32", "shape": [0, 4], "data_offsets": [0, 0]}})
    st = orn.SafeTensors(paths=[p])
    assert st.info("e")[1] == (0, 4)
    st.close()
    _raw_file(p, {})
    st = orn.SafeTensors(paths=[p])
    assert st.counts() == (0, 1)
    st.close()


def test_index_resolves_shards_and_extra_files(tmp_path):
    s = synth.SynthModel(synth.TINY, seed=5, with_oracle=False)
    d = str(tmp_path / "model")
    side = synth.write_artifact(s, d, shards=3)
    st = orn.SafeTensors(model_dir=d)
    n_trunk = sum(1 for n in s.tensors if not n.startswith("mtp."))
    assert st.counts() == (n_trunk, 3)
    for n in ("language_model.model.embed_tokens.weight",
              "language_model.model.layers.3.self_attn.q_proj.dm",
              "language_model.model.layers.0.mlp.switch_mlp.down_proj.scales"):
        dt, shape, raw = st.info(n)
        arr, code = s.tensors[n]
        assert (dt, shape) == (code, arr.shape)
        assert raw.tobytes() == arr.tobytes()
    st.close()
    st = orn.SafeTensors(model_dir=d, extra=[side])
    E = synth.TINY["num_experts"]
    assert st.counts()[1] == 4
    dt, shape, raw = st.info(f"mtp.layers.0.mlp.experts.{E - 1}.down_proj.weight")
    want = s.tensors["mtp.layers.0.mlp.switch_mlp.down_proj.weight"][0][E - 1]
    assert shape == want.shape and raw.tobytes() == want.tobytes()
    st.close()
    os.remove(os.path.join(d, "model.safetensors.index.json"))
    assert "model.safetensors.index.json" in _err(orn.SafeTensors, model_dir=d)


@pytest.mark.parametrize("nested", [True, False])
def test_text_config(tmp_path, nested):
    s = synth.SynthModel(synth.TINY, seed=5, with_oracle=False)
    d = str(tmp_path / "model")
    synth.write_artifact(s, d, nested=nested)
    cfg, mtp = orn.TextConfig.load(d)
    assert mtp == 1
    for k, v in synth.TINY.items():
        got = getattr(cfg, k)
        assert got == (np.float32(v) if k == "rms_norm_eps" else v), k


def test_text_config_defaults_and_errors(tmp_path):
    d = str(tmp_path)
    base = dict(hidden_size=1024, num_attention_heads=8, num_hidden_layers=2, num_key_value_heads=2,
                vocab_size=100, linear_num_value_heads=4, linear_num_key_heads=2, linear_key_head_dim=128,
                linear_value_head_dim=128, linear_conv_kernel_dim=4)
    json.dump(base, open(os.path.join(d, "config.json"), "w"))
    cfg, mtp = orn.TextConfig.load(d)
    assert mtp == 0
    assert cfg.head_dim == 128 and cfg.rope_dims == 32          # hidden / heads, factor 0.25
    assert cfg.full_attention_interval == 4 and cfg.norm_topk_prob == 1
    assert cfg.rms_norm_eps == np.float32(1e-6) and cfg.rope_theta == 100000.0
    assert cfg.num_experts == 0
    # rope_theta is read as fp32, top-level keys are the fallback for rope_parameters
    json.dump(dict(base, rope_theta=1234567.891, partial_rotary_factor=0.5, head_dim=64),
              open(os.path.join(d, "config.json"), "w"))
    cfg, _ = orn.TextConfig.load(d)
    assert cfg.rope_theta == float(np.float32(1234567.891)) and cfg.rope_dims == 32
    del base["vocab_size"]
    json.dump(base, open(os.path.join(d, "config.json"), "w"))
    assert "missing vocab_size" in _err(orn.TextConfig.load, d)
    os.remove(os.path.join(d, "config.json"))
    assert "config.json" in _err(orn.TextConfig.load, d)


def test_quant_config_overrides(tmp_path):
    d = str(tmp_path)
    q = {"group_size": 64, "bits": 4,
         "language_model.model.layers.0.mlp.gate": {"group_size": 64, "bits": 8},
         "language_model.lm_head": {"group_size": 256, "bits": 4, "mode": "q4k"},
         "language_model.model.layers.3.self_attn.q_proj": {"group_size": 256, "bits": 6, "mode": "q6k"},
         "x.partial": {"bits": 8}}
    json.dump({"quantization": q}, open(os.path.join(d, "config.json"), "w"))
    look = lambda p: orn.quant_config_load(d, p)
    assert look("anything.else") == (64, 4, orn.QM_AFFINE)          # no mode key: affine
    assert look("language_model.model.layers.0.mlp.gate") == (64, 8, orn.QM_AFFINE)
    assert look("language_model.lm_head") == (256, 4, orn.QM_Q4K)
    assert look("language_model.model.layers.3.self_attn.q_proj") == (256, 6, orn.QM_Q6K)
    assert look("x.partial") == (64, 8, orn.QM_AFFINE)               # missing fields inherit
    json.dump({"quantization": dict(q, mode="nvfp4")}, open(os.path.join(d, "config.json"), "w"))
    assert "not carried" in _err(look, "a")
    json.dump({"quantization": dict(q, mode="int3")}, open(os.path.join(d, "config.json"), "w"))
    assert "unknown quantization mode" in _err(look, "a")
    json.dump({"quantization": {"bits": 4}}, open(os.path.join(d, "config.json"), "w"))
    assert "group_size" in _err(look, "a")
    json.dump({}, open(os.path.join(d, "config.json"), "w"))
    assert "no quantization block" in _err(look, "a")
