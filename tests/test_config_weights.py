"""Configuration, registry, safetensors I/O, loader errors and the random-weights mode."""
import json
import os

import pytest
import torch

import mini_llm_amd.models  # noqa: F401  (registers the architecture)
from conftest import TINY_A, TINY_B
from mini_llm_amd.config.base import ConfigError, LayerCall
from mini_llm_amd.config.gpt2 import GPT2Config
from mini_llm_amd.config.registry import (architecture_of, get_architecture, load_config,
                                          registered_architectures)
from mini_llm_amd.models import load_model
from mini_llm_amd.weights.loader import WeightsError, load_weights
from mini_llm_amd.weights.random_init import write_random_model
from mini_llm_amd.weights.safetensors_io import SafetensorsError, SafetensorsFile, save_file


def test_config_reads_its_own_keys():
    a, b = GPT2Config.from_dict(TINY_A), GPT2Config.from_dict(TINY_B)
    assert (a.n_layer, a.n_embd, a.n_head, a.head_dim, a.inner_dim, a.vocab_size, a.n_positions) == \
           (2, 64, 4, 16, 256, 512, 128)
    assert (b.n_layer, b.n_embd, b.n_head, b.head_dim, b.inner_dim, b.vocab_size, b.n_positions) == \
           (3, 96, 3, 32, 320, 1000, 256)
    assert a.layer_norm_epsilon == 1e-5 and b.layer_norm_epsilon == 1e-6
    assert a.eos_token_id == 511 and b.max_positions == 256
    sa, sb = a.layer_specs(), b.layer_specs()
    assert len(sa) == 2 and len(sb) == 3
    assert sa[0].feed_forward.params["activation"] == "gelu_tanh"
    assert sb[0].feed_forward.params["activation"] == "gelu_erf"
    assert sb[2].mixer.params["scale"] == pytest.approx(32 ** -0.5) and sb[2].weight_prefix == "h.2."
    assert a.layer_order() == [LayerCall(0, 0, True), LayerCall(1, 1, True)]
    assert GPT2Config.from_dict(a.to_dict()) == a


@pytest.mark.parametrize("change,match", [
    ({"n_embd": None}, "n_embd"), ({"vocab_size": "x"}, "vocab_size"), ({"n_head": 5}, "divisible"),
    ({"activation_function": "relu"}, "activation_function"), ({"layer_norm_epsilon": 0}, "positive"),
    ({"scale_attn_by_inverse_layer_idx": True}, "not supported"), ({"reorder_and_upcast_attn": True}, "not supported"),
    ({"tie_word_embeddings": False}, "untied"), ({"n_layer": 0}, "positive"), ({"n_inner": 1.5}, "n_inner"),
])
def test_config_refuses(change, match):
    d = dict(TINY_A, **change)
    d = {k: v for k, v in d.items() if not (k in change and change[k] is None and k != "n_inner")}
    with pytest.raises(ConfigError, match=match):
        GPT2Config.from_dict(d)


def test_registry(tmp_path):
    assert "GPT2LMHeadModel" in registered_architectures()
    assert architecture_of({"model_type": "gpt2"}).name == "GPT2LMHeadModel"
    with pytest.raises(ConfigError, match="unknown architecture 'LlamaForCausalLM'.*GPT2LMHeadModel"):
        get_architecture("LlamaForCausalLM")
    with pytest.raises(ConfigError, match="names no architecture"):
        architecture_of({"n_embd": 4})
    with pytest.raises(ConfigError, match="no such file"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="not valid JSON"):
        load_config(str(tmp_path))


def test_safetensors_roundtrip_and_interop(tmp_path):
    from safetensors.torch import load_file, save_file as st_save
    g = torch.Generator().manual_seed(0)
    tensors = {"a.weight": torch.randn(3, 5, generator=g).bfloat16(), "b": torch.randn(7, generator=g),
               "c.table": torch.arange(6, dtype=torch.int32).reshape(2, 3), "d": torch.tensor(2.5)}
    p = str(tmp_path / "x.safetensors")
    save_file(tensors, p, metadata={"format": "pt"})
    theirs = load_file(p)                                   # the library reads what we wrote
    with SafetensorsFile(p) as f:
        assert sorted(f.names()) == sorted(tensors)
        for k, v in tensors.items():
            assert f.info(k) == (v.dtype, tuple(v.shape))
            assert torch.equal(f.tensor(k), v) and torch.equal(theirs[k], v)
    q = str(tmp_path / "y.safetensors")
    st_save({k: v for k, v in tensors.items()}, q)          # we read what the library wrote
    with SafetensorsFile(q) as f:
        for k, v in tensors.items():
            assert torch.equal(f.tensor(k), v)


def test_safetensors_refuses_broken_files(tmp_path):
    p = tmp_path / "short.safetensors"
    p.write_bytes(b"\x01\x02")
    with pytest.raises(SafetensorsError, match="too short"):
        SafetensorsFile(str(p))
    save_file({"a": torch.zeros(4, 4)}, str(p))
    raw = p.read_bytes()
    p.write_bytes(raw[:-8])                                  # data cut off
    with pytest.raises(SafetensorsError, match="offsets"):
        SafetensorsFile(str(p))
    p.write_bytes((10 ** 9).to_bytes(8, "little") + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        SafetensorsFile(str(p))


def _tensors(model_dir):
    with SafetensorsFile(os.path.join(model_dir, "model.safetensors")) as f:
        return {n: f.tensor(n) for n in f.names()}


def test_random_model_folder(tmp_path):
    d = write_random_model(dict(TINY_B), str(tmp_path / "m"), seed=1)
    cfg = json.load(open(os.path.join(d, "config.json")))
    assert cfg["architectures"] == ["GPT2LMHeadModel"] and cfg["n_inner"] == 320
    t = _tensors(d)
    assert len(t) == 2 + 3 * 12 + 2
    assert t["wte.weight"].shape == (1000, 96) and t["wte.weight"].dtype == torch.bfloat16
    assert t["h.1.attn.c_attn.weight"].shape == (96, 288)          # Conv1D: [in, out]
    assert t["h.2.mlp.c_fc.weight"].shape == (96, 320) and t["h.2.mlp.c_proj.weight"].shape == (320, 96)
    assert t["h.0.ln_1.weight"].dtype == torch.float32 and t["h.0.attn.c_attn.bias"].dtype == torch.float32
    # the distributions BASELINE names: N(0, .02); residual projections N(0, .02/sqrt(2L)); gains N(1, .1)
    assert t["wte.weight"].float().std().item() == pytest.approx(0.02, rel=0.05)
    assert t["h.0.mlp.c_proj.weight"].float().std().item() == pytest.approx(0.02 / 6 ** 0.5, rel=0.05)
    assert t["h.0.attn.c_proj.weight"].float().std().item() == pytest.approx(0.02 / 6 ** 0.5, rel=0.08)
    assert t["ln_f.weight"].mean().item() == pytest.approx(1.0, abs=0.05)
    assert t["ln_f.weight"].std().item() == pytest.approx(0.1, rel=0.3)
    # same seed, same bytes; another seed, other values
    d2 = write_random_model(dict(TINY_B), str(tmp_path / "m2"), seed=1)
    d3 = write_random_model(dict(TINY_B), str(tmp_path / "m3"), seed=2)
    assert open(os.path.join(d, "model.safetensors"), "rb").read() == open(os.path.join(d2, "model.safetensors"), "rb").read()
    assert not torch.equal(_tensors(d3)["wpe.weight"], t["wpe.weight"])


def test_random_values_follow_the_published_recipe():
    """The generator is a specification, not a library call: element i of tensor `name` under `seed`
    is recomputed here with Python integers and math.* only, and a fixed vector pins the constants."""
    import math
    from mini_llm_amd.weights.random_init import normal_values
    M = (1 << 64) - 1

    def mix(x):
        z = (x + 0x9E3779B97F4A7C15) & M
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M
        return z ^ (z >> 31)

    def fnv(b):
        h = 0xCBF29CE484222325
        for c in b:
            h = ((h ^ c) * 0x100000001B3) & M
        return h

    def value(seed, name, i, mean, std):
        key = mix(seed) ^ fnv(name.encode())
        a, b = mix((key + 2 * i) & M), mix((key + 2 * i + 1) & M)
        u1, u2 = ((a >> 11) + 1) / 2.0 ** 53, (b >> 11) / 2.0 ** 53
        return mean + std * math.sqrt(-2.0 * math.log(u1)) * math.cos(2.0 * math.pi * u2)

    assert mix(0) == 0xE220A8397B1DCDAF and fnv(b"wte.weight") == 0x61D3A46D83BC4189
    got = normal_values(2, "wte.weight", 6, 0.0, 0.02)
    assert [round(float(v), 9) for v in got[:3]] == [-0.011919891, 0.005637622, -0.020101186]
    for seed, name, mean, std in ((2, "wte.weight", 0.0, 0.02), (7, "h.3.ln_1.weight", 1.0, 0.1)):
        v = normal_values(seed, name, 1000, mean, std)
        for i in (0, 1, 17, 999):
            assert abs(float(v[i]) - value(seed, name, i, mean, std)) <= 1e-7 * max(1.0, abs(mean))
    # a value depends on (seed, name, index) only: a window of a tensor equals the same window of the whole
    whole = normal_values(5, "t", (1 << 18) * 3 + 11, 0.0, 1.0)
    assert (normal_values(5, "t", 4097, 0.0, 1.0, first=(1 << 18) - 100) == whole[(1 << 18) - 100:(1 << 18) + 3997]).all()
    assert abs(float(whole.mean())) < 5e-3 and abs(float(whole.std()) - 1.0) < 5e-3
    assert abs(float((whole ** 4).mean()) - 3.0) < 0.05                                  # normal, not merely unit variance
    assert not (normal_values(6, "t", 64, 0.0, 1.0) == whole[:64]).any()
    assert not (normal_values(5, "u", 64, 0.0, 1.0) == whole[:64]).any()


def test_a_tensor_keeps_its_values_when_the_model_changes(tmp_path):
    """Random weights are keyed by tensor name: a model with one more layer has the same first layers."""
    d2 = write_random_model(dict(TINY_A), str(tmp_path / "l2"), seed=3)
    d3 = write_random_model(dict(TINY_A, n_layer=3), str(tmp_path / "l3"), seed=3)
    t2, t3 = _tensors(d2), _tensors(d3)
    assert set(t2) < set(t3)
    same = [n for n in t2 if torch.equal(t2[n], t3[n])]
    # (the residual projections' spread depends on the number of layers, so they differ)
    assert sorted(set(t2) - set(same)) == sorted(f"h.{i}.{p}.c_proj.weight" for i in range(2) for p in ("attn", "mlp"))


def test_loader_reads_shards_and_half_precision(tmp_path):
    """A checkpoint split over two files named by model.safetensors.index.json, stored in float16."""
    d = write_random_model(dict(TINY_B), str(tmp_path / "whole"), seed=4, weights_dtype="float16")
    t = _tensors(d)
    assert t["wte.weight"].dtype == torch.float16
    sharded = tmp_path / "sharded"
    sharded.mkdir()
    names = sorted(t)
    parts = {"model-00001-of-00002.safetensors": names[:len(names) // 2],
             "model-00002-of-00002.safetensors": names[len(names) // 2:]}
    for fname, ns in parts.items():
        save_file({n: t[n] for n in ns}, str(sharded / fname))
    json.dump({"metadata": {}, "weight_map": {n: f for f, ns in parts.items() for n in ns}},
              open(sharded / "model.safetensors.index.json", "w"))
    json.dump(json.load(open(os.path.join(d, "config.json"))), open(sharded / "config.json", "w"))
    for dtype in (torch.float32, torch.bfloat16):
        a, b = load_model(d, dtype, "cpu"), load_model(str(sharded), dtype, "cpu")
        for sa, sb in zip(a.param_specs(), b.param_specs()):
            assert sa.name == sb.name
        assert torch.equal(a.embedding.weight, b.embedding.weight) and a.embedding.weight.dtype == dtype
        assert torch.equal(a.embedding.weight, t["wte.weight"].to(dtype))
        assert torch.equal(a.layers[2].feed_forward.down.weight, b.layers[2].feed_forward.down.weight)
        assert torch.equal(b.layers[2].feed_forward.down.weight, t["h.2.mlp.c_proj.weight"].t().to(dtype))
        assert torch.equal(b.layers[1].norm1.gamma, t["h.1.ln_1.weight"])
    # a tensor in two shards is an error that names it; a shard the index names but that is not there too
    save_file({names[0]: t[names[0]], **{n: t[n] for n in parts["model-00002-of-00002.safetensors"]}},
              str(sharded / "model-00002-of-00002.safetensors"))
    with pytest.raises(WeightsError, match="two files"):
        load_model(str(sharded), "float32", "cpu")
    os.remove(sharded / "model-00001-of-00002.safetensors")
    with pytest.raises((WeightsError, SafetensorsError, OSError)):
        load_model(str(sharded), "float32", "cpu")


def test_loader_places_and_converts(tmp_path):
    d = write_random_model(dict(TINY_A), str(tmp_path / "m"), seed=0, weights_dtype="float32")
    t = _tensors(d)
    for dtype in (torch.float32, torch.bfloat16):
        m = load_model(d, dtype, "cpu")
        att = m.layers[1].mixer
        assert att.qkv.weight.dtype == dtype and att.qkv.weight.shape == (192, 64)       # held [out, in]
        assert torch.equal(att.qkv.weight, t["h.1.attn.c_attn.weight"].t().to(dtype))
        assert att.qkv.bias.dtype == torch.float32 and torch.equal(att.qkv.bias, t["h.1.attn.c_attn.bias"])
        assert m.layers[0].norm2.gamma.dtype == torch.float32           # stored in 32-bit, stays so
        assert torch.equal(m.final_norm.beta, t["ln_f.bias"])
        assert m.embedding.weight.dtype == dtype and m.position.table.shape == (128, 64)
        assert m.head.embedding is m.embedding                           # tied head


def test_loader_accepts_prefix_and_mask_buffers(tmp_path):
    d = write_random_model(dict(TINY_A), str(tmp_path / "m"), seed=0)
    t = {"transformer." + k: v for k, v in _tensors(d).items()}
    t["transformer.h.0.attn.bias"] = torch.ones(1, 1, 8, 8)
    t["transformer.h.1.attn.masked_bias"] = torch.tensor(-1e4)
    t["lm_head.weight"] = t["transformer.wte.weight"].clone()
    save_file(t, os.path.join(d, "model.safetensors"))
    load_model(d, "float32", "cpu")


def test_loader_lists_every_mismatch(tmp_path):
    d = write_random_model(dict(TINY_A), str(tmp_path / "m"), seed=0)
    t = _tensors(d)
    del t["h.1.ln_2.bias"], t["wpe.weight"]
    t["h.0.mlp.c_fc.weight"] = torch.zeros(256, 64, dtype=torch.bfloat16)     # transposed by mistake
    t["h.0.attn.c_attn.bias"] = torch.zeros(64)
    t["h.7.extra.weight"] = torch.zeros(2)
    save_file(t, os.path.join(d, "model.safetensors"))
    with pytest.raises(WeightsError) as ei:
        load_model(d, "float32", "cpu")
    e = ei.value
    assert e.missing == ["h.1.ln_2.bias", "wpe.weight"]
    assert e.unexpected == ["h.7.extra.weight"]
    assert sorted(n for n, _, _ in e.wrong_shape) == ["h.0.attn.c_attn.bias", "h.0.mlp.c_fc.weight"]
    msg = str(e)
    for piece in ("missing tensors (2)", "h.1.ln_2.bias", "unexpected tensors (1)", "h.7.extra.weight",
                  "wrong shapes (2)", "expected [64, 256], found [256, 64]"):
        assert piece in msg
    os.remove(os.path.join(d, "model.safetensors"))
    with pytest.raises(WeightsError, match="neither model.safetensors"):
        load_model(d, "float32", "cpu")


def test_sizes_the_kernels_cannot_take_are_refused_when_the_model_is_built(tmp_path):
    """A feed-forward width that is no multiple of 8 has no bfloat16 kernel: building the model says
    so (float32 takes it); a head size that is no multiple of 16 is refused for every dtype."""
    from mini_llm_amd import load_model, write_random_model
    cfg = dict(json.load(open(os.path.join(os.path.dirname(__file__), "..", "mini_llm_amd", "config", "presets",
                                          "tiny-a.json"))))
    cfg["n_inner"] = 100
    d = str(tmp_path / "odd")
    write_random_model(cfg, d, seed=0)
    with pytest.raises(ValueError, match="multiple of 8"):
        load_model(d, "bfloat16", "cpu")
    assert load_model(d, "float32", "cpu") is not None
    cfg2 = dict(cfg, n_inner=256, n_embd=40, n_head=4)     # head size 10
    d2 = str(tmp_path / "odd2")
    with pytest.raises(ValueError, match="head"):
        write_random_model(cfg2, d2, seed=0)
        load_model(d2, "float32", "cpu")


def test_the_native_program_writes_the_same_model_folder(tmp_path):
    """`mini-llm make-model` (C++: its own JSON, generator and safetensors writer) and `write_random_model`
    (Python) make the same folder from a preset and a seed: the tensor file byte for byte, the same
    configuration. No GPU is needed for it."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    native = str(tmp_path / "native")
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "mini-llm"), "make-model", "--preset", "tiny-b",
                        "--seed", "5", "--out", native], capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stderr
    preset = json.load(open(os.path.join(root, "mini_llm_amd", "config", "presets", "tiny-b.json")))
    python = write_random_model(dict(preset), str(tmp_path / "python"), seed=5)
    with open(os.path.join(native, "model.safetensors"), "rb") as a, open(os.path.join(python, "model.safetensors"), "rb") as b:
        assert a.read() == b.read()
    assert json.load(open(os.path.join(native, "config.json"))) == json.load(open(os.path.join(python, "config.json")))
    for dtype in ("float32",):
        r = subprocess.run([sys.executable, os.path.join(root, "bin", "mini-llm"), "make-model", "--preset", "tiny-a",
                            "--seed", "0", "--weights-dtype", dtype, "--out", native + dtype], capture_output=True, text=True, timeout=900)
        assert r.returncode == 0, r.stderr
        preset = json.load(open(os.path.join(root, "mini_llm_amd", "config", "presets", "tiny-a.json")))
        python = write_random_model(dict(preset), str(tmp_path / ("python" + dtype)), seed=0, weights_dtype=dtype)
        with open(os.path.join(native + dtype, "model.safetensors"), "rb") as a, open(os.path.join(python, "model.safetensors"), "rb") as b:
            assert a.read() == b.read()
    bad = subprocess.run([sys.executable, os.path.join(root, "bin", "mini-llm"), "make-model", "--preset", "nothing",
                          "--seed", "0", "--out", native + "x"], capture_output=True, text=True, timeout=900)
    assert bad.returncode == 1 and "unknown preset" in bad.stderr


def _native_check(folder):
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "mini-llm"), "check", "--model", str(folder)],
                       capture_output=True, text=True, timeout=900)
    return r.returncode, r.stdout + r.stderr


def test_the_native_loader_checks_a_folder_without_a_gpu(tmp_path):
    """`mini-llm check` runs the C++ side's configuration, safetensors reader and name/shape check: the
    same findings as the Python loader, every mismatch in one message."""
    d = write_random_model(dict(TINY_A), str(tmp_path / "m"), seed=0)
    rc, out = _native_check(d)
    good = _tensors(d)
    n_params = sum(t.numel() for t in good.values())
    assert rc == 0 and f"ok: GPT2LMHeadModel, {len(good)} tensors, {n_params} parameters" in out, out
    # the prefix and the mask buffers of exported checkpoints are accepted
    t = {"transformer." + k: v for k, v in good.items()}
    t["transformer.h.0.attn.bias"] = torch.ones(1, 1, 8, 8)
    t["lm_head.weight"] = t["transformer.wte.weight"].clone()
    save_file(t, os.path.join(d, "model.safetensors"))
    assert _native_check(d)[0] == 0
    # every mismatch in one message
    t = dict(good)
    del t["h.1.ln_2.bias"], t["wpe.weight"]
    t["h.0.mlp.c_fc.weight"] = torch.zeros(256, 64, dtype=torch.bfloat16)
    t["h.7.extra.weight"] = torch.zeros(2)
    save_file(t, os.path.join(d, "model.safetensors"))
    rc, out = _native_check(d)
    assert rc == 1
    for piece in ("missing tensors (2)", "h.1.ln_2.bias", "wpe.weight", "unexpected tensors (1)", "h.7.extra.weight",
                  "wrong shapes (1)", "expected [64, 256], found [256, 64]"):
        assert piece in out, (piece, out)
    # files that are no safetensors files
    raw = open(os.path.join(d, "model.safetensors"), "rb").read()
    for broken, match in ((raw[:5], "too short"), ((10 ** 9).to_bytes(8, "little") + raw[8:], "header length"),
                          (raw[:8] + b"{" * 20 + raw[28:], "JSON"), (raw[:len(raw) // 2], "offsets")):
        open(os.path.join(d, "model.safetensors"), "wb").write(broken)
        rc, out = _native_check(d)
        assert rc == 1 and match in out, (match, out)
    os.remove(os.path.join(d, "model.safetensors"))
    rc, out = _native_check(d)
    assert rc == 1 and "neither model.safetensors" in out
    # the configuration is judged first
    cfg = json.load(open(os.path.join(d, "config.json")))
    json.dump(dict(cfg, n_head=5), open(os.path.join(d, "config.json"), "w"))
    rc, out = _native_check(d)
    assert rc == 1 and "divisible" in out
    json.dump(dict(cfg, architectures=["Other"], model_type="other"), open(os.path.join(d, "config.json"), "w"))
    rc, out = _native_check(d)
    assert rc == 1 and "no known architecture" in out and "GPT2LMHeadModel" in out
    open(os.path.join(d, "config.json"), "w").write("{not json")
    assert _native_check(d)[0] == 1
