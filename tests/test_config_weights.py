"""Configuration, registry, model folders and weight errors, on the CPU: the engine's own native code
(csrc/engine/arch.cc, gpt2.cc, weights.cc, json.cc) through its Python faces and its program. Files are read back
and made wrong with the `safetensors` package, which the engine does not use."""
import json
import math
import os
import subprocess
import sys

import pytest
import torch
from safetensors import safe_open
from safetensors.torch import save_file

from conftest import TINY_A, TINY_B
from mini_llm_amd import (check_model_dir, describe_config, load_plugin, read_preset, registered_architectures,
                          write_random_model)
from mini_llm_amd.config import ConfigError
from mini_llm_amd.weights import WeightsError, normal_values

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLI = os.path.join(ROOT, "bin", "mini-llm")


def _tensors(model_dir):
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as f:
        return {k: f.get_tensor(k) for k in f.keys()}


def _shapes(config):
    return {t["name"]: t for t in describe_config(config)["tensors"]}


def test_config_reads_its_own_keys():
    """Every size of the tensors a model expects comes from config.json's keys (two configurations that differ in all)."""
    a, b = _shapes(TINY_A), _shapes(TINY_B)
    assert len(a) == 2 + 2 * 12 + 2 and len(b) == 2 + 3 * 12 + 2
    assert a["wte.weight"]["shape"] == [512, 64] and b["wte.weight"]["shape"] == [1000, 96]
    assert a["wpe.weight"]["shape"] == [128, 64] and b["wpe.weight"]["shape"] == [256, 96]
    # Conv1D weights are stored [in, out] and turned once; n_inner null means four times the width
    assert a["h.1.attn.c_attn.weight"] == dict(name="h.1.attn.c_attn.weight", shape=[64, 192], role="matrix", transpose=True,
                                              mean=0, std=0.02)
    assert a["h.0.mlp.c_fc.weight"]["shape"] == [64, 256] and b["h.2.mlp.c_fc.weight"]["shape"] == [96, 320]
    assert b["h.2.mlp.c_proj.weight"]["shape"] == [320, 96] and "h.3.ln_1.weight" not in b
    assert a["h.0.ln_1.weight"]["role"] == "vector" and a["h.0.ln_1.weight"]["mean"] == 1 and a["ln_f.bias"]["shape"] == [64]
    # residual projections: std 0.02 / sqrt(2 n_layer)
    assert a["h.0.attn.c_proj.weight"]["std"] == pytest.approx(0.02 / 2.0) and b["h.0.mlp.c_proj.weight"]["std"] == pytest.approx(0.02 / math.sqrt(6))
    assert describe_config(TINY_A)["architecture"] == "GPT2LMHeadModel"
    assert _shapes("tiny-b") == b and read_preset("tiny-a")["n_embd"] == 64


@pytest.mark.parametrize("change,match", [
    ({"n_embd": None}, "n_embd"), ({"vocab_size": "x"}, "vocab_size"), ({"n_head": 5}, "divisible"),
    ({"activation_function": "relu"}, "activation_function"), ({"layer_norm_epsilon": 0}, "positive"),
    ({"scale_attn_by_inverse_layer_idx": True}, "not supported"), ({"reorder_and_upcast_attn": True}, "not supported"),
    ({"add_cross_attention": True}, "not supported"), ({"scale_attn_weights": False}, "not supported"),
    ({"tie_word_embeddings": False}, "untied"), ({"n_layer": 0}, "positive"), ({"n_inner": 1.5}, "n_inner"),
    ({"n_positions": -4}, "positive"),
])
def test_config_refuses(change, match):
    d = dict(TINY_A, **change)
    d = {k: v for k, v in d.items() if not (k in change and change[k] is None and k != "n_inner")}
    with pytest.raises(ConfigError, match=match):
        describe_config(d)


def test_registry(tmp_path):
    assert "GPT2LMHeadModel" in registered_architectures()
    only_type = {k: v for k, v in TINY_A.items() if k != "architectures"}
    assert describe_config(only_type)["architecture"] == "GPT2LMHeadModel"          # by model_type
    with pytest.raises(ConfigError, match="no known architecture.*LlamaForCausalLM.*registered: .*GPT2LMHeadModel"):
        describe_config(dict(TINY_A, architectures=["LlamaForCausalLM"], model_type="llama"))
    with pytest.raises(ConfigError, match="no known architecture"):
        describe_config({"n_embd": 4})
    with pytest.raises(ConfigError, match="unknown preset"):
        describe_config("no-such-size")
    with pytest.raises(ConfigError, match="cannot be loaded"):
        load_plugin(str(tmp_path / "nothing.so"))
    with pytest.raises(WeightsError, match="config.json"):
        check_model_dir(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(WeightsError, match="config.json"):
        check_model_dir(str(tmp_path))


def test_an_architecture_registered_from_outside_the_package(tmp_path):
    """The tests' plugin (tests/native/toy_plugin.hip) registers three toy architectures and their parts; their
    configurations, tensors and folders are then handled like GPT-2's, without a GPU."""
    import toy
    toy.load()
    assert {"ToyLM", "ToyRoutedLM", "ToyBareMixer"} <= set(registered_architectures())
    cfg = dict(architectures=["ToyLM"], vocab=203, width=48, heads=3, decay=0.75, eps=1e-5)
    t = _shapes(cfg)
    assert t["l0.qkv.weight"]["shape"] == [48 + 2 * 16, 48] and t["l1.mean.gain"]["shape"] == [48] and "l1.up.weight" not in t
    with pytest.raises(ConfigError, match="divisible"):
        describe_config(dict(cfg, heads=5))
    d = write_random_model(cfg, str(tmp_path / "toy"), seed=3)
    assert check_model_dir(d) == ("ToyLM", 13, sum(v.numel() for v in _tensors(d).values()))
    rc = subprocess.run([sys.executable, CLI, "check", "--model", d, "--plugin", toy.plugin_path()], capture_output=True, text=True, timeout=900)
    assert rc.returncode == 0 and "ok: ToyLM, 13 tensors" in rc.stdout, rc.stderr


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
    # the distributions of the benchmark configurations: N(0, .02); residual projections N(0, .02/sqrt(2L)); gains N(1, .1)
    assert t["wte.weight"].float().std().item() == pytest.approx(0.02, rel=0.05)
    assert t["h.0.mlp.c_proj.weight"].float().std().item() == pytest.approx(0.02 / 6 ** 0.5, rel=0.05)
    assert t["h.0.attn.c_proj.weight"].float().std().item() == pytest.approx(0.02 / 6 ** 0.5, rel=0.08)
    assert t["ln_f.weight"].mean().item() == pytest.approx(1.0, abs=0.05)
    assert t["ln_f.weight"].std().item() == pytest.approx(0.1, rel=0.3)
    # same seed, same bytes; another seed, other values; 32-bit storage on request
    d2 = write_random_model(dict(TINY_B), str(tmp_path / "m2"), seed=1)
    d3 = write_random_model(dict(TINY_B), str(tmp_path / "m3"), seed=2)
    assert open(os.path.join(d, "model.safetensors"), "rb").read() == open(os.path.join(d2, "model.safetensors"), "rb").read()
    assert not torch.equal(_tensors(d3)["wpe.weight"], t["wpe.weight"])
    d4 = write_random_model(dict(TINY_B), str(tmp_path / "m4"), seed=1, weights_dtype="float32")
    t4 = _tensors(d4)
    assert t4["wte.weight"].dtype == torch.float32 and torch.equal(t4["wte.weight"].bfloat16(), t["wte.weight"])
    with pytest.raises(WeightsError, match="bfloat16 or float32"):
        write_random_model(dict(TINY_B), str(tmp_path / "m5"), seed=1, weights_dtype="int8")


def test_random_values_follow_the_published_recipe():
    """The generator is a specification, not a library call: element i of tensor `name` under `seed`
    is recomputed here with Python integers and math.* only, and a fixed vector pins the constants."""
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
    got = normal_values(2, "wte.weight", 0, 6, 0.0, 0.02)
    assert [round(float(v), 9) for v in got[:3]] == [-0.011919891, 0.005637622, -0.020101186]
    for seed, name, mean, std in ((2, "wte.weight", 0.0, 0.02), (7, "h.3.ln_1.weight", 1.0, 0.1)):
        v = normal_values(seed, name, 0, 1000, mean, std)
        for i in (0, 1, 17, 999):
            assert abs(float(v[i]) - value(seed, name, i, mean, std)) <= 1e-7 * max(1.0, abs(mean))
    # a value depends on (seed, name, index) only: a window of a tensor equals the same window of the whole
    whole = normal_values(5, "t", 0, (1 << 18) * 3 + 11)
    assert (normal_values(5, "t", (1 << 18) - 100, 4097) == whole[(1 << 18) - 100:(1 << 18) + 3997]).all()
    assert abs(float(whole.mean())) < 5e-3 and abs(float(whole.std()) - 1.0) < 5e-3
    assert abs(float((whole.astype("float64") ** 4).mean()) - 3.0) < 0.05                # normal, not merely unit variance
    assert not (normal_values(6, "t", 0, 64) == whole[:64]).any()
    assert not (normal_values(5, "u", 0, 64) == whole[:64]).any()


def test_a_tensor_keeps_its_values_when_the_model_changes(tmp_path):
    """Random weights are keyed by tensor name: a model with one more layer has the same first layers."""
    d2 = write_random_model(dict(TINY_A), str(tmp_path / "l2"), seed=3)
    d3 = write_random_model(dict(TINY_A, n_layer=3), str(tmp_path / "l3"), seed=3)
    t2, t3 = _tensors(d2), _tensors(d3)
    assert set(t2) < set(t3)
    same = [n for n in t2 if torch.equal(t2[n], t3[n])]
    # (the residual projections' spread depends on the number of layers, so they differ)
    assert sorted(set(t2) - set(same)) == sorted(f"h.{i}.{p}.c_proj.weight" for i in range(2) for p in ("attn", "mlp"))


def _check(folder):
    """Through the program, as a user checks a download."""
    r = subprocess.run([sys.executable, CLI, "check", "--model", str(folder)], capture_output=True, text=True, timeout=900)
    return r.returncode, r.stdout + r.stderr


def test_a_folder_is_checked_without_a_gpu_and_every_mismatch_is_listed(tmp_path):
    d = write_random_model(dict(TINY_A), str(tmp_path / "m"), seed=0)
    good = _tensors(d)
    n_params = sum(t.numel() for t in good.values())
    assert check_model_dir(d) == ("GPT2LMHeadModel", len(good), n_params)
    rc, out = _check(d)
    assert rc == 0 and f"ok: GPT2LMHeadModel, {len(good)} tensors, {n_params} parameters" in out, out
    # the prefix and the mask buffers of exported checkpoints are accepted; float16 and float32 storage too
    t = {"transformer." + k: (v.half() if v.dim() == 2 else v) for k, v in good.items()}
    t["transformer.h.0.attn.bias"] = torch.ones(1, 1, 8, 8)
    t["transformer.h.1.attn.masked_bias"] = torch.tensor(-1e4)
    t["lm_head.weight"] = t["transformer.wte.weight"].clone()
    save_file(t, os.path.join(d, "model.safetensors"))
    assert check_model_dir(d)[0] == "GPT2LMHeadModel" and _check(d)[0] == 0
    # every mismatch in one message
    t = dict(good)
    del t["h.1.ln_2.bias"], t["wpe.weight"]
    t["h.0.mlp.c_fc.weight"] = torch.zeros(256, 64, dtype=torch.bfloat16)     # transposed by mistake
    t["h.0.attn.c_attn.bias"] = torch.zeros(64)
    t["h.7.extra.weight"] = torch.zeros(2)
    save_file(t, os.path.join(d, "model.safetensors"))
    with pytest.raises(WeightsError) as ei:
        check_model_dir(d)
    rc, out = _check(d)
    assert rc == 1
    for text in (str(ei.value), out):
        for piece in ("missing tensors (2)", "h.1.ln_2.bias", "wpe.weight", "unexpected tensors (1)", "h.7.extra.weight",
                      "wrong shapes (2)", "expected [64, 256], found [256, 64]", "h.0.attn.c_attn.bias"):
            assert piece in text, (piece, text)
    # files that are no safetensors files: each is refused with an error that says why
    save_file(good, os.path.join(d, "model.safetensors"))
    raw = open(os.path.join(d, "model.safetensors"), "rb").read()
    hlen = int.from_bytes(raw[:8], "little")
    deep = b"[" * 3_000_000
    negative = raw[8:8 + hlen].replace(b'"shape":[64]', b'"shape":[-64]', 1)
    huge = raw[8:8 + hlen].replace(b'"shape":[64]', b'"shape":[3000000000,3000000000,4]', 1)
    for broken, match in ((raw[:5], "too short"), ((10 ** 9).to_bytes(8, "little") + raw[8:], "header length"),
                          ((2 ** 64 - 1).to_bytes(8, "little") + raw[8:], "header length"),
                          ((2 ** 64 - 8).to_bytes(8, "little") + raw[8:], "header length"),
                          (raw[:8] + b"{" * 20 + raw[28:], "JSON"), (raw[:len(raw) // 2], "offsets"),
                          (len(deep).to_bytes(8, "little") + deep, "nested deeper"),
                          (len(negative).to_bytes(8, "little") + negative + raw[8 + hlen:], "negative dimension"),
                          (len(huge).to_bytes(8, "little") + huge + raw[8 + hlen:], "more elements than can be counted")):
        open(os.path.join(d, "model.safetensors"), "wb").write(broken)
        rc, out = _check(d)
        assert rc == 1 and match in out, (match, out[-300:])
        with pytest.raises(WeightsError, match=match):
            check_model_dir(d)
    os.remove(os.path.join(d, "model.safetensors"))
    rc, out = _check(d)
    assert rc == 1 and "neither model.safetensors" in out
    # the configuration is judged first
    cfg = json.load(open(os.path.join(d, "config.json")))
    json.dump(dict(cfg, n_head=5), open(os.path.join(d, "config.json"), "w"))
    rc, out = _check(d)
    assert rc == 1 and "divisible" in out
    json.dump(dict(cfg, architectures=["Other"], model_type="other"), open(os.path.join(d, "config.json"), "w"))
    rc, out = _check(d)
    assert rc == 1 and "no known architecture" in out and "GPT2LMHeadModel" in out
    open(os.path.join(d, "config.json"), "w").write("{not json")
    assert _check(d)[0] == 1


def test_shards_are_checked_like_one_file(tmp_path):
    d = write_random_model(dict(TINY_B), str(tmp_path / "whole"), seed=4)
    t = _tensors(d)
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
    assert check_model_dir(str(sharded)) == check_model_dir(d)
    # a tensor in two shards is an error that names it; a shard the index names but that is not there too
    save_file({names[0]: t[names[0]], **{n: t[n] for n in parts["model-00002-of-00002.safetensors"]}},
              str(sharded / "model-00002-of-00002.safetensors"))
    with pytest.raises(WeightsError, match="two files"):
        check_model_dir(str(sharded))
    os.remove(sharded / "model-00001-of-00002.safetensors")
    with pytest.raises(WeightsError, match="cannot be opened"):
        check_model_dir(str(sharded))


def test_the_program_writes_model_folders(tmp_path):
    """`mini-llm make-model` and `write_random_model` are one writer: the same folder from a preset or a
    configuration file and a seed. No GPU is needed for it."""
    made = str(tmp_path / "made")
    r = subprocess.run([sys.executable, CLI, "make-model", "--preset", "tiny-b", "--seed", "5", "--out", made],
                       capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stderr
    face = write_random_model("tiny-b", str(tmp_path / "face"), seed=5)
    with open(os.path.join(made, "model.safetensors"), "rb") as a, open(os.path.join(face, "model.safetensors"), "rb") as b:
        assert a.read() == b.read()
    assert json.load(open(os.path.join(made, "config.json"))) == json.load(open(os.path.join(face, "config.json")))
    (tmp_path / "c.json").write_text(json.dumps(TINY_A))
    r = subprocess.run([sys.executable, CLI, "make-model", "--config", str(tmp_path / "c.json"), "--seed", "0", "--weights-dtype", "float32",
                        "--out", made + "32"], capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stderr
    assert _tensors(made + "32")["wte.weight"].dtype == torch.float32 and check_model_dir(made + "32")[1] == 28
    bad = subprocess.run([sys.executable, CLI, "make-model", "--preset", "nothing", "--seed", "0", "--out", made + "x"],
                         capture_output=True, text=True, timeout=900)
    assert bad.returncode == 1 and "unknown preset" in bad.stderr
