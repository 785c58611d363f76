"""The native engine and its command line (csrc/engine: loader, runner, engine loop, main.cc) on the
GPU: replay against the plain implementation, generation against the plain implementation and
against the Python engine, which composes the same native parts."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_gpt2
import replay_cases as rc
import replay_util as ru
from conftest import TINY

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLI = os.path.join(ROOT, "bin", "mini-llm")


def _run(args, stdin=None, timeout=300):
    r = subprocess.run([sys.executable, CLI] + args, input=stdin, capture_output=True, text=True, timeout=timeout)
    assert r.returncode == 0, r.stderr
    return r.stdout


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["a", "b"])
def test_native_replay_matches_plain(tiny_model_dirs, tmp_path, name, dtype):
    """`mini-llm replay`: the native loader, cache storage and runner under a mixed trace with a pool made for
    exactly what the trace needs, page size 16 (the pages are used again)."""
    reqs = rc.requests_for(name, seed=4, lengths=rc.LENGTHS[name][:4] + [2, 64])
    steps, _ = ru.trace_mixed(reqs, seed=4)
    out_dir = str(tmp_path / "out")
    cmd = [sys.executable, CLI, "replay", "--model", tiny_model_dirs[name], "--dtype", dtype, "--out", out_dir,
           "--max-tokens", str(ru.peak_tokens(steps))]
    p = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for s in steps:
            p.stdin.write(json.dumps(s) + "\n")
            p.stdin.flush()
            assert p.stdout.readline().strip() == f"done {s['step']}"
        p.stdin.close()
        assert p.wait(timeout=120) == 0
    finally:
        if p.poll() is None:
            p.kill()
    out = {}
    for s in steps:
        n = sum(len(e["want"]) for e in s["entries"])
        if n:
            out[s["step"]] = np.fromfile(os.path.join(out_dir, f"{s['step']}.f32"), dtype="<f4").reshape(n, -1)
    rc.check_against_plain(tiny_model_dirs[name], name, reqs, steps, out, dtype, label="native replay")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_native_generation_matches_plain_and_the_python_engine(tiny_model_dirs, dtype):
    """Greedy and sampled generation through the native program: continuous batching of more requests than
    a step holds, prompts cut into portions, so few pages that requests are deferred or preempted."""
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    cfg, w = plain_gpt2.read_model(tiny_model_dirs["b"])
    g = torch.Generator().manual_seed(8)
    prompts = [torch.randint(0, 999, (n,), generator=g).tolist() for n in (1, 9, 40, 100, 17, 33, 64)]
    lines = "\n".join(" ".join(map(str, p)) for p in prompts) + "\n"
    common = ["--model", tiny_model_dirs["b"], "--dtype", dtype, "--max-new-tokens", "12", "--ignore-eos",
              "--kv-block-size", "8", "--total-kv-blocks", "34", "--max-batch-num", "4", "--max-tokens-per-step", "40",
              "--prefill-chunk", "16"]
    opts = EngineOptions(kv_block_size=8, total_kv_blocks=34, max_batch_num=4, max_tokens_per_step=40, prefill_chunk=16)
    # greedy
    out = _run(["generate"] + common, stdin=lines).strip().splitlines()
    assert len(out) == len(prompts) and all(l.endswith("[DONE]") for l in out)
    native = [[int(t) for t in l[:-6].split()] for l in out]
    for p, o in zip(prompts, native):
        assert len(o) == 12
        if dtype == "float32":
            assert o == plain_gpt2.greedy_generate(cfg, w, p, 12)
        else:
            ids = list(p)
            for t in o:
                row = plain_gpt2.forward_logits(cfg, w, ids)[-1]
                assert row[t] >= row.max() - 0.05, (t, int(row.argmax()))
                ids.append(t)
    python = Engine.from_pretrained(tiny_model_dirs["b"], dtype=dtype, options=opts).generate(
        prompts, SamplingParams(max_new_tokens=12, ignore_eos=True))
    if dtype == "float32":
        assert native == python
    # temperature sampling: the same draws as the Python engine (seed + request index, counter hash per output)
    out = _run(["generate"] + common + ["--temperature", "0.8", "--seed", "10", "--stats"], stdin=lines).strip().splitlines()
    native = [[int(t) for t in l[:-6].split()] for l in out]
    python = Engine.from_pretrained(tiny_model_dirs["b"], dtype=dtype, options=opts).generate(
        prompts, [SamplingParams(temperature=0.8, seed=10 + i, max_new_tokens=12, ignore_eos=True) for i in range(len(prompts))])
    if dtype == "float32":
        assert native == python
    else:
        same = sum(a == b for x, y in zip(native, python) for a, b in zip(x, y))
        assert same >= 0.85 * 12 * len(prompts)
    assert len({tuple(o) for o in native}) == len(prompts)


def test_native_engine_ends_requests_at_the_end_of_sequence_token(tiny_model_dirs):
    """Without --ignore-eos a request ends with the model's end-of-sequence token (read one step late while the
    next step is already in flight); --no-overlap waits for every step and must give the same lines."""
    g = torch.Generator().manual_seed(2)
    prompts = [torch.randint(0, 510, (n,), generator=g).tolist() for n in (7, 19, 30)]
    lines = "\n".join(" ".join(map(str, p)) for p in prompts) + "\n"
    base = ["generate", "--model", tiny_model_dirs["a"], "--dtype", "float32", "--max-new-tokens", "14", "--temperature", "1.5",
            "--seed", "3", "--kv-block-size", "4", "--total-kv-blocks", "60", "--max-batch-num", "4"]
    free = [[int(t) for t in l[:-6].split()] for l in _run(base + ["--ignore-eos"], stdin=lines).strip().splitlines()]
    cfg = json.load(open(os.path.join(tiny_model_dirs["a"], "config.json")))
    eos = cfg["eos_token_id"]
    # make a copy of the model whose end-of-sequence token is one that request 0 samples
    j = next(j for j in range(2, 14) if free[0][j] not in free[0][:j])
    import shutil
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        shutil.copy(os.path.join(tiny_model_dirs["a"], "model.safetensors"), d)
        json.dump(dict(cfg, eos_token_id=free[0][j]), open(os.path.join(d, "config.json"), "w"))
        expect = [o[:o.index(free[0][j]) + 1] if free[0][j] in o else o for o in free]
        for extra in ([], ["--no-overlap"]):
            args = [a if a != tiny_model_dirs["a"] else d for a in base] + extra
            got = [[int(t) for t in l[:-6].split()] for l in _run(args, stdin=lines).strip().splitlines()]
            assert got == expect, extra
    assert eos == 511 and len(expect[0]) == j + 1


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_native_engine_through_its_python_face(tiny_model_dirs, dtype):
    """`NativeEngine` (the C ABI mllm_engine_*): the same tokens as the Python engine, request by request
    through add_request/step, random weights made in memory equal to a written folder's, counters and pages
    accounted for, an unknown token refused."""
    from mini_llm_amd import Engine, EngineOptions, NativeEngine, SamplingParams
    g = torch.Generator().manual_seed(12)
    prompts = [torch.randint(0, 511, (n,), generator=g).tolist() for n in (5, 17, 33, 3, 60)]
    o = EngineOptions(kv_block_size=4, total_kv_blocks=24, max_batch_num=3, max_tokens_per_step=24, prefill_chunk=16)
    sp = [SamplingParams(temperature=0.0 if i % 2 else 0.9, seed=i, max_new_tokens=10, ignore_eos=True) for i in range(5)]
    native = NativeEngine.from_pretrained(tiny_model_dirs["a"], dtype=dtype, options=o)
    python = Engine.from_pretrained(tiny_model_dirs["a"], dtype=dtype, options=o)
    a, b = native.generate(prompts, sp), python.generate(prompts, sp)
    if dtype == "float32":
        assert a == b
    else:
        assert sum(x == y for p, q in zip(a, b) for x, y in zip(p, q)) >= 0.85 * 50
    st = native.stats()
    assert st["free_pages"] == st["total_pages"] == 24 and st["finished"] == 5 and st["failures"] == 0
    assert st["deferred_prefills"] + st["deferred_decodes"] + st["preemptions"] > 0
    # step by step, with an abort in flight
    r0 = native.add_request(prompts[0], SamplingParams(max_new_tokens=6, ignore_eos=True))
    r1 = native.add_request(prompts[1], SamplingParams(max_new_tokens=9, ignore_eos=True))
    seen = {r0: [], r1: []}
    steps = 0
    while native.has_unfinished():
        for out in native.step():
            seen[out.request_id].append((out.token, out.finished))
        steps += 1
        if steps == 4:
            native.abort(r1)
    assert [f for _, f in seen[r0]] == [False] * 5 + [True] and 0 < len(seen[r1]) < 9
    assert native.stats()["free_pages"] == 24
    with pytest.raises(ValueError, match="token ids"):
        native.add_request([5, 512])
    # random weights in memory: the same model as the folder the generator writes
    from conftest import TINY_A
    mem = NativeEngine.from_random(dict(TINY_A), seed=0, dtype=dtype, options=o)
    greedy = SamplingParams(max_new_tokens=8, ignore_eos=True)
    assert mem.generate(prompts[:3], greedy) == native.generate(prompts[:3], greedy)


def test_pool_sized_from_free_device_memory(tiny_model_dirs):
    """`kv_memory_fraction`: both engines size the page pool from the device memory that is free once the
    weights are loaded (tiny A in bfloat16 holds 512 bytes per token: 2 caches x K and V x 64 columns)."""
    from mini_llm_amd import Engine, EngineOptions, NativeEngine, SamplingParams
    free_before, _ = torch.cuda.mem_get_info()
    o = EngineOptions(kv_block_size=4, total_kv_blocks=7, kv_memory_fraction=0.002, max_batch_num=2)
    native = NativeEngine.from_pretrained(tiny_model_dirs["a"], dtype="bfloat16", options=o)
    pages = native.stats()["total_pages"]
    expect = 0.002 * free_before / (4 * 512)
    assert 0.5 * expect <= pages <= 1.05 * expect and pages > 1000, (pages, expect)
    python = Engine.from_pretrained(tiny_model_dirs["a"], dtype="bfloat16", options=o)
    assert 0.5 * expect <= python.stats()["total_pages"] <= 1.05 * expect
    sp = SamplingParams(max_new_tokens=5, ignore_eos=True)
    assert native.generate([[1, 2, 3]], sp) == python.generate([[1, 2, 3]], sp)
    with pytest.raises((RuntimeError, ValueError), match="at most 1"):
        NativeEngine.from_pretrained(tiny_model_dirs["a"], dtype="bfloat16", options=EngineOptions(kv_memory_fraction=1.5))


def test_native_loader_lists_every_mismatch_and_reads_shards(tmp_path):
    """The C++ loader: ONE error that lists missing, unexpected and wrong-shape tensors; a checkpoint in two
    float16 shards gives the logits of the whole one; a configuration it cannot honour is refused by name."""
    import json
    from safetensors import safe_open
    from safetensors.torch import save_file
    from conftest import TINY_A, TINY_B
    from mini_llm_amd import EngineOptions, NativeEngine, SamplingParams, write_random_model
    o = EngineOptions(kv_block_size=4, total_kv_blocks=64, max_batch_num=2)

    def tensors(d):
        with safe_open(os.path.join(d, "model.safetensors"), framework="pt") as f:
            return {k: f.get_tensor(k) for k in f.keys()}

    d = write_random_model(dict(TINY_A), str(tmp_path / "m"), seed=0)
    t = tensors(d)
    del t["h.1.ln_2.bias"], t["wpe.weight"]
    t["h.0.mlp.c_fc.weight"] = torch.zeros(256, 64, dtype=torch.bfloat16)     # transposed by mistake
    t["h.0.attn.c_attn.bias"] = torch.zeros(64)
    t["h.7.extra.weight"] = torch.zeros(2)
    save_file(t, os.path.join(d, "model.safetensors"))
    with pytest.raises(RuntimeError) as ei:
        NativeEngine.from_pretrained(d, dtype="float32", options=o)
    msg = str(ei.value)
    for piece in ("missing tensors (2)", "h.1.ln_2.bias", "wpe.weight", "unexpected tensors (1)", "h.7.extra.weight",
                  "wrong shapes (2)", "h.0.mlp.c_fc.weight", "h.0.attn.c_attn.bias", "[64, 256]", "[256, 64]"):
        assert piece in msg, (piece, msg)
    os.remove(os.path.join(d, "model.safetensors"))
    with pytest.raises(RuntimeError, match="neither model.safetensors"):
        NativeEngine.from_pretrained(d, dtype="float32", options=o)

    # two float16 shards against the whole file
    whole = write_random_model(dict(TINY_B), str(tmp_path / "whole"), seed=4, weights_dtype="float16")
    t = tensors(whole)
    sharded = tmp_path / "sharded"
    sharded.mkdir()
    names = sorted(t)
    parts = {"model-00001-of-00002.safetensors": names[:len(names) // 2],
             "model-00002-of-00002.safetensors": names[len(names) // 2:]}
    for fname, ns in parts.items():
        save_file({n: t[n] for n in ns}, str(sharded / fname))
    json.dump({"metadata": {}, "weight_map": {n: f for f, ns in parts.items() for n in ns}},
              open(sharded / "model.safetensors.index.json", "w"))
    json.dump(json.load(open(os.path.join(whole, "config.json"))), open(sharded / "config.json", "w"))
    sp = SamplingParams(max_new_tokens=12, ignore_eos=True)
    prompts = [[3, 1, 4, 1, 5, 9, 2, 6], [27, 18, 28]]
    o8 = EngineOptions(kv_block_size=8, total_kv_blocks=32, max_batch_num=2)
    a = NativeEngine.from_pretrained(whole, dtype="float32", options=o8).generate(prompts, sp)
    b = NativeEngine.from_pretrained(str(sharded), dtype="float32", options=o8).generate(prompts, sp)
    assert a == b and all(len(x) == 12 for x in a)
    save_file({names[0]: t[names[0]], **{n: t[n] for n in parts["model-00002-of-00002.safetensors"]}},
              str(sharded / "model-00002-of-00002.safetensors"))
    with pytest.raises(RuntimeError, match="two files"):
        NativeEngine.from_pretrained(str(sharded), dtype="float32", options=o8)

    # configurations
    for change, match in [({"n_head": 5}, "divisible"), ({"activation_function": "relu"}, "activation_function"),
                          ({"tie_word_embeddings": False}, "untied"), ({"scale_attn_by_inverse_layer_idx": True}, "not supported"),
                          ({"architectures": ["SomethingElse"], "model_type": "other"}, "no known architecture")]:
        with pytest.raises(RuntimeError, match=match):
            NativeEngine.from_random(dict(TINY_A, **change), seed=0, dtype="float32", options=o)


def test_native_and_python_engines_agree_under_random_options(tiny_model_dirs):
    """Thirty random workloads (page sizes, pools down to one request's worth of pages plus one, batch and
    token budgets, portions, greedy and temperature sampling, end-of-sequence on and off, steps run ahead or
    not): the C++ engine loop and the Python one produce the same tokens in 32-bit, make the same number of
    preemptions, and give every page back."""
    import random
    from mini_llm_amd import Engine, EngineOptions, NativeEngine, SamplingParams
    preempted = 0
    for trial in range(30):
        rnd = random.Random(19000 + trial)
        name = rnd.choice(["a", "b"])
        cfg = TINY[name][0]
        P, V = cfg["n_positions"], cfg["vocab_size"]
        page, n, new = rnd.choice([4, 8, 16]), rnd.randint(1, 9), rnd.randint(1, 20)
        lens = [rnd.choice([1, 2, rnd.randint(3, P - new - 1), rnd.randint(3, 40)]) for _ in range(n)]
        need_one = -(-(max(lens) + new) // page)
        pages = rnd.randint(need_one + 1, need_one * rnd.randint(1, 2) + 2)
        chunk = rnd.choice([4, 8, 16, 32, 64])
        o = EngineOptions(kv_block_size=page, total_kv_blocks=pages, max_batch_num=rnd.randint(1, 8),
                          max_tokens_per_step=rnd.choice([chunk, 2 * chunk, 64, 128]) + 8, prefill_chunk=chunk,
                          overlap_decode=rnd.random() < 0.8)
        g = torch.Generator().manual_seed(trial)
        prompts = [torch.randint(0, V - 1, (l,), generator=g).tolist() for l in lens]
        sps = [SamplingParams(temperature=rnd.choice([0.0, 0.0, 0.7, 1.2]), seed=rnd.randint(0, 99), max_new_tokens=new,
                              ignore_eos=rnd.random() < 0.7) for _ in range(n)]
        a = NativeEngine.from_pretrained(tiny_model_dirs[name], dtype="float32", options=o)
        b = Engine.from_pretrained(tiny_model_dirs[name], dtype="float32", device="cuda:0", options=o)
        assert a.generate(prompts, sps) == b.generate(prompts, sps), (trial, o, lens, new)
        sa, sb = a.stats(), b.stats()
        assert sa["free_pages"] == sa["total_pages"] == pages and sb["free_pages"] == pages, (trial, sa, sb)
        assert sa["preemptions"] == sb["preemptions"] and sa["deferred_decodes"] == sb["deferred_decodes"], (trial, sa, sb)
        preempted += sa["preemptions"] > 0
    assert preempted >= 3              # (the workloads do run out of pages)


def test_stage_times_of_the_native_forward_pass(tiny_model_dirs):
    """MINI_LLM_STAGE_TIMES: one line per stage and step on standard error, in the reference's format
    (kind,batch_size,total_tokens,layer,stage,ms); the tokens on standard output are unchanged."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cmd = [sys.executable, os.path.join(root, "bin", "mini-llm"), "generate", "--model", tiny_model_dirs["a"],
           "--prompt-ids", "5 17 3 9 100", "--max-new-tokens", "4", "--ignore-eos", "--kv-block-size", "4",
           "--total-kv-blocks", "32", "--no-overlap"]
    plain = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    timed = subprocess.run(cmd, capture_output=True, text=True, timeout=300, env=dict(os.environ, MINI_LLM_STAGE_TIMES="1"))
    assert plain.returncode == 0 and timed.returncode == 0, (plain.stderr, timed.stderr)
    assert plain.stdout == timed.stdout and plain.stdout.strip().endswith("[DONE]")
    assert "kind,batch_size" not in plain.stderr
    lines = [l for l in timed.stderr.splitlines() if l.count(",") == 5]
    assert lines[0] == "kind,batch_size,total_tokens,layer,stage,ms"
    rows = [l.split(",") for l in lines[1:]]
    # four steps (the prompt, then three single tokens), each: embed, 2 layers x 5 stages, head
    assert len(rows) == 4 * 12, timed.stderr
    assert [r[4] for r in rows[:12]] == ["embed"] + ["qkv", "attention", "out_proj", "fc1", "fc2"] * 2 + ["head"]
    assert [r[3] for r in rows[:12]] == ["-1"] + ["0"] * 5 + ["1"] * 5 + ["-1"]
    assert rows[0][:3] == ["prefill", "1", "5"] and rows[12][:3] == ["decode", "1", "1"]
    assert all(0.0 < float(r[5]) < 100.0 for r in rows)
