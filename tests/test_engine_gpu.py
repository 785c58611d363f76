"""Generation through the entry points on the GPU: the engine from Python, the command line, greedy and
temperature sampling that do not depend on batching, the end-of-sequence token, page pressure, the loader's
errors, and two engines side by side. Tokens are compared with the plain implementation's."""
import json
import os
import random
import shutil
import subprocess
import sys

import pytest
import torch

import plain_gpt2
from conftest import TINY, TINY_A, TINY_B

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLI = os.path.join(ROOT, "bin", "mini-llm")
_MASK = (1 << 64) - 1


def _prompts(name, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    v = TINY[name][0]["vocab_size"]
    return [torch.randint(0, v - 1, (n,), generator=g).tolist() for n in lengths]


def _run(args, stdin=None, env=None, timeout=300):
    r = subprocess.run([sys.executable, CLI] + args, input=stdin, capture_output=True, text=True, timeout=timeout, env=env)
    assert r.returncode == 0, r.stderr
    return r.stdout


def _lines(out):
    return [[int(t) for t in l[:-6].split()] for l in out.strip().splitlines()]


def _near_ties_only(cfg, w, prompt, out, slack):
    """Every token is the one the plain model chooses given the tokens before it, or one whose logit lies
    within `slack` of the largest (32-bit: rounding of the sums; bfloat16: of the activations too)."""
    ids = list(prompt)
    for t in out:
        row = plain_gpt2.forward_logits(cfg, w, ids)[-1]
        assert row[t] >= row.max() - slack, (t, int(row.argmax()), float(row.max() - row[t]))
        ids.append(t)


# bfloat16 logits differ from the plain model's by up to 7e-3 at the tiny sizes (replay_cases.TOL): a token
# chosen instead of the plain model's best can lie that far below it on each side
SLACK = {"float32": 1e-5, "bfloat16": 1.5e-2}


def _splitmix64(x):
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def _uniform01(seed, index):
    """The engine's rule: 24 bits of a counter hash of (seed, index of the output among the request's)."""
    return (_splitmix64(_splitmix64(seed & _MASK) ^ (index & _MASK)) >> 40) / float(1 << 24)


def _check_sampled(cfg, w, prompt, out, temperature, seed, slack=1e-5):
    """Every sampled token is the inverse-CDF draw of softmax(plain logits / temperature) at the engine's
    uniform number for (seed, output index), up to `slack` of cumulative probability at a boundary."""
    ids = list(prompt)
    for i, t in enumerate(out):
        row = plain_gpt2.forward_logits(cfg, w, ids)[-1].double()
        c = torch.cumsum(torch.softmax(row / temperature, 0), 0)
        u = _uniform01(seed, i)
        lo = float(c[t - 1]) if t > 0 else 0.0
        assert lo - slack <= u <= float(c[t]) + slack, (i, t, lo, u, float(c[t]))
        ids.append(t)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,lengths,n_new", [("a", (5, 17, 33), 16), ("b", (1, 9, 40, 100), 24)])
def test_greedy_generation_matches_plain(tiny_model_dirs, name, lengths, n_new, dtype):
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    cfg, w = plain_gpt2.read_model(tiny_model_dirs[name])
    prompts = _prompts(name, lengths, 1)
    engine = Engine.from_pretrained(tiny_model_dirs[name], dtype=dtype,
                                    options=EngineOptions(kv_block_size=TINY[name][2], total_kv_blocks=64,
                                                          max_batch_num=4, max_tokens_per_step=48, prefill_chunk=16))
    engine.runner.poison_cache()
    outs = engine.generate(prompts, SamplingParams(max_new_tokens=n_new, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert len(o) == n_new
        if dtype == "float32":
            assert o == plain_gpt2.greedy_generate(cfg, w, p, n_new)
        else:
            _near_ties_only(cfg, w, p, o, SLACK[dtype])
    assert engine.stats()["free_pages"] == 64 and engine.runner.check() == ""


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generation_with_pages_of_twelve_tokens(tiny_model_dirs, dtype):
    """A page size that is no power of two (the command line accepts any): the attention kernels made
    for powers of two step aside for the general one, and prompts that end at, before and after a page's
    edge (11, 12, 13, 24, 25) still decode as the plain model does."""
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    cfg, w = plain_gpt2.read_model(tiny_model_dirs["b"])
    prompts = _prompts("b", (11, 12, 13, 24, 25, 70), 7)
    engine = Engine.from_pretrained(tiny_model_dirs["b"], dtype=dtype,
                                    options=EngineOptions(kv_block_size=12, total_kv_blocks=30, max_batch_num=6,
                                                          max_tokens_per_step=40, prefill_chunk=20))
    engine.runner.poison_cache()
    outs = engine.generate(prompts, SamplingParams(max_new_tokens=14, ignore_eos=True))
    for p, o in zip(prompts, outs):
        if dtype == "float32":
            assert o == plain_gpt2.greedy_generate(cfg, w, p, 14)
        else:
            _near_ties_only(cfg, w, p, o, SLACK[dtype])
    assert engine.stats()["free_pages"] == 30 and engine.runner.check() == ""


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_temperature_sampling_follows_the_plain_distribution_whatever_the_batching(tiny_model_dirs, dtype):
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    cfg, w = plain_gpt2.read_model(tiny_model_dirs["b"])
    prompts = _prompts("b", (1, 9, 40, 100), 4)
    params = [SamplingParams(temperature=0.8, seed=10 + i, max_new_tokens=24, ignore_eos=True) for i in range(4)]
    opts = dict(kv_block_size=8, max_batch_num=4)
    alone = [Engine.from_pretrained(tiny_model_dirs["b"], dtype=dtype, options=EngineOptions(total_kv_blocks=64, **opts))
             .generate([p], sp)[0] for p, sp in zip(prompts, params)]
    assert len({tuple(o) for o in alone}) == 4 and all(len(set(o)) > 3 for o in alone)
    if dtype == "float32":
        for p, sp, o in zip(prompts, params, alone):
            _check_sampled(cfg, w, p, o, sp.temperature, sp.seed)
    tight = Engine.from_pretrained(tiny_model_dirs["b"], dtype=dtype,
                                   options=EngineOptions(total_kv_blocks=26, max_tokens_per_step=32,
                                                         prefill_chunk=16, **opts))
    together = tight.generate(prompts, params)
    st = tight.stats()
    assert st["deferred_prefills"] + st["deferred_decodes"] + st["preemptions"] > 0 and st["free_pages"] == 26
    if dtype == "float32":
        assert together == alone
    else:
        same = sum(a == b for x, y in zip(alone, together) for a, b in zip(x, y))
        assert same >= 0.9 * 96           # rounding may move a draw that sits on a boundary
    # another seed, another sequence; temperature -> 0 is greedy
    e = Engine.from_pretrained(tiny_model_dirs["b"], dtype=dtype, options=EngineOptions(total_kv_blocks=64, **opts))
    other = e.generate([prompts[2]], SamplingParams(temperature=0.8, seed=99, max_new_tokens=24, ignore_eos=True))[0]
    assert other != alone[2]
    cold = e.generate([prompts[2]], SamplingParams(temperature=1e-4, seed=5, max_new_tokens=8, ignore_eos=True))[0]
    greedy = e.generate([prompts[2]], SamplingParams(max_new_tokens=8, ignore_eos=True))[0]
    assert cold == greedy


def test_random_workloads_match_plain_and_give_every_page_back(tiny_model_dirs):
    """Thirty random workloads (page sizes, pools down to one request's worth of pages plus one, batch and
    token budgets, portions, greedy and temperature sampling, steps run ahead or not) in 32-bit: greedy
    requests produce the plain model's tokens, sampled ones its inverse-CDF draws; the workloads do run out
    of pages, nothing fails, and every page comes back."""
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    models = {name: plain_gpt2.read_model(tiny_model_dirs[name]) for name in ("a", "b")}
    preempted = deferred = 0
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
                              ignore_eos=True) for _ in range(n)]
        e = Engine.from_pretrained(tiny_model_dirs[name], dtype="float32", options=o)
        outs = e.generate(prompts, sps)
        for p, sp, out in zip(prompts[:3], sps, outs):          # (the plain model is slow: three requests a workload)
            assert len(out) == new
            if sp.temperature == 0:
                _near_ties_only(*models[name], p, out, SLACK["float32"])
            else:
                _check_sampled(*models[name], p, out, sp.temperature, sp.seed)
        st = e.stats()
        assert st["free_pages"] == st["total_pages"] == pages and st["failures"] == 0, (trial, st)
        assert e.runner.check() == ""
        preempted += st["preemptions"] > 0
        deferred += st["deferred_decodes"] + st["deferred_prefills"] > 0
    assert preempted >= 3 and deferred >= 5


@pytest.mark.parametrize("overlap", [True, False])
def test_generation_stops_at_the_last_position(tiny_model_dirs, overlap):
    """Prompts that end 0, 1, 3 and 10 tokens before the model's last position ask for 10 tokens and get what fits
    (the token after the last position is still chosen: 1, 2, 4 and 10), the plain model's; a prompt longer than
    the positions is refused when it is added."""
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    cfg, w = plain_gpt2.read_model(tiny_model_dirs["a"])
    P = TINY_A["n_positions"]
    e = Engine.from_pretrained(tiny_model_dirs["a"], dtype="float32",
                               options=EngineOptions(kv_block_size=4, total_kv_blocks=200, max_batch_num=8, overlap_decode=overlap))
    g = torch.Generator().manual_seed(1)
    reqs = {}
    for length in (P, P - 1, P - 3, P - 10):
        prompt = torch.randint(0, TINY_A["vocab_size"] - 1, (length,), generator=g).tolist()
        reqs[e.add_request(prompt, SamplingParams(max_new_tokens=10, ignore_eos=True))] = (prompt, [])
    with pytest.raises(ValueError, match="prompt of %d tokens" % (P + 1)):
        e.add_request([1] * (P + 1), SamplingParams(max_new_tokens=2))
    last = {}
    while e.has_unfinished():
        for o in e.step():
            assert o.token >= 0 and o.request_id not in last
            reqs[o.request_id][1].append(o.token)
            if o.finished:
                last[o.request_id] = True
    for rid, (prompt, toks) in reqs.items():
        want = min(10, P - len(prompt) + 1)
        assert len(toks) == want and last.get(rid), (len(prompt), toks)
        _near_ties_only(cfg, w, prompt, toks, SLACK["float32"])
    st = e.stats()
    assert st["free_pages"] == st["total_pages"] and st["failures"] == 0 and st["finished"] == 4


def test_end_of_sequence_token_ends_a_request(tiny_model_dirs, tmp_path):
    """Without --ignore-eos a request ends with the model's end-of-sequence token (read one step late while the
    next step is already in flight); --no-overlap waits for every step and must give the same lines; so must the
    Python entry."""
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    g = torch.Generator().manual_seed(2)
    prompts = [torch.randint(0, 510, (n,), generator=g).tolist() for n in (7, 19, 30)]
    lines = "\n".join(" ".join(map(str, p)) for p in prompts) + "\n"
    base = ["generate", "--model", tiny_model_dirs["a"], "--dtype", "float32", "--max-new-tokens", "14", "--temperature", "1.5",
            "--seed", "3", "--kv-block-size", "4", "--total-kv-blocks", "60", "--max-batch-num", "4"]
    free = _lines(_run(base + ["--ignore-eos"], stdin=lines))
    cfg = json.load(open(os.path.join(tiny_model_dirs["a"], "config.json")))
    # a copy of the model whose end-of-sequence token is one that request 0 samples
    j = next(j for j in range(2, 14) if free[0][j] not in free[0][:j])
    d = str(tmp_path / "eos")
    os.makedirs(d)
    shutil.copy(os.path.join(tiny_model_dirs["a"], "model.safetensors"), d)
    json.dump(dict(cfg, eos_token_id=free[0][j]), open(os.path.join(d, "config.json"), "w"))
    expect = [o[:o.index(free[0][j]) + 1] if free[0][j] in o else o for o in free]
    for extra in ([], ["--no-overlap"]):
        args = [a if a != tiny_model_dirs["a"] else d for a in base] + extra
        assert _lines(_run(args, stdin=lines)) == expect, extra
    assert cfg["eos_token_id"] == 511 and len(expect[0]) == j + 1
    e = Engine.from_pretrained(d, dtype="float32", options=EngineOptions(kv_block_size=4, total_kv_blocks=60, max_batch_num=4))
    got = e.generate(prompts, [SamplingParams(temperature=1.5, seed=3 + i, max_new_tokens=14) for i in range(3)])
    assert got == expect and e.stats()["free_pages"] == 60


def test_steps_launched_ahead_give_the_same_tokens(tiny_model_dirs):
    """Decode steps launched before the previous step's tokens are read (tokens fed on the device) produce what
    step-by-step decoding produces, also when pages run out on the way."""
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    g = torch.Generator().manual_seed(11)
    prompts = [torch.randint(0, 1000, (n,), generator=g).tolist() for n in (3, 20, 41, 64)]
    params = [SamplingParams(temperature=0.7 if i % 2 else 0.0, seed=10 + i, max_new_tokens=12 + 5 * i,
                             ignore_eos=True) for i in range(4)]
    for pages in (64, 24):
        outs = []
        for overlap in (False, True):
            e = Engine.from_pretrained(tiny_model_dirs["b"], dtype="float32", options=EngineOptions(
                kv_block_size=8, total_kv_blocks=pages, max_batch_num=4, max_tokens_per_step=32, prefill_chunk=16,
                overlap_decode=overlap))
            outs.append(e.generate(prompts, params))
            assert e.stats()["free_pages"] == pages and e.runner.check() == ""
        assert outs[0] == outs[1]
        assert [len(o) for o in outs[0]] == [12, 17, 22, 27]


def test_outputs_arrive_in_order_and_a_request_is_aborted_in_flight(tiny_model_dirs):
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    o = EngineOptions(kv_block_size=4, total_kv_blocks=60, max_batch_num=4)
    e = Engine.from_pretrained(tiny_model_dirs["a"], dtype="float32", options=o)
    a = e.add_request([5, 6, 7, 8], SamplingParams(max_new_tokens=6, ignore_eos=True))
    b = e.add_request([9, 10, 11], SamplingParams(max_new_tokens=9, ignore_eos=True))
    seen = {a: [], b: []}
    steps = 0
    while e.has_unfinished():
        for out in e.step():
            seen[out.request_id].append((out.token, out.finished))
        steps += 1
        if steps == 4:
            e.abort(b)               # b has a token in flight; it is dropped
    assert len(seen[a]) == 6 and [f for _, f in seen[a]] == [False] * 5 + [True]
    whole = Engine.from_pretrained(tiny_model_dirs["a"], dtype="float32", options=o).generate(
        [[5, 6, 7, 8], [9, 10, 11]], SamplingParams(max_new_tokens=9, ignore_eos=True))
    assert [t for t, _ in seen[a]] == whole[0][:6]
    assert 0 < len(seen[b]) < 9 and [t for t, _ in seen[b]] == whole[1][:len(seen[b])] and not any(f for _, f in seen[b])
    assert e.stats()["free_pages"] == 60 and e.runner.check() == ""
    assert e.stats()["aborted"] == 1 and e.stats()["failures"] == 0 and e.stats()["finished"] == 1
    with pytest.raises(KeyError):
        e.abort(b)
    # nothing of a finished or aborted request stays behind: its id can be used again
    again = e.add_request([5, 6, 7, 8], SamplingParams(max_new_tokens=6, ignore_eos=True), request_id=a)
    toks = []
    while e.has_unfinished():
        toks += [o.token for o in e.step() if o.request_id == again]
    assert toks == whole[0][:6]
    # requests the engine refuses say why
    with pytest.raises(ValueError, match="token ids"):
        e.add_request([5, 100000], SamplingParams())
    with pytest.raises(ValueError, match="prompt of 0 tokens"):
        e.add_request([], SamplingParams())


def test_command_line(tiny_model_dirs, tmp_path):
    cfg, w = plain_gpt2.read_model(tiny_model_dirs["a"])
    prompts = _prompts("a", (5, 17), 1)
    lines = [" ".join(map(str, p)) for p in prompts] + ["12 x 3", "999999"]
    out = _run(["generate", "--model", tiny_model_dirs["a"], "--dtype", "float32", "--max-new-tokens", "6", "--ignore-eos",
                "--kv-block-size", "4", "--total-kv-blocks", "32", "--max-batch-num", "4"],
               stdin="\n".join(lines) + "\n").strip().splitlines()
    assert len(out) == 4
    for p, line in zip(prompts, out):
        assert line.endswith(" [DONE]")
        assert [int(t) for t in line[:-7].split()] == plain_gpt2.greedy_generate(cfg, w, p, 6)
    assert out[2] == "invalid request" and out[3].startswith("invalid request")
    # a model folder from the command line, then a streamed run of it
    made = str(tmp_path / "made")
    _run(["make-model", "--preset", "tiny-b", "--seed", "1", "--out", made])
    assert os.path.isfile(os.path.join(made, "model.safetensors"))
    s = _run(["generate", "--model", made, "--prompt-ids", "1 2 3", "--max-new-tokens", "3", "--ignore-eos", "--stream"]).strip().splitlines()
    assert len(s) == 3 and s[-1].endswith("[DONE]") and all(l.startswith("0 ") for l in s)
    # the GPU only
    r = subprocess.run([sys.executable, CLI, "generate", "--model", made, "--device", "cpu", "--prompt-ids", "1"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 1 and "no CPU path" in r.stderr


def test_pool_sized_from_free_device_memory_through_every_entry(tiny_model_dirs):
    """`kv_memory_fraction` / `--kv-memory-fraction`: the page pool is sized from the device memory that is free once
    the weights and the largest step's buffers are there (tiny A in bfloat16 holds 512 bytes per token: 2 caches x
    K and V x 64 columns)."""
    from mini_llm_amd import Engine, EngineError, EngineOptions, SamplingParams
    free_before, _ = torch.cuda.mem_get_info()
    o = EngineOptions(kv_block_size=4, total_kv_blocks=7, kv_memory_fraction=0.002, max_batch_num=2)
    e = Engine.from_pretrained(tiny_model_dirs["a"], dtype="bfloat16", options=o)
    pages = e.stats()["total_pages"]
    expect = 0.002 * free_before / (4 * 512)
    assert 0.5 * expect <= pages <= 1.05 * expect and pages > 1000, (pages, expect)
    sp = SamplingParams(max_new_tokens=5, ignore_eos=True)
    toks = e.generate([[1, 2, 3]], sp)[0]
    with pytest.raises(EngineError, match=r"\[0, 1\]"):
        Engine.from_pretrained(tiny_model_dirs["a"], dtype="bfloat16", options=EngineOptions(kv_memory_fraction=1.5))
    # the program: the same option, the same tokens, and its pool in the statistics
    r = subprocess.run([sys.executable, CLI, "generate", "--model", tiny_model_dirs["a"], "--kv-block-size", "4",
                        "--kv-memory-fraction", "0.002", "--max-batch-num", "2", "--prompt-ids", "1 2 3", "--max-new-tokens", "5",
                        "--ignore-eos", "--stats"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert _lines(r.stdout) == [toks]
    stats = json.loads(r.stderr.strip().splitlines()[-1])
    assert 0.5 * expect <= stats["total_pages"] <= 1.05 * expect
    bad = subprocess.run([sys.executable, CLI, "generate", "--model", tiny_model_dirs["a"], "--kv-memory-fraction", "lots",
                          "--prompt-ids", "1"], capture_output=True, text=True, timeout=120)
    assert bad.returncode == 1 and "wants a number" in bad.stderr


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_random_preset_entry_points_give_one_model(tmp_path, dtype):
    """`--preset` on the command line, `Engine.from_random` and a folder written by `make-model` or
    `write_random_model` with that seed are the same model in both precisions; `step_logits` is the step function."""
    from mini_llm_amd import Engine, EngineOptions, SamplingParams, StepEntry, write_random_model
    made = str(tmp_path / "made")
    _run(["make-model", "--preset", "tiny-b", "--seed", "5", "--out", made])
    written = write_random_model("tiny-b", str(tmp_path / "written"), 5)
    assert open(os.path.join(made, "model.safetensors"), "rb").read() == open(os.path.join(written, "model.safetensors"), "rb").read()
    common = ["--dtype", dtype, "--prompt-ids", "4 5 6 7", "--max-new-tokens", "9", "--ignore-eos", "--kv-block-size", "8",
              "--total-kv-blocks", "16", "--max-batch-num", "2"]
    a = _run(["generate", "--model", made] + common)
    b = _run(["generate", "--preset", "tiny-b", "--weights-seed", "5"] + common)
    assert a == b and a.strip().endswith("[DONE]")
    o = EngineOptions(kv_block_size=8, total_kv_blocks=16, max_batch_num=2)
    sp = SamplingParams(max_new_tokens=9, ignore_eos=True)
    e = Engine.from_random("tiny-b", 5, dtype=dtype, options=o)
    out = e.generate([[4, 5, 6, 7]], sp)[0]
    assert [out] == _lines(a)
    assert Engine.from_pretrained(written, dtype=dtype, options=o).generate([[4, 5, 6, 7]], sp)[0] == out
    if dtype == "float32":
        cfg, w = plain_gpt2.read_model(made)
        assert out == plain_gpt2.greedy_generate(cfg, w, [4, 5, 6, 7], 9)
    logits = e.step_logits([StepEntry(77, [4, 5, 6, 7], [3])])
    assert logits.shape == (1, TINY_B["vocab_size"]) and int(logits[0].argmax()) == out[0]
    e.runner.end_request(77)
    with pytest.raises(ValueError, match="unknown preset"):
        Engine.from_random("no-such-size")
    bad = subprocess.run([sys.executable, CLI, "generate", "--preset", "no-such-size", "--prompt-ids", "1"],
                         capture_output=True, text=True, timeout=120)
    assert bad.returncode == 1 and "unknown preset" in bad.stderr


def test_loader_lists_every_mismatch_and_reads_shards(tmp_path):
    """ONE error that lists missing, unexpected and wrong-shape tensors; a checkpoint in two float16 shards gives
    the tokens of the whole one; a configuration the architecture cannot honour is refused by name."""
    from safetensors import safe_open
    from safetensors.torch import save_file
    from mini_llm_amd import Engine, EngineError, EngineOptions, SamplingParams, write_random_model
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
    with pytest.raises(EngineError) as ei:
        Engine.from_pretrained(d, dtype="float32", options=o)
    msg = str(ei.value)
    for piece in ("missing tensors (2)", "h.1.ln_2.bias", "wpe.weight", "unexpected tensors (1)", "h.7.extra.weight",
                  "wrong shapes (2)", "h.0.mlp.c_fc.weight", "h.0.attn.c_attn.bias", "[64, 256]", "[256, 64]"):
        assert piece in msg, (piece, msg)
    os.remove(os.path.join(d, "model.safetensors"))
    with pytest.raises(EngineError, match="neither model.safetensors"):
        Engine.from_pretrained(d, dtype="float32", options=o)

    # two float16 shards against the whole file
    whole = write_random_model(dict(TINY_B), str(tmp_path / "whole"), seed=4, weights_dtype="float32")
    t = {k: (v.half() if v.dim() == 2 else v) for k, v in tensors(whole).items()}
    save_file(t, os.path.join(whole, "model.safetensors"))
    sharded = tmp_path / "sharded"
    sharded.mkdir()
    names = sorted(t)
    parts = {"model-00001-of-00002.safetensors": names[:len(names) // 2],
             "model-00002-of-00002.safetensors": names[len(names) // 2:]}
    for fname, ns in parts.items():
        save_file({n: t[n] for n in ns}, str(sharded / fname))
    json.dump({"metadata": {}, "weight_map": {n: f for f, ns in parts.items() for n in ns}},
              open(sharded / "model.safetensors.index.json", "w"))
    shutil.copy(os.path.join(whole, "config.json"), sharded / "config.json")
    sp = SamplingParams(max_new_tokens=12, ignore_eos=True)
    prompts = [[3, 1, 4, 1, 5, 9, 2, 6], [27, 18, 28]]
    o8 = EngineOptions(kv_block_size=8, total_kv_blocks=32, max_batch_num=2)
    a = Engine.from_pretrained(whole, dtype="float32", options=o8).generate(prompts, sp)
    b = Engine.from_pretrained(str(sharded), dtype="float32", options=o8).generate(prompts, sp)
    cfg, w = plain_gpt2.read_model(whole)
    assert a == b and a == [plain_gpt2.greedy_generate(cfg, w, p, 12) for p in prompts]
    save_file({names[0]: t[names[0]], **{n: t[n] for n in parts["model-00002-of-00002.safetensors"]}},
              str(sharded / "model-00002-of-00002.safetensors"))
    with pytest.raises(EngineError, match="two files"):
        Engine.from_pretrained(str(sharded), dtype="float32", options=o8)

    # configurations
    for change, match in [({"n_head": 5}, "divisible"), ({"activation_function": "relu"}, "activation_function"),
                          ({"tie_word_embeddings": False}, "untied"), ({"scale_attn_by_inverse_layer_idx": True}, "not supported"),
                          ({"architectures": ["SomethingElse"], "model_type": "other"}, "no known architecture")]:
        with pytest.raises(EngineError, match=match):
            Engine.from_random(dict(TINY_A, **change), seed=0, dtype="float32", options=o)


def test_sizes_the_kernels_cannot_take_are_refused_when_the_model_is_built():
    """A head size that is no multiple of 16 is refused with the sizes in the message, not computed wrongly."""
    from mini_llm_amd import Engine, EngineError
    with pytest.raises(EngineError, match="head_dim=12"):
        Engine.from_random(dict(TINY_A, n_embd=48, n_head=4), seed=0)


def test_more_failed_requests_than_a_step_call_has_room_for(tiny_model_dirs):
    """Sixty prompts that can never fit the pool fail in one iteration; the outputs arrive over several calls of
    `step` (whose buffers hold 2 x 4 + 16) and none is lost; requests that fit still generate."""
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    e = Engine.from_pretrained(tiny_model_dirs["a"], dtype="float32",
                               options=EngineOptions(kv_block_size=4, total_kv_blocks=8, max_batch_num=4, prefill_chunk=16))
    sp = SamplingParams(max_new_tokens=3, ignore_eos=True)
    big = [e.add_request([1] * 60, sp) for _ in range(60)]          # 15 pages each, the pool has 8
    small = [e.add_request([5, 6, 7], sp) for _ in range(2)]
    failed, tokens, calls = {}, {r: [] for r in small}, 0
    while e.has_unfinished():
        calls += 1
        outs = e.step()
        assert len(outs) <= 24
        for o in outs:
            if o.token < 0:
                assert o.finished and "pool" in o.error
                failed[o.request_id] = o.error
            else:
                tokens[o.request_id].append(o.token)
    assert sorted(failed) == big and all(len(t) == 3 for t in tokens.values()) and calls >= 4
    assert e.stats()["failures"] == 60 and e.stats()["free_pages"] == 8


def test_a_step_that_fails_leaves_the_runner_as_it_was(tiny_model_dirs):
    """A step with a token outside the vocabulary, with a wanted place outside its tokens, or with counts that make
    no sense is refused with a message; the requests it would have registered hold nothing afterwards, and the
    same ids step normally after it."""
    import ctypes
    import numpy as np
    from mini_llm_amd import EngineError, Runner, StepEntry, native
    cfg = TINY["a"][0]
    runner = Runner(model_dir=tiny_model_dirs["a"], dtype="float32", page_size=4, n_pages=16, max_num_seqs=4)
    with pytest.raises(EngineError, match="token ids must lie in"):
        runner.step([StepEntry(1, [3, 4, 5], want=[2]), StepEntry(2, [7, cfg["vocab_size"]], want=[])])
    with pytest.raises(EngineError, match="wanted index 3 is outside its 3 tokens"):
        runner.step([StepEntry(1, [3, 4, 5], want=[3])])
    info = runner.info()
    assert info["n_requests"] == 0 and info["free_pages"] == 16 and runner.check() == ""
    # the C function itself refuses counts below zero (the Python face cannot produce them)
    lib = native.lib()
    ids, n_tok, toks = np.array([1], np.int64), np.array([-1], np.int32), np.array([3], np.int32)
    n_want, want, out = np.array([0], np.int32), np.array([0], np.int32), np.zeros(cfg["vocab_size"], np.float32)
    rc = lib.mllm_runner_step(runner._h, ids.ctypes.data, n_tok.ctypes.data, toks.ctypes.data, n_want.ctypes.data,
                              want.ctypes.data, 1, out.ctypes.data, 1)
    assert rc == -1 and "brings -1 tokens" in native.last_error()
    assert lib.mllm_runner_step(runner._h, None, None, None, None, None, -2, None, 0) == -1
    # and the ids are free for a proper step
    got = runner.step([StepEntry(1, [3, 4, 5], want=[2]), StepEntry(2, [7, 8], want=[1])])
    assert got.shape == (2, cfg["vocab_size"]) and np.isfinite(got).all()
    runner.end_request(1)
    runner.end_request(2)
    assert runner.info()["free_pages"] == 16


XL_WIDTH = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=2, n_embd=1600, n_head=25, n_inner=6400,
                vocab_size=5003, n_positions=1024, layer_norm_epsilon=1e-5, activation_function="gelu_new",
                eos_token_id=5002, bos_token_id=5002)


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_two_engines_stepped_in_turn_do_not_share_scratch(dtype):
    """Two engines in one process, different weights and prompts, stepped alternately with steps launched ahead
    of the host, so that their kernels overlap on the device: each produces the tokens it produces alone. At
    GPT-2 XL layer widths, 8 requests each: the products that share tiles among workgroups (K = 6400), attention
    split over several workgroups a pair, and the two-stage argmax all use scratch memory, which belongs to an
    engine's own stream."""
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    o = EngineOptions(kv_block_size=16, total_kv_blocks=200, max_batch_num=8, max_tokens_per_step=2048, prefill_chunk=256)
    sp = SamplingParams(max_new_tokens=24, ignore_eos=True)
    g = torch.Generator().manual_seed(5)
    prompts = [[torch.randint(0, 5000, (200 + 7 * i + 50 * k,), generator=g).tolist() for i in range(8)] for k in range(2)]
    alone = []
    for k in range(2):
        e = Engine.from_random(XL_WIDTH, seed=40 + k, dtype=dtype, options=o)
        alone.append(e.generate(prompts[k], sp))
        e.close()
    engines = [Engine.from_random(XL_WIDTH, seed=40 + k, dtype=dtype, options=o) for k in range(2)]
    ids = [[e.add_request(p, sp) for p in prompts[k]] for k, e in enumerate(engines)]
    got = [{r: [] for r in ids[k]} for k in range(2)]
    while any(e.has_unfinished() for e in engines):
        for k, e in enumerate(engines):
            if e.has_unfinished():
                for out in e.step():
                    got[k][out.request_id].append(out.token)
    for k in range(2):
        assert [got[k][r] for r in ids[k]] == alone[k], k
    assert alone[0] != alone[1]


def test_engines_give_their_memory_back(tiny_model_dirs):
    """An engine owns a stream, and the kernels' scratch memory belongs to that stream: closing the engine frees
    both, so that engines made and dropped one after the other do not pile up device memory."""
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    from mini_llm_amd.kernels import ops
    o = EngineOptions(kv_block_size=8, total_kv_blocks=64, max_batch_num=4)
    sp = SamplingParams(max_new_tokens=4, ignore_eos=True)

    def once():
        e = Engine.from_pretrained(tiny_model_dirs["b"], dtype="bfloat16", options=o)
        out = e.generate([[1, 2, 3, 4, 5]], sp)
        held = ops.scratch_bytes()
        e.close()
        return out, held

    first, held = once()
    torch.cuda.synchronize()
    base_scratch, (base_free, _) = ops.scratch_bytes(), torch.cuda.mem_get_info()
    assert held > base_scratch                  # (the engine's stream held scratch of its own while it lived)
    for _ in range(12):
        out, _ = once()
        assert out == first
    torch.cuda.synchronize()
    assert ops.scratch_bytes() == base_scratch
    free, _ = torch.cuda.mem_get_info()
    assert base_free - free < 8 << 20, (base_free, free)


def test_stage_times_of_the_forward_pass(tiny_model_dirs):
    """MINI_LLM_STAGE_TIMES: one line per stage and step on standard error, in the reference's format
    (kind,batch_size,total_tokens,layer,stage,ms); the tokens on standard output are unchanged."""
    cmd = [sys.executable, CLI, "generate", "--model", tiny_model_dirs["a"],
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
