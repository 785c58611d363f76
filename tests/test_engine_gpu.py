"""Generation through the entry points on the GPU: the Python Engine, the command line, and
sampling that does not depend on batching."""
import os
import subprocess
import sys

import pytest
import torch

import plain_gpt2
from conftest import TINY

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _prompts(name, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    v = TINY[name][0]["vocab_size"]
    return [torch.randint(0, v - 1, (n,), generator=g).tolist() for n in lengths]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,lengths,n_new", [("a", (5, 17, 33), 16), ("b", (1, 9, 40, 100), 24)])
def test_greedy_generation_matches_plain(tiny_model_dirs, name, lengths, n_new, dtype):
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    cfg, w = plain_gpt2.read_model(tiny_model_dirs[name])
    prompts = _prompts(name, lengths, 1)
    engine = Engine.from_pretrained(tiny_model_dirs[name], dtype=dtype,
                                    options=EngineOptions(kv_block_size=TINY[name][2], total_kv_blocks=64,
                                                          max_batch_num=4, max_tokens_per_step=48, prefill_chunk=16))
    outs = engine.generate(prompts, SamplingParams(max_new_tokens=n_new, ignore_eos=True))
    for p, o in zip(prompts, outs):
        ref = plain_gpt2.greedy_generate(cfg, w, p, n_new)
        if dtype == "float32":
            assert o == ref
        else:
            # bf16 may turn a near-tie; every token must be one the plain model nearly chose
            ids = list(p)
            for t in o:
                row = plain_gpt2.forward_logits(cfg, w, ids)[-1]
                assert row[t] >= row.max() - 0.05, (t, int(row.argmax()))
                ids.append(t)
    assert engine.stats()["free_pages"] == 64 and engine.runner.manager.check() == ""


def _near_ties_only(cfg, w, prompt, out, slack=0.05):
    """Every token is one that the plain model chose or nearly chose, given the tokens before it."""
    ids = list(prompt)
    for t in out:
        row = plain_gpt2.forward_logits(cfg, w, ids)[-1]
        assert row[t] >= row.max() - slack, (t, int(row.argmax()))
        ids.append(t)


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
    engine.runner.cache.poison()
    outs = engine.generate(prompts, SamplingParams(max_new_tokens=14, ignore_eos=True))
    for p, o in zip(prompts, outs):
        if dtype == "float32":
            assert o == plain_gpt2.greedy_generate(cfg, w, p, 14)
        else:
            _near_ties_only(cfg, w, p, o)
    assert engine.stats()["free_pages"] == 30 and engine.runner.manager.check() == ""


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_temperature_sampling_does_not_depend_on_batching(tiny_model_dirs, dtype):
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    prompts = _prompts("b", (1, 9, 40, 100), 4)
    params = [SamplingParams(temperature=0.8, seed=10 + i, max_new_tokens=24, ignore_eos=True) for i in range(4)]
    opts = dict(kv_block_size=8, max_batch_num=4)
    alone = [Engine.from_pretrained(tiny_model_dirs["b"], dtype=dtype, options=EngineOptions(total_kv_blocks=64, **opts))
             .generate([p], sp)[0] for p, sp in zip(prompts, params)]
    assert len({tuple(o) for o in alone}) == 4 and all(len(set(o)) > 3 for o in alone)
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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_decode_matches_eager_steps(tiny_model_dirs, dtype):
    """Decode steps replay as HIP graphs (padded to a bucket of 16 for 11 requests), each launched
    before the previous one's tokens are read; the tokens equal those of the same engine waiting
    for every step, running the static buffers without a graph, and stepping through the general
    step function, replay after replay."""
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    prompts = _prompts("a", (3, 5, 8, 13, 21, 34, 4, 9, 16, 25, 1), 7)
    params = [SamplingParams(temperature=0.0 if i % 2 else 0.7, seed=i, max_new_tokens=20, ignore_eos=True)
              for i in range(len(prompts))]
    outs = {}
    for mode in ("graph", "graph, waited for", "static buffers", "general steps"):
        e = Engine.from_pretrained(tiny_model_dirs["a"], dtype=dtype,
                                   options=EngineOptions(kv_block_size=4, total_kv_blocks=256, max_batch_num=16,
                                                         overlap_decode=(mode != "graph, waited for")))
        assert e.runner.use_graphs and e.runner.fast_decode
        if mode == "static buffers":
            e.runner.use_graphs = False
        if mode == "general steps":
            e.runner.fast_decode = False
        outs[mode] = e.generate(prompts, params)
        graphs = list(e.runner._graphs.values())
        assert (len(graphs) > 0) == (mode != "general steps")
        assert all((g.graph is not None) == mode.startswith("graph") for g in graphs)
        assert e.stats()["free_pages"] == 256 and not e.has_unfinished()
    assert all(o == outs["graph"] for o in outs.values())
    assert all(len(o) == 20 for o in outs["graph"])


def test_scratch_stays_put_while_decode_graphs_of_growing_batches_are_captured(tmp_path):
    """A vocabulary of 50,257 (25 argmax chunks a row) and up to 176 requests, no warm-up: a batch of 8
    captures its graph first, then 176 requests capture the larger ones, then 8 again replay the first
    graph. The kernels' scratch is sized for the largest batch when the runner is built, so its
    addresses never change and the early graph still writes where its replays read; tokens equal those
    of general steps that wait for every token."""
    from mini_llm_amd import Engine, EngineOptions, SamplingParams, write_random_model
    from mini_llm_amd.kernels import ops
    cfg = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=2, n_embd=64, n_head=2, n_inner=128,
               vocab_size=50257, n_positions=48, layer_norm_epsilon=1e-5, activation_function="gelu_new",
               eos_token_id=50256, bos_token_id=50256)
    d = write_random_model(cfg, str(tmp_path / "wide"), seed=6)
    g = torch.Generator().manual_seed(3)
    few = [torch.randint(0, 50256, (3 + i,), generator=g).tolist() for i in range(8)]
    many = [torch.randint(0, 50256, (2 + i % 7,), generator=g).tolist() for i in range(176)]
    sp = SamplingParams(max_new_tokens=5, ignore_eos=True)
    names = ("argmax_values", "argmax_indices", "decode_partials", "decode_counters")

    def run(graphs: bool):
        e = Engine.from_pretrained(d, dtype="float32", options=EngineOptions(
            kv_block_size=4, total_kv_blocks=176 * 4 + 8, max_batch_num=176, max_tokens_per_step=1024,
            prefill_chunk=16, overlap_decode=graphs))
        if not graphs:
            e.runner.fast_decode = False
        before = [ops.scratch_address("cuda:0", n) for n in names]
        assert all(before), "the runner reserves the scratch when it is built"
        outs = [e.generate(few, sp)]
        first = dict(e.runner._graphs)
        outs.append(e.generate(many, sp))
        outs.append(e.generate(few, sp))
        if graphs:
            assert first and all(e.runner._graphs.get(k) is v for k, v in first.items()), "an early graph was dropped"
            assert any(k[0] == 176 for k in e.runner._graphs)
            assert [ops.scratch_address("cuda:0", n) for n in names] == before
        assert e.stats()["free_pages"] == 176 * 4 + 8
        return outs

    with_graphs, general = run(True), run(False)
    assert with_graphs[0] == with_graphs[2]
    assert with_graphs == general


def test_command_line(tiny_model_dirs, tmp_path):
    cfg, w = plain_gpt2.read_model(tiny_model_dirs["a"])
    prompts = _prompts("a", (5, 17), 1)
    lines = [" ".join(map(str, p)) for p in prompts] + ["12 x 3", "999999"]
    cmd = [sys.executable, os.path.join(ROOT, "bin", "mini-llm"), "generate", "--model", tiny_model_dirs["a"],
           "--dtype", "float32", "--max-new-tokens", "6", "--ignore-eos", "--kv-block-size", "4",
           "--total-kv-blocks", "32", "--max-batch-num", "4"]
    r = subprocess.run(cmd, input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    out = r.stdout.strip().splitlines()
    assert len(out) == 4
    for p, line in zip(prompts, out):
        assert line.endswith(" [DONE]")
        assert [int(t) for t in line[:-7].split()] == plain_gpt2.greedy_generate(cfg, w, p, 6)
    assert out[2] == "invalid request" and out[3].startswith("invalid request")
    # a model folder from the command line, then a streamed run of it
    made = str(tmp_path / "made")
    mk = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "mini-llm"), "make-model", "--preset", "tiny-b",
                         "--seed", "1", "--out", made], capture_output=True, text=True, timeout=120)
    assert mk.returncode == 0 and os.path.isfile(os.path.join(made, "model.safetensors"))
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "mini-llm"), "generate", "--model", made,
                        "--prompt-ids", "1 2 3", "--max-new-tokens", "3", "--ignore-eos", "--stream"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    s = r.stdout.strip().splitlines()
    assert len(s) == 3 and s[-1].endswith("[DONE]") and all(l.startswith("0 ") for l in s)


def test_random_preset_entry_points(tmp_path):
    """`--preset` on the command line and `Engine.from_random` generate with the same random
    weights as a folder written by `make-model` with that seed; `step_logits` is the step function."""
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    from mini_llm_amd.engine.step import StepEntry
    cli = os.path.join(ROOT, "bin", "mini-llm")
    made = str(tmp_path / "made")
    mk = subprocess.run([sys.executable, cli, "make-model", "--preset", "tiny-b", "--seed", "5", "--out", made],
                        capture_output=True, text=True, timeout=120)
    assert mk.returncode == 0, mk.stderr
    common = ["--prompt-ids", "4 5 6 7", "--max-new-tokens", "5", "--ignore-eos", "--kv-block-size", "8",
              "--total-kv-blocks", "16", "--max-batch-num", "2"]
    a = subprocess.run([sys.executable, cli, "generate", "--model", made] + common,
                       capture_output=True, text=True, timeout=300)
    b = subprocess.run([sys.executable, cli, "generate", "--preset", "tiny-b", "--weights-seed", "5"] + common,
                       capture_output=True, text=True, timeout=300)
    assert a.returncode == 0 and b.returncode == 0, (a.stderr, b.stderr)
    assert a.stdout == b.stdout and a.stdout.strip().endswith("[DONE]")
    e = Engine.from_random("tiny-b", 5, options=EngineOptions(kv_block_size=8, total_kv_blocks=16, max_batch_num=2))
    out = e.generate([[4, 5, 6, 7]], SamplingParams(max_new_tokens=5, ignore_eos=True))[0]
    assert " ".join(map(str, out)) + " [DONE]" == a.stdout.strip()
    logits = e.step_logits([StepEntry(77, [4, 5, 6, 7], [3])])
    assert logits.shape == (1, e.model.vocab_size) and int(logits[0].argmax()) == out[0]
    e.runner.end_request(77)
    with pytest.raises(ValueError, match="unknown preset"):
        Engine.from_random("no-such-size")
    bad = subprocess.run([sys.executable, cli, "generate", "--preset", "no-such-size", "--prompt-ids", "1"],
                         capture_output=True, text=True, timeout=120)
    assert bad.returncode == 1 and "unknown preset" in bad.stderr


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_end_of_sequence_under_overlapped_graph_decode(tiny_model_dirs, dtype):
    """A decoded end-of-sequence token is read one step late while HIP graphs replay: generation
    still ends with that token for that request only, under page pressure too, and all pages return."""
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    prompts = _prompts("b", (7, 19, 30, 52), 3)

    def run(eos, pages, overlap, **sp):
        e = Engine.from_pretrained(tiny_model_dirs["b"], dtype=dtype,
                                   options=EngineOptions(kv_block_size=8, total_kv_blocks=pages, max_batch_num=4,
                                                         overlap_decode=overlap))
        e.eos_token_id = eos
        out = e.generate(prompts, [SamplingParams(temperature=1.3, seed=20 + i, max_new_tokens=18, **sp)
                                   for i in range(len(prompts))])
        assert e.stats()["free_pages"] == pages and e.runner.manager.check() == "" and not e.has_unfinished()
        return out

    full = run(None, 64, True, ignore_eos=True)
    j = next(j for j in range(2, 18) if full[1][j] not in full[1][:j])
    eos = full[1][j]
    expect = [o[:o.index(eos) + 1] if eos in o else o for o in full]
    assert len(expect[1]) == j + 1
    for pages, overlap in ((64, True), (64, False), (22, True)):
        assert run(eos, pages, overlap) == expect


def test_a_dropped_engine_is_not_collected_while_a_graph_is_captured(tiny_model_dirs):
    """An engine that nobody holds any more, but that sits in a reference cycle, keeps its HIP graphs
    until Python's collector runs. Destroying a graph while another is captured ends the process,
    so the collector runs before a capture and not during it: engines made one after the other,
    with the collector set to run as often as it can, all generate the same tokens."""
    import gc
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    prompts = _prompts("a", (9, 21), 6)
    params = SamplingParams(max_new_tokens=6, ignore_eos=True)
    old = gc.get_threshold()
    gc.set_threshold(1, 1, 1)
    try:
        outs = []
        for _ in range(4):
            e = Engine.from_pretrained(tiny_model_dirs["a"], dtype="bfloat16",
                                       options=EngineOptions(kv_block_size=8, total_kv_blocks=32, max_batch_num=4))
            outs.append(e.generate(prompts, params))
            cycle = [e]
            cycle.append(cycle)                 # garbage only the collector can free
            del e, cycle
    finally:
        gc.set_threshold(*old)
    assert all(o == outs[0] for o in outs) and all(len(x) == 6 for x in outs[0])


def test_warmup_captures_the_decode_graphs_and_changes_nothing(tiny_model_dirs):
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    prompts = _prompts("b", (3, 30, 11), 8)
    params = [SamplingParams(temperature=t, seed=4, max_new_tokens=9, ignore_eos=True) for t in (0.0, 0.9, 0.0)]
    opts = dict(kv_block_size=8, total_kv_blocks=40, max_batch_num=20)
    cold = Engine.from_pretrained(tiny_model_dirs["b"], dtype="bfloat16", options=EngineOptions(**opts))
    expect = cold.generate(prompts, params)
    warm = Engine.from_pretrained(tiny_model_dirs["b"], dtype="bfloat16", options=EngineOptions(**opts))
    sizes = warm.warmup(sampling=True)
    assert sizes == [20, 16, 8, 7, 6, 5, 4, 3, 2, 1]
    captured = dict(warm.runner._graphs)
    assert {k[0] for k in captured} == {24, 16, 8, 7, 6, 5, 4, 3, 2, 1} and len(captured) == 20
    assert warm.stats()["free_pages"] == 40 and not warm.has_unfinished() and not warm.requests
    assert warm.generate(prompts, params) == expect
    assert all(warm.runner._graphs[k] is g for k, g in captured.items())        # nothing captured again
