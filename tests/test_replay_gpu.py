"""The engine on the GPU against the plain implementation, in 32-bit and in bfloat16:
each request alone and whole; most of it in one step and the last 32 tokens one by one;
portions of changing size down to two tokens; and mixed batches of up to four live requests
with so few pages that they are used again. Through the engine's runner in this process, and
through bin/trace_run (the engine's `mini-llm replay`) as a user drives it: one runner either way."""
import numpy as np
import pytest

import plain_gpt2
import replay_cases as rc
import replay_util as ru
from conftest import CONFIGS, TINY

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
FAMILIES = ["whole", "decode_tail", "chunks", "mixed"]


def _runner(model_dir, name, dtype, n_pages, page=None, max_num_seqs=8):
    from mini_llm_amd import Runner
    runner = Runner(model_dir=model_dir, dtype=dtype, page_size=page or CONFIGS[name][2], n_pages=n_pages,
                    max_num_seqs=max_num_seqs)
    runner.poison_cache()          # an unwritten or stale page that is read shows up as NaN
    return runner


def _all_pages_back(runner, n_pages):
    assert runner.check() == ""
    info = runner.info()
    assert info["free_pages"] == n_pages and info["n_requests"] == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["a", "b"])
@pytest.mark.parametrize("family", FAMILIES)
def test_schedule_families_match_plain(tiny_model_dirs, name, family, dtype):
    reqs = rc.requests_for(name)
    steps = rc.families(reqs)[family]
    page = TINY[name][2]
    n_pages = ru.peak_tokens(steps) // page
    runner = _runner(tiny_model_dirs[name], name, dtype, n_pages)
    out = ru.run_in_process(runner, steps)
    rc.check_against_plain(tiny_model_dirs[name], name, reqs, steps, out, dtype, label=family)
    _all_pages_back(runner, n_pages)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["small2", "xl2"])
@pytest.mark.parametrize("family", FAMILIES)
def test_schedule_families_match_plain_at_real_layer_sizes(real_model_dirs, name, family, dtype):
    """The same four families at the layer sizes of GPT-2 small and XL (two layers, the real vocabulary):
    the sizes at which the engine picks the matrix-core attention, the 64-wide decode attention, the
    two-tile and shared-tile few-row products, the large tiles and the staged head. Requests of the
    reference's page-edge lengths (5, 15, 16, 17) and of 41, 130 and 300 tokens."""
    reqs = rc.requests_for(name)
    steps = rc.families(reqs, large=True)[family]
    skip = rc.thin(steps)
    n_pages = ru.peak_tokens(steps) // 16
    runner = _runner(real_model_dirs[name], name, dtype, n_pages)
    out = ru.run_in_process(runner, steps)
    rc.check_against_plain(real_model_dirs[name], name, reqs, steps, out, dtype, skip=skip, label=family)
    _all_pages_back(runner, n_pages)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["a", "b"])
@pytest.mark.parametrize("family", FAMILIES)
def test_trace_run_program_families(tiny_model_dirs, tmp_path, name, family, dtype):
    """Every family through bin/trace_run with its default page size, the pool made for exactly --max-tokens."""
    reqs = rc.requests_for(name, seed=2, lengths=rc.LENGTHS[name][:4] + [2, 64])
    steps = rc.families(reqs, seed=2)[family]
    skip = set()
    if family == "mixed":
        # a step in which nothing is wanted writes no file
        for e in steps[0]["entries"]:
            e["want"] = []
            skip |= {(e["id"], p) for p in range(len(e["tokens"]))}
    out = ru.run_trace_run(tiny_model_dirs[name], dtype, steps, str(tmp_path / "out"), ru.peak_tokens(steps))
    if family == "mixed":
        assert 0 not in out
    rc.check_against_plain(tiny_model_dirs[name], name, reqs, steps, out, dtype, skip=skip, label="program " + family)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["small2", "xl2"])
@pytest.mark.parametrize("family", ["decode_tail", "mixed"])
def test_trace_run_program_at_real_layer_sizes(real_model_dirs, tmp_path, name, family, dtype):
    reqs = rc.requests_for(name, seed=4, lengths=[15, 17, 130, 300])
    steps = rc.families(reqs, seed=4, large=True)[family]
    skip = rc.thin(steps)
    out = ru.run_trace_run(real_model_dirs[name], dtype, steps, str(tmp_path / "out"), ru.peak_tokens(steps))
    rc.check_against_plain(real_model_dirs[name], name, reqs, steps, out, dtype, skip=skip, label="program " + family)


def test_trace_run_program_names_and_refusals(tiny_model_dirs, tmp_path):
    """Steps may be named by words, request ids may be numbers or strings, the output folder is made with the
    folders above it; a step that cannot run ends the program with a message that names the step and says which
    of the trace's ids the request is, and with a status other than 0."""
    import json
    import os
    import subprocess
    import sys
    name, dtype = "a", "float32"
    reqs = rc.requests_for(name, seed=6, lengths=[9, 5])
    a, b = reqs["r0"], reqs["r1"]
    steps = [{"step": "first", "entries": [{"id": "a", "tokens": a[:7], "want": [6]}, {"id": 7, "tokens": b, "want": [0, 4]}], "end": [7]},
             {"step": 1, "entries": [{"id": "a", "tokens": a[7:], "want": [0, 1]}], "end": ["a"]}]
    out_dir = str(tmp_path / "deep" / "er" / "out")
    out = ru.run_trace_run(tiny_model_dirs[name], dtype, steps, out_dir, 128)
    assert sorted(os.listdir(out_dir)) == ["1.f32", "first.f32"]
    cfg, w = plain_gpt2.read_model(tiny_model_dirs[name])
    ref_a, ref_b = plain_gpt2.forward_logits(cfg, w, a).numpy(), plain_gpt2.forward_logits(cfg, w, b).numpy()
    tol = rc.TOL[(name, dtype)]["max_abs"]
    assert np.abs(out["first"] - np.stack([ref_a[6], ref_b[0], ref_b[4]])).max() <= tol
    assert np.abs(out[1] - np.stack([ref_a[7], ref_a[8]])).max() <= tol
    bad = {"step": 3, "entries": [{"id": "x", "tokens": [1, 2], "want": [5]}], "end": []}
    r = subprocess.run([sys.executable, os.path.join(ru.ROOT, "bin", "trace_run"), "--model", tiny_model_dirs[name], "--dtype", dtype,
                        "--out", out_dir, "--max-tokens", "64"], input=json.dumps(bad) + "\n", capture_output=True, text=True, timeout=300)
    assert r.returncode != 0 and "done" not in r.stdout
    assert "step 3" in r.stderr and "wanted index 5 is outside its 2 tokens" in r.stderr and 'is "x"' in r.stderr


@pytest.mark.parametrize("dtype", DTYPES)
def test_schedules_agree_with_each_other(tiny_model_dirs, dtype):
    """Cutting, batching and page placement change the logits by rounding only."""
    reqs = rc.requests_for("b", seed=5, lengths=[25, 64, 124, 9])
    outs = {}
    for fam, steps in rc.families(reqs, seed=5).items():
        runner = _runner(tiny_model_dirs["b"], "b", dtype, 64)
        outs[fam] = ru.collect(steps, ru.run_in_process(runner, steps), 1000)
    tol = 2e-6 if dtype == "float32" else 8e-3
    worst = 0.0
    for rid, toks in reqs.items():
        for pos in range(len(toks)):
            base = outs["whole"][rid][pos]
            for fam in ("decode_tail", "chunks", "mixed"):
                d = np.abs(outs[fam][rid][pos] - base).max()
                worst = max(worst, d)
                assert d <= tol, (fam, rid, pos, d)
    print(f"worst difference between schedules [{dtype}]: {worst:.3e} (allowed {tol:.1e})")


@pytest.mark.parametrize("dtype", DTYPES)
def test_first_tokens_and_long_decoding(tiny_model_dirs, dtype):
    """The first tokens of a sequence one by one, then decoding up to the last position."""
    name = "b"
    n = TINY[name][0]["n_positions"]
    reqs = rc.requests_for(name, seed=9, lengths=[n])
    toks = reqs["r0"]
    steps = [{"step": i, "entries": [{"id": "r0", "tokens": [toks[i]], "want": [0]}],
              "end": ["r0"] if i == n - 1 else []} for i in range(n)]
    runner = _runner(tiny_model_dirs[name], name, dtype, n // TINY[name][2])
    out = ru.run_in_process(runner, steps)
    rc.check_against_plain(tiny_model_dirs[name], name, reqs, steps, out, dtype)


def _other(L, H, dh, F, V, P, eps, act):
    return dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=L, n_embd=H * dh, n_head=H, n_inner=F,
                vocab_size=V, n_positions=P, layer_norm_epsilon=eps, activation_function=act, eos_token_id=V - 1,
                bos_token_id=V - 1)


# sizes that neither the tiny nor the real configurations have: seven heads of 16, three of 48, two of 80, one of 256;
# widths, inner widths and vocabularies that are no power of two; one to five layers; four eps; the three activation names
OTHER_SIZES = {
    "7x16": _other(2, 7, 16, 200, 517, 192, 1e-3, "gelu"),
    "3x48": _other(3, 3, 48, 576, 777, 200, 1e-6, "gelu_pytorch_tanh"),
    "2x80": _other(5, 2, 80, 328, 4099, 300, 1e-5, "gelu_new"),
    "1x256": _other(1, 1, 256, 1000, 333, 130, 1e-4, "gelu"),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(OTHER_SIZES))
def test_other_sizes_end_to_end(tmp_path, name, dtype):
    """Whole prompts and mixed batches at further sizes, against the plain implementation. Allowed: about three
    times the worst seen over these four (float32 1.5e-6 of a row, mean 2.0e-7; bfloat16 4.3e-3 and 1.0e-3; the
    logits' own standard deviation is 0.2 to 0.3)."""
    from mini_llm_amd import Runner, write_random_model
    cfg = OTHER_SIZES[name]
    d = write_random_model(cfg, str(tmp_path / name), seed=50 + len(name))
    pc, w = plain_gpt2.read_model(d)
    P, V = cfg["n_positions"], cfg["vocab_size"]
    reqs = ru.random_requests(V, [1, 2, 15, 16, 17, P // 3, P - 1, P], seed=300)
    ref = {rid: plain_gpt2.forward_logits(pc, w, list(t)).numpy() for rid, t in reqs.items()}
    tol = dict(max_abs=4.5e-6, mean_abs=6e-7) if dtype == "float32" else dict(max_abs=1.3e-2, mean_abs=3e-3)
    worst = worst_mean = 0.0
    for fam, steps, page in (("whole", ru.trace_whole(reqs), 16), ("mixed", ru.trace_mixed(reqs, seed=3)[0], 8)):
        n_pages = -(-ru.peak_tokens(steps) // page)
        runner = Runner(model_dir=d, dtype=dtype, page_size=page, n_pages=n_pages, max_num_seqs=8)
        runner.poison_cache()
        got = ru.collect(steps, ru.run_in_process(runner, steps), V)
        for rid, rows in got.items():
            assert len(rows) == len(reqs[rid])
            for pos, row in rows.items():
                assert np.isfinite(row).all(), (fam, rid, pos)
                diff = np.abs(row.astype(np.float64) - ref[rid][pos])
                worst, worst_mean = max(worst, diff.max()), max(worst_mean, diff.mean())
                assert diff.max() <= tol["max_abs"] and diff.mean() <= tol["mean_abs"], (fam, rid, pos, diff.max(), diff.mean())
        _all_pages_back(runner, n_pages)
    print(f"worst difference from plain at {name} [{dtype}]: max {worst:.3e}, mean {worst_mean:.3e} "
          f"(allowed {tol['max_abs']:.1e}, {tol['mean_abs']:.1e})")


# A context far beyond GPT-2's own: n_positions is a free key of config.json. Narrow (two heads of 64), so
# that the plain implementation's 4,700 x 4,700 scores stay cheap.
LONG = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=2, n_embd=128, n_head=2, n_inner=256,
            vocab_size=300, n_positions=8192, layer_norm_epsilon=1e-5, activation_function="gelu_new",
            eos_token_id=299, bos_token_id=299)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_context_decode_splits_keys_over_the_chip(tmp_path, dtype):
    """One request of 4,732 tokens: 4,700 in one step, the last 32 one by one, beside a short request that
    decodes with it; before it a request that ends, so that the long one writes pages that were used. With
    so few (token, head) pairs and so many keys the decode kernel splits every pair's keys over at least
    eight workgroups and a second kernel merges their states: read back from the ops, not taken on faith.
    Block tables have 296 entries."""
    from mini_llm_amd import write_random_model
    from mini_llm_amd.kernels import ops
    d = write_random_model(LONG, str(tmp_path / "long"), seed=11)
    cfg, w = plain_gpt2.read_model(d)
    reqs = ru.random_requests(LONG["vocab_size"], [4732, 40, 70], seed=21)
    long_, short, first = reqs["r0"], reqs["r1"], reqs["r2"]
    steps = [{"step": 0, "entries": [{"id": "first", "tokens": first, "want": [len(first) - 1]}], "end": ["first"]},
             {"step": 1, "entries": [{"id": "long", "tokens": long_[:4700], "want": [0, 1, 2047, 4095, 4096, 4699]},
                                     {"id": "short", "tokens": short[:8], "want": [7]}], "end": []}]
    for i in range(32):
        steps.append({"step": 2 + i, "entries": [{"id": "short", "tokens": [short[8 + i]], "want": [0]},
                                                  {"id": "long", "tokens": [long_[4700 + i]], "want": [0]}],
                      "end": ["long", "short"] if i == 31 else []})
    n_pages = ru.peak_tokens(steps) // 16
    from mini_llm_amd import Runner
    runner = Runner(model_dir=d, dtype=dtype, page_size=16, n_pages=n_pages, max_num_seqs=4)
    runner.poison_cache()
    ops.reset_seen()
    out = ru.run_in_process(runner, steps)
    assert ops.seen("max_decode_splits") >= 8 and ops.seen("merge_kernel_launches") >= 32 * LONG["n_layer"]
    got = ru.collect(steps, out, LONG["vocab_size"])
    # about three times the worst seen (float32: max 2.6e-7 of a row, mean 4e-8; bfloat16: 2.2e-3 and 4e-4; the
    # logits' own standard deviation is about 0.2)
    tol = dict(max_abs=1e-6, mean_abs=1.5e-7) if dtype == "float32" else dict(max_abs=7e-3, mean_abs=1.5e-3)
    worst = worst_mean = 0.0
    for rid, toks in (("long", long_), ("short", short), ("first", first)):
        ref = plain_gpt2.forward_logits(cfg, w, list(toks)).numpy()
        assert got[rid], rid
        for pos, row in got[rid].items():
            assert np.isfinite(row).all(), (rid, pos)
            diff = np.abs(row.astype(np.float64) - ref[pos])
            worst, worst_mean = max(worst, diff.max()), max(worst_mean, diff.mean())
            assert diff.max() <= tol["max_abs"] and diff.mean() <= tol["mean_abs"], (rid, pos, diff.max(), diff.mean())
    print(f"worst difference from plain at 4,732 tokens [{dtype}]: max {worst:.3e}, mean {worst_mean:.3e} "
          f"(allowed {tol['max_abs']:.1e}, {tol['mean_abs']:.1e})")
    _all_pages_back(runner, n_pages)
