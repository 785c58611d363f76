"""The engine on the GPU against the plain implementation, in 32-bit and in bfloat16:
each request alone and whole; most of it in one step and the last 32 tokens one by one;
portions of changing size down to two tokens; and mixed batches of up to four live requests
with so few pages that they are used again. In-process through ModelRunner, and through
bin/trace_run as a user drives it."""
import os

import numpy as np
import pytest
import torch

import replay_cases as rc
import replay_util as ru
from conftest import TINY

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


def _runner(model_dir, name, dtype, n_pages, page=None):
    from mini_llm_amd.engine.step import ModelRunner
    from mini_llm_amd.models import load_model
    model = load_model(model_dir, dtype, "cuda:0")
    runner = ModelRunner(model, page or TINY[name][2], n_pages, 8)
    runner.cache.poison()          # an unwritten or stale page that is read shows up as NaN
    return runner


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["a", "b"])
@pytest.mark.parametrize("family", ["whole", "decode_tail", "chunks", "mixed"])
def test_schedule_families_match_plain(tiny_model_dirs, name, family, dtype):
    reqs = rc.requests_for(name)
    steps = rc.families(reqs)[family]
    page = TINY[name][2]
    n_pages = ru.peak_tokens(steps) // page
    runner = _runner(tiny_model_dirs[name], name, dtype, n_pages)
    out = ru.run_in_process(runner, steps)
    rc.check_against_plain(tiny_model_dirs[name], name, reqs, steps, out, dtype)
    assert runner.manager.check() == ""
    assert runner.manager.free_pages(0) == n_pages and runner.manager.n_requests() == 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_schedules_agree_with_each_other(tiny_model_dirs, dtype):
    """Cutting, batching and page placement change the logits by rounding only."""
    reqs = rc.requests_for("b", seed=5, lengths=[25, 64, 124, 9])
    outs = {}
    for fam, steps in rc.families(reqs, seed=5).items():
        runner = _runner(tiny_model_dirs["b"], "b", dtype, 64)
        outs[fam] = ru.collect(steps, ru.run_in_process(runner, steps), 1000)
    tol = 2e-5 if dtype == "float32" else 4e-2
    for rid, toks in reqs.items():
        for pos in range(len(toks)):
            base = outs["whole"][rid][pos]
            for fam in ("decode_tail", "chunks", "mixed"):
                assert np.abs(outs[fam][rid][pos] - base).max() <= tol, (fam, rid, pos)


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


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["a", "b"])
def test_trace_run_program(tiny_model_dirs, tmp_path, name, dtype):
    """bin/trace_run with its default page size, pool made for exactly --max-tokens."""
    reqs = rc.requests_for(name, seed=2, lengths=rc.LENGTHS[name][:4] + [2, 64])
    steps, _ = ru.trace_mixed(reqs, seed=2)
    # a step in which nothing is wanted writes no file
    skip = set()
    for e in steps[0]["entries"]:
        e["want"] = []
        skip |= {(e["id"], p) for p in range(len(e["tokens"]))}
    out = ru.run_trace_run(tiny_model_dirs[name], dtype, steps, str(tmp_path / "out"), ru.peak_tokens(steps))
    assert 0 not in out
    rc.check_against_plain(tiny_model_dirs[name], name, reqs, steps, out, dtype, skip=skip)
