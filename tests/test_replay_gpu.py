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
from conftest import CONFIGS, TINY

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


def _runner(model_dir, name, dtype, n_pages, page=None):
    from mini_llm_amd.engine.step import ModelRunner
    from mini_llm_amd.models import load_model
    model = load_model(model_dir, dtype, "cuda:0")
    runner = ModelRunner(model, page or CONFIGS[name][2], n_pages, 8)
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
    rc.check_against_plain(tiny_model_dirs[name], name, reqs, steps, out, dtype, label=family)
    assert runner.manager.check() == ""
    assert runner.manager.free_pages(0) == n_pages and runner.manager.n_requests() == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["small2", "xl2"])
@pytest.mark.parametrize("family", ["whole", "decode_tail", "chunks", "mixed"])
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
    assert runner.manager.check() == ""
    assert runner.manager.free_pages(0) == n_pages and runner.manager.n_requests() == 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_native_step_equals_the_parts_python_forward(tiny_model_dirs, dtype):
    """A model whose parts are all native runs its step in one native call; with `use_native` off the
    parts' Python forward methods run instead. Same kernels, same arguments: the logits are equal
    bit for bit, and both match the plain implementation."""
    reqs = rc.requests_for("b", seed=3, lengths=[40, 9, 100, 70])
    steps, _ = ru.trace_mixed(reqs, seed=3)
    outs = []
    for native in (True, False):
        runner = _runner(tiny_model_dirs["b"], "b", dtype, ru.peak_tokens(steps) // 8)
        runner.model.use_native = native
        assert (runner.model.native() is not None)
        outs.append(ru.run_in_process(runner, steps))
    assert outs[0].keys() == outs[1].keys()
    for k in outs[0]:
        assert np.array_equal(outs[0][k], outs[1][k]), k
    rc.check_against_plain(tiny_model_dirs["b"], "b", reqs, steps, outs[0], dtype, label="native")


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
