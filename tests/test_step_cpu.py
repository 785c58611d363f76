"""The step function, the cache and the model assembly on the CPU: the engine runs over the
plain reference ops (tests/plain_ops.py) instead of the HIP kernels, and every schedule
family must reproduce the plain implementation's logits."""
import numpy as np
import pytest
import torch

import plain_ops
import replay_cases as rc
import replay_util as ru
from conftest import TINY


@pytest.fixture()
def cpu_ops(monkeypatch):
    plain_ops.install(monkeypatch)


def _runner(model_dir, name, n_pages):
    from mini_llm_amd.engine.step import ModelRunner
    from mini_llm_amd.models import load_model
    model = load_model(model_dir, "float32", "cpu")
    runner = ModelRunner(model, TINY[name][2], n_pages, 8)
    runner.cache.poison()
    return runner


@pytest.mark.parametrize("name", ["a", "b"])
@pytest.mark.parametrize("family", ["whole", "decode_tail", "chunks", "mixed"])
def test_schedule_families_match_plain(cpu_ops, tiny_model_dirs, name, family):
    lengths = rc.LENGTHS[name][:5] + [rc.LENGTHS[name][-1]]
    reqs = rc.requests_for(name, lengths=lengths)
    steps = rc.families(reqs)[family]
    page = TINY[name][2]
    n_pages = ru.peak_tokens(steps) // page          # exactly what the trace needs: pages are reused
    runner = _runner(tiny_model_dirs[name], name, n_pages)
    out = ru.run_in_process(runner, steps)
    rc.check_against_plain(tiny_model_dirs[name], name, reqs, steps, out, "float32")
    assert runner.manager.check() == ""
    assert runner.manager.free_pages(0) == n_pages and runner.manager.n_requests() == 0


def test_schedules_agree_bitwise_on_cpu(cpu_ops, tiny_model_dirs):
    """With row-independent reference ops, cutting and batching change nothing at all."""
    reqs = rc.requests_for("a", lengths=[21, 33, 49, 4])
    fams = rc.families(reqs, seed=3)
    outs = {}
    for fam, steps in fams.items():
        runner = _runner(tiny_model_dirs["a"], "a", 64)
        outs[fam] = ru.collect(steps, ru.run_in_process(runner, steps), 512)
    for rid, toks in reqs.items():
        for pos in range(len(toks)):
            base = outs["whole"][rid][pos]
            for fam in ("decode_tail", "chunks", "mixed"):
                assert np.array_equal(outs[fam][rid][pos], base), (fam, rid, pos)


def test_step_errors(cpu_ops, tiny_model_dirs):
    from mini_llm_amd.cache.manager import OutOfPages
    from mini_llm_amd.engine.step import StepEntry, StepError
    runner = _runner(tiny_model_dirs["a"], "a", 4)          # 16 tokens of cache
    with pytest.raises(StepError, match="token ids"):
        runner.step([StepEntry(1, [0, 512], [])])
    with pytest.raises(StepError, match="twice"):
        runner.step([StepEntry(2, [1], []), StepEntry(2, [2], [])])
    with pytest.raises(StepError, match="wanted index"):
        runner.step([StepEntry(3, [1, 2], [2])])
    with pytest.raises(OutOfPages):
        runner.step([StepEntry(4, list(range(17)), [])])
    assert runner.manager.check() == ""
    for rid in (1, 2, 3):
        if runner.manager.has_request(rid):
            runner.end_request(rid)
    assert runner.manager.free_pages(0) == 4 and runner.manager.n_requests() == 0
    # no logits wanted: nothing is returned, the cache still advances
    assert runner.step([StepEntry(5, [1, 2, 3], [])]) is None
    assert runner.manager.length(5) == 3
    runner2 = _runner(tiny_model_dirs["a"], "a", 64)
    with pytest.raises(StepError, match="positions"):
        runner2.step([StepEntry(1, [1] * 129, [])])
