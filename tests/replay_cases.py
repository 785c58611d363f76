"""The replay comparisons shared by the CPU tests (engine over plain ops) and the GPU tests
(engine over the HIP kernels): every schedule family against the plain implementation."""
from __future__ import annotations

from typing import Dict

import numpy as np
import torch

import plain_gpt2
import replay_util as ru
from conftest import TINY

# request lengths: BASELINE's prompt lengths plus generated tokens, and page-edge cases
LENGTHS = {"a": [5 + 16, 17 + 16, 33 + 16, 1, 3, 4, 5, 64, 128], "b": [1 + 24, 9 + 24, 40 + 24, 100 + 24, 7, 8, 9, 256]}

# fp32: the engine against float64; bf16: bf16 activations against float64 on the same weights
TOL = {"float32": dict(max_abs=2e-5, mean_abs=2e-6), "bfloat16": dict(max_abs=4e-2, mean_abs=6e-3)}

_plain_cache: Dict[tuple, torch.Tensor] = {}


def plain_logits(model_dir: str, name: str, rid: str, toks) -> np.ndarray:
    key = (name, tuple(toks))
    if key not in _plain_cache:
        cfg, w = plain_gpt2.read_model(model_dir)
        _plain_cache[key] = plain_gpt2.forward_logits(cfg, w, list(toks)).numpy()
    return _plain_cache[key]


def requests_for(name: str, seed: int = 0, lengths=None):
    cfg = TINY[name][0]
    return ru.random_requests(cfg["vocab_size"], lengths or LENGTHS[name], seed=100 + seed)


def check_against_plain(model_dir, name, reqs, steps, outputs, dtype: str, skip=()):
    vocab = TINY[name][0]["vocab_size"]
    got = ru.collect(steps, outputs, vocab)
    tol = TOL[dtype]
    worst = 0.0
    for rid, toks in reqs.items():
        ref = plain_logits(model_dir, name, rid, toks)
        wanted = [p for p in range(len(toks)) if (rid, p) not in skip]
        assert sorted(got.get(rid, {})) == wanted, f"{rid}: positions missing or unasked"
        for pos in wanted:
            row = got[rid][pos].astype(np.float64)
            assert np.isfinite(row).all(), f"{rid} position {pos}: non-finite logits"
            d = np.abs(row - ref[pos])
            worst = max(worst, d.max())
            assert d.max() <= tol["max_abs"], (
                f"{rid} position {pos} (of {len(toks)}): max |diff| {d.max():.3e} > {tol['max_abs']:.1e}")
            assert d.mean() <= tol["mean_abs"], (
                f"{rid} position {pos} (of {len(toks)}): mean |diff| {d.mean():.3e} > {tol['mean_abs']:.1e}")
    return worst


def families(reqs, seed=0):
    mixed, _ = ru.trace_mixed(reqs, seed=seed)
    return {
        "whole": ru.trace_whole(reqs),
        "decode_tail": ru.trace_decode_tail(reqs),
        "chunks": ru.trace_chunks(reqs, seed=seed),
        "mixed": mixed,
    }
