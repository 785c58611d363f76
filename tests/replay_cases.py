"""The replay comparisons of the GPU tests: request sets, the four schedule families, tolerances, and the
check of an engine's logits against the plain implementation's, position by position."""
from __future__ import annotations

from typing import Dict

import numpy as np
import torch

import plain_gpt2
import replay_util as ru
from conftest import CONFIGS

# request lengths: the tiny workloads' prompt lengths (5, 17, 33 and 1, 9, 40, 100) plus their generated tokens, and page-edge cases
LENGTHS = {"a": [5 + 16, 17 + 16, 33 + 16, 1, 3, 4, 5, 64, 128], "b": [1 + 24, 9 + 24, 40 + 24, 100 + 24, 7, 8, 9, 256]}

# at GPT-2 small / XL layer sizes: the reference's own page-edge lengths (5, 15, 16, 17 around its 16-token
# pages: /root/reference/scripts/dump_gpt2_batch_prefill_golden.py:49-54), then about 40, 130 and 300 tokens
LENGTHS.update({"small2": [5, 15, 16, 17, 41, 130, 300], "xl2": [5, 15, 16, 17, 41, 130, 300]})

# What the engine's logits may differ by from the plain implementation's (float64 on the same stored
# weights). fp32: rounding of 32-bit sums. bf16: activations rounded to bfloat16 between the kernels.
# The figures are about three times the worst difference seen over all four schedule families, per
# configuration (seen, max / mean of a row: a 4.4e-7 / 4.8e-8 and 1.5e-3 / 3.4e-4; b 4.4e-7 / 4.8e-8 and
# 2.2e-3 / 4.2e-4; small2 5.2e-6 / 6.8e-7 and 1.4e-2 / 2.3e-3; xl2 1.1e-5 / 1.5e-6 and 2.1e-2 / 3.3e-3;
# the logits' own spread: standard deviation 0.16 / 0.20 at the tiny sizes, about 0.55 at the real ones).
# Every comparison prints its worst, so a drift shows in the test report before it fails.
TOL = {
    ("a", "float32"): dict(max_abs=2e-6, mean_abs=2e-7), ("b", "float32"): dict(max_abs=2e-6, mean_abs=2.5e-7),
    ("small2", "float32"): dict(max_abs=2e-5, mean_abs=2.5e-6), ("xl2", "float32"): dict(max_abs=4e-5, mean_abs=5e-6),
    ("a", "bfloat16"): dict(max_abs=5e-3, mean_abs=1.1e-3), ("b", "bfloat16"): dict(max_abs=7e-3, mean_abs=1.3e-3),
    ("small2", "bfloat16"): dict(max_abs=4.5e-2, mean_abs=7e-3), ("xl2", "bfloat16"): dict(max_abs=6.5e-2, mean_abs=1e-2),
}
WORST: Dict[tuple, tuple] = {}       # (configuration, dtype, label) -> worst (max |diff|, mean |diff|) seen

_plain_cache: Dict[tuple, Dict[int, np.ndarray]] = {}
_weights_cache: Dict[str, tuple] = {}


def plain_logits(model_dir: str, name: str, toks, positions) -> Dict[int, np.ndarray]:
    """Rows of the plain implementation's logits for one whole sequence, at the given positions."""
    key = (name, tuple(toks))
    have = _plain_cache.setdefault(key, {})
    if any(p not in have for p in positions):
        if model_dir not in _weights_cache:
            _weights_cache.clear()                   # one model's float64 weights at a time
            _weights_cache[model_dir] = plain_gpt2.read_model(model_dir)
        cfg, w = _weights_cache[model_dir]
        full = plain_gpt2.forward_logits(cfg, w, list(toks)).numpy()
        for p in positions:
            have[p] = full[p].copy()
    return have


def requests_for(name: str, seed: int = 0, lengths=None):
    cfg = CONFIGS[name][0]
    return ru.random_requests(cfg["vocab_size"], lengths or LENGTHS[name], seed=100 + seed)


def thin(steps, page: int = 16, every: int = 7, tail: int = 33):
    """Keeps of every request's wanted places those at the first positions, around page edges, every
    ``every``-th one and the last ``tail`` (a vocabulary of 50,257 makes every row 200 KB). Returns the
    set of (request, position) that are no longer asked for."""
    total: Dict[str, int] = {}
    for s in steps:
        for e in s["entries"]:
            total[e["id"]] = total.get(e["id"], 0) + len(e["tokens"])
    fed: Dict[str, int] = {}
    dropped = set()
    for s in steps:
        for e in s["entries"]:
            base = fed.get(e["id"], 0)
            keep = []
            for w in e["want"]:
                p = base + w
                if p < 3 or p % every == 0 or p % page in (0, 1, page - 1) or p >= total[e["id"]] - tail:
                    keep.append(w)
                else:
                    dropped.add((e["id"], p))
            e["want"] = keep
            fed[e["id"]] = base + len(e["tokens"])
    return dropped


def check_against_plain(model_dir, name, reqs, steps, outputs, dtype: str, skip=(), label: str = ""):
    vocab = CONFIGS[name][0]["vocab_size"]
    got = ru.collect(steps, outputs, vocab)
    tol = TOL[(name, dtype)]
    worst = worst_mean = 0.0
    for rid, toks in reqs.items():
        wanted = [p for p in range(len(toks)) if (rid, p) not in skip]
        ref = plain_logits(model_dir, name, toks, wanted)
        assert sorted(got.get(rid, {})) == wanted, f"{rid}: positions missing or unasked"
        for pos in wanted:
            row = got[rid][pos].astype(np.float64)
            assert np.isfinite(row).all(), f"{rid} position {pos}: non-finite logits"
            d = np.abs(row - ref[pos])
            worst, worst_mean = max(worst, d.max()), max(worst_mean, d.mean())
            assert d.max() <= tol["max_abs"], (
                f"{rid} position {pos} (of {len(toks)}): max |diff| {d.max():.3e} > {tol['max_abs']:.1e}")
            assert d.mean() <= tol["mean_abs"], (
                f"{rid} position {pos} (of {len(toks)}): mean |diff| {d.mean():.3e} > {tol['mean_abs']:.1e}")
    key = (name, dtype, label)
    old = WORST.get(key, (0.0, 0.0))
    WORST[key] = (max(old[0], worst), max(old[1], worst_mean))
    print(f"worst difference from plain [{name} {dtype} {label}]: max {worst:.3e}, mean {worst_mean:.3e} "
          f"(allowed {tol['max_abs']:.1e}, {tol['mean_abs']:.1e})")
    return worst


def families(reqs, seed=0, large=False):
    """The four schedule families. ``large``: portions of up to 130 tokens among the small ones (steps of
    more than 64 and more than 256 rows run other kernels than short steps)."""
    if large:
        mixed, _ = ru.trace_mixed(reqs, seed=seed, sizes=(2, 3, 70, 9, 16, 2, 130))
        chunks = ru.trace_chunks(reqs, seed=seed, sizes=(2, 3, 65, 7, 16, 130, 2, 31, 4, 64))
    else:
        mixed, _ = ru.trace_mixed(reqs, seed=seed)
        chunks = ru.trace_chunks(reqs, seed=seed)
    return {
        "whole": ru.trace_whole(reqs),
        "decode_tail": ru.trace_decode_tail(reqs),
        "chunks": chunks,
        "mixed": mixed,
    }
