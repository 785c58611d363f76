"""The step function, seen from Python: a face over the native runner (csrc/engine/engine.cc,
``ModelRunner``), which owns a model's caches and runs steps on a stream of its own.

One step is any mixture of (request, its next tokens): portions of prompts beside single decoded tokens,
cut anywhere. It runs only the tokens it is given, from the cache that earlier steps left, and returns
the fp32 logits at the wanted places. The runner takes pages and commits lengths itself here; under the
engine the scheduler does.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Union

import numpy as np

from .. import native
from ..config import as_config


@dataclass
class StepEntry:
    request_id: int
    tokens: Sequence[int]               # the request's next tokens (a list, or an int32 array: no conversion then)
    want: Sequence[int] = field(default_factory=list)     # indices into ``tokens`` whose logits are wanted


class Runner:
    """``Runner(model_dir=...)`` or ``Runner(config=..., seed=...)`` (random weights, the values a written
    folder holds) owns its model; ``Engine.runner`` is the engine's own."""

    def __init__(self, model_dir: Optional[str] = None, config: Union[None, str, dict] = None, seed: int = 0,
                 dtype: str = "bfloat16", page_size: int = 16, n_pages: int = 256, max_num_seqs: int = 16,
                 _borrowed: Optional[int] = None, _owner=None):
        self._lib = native.lib()
        self._box = None
        self._owner = _owner            # keeps the engine alive while its runner is in use
        if _borrowed is not None:
            self._h = _borrowed
        else:
            if (model_dir is None) == (config is None):
                raise ValueError("give either model_dir or config")
            text = b"" if config is None else json.dumps(as_config(config)).encode()
            self._box = self._lib.mllm_runner_create(os.fsencode(model_dir) if model_dir else b"", text, int(seed),
                                                     native.dtype_code(dtype), int(page_size), int(n_pages),
                                                     int(max_num_seqs))
            if not self._box:
                raise native.EngineError(native.last_error())
            self._h = self._lib.mllm_runner_of_box(self._box)
        self._info = self.info()
        self.vocab_size = self._info["vocab_size"]

    def __del__(self):
        box, self._box = getattr(self, "_box", None), None
        if box:
            self._lib.mllm_runner_destroy(box)

    def step(self, entries: Sequence[StepEntry]) -> Optional[np.ndarray]:
        """Runs one batch; returns float32 logits [wanted, vocab] in the order of the entries and of each
        entry's ``want``, or None if nothing is wanted."""
        ids = np.asarray([e.request_id for e in entries], dtype=np.int64)
        n_tok = np.asarray([len(e.tokens) for e in entries], dtype=np.int32)
        toks = np.concatenate([np.asarray(e.tokens, dtype=np.int32).reshape(-1) for e in entries]) if entries \
            else np.empty(0, dtype=np.int32)
        n_want = np.asarray([len(e.want) for e in entries], dtype=np.int32)
        want = np.asarray([w for e in entries for w in e.want], dtype=np.int32)
        rows = int(n_want.sum())
        out = np.empty((max(rows, 1), self.vocab_size), dtype=np.float32)
        n = self._lib.mllm_runner_step(self._h, ids.ctypes.data, n_tok.ctypes.data, toks.ctypes.data, n_want.ctypes.data,
                                       want.ctypes.data, len(entries), out.ctypes.data, rows)
        if n < 0:
            raise native.EngineError(native.last_error())
        return out[:n] if n > 0 else None

    def end_request(self, request_id: int) -> None:
        native.check(self._lib.mllm_runner_end_request(self._h, int(request_id)))

    def poison_cache(self) -> None:
        """Fills every page and state slot with NaN: a stale or unwritten one that is read shows (tests)."""
        native.check(self._lib.mllm_runner_poison(self._h))

    def check(self) -> str:
        """Empty when no page or slot is lost, held twice, or both held and free."""
        return native.text_of(lambda buf, cap: self._lib.mllm_runner_check(self._h, buf, cap))

    def info(self) -> Dict:
        """Sizes (architecture, vocab_size, hidden_size, max_positions, n_layers, n_caches, n_groups, page_size,
        n_pages, free_pages, n_requests, cache_bytes_per_token) and what a step costs through the model's parts
        (weight_bytes, flops_per_token, attention_flops_per_key, flops_per_logits_row)."""
        return json.loads(native.text_of(lambda buf, cap: self._lib.mllm_runner_info(self._h, buf, cap)))

    def synchronize(self) -> None:
        self._lib.mllm_runner_synchronize(self._h)
