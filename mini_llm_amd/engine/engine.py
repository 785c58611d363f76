"""The engine, seen from Python: requests in, tokens out. A face over the native engine
(csrc/engine/engine.cc), the one behind ``bin/mini-llm``: scheduler above, step function below.

    engine = Engine.from_pretrained(model_dir, dtype="bfloat16")
    new_tokens = engine.generate([[15496, 11, 616]], SamplingParams(max_new_tokens=8))

The reference's loop: /root/reference/src/runtime/scheduler.cpp:322-356; its offline use of the model:
/root/reference/benchmarks/gpt2/bench_batch_vs_single_wall.cu:157-171.
"""
from __future__ import annotations

import ctypes
import json
import os
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Union

import numpy as np

from .. import native
from ..config import as_config
from .runner import Runner, StepEntry

_STATS = ("steps", "scheduled_tokens", "prefill_tokens", "decode_tokens", "deferred_decodes", "deferred_prefills",
          "preemptions", "failures", "finished", "peak_pages_used", "free_pages", "total_pages", "aborted")


@dataclass
class EngineOptions:
    kv_block_size: int = 16             # tokens per page (reference: DEFAULT_KV_BLOCK_SIZE, constants.h:16)
    total_kv_blocks: int = 4096         # pages in the pool (reference: DEFAULT_TOTAL_KV_BLOCKS, constants.h:17)
    kv_memory_fraction: float = 0.0     # > 0: the pool takes this share of the device memory that is free once the
                                        # weights and the largest step's buffers are there, whatever total_kv_blocks says
    max_batch_num: int = 16             # sequences in one step (reference: MAX_BATCH_NUM, constants.h:20)
    max_tokens_per_step: int = 2048     # token budget of one step
    prefill_chunk: int = 512            # longest prompt portion
    overlap_decode: bool = True         # launch a step before the previous one's tokens are read
    preempt_for_decode: bool = True     # a decode that gets no page preempts a younger request at once; False: it
                                        # waits on its pages until somebody finishes (the reference's manner)


@dataclass
class SamplingParams:
    temperature: float = 0.0            # 0: greedy (lowest index on ties: /root/reference/src/kernels/argmax.cu:12-20)
    seed: int = 0                       # the draw for output i of a request depends on (seed, i) only
    max_new_tokens: int = 8             # the reference's default (/root/reference/include/constants.h:14)
    ignore_eos: bool = False

    def __post_init__(self):
        if self.temperature < 0:
            raise ValueError("temperature must be >= 0")
        if self.max_new_tokens < 1:
            raise ValueError("max_new_tokens must be >= 1")


@dataclass
class RequestOutput:
    request_id: int
    token: int                          # -1: no token (the request failed)
    finished: bool
    error: Optional[str] = None         # why a request failed


class Engine:
    def __init__(self, handle: int, options: EngineOptions):
        self._lib = native.lib()
        self._h = handle
        self.options = options
        cap = max(options.max_batch_num, 1) * 2 + 16
        self._ids = np.empty(cap, dtype=np.int64)
        self._toks = np.empty(cap, dtype=np.int32)
        self._fin = np.empty(cap, dtype=np.int32)
        self.runner = Runner(_borrowed=self._lib.mllm_engine_runner(handle), _owner=self)

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.mllm_engine_destroy(h)

    def close(self) -> None:
        """Frees the model, the caches and the stream now (otherwise: when the object is collected)."""
        self.runner = None
        self.__del__()

    @staticmethod
    def _options(options: Optional[EngineOptions], kw) -> EngineOptions:
        if kw:
            options = EngineOptions(**{**(options.__dict__ if options else {}), **kw})
        return options or EngineOptions()

    @staticmethod
    def _pack(o: EngineOptions):
        return (ctypes.c_int * 8)(o.kv_block_size, o.total_kv_blocks, o.max_batch_num, o.max_tokens_per_step,
                                  o.prefill_chunk, 1 if o.overlap_decode else 0, int(round(o.kv_memory_fraction * 1e6)),
                                  1 if o.preempt_for_decode else 0)

    @classmethod
    def from_pretrained(cls, model_dir: str, dtype: str = "bfloat16", options: Optional[EngineOptions] = None, **kw):
        lb, o = native.lib(), cls._options(options, kw)
        h = lb.mllm_engine_from_pretrained(os.fsencode(model_dir), native.dtype_code(dtype), cls._pack(o))
        if not h:
            raise native.EngineError(native.last_error())
        return cls(h, o)

    @classmethod
    def from_random(cls, preset: Union[str, dict], seed: int = 0, dtype: str = "bfloat16",
                    options: Optional[EngineOptions] = None, **kw):
        """``preset``: a size under config/presets, or a config.json dictionary. The weights are made in memory
        by the specified generator and are the values a written folder holds (matrices rounded to bfloat16
        whatever ``dtype`` computes in): the same model as ``write_random_model`` + ``from_pretrained``."""
        lb, o = native.lib(), cls._options(options, kw)
        h = lb.mllm_engine_from_random(json.dumps(as_config(preset)).encode(), int(seed), native.dtype_code(dtype),
                                       cls._pack(o))
        if not h:
            raise native.EngineError(native.last_error())
        return cls(h, o)

    def add_request(self, prompt_ids: Sequence[int], params: Optional[SamplingParams] = None,
                    request_id: Optional[int] = None) -> int:
        p = params or SamplingParams()
        toks = np.asarray(list(prompt_ids), dtype=np.int32)
        rid = self._lib.mllm_engine_add_request(self._h, toks.ctypes.data, len(toks), p.temperature, p.seed,
                                                p.max_new_tokens, 1 if p.ignore_eos else 0,
                                                -1 if request_id is None else int(request_id))
        if rid < 0:
            raise ValueError(native.last_error())
        return rid

    def has_unfinished(self) -> bool:
        return bool(self._lib.mllm_engine_has_unfinished(self._h))

    def step(self) -> List[RequestOutput]:
        """One iteration of the engine. Outputs beyond the buffer's room arrive with the next calls."""
        n = self._lib.mllm_engine_step(self._h, self._ids.ctypes.data, self._toks.ctypes.data, self._fin.ctypes.data,
                                       len(self._ids))
        if n < 0:
            raise native.EngineError(native.last_error())
        return [RequestOutput(int(self._ids[k]), int(self._toks[k]), bool(self._fin[k]),
                              self._lib.mllm_engine_output_error(k).decode("utf-8", "replace") if self._toks[k] < 0 else None)
                for k in range(n)]

    def abort(self, request_id: int) -> None:
        if self._lib.mllm_engine_abort(self._h, request_id) != 0:
            raise KeyError(native.last_error())

    def generate(self, prompts: Sequence[Sequence[int]],
                 params: Union[None, SamplingParams, Sequence[SamplingParams]] = None) -> List[List[int]]:
        """Generates for every prompt (continuous batching) and returns the new tokens of each."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        rids = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        got: Dict[int, List[int]] = {rid: [] for rid in rids}
        failed: Dict[int, str] = {}
        while self.has_unfinished():
            for o in self.step():
                if o.request_id in got:
                    if o.token < 0:
                        failed[o.request_id] = o.error or "failed"
                    else:
                        got[o.request_id].append(o.token)
        if failed:
            rid, why = next(iter(failed.items()))
            raise native.EngineError(f"request {rid} failed: {why}")
        return [got[rid] for rid in rids]

    def step_logits(self, entries: Sequence[StepEntry]) -> Optional[np.ndarray]:
        """The step function itself, on the engine's runner (ids must differ from those of added requests)."""
        return self.runner.step(entries)

    def stats(self) -> Dict[str, int]:
        buf = np.zeros(len(_STATS), dtype=np.int64)
        native.check(self._lib.mllm_engine_stats(self._h, buf.ctypes.data))
        return dict(zip(_STATS, (int(v) for v in buf)))

    def synchronize(self) -> None:
        self._lib.mllm_engine_synchronize(self._h)
