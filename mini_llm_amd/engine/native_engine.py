"""The native engine (csrc/engine/engine.cc) seen from Python: a thin face over its C ABI.

Everything between a request's tokens and its next token happens natively here: loader, cache
manager, scheduler, step function, kernels, sampler. It serves the architectures that are registered
natively; a model with parts written in Python runs through ``Engine`` (engine.py), which composes
the same native parts and ops from Python.
"""
from __future__ import annotations

import ctypes
import json
import os
from typing import Dict, List, Optional, Sequence, Union

import numpy as np

from ..kernels import ops
from ..sampling.sampler import SamplingParams
from .engine import EngineOptions, RequestOutput

_typed = False
_STATS = ("steps", "scheduled_tokens", "prefill_tokens", "decode_tokens", "deferred_decodes", "deferred_prefills",
          "preemptions", "failures", "finished", "peak_pages_used", "free_pages", "total_pages")
_DTYPES = {"bfloat16": 1, "bf16": 1, "float32": 0, "fp32": 0}


def _lib():
    global _typed
    lib = ops.engine_library()
    if not _typed:
        vp, i, ll, ull = ctypes.c_void_p, ctypes.c_int, ctypes.c_longlong, ctypes.c_ulonglong
        sigs = {
            "mllm_engine_from_pretrained": (vp, [ctypes.c_char_p, i, vp]),
            "mllm_engine_from_random": (vp, [ctypes.c_char_p, ull, i, vp]),
            "mllm_engine_destroy": (None, [vp]),
            "mllm_engine_add_request": (ll, [vp, vp, i, ctypes.c_float, ull, i, i, ll]),
            "mllm_engine_has_unfinished": (i, [vp]),
            "mllm_engine_step": (i, [vp, vp, vp, vp, i]),
            "mllm_engine_abort": (i, [vp, ll]),
            "mllm_engine_stats": (None, [vp, vp]),
            "mllm_engine_vocab_size": (i, [vp]),
            "mllm_engine_cache_bytes_per_token": (ull, [vp]),
            "mllm_engine_synchronize": (None, [vp]),
        }
        for name, (res, args) in sigs.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _typed = True
    return lib


def _error(lib) -> str:
    return lib.mllm_last_error().decode("utf-8", "replace")


class NativeEngine:
    def __init__(self, handle: int, options: EngineOptions):
        self._lib = _lib()
        self._h = handle
        self.options = options
        cap = max(options.max_batch_num, 1) * 2 + 16
        self._ids = np.empty(cap, dtype=np.int64)
        self._toks = np.empty(cap, dtype=np.int32)
        self._fin = np.empty(cap, dtype=np.int32)

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.mllm_engine_destroy(h)

    @staticmethod
    def _options(options: Optional[EngineOptions], kw) -> EngineOptions:
        if kw:
            options = EngineOptions(**{**(options.__dict__ if options else {}), **kw})
        return options or EngineOptions()

    @staticmethod
    def _pack(o: EngineOptions):
        return (ctypes.c_int * 7)(o.kv_block_size, o.total_kv_blocks, o.max_batch_num, o.max_tokens_per_step,
                                  o.prefill_chunk, 1 if o.overlap_decode else 0, int(round(o.kv_memory_fraction * 1e6)))

    @classmethod
    def from_pretrained(cls, model_dir: str, dtype="bfloat16", options: Optional[EngineOptions] = None, **kw):
        lib, o = _lib(), cls._options(options, kw)
        h = lib.mllm_engine_from_pretrained(os.fsencode(model_dir), _DTYPES[dtype], cls._pack(o))
        if not h:
            raise RuntimeError(_error(lib))
        return cls(h, o)

    @classmethod
    def from_random(cls, preset: Union[str, dict], seed: int = 0, dtype="bfloat16",
                    options: Optional[EngineOptions] = None, **kw):
        """``preset``: a size under config/presets, or a config.json dictionary. The weights are made by the
        specified generator in memory (the values a written folder would hold)."""
        if isinstance(preset, str):
            d = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "config", "presets")
            path = os.path.join(d, preset + ".json")
            if not os.path.isfile(path):
                raise ValueError(f"unknown preset '{preset}'")
            with open(path) as f:
                preset = json.load(f)
        lib, o = _lib(), cls._options(options, kw)
        h = lib.mllm_engine_from_random(json.dumps(preset).encode(), int(seed), _DTYPES[dtype], cls._pack(o))
        if not h:
            raise RuntimeError(_error(lib))
        return cls(h, o)

    def add_request(self, prompt_ids: Sequence[int], params: Optional[SamplingParams] = None,
                    request_id: Optional[int] = None) -> int:
        p = params or SamplingParams()
        toks = np.asarray(list(prompt_ids), dtype=np.int32)
        rid = self._lib.mllm_engine_add_request(self._h, toks.ctypes.data, len(toks), p.temperature, p.seed,
                                                p.max_new_tokens, 1 if p.ignore_eos else 0,
                                                -1 if request_id is None else int(request_id))
        if rid < 0:
            raise ValueError(_error(self._lib))
        return rid

    def has_unfinished(self) -> bool:
        return bool(self._lib.mllm_engine_has_unfinished(self._h))

    def step(self) -> List[RequestOutput]:
        n = self._lib.mllm_engine_step(self._h, self._ids.ctypes.data, self._toks.ctypes.data, self._fin.ctypes.data,
                                       len(self._ids))
        if n < 0:
            raise RuntimeError(_error(self._lib))
        return [RequestOutput(int(self._ids[k]), int(self._toks[k]), bool(self._fin[k]),
                              _error(self._lib) if self._toks[k] < 0 else None) for k in range(n)]

    def abort(self, request_id: int) -> None:
        if self._lib.mllm_engine_abort(self._h, request_id) != 0:
            raise KeyError(_error(self._lib))

    def generate(self, prompts: Sequence[Sequence[int]],
                 params: Union[None, SamplingParams, Sequence[SamplingParams]] = None) -> List[List[int]]:
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        rids = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        got: Dict[int, List[int]] = {rid: [] for rid in rids}
        while self.has_unfinished():
            for o in self.step():
                if o.request_id in got:
                    if o.token < 0:
                        raise RuntimeError(f"request {o.request_id} failed: {o.error}")
                    got[o.request_id].append(o.token)
        return [got[rid] for rid in rids]

    def stats(self) -> Dict[str, int]:
        buf = np.zeros(12, dtype=np.int64)
        self._lib.mllm_engine_stats(self._h, buf.ctypes.data)
        return dict(zip(_STATS, (int(v) for v in buf)))

    def cache_bytes_per_token(self) -> int:
        return int(self._lib.mllm_engine_cache_bytes_per_token(self._h))

    def synchronize(self) -> None:
        self._lib.mllm_engine_synchronize(self._h)
