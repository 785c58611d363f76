"""The engine: requests in, tokens out. Scheduler above, step function below.

One iteration: the scheduler plans a mixed batch (decoded tokens first, then prompt
portions under the token budget), the model runner runs it, the sampler chooses a token
for every request whose newest token was in the batch, finished requests give their
pages back. The reference's loop: /root/reference/src/runtime/scheduler.cpp:322-356;
its offline use of the model: /root/reference/benchmarks/gpt2/bench_batch_vs_single_wall.cu:157-171.

Steps run one ahead of the host: a step is launched with the decoded tokens among its
inputs taken on the device from the step before, and only then are that earlier step's
tokens read. The GPU so never waits for the host between steps. What the host learns
late is only whether a token was the end of sequence; such a request has then run one step
too many, whose token is dropped.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Union

import torch

from ..models import load_model
from ..sampling.sampler import SamplingParams, uniform01
from .scheduler import Scheduler
from .step import ModelRunner, StepEntry


@dataclass
class EngineOptions:
    kv_block_size: int = 16             # tokens per page (reference: DEFAULT_KV_BLOCK_SIZE, constants.h:16)
    total_kv_blocks: int = 4096         # pages in the pool (reference: DEFAULT_TOTAL_KV_BLOCKS, constants.h:17)
    kv_memory_fraction: float = 0.0     # > 0: the pool takes this share of the device memory that is free once the
                                        # weights are loaded, whatever total_kv_blocks says
    max_batch_num: int = 16             # sequences in one step (reference: MAX_BATCH_NUM, constants.h:20)
    max_tokens_per_step: int = 2048     # token budget of one step
    prefill_chunk: int = 512            # longest prompt portion
    overlap_decode: bool = True         # launch a step before the previous one's tokens are read


@dataclass
class RequestOutput:
    request_id: int
    token: int                          # -1: no token (the request failed)
    finished: bool
    error: Optional[str] = None         # why a request failed


# A request's record leaves the engine (and the scheduler) with its final output: what a caller
# wants to keep of it has arrived in the outputs by then, and its id may be used again.


@dataclass
class _Request:
    request_id: int
    tokens: List[int]
    prompt_len: int
    params: SamplingParams
    finished: bool = False
    failed: Optional[str] = None
    n_launched: int = 0                 # output tokens whose sampling has been launched
    ended_early: bool = False           # an end-of-sequence token was read after later steps were planned

    @property
    def output(self) -> List[int]:
        return self.tokens[self.prompt_len:]


def pages_for_memory_fraction(model, page_size: int, fraction: float) -> int:
    """Pages that ``fraction`` of the device memory free now holds, for the caches this model asks for."""
    from ..cache.manager import KVCacheSpec
    if fraction > 1:
        raise ValueError("kv_memory_fraction must be at most 1")
    esize = torch.empty((), dtype=model.dtype).element_size()
    per_token = sum(2 * s.n_kv_heads * s.head_dim * esize for s in model.cache_specs() if isinstance(s, KVCacheSpec))
    if per_token == 0:
        return 1
    free_bytes, _ = torch.cuda.mem_get_info(model.device)
    pages = int(fraction * free_bytes / (per_token * page_size))
    if pages < 1:
        raise ValueError("kv_memory_fraction leaves no room for a single page")
    return min(pages, (2 ** 31 - 1) // page_size)          # rows of a pool are indexed with 32 bits


class Engine:
    def __init__(self, model, options: Optional[EngineOptions] = None):
        self.model = model
        self.options = options or EngineOptions()
        o = self.options
        n_pages = o.total_kv_blocks
        if o.kv_memory_fraction > 0:
            n_pages = pages_for_memory_fraction(model, o.kv_block_size, o.kv_memory_fraction)
        self.runner = ModelRunner(model, o.kv_block_size, n_pages, o.max_batch_num)
        self.scheduler = Scheduler(self.runner.manager, o.max_batch_num, o.max_tokens_per_step,
                                   o.prefill_chunk, model.max_positions)
        self.eos_token_id = model.config.eos_token_id
        self.requests: Dict[int, _Request] = {}     # live requests only
        self._next_id = 0
        self._pending = None            # (PendingTokens, [(request, finished by that token)]) of the step in flight

    @classmethod
    def from_pretrained(cls, model_dir: str, dtype="bfloat16", device="cuda:0",
                        options: Optional[EngineOptions] = None, **kw) -> "Engine":
        if kw:
            options = EngineOptions(**{**(options.__dict__ if options else {}), **kw})
        return cls(load_model(model_dir, dtype, device), options)

    @classmethod
    def from_random(cls, preset: Union[str, dict], seed: int = 0, dtype="bfloat16", device="cuda:0",
                    options: Optional[EngineOptions] = None, **kw) -> "Engine":
        """An engine over random weights: ``preset`` names a size under config/presets (or is a
        config.json dictionary); the model folder is written to a temporary place and loaded as
        any other."""
        import json
        import os
        import tempfile
        from ..weights.random_init import write_random_model
        if isinstance(preset, str):
            d = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "config", "presets")
            path = os.path.join(d, preset + ".json")
            if not os.path.isfile(path):
                names = sorted(f[:-5] for f in os.listdir(d) if f.endswith(".json"))
                raise ValueError(f"unknown preset '{preset}'; known: {names}")
            with open(path) as f:
                preset = json.load(f)
        with tempfile.TemporaryDirectory() as tmp:
            write_random_model(dict(preset), tmp, seed, "float32" if dtype == "float32" else "bfloat16")
            return cls.from_pretrained(tmp, dtype=dtype, device=device, options=options, **kw)

    def step_logits(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """The step function itself, for callers that bring their own tokens (tests, replay):
        runs the entries through the model and the cache and returns fp32 logits at the wanted
        places. Requests stepped this way are not known to the scheduler."""
        return self.runner.step(entries, manage_cache=True)

    # -- requests ------------------------------------------------------------------------
    def add_request(self, prompt_ids: Sequence[int], params: Optional[SamplingParams] = None,
                    request_id: Optional[int] = None) -> int:
        params = params or SamplingParams()
        ids = [int(t) for t in prompt_ids]
        if any(t < 0 or t >= self.model.vocab_size for t in ids):
            raise ValueError(f"token ids must lie in [0, {self.model.vocab_size})")
        rid = self._next_id if request_id is None else int(request_id)
        self._next_id = max(self._next_id, rid) + 1
        self.scheduler.add_request(rid, len(ids), params.max_new_tokens)
        self.requests[rid] = _Request(rid, ids, len(ids), params)
        return rid

    def abort(self, request_id: int) -> List[int]:
        """Ends a live request now; a token of it that is still in flight is dropped. Returns the
        tokens it has generated so far."""
        r = self.requests[request_id]
        self.scheduler.abort(request_id)
        r.finished, r.failed = True, "aborted"
        self._drop(r)
        return r.output

    def _drop(self, r: _Request) -> None:
        """Forgets a request whose final output is on its way to the caller."""
        if self.requests.get(r.request_id) is r:
            del self.requests[r.request_id]
            self.scheduler.forget(r.request_id)

    def has_unfinished(self) -> bool:
        return self.scheduler.has_work() or self._pending is not None

    # -- one iteration -------------------------------------------------------------------
    def _is_eos(self, r: _Request, tok: int) -> bool:
        return (not r.params.ignore_eos) and self.eos_token_id is not None and tok == self.eos_token_id

    def _collect(self) -> List[RequestOutput]:
        """Reads the tokens of the step in flight, if any. A request that an earlier token
        already ended (seen late) or that was aborted drops its token."""
        if self._pending is None:
            return []
        (handle, rows), self._pending = self._pending, None
        outputs = []
        for (r, done), tok in zip(rows, handle.result()):
            if r.finished or self.requests.get(r.request_id) is not r:
                continue                      # ended by an earlier token, or aborted
            rid = r.request_id
            r.tokens.append(tok)
            if not done and self._is_eos(r, tok):
                # the scheduler has planned on without knowing: take the request out now
                self.scheduler.stop(rid)
                r.ended_early = done = True
            r.finished = done
            outputs.append(RequestOutput(rid, tok, done))
            if done:
                self._drop(r)
        return outputs

    def step(self) -> List[RequestOutput]:
        plan = self.scheduler.schedule()
        outputs: List[RequestOutput] = []
        for rid, kind in self.scheduler.pop_events():
            if kind == "failed":
                r = self.requests.get(rid)
                if r is None:                  # aborted by the caller, who knows
                    continue
                r.finished, r.failed = True, "the page pool cannot hold this request"
                outputs.append(RequestOutput(rid, -1, True, r.failed))
                self._drop(r)
        if not plan:
            return outputs + self._collect()
        sampled = [e for e in plan if e.want_last]
        fast = (self.runner.fast_decode and len(sampled) == len(plan) and all(e.n_tokens == 1 for e in plan))
        # only a single decoded token can be fed on the device; a portion that reaches past what the
        # host has read (a request recomputed right after it was preempted) waits for the read
        unread_portion = any(e.n_tokens > 1 and e.start + e.n_tokens > len(self.requests[e.request_id].tokens)
                             for e in plan)
        if not self.options.overlap_decode or unread_portion:
            # the host knows every token it feeds: read what is in flight first
            outputs += self._collect()
            live = [e for e in plan if e.request_id in self.requests]
            if len(live) != len(plan):        # ended by a token just read; the scheduler dropped them too
                plan, sampled = live, [e for e in live if e.want_last]
                if not plan:
                    return outputs
        temps, us = [], []
        for e in sampled:
            r = self.requests[e.request_id]
            temps.append(r.params.temperature)
            us.append(uniform01(r.params.seed, r.n_launched) if r.params.temperature > 0 else 0.0)
            r.n_launched += 1
        # A token that the step in flight has sampled and the host has not read is fed on the device:
        # its row among that step's sampled tokens stands in for it.
        in_flight = {r.request_id: i for i, (r, _) in enumerate(self._pending[1])} if self._pending else {}
        if fast:
            # every entry is one decoded token: the whole step runs from static buffers (a HIP graph)
            toks, src = [], []
            for e in plan:
                r = self.requests[e.request_id]
                if e.start < len(r.tokens):
                    toks.append(r.tokens[e.start])
                    src.append(-1)
                else:
                    toks.append(0)
                    src.append(in_flight[e.request_id])
            handle = self.runner.launch_decode([e.request_id for e in plan], toks, src, temps, us)
        else:
            entries, feed = [], []
            for e in plan:
                r = self.requests[e.request_id]
                known = r.tokens[e.start:e.start + e.n_tokens]
                if len(known) < e.n_tokens:        # a decoded token still in flight
                    known, row = [0], in_flight[e.request_id]
                else:
                    row = -1
                entries.append(StepEntry(e.request_id, known, [e.n_tokens - 1] if e.want_last else []))
                feed.append(row)
            handle = self.runner.launch_step(entries, feed, temps, us)
        self.scheduler.commit()
        # the scheduler moves on as if no token were the end of sequence; `_collect` corrects it
        rows = [(self.requests[e.request_id], self.scheduler.on_token(e.request_id, False)) for e in sampled]
        outputs += self._collect()
        self._pending = (handle, rows) if handle is not None else None
        if not self.options.overlap_decode:
            outputs += self._collect()
        return outputs

    # -- offline generation --------------------------------------------------------------
    def generate(self, prompts: Sequence[Sequence[int]],
                 params: Union[None, SamplingParams, Sequence[SamplingParams]] = None) -> List[List[int]]:
        """Generates for every prompt (continuous batching) and returns the new tokens of each."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        rids = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        got: Dict[int, List[int]] = {rid: [] for rid in rids}
        errors: Dict[int, str] = {}
        while self.has_unfinished():
            for o in self.step():
                if o.request_id not in got:
                    continue                  # a request the caller added beside these
                if o.token < 0:
                    errors[o.request_id] = o.error or "failed"
                else:
                    got[o.request_id].append(o.token)
        for rid in rids:
            if rid in errors:
                raise RuntimeError(f"request {rid} failed: {errors[rid]}")
        return [got[rid] for rid in rids]

    def warmup(self, sampling: bool = False) -> List[int]:
        """Captures the decode graphs before the first real request needs them: for every batch size
        that decode steps are captured at (1 to 8, then multiples of 8 up to ``max_batch_num``) that
        many one-token requests run one step. With ``sampling`` the graphs that sample at a
        temperature are captured too. Returns the batch sizes. Call it on an idle engine."""
        if self.has_unfinished():
            raise RuntimeError("warmup wants an idle engine")
        if not self.runner.fast_decode:
            return []
        top = self.options.max_batch_num
        sizes = sorted({b for b in range(1, min(top, 8) + 1)} | {b for b in range(16, top + 1, 8)} | {top}, reverse=True)
        pages = self.runner.manager.total_pages(0) if self.runner.cache.n_groups else top
        sizes = [b for b in sizes if b <= pages]
        for temperature in ([0.0, 1.0] if sampling else [0.0]):
            for b in sizes:
                self.generate([[0]] * b, SamplingParams(temperature=temperature, max_new_tokens=1, ignore_eos=True))
        return sizes

    def stats(self) -> Dict[str, int]:
        s = self.scheduler.counters()
        s["free_pages"] = self.runner.manager.free_pages(0) if self.runner.cache.n_groups else 0
        s["total_pages"] = self.runner.manager.total_pages(0) if self.runner.cache.n_groups else 0
        return s
