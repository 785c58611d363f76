"""The engine: requests in, tokens out. Scheduler above, step function below.

One iteration: the scheduler plans a mixed batch (decoded tokens first, then prompt
portions under the token budget), the model runner runs it, the sampler chooses a token
for every request whose newest token was in the batch, finished requests give their
pages back. The reference's loop: /root/reference/src/runtime/scheduler.cpp:322-356;
its offline use of the model: /root/reference/benchmarks/gpt2/bench_batch_vs_single_wall.cu:157-171.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Union

import torch

from ..models import load_model
from ..sampling.sampler import Sampler, SamplingParams, uniform01
from .scheduler import Scheduler
from .step import ModelRunner, StepEntry


@dataclass
class EngineOptions:
    kv_block_size: int = 16             # tokens per page (reference: DEFAULT_KV_BLOCK_SIZE, constants.h:16)
    total_kv_blocks: int = 4096         # pages in the pool (reference: DEFAULT_TOTAL_KV_BLOCKS, constants.h:17)
    max_batch_num: int = 16             # sequences in one step (reference: MAX_BATCH_NUM, constants.h:20)
    max_tokens_per_step: int = 2048     # token budget of one step
    prefill_chunk: int = 512            # longest prompt portion


@dataclass
class RequestOutput:
    request_id: int
    token: int
    finished: bool


@dataclass
class _Request:
    request_id: int
    tokens: List[int]
    prompt_len: int
    params: SamplingParams
    finished: bool = False
    failed: Optional[str] = None

    @property
    def output(self) -> List[int]:
        return self.tokens[self.prompt_len:]


class Engine:
    def __init__(self, model, options: Optional[EngineOptions] = None):
        self.model = model
        self.options = options or EngineOptions()
        o = self.options
        self.runner = ModelRunner(model, o.kv_block_size, o.total_kv_blocks, o.max_batch_num)
        self.scheduler = Scheduler(self.runner.manager, o.max_batch_num, o.max_tokens_per_step,
                                   o.prefill_chunk, model.max_positions)
        self.sampler = Sampler(model.device, o.max_batch_num)
        self.eos_token_id = model.config.eos_token_id
        self.requests: Dict[int, _Request] = {}
        self._next_id = 0

    @classmethod
    def from_pretrained(cls, model_dir: str, dtype="bfloat16", device="cuda:0",
                        options: Optional[EngineOptions] = None, **kw) -> "Engine":
        if kw:
            options = EngineOptions(**{**(options.__dict__ if options else {}), **kw})
        return cls(load_model(model_dir, dtype, device), options)

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

    def abort(self, request_id: int) -> None:
        self.scheduler.abort(request_id)
        r = self.requests[request_id]
        r.finished, r.failed = True, "aborted"

    def has_unfinished(self) -> bool:
        return self.scheduler.has_work()

    # -- one iteration -------------------------------------------------------------------
    def step(self) -> List[RequestOutput]:
        plan = self.scheduler.schedule()
        outputs: List[RequestOutput] = []
        for rid, kind in self.scheduler.pop_events():
            if kind == "failed":
                r = self.requests[rid]
                r.finished, r.failed = True, "the page pool cannot hold this request"
                outputs.append(RequestOutput(rid, -1, True))
        if not plan:
            return outputs
        sampled = [e for e in plan if e.want_last]
        temps, us = [], []
        for e in sampled:
            r = self.requests[e.request_id]
            temps.append(r.params.temperature)
            us.append(uniform01(r.params.seed, len(r.tokens) - r.prompt_len) if r.params.temperature > 0 else 0.0)
        if self.runner.use_graphs and len(sampled) == len(plan) and all(e.n_tokens == 1 for e in plan):
            # every entry is one decoded token: the whole step replays as a HIP graph
            tokens = self.runner.decode_step([e.request_id for e in plan],
                                             [self.requests[e.request_id].tokens[e.start] for e in plan],
                                             temps, us)
            self.scheduler.commit()
        else:
            entries = []
            for e in plan:
                r = self.requests[e.request_id]
                entries.append(StepEntry(e.request_id, r.tokens[e.start:e.start + e.n_tokens],
                                         [e.n_tokens - 1] if e.want_last else []))
            logits = self.runner.step(entries, manage_cache=False)
            self.scheduler.commit()
            tokens = self.sampler.sample(logits, temps, us) if sampled else []
        if sampled:
            for e, tok in zip(sampled, tokens):
                r = self.requests[e.request_id]
                r.tokens.append(tok)
                is_eos = (not r.params.ignore_eos) and self.eos_token_id is not None and tok == self.eos_token_id
                r.finished = self.scheduler.on_token(e.request_id, is_eos)
                outputs.append(RequestOutput(e.request_id, tok, r.finished))
        return outputs

    # -- offline generation --------------------------------------------------------------
    def generate(self, prompts: Sequence[Sequence[int]],
                 params: Union[None, SamplingParams, Sequence[SamplingParams]] = None) -> List[List[int]]:
        """Generates for every prompt (continuous batching) and returns the new tokens of each."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        rids = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        while self.has_unfinished():
            self.step()
        out = []
        for rid in rids:
            r = self.requests.pop(rid)
            if r.failed:
                raise RuntimeError(f"request {rid} failed: {r.failed}")
            out.append(r.output)
        return out

    def stats(self) -> Dict[str, int]:
        s = self.scheduler.counters()
        s["free_pages"] = self.runner.manager.free_pages(0) if self.runner.cache.n_groups else 0
        s["total_pages"] = self.runner.manager.total_pages(0) if self.runner.cache.n_groups else 0
        return s
