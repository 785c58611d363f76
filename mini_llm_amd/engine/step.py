"""The step function: one batch of (request, its next tokens) through the model.

A step holds any mixture of prompt portions and single decoded tokens, cut anywhere.
It runs only the tokens it is given, reads everything earlier from the cache, writes
the new keys/values (or state) to the cache, and returns fp32 logits at the wanted
places only.

The reference has two entry points that never mix, whole prompts and single tokens
(/root/reference/include/model/gpt2_model.cuh:89-95), and rebuilds its index arrays
on the host for every layer (/root/reference/src/model/gpt2_model.cu:214-248,505-588);
here they are built once per step and reach the device in one copy.
"""
from __future__ import annotations

import os

import gc
import weakref
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheStorage
from ..sampling.sampler import Sampler


@dataclass
class StepEntry:
    """A request's share of a step: its next tokens, and where logits are wanted."""
    request_id: int
    tokens: Sequence[int]
    want: Sequence[int] = ()      # indices into ``tokens`` whose logits are returned


@dataclass
class StepContext:
    """Everything a part may need to know about the step's batch (device tensors are int32)."""
    n_tokens: int
    n_seqs: int
    n_logits: int
    token_ids: torch.Tensor       # [T]
    positions: torch.Tensor       # [T] position of each token in its own sequence
    token_seq: torch.Tensor       # [T] batch row of each token
    cu_q: torch.Tensor            # [B+1] row range of each sequence
    ctx_len: torch.Tensor         # [B] tokens cached once this step is done
    starts: torch.Tensor          # [B] tokens cached before this step
    state_slots: torch.Tensor     # [B] per-request state slot; < 0: a padding row, whose state is neither
                                  #     read nor written (as a token whose page row in ``slots`` is < 0
                                  #     writes no key or value)
    logit_rows: torch.Tensor      # [n_logits] rows whose logits are wanted
    block_tables: List[torch.Tensor]   # per group [B, max_blocks]
    slots: List[torch.Tensor]          # per group [T] row of the page pool each token writes
    max_q_len: int
    max_ctx_len: int
    n_single: int = 0             # the first n_single sequences bring one token each (decoded tokens stand
                                  #     first in a scheduler's mixed step); kernels may treat them apart
    static_buffers: bool = False  # the step runs from buffers whose addresses never change (a captured
                                  #     graph replays it): its temporaries must stay where they are too
    # host copies, for parts that plan on the host
    h_cu_q: np.ndarray = None
    h_starts: np.ndarray = None
    h_state_slots: np.ndarray = None
    request_ids: List[int] = field(default_factory=list)


class StepError(ValueError):
    pass


class _Staging:
    """Pinned host buffers used in turn, each with the device buffer it is copied to: the host
    may fill one while the copy out of the other is still queued on the stream."""

    def __init__(self, device, n_buffers: int = 2):
        self.device = torch.device(device)
        self._bufs: List[list] = [[None, None, None] for _ in range(n_buffers)]   # pinned, device, event
        self._turn = 0

    def take(self, n_ints: int):
        """A host numpy view of n_ints int32 and the matching device tensor (not yet copied)."""
        self._turn = (self._turn + 1) % len(self._bufs)
        b = self._bufs[self._turn]
        if b[0] is None or b[0].numel() < n_ints:
            cap = max(n_ints, 4096) * 2
            on_gpu = self.device.type == "cuda"
            b[0] = torch.empty(cap, dtype=torch.int32, pin_memory=on_gpu)
            b[1] = torch.empty(cap, dtype=torch.int32, device=self.device)
            b[2] = torch.cuda.Event() if on_gpu else None
        elif b[2] is not None:
            b[2].synchronize()            # the copy that last read this buffer is done
        return b[0].numpy()[:n_ints], b

    @staticmethod
    def upload(b, n_ints: int, dst: Optional[torch.Tensor] = None) -> torch.Tensor:
        dev = b[1] if dst is None else dst
        dev[:n_ints].copy_(b[0][:n_ints], non_blocking=True)
        if b[2] is not None:
            b[2].record()
        return dev


def _layout(T: int, B: int, n_logits: int, max_blocks: Sequence[int]):
    """Offsets of the step's int32 arrays in one packed buffer."""
    sizes = [T, T, T, B + 1, B, B, B, max(n_logits, 1)]
    for mb in max_blocks:
        sizes += [B * mb, T]
    offs = [0]
    for n in sizes:
        offs.append(offs[-1] + n)
    return offs


class ModelRunner:
    """Owns a model and its cache storage, and runs steps."""

    def __init__(self, model, page_size: int, n_pages: int, max_num_seqs: int):
        self.model = model
        self.device = model.device
        self.cache = CacheStorage(model.cache_specs(), page_size, n_pages, max_num_seqs, model.dtype,
                                  model.device)
        self.manager = self.cache.manager
        self.page_size = page_size
        self.n_pages = n_pages
        self._staging = _Staging(self.device)
        self._staging_src = _Staging(self.device)      # rows that feed tokens from the previous launch
        self._graphs: Dict[tuple, "DecodeGraph"] = {}
        self._tok_out: Optional[torch.Tensor] = None      # sampled tokens of the last launched step
        self._host_tok = None
        self._turn_out = 0
        self.sampler = Sampler(self.device, max_num_seqs)
        # Pure-decode batches may run from static buffers (`launch_decode`) unless a part of the model
        # plans on the host; on the GPU those steps are captured and replayed as HIP graphs.
        self.fast_decode = bool(getattr(model, "graph_safe", True))
        # (with MINI_LLM_STAGE_TIMES set the native forward pass times its stages with events, which a
        # replayed graph would not hold: every step is then launched as it is)
        self.use_graphs = (self.device.type == "cuda" and self.fast_decode
                           and os.environ.get("MINI_LLM_STAGE_TIMES") is None)
        # Kernel scratch is sized now for the largest decode batch, so that no captured graph is left
        # with the address of a buffer that a larger batch replaced; should one grow after all (a
        # step that wants more logits rows than that), the graphs are dropped and captured again.
        from ..kernels import ops
        if self.device.type == "cuda":
            rows = -(-max(max_num_seqs, 1) // 8) * 8
            n_heads = max((getattr(m, "n_heads", 0) for m in self._mixers()), default=0)
            head_dim = max((getattr(m, "head_dim", 0) for m in self._mixers()), default=0)
            ops.reserve_scratch(self.device, rows, model.vocab_size, n_heads, head_dim)
            ops.on_scratch_growth(self._drop_graphs)
            native = model.native() if getattr(model, "use_native", False) and hasattr(model, "native") else None
            if native is not None:
                native.reserve_static(rows)
                native.on_static_arena_replaced = weakref.WeakMethod(self._drop_graphs)

    def _mixers(self):
        return [getattr(layer, "mixer", None) for layer in getattr(self.model, "layers", [])]

    def _drop_graphs(self) -> None:
        self._graphs.clear()

    def forward(self, ctx: "StepContext") -> Optional[torch.Tensor]:
        """The model over one batch: fresh requests (no token cached yet) get their fixed-size state
        cleared on the device first, then every layer runs."""
        self.cache.reset_fresh_states(ctx)
        return self.model.forward(ctx, self.cache)

    # -- cache bookkeeping for callers without a scheduler ---------------------------
    def ensure_request(self, rid: int) -> None:
        if not self.manager.has_request(rid):
            self.manager.add_request(rid)

    def end_request(self, rid: int) -> None:
        self.manager.free_request(rid)

    # -- the step ----------------------------------------------------------------------
    def _fill(self, host: np.ndarray, offs, ids: np.ndarray, n_tok: np.ndarray, max_blocks: Sequence[int]):
        """Fills the packed index arrays (all but token ids and logit rows) natively."""
        seg = [host[offs[i]:offs[i + 1]] for i in range(len(offs) - 1)]
        self.manager.fill_step_common(ids, n_tok, seg[1], seg[2], seg[3], seg[5], seg[4], seg[6])
        for g, mb in enumerate(max_blocks):
            self.manager.fill_step_group(ids, n_tok, g, mb, seg[8 + 2 * g], seg[9 + 2 * g])
        return seg

    def _context(self, dev: torch.Tensor, offs, T, B, n_logits, max_blocks, max_q_len, max_ctx_len,
                 seg=None, request_ids=(), n_single=0) -> StepContext:
        d = [dev[offs[i]:offs[i + 1]] for i in range(len(offs) - 1)]
        G = len(max_blocks)
        return StepContext(
            n_tokens=T, n_seqs=B, n_logits=n_logits,
            token_ids=d[0], positions=d[1], token_seq=d[2], cu_q=d[3], ctx_len=d[4], starts=d[5],
            state_slots=d[6], logit_rows=d[7][:n_logits],
            block_tables=[d[8 + 2 * g].view(B, max_blocks[g]) for g in range(G)],
            slots=[d[9 + 2 * g] for g in range(G)],
            max_q_len=max_q_len, max_ctx_len=max_ctx_len, n_single=n_single,
            h_cu_q=None if seg is None else seg[3].copy(),
            h_starts=None if seg is None else seg[5].copy(),
            h_state_slots=None if seg is None else seg[6].copy(),
            request_ids=list(request_ids))

    def build_context(self, entries: Sequence[StepEntry]) -> StepContext:
        B = len(entries)
        if B == 0:
            raise StepError("a step needs at least one entry")
        vocab, max_pos = self.model.vocab_size, self.model.max_positions
        ids = np.fromiter((e.request_id for e in entries), dtype=np.int64, count=B)
        if len(set(ids.tolist())) != B:
            dup = [r for r in ids.tolist() if (ids == r).sum() > 1][0]
            raise StepError(f"request {dup} appears twice in one step")
        n_tok = np.fromiter((len(e.tokens) for e in entries), dtype=np.int32, count=B)
        if n_tok.min() < 1:
            raise StepError(f"request {entries[int(n_tok.argmin())].request_id}: an entry needs at least one token")
        T = int(n_tok.sum())
        n_logits = 0
        for e in entries:
            for w in e.want:
                if not (0 <= w < len(e.tokens)):
                    raise StepError(f"request {e.request_id}: wanted index {w} is outside its "
                                    f"{len(e.tokens)} tokens")
            n_logits += len(e.want)
        lengths = np.fromiter((self.manager.length(int(r)) for r in ids), dtype=np.int64, count=B)
        ctx = lengths + n_tok
        if max_pos is not None and int(ctx.max()) > max_pos:
            i = int(ctx.argmax())
            raise StepError(f"request {entries[i].request_id}: {int(ctx[i])} tokens exceed the model's "
                            f"{max_pos} positions")
        G = self.cache.n_groups
        max_blocks = [max(1, -(-int(ctx.max()) // self.page_size))] * G
        offs = _layout(T, B, n_logits, max_blocks)
        host, buf = self._staging.take(offs[-1])
        try:
            seg = self._fill(host, offs, ids, n_tok, max_blocks)
        except KeyError as err:
            raise StepError(str(err.args[0])) from None
        tok, lrows = seg[0], seg[7]
        r = t = 0
        for e in entries:
            n = len(e.tokens)
            tok[t:t + n] = e.tokens
            for w in e.want:
                lrows[r] = t + w
                r += 1
            t += n
        if tok.min() < 0 or tok.max() >= vocab:
            raise StepError(f"token ids must lie in [0, {vocab})")
        dev = self._staging.upload(buf, offs[-1])
        many = np.flatnonzero(n_tok != 1)
        n_single = int(many[0]) if many.size else B
        return self._context(dev, offs, T, B, n_logits, max_blocks, int(n_tok.max()), int(ctx.max()), seg,
                             ids.tolist(), n_single)

    def step(self, entries: Sequence[StepEntry], manage_cache: bool = True) -> Optional[torch.Tensor]:
        """Runs one batch. With ``manage_cache`` the runner registers new requests, takes
        their pages and commits the new lengths itself (replay and tests); a scheduler
        that has done so already passes False. Returns fp32 logits ``[wanted, vocab]`` in
        the order of the entries and of each entry's ``want``, or None if nothing is wanted.
        """
        mgr = self.manager
        if manage_cache:
            fresh = []
            try:
                for e in entries:
                    if not mgr.has_request(e.request_id):
                        mgr.add_request(e.request_id)
                        fresh.append(e.request_id)
                    mgr.reserve(e.request_id, mgr.length(e.request_id) + len(e.tokens))
            except Exception:
                for rid in fresh:
                    mgr.free_request(rid)
                raise
        ctx = self.build_context(entries)
        logits = self.forward(ctx)
        if manage_cache:
            for e in entries:
                mgr.commit(e.request_id, mgr.length(e.request_id) + len(e.tokens))
        return logits

    # -- steps whose sampled tokens stay on the device until asked for -------------------------
    def _room_for_tokens(self, n_rows: int) -> None:
        if self._tok_out is None or self._tok_out.numel() < n_rows:
            # (sized for the most requests the cache manager admits, so this happens once)
            n = max(n_rows, -(-self.manager.n_state_slots // 8) * 8, 8)
            grown = torch.zeros(n, dtype=torch.int32, device=self.device)
            if self._tok_out is not None:
                grown[:self._tok_out.numel()].copy_(self._tok_out)     # tokens a later launch may still take
                self._drop_graphs()                                    # captured graphs hold the old address
            self._tok_out = grown

    def launch_step(self, entries: Sequence[StepEntry], feed_rows: Sequence[int],
                    temperatures: Sequence[float], uniforms: Sequence[float]) -> Optional["PendingTokens"]:
        """Starts one step of any mixture (pages already reserved; the caller commits the lengths)
        and returns at once. Entry i's single token is taken from row ``feed_rows[i]`` of what the
        previous launch sampled where that is >= 0 (the host need not have read it); other entries
        bring their tokens. One token is sampled for every wanted place, in the order of the
        entries, and left on the device for the next launch; ``PendingTokens.result()`` waits for
        them. None if nothing is wanted."""
        from ..kernels import ops
        ctx = self.build_context(entries)
        if any(f >= 0 for f in feed_rows):
            src = np.full(ctx.n_tokens, -1, dtype=np.int32)
            t = 0
            for e, f in zip(entries, feed_rows):
                if f >= 0:
                    if len(e.tokens) != 1:
                        raise StepError("only a single token can come from the previous launch")
                    src[t] = f
                t += len(e.tokens)
            if self._tok_out is None:
                raise StepError("no earlier launch has sampled a token")
            host, buf = self._staging_src.take(ctx.n_tokens)
            host[:] = src
            ops.select_tokens(ctx.token_ids, _Staging.upload(buf, ctx.n_tokens)[:ctx.n_tokens], self._tok_out)
        logits = self.forward(ctx)
        if logits is None:
            return None
        n = logits.shape[0]
        self._room_for_tokens(n)
        out = self._tok_out[:n]
        self.sampler.choose(logits, temperatures, uniforms, out)
        self._turn_out ^= 1
        host_out = self._host_tokens(n)[self._turn_out]
        host_out[:n].copy_(out, non_blocking=True)
        event = None
        if self.device.type == "cuda":
            event = torch.cuda.Event()
            event.record()
        return PendingTokens(host_out, n, event)

    def _host_tokens(self, n: int):
        # two host buffers in turn: one may still be unread when the next step's copy is queued
        if self._host_tok is None or self._host_tok[0].numel() < n:
            cap = max(n, 64)
            pin = self.device.type == "cuda"
            self._host_tok = [torch.zeros(cap, dtype=torch.int32, pin_memory=pin) for _ in range(2)]
        return self._host_tok

    # -- decode steps through a captured HIP graph ------------------------------------------
    def launch_decode(self, request_ids: Sequence[int], tokens: Sequence[int], src_rows: Sequence[int],
                      temperatures: Optional[Sequence[float]] = None,
                      uniforms: Optional[Sequence[float]] = None) -> "PendingTokens":
        """Starts one decode step for the given requests (pages already reserved; the caller commits
        the lengths) and returns at once. Row i's input token is ``tokens[i]``, or, where
        ``src_rows[i] >= 0``, the token that the previous launch sampled in that row (the host need
        not have read it). The model and the sampler run from static buffers, on the GPU as one HIP
        graph captured at a batch size's first use. ``PendingTokens.result()`` waits for the
        sampled tokens."""
        B = len(request_ids)
        greedy = temperatures is None or all(t <= 0 for t in temperatures)
        bucket = B if B <= 8 else -(-B // 8) * 8
        self._room_for_tokens(bucket)
        if self.use_graphs:
            from ..kernels import ops
            ops.notify_scratch_growth()           # a scratch buffer replaced since the last step: graphs are dropped
        key = (bucket, greedy)
        g = self._graphs.get(key)
        if g is None:
            g = self._graphs[key] = DecodeGraph(self, bucket, greedy)
        return g.launch(request_ids, tokens, src_rows, temperatures, uniforms)

    def decode_step(self, request_ids: Sequence[int], tokens: Sequence[int],
                    temperatures: Optional[Sequence[float]] = None,
                    uniforms: Optional[Sequence[float]] = None) -> List[int]:
        """One decoded token for each request, waited for: ``launch_decode`` with every input token
        known to the host."""
        return self.launch_decode(request_ids, tokens, [-1] * len(request_ids), temperatures, uniforms).result()


class PendingTokens:
    """The sampled tokens of a launched decode step; ``result()`` waits until they have reached
    the host."""

    def __init__(self, host: torch.Tensor, n: int, event):
        self._host, self._n, self._event = host, n, event

    def result(self) -> List[int]:
        if self._event is not None:
            self._event.synchronize()
        return self._host[:self._n].tolist()


class DecodeGraph:
    """A decode step of fixed batch size on static buffers: embedding, every layer, the head and
    the sampler; on the GPU captured once and replayed as a HIP graph. Per step the host only
    refreshes the index arrays (one copy: temperatures and uniform numbers travel in the same
    buffer) and later reads the sampled tokens, which every graph of a runner leaves in the same
    device buffer, so that the next step can take its input tokens from there before the host has
    seen them.

    Rows beyond the live batch repeat row 0 but write nothing: their page rows and their state
    slots are -1. So one graph serves every batch size up to its own. The run that precedes the
    capture (it loads the kernels) is made of such rows only, so a step's effects on keys, values
    and state happen once, in the replay.
    """

    def __init__(self, runner: ModelRunner, batch: int, greedy: bool):
        from ..kernels import ops
        self.runner = weakref.proxy(runner)      # the runner owns this object: no reference cycle between them
        self.batch, self.greedy = batch, greedy
        model, cache = runner.model, runner.cache
        dev = runner.device
        on_gpu = dev.type == "cuda"
        max_pos = model.max_positions
        cap_blocks = runner.n_pages if max_pos is None else min(runner.n_pages, -(-max_pos // runner.page_size))
        self.max_blocks = [max(1, cap_blocks)] * cache.n_groups
        B = batch
        self.offs = _layout(B, B, B, self.max_blocks)
        self.n_ctx_ints = self.offs[-1]
        # then: the row of the last launch each token comes from, temperatures, uniform numbers
        self.n_ints = self.n_ctx_ints + 3 * B
        self.dev_ints = torch.zeros(self.n_ints, dtype=torch.int32, device=dev)
        self.src_rows = self.dev_ints[self.n_ctx_ints:self.n_ctx_ints + B]
        self.d_float = self.dev_ints[self.n_ctx_ints + B:].view(torch.float32).view(2, B)
        self.ctx = runner._context(self.dev_ints, self.offs, B, B, B, self.max_blocks, 1,
                                   self.max_blocks[0] * runner.page_size if self.max_blocks else 1, n_single=B)
        self.ctx.static_buffers = True
        self.out = runner._tok_out[:B]
        # two host buffers in turn: one may still be unread when the next step's copy is queued
        self.h_out = [torch.zeros(B, dtype=torch.int32, pin_memory=on_gpu) for _ in range(2)]
        self._turn = 0
        self.capture = runner.use_graphs
        self.graph: Optional["torch.cuda.CUDAGraph"] = None
        self._ops = ops

    def _forward(self) -> None:
        self._ops.select_tokens(self.ctx.token_ids, self.src_rows, self.runner._tok_out)
        logits = self.runner.forward(self.ctx)
        if self.greedy:
            self._ops.argmax(logits, self.out)
        else:
            self._ops.sample(logits, self.d_float[0], self.d_float[1], self.out)

    def _fill(self, request_ids, tokens, src_rows, temperatures, uniforms, live: bool = True) -> None:
        """Refreshes the static buffers for this batch. ``live`` False: every row is a padding row."""
        r, B, n = self.runner, self.batch, len(request_ids)
        ids = np.empty(B, dtype=np.int64)
        ids[:n] = request_ids
        ids[n:] = request_ids[0]
        n_tok = np.ones(B, dtype=np.int32)
        host, buf = r._staging.take(self.n_ints)
        seg = r._fill(host[:self.n_ctx_ints], self.offs, ids, n_tok, self.max_blocks)
        tok = seg[0]
        tok[:n] = tokens
        tok[n:] = tokens[0]
        if tok.min() < 0 or tok.max() >= r.model.vocab_size:
            raise StepError(f"token ids must lie in [0, {r.model.vocab_size})")
        seg[7][:] = np.arange(B, dtype=np.int32)
        first_pad = n if live else 0
        seg[6][first_pad:] = -1                      # padding rows touch no state
        for g in range(len(self.max_blocks)):
            seg[9 + 2 * g][first_pad:] = -1          # and write nothing to the pages
        src = host[self.n_ctx_ints:self.n_ctx_ints + B]
        src[:n] = src_rows
        src[n:] = src_rows[0]
        fl = host[self.n_ctx_ints + B:self.n_ints].view(np.float32).reshape(2, B)
        fl[:] = 0.0
        if not self.greedy:
            fl[0, :n] = temperatures
            fl[1, :n] = uniforms
        _Staging.upload(buf, self.n_ints, self.dev_ints)

    def launch(self, request_ids, tokens, src_rows, temperatures, uniforms) -> PendingTokens:
        n = len(request_ids)
        if self.capture and self.graph is None:
            # First use: run once eagerly (loads the kernels), with rows that write nothing, then
            # capture. The run overwrites the sampled tokens that this step may be fed from, so they
            # are set aside.
            self._fill(request_ids, tokens, src_rows, temperatures, uniforms, live=False)
            fed = self.runner._tok_out.clone()
            self._forward()
            torch.cuda.synchronize()
            self.runner._tok_out.copy_(fed)
            self.graph = torch.cuda.CUDAGraph()
            # No graph may be destroyed while the stream captures (HIP refuses it and the process
            # ends), and a dropped engine's graphs may sit in a reference cycle until the collector
            # runs: so it does not run during the capture. (Running it before every capture instead
            # costs more than the capture.)
            gc_was_enabled = gc.isenabled()
            gc.disable()
            try:
                with torch.cuda.graph(self.graph):
                    self._forward()
            finally:
                if gc_was_enabled:
                    gc.enable()
        self._fill(request_ids, tokens, src_rows, temperatures, uniforms)
        if self.capture:
            self.graph.replay()
        else:
            self._forward()
        self._turn ^= 1
        host = self.h_out[self._turn]
        host.copy_(self.out, non_blocking=True)
        event = None
        if self.capture:
            event = torch.cuda.Event()
            event.record()
        return PendingTokens(host, n, event)
