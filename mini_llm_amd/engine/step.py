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

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheStorage


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
    state_slots: torch.Tensor     # [B] per-request state slot
    logit_rows: torch.Tensor      # [n_logits] rows whose logits are wanted
    block_tables: List[torch.Tensor]   # per group [B, max_blocks]
    slots: List[torch.Tensor]          # per group [T] row of the page pool each token writes
    max_q_len: int
    max_ctx_len: int
    # host copies, for parts that plan on the host
    h_cu_q: np.ndarray = None
    h_starts: np.ndarray = None
    h_state_slots: np.ndarray = None
    request_ids: List[int] = field(default_factory=list)


class StepError(ValueError):
    pass


class ModelRunner:
    """Owns a model and its cache storage, and runs steps."""

    def __init__(self, model, page_size: int, n_pages: int, max_num_seqs: int):
        self.model = model
        self.device = model.device
        self.cache = CacheStorage(model.cache_specs(), page_size, n_pages, max_num_seqs, model.dtype,
                                  model.device)
        self.manager = self.cache.manager
        self.page_size = page_size
        # Two staging buffers used in turn: the host may fill one while the copy out of
        # the other is still queued on the stream.
        self._staging: List[list] = [[None, None, None], [None, None, None]]   # pinned, device, event
        self._turn = 0

    # -- cache bookkeeping for callers without a scheduler ---------------------------
    def ensure_request(self, rid: int) -> None:
        if not self.manager.has_request(rid):
            self.manager.add_request(rid)

    def end_request(self, rid: int) -> None:
        self.manager.free_request(rid)

    # -- the step ----------------------------------------------------------------------
    def build_context(self, entries: Sequence[StepEntry]) -> StepContext:
        mgr, B = self.manager, len(entries)
        if B == 0:
            raise StepError("a step needs at least one entry")
        vocab, max_pos = self.model.vocab_size, self.model.max_positions
        seen = set()
        q_lens = np.empty(B, dtype=np.int64)
        starts = np.empty(B, dtype=np.int64)
        for i, e in enumerate(entries):
            if e.request_id in seen:
                raise StepError(f"request {e.request_id} appears twice in one step")
            seen.add(e.request_id)
            n = len(e.tokens)
            if n < 1:
                raise StepError(f"request {e.request_id}: an entry needs at least one token")
            q_lens[i] = n
            starts[i] = mgr.length(e.request_id)
            for w in e.want:
                if not (0 <= w < n):
                    raise StepError(f"request {e.request_id}: wanted index {w} is outside its {n} tokens")
        T = int(q_lens.sum())
        ctx = starts + q_lens
        if max_pos is not None and int(ctx.max()) > max_pos:
            i = int(ctx.argmax())
            raise StepError(f"request {entries[i].request_id}: {int(ctx[i])} tokens exceed the model's "
                            f"{max_pos} positions")
        n_logits = sum(len(e.want) for e in entries)
        G = self.cache.n_groups
        max_blocks = [max(1, -(-int(ctx.max()) // self.page_size)) for _ in range(G)]

        # one packed int32 buffer: a single host-to-device copy
        sizes = [T, T, T, B + 1, B, B, B, max(n_logits, 1)]
        for g in range(G):
            sizes += [B * max_blocks[g], T]
        offs = np.concatenate([[0], np.cumsum(sizes)])
        total = int(offs[-1])
        self._turn ^= 1
        stage = self._staging[self._turn]
        if stage[0] is None or stage[0].numel() < total:
            cap = max(total, 4096) * 2
            on_gpu = self.device.type == "cuda"
            stage[0] = torch.empty(cap, dtype=torch.int32, pin_memory=on_gpu)
            stage[1] = torch.empty(cap, dtype=torch.int32, device=self.device)
            stage[2] = torch.cuda.Event() if on_gpu else None
        elif stage[2] is not None:
            stage[2].synchronize()        # the copy that last read this buffer is done
        host = stage[0].numpy()
        host[:total] = 0
        seg = [host[offs[i]:offs[i + 1]] for i in range(len(sizes))]
        tok, pos, tseq, cu_q, ctxl, st, slot_ids, lrows = seg[:8]
        cu_q[0] = 0
        np.cumsum(q_lens, out=cu_q[1:])
        ctxl[:] = ctx
        st[:] = starts
        r = 0
        for i, e in enumerate(entries):
            a, b = int(cu_q[i]), int(cu_q[i + 1])
            tok[a:b] = np.asarray(e.tokens, dtype=np.int64)
            pos[a:b] = np.arange(starts[i], ctx[i])
            tseq[a:b] = i
            slot_ids[i] = mgr.state_slot(e.request_id)
            for w in e.want:
                lrows[r] = a + w
                r += 1
        if T and (tok[:T].min() < 0 or tok[:T].max() >= vocab):
            raise StepError(f"token ids must lie in [0, {vocab})")
        for g in range(G):
            tab = seg[8 + 2 * g].reshape(B, max_blocks[g])
            slots = seg[9 + 2 * g]
            for i, e in enumerate(entries):
                row = mgr.block_table(e.request_id, g, out=tab[i])
                a, b = int(cu_q[i]), int(cu_q[i + 1])
                p = pos[a:b]
                blk = p // self.page_size
                if len(row) * self.page_size < int(ctx[i]) or (tab[i][blk] < 0).any():
                    raise StepError(f"request {e.request_id}: no pages are reserved for positions "
                                    f"[{int(starts[i])}, {int(ctx[i])}) (reserve before the step)")
                slots[a:b] = tab[i][blk] * self.page_size + p % self.page_size
        dev = stage[1]
        dev[:total].copy_(stage[0][:total], non_blocking=True)
        if stage[2] is not None:
            stage[2].record()
        d = [dev[int(offs[i]):int(offs[i + 1])] for i in range(len(sizes))]
        return StepContext(
            n_tokens=T, n_seqs=B, n_logits=n_logits,
            token_ids=d[0], positions=d[1], token_seq=d[2], cu_q=d[3], ctx_len=d[4], starts=d[5],
            state_slots=d[6], logit_rows=d[7][:n_logits],
            block_tables=[d[8 + 2 * g].view(B, max_blocks[g]) for g in range(G)],
            slots=[d[9 + 2 * g] for g in range(G)],
            max_q_len=int(q_lens.max()), max_ctx_len=int(ctx.max()),
            h_cu_q=cu_q.copy(), h_starts=starts.astype(np.int32), h_state_slots=slot_ids.copy(),
            request_ids=[e.request_id for e in entries])

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
        logits = self.model.forward(ctx, self.cache)
        if manage_cache:
            for e in entries:
                mgr.commit(e.request_id, mgr.length(e.request_id) + len(e.tokens))
        return logits
