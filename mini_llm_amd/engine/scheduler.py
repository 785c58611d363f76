"""Python face of the native scheduler (csrc/runtime/scheduler.cc)."""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import numpy as np

from ..cache.manager import CacheManager, _rt

STATE_NAMES = {
    0: "waiting_prefill", 1: "deferred_prefill", 2: "prefill", 3: "decode_ready",
    4: "deferred_decode", 5: "finished", 6: "failed", 7: "aborted", -1: "unknown",
}
EVENT_NAMES = {1: "preempted", 2: "failed", 3: "deferred"}
QUEUES = {"waiting_prefill": 0, "deferred_prefill": 1, "prefill": 2, "decode": 3, "deferred_decode": 4}
COUNTER_NAMES = ("steps", "scheduled_tokens", "prefill_tokens", "decode_tokens", "deferred_decodes",
                 "deferred_prefills", "preemptions", "failures", "finished", "peak_pages_used", "aborted")


@dataclass(frozen=True)
class PlanEntry:
    request_id: int
    start: int          # tokens already cached
    n_tokens: int       # tokens fed by this step
    want_last: bool     # the last of them is the request's newest token: sample after it


class Scheduler:
    def __init__(self, cache: CacheManager, max_num_seqs: int, max_tokens_per_step: int,
                 prefill_chunk: int, max_positions: Optional[int], preempt_for_decode: bool = False):
        self._lib = _rt()
        self._cache = cache       # keeps the native cache manager alive
        self.max_num_seqs = int(max_num_seqs)
        self._h = self._lib.mllm_sched_create(cache.handle, int(max_num_seqs), int(max_tokens_per_step),
                                              int(prefill_chunk), int(max_positions or 0),
                                              1 if preempt_for_decode else 0)
        cap = self.max_num_seqs
        self._ids = np.empty(cap, dtype=np.int64)
        self._start = np.empty(cap, dtype=np.int32)
        self._n = np.empty(cap, dtype=np.int32)
        self._want = np.empty(cap, dtype=np.int32)

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.mllm_sched_destroy(h)

    def add_request(self, rid: int, prompt_len: int, max_new_tokens: int) -> None:
        rc = self._lib.mllm_sched_add(self._h, rid, prompt_len, max_new_tokens)
        if rc == -2:
            raise KeyError(f"request {rid} already exists")
        if rc != 0:
            raise ValueError(
                f"request {rid} refused: prompt of {prompt_len} tokens (must be 1..max positions) "
                f"and max_new_tokens={max_new_tokens} (must be >= 1)")

    def schedule(self) -> List[PlanEntry]:
        n = self._lib.mllm_sched_schedule(self._h, self._ids.ctypes.data, self._start.ctypes.data,
                                          self._n.ctypes.data, self._want.ctypes.data, self._ids.shape[0])
        assert n <= self._ids.shape[0]
        return [PlanEntry(int(self._ids[i]), int(self._start[i]), int(self._n[i]), bool(self._want[i]))
                for i in range(n)]

    def commit(self) -> None:
        self._lib.mllm_sched_commit(self._h)

    def on_token(self, rid: int, is_eos: bool) -> bool:
        rc = self._lib.mllm_sched_on_token(self._h, rid, 1 if is_eos else 0)
        if rc < 0:
            raise KeyError(f"request {rid} is unknown")
        return rc == 1

    def abort(self, rid: int) -> None:
        if self._lib.mllm_sched_abort(self._h, rid) != 0:
            raise KeyError(f"request {rid} is unknown")

    def stop(self, rid: int) -> None:
        """The request ended with a token sampled earlier: finished (not failed), pages freed."""
        if self._lib.mllm_sched_stop(self._h, rid) != 0:
            raise KeyError(f"request {rid} is unknown")

    def forget(self, rid: int) -> None:
        """Drops the record of a finished or failed request; its id may then be used again."""
        self._lib.mllm_sched_forget(self._h, rid)

    def n_known(self) -> int:
        return self._lib.mllm_sched_n_known(self._h)

    def has_work(self) -> bool:
        return bool(self._lib.mllm_sched_has_work(self._h))

    def state(self, rid: int) -> str:
        return STATE_NAMES[self._lib.mllm_sched_state(self._h, rid)]

    def generated(self, rid: int) -> int:
        return self._lib.mllm_sched_generated(self._h, rid)

    def pop_events(self) -> List[Tuple[int, str]]:
        out = []
        rid, kind = ctypes.c_int64(), ctypes.c_int()
        while self._lib.mllm_sched_pop_event(self._h, ctypes.byref(rid), ctypes.byref(kind)):
            out.append((rid.value, EVENT_NAMES[kind.value]))
        return out

    def queue_length(self, name: str) -> int:
        return self._lib.mllm_sched_queue_length(self._h, QUEUES[name])

    def counters(self) -> Dict[str, int]:
        buf = np.zeros(len(COUNTER_NAMES), dtype=np.int64)
        self._lib.mllm_sched_counters(self._h, buf.ctypes.data)
        return dict(zip(COUNTER_NAMES, (int(v) for v in buf)))
