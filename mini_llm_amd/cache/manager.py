"""Python face of the native cache manager (tests drive it from here).

``CacheManager`` (C++: csrc/runtime/cache_manager.cc) decides which pages and state
slots a request holds; it never touches device memory. The device memory behind the
pages belongs to the engine's ``CacheStorage`` (csrc/engine/engine.cc): for every group
of layers one pool of pages shared by the layers of the group, and for state caches one
array of slots.

The reference's pool and block manager:
/root/reference/include/runtime/pool.cuh:11-68,
/root/reference/src/runtime/block_manager.cu:39-99.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from ..build import load_library

_i32p = ctypes.POINTER(ctypes.c_int)


def _rt():
    lib = load_library("runtime")
    if getattr(lib, "_mllm_typed", False):
        return lib
    vp, i64, i = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    sigs = {
        "mllm_cache_create": (vp, [i, _i32p, _i32p, _i32p, i]),
        "mllm_cache_destroy": (None, [vp]),
        "mllm_cache_add_request": (i, [vp, i64]),
        "mllm_cache_has_request": (i, [vp, i64]),
        "mllm_cache_pages_needed": (i, [vp, i64, i, i]),
        "mllm_cache_can_reserve": (i, [vp, i64, i]),
        "mllm_cache_reserve": (i, [vp, i64, i]),
        "mllm_cache_commit": (i, [vp, i64, i]),
        "mllm_cache_free_request": (i, [vp, i64]),
        "mllm_cache_length": (i, [vp, i64]),
        "mllm_cache_state_slot": (i, [vp, i64]),
        "mllm_cache_block_table": (i, [vp, i64, i, ctypes.c_void_p, i]),
        "mllm_cache_fill_step_common": (i, [vp] * 3 + [i] + [vp] * 6),
        "mllm_cache_fill_step_group": (i, [vp, vp, vp, i, i, i, vp, vp]),
        "mllm_cache_free_pages": (i, [vp, i]),
        "mllm_cache_total_pages": (i, [vp, i]),
        "mllm_cache_free_state_slots": (i, [vp]),
        "mllm_cache_n_requests": (i, [vp]),
        "mllm_cache_check": (i, [vp, ctypes.c_char_p, i]),
        "mllm_sched_create": (vp, [vp, i, i, i, i, i]),
        "mllm_sched_destroy": (None, [vp]),
        "mllm_sched_add": (i, [vp, i64, i, i]),
        "mllm_sched_schedule": (i, [vp, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, i]),
        "mllm_sched_commit": (None, [vp]),
        "mllm_sched_on_token": (i, [vp, i64, i]),
        "mllm_sched_abort": (i, [vp, i64]),
        "mllm_sched_stop": (i, [vp, i64]),
        "mllm_sched_forget": (i, [vp, i64]),
        "mllm_sched_n_known": (i, [vp]),
        "mllm_sched_has_work": (i, [vp]),
        "mllm_sched_state": (i, [vp, i64]),
        "mllm_sched_generated": (i, [vp, i64]),
        "mllm_sched_pop_event": (i, [vp, ctypes.POINTER(i64), ctypes.POINTER(i)]),
        "mllm_sched_queue_length": (i, [vp, i]),
        "mllm_sched_counters": (None, [vp, ctypes.c_void_p]),
    }
    for name, (res, args) in sigs.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    lib._mllm_typed = True
    return lib


class OutOfPages(RuntimeError):
    """A request asked for more pages than are free."""


@dataclass(frozen=True)
class GroupSpec:
    """A group of caches with the same needs; it owns a pool of pages."""
    page_size: int
    n_pages: int
    window: int = 0      # 0: all keys are kept; W > 0: only the last W keys are needed


class CacheManager:
    """Pages and state slots of live requests (bookkeeping only, no device memory)."""

    def __init__(self, groups: Sequence[GroupSpec], n_state_slots: int):
        self._lib = _rt()
        self.groups = list(groups)
        self.n_state_slots = int(n_state_slots)
        n = len(self.groups)
        ps = (ctypes.c_int * max(n, 1))(*[g.page_size for g in self.groups])
        npg = (ctypes.c_int * max(n, 1))(*[g.n_pages for g in self.groups])
        win = (ctypes.c_int * max(n, 1))(*[g.window for g in self.groups])
        self._h = self._lib.mllm_cache_create(n, ps, npg, win, self.n_state_slots)
        if not self._h:
            raise ValueError(f"invalid cache groups {self.groups} or slots {n_state_slots}")

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.mllm_cache_destroy(h)

    @property
    def handle(self):
        return self._h

    def add_request(self, rid: int) -> int:
        slot = self._lib.mllm_cache_add_request(self._h, rid)
        if slot == -2:
            raise KeyError(f"request {rid} is already registered")
        if slot == -1:
            raise OutOfPages("no free state slot")
        return slot

    def has_request(self, rid: int) -> bool:
        return bool(self._lib.mllm_cache_has_request(self._h, rid))

    def pages_needed(self, rid: int, group: int, new_len: int) -> int:
        return self._lib.mllm_cache_pages_needed(self._h, rid, group, new_len)

    def can_reserve(self, rid: int, new_len: int) -> bool:
        return bool(self._lib.mllm_cache_can_reserve(self._h, rid, new_len))

    def reserve(self, rid: int, new_len: int) -> None:
        rc = self._lib.mllm_cache_reserve(self._h, rid, new_len)
        if rc == -1:
            raise OutOfPages(f"request {rid}: not enough free pages to hold {new_len} tokens")
        if rc != 0:
            raise KeyError(f"request {rid}: unknown, or {new_len} is below its committed length")

    def try_reserve(self, rid: int, new_len: int) -> bool:
        return self._lib.mllm_cache_reserve(self._h, rid, new_len) == 0

    def commit(self, rid: int, new_len: int) -> None:
        if self._lib.mllm_cache_commit(self._h, rid, new_len) != 0:
            raise KeyError(f"request {rid}: cannot commit length {new_len}")

    def free_request(self, rid: int) -> int:
        n = self._lib.mllm_cache_free_request(self._h, rid)
        if n == -2:
            raise KeyError(f"request {rid} is not registered (freed twice?)")
        return n

    def length(self, rid: int) -> int:
        n = self._lib.mllm_cache_length(self._h, rid)
        if n < 0:
            raise KeyError(f"request {rid} is not registered")
        return n

    def state_slot(self, rid: int) -> int:
        n = self._lib.mllm_cache_state_slot(self._h, rid)
        if n < 0:
            raise KeyError(f"request {rid} is not registered")
        return n

    def block_table(self, rid: int, group: int, out: Optional[np.ndarray] = None) -> np.ndarray:
        """Page ids of the request's logical blocks in a group (-1 where released)."""
        if out is None:
            n = self._lib.mllm_cache_block_table(self._h, rid, group, None, 0)
            if n < 0:
                raise KeyError(f"request {rid} is not registered")
            out = np.empty(n, dtype=np.int32)
        n = self._lib.mllm_cache_block_table(self._h, rid, group, out.ctypes.data, out.shape[0])
        if n < 0:
            raise KeyError(f"request {rid} is not registered")
        return out[:min(n, out.shape[0])]

    def fill_step_common(self, ids: np.ndarray, n_tokens: np.ndarray, positions, token_seq, cu_q, starts,
                         ctx_len, state_slots) -> None:
        """Fills the step's group-independent int32 index arrays (numpy views) in one native call."""
        rc = self._lib.mllm_cache_fill_step_common(
            self._h, ids.ctypes.data, n_tokens.ctypes.data, len(ids), positions.ctypes.data,
            token_seq.ctypes.data, cu_q.ctypes.data, starts.ctypes.data, ctx_len.ctypes.data,
            state_slots.ctypes.data)
        if rc != 0:
            raise KeyError(f"request {int(ids[-rc - 1])} is not registered")

    def fill_step_group(self, ids: np.ndarray, n_tokens: np.ndarray, group: int, max_blocks: int,
                        tables, slots) -> None:
        """Fills one group's block tables [n, max_blocks] and per-token page rows."""
        rc = self._lib.mllm_cache_fill_step_group(
            self._h, ids.ctypes.data, n_tokens.ctypes.data, len(ids), group, max_blocks,
            tables.ctypes.data, slots.ctypes.data)
        if rc != 0:
            raise KeyError(f"request {int(ids[-rc - 1])}: not registered, no pages reserved for its tokens "
                           f"(reserve before the step), or more than {max_blocks} blocks")

    def free_pages(self, group: int = 0) -> int:
        return self._lib.mllm_cache_free_pages(self._h, group)

    def total_pages(self, group: int = 0) -> int:
        return self._lib.mllm_cache_total_pages(self._h, group)

    def free_state_slots(self) -> int:
        return self._lib.mllm_cache_free_state_slots(self._h)

    def n_requests(self) -> int:
        return self._lib.mllm_cache_n_requests(self._h)

    def check(self) -> str:
        """Empty when no page or slot is lost, held twice, or both held and free."""
        buf = ctypes.create_string_buffer(4096)
        self._lib.mllm_cache_check(self._h, buf, 4096)
        return buf.value.decode()
