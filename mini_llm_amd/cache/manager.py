"""Python face of the native cache manager, and the device storage behind its pages.

``CacheManager`` (C++: csrc/runtime/cache_manager.cc) decides which pages and state
slots a request holds; it never touches device memory. ``CacheStorage`` owns the
device tensors: for every group of layers one pool of pages shared by the layers of
the group, and for state caches one array of slots.

The reference's pool and block manager:
/root/reference/include/runtime/pool.cuh:11-68,
/root/reference/src/runtime/block_manager.cu:39-99.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

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
        "mllm_sched_create": (vp, [vp, i, i, i, i]),
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


# --------------------------------------------------------------------------------
# What a mixer asks of the cache
# --------------------------------------------------------------------------------

@dataclass(frozen=True)
class KVCacheSpec:
    """Keys and values of every token (or of a window of them), in pages."""
    n_kv_heads: int
    head_dim: int
    window: int = 0

    def group_key(self):
        return ("kv", self.n_kv_heads, self.head_dim, self.window)


@dataclass(frozen=True)
class StateCacheSpec:
    """A state of fixed size per request, in a slot."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32

    def group_key(self):
        return ("state", tuple(self.shape), self.dtype)


@dataclass
class KVCacheView:
    """What a mixer sees of its cache during a step."""
    k_pages: torch.Tensor      # [n_pages * page_size, n_kv_heads * head_dim]
    v_pages: torch.Tensor
    group: int                 # index into the step's per-group tables
    page_size: int
    window: int


@dataclass
class StateCacheView:
    slots: torch.Tensor        # [n_state_slots, *shape]


class CacheStorage:
    """Device memory for the caches of a model, grouped by need.

    ``specs[c]`` is what cache ``c`` of the model's execution order asks for. Caches
    with equal KV specs form a group and share page ids, so one block table serves
    all of them: pool layout ``[caches in group][K|V][n_pages * page_size][kv_dim]``.
    """

    def __init__(self, specs: Sequence[object], page_size: int, n_pages: int, n_state_slots: int,
                 dtype: torch.dtype, device, n_pages_by_group: Optional[Dict[int, int]] = None):
        self.page_size = int(page_size)
        self.dtype = dtype
        self.device = torch.device(device)
        self.n_state_slots = int(n_state_slots)
        keys: List[object] = []
        self.cache_group: List[int] = []      # cache index -> kv group index, or -1 for state
        members: List[List[int]] = []
        for c, spec in enumerate(specs):
            if isinstance(spec, KVCacheSpec):
                k = spec.group_key()
                if k not in keys:
                    keys.append(k)
                    members.append([])
                g = keys.index(k)
                members[g].append(c)
                self.cache_group.append(g)
            elif isinstance(spec, StateCacheSpec) or spec is None:
                self.cache_group.append(-1)
            else:
                raise TypeError(f"cache {c}: unknown cache spec {spec!r}")
        self.group_specs: List[GroupSpec] = []
        self._pools: List[torch.Tensor] = []
        self._views: List[Optional[object]] = [None] * len(specs)
        for g, k in enumerate(keys):
            _, hkv, hd, window = k
            npg = (n_pages_by_group or {}).get(g, n_pages)
            self.group_specs.append(GroupSpec(self.page_size, npg, window))
            pool = torch.zeros((len(members[g]), 2, npg * self.page_size, hkv * hd),
                               dtype=dtype, device=self.device)
            self._pools.append(pool)
            for j, c in enumerate(members[g]):
                self._views[c] = KVCacheView(pool[j, 0], pool[j, 1], g, self.page_size, window)
        self._state_views: List[StateCacheView] = []
        for c, spec in enumerate(specs):
            if isinstance(spec, StateCacheSpec):
                slots = torch.zeros((self.n_state_slots,) + tuple(spec.shape), dtype=spec.dtype,
                                    device=self.device)
                self._views[c] = StateCacheView(slots)
                self._state_views.append(self._views[c])
        self.manager = CacheManager(self.group_specs, self.n_state_slots)

    @property
    def n_groups(self) -> int:
        return len(self.group_specs)

    def view(self, cache: int):
        return self._views[cache]

    def reset_fresh_states(self, ctx) -> None:
        """Clears, on the device, the state slot of every request of the step that has no token
        cached yet (``ctx.starts == 0``; a request that begins, or begins again after it was
        preempted). Nothing to do for a model without state caches."""
        if not self._state_views:
            return
        from ..kernels import ops
        for view in self._state_views:
            ops.reset_state(view.slots, ctx.state_slots, ctx.starts)

    def bytes_per_token(self) -> int:
        return sum(p.shape[0] * 2 * p.shape[3] * p.element_size() for p in self._pools)

    def state_bytes_per_request(self) -> int:
        return sum(v.slots[0].numel() * v.slots.element_size() for v in self._state_views)

    def poison(self, value: float = float("nan")) -> None:
        """Fills every page and every state slot with a value (tests: a stale or unwritten page, or
        a state that was not cleared when its request began, must never be read)."""
        for p in self._pools:
            p.fill_(value)
        for v in self._state_views:
            v.slots.fill_(value)
