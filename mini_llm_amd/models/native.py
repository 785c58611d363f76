"""The model's step function, natively: a model whose parts all have a native kind is handed
to the native engine (csrc/engine/parts.cc), which runs embedding, every call of the execution
order, the final norm and the head in one call without returning to Python between kernels.

A part offers itself by ``native_kind`` (the name it is registered under natively, in the
category of its interface) and ``native_params()`` (numbers, strings and tensors it is built
from). A model with a part that does not (a part written in Python) runs through the parts'
Python ``forward`` methods instead; both paths launch the same kernels through the same native
ops.
"""
from __future__ import annotations

import ctypes
from typing import Dict, List, Optional

import torch

from ..cache.manager import KVCacheView, StateCacheView
from ..kernels import ops
from ..kernels.ops import Tensor2, t2

_vp, _i = ctypes.c_void_p, ctypes.c_int


class StepViewC(ctypes.Structure):
    _fields_ = [("n_tokens", _i), ("n_seqs", _i), ("n_logits", _i), ("max_q_len", _i), ("max_ctx_len", _i),
                ("n_single", _i), ("token_ids", _vp), ("positions", _vp), ("token_seq", _vp), ("cu_q", _vp),
                ("ctx_len", _vp), ("starts", _vp), ("state_slots", _vp), ("logit_rows", _vp), ("n_groups", _i),
                ("block_tables", ctypes.POINTER(_vp)), ("max_blocks", ctypes.POINTER(_i)),
                ("slots", ctypes.POINTER(_vp))]


class CacheViewC(ctypes.Structure):
    _fields_ = [("kind", _i), ("k_pages", Tensor2), ("v_pages", Tensor2), ("group", _i), ("page_size", _i),
                ("window", _i), ("state", _vp), ("slot_bytes", ctypes.c_size_t), ("n_slots", _i)]


_typed = False


def _lib():
    global _typed
    lib = ops.engine_library()
    if not _typed:
        T2p, sz = ctypes.POINTER(Tensor2), ctypes.c_size_t
        sigs = {
            "mllm_params_create": (_vp, []), "mllm_params_destroy": (None, [_vp]),
            "mllm_params_set_number": (None, [_vp, ctypes.c_char_p, ctypes.c_double]),
            "mllm_params_set_string": (None, [_vp, ctypes.c_char_p, ctypes.c_char_p]),
            "mllm_params_set_tensor": (None, [_vp, ctypes.c_char_p, T2p]),
            "mllm_has_part": (_i, [ctypes.c_char_p, ctypes.c_char_p]),
            "mllm_norm_create": (_vp, [ctypes.c_char_p, _vp]), "mllm_mixer_create": (_vp, [ctypes.c_char_p, _vp]),
            "mllm_feed_forward_create": (_vp, [ctypes.c_char_p, _vp]),
            "mllm_block_create": (_vp, [ctypes.c_char_p, _vp, _vp, ctypes.POINTER(_vp), _i]),
            "mllm_model_create": (_vp, [T2p, T2p, _i]), "mllm_model_destroy": (None, [_vp]),
            "mllm_model_add_layer": (_i, [_vp, _vp]),
            "mllm_model_set_order": (None, [_vp, ctypes.POINTER(_i), ctypes.POINTER(_i), ctypes.POINTER(_i), _i]),
            "mllm_model_set_final_norm": (None, [_vp, _vp]),
            "mllm_model_workspace_bytes": (sz, [_vp, _i, _i]),
            "mllm_model_forward": (_i, [_vp, ctypes.POINTER(StepViewC), ctypes.POINTER(CacheViewC), _i, _vp, sz,
                                        T2p, _vp]),
        }
        for name, (res, args) in sigs.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _typed = True
    return lib


def _params(lib, values: Dict[str, object]):
    p = lib.mllm_params_create()
    for key, v in values.items():
        k = key.encode()
        if v is None:
            continue
        if isinstance(v, torch.Tensor):
            lib.mllm_params_set_tensor(p, k, ctypes.byref(t2(v, key)))
        elif isinstance(v, str):
            lib.mllm_params_set_string(p, k, v.encode())
        else:
            lib.mllm_params_set_number(p, k, float(v))
    return p


def _native_kind(part) -> Optional[str]:
    """The native kind a part's own class names (a subclass that changes the part's behaviour in Python
    does not inherit it)."""
    kind = type(part).__dict__.get("native_kind")
    return kind.fget(part) if isinstance(kind, property) else kind


def _part(lib, category: str, part) -> Optional[int]:
    kind = _native_kind(part)
    if kind is None or not lib.mllm_has_part(category.encode(), kind.encode()):
        return None
    create = {"norm": lib.mllm_norm_create, "mixer": lib.mllm_mixer_create,
              "feed_forward": lib.mllm_feed_forward_create}[category]
    p = _params(lib, part.native_params())
    try:
        h = create(kind.encode(), p)
    finally:
        lib.mllm_params_destroy(p)
    if not h:
        raise ops.KernelError(lib.mllm_last_error().decode("utf-8", "replace"))
    return h


class NativeModel:
    """The native twin of a ``DecoderModel`` (same weights: it holds pointers into the model's
    tensors, which the Python model keeps alive)."""

    def __init__(self, handle: int, model):
        self._h = handle
        self._lib = _lib()
        self._model = model                     # keeps the weights alive
        self._arena: Optional[torch.Tensor] = None      # temporaries of steps whose sizes change
        self._static_arena: Optional[torch.Tensor] = None      # temporaries of steps on static buffers (graphs)
        self.on_static_arena_replaced = None           # called when captured graphs have lost their arena
        self._cache_views = None
        self._cache_key = None

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.mllm_model_destroy(h)

    @classmethod
    def build(cls, model) -> Optional["NativeModel"]:
        """The native model, or None if the model is not on the GPU or one of its parts has no native kind."""
        if model.device.type != "cuda":
            return None
        from ..parts.embedding import TiedHead
        lib = _lib()
        if not isinstance(model.head, TiedHead) or model.head.embedding is not model.embedding:
            return None
        from ..parts.base import PositionEncoding
        position = model.position
        table = getattr(position, "table", None) if position is not None else None
        if position is not None:
            # natively: a learned table added where tokens are embedded, or no encoding at all
            if position.applies_in_mixer:
                return None
            if table is None and type(position).at_embedding is not PositionEncoding.at_embedding:
                return None
        blocks: List[int] = []
        try:
            for layer in model.layers:
                kind = _native_kind(layer)
                if kind is None or not lib.mllm_has_part(b"block", kind.encode()):
                    raise _NotNative()
                if getattr(layer.mixer, "position", None) is not None:
                    raise _NotNative()
                mixer = _part(lib, "mixer", layer.mixer)
                ff = _part(lib, "feed_forward", layer.feed_forward)
                norms = [_part(lib, "norm", n) for n in layer.native_norms()]
                if mixer is None or ff is None or any(n is None for n in norms):
                    raise _NotNative()         # (handles made so far leak a few bytes; models are built once)
                arr = (_vp * len(norms))(*norms)
                b = lib.mllm_block_create(kind.encode(), mixer, ff, arr, len(norms))
                if not b:
                    raise ops.KernelError(lib.mllm_last_error().decode("utf-8", "replace"))
                blocks.append(b)
            final = _part(lib, "norm", model.final_norm)
            if final is None:
                raise _NotNative()
        except _NotNative:
            return None
        wte = t2(model.embedding.weight, "wte")
        wpe = t2(table, "wpe") if table is not None else None
        h = lib.mllm_model_create(ctypes.byref(wte), ctypes.byref(wpe) if wpe is not None else None,
                                  ops._DT[model.dtype])
        for b in blocks:
            lib.mllm_model_add_layer(h, b)
        n = len(model.order)
        arr = lambda vals: (_i * n)(*vals)
        lib.mllm_model_set_order(h, arr([c.layer for c in model.order]), arr([c.cache for c in model.order]),
                                 arr([1 if c.write else 0 for c in model.order]), n)
        lib.mllm_model_set_final_norm(h, final)
        return cls(h, model)

    def _views(self, cache):
        if self._cache_key is not cache:
            n = len(cache._views)
            arr = (CacheViewC * max(n, 1))()
            for i, v in enumerate(cache._views):
                if isinstance(v, KVCacheView):
                    arr[i].kind = 1
                    arr[i].k_pages, arr[i].v_pages = t2(v.k_pages, "k_pages"), t2(v.v_pages, "v_pages")
                    arr[i].group, arr[i].page_size, arr[i].window = v.group, v.page_size, int(v.window or 0)
                elif isinstance(v, StateCacheView):
                    arr[i].kind = 2
                    arr[i].state = v.slots.data_ptr()
                    arr[i].n_slots = v.slots.shape[0]
                    arr[i].slot_bytes = (v.slots.numel() // max(v.slots.shape[0], 1)) * v.slots.element_size()
            self._cache_views, self._cache_key, self._n_caches = arr, cache, n
        return self._cache_views

    def reserve_static(self, rows: int) -> None:
        """Room for the temporaries of decode steps of up to ``rows`` tokens on static buffers: graphs
        captured later keep this memory's address, so it is made once, for the largest batch."""
        need = self._lib.mllm_model_workspace_bytes(self._h, int(rows), int(rows))
        if self._static_arena is None or self._static_arena.numel() < need:
            replaced = self._static_arena is not None
            self._static_arena = torch.empty(int(need) + 4096, dtype=torch.uint8, device=self._model.device)
            hook = self.on_static_arena_replaced
            fn = hook() if isinstance(hook, __import__("weakref").WeakMethod) else hook
            if replaced and fn is not None:
                fn()

    def _arena_for(self, ctx) -> torch.Tensor:
        need = self._lib.mllm_model_workspace_bytes(self._h, int(ctx.n_tokens), int(ctx.n_logits))
        if getattr(ctx, "static_buffers", False):
            if self._static_arena is None or self._static_arena.numel() < need:
                self.reserve_static(max(ctx.n_tokens, ctx.n_logits))
            return self._static_arena
        if self._arena is None or self._arena.numel() < need:
            self._arena = torch.empty(int(need * 1.25) + 4096, dtype=torch.uint8, device=self._model.device)
        return self._arena

    def forward(self, ctx, cache) -> Optional[torch.Tensor]:
        lib = self._lib
        ops.push_tuning()
        G = len(ctx.block_tables)
        sv = StepViewC()
        sv.n_tokens, sv.n_seqs, sv.n_logits = ctx.n_tokens, ctx.n_seqs, ctx.n_logits
        sv.max_q_len, sv.max_ctx_len, sv.n_single = ctx.max_q_len, ctx.max_ctx_len, ctx.n_single
        sv.token_ids, sv.positions, sv.token_seq = ctx.token_ids.data_ptr(), ctx.positions.data_ptr(), ctx.token_seq.data_ptr()
        sv.cu_q, sv.ctx_len, sv.starts = ctx.cu_q.data_ptr(), ctx.ctx_len.data_ptr(), ctx.starts.data_ptr()
        sv.state_slots = ctx.state_slots.data_ptr()
        sv.logit_rows = ctx.logit_rows.data_ptr() if ctx.n_logits else None
        sv.n_groups = G
        tables = (_vp * max(G, 1))(*[t.data_ptr() for t in ctx.block_tables])
        maxb = (_i * max(G, 1))(*[t.shape[1] for t in ctx.block_tables])
        slots = (_vp * max(G, 1))(*[t.data_ptr() for t in ctx.slots])
        sv.block_tables, sv.max_blocks, sv.slots = tables, maxb, slots
        logits = None
        if ctx.n_logits:
            logits = torch.empty((ctx.n_logits, self._model.vocab_size), dtype=torch.float32, device=self._model.device)
        arena = self._arena_for(ctx)
        views = self._views(cache)
        rc = lib.mllm_model_forward(self._h, ctypes.byref(sv), views, self._n_caches, arena.data_ptr(), arena.numel(),
                                    ctypes.byref(t2(logits, "logits")) if logits is not None else None, ops._stream())
        if rc != 0:
            raise ops.KernelError(lib.mllm_last_error().decode("utf-8", "replace"))
        return logits


class _NotNative(Exception):
    pass
