"""Single parts of the engine, built and run alone from a test: a thin face over the C functions that
the engine library offers for this (mllm_params_*, mllm_norm_*, mllm_feed_forward_*, mllm_embedding_*,
mllm_head_*). Tensors are torch tensors on the GPU; the parts launch on torch's current stream."""
import ctypes

import torch

from mini_llm_amd import native
from mini_llm_amd.kernels import ops


class Params:
    """A bag of parameters for a part: numbers, strings and tensors by name (kept alive here)."""

    def __init__(self, **kw):
        self._lib = native.lib()
        self.h = self._lib.mllm_params_create()
        self._keep = []
        for k, v in kw.items():
            self.set(k, v)

    def set(self, key, v):
        k = key.replace("__", ".").encode()
        if isinstance(v, torch.Tensor):
            self._keep.append(v)
            self._lib.mllm_params_set_tensor(self.h, k, ctypes.byref(ops.t2(v, key)))
        elif isinstance(v, str):
            self._lib.mllm_params_set_string(self.h, k, v.encode())
        else:
            self._lib.mllm_params_set_number(self.h, k, float(v))

    def __del__(self):
        self._lib.mllm_params_destroy(self.h)


DT = {torch.float32: 0, torch.bfloat16: 1}


def _arena(n_bytes=1 << 22):
    return torch.empty(n_bytes, dtype=torch.uint8, device="cuda:0")


class _Part:
    create = destroy = None

    def __init__(self, kind, params):
        self._lib = native.lib()
        self.params = params
        self.h = getattr(self._lib, self.create)(kind.encode(), params.h)
        if not self.h:
            raise native.EngineError(native.last_error())

    def __del__(self):
        if getattr(self, "h", None):
            getattr(self._lib, self.destroy)(self.h)


class Norm(_Part):
    create, destroy = "mllm_norm_create", "mllm_norm_destroy"

    def forward(self, x, dtype, rows=None):
        n = x.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, x.shape[1]), dtype=dtype, device=x.device)
        a = _arena()
        native.check(self._lib.mllm_norm_forward(self.h, ctypes.byref(ops.t2(x)), ops._p(rows), ctypes.byref(ops.t2(out)),
                                                 a.data_ptr(), a.numel(), ops._stream()))
        return out


class FeedForward(_Part):
    create, destroy = "mllm_feed_forward_create", "mllm_feed_forward_destroy"

    def forward(self, h, x):
        """x += feed_forward(h)"""
        a = _arena()
        native.check(self._lib.mllm_feed_forward_forward(self.h, ctypes.byref(ops.t2(h)), ctypes.byref(ops.t2(x)),
                                                         a.data_ptr(), a.numel(), ops._stream()))
        return x


class Embedding(_Part):
    create, destroy = "mllm_embedding_create", "mllm_embedding_destroy"

    def forward(self, ids, positions, size, position_kind="", position_params=None):
        x = torch.empty((ids.numel(), size), dtype=torch.float32, device=ids.device)
        native.check(self._lib.mllm_embedding_forward(self.h, position_kind.encode(),
                                                      position_params.h if position_params else None, ops._p(ids),
                                                      ops._p(positions), ctypes.byref(ops.t2(x)), ops._stream()))
        return x


class Head(_Part):
    create, destroy = "mllm_head_create", "mllm_head_destroy"

    def forward(self, x, norm, vocab, rows=None):
        n = x.shape[0] if rows is None else rows.numel()
        logits = torch.empty((n, vocab), dtype=torch.float32, device=x.device)
        a = _arena()
        native.check(self._lib.mllm_head_forward(self.h, norm.h, ctypes.byref(ops.t2(x)), ops._p(rows),
                                                 ctypes.byref(ops.t2(logits)), a.data_ptr(), a.numel(), ops._stream()))
        return logits
