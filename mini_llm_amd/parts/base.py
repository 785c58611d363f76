"""Interfaces of the parts a model is put together from, and their registries.

A part knows its own sizes and constants (given as parameters), the tensors it owns
and what it needs from the cache. It does not know which model it is in.

Interfaces (``ctx`` is the step's ``StepContext``; ``x`` is the fp32 residual
stream ``[T, hidden]``; ``h`` a normalised activation ``[T, hidden]`` in the compute
dtype):

* ``Norm.forward(x, rows=None) -> h``
* ``Mixer.forward(h, ctx, cache_view, x, write=True)``: adds the mixer's output into ``x``
  in place; ``cache_spec()`` says what cache it needs (or None).
* ``FeedForward.forward(h, ctx, x)``: adds its output into ``x`` in place.
* ``PositionEncoding.at_embedding(x, ctx)`` / ``.table``: acts where tokens are
  embedded; ``.in_mixer(qkv, mixer, ctx)``: turns queries/keys in place inside a mixer.
* ``Block.forward(x, ctx, cache_view, write)``: runs one layer on the stream.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Tuple

import torch


@dataclass
class ParamSpec:
    """One tensor a part expects from the checkpoint.

    role: "matrix" (kept in the compute dtype), "vector" (kept in fp32),
          "table" (integers, kept as int32).
    layout: "as_stored" or "transpose" (stored [in, out], used as [out, in]).
    init: (mean, std) of the random-weights mode.
    """
    name: str
    shape: Tuple[int, ...]           # as stored in the checkpoint
    role: str
    assign: Callable[[torch.Tensor], None]
    init: Tuple[float, float] = (0.0, 0.02)
    layout: str = "as_stored"


class Part:
    def __init__(self, dtype: torch.dtype, device):
        self.dtype = dtype
        self.device = torch.device(device)

    def param_specs(self, prefix: str) -> List[ParamSpec]:
        return []


class Norm(Part):
    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        raise NotImplementedError

    def linear(self, x: torch.Tensor, lin, out: torch.Tensor, epilogue: str = "store",
               rows: Optional[torch.Tensor] = None, **linear_options) -> torch.Tensor:
        """out = epilogue(lin(norm(x[rows]))); ``linear_options`` are options of the linear map itself
        (such as a key/value scatter) and are passed through. A norm with a fused kernel overrides this."""
        return lin(self.forward(x, rows), out, epilogue, **linear_options)


class NormedInput:
    """The input of a sub-layer as (stream, norm), not yet normalised. A part that sets
    ``accepts_normed_input`` receives this instead of a tensor and can let its first linear
    map absorb the norm (``linear``); ``tensor()`` gives the normalised activation."""

    def __init__(self, norm: "Norm", x: torch.Tensor):
        self.norm, self.x = norm, x
        self._h = None
        self.shape = x.shape
        self.device = x.device

    def tensor(self) -> torch.Tensor:
        if self._h is None:
            self._h = self.norm.forward(self.x)
        return self._h

    def linear(self, lin, out: torch.Tensor, epilogue: str = "store", **linear_options) -> torch.Tensor:
        """``lin`` applied to the normalised input; ``linear_options`` are options of the linear map
        itself (such as a key/value scatter)."""
        if self._h is not None:
            return lin(self._h, out, epilogue, **linear_options)
        return self.norm.linear(self.x, lin, out, epilogue, **linear_options)


class Mixer(Part):
    accepts_normed_input = False     # True: forward() takes a NormedInput instead of a tensor
    graph_safe = True                # False: forward() plans on the host (reads ctx.h_*), so a decode
                                     # step that contains it cannot be replayed as a HIP graph

    def cache_spec(self):
        """KVCacheSpec, StateCacheSpec or None."""
        return None

    def forward(self, h, ctx, cache_view, x, write: bool = True) -> None:
        raise NotImplementedError


class FeedForward(Part):
    accepts_normed_input = False
    graph_safe = True

    def forward(self, h, ctx, x) -> None:
        raise NotImplementedError


class PositionEncoding(Part):
    """How positions enter the model. Three places, any of which an encoding may use: a learned
    table added where tokens are embedded (``table``, fused into the embedding kernel),
    ``at_embedding`` (anything else done to the embedded stream), and ``in_mixer`` (queries and
    keys turned by position inside every mixer that takes positions: set ``applies_in_mixer``)."""

    table: Optional[torch.Tensor] = None     # learned absolute table, if the encoding is one
    applies_in_mixer = False                 # True: mixers call in_mixer() before keys are written

    def at_embedding(self, x, ctx) -> None:
        pass

    def in_mixer(self, qkv: torch.Tensor, mixer, ctx) -> None:
        """Changes, in place, the query and key columns of ``qkv`` ([T, q | k | v], the mixer says
        where: mixer.q_dim, mixer.kv_dim, mixer.head_dim) for the positions ``ctx.positions``."""


class Block(Part):
    def forward(self, x, ctx, cache_view, write: bool = True) -> None:
        raise NotImplementedError

    @property
    def graph_safe(self) -> bool:
        return all(getattr(getattr(self, name, None), "graph_safe", True) for name in ("mixer", "feed_forward"))

    def cache_spec(self):
        return None


# ---------------------------------------------------------------------------------
# registries: kind name -> class. A part class is built as cls(dtype=, device=, **params)
# (blocks: cls(mixer=, feed_forward=, norms=, dtype=, device=)).
# ---------------------------------------------------------------------------------
MIXERS: Dict[str, type] = {}
FEED_FORWARDS: Dict[str, type] = {}
NORMS: Dict[str, type] = {}
POSITIONS: Dict[str, type] = {}
BLOCKS: Dict[str, type] = {}


def _register(table: Dict[str, type], what: str):
    def deco(kind: str, replace: bool = False):
        def wrap(cls):
            if kind in table and not replace:
                raise ValueError(f"{what} '{kind}' is already registered")
            table[kind] = cls
            return cls
        return wrap
    return deco


register_mixer = _register(MIXERS, "mixer")
register_feed_forward = _register(FEED_FORWARDS, "feed-forward")
register_norm = _register(NORMS, "norm")
register_position = _register(POSITIONS, "position encoding")
register_block = _register(BLOCKS, "block")


def build_part(table: Dict[str, type], spec, dtype, device, what: str):
    if spec.kind not in table:
        raise KeyError(f"unknown {what} '{spec.kind}'; registered: {sorted(table)}")
    return table[spec.kind](dtype=dtype, device=device, **spec.params)
