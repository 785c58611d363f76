"""A decoder-only model assembled from parts by configuration.

Nothing here is specific to an architecture: the layers come from
``config.layer_specs()``, their execution order from ``config.layer_order()``.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from ..config.base import LayerCall, LayerSpec, ModelConfig, PartSpec
from ..parts import base as parts_base
from ..parts.base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, Block, Norm, ParamSpec,
                          PositionEncoding, build_part)
from ..parts.embedding import TiedHead, TokenEmbedding


class DecoderModel:
    def __init__(self, config: ModelConfig, embedding: TokenEmbedding, position: Optional[PositionEncoding],
                 layers: Sequence[Block], layer_prefixes: Sequence[str], order: Sequence[LayerCall],
                 final_norm: Norm, final_norm_name: str, head, dtype: torch.dtype, device,
                 weight_prefix: str = ""):
        self.config = config
        self.embedding, self.position = embedding, position
        self.layers, self.layer_prefixes = list(layers), list(layer_prefixes)
        self.order = list(order)
        self.final_norm, self.final_norm_name, self.head = final_norm, final_norm_name, head
        self.dtype, self.device = dtype, torch.device(device)
        self.weight_prefix = weight_prefix
        self.vocab_size = embedding.vocab_size
        for c in self.order:
            if not (0 <= c.layer < len(self.layers)):
                raise ValueError(f"execution order names layer {c.layer}, the model has {len(self.layers)}")
        n_caches = 1 + max((c.cache for c in self.order), default=-1)
        self._cache_specs: List[object] = [None] * n_caches
        written = [False] * n_caches
        for c in self.order:
            spec = self.layers[c.layer].cache_spec()
            if c.write:
                if written[c.cache]:
                    raise ValueError(f"cache {c.cache} is written by two calls of the execution order")
                written[c.cache] = True
                self._cache_specs[c.cache] = spec
            else:
                if not written[c.cache]:
                    raise ValueError(f"a call reads cache {c.cache} before any call has written it")
                if spec != self._cache_specs[c.cache]:
                    raise ValueError(f"a call reads cache {c.cache} whose shape differs from its own")

    @property
    def max_positions(self) -> Optional[int]:
        return self.config.max_positions

    @property
    def graph_safe(self) -> bool:
        """True when a decode step of this model may be captured and replayed as a HIP graph."""
        return all(layer.graph_safe for layer in self.layers)

    def cache_specs(self) -> List[object]:
        return list(self._cache_specs)

    def param_specs(self) -> List[ParamSpec]:
        p = self.weight_prefix
        specs = self.embedding.param_specs(p)
        if self.position is not None:
            specs += self.position.param_specs(p)
        for layer, prefix in zip(self.layers, self.layer_prefixes):
            specs += layer.param_specs(p + prefix)
        specs += self.final_norm.param_specs(p + self.final_norm_name)
        if hasattr(self.head, "param_specs"):
            specs += self.head.param_specs(p)
        return specs

    def forward(self, ctx, cache) -> Optional[torch.Tensor]:
        """Runs the step's tokens through every call of the execution order and returns
        fp32 logits ``[len(ctx.logit_rows), vocab]`` (None if no logits are wanted)."""
        x = self.embedding.forward(ctx, self.position)
        for call in self.order:
            self.layers[call.layer].forward(x, ctx, cache.view(call.cache), call.write)
        if ctx.n_logits == 0:
            return None
        if hasattr(self.head, "forward_normed"):
            return self.head.forward_normed(self.final_norm, x, ctx.logit_rows)
        return self.head.forward(self.final_norm.forward(x, rows=ctx.logit_rows))


def build_layers(specs: Sequence[LayerSpec], dtype, device, position: Optional[PositionEncoding] = None):
    layers, prefixes = [], []
    for ls in specs:
        if ls.block not in BLOCKS:
            raise KeyError(f"unknown block arrangement '{ls.block}'; registered: {sorted(BLOCKS)}")
        mixer = build_part(MIXERS, ls.mixer, dtype, device, "mixer")
        if position is not None and position.applies_in_mixer and hasattr(mixer, "position"):
            mixer.position = position        # an encoding that turns queries and keys inside the mixer
        ff = build_part(FEED_FORWARDS, ls.feed_forward, dtype, device, "feed-forward")
        block_cls = BLOCKS[ls.block]
        norms = [build_part(NORMS, ls.norm, dtype, device, "norm") for _ in range(block_cls.n_norms)]
        layers.append(block_cls(mixer=mixer, feed_forward=ff, norms=norms, norm_names=ls.norm_names,
                                dtype=dtype, device=device))
        prefixes.append(ls.weight_prefix)
    return layers, prefixes
