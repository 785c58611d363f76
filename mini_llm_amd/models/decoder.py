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

    def step_cost(self) -> dict:
        """What a step costs, read off the parts (for roofline arithmetic, whatever the architecture):

        ``weight_bytes``      bytes of weights that every step reads once whatever its batch (every linear
                              map's matrix and bias, norm gains and shifts, the head's matrix; embedding
                              and position tables are gathered by row and not counted);
        ``flops_per_token``   matrix-product flops of the layers per token (2 x in x out of every linear
                              map, per call of the execution order);
        ``flops_per_logits_row``  the head's product for one wanted row;
        ``attention_flops_per_key``  flops per (token, attended key) summed over the attention calls
                              (4 x query width: scores and value mix).
        """
        from ..parts.linear import Linear

        def linears(part):
            return [v for v in vars(part).values() if isinstance(v, Linear)] if part is not None else []

        def vectors(part):
            out = []
            for v in (vars(part).values() if part is not None else ()):
                if isinstance(v, torch.Tensor) and v.dim() == 1:
                    out.append(v)
                elif isinstance(v, Norm):
                    out += vectors(v)
            return out

        nbytes = lambda t: 0 if t is None else t.numel() * t.element_size()
        weight_bytes = 0
        for layer in self.layers:
            for part in (layer, getattr(layer, "mixer", None), getattr(layer, "feed_forward", None)):
                for lin in linears(part):
                    weight_bytes += nbytes(lin.weight) + nbytes(lin.bias)
                weight_bytes += sum(nbytes(v) for v in vectors(part))
        weight_bytes += sum(nbytes(v) for v in vectors(self.final_norm))
        head_w = self.embedding.weight if isinstance(self.head, TiedHead) else getattr(self.head, "weight", None)
        weight_bytes += nbytes(head_w)
        flops = attn = 0
        for call in self.order:
            layer = self.layers[call.layer]
            for part in (getattr(layer, "mixer", None), getattr(layer, "feed_forward", None)):
                flops += sum(2 * lin.in_features * lin.out_features for lin in linears(part))
            q_dim = getattr(getattr(layer, "mixer", None), "q_dim", 0)
            attn += 4 * q_dim
        head_flops = 2 * self.embedding.size * self.vocab_size
        return {"weight_bytes": weight_bytes, "flops_per_token": flops, "flops_per_logits_row": head_flops,
                "attention_flops_per_key": attn}

    use_native = True        # False: always run through the parts' Python forward methods (tests compare the two)

    def native(self):
        """The native twin of this model (built at first use, once the weights are loaded), or None when
        a part has no native kind or the model is not on the GPU."""
        if not hasattr(self, "_native"):
            from .native import NativeModel
            self._native = NativeModel.build(self)
        return self._native

    def forward(self, ctx, cache) -> Optional[torch.Tensor]:
        """Runs the step's tokens through every call of the execution order and returns
        fp32 logits ``[len(ctx.logit_rows), vocab]`` (None if no logits are wanted). A model whose
        parts are all native runs the whole step in one native call; otherwise the parts' Python
        ``forward`` methods run one after the other (the same kernels either way)."""
        native = self.native() if self.use_native else None
        if native is not None:
            return native.forward(ctx, cache)
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
        mixer = None if ls.mixer is None else build_part(MIXERS, ls.mixer, dtype, device, "mixer")
        if position is not None and position.applies_in_mixer and hasattr(mixer, "position"):
            mixer.position = position        # an encoding that turns queries and keys inside the mixer
        ff = None if ls.feed_forward is None else build_part(FEED_FORWARDS, ls.feed_forward, dtype, device, "feed-forward")
        block_cls = BLOCKS[ls.block]
        norms = [build_part(NORMS, ls.norm_at(i), dtype, device, "norm") for i in range(block_cls.n_norms)]
        layers.append(block_cls(mixer=mixer, feed_forward=ff, norms=norms, norm_names=ls.norm_names,
                                dtype=dtype, device=device))
        prefixes.append(ls.weight_prefix)
    return layers, prefixes
